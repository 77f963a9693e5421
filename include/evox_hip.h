/* C ABI of libevox_hip.so: MI355X (gfx950) kernels for EvoX's multi-objective environmental
 * selection.  Plain pointers and sizes only; every pointer is DEVICE memory unless said otherwise.
 *
 * Conventions
 *   - Return value: 0 on success, a negative library code (EVOX_HIP_E_*) or a positive hipError_t.
 *     No exceptions cross the boundary and nothing aborts.
 *   - The caller owns every buffer, including the workspace; the library allocates no device memory
 *     and synchronises only in evox_hip_read_status().  (One entry point brings its own scratch memory
 *     instead of taking a workspace: evox_hip_nd_environmental_selection_static.)  All work is enqueued on `stream`
 *     (a hipStream_t passed as void*).
 *   - What the library keeps between calls, per process: the tunables; per device, small host-side tables of what it
 *     has asked the runtime once (compute units, resident workgroups, LDS grants); the scratch buffer of the entry
 *     point named above (EVOX_HIP_STATIC_SCRATCH_BYTES of device memory on every GPU that the process touches,
 *     whether or not that entry point is ever called: it is part of the device image); and 64 bytes of pinned host
 *     memory per device, allocated at the first selection, in which the last kernel of a selection notes whether the
 *     peel kernel ordered the last front (for a selection of 8-byte fitness: whether its last front held more than
 *     8192 rows; for a large population whose matrix comes from the per-objective orders: whether front 0 held
 *     every row kept) -- the next selection of a like shape picks its launches by it (tunable "launch_memory"; 0 =
 *     never looked at).  Results never depend on any of it; the time of a call can, by a few microseconds (a first
 *     call, or calls whose last fronts alternate between small and large, take the other set of launches; with 8-byte
 *     fitness and a front of all of 20 000 rows the other set costs 0.7 ms more, once; so does, at 200 000 rows of
 *     eight objectives, the first selection with a short front 0 after two or more with a full one).
 *   - Fitness `f` is float32, addressed as f[i * stride_row + k * stride_col] (strides in elements),
 *     minimisation, n rows (individuals) by m columns (objectives).
 *   - The workspace must hold evox_hip_workspace_bytes(n, m) bytes, 256-byte aligned.  Calls that
 *     share a workspace must be ordered on one stream.
 */
#ifndef EVOX_HIP_H
#define EVOX_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define EVOX_HIP_ABI_VERSION 1

#define EVOX_HIP_E_BAD_ARG (-1)         /* null pointer, n < 1, m < 1, topk outside [1, n], ... */
#define EVOX_HIP_E_WORKSPACE (-2)       /* workspace too small or misaligned */
#define EVOX_HIP_E_BARRIER_TIMEOUT (-3) /* reported by evox_hip_read_status(): a bounded device-side wait ran out; the call's
                                           outputs then hold no partial result: ranks and orders -1, distances and fitness NaN,
                                           decision vectors all-ones bytes, first-front masks 0 */
#define EVOX_HIP_E_STATIC_LIMIT (-4)    /* the population needs more scratch than the library's own buffer holds */

int evox_hip_abi_version(void);

/* Bytes of workspace needed by every entry point below for an (n, m) population.  0 if the
 * arguments are invalid. */
size_t evox_hip_workspace_bytes(int64_t n, int64_t m);

/* rank_out[j] (int32, n entries) = non-domination rank of row j.
 * Replaces evox.operators.selection.non_dominate_rank
 * (src/evox/operators/selection/non_dominate.py:172-195, with dominate_relation :6-26,
 * the column sum :188 and the peeling loop :29-59, :161-169). */
int evox_hip_non_dominate_rank(const float* f, int64_t n, int64_t m, int64_t stride_row, int64_t stride_col,
                               int32_t* rank_out, void* workspace, size_t workspace_bytes, void* stream);

/* The same ranking, stopped after the front that holds the stop_count-th best row: rows of that front and of
 * the better ones get their rank, all others EVOX_HIP_RANK_UNSET.  It serves the callers that rank a merged
 * population only to cut it at a front, `worst = topk(rank, k, largest=False)[0][-1]; keep = rank <= worst`
 * (src/evox/algorithms/mo/nsga3.py:169-171 with k = pop_size + 1, src/evox/algorithms/mo/hype.py:135-138 with
 * k = pop_size): both statements give the same result on the truncated ranks, and the fronts behind the cut are
 * never peeled (C3 shape: 24 of 61 fronts). */
#define EVOX_HIP_RANK_UNSET 0x7FFFFFFF
int evox_hip_non_dominate_rank_until(const float* f, int64_t n, int64_t m, int64_t stride_row, int64_t stride_col,
                                     int64_t stop_count, int32_t* rank_out, void* workspace, size_t workspace_bytes,
                                     void* stream);

/* mask_out[j] (one byte per row, n entries) = 1 when no row dominates row j, else 0: the rows of rank 0,
 * without building the dominance matrix or peeling.  Replaces the pair
 * `rank = non_dominate_rank(all_fitness); ... [rank == 0]` of EvalMonitor.get_pf_fitness / get_pf
 * (src/evox/workflows/eval_monitor.py:301-302 and :333-335), which ranks the whole evaluation history only
 * to keep its first front.  Needs evox_hip_first_front_workspace_bytes(n, m) bytes of workspace (a few
 * arrays of n entries; a workspace of evox_hip_workspace_bytes(n, m) is also accepted). */
size_t evox_hip_first_front_workspace_bytes(int64_t n, int64_t m);
int evox_hip_first_front_mask(const float* f, int64_t n, int64_t m, int64_t stride_row, int64_t stride_col,
                              uint8_t* mask_out, void* workspace, size_t workspace_bytes, void* stream);

/* dist_out[j] (float32, n entries) = crowding distance of row j among the rows with mask[j] != 0,
 * -inf for the others.  `mask` is a byte per row at mask[j * mask_stride]; NULL selects every row.
 * Replaces evox.operators.selection.crowding_distance
 * (src/evox/operators/selection/non_dominate.py:198-231; ordering rules of
 * src/evox/utils/jit_fix_operator.py:246-252). */
int evox_hip_crowding_distance(const float* costs, int64_t n, int64_t m, int64_t stride_row, int64_t stride_col,
                               const uint8_t* mask, int64_t mask_stride, float* dist_out, void* workspace,
                               size_t workspace_bytes, void* stream);

/* The same distance for costs of 8-byte elements, which the reference also accepts (it computes the differences in
 * the costs' dtype and the quotients in torch's default float dtype, non_dominate.py:222-225): kind 0 = float64
 * costs, 1 = int64 costs (exact wrapping differences, divided as floats); out_kind 0 = float64 distances, 1 =
 * float32 (integer costs under a float32 default).  Strides in elements.  The per-objective orders
 * (jit_fix_operator.py:246-250) come from the stable argsort steps below on the halves of an order-preserving 64-bit
 * image of the cost.  Workspace: evox_hip_wide_workspace_bytes(n, m). */
size_t evox_hip_wide_workspace_bytes(int64_t n, int64_t m);
int evox_hip_crowding_distance_wide(const void* costs, int kind, int64_t n, int64_t m, int64_t stride_row, int64_t stride_col,
                                    const uint8_t* mask, int64_t mask_stride, void* dist_out, int out_kind, void* workspace,
                                    size_t workspace_bytes, void* stream);

/* The float32 image of such fitness that the ranking entry points take: dominance (non_dominate.py:6-26) only looks
 * at the order of the values inside an objective, so the ranks of fitness of any ordered dtype are the ranks of its
 * per-objective dense ranks.  sorted: (batch, m, n) values of kind 0 = float64 or 1 = int64, every row ascending
 * with NaN last; index: (batch, m, n) int64, the row that each value came from (what a sort of every objective
 * returns).  out: (batch, n, m) float32: the number of distinct values of the objective below the row's (-0.0 and
 * 0.0 are one value), NaN where the value is NaN; n below 2^24.  Nothing of this shape exists in the reference, which
 * compares the values themselves (:20-24); it stands in for those comparisons. */
int evox_hip_dense_rank_rows(const void* sorted, int kind, const int64_t* index, int64_t batch, int64_t n, int64_t m,
                             float* out, void* stream);

/* The selection steps after the ranking for such fitness (non_dominate.py:249-254): given rank (int32, n entries,
 * EVOX_HIP_RANK_UNSET behind the front that holds the topk-th row, as evox_hip_non_dominate_rank_until leaves them on
 * any order-preserving float32 image of the fitness), the distances of the rows of the largest set rank (the mask
 * rank == worst of :250-252), the order by (rank, distance descending with NaN last, row index) and the gathers:
 * out_x rows of x_row_bytes, out_f rows of f_row_bytes taken from f_rows (the caller's fitness rows as raw bytes, of
 * whatever dtype they have), out_rank int32, out_dist float64 (out_kind 0) or float32 (1).  costs / kind / strides as
 * above.  Workspace: evox_hip_wide_workspace_bytes(n, m). */
int evox_hip_nd_environmental_selection_wide(const void* x, int64_t x_row_bytes, int64_t x_row_stride_bytes, const void* f_rows,
                                             int64_t f_row_bytes, int64_t f_row_stride_bytes, const void* costs, int kind,
                                             int64_t n, int64_t m, int64_t stride_row, int64_t stride_col, const int32_t* rank,
                                             int64_t topk, void* out_x, void* out_f, int32_t* out_rank, void* out_dist,
                                             int out_kind, void* workspace, size_t workspace_bytes, void* stream);

/* The same for `batch` populations of one shape in the same launches (what a vmapped caller of the reference's
 * nd_environmental_selection gets, utils/op_register.py:26-51): x, f_rows and costs of population b lie
 * x_batch_stride_bytes, f_batch_stride_bytes and stride_batch elements further; rank is (batch, n), the outputs are
 * contiguous (batch, topk, ...) arrays.  workspace: batch copies of evox_hip_wide_workspace_bytes(n, m), each rounded
 * up to a multiple of 256 bytes; with a smaller one (at least one copy), more than 24 576 rows, or after a selection
 * of the shape whose last front held more than 8192 rows, the populations are taken one after the other. */
int evox_hip_many_nd_environmental_selection_wide(const void* x, int64_t x_row_bytes, int64_t x_row_stride_bytes,
                                                  int64_t x_batch_stride_bytes, const void* f_rows, int64_t f_row_bytes,
                                                  int64_t f_row_stride_bytes, int64_t f_batch_stride_bytes, const void* costs,
                                                  int kind, int64_t batch, int64_t n, int64_t m, int64_t stride_batch,
                                                  int64_t stride_row, int64_t stride_col, const int32_t* rank, int64_t topk,
                                                  void* out_x, void* out_f, int32_t* out_rank, void* out_dist, int out_kind,
                                                  void* workspace, size_t workspace_bytes, void* stream);

/* NSGA-II survivor selection: ranks f, takes the topk best rows by (rank ascending, crowding
 * distance within the last admitted front descending, row index ascending) and gathers them.
 *   x            decision vectors as raw bytes, row i at x + i * x_row_stride_bytes, x_row_bytes each
 *                (may be NULL together with out_x when only f / rank / distance are wanted)
 *   out_x        topk rows of x_row_bytes, contiguous
 *   out_f        (topk, m) float32 contiguous
 *   out_rank     topk int32
 *   out_dist     topk float32 (crowding distance; -inf for rows of better fronts than the last one)
 *   out_order    optional (may be NULL): the topk selected row indices, int32
 * Replaces evox.operators.selection.nd_environmental_selection
 * (src/evox/operators/selection/non_dominate.py:234-254). */
int evox_hip_nd_environmental_selection(const void* x, int64_t x_row_bytes, int64_t x_row_stride_bytes, const float* f,
                                        int64_t n, int64_t m, int64_t stride_row, int64_t stride_col, int64_t topk,
                                        void* out_x, float* out_f, int32_t* out_rank, float* out_dist,
                                        int32_t* out_order, void* workspace, size_t workspace_bytes, void* stream);

/* The same selection over a population that is given in two parts (rows 0..n_a-1 = part a, rows n_a.. = part
 * b), with the results exactly those of the entry point above on their concatenation.  Replaces, together
 * with it, the merge step of NSGA-II
 *     merge_pop = torch.cat([self.pop, offspring]); merge_fit = torch.cat([self.fit, off_fit])
 *     ... = nd_environmental_selection(merge_pop, merge_fit, self.pop_size)
 * (src/evox/algorithms/mo/nsga2.py:99-102): parents and offspring are read where they lie and the
 * concatenated copies are never made.  A part with no rows may pass NULL pointers.
 * Workspace: evox_hip_workspace_bytes(n_a + n_b, m). */
int evox_hip_nd_environmental_selection_two_part(const void* x_a, int64_t x_a_row_stride_bytes, const void* x_b,
                                                 int64_t x_b_row_stride_bytes, int64_t x_row_bytes, const float* f_a,
                                                 int64_t n_a, int64_t f_a_stride_row, int64_t f_a_stride_col,
                                                 const float* f_b, int64_t n_b, int64_t f_b_stride_row,
                                                 int64_t f_b_stride_col, int64_t m, int64_t topk, void* out_x, float* out_f,
                                                 int32_t* out_rank, float* out_dist, int32_t* out_order, void* workspace,
                                                 size_t workspace_bytes, void* stream);

/* The same selection for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc): no counterpart in the reference.  It takes no workspace: the scratch
 * memory is a buffer of EVOX_HIP_STATIC_SCRATCH_BYTES bytes that is part of the library's device image, one copy per
 * GPU, held until the process ends.  The call allocates and frees nothing.  Results are those of
 * evox_hip_nd_environmental_selection.  A population with evox_hip_workspace_bytes(n, m) >
 * EVOX_HIP_STATIC_SCRATCH_BYTES (about 14 000 rows of 3 objectives, 9800 of 16) is refused with
 * EVOX_HIP_E_STATIC_LIMIT.  All calls on one GPU share the buffer: calls on different streams of one GPU that
 * overlap in time race, the caller must order them. */
#define EVOX_HIP_STATIC_SCRATCH_BYTES (32u << 20)
int evox_hip_nd_environmental_selection_static(const void* x, int64_t x_row_bytes, int64_t x_row_stride_bytes,
                                               const float* f, int64_t n, int64_t m, int64_t stride_row, int64_t stride_col,
                                               int64_t topk, void* out_x, float* out_f, int32_t* out_rank, float* out_dist,
                                               int32_t* out_order, void* stream);

/* ---- many small populations at once (what the reference reaches through vmap: non_dominate.py:107-125
 * for the peeling, the rest of the path batching natively).  One workgroup per population, no workspace.
 * n <= evox_hip_batched_max_rows(m) (1024 rows for m <= 16, 4096 rows for m = 2, which has a kernel of its own that
 * builds no dominance matrix and takes populations of at least "two_small_min_rows" rows; 0 = unsupported); f is addressed as
 * f[b * stride_batch + i * stride_row + k * stride_col]; outputs are contiguous (batch, ...) arrays.
 * Per population the results equal those of the single-population entry points. */
int64_t evox_hip_batched_max_rows(int64_t m);
int evox_hip_batched_non_dominate_rank(const float* f, int64_t batch, int64_t n, int64_t m, int64_t stride_batch,
                                       int64_t stride_row, int64_t stride_col, int32_t* rank_out, void* stream);
int evox_hip_batched_nd_environmental_selection(const void* x, int64_t x_row_bytes, int64_t x_row_stride_bytes,
                                                int64_t x_batch_stride_bytes, const float* f, int64_t batch, int64_t n,
                                                int64_t m, int64_t stride_batch, int64_t stride_row, int64_t stride_col,
                                                int64_t topk, void* out_x, float* out_f, int32_t* out_rank, float* out_dist,
                                                void* stream);

/* ---- many populations of one shape, of any size (the same reference loop, non_dominate.py:107-125, and
 * utils/op_register.py:26-51, through which a vmapped caller reaches it -- problems/hpo_wrapper.py:214-223 maps whole
 * workflows).  The stages of the single-population pipeline run once for several populations at a time, each in
 * its own workgroups on its own copy of the workspace, wherever the kernels whose workgroups wait for each other
 * can all be resident with a share of the device each: populations of up to 32 768 rows whose bit matrix fits the
 * LDS of that share; of two objectives and more than 4096 rows, as many as have their chains of workgroups resident
 * together (two per compute unit, a workgroup to 3840 rows).  evox_hip_many_populations_per_launch says how many share a launch (1: the entry points below
 * then run the populations one after the other, which is always correct); evox_hip_many_workspace_bytes is the
 * workspace for it (that many single-population workspaces).  `stop_count` is the topk of the selection, or the
 * count of evox_hip_non_dominate_rank_until (n: every row is ranked).  Addressing as in evox_hip_batched_*; outputs
 * are contiguous (batch, ...) arrays; per population the results equal those of the single-population entry points. */
size_t evox_hip_many_workspace_bytes(int64_t batch, int64_t n, int64_t m, int64_t stop_count);
int64_t evox_hip_many_populations_per_launch(int64_t batch, int64_t n, int64_t m, int64_t stop_count);
int evox_hip_many_non_dominate_rank_until(const float* f, int64_t batch, int64_t n, int64_t m, int64_t stride_batch,
                                          int64_t stride_row, int64_t stride_col, int64_t stop_count, int32_t* rank_out,
                                          void* workspace, size_t workspace_bytes, void* stream);
int evox_hip_many_nd_environmental_selection(const void* x, int64_t x_row_bytes, int64_t x_row_stride_bytes,
                                             int64_t x_batch_stride_bytes, const float* f, int64_t batch, int64_t n, int64_t m,
                                             int64_t stride_batch, int64_t stride_row, int64_t stride_col, int64_t topk,
                                             void* out_x, float* out_f, int32_t* out_rank, float* out_dist, void* workspace,
                                             size_t workspace_bytes, void* stream);

/* The first-front mask and the crowding distances of many populations of one shape (evox_hip_first_front_mask and
 * evox_hip_crowding_distance under vmap / leading batch dimensions): the same launches for all of them where the
 * workspace for it (the query beside each) stays below 1 GiB, else in passes.  Masks and distances are contiguous
 * (batch, n) arrays; the optional input mask of the crowding distances is addressed as
 * mask[b * mask_batch_stride + i * mask_stride] (bytes). */
size_t evox_hip_many_first_front_workspace_bytes(int64_t batch, int64_t n, int64_t m);
int evox_hip_many_first_front_mask(const float* f, int64_t batch, int64_t n, int64_t m, int64_t stride_batch, int64_t stride_row,
                                   int64_t stride_col, uint8_t* mask_out, void* workspace, size_t workspace_bytes, void* stream);
size_t evox_hip_many_crowding_workspace_bytes(int64_t batch, int64_t n, int64_t m);
int evox_hip_many_crowding_distance(const float* costs, int64_t batch, int64_t n, int64_t m, int64_t stride_batch,
                                    int64_t stride_row, int64_t stride_col, const uint8_t* mask, int64_t mask_batch_stride,
                                    int64_t mask_stride, float* dist_out, void* workspace, size_t workspace_bytes, void* stream);

/* One small population given in two parts of equal strides (parents and offspring of NSGA-II,
 * src/evox/algorithms/mo/nsga2.py:99-102, at the population sizes such runs mostly have: a few hundred rows): the
 * selection of evox_hip_nd_environmental_selection_two_part in the one-workgroup kernel of the entry points above,
 * one launch and no workspace.  n_a, n_b >= 1, n_a + n_b <= evox_hip_batched_max_rows(m); both fitness parts are
 * addressed as f[i * stride_row + k * stride_col], both parts of x as rows of x_row_bytes bytes x_row_stride_bytes
 * apart.  Results equal those of the other entry points on the concatenation. */
int evox_hip_small_nd_environmental_selection_two_part(const void* x_a, const void* x_b, int64_t x_row_bytes,
                                                       int64_t x_row_stride_bytes, const float* f_a, int64_t n_a,
                                                       const float* f_b, int64_t n_b, int64_t m, int64_t stride_row,
                                                       int64_t stride_col, int64_t topk, void* out_x, float* out_f,
                                                       int32_t* out_rank, float* out_dist, void* stream);

/* out[r] (int64) = the winner of tournament r: among parents[r * tournament_size + 0 .. tournament_size-1]
 * (int64 candidate indices, values in [0, n_candidates)) the one that sorts first by the LAST key column of
 * fit, ties by the column before it, ..., ties by position in the tournament; NaN after every number.
 * fit is float32 (n_candidates, n_keys) addressed as fit[c * stride_row + k * stride_col].
 * Replaces the ordering step of evox.operators.selection.tournament_selection_multifit
 * (src/evox/operators/selection/tournament_selection.py:21-27; the random draw of `parents`, :21, stays in
 * torch so that the caller's generator is consumed exactly as before). */
int evox_hip_tournament_pick(const int64_t* parents, int64_t n_round, int64_t tournament_size, const float* fit,
                             int64_t n_candidates, int64_t n_keys, int64_t stride_row, int64_t stride_col, int64_t* out,
                             void* stream);

/* The same tournaments on the caller's list of key tensors as it is, without the stacked copy that
 * tournament_selection_multifit makes of it (tournament_selection.py:23: torch.stack(fitnesses, dim=1), with int32
 * ranks promoted to float32 beside float32 distances): keys, kinds and strides are HOST arrays of n_keys (1 .. 4)
 * entries, read during the call -- keys[k] a device pointer to n_candidates values stride[k] elements apart, kinds[k]
 * 0 for float32 and 1 for int32 (compared as the float32 it converts to, as after the stack).  The LAST key decides
 * first, as above. */
int evox_hip_tournament_pick_keys(const int64_t* parents, int64_t n_round, int64_t tournament_size, int64_t n_candidates,
                                  int64_t n_keys, const void* const* keys, const int32_t* kinds, const int64_t* strides,
                                  int64_t* out, void* stream);

/* One step of evox.utils.lexsort (src/evox/utils/jit_fix_operator.py:246-250): order_out = prev_order
 * rearranged by a stable ascending sort of key[prev_order[.]] (NaN after every number, -0.0 and 0.0 tied);
 * prev_order == NULL is the identity (the first key, :246).  Chaining one call per key, in the order of the
 * list, gives lexsort(keys) for a one-dimensional sort: the last key is primary, ties fall to the earlier
 * keys and then to the index.  kind: 0 float32 keys, 1 int32 keys, 2 uint32 keys; stride in elements;
 * order_out must not alias prev_order.  Workspace: evox_hip_argsort_workspace_bytes(n). */
size_t evox_hip_argsort_workspace_bytes(int64_t n);
int evox_hip_stable_argsort_step(const void* key, int kind, int64_t stride, int64_t n, const int32_t* prev_order,
                                 int32_t* order_out, void* workspace, size_t workspace_bytes, void* stream);

/* The same step for `batch` independent sorts of n positions each, which is lexsort along one dimension of
 * keys with more dimensions (jit_fix_operator.py:246-250 with dim, the shape tournament selection sorts in,
 * src/evox/operators/selection/tournament_selection.py:26): sort b reads key[b * batch_stride + i * stride]
 * (strides in elements; batch_stride may be negative only if the addressed elements stay inside the buffer),
 * prev_order + b * n and writes order_out + b * n.  Sorts of up to 8192 positions run together in one launch;
 * longer ones run one after the other on the stream.  Workspace: evox_hip_argsort_workspace_bytes(n). */
int evox_hip_stable_argsort_step_batched(const void* key, int kind, int64_t batch_stride, int64_t stride, int64_t batch,
                                         int64_t n, const int32_t* prev_order, int32_t* order_out, void* workspace,
                                         size_t workspace_bytes, void* stream);

/* Monte-Carlo hypervolume contributions of HypE (src/evox/algorithms/mo/hype.py:29-39, the part of cal_hv
 * after the samples are drawn): out[i] = scale * sum over the samples s that point i covers
 * (all_k fit[i,k] <= sample[s,k]) of alpha[max(c_s - 1, 0)], c_s = the number of points that cover s.
 * fit_t is (m, n) row-major (objectives by points), samples_t is (m, n_sample), alpha has n entries
 * (hype.py:14-24), scale = prod(ref - f_min) / n_sample (:38).  Workspace: evox_hip_hv_workspace_bytes. */
size_t evox_hip_hv_workspace_bytes(int64_t n, int64_t n_sample);
int evox_hip_hv_contributions(const float* fit_t, const float* samples_t, const float* alpha, int64_t n, int64_t m,
                              int64_t n_sample, float scale, float* out, void* workspace, size_t workspace_bytes,
                              void* stream);

/* Monte-Carlo hypervolume metric (src/evox/metrics/hv.py:18, the sample-against-points test after the samples
 * are drawn): out_count[0] = the number of samples s with some point i strictly greater in every objective
 * (all_k samples[s,k] < points[i,k]; a NaN on either side compares false).  points_t is (m, n) row-major,
 * samples_t is (m, n_sample); hv.py:19 turns the count into the estimate count / n_sample * prod(bound).
 * Workspace: evox_hip_hv_covered_workspace_bytes(n_sample). */
size_t evox_hip_hv_covered_workspace_bytes(int64_t n_sample);
int evox_hip_hv_covered_count(const float* points_t, const float* samples_t, int64_t n, int64_t m, int64_t n_sample,
                              int64_t* out_count, void* workspace, size_t workspace_bytes, void* stream);

/* No counterpart in the reference: launches `blocks` workgroups of 256 threads that issue, `iterations` times,
 * 16 independent v_add_f32 (kind 0), 16 independent v_cmp_le_f32 with SGPR results (kind 1), twice the
 * three-objective unit of the dominance kernel's compare form, 10 vector and 6 scalar instructions (kind 2), or
 * twice that of its arithmetic form, 12 vector instructions (kind 3).  The benchmark times it to report the
 * vector issue rates that the device sustains for the instruction kinds of the dominance kernel.
 * scratch_out: one float of device memory (never written in practice). */
int evox_hip_calibration_launch(int kind, int64_t blocks, int64_t iterations, float* scratch_out, void* stream);

/* ---- stages of the calls above, exposed so that each kernel can be tested and timed alone.
 * They operate on the state left in the workspace by the previous stage, in this order:
 *   prepare -> dominance -> count -> peel -> (crowding -> order -> gather).                                 */

/* Fitness -> structure-of-arrays copy + row keys, clears the small state, sorts the rows into slots
 * by key (a relabelling under which every dominator precedes the rows it dominates). */
int evox_hip_stage_prepare(const float* f, int64_t n, int64_t m, int64_t stride_row, int64_t stride_col, void* workspace,
                           size_t workspace_bytes, void* stream);
/* The pairwise dominance bit matrix (non_dominate.py:6-26) in slot space.  variant 0 = production
 * path (large finite populations: from the order of the rows in every objective; else pair by pair, by the signs
 * of differences when every value is finite, else by compares plus "differs somewhere" from a 32-bit stand-in of
 * the row key), 1 = check kernel that evaluates both `<=` and `<` per objective as the reference does, 2 = the
 * compare form on the 64-bit row keys themselves, 3 = the compare form whatever the values, 5 = only the
 * per-objective orders of the production path (an error where that path does not apply; for measurements). */
int evox_hip_stage_dominance(int64_t n, int64_t m, int variant, void* workspace, size_t workspace_bytes, void* stream);
/* Domination counts by row popcount (non_dominate.py:188) and front 0 (:192).  Resets the peeling
 * state first, so count -> peel can be repeated on one dominance matrix. */
int evox_hip_stage_count(int64_t n, int64_t m, void* workspace, size_t workspace_bytes, void* stream);
/* Front peeling (non_dominate.py:29-59, :161-169) until stop_count rows are ranked (stop_count = n
 * ranks every row).  rank_out may be NULL (ranks stay in the workspace). */
int evox_hip_stage_peel(int64_t n, int64_t m, int64_t stop_count, int32_t* rank_out, void* workspace,
                        size_t workspace_bytes, void* stream);
/* Crowding distance of the last peeled front (non_dominate.py:198-231 with mask = rank == worst). */
int evox_hip_stage_crowding(int64_t n, int64_t m, void* workspace, size_t workspace_bytes, void* stream);
/* Index-stable top-k on the last front + listing of the better fronts (non_dominate.py:253). */
int evox_hip_stage_order(int64_t n, int64_t m, void* workspace, size_t workspace_bytes, void* stream);

/* Byte offsets of the workspace regions, for tests and tools:
 *   out[0] dominance bit matrix (uint64, row j at + j * out[1] words)   out[1] row stride in words
 *   out[2] words per row in use      out[3] count (int32 n)             out[4] rank (int32 n)
 *   out[5] distance (float32 n)      out[6] rank-ordered listing (int32 n)
 *   out[7] front starts (int32 n+2)  out[8] selected order (int32 n)    out[9] control block
 *   out[10] slot -> original row index (int32 n)
 * The bit matrix and the counts are indexed by SLOT (rows relabelled by ascending row key, which makes
 * the matrix strictly lower triangular): bit b of word w of row s says that the row in slot 64 w + b
 * dominates the row in slot s.  Ranks, distances, listings and the order use original row indices. */
int evox_hip_workspace_layout(int64_t n, int64_t m, int64_t* out11);

/* Byte offsets of what the slot sort leaves, for tests: out[0] row keys by slot (uint64, out[4] entries: all-ones behind
 * the n-th), out[1] first slot that holds the same key (uint32, out[4] entries), out[2] fitness by slot as a structure of
 * arrays (float32, objective k at + k * out[4]; NaN behind the n-th row), out[3] fitness by original index, same shape,
 * out[4] padded row count, out[5] original row index -> slot (int32 n; written for populations of more than 4096 rows). */
int evox_hip_slot_sort_layout(int64_t n, int64_t m, int64_t* out6);

/* How a population of this shape is peeled, for tools and benchmarks: out[0] = 1 when every sweeping workgroup keeps
 * its rows of the bit matrix in LDS (the matrix fits the LDS of the device; counts and peeling are then one kernel),
 * 0 when rows are rescanned in memory; out[1] = sweeping workgroups of that kernel, out[2] = bytes of LDS of each
 * (both 0 when out[0] is 0).  Depends on the device that is current and on the tunables. */
int evox_hip_peel_plan(int64_t n, int64_t m, int64_t* out3);

/* How the dominance matrix of a population of this shape is built, for tools and benchmarks: out[1] = 1 when a finite
 * population gets it from the order of its rows in every objective (no pairwise test; out[0] is then 0), else out[0] =
 * words of a row that one wave of the pairwise kernel produces (it evaluates whole tiles of 64 rows x 64 out[0] slots on
 * or below the diagonal).  Depends on the tunables. */
int evox_hip_dominance_plan(int64_t n, int64_t m, int64_t* out2);

/* Waits for `stream`, then copies the control block's eight leading ints to HOST memory (workspace == NULL: those of
 * the library's own scratch buffer on the current device, i.e. of evox_hip_nd_environmental_selection_static):
 * out[0] error (0 or EVOX_HIP_E_BARRIER_TIMEOUT), out[1] fronts peeled, out[2] last front's rank,
 * out[3] rows in better fronts, out[4] last front's size, out[5] rows taken from it, out[6] sweep passes.
 * Returns out[0] when it is non-zero. */
int evox_hip_read_status(const void* workspace, void* stream, int32_t* host_out8);

/* Tunables (process-wide): "peel_lds" (1 = populations whose bit matrix fits the LDS of the device are peeled from LDS), "peel_lds_blocks"
 * (0 = by size, or 8 .. 255 sweeping workgroups of that kernel), "peel_tail" (1 = that kernel also orders a small last front), "tail_merged"
 * (1 = after such a peel the two ordering stages and the gather share one launch, up to three objectives), "launch_memory" (1 = ... unless
 * the last selection of that shape on the device had a last front that the peel kernel left to the ordering kernels, which a word of
 * pinned host memory tells: the library allocates 64 bytes of it per device at the first selection; 0 = never looked at),
 * "peel_blocks_per_cu" (default 2), "peel_witness" (1 = witness pass, 0 = popcount sweep), "peel_records" (1 = record
 * protocol, 0 = master barrier and front bitmaps), "peel_record_blocks" (0 = by size, or 16 .. 255), "spin_limit" (the bound of every device-side wait: a value above 65535 is a time in units of 10 ns on the device's constant clock, default 4000000 = 40 ms; a value up to 65535 counts failed polls, for tests that force a wait to give up), "two_small_min_rows" (default 128: from this many rows on, a population of two objectives that goes to a one-workgroup kernel takes the one without a dominance matrix, which also raises evox_hip_batched_max_rows(2) to 4096; 0 = never), "two_min_rows" (default 4097: smallest population of two objectives that is ranked without a dominance matrix -- rows sorted by (f1, f2, index), every front the strict prefix minima of f2 among the rows that remain; 0 = never) and "two_min_rows_partial" (default 4097: the same where the ranking may stop at a front, as in a selection; there the peeling ends once the fronts so far hold the rows asked for), "peel_stepped" (0 = the fronts are peeled by one persistent kernel where its grid can be resident at once, 1 = always by one launch per front and the last front by kernels that never wait for each other: slower, needs no co-residency, and waits for the stream between groups of sixteen launches), "dominance_tile_words" (0 = by size: 2 or 4; or 2, 4, 8, 16), "dominance_folded" (1 = only the blocks at or below the diagonal are launched; 0 = the whole rectangle), "mid_argsort" (1 = an argsort step of 8193 to 32768 positions, and a last front of 1025 to 32768 rows, are ordered by workgroups that sort in LDS without waiting for each other; 0 = the radix sort and ranking by counting), "small_sort" (1 = one-kernel slot sort up to 4096 rows),
 * "prefix_min_rows" (default 65536: smallest finite population of three objectives whose matrix is built from the per-objective orders -- a quarter more rows with two, fewer with more: 28672 at eight, 10240 at sixteen; 0 = never),
 * "prefix_bands" (default 1), "prefix_double_tile" (default 131072 rows, 0 = never), "prefix_mode" (default 3; 1 and 2 build only half of that kernel's output, for measurements),
 * "batched_stage" (default 1: the one-workgroup kernel reads the dominators of populations of at most 256 rows and eight objectives from a copy of the fitness in LDS when the launch holds no more populations than the device has compute units; 0 = by scalar loads from memory always),
 * "order_stream" (default 1: for more than 32768 rows those orders come from workgroups that read their objective's keys once and sort a share of the order in LDS, without waiting for each other, while shares of 3200 rows need no more workgroups than the device has compute units -- up to 102400 rows of eight objectives; 0 = from the radix sort, whose workgroups wait for each other twelve times), "order_stream_capacity" (default 16384, 1 .. 16384: entries that such a workgroup sorts at once; a larger share is taken in pieces -- tests make it small),
 * "prefix_count_first" (default 1: a selection of such a population whose last two of the same shape on the device found all the rows they keep in front 0 -- told by a word of the pinned host memory of "launch_memory" -- has that kernel count the dominators of every row first and build the matrix, in a second launch, only if front 0 falls short this time; 0 = always both at once).
 * Returns EVOX_HIP_E_BAD_ARG for an unknown name or a value out of range. */
int evox_hip_set_option(const char* name, int64_t value);

/* The same tunables for the calls of one thread, without touching process-wide state: a set of tunables is created
 * as a copy of the process-wide ones (NULL when memory runs out), changed by name like evox_hip_set_option, and
 * handed to evox_hip_options_use, after which every call that THIS thread makes into the library reads its tunables
 * from there, until the thread hands over another set or NULL (the process-wide ones again).  A set in use must
 * outlive the calls that read it; destroying the set that the calling thread uses puts that thread back on the
 * process-wide ones.  evox_hip_set_option remains for configuration at start-up. */
typedef struct evox_hip_options evox_hip_options;
evox_hip_options* evox_hip_options_create(void);
void evox_hip_options_destroy(evox_hip_options* options);
int evox_hip_options_set(evox_hip_options* options, const char* name, int64_t value);
int evox_hip_options_use(const evox_hip_options* options);

#ifdef __cplusplus
}
#endif
#endif /* EVOX_HIP_H */
