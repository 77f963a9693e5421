/* TEST INFRASTRUCTURE ONLY -- plain-C restatement of the reference's environmental selection for
 * populations where its dense formulation cannot allocate (N = 200000 needs a 40 GB bool matrix
 * plus two 320 GB temporaries, src/evox/operators/selection/non_dominate.py:16-24).
 *
 * Same algorithm as the reference, with the (N, N) bool matrix held as bits:
 *   dominance   A[i][j] = all_k x[i][k] <= x[j][k] and any_k x[i][k] < x[j][k]      non_dominate.py:6-26
 *   count[j]    = sum_i A[i][j]                                                      non_dominate.py:188
 *   peeling     rank[front] = level; count -= sum_{i in front} A[i][:]; count -= front;
 *               level += 1; front = count == 0, until the front is empty             non_dominate.py:29-59, 161-169
 *   crowding    per objective: stable sort of the masked rows by cost (NaN last), +inf for the first and
 *               last row of any objective, (next - prev) / (last - first) summed over objectives for the
 *               others, -inf outside the mask                                         non_dominate.py:198-231
 *   selection   order by (rank, -distance with NaN last, index), first topk          non_dominate.py:234-254
 *   first front rank == 0, i.e. "no row dominates it"                                 eval_monitor.py:301-302
 *
 * Pinned by tests/test_oracle_c.py against the torch restatement (itself pinned by brute force and by
 * the reference's golden vectors) on every small case.  Only tests/ may load this library.
 */
#include <math.h>
#include <omp.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

typedef uint64_t u64;

/* Threads that the parallel loops below run on (for reports of timings). */
int oracle_threads(void) { return omp_get_max_threads(); }

static int dominates(const float* a, const float* b, int m) {
  int lt = 0;
  for (int k = 0; k < m; ++k) {
    if (!(a[k] <= b[k])) return 0;
    lt |= a[k] < b[k];
  }
  return lt;
}

/* rank[j] for all rows.  Row j of `bits` lists the dominators of j.  Returns the number of fronts,
 * or -1 when memory runs out. */
int oracle_nd_rank(const float* f, int64_t n, int m, int32_t* rank) {
  const int64_t w = (n + 63) / 64;
  u64* bits = (u64*)calloc((size_t)n * (size_t)w, sizeof(u64));
  int64_t* count = (int64_t*)calloc((size_t)n, sizeof(int64_t));
  u64* front = (u64*)calloc((size_t)w, sizeof(u64));
  if (!bits || !count || !front) {
    free(bits); free(count); free(front);
    return -1;
  }
#pragma omp parallel for schedule(dynamic, 16)
  for (int64_t j = 0; j < n; ++j) {
    u64* row = bits + j * w;
    int64_t c = 0;
    for (int64_t i = 0; i < n; ++i)
      if (dominates(f + i * m, f + j * m, m)) {
        row[i >> 6] |= 1ull << (i & 63);
        ++c;
      }
    count[j] = c;
  }
  for (int64_t j = 0; j < n; ++j) rank[j] = 0;
  int level = 0;
  for (;;) {
    int any = 0;
    memset(front, 0, (size_t)w * sizeof(u64));
    for (int64_t j = 0; j < n; ++j)
      if (count[j] == 0) {
        front[j >> 6] |= 1ull << (j & 63);
        any = 1;
      }
    if (!any) break;
#pragma omp parallel for schedule(dynamic, 64)
    for (int64_t j = 0; j < n; ++j) {
      if ((front[j >> 6] >> (j & 63)) & 1) {
        rank[j] = level;
        count[j] -= 1; /* count -= front: ranked rows drop to -1 for good */
      } else if (count[j] > 0) {
        const u64* row = bits + j * w;
        int64_t c = 0;
        for (int64_t q = 0; q < w; ++q) c += __builtin_popcountll(row[q] & front[q]);
        count[j] -= c;
      }
    }
    ++level;
  }
  free(bits); free(count); free(front);
  return level;
}

/* mask[j] = 1 when no row dominates row j (the rows of rank 0: all that
 * src/evox/workflows/eval_monitor.py:301-302 keeps of the ranking), by direct search.  No matrix. */
int oracle_first_front(const float* f, int64_t n, int m, uint8_t* mask) {
#pragma omp parallel for schedule(dynamic, 256)
  for (int64_t j = 0; j < n; ++j) {
    uint8_t free_row = 1;
    for (int64_t i = 0; i < n && free_row; ++i)
      if (dominates(f + i * m, f + j * m, m)) free_row = 0;
    mask[j] = free_row;
  }
  return 0;
}

/* ---- stable ordering helpers: torch.argsort(stable=True) puts NaN last and ties by index */
typedef struct { float key; int64_t idx; } keyed;

static int cmp_keyed(const void* pa, const void* pb) {
  const keyed* a = (const keyed*)pa;
  const keyed* b = (const keyed*)pb;
  const int an = isnan(a->key), bn = isnan(b->key);
  if (an != bn) return an - bn;
  if (!an) {
    if (a->key < b->key) return -1;
    if (a->key > b->key) return 1;
  }
  return a->idx < b->idx ? -1 : (a->idx > b->idx ? 1 : 0);
}

/* dist[j] for all rows; mask may be NULL (every row). */
int oracle_crowding(const float* costs, int64_t n, int m, const uint8_t* mask, float* dist) {
  int64_t nv = 0;
  for (int64_t j = 0; j < n; ++j) nv += mask ? (mask[j] != 0) : 1;
  keyed* s = (keyed*)malloc((size_t)(nv > 0 ? nv : 1) * sizeof(keyed));
  float* part = (float*)calloc((size_t)n * (size_t)m, sizeof(float));
  uint8_t* boundary = (uint8_t*)calloc((size_t)n, 1);
  if (!s || !part || !boundary) {
    free(s); free(part); free(boundary);
    return -1;
  }
  for (int k = 0; k < m && nv > 0; ++k) {
    int64_t t = 0;
    for (int64_t j = 0; j < n; ++j)
      if (!mask || mask[j]) {
        s[t].key = costs[j * m + k];
        s[t].idx = j;
        ++t;
      }
    qsort(s, (size_t)nv, sizeof(keyed), cmp_keyed);
    const float span = s[nv - 1].key - s[0].key;
    boundary[s[0].idx] = 1;
    boundary[s[nv - 1].idx] = 1;
    for (int64_t p = 1; p + 1 < nv; ++p) part[s[p].idx * m + k] = (s[p + 1].key - s[p - 1].key) / span;
  }
  for (int64_t j = 0; j < n; ++j) {
    if (mask && !mask[j]) {
      dist[j] = -INFINITY;
    } else if (boundary[j]) {
      dist[j] = INFINITY;
    } else {
      float acc = 0.0f;
      for (int k = 0; k < m; ++k) acc = k == 0 ? part[j * m + k] : acc + part[j * m + k];
      dist[j] = acc;
    }
  }
  free(s); free(part); free(boundary);
  return 0;
}

typedef struct { int32_t rank; float negd; int64_t idx; } sel;

static int cmp_sel(const void* pa, const void* pb) {
  const sel* a = (const sel*)pa;
  const sel* b = (const sel*)pb;
  if (a->rank != b->rank) return a->rank < b->rank ? -1 : 1;
  const int an = isnan(a->negd), bn = isnan(b->negd);
  if (an != bn) return an - bn;
  if (!an) {
    if (a->negd < b->negd) return -1;
    if (a->negd > b->negd) return 1;
  }
  return a->idx < b->idx ? -1 : (a->idx > b->idx ? 1 : 0);
}

/* Full selection: rank (n), dist (n), order (topk).  Returns the number of fronts or a negative code. */
int oracle_select(const float* f, int64_t n, int m, int64_t topk, int32_t* rank, float* dist, int64_t* order) {
  if (topk < 1 || topk > n) return -2;
  const int fronts = oracle_nd_rank(f, n, m, rank);
  if (fronts < 0) return fronts;
  int32_t* sorted = (int32_t*)malloc((size_t)n * sizeof(int32_t));
  uint8_t* mask = (uint8_t*)malloc((size_t)n);
  sel* s = (sel*)malloc((size_t)n * sizeof(sel));
  if (!sorted || !mask || !s) {
    free(sorted); free(mask); free(s);
    return -1;
  }
  /* worst = topk-th smallest rank (counting sort over ranks) */
  int64_t* hist = (int64_t*)calloc((size_t)fronts + 1, sizeof(int64_t));
  for (int64_t j = 0; j < n; ++j) hist[rank[j]]++;
  int32_t worst = 0;
  for (int64_t acc = 0; worst < fronts; ++worst) {
    acc += hist[worst];
    if (acc >= topk) break;
  }
  free(hist);
  for (int64_t j = 0; j < n; ++j) mask[j] = rank[j] == worst;
  if (oracle_crowding(f, n, m, mask, dist) != 0) {
    free(sorted); free(mask); free(s);
    return -1;
  }
  for (int64_t j = 0; j < n; ++j) {
    s[j].rank = rank[j];
    s[j].negd = -dist[j];
    s[j].idx = j;
  }
  qsort(s, (size_t)n, sizeof(sel), cmp_sel);
  for (int64_t p = 0; p < topk; ++p) order[p] = s[p].idx;
  free(sorted); free(mask); free(s);
  return fronts;
}
