"""GPU parity: the HIP path (through the C ABI) against the CPU oracle and the golden vectors.

Tolerances (from the task statement): ranks bit-exact; crowding distance within 1e-5 relative on
finite values with infinities and NaN positions exact; selected order exact."""

import ctypes
import sys

import numpy as np
import pytest
import torch

from evox_amd import _lib, runtime, workloads
from evox_amd.operators.selection import (crowding_distance, nd_environmental_selection, nd_environmental_selection_two_part,
                                          non_dominate_rank)
from oracle import eager_restatement as er
from tests import golden_io
from tests.cases import as_np, edge_cases

pytestmark = pytest.mark.gpu

EDGE = edge_cases()
IDS = [c[0] for c in EDGE]
DEV = "cuda"


def say(*a):
    print(*a, flush=True, file=sys.stderr)


@pytest.fixture(autouse=True, params=["pipeline", "small-kernel"])
def population_path(request):
    """Every test runs twice: with small populations (<= 1024 rows, <= 16 objectives) served by the
    one-workgroup-per-population kernel, as in production, and with everything forced through the
    bit-matrix pipeline."""
    runtime.use_small_population_kernel = request.param == "small-kernel"
    yield request.param
    runtime.use_small_population_kernel = None


def assert_dist_close(got, want, what=""):
    got, want = as_np(got), as_np(want)
    assert got.shape == want.shape, what
    fin = np.isfinite(want)
    assert np.array_equal(np.isfinite(got), fin), what
    assert np.array_equal(np.isnan(got), np.isnan(want)), what
    assert np.array_equal(got[np.isinf(want)], want[np.isinf(want)]), what
    np.testing.assert_allclose(got[fin], want[fin], rtol=1e-5, atol=0, err_msg=what)


def run_stages(f, topk, variant=0):
    """dominance -> count -> peel through the stage entry points; returns the workspace views."""
    n, m = f.shape
    ws = runtime.workspace(n, m, f.device)
    s = runtime.stream_handle(f.device)
    _lib.call("evox_hip_stage_prepare", f.data_ptr(), n, m, f.stride(0), f.stride(1), ws.data_ptr(), ws.numel(), s)
    _lib.call("evox_hip_stage_dominance", n, m, variant, ws.data_ptr(), ws.numel(), s)
    _lib.call("evox_hip_stage_count", n, m, ws.data_ptr(), ws.numel(), s)
    _lib.call("evox_hip_stage_peel", n, m, topk, None, ws.data_ptr(), ws.numel(), s)
    runtime.note_call(ws, s)
    status = runtime.last_status()
    return runtime.workspace_views(ws, n, m), status


def defined_words(n, nwords):
    """1 where word w of the row of slot j is written by the dominance kernel: w < 2 * (j // 128 + 1).
    Words beyond that lie above the diagonal, are never stored and never read."""
    limit = 2 * (np.arange(n) // 128 + 1)
    return (np.arange(nwords)[None, :] < limit[:, None]).astype(np.uint8)


def unpack_bits(views, n):
    """Workspace bit matrix (slot space) -> bool (n, n) in ORIGINAL indices with [j, i] = i dominates j.
    Also checks the slot properties: a permutation, and nothing on or above the diagonal."""
    words = np.ascontiguousarray(as_np(views["dom"])[:, : views["nwords"]]).view(np.uint64)  # words in use
    words = words.copy()
    words[defined_words(words.shape[0], words.shape[1]) == 0] = 0
    bits = np.unpackbits(words.view(np.uint8), axis=1, bitorder="little")
    assert not bits[:, n:].any()  # padding columns
    bits = bits[:, :n].astype(bool)
    assert not np.triu(bits).any()  # strictly lower triangular in slot space
    orig = as_np(views["orig_of"]).astype(np.int64)
    assert np.array_equal(np.sort(orig), np.arange(n))
    out = np.zeros((n, n), dtype=bool)
    out[np.ix_(orig, orig)] = bits
    return out


# ------------------------------------------------------------ dominance bits


@pytest.mark.parametrize("variant", [0, 1, 2, 3])
@pytest.mark.parametrize("name,f,ks", EDGE, ids=IDS)
def test_dominance_bits_edge(name, f, ks, variant):
    say("dominance_bits", name, "variant", variant, tuple(f.shape))
    fd = f.to(DEV)
    n, m = f.shape
    ws = runtime.workspace(n, m, fd.device)
    s = runtime.stream_handle(fd.device)
    _lib.call("evox_hip_stage_prepare", fd.data_ptr(), n, m, fd.stride(0), fd.stride(1), ws.data_ptr(), ws.numel(), s)
    _lib.call("evox_hip_stage_dominance", n, m, variant, ws.data_ptr(), ws.numel(), s)
    _lib.call("evox_hip_stage_count", n, m, ws.data_ptr(), ws.numel(), s)
    torch.cuda.synchronize()
    views = runtime.workspace_views(ws, n, m)
    got = unpack_bits(views, n)  # [j, i] = i dominates j
    want = as_np(er.pareto_dominance(f, f))
    assert np.array_equal(got, want.T)
    orig = as_np(views["orig_of"]).astype(np.int64)
    assert np.array_equal(as_np(views["count"]), want.sum(axis=0)[orig])  # non_dominate.py:188, by slot
    _lib.call("evox_hip_stage_peel", n, m, n, None, ws.data_ptr(), ws.numel(), s)
    runtime.note_call(ws, s)
    assert runtime.last_status()["error"] == 0
    assert np.array_equal(as_np(views["rank"]), as_np(er.ranks_by_peeling(f)))


@pytest.mark.parametrize("m", [1, 2, 3, 4, 5, 6, 7, 8, 9, 12, 16, 17])
def test_dominance_bits_all_m(m):
    say("dominance_bits_all_m", m)
    g = torch.Generator("cpu").manual_seed(40 + m)
    finite = (torch.randint(0, 3 + m, (333, m), generator=g).float() / 4.0).contiguous()
    other = finite.clone()  # with values that are not finite: the kernels then take the compare form
    other[torch.rand(333, m, generator=g) < 0.02] = float("nan")
    other[torch.rand(333, m, generator=g) < 0.02] = float("inf")
    other[torch.rand(333, m, generator=g) < 0.02] = -float("inf")
    for f in (finite, other):
        n = f.size(0)
        fd = f.to(DEV)
        ws = runtime.workspace(n, m, fd.device)
        s = runtime.stream_handle(fd.device)
        want = as_np(er.pareto_dominance(f, f)).T
        for variant in ([0, 1, 2, 3] if m <= 8 else [0, 1]):
            _lib.call("evox_hip_stage_prepare", fd.data_ptr(), n, m, fd.stride(0), fd.stride(1), ws.data_ptr(), ws.numel(), s)
            _lib.call("evox_hip_stage_dominance", n, m, variant, ws.data_ptr(), ws.numel(), s)
            torch.cuda.synchronize()
            got = unpack_bits(runtime.workspace_views(ws, n, m), n)
            assert np.array_equal(got, want), (m, variant, bool(torch.isfinite(f).all()))


@pytest.mark.parametrize("n,m", [(65535, 3), (65536, 3), (65537, 4), (65664, 8), (81919, 2), (81920, 2), (70001, 10), (49151, 9), (49152, 16), (66000, 17),
                                 (45055, 5), (45056, 4), (40960, 6), (36863, 7), (28671, 8), (28672, 8), (32768, 8), (18431, 9), (18432, 10),
                                 (14336, 12), (12288, 14), (10239, 16), (10240, 16), (24577, 16)])
def test_ranks_across_the_switch_to_the_order_based_matrix(n, m):
    """Populations just below and above the size at which the matrix comes from the per-objective orders -- 65 536 rows
    of three objectives, fewer with more objectives, down to 10 240 of sixteen -- and 65536 rows, where the padded
    column length steps off a multiple of 4096: same ranks and same selection whichever kernel builds the matrix, and
    both the ranks and the selection of the plain-C checker."""
    from oracle import c_oracle

    say("switch", n, m)
    g = torch.Generator("cpu").manual_seed(n + m)
    f_cpu = torch.randint(0, 1 << 12, (n, m), generator=g).float() / 64  # ties in every objective
    f = f_cpu.to(DEV)
    x = torch.arange(n, dtype=torch.int32, device=DEV)[:, None]
    try:
        got_rank = non_dominate_rank(f)
        got = nd_environmental_selection(x, f, n // 2)
        order, rank, dist, _ = c_oracle.select(as_np(f_cpu), n // 2)
        assert np.array_equal(as_np(got_rank), rank)
        assert np.array_equal(as_np(got[0])[:, 0].astype(np.int64), order)
        assert np.array_equal(as_np(got[2]), rank[order])
        assert_dist_close(got[3], dist[order])
        with runtime.options(prefix_min_rows=0):
            assert torch.equal(got_rank, non_dominate_rank(f))
            want = nd_environmental_selection(x, f, n // 2)
        assert all(torch.equal(a, b) for a, b in zip(got, want))
    finally:
        runtime.release_workspaces()


def _matrix_words(f, variant, views_out=None):
    """Raw words of the bit matrix (slot space) that readers look at, after prepare + dominance."""
    n, m = f.shape
    fd = f.to(DEV)
    ws = runtime.workspace(n, m, fd.device)
    s = runtime.stream_handle(fd.device)
    _lib.call("evox_hip_stage_prepare", fd.data_ptr(), n, m, fd.stride(0), fd.stride(1), ws.data_ptr(), ws.numel(), s)
    _lib.call("evox_hip_stage_dominance", n, m, variant, ws.data_ptr(), ws.numel(), s)
    _lib.call("evox_hip_stage_count", n, m, ws.data_ptr(), ws.numel(), s)
    torch.cuda.synchronize()
    views = runtime.workspace_views(ws, n, m)
    words = np.ascontiguousarray(as_np(views["dom"])[:, : views["nwords"]]).view(np.uint64).copy()
    words[defined_words(words.shape[0], words.shape[1]) == 0] = 0
    if views_out is not None:
        views_out.update({k: as_np(views[k]).copy() for k in ("count", "rank")})
    return words


@pytest.mark.parametrize("m", [2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 13, 16])
def test_matrix_from_objective_orders_equals_the_pairwise_matrix(m):
    """Large finite populations get their matrix from the order of the rows in every objective; it must be
    the matrix of the pairwise test, word for word: ties, duplicate rows, constant objectives, a population
    whose rows are all equal, signed zeros; and a NaN or an infinity hands the work back to the pairwise kernel."""
    g = torch.Generator("cpu").manual_seed(700 + m)
    cases = {}
    cases["uniform"] = torch.rand(12345, m, generator=g)
    cases["ties"] = torch.randint(0, 40, (9000, m), generator=g).float() / 8 - 2
    dup = torch.rand(3000, m, generator=g)
    cases["duplicates"] = dup[torch.randint(0, 3000, (8500,), generator=g)]
    cases["all_equal"] = torch.full((8300, m), 1.5)
    const = torch.rand(8400, m, generator=g)
    const[:, m - 1] = -0.0
    const[::3, m - 1] = 0.0
    cases["constant_objective_signed_zeros"] = const
    front = torch.rand(8200, m, generator=g)
    front = front / front.sum(dim=1, keepdim=True)
    cases["one_front"] = front
    chain = torch.arange(8193, dtype=torch.float32)[:, None].repeat(1, m)
    cases["chain"] = chain[torch.randperm(8193, generator=g)]
    nan = torch.rand(8600, m, generator=g)
    nan[17, 0] = float("nan")
    nan[4000, m - 1] = float("inf")
    cases["nonfinite"] = nan
    cases["large"] = torch.rand(40000, m, generator=g)
    for name, f in cases.items():
        say("prefix_matrix", m, name, tuple(f.shape))
        want_state = {}
        with runtime.options(prefix_min_rows=0):
            want = _matrix_words(f.contiguous(), 0, want_state)
        # up to four objectives also with both tiles of a 128-byte line in one workgroup (by default from 131072 rows on)
        for double_from in (131072, 1) if m <= 4 else (131072,):
            with runtime.options(prefix_min_rows=4097, prefix_double_tile=double_from):  # (a quarter more rows with two objectives)
                got_state = {}
                got = _matrix_words(f.contiguous(), 0, got_state)
            assert np.array_equal(got, want), (m, name, double_from, int((got != want).sum()))
            if double_from == 1:
                assert np.array_equal(got_state["count"], want_state["count"]), (m, name)
        # the counts and front 0 that the count stage derives from what the order-based kernel left behind
        assert np.array_equal(got_state["count"], want_state["count"]), (m, name)
        assert np.array_equal(got_state["count"], np.bitwise_count(want).sum(axis=1)), (m, name)
        assert np.array_equal(got_state["rank"], want_state["rank"]), (m, name)
        if name in ("ties", "duplicates", "large"):  # and the whole ranking on top of them (the passes start from
            fd = f.contiguous().to(DEV)              # the highest non-empty word of every row)
            with runtime.options(prefix_min_rows=4097):
                ranks = non_dominate_rank(fd)
            with runtime.options(prefix_min_rows=0):
                assert torch.equal(ranks, non_dominate_rank(fd)), (m, name)


@pytest.mark.parametrize("m", [2, 3, 5, 8, 16])
def test_objective_orders_of_more_than_32768_rows(m):
    """Above 32 768 rows the per-objective orders come from workgroups that read their objective's keys once and sort a
    share of the order in LDS (the shares are cut between members of a sorted sample).  The matrix built from them
    must be that of the radix sort's orders, word for word: uniform values, few distinct values, a constant objective,
    values with the period of the sample, and a crowd of equal values that the sample does not see (a share too large
    for the workgroup's LDS, taken in pieces); then the same with room for 700 entries only, so that every share is
    taken in pieces."""
    n = 36000
    g = torch.Generator("cpu").manual_seed(800 + m)
    cases = {}
    cases["uniform"] = torch.rand(n, m, generator=g)
    cases["few_values"] = torch.randint(0, 7, (n, m), generator=g).float()
    const = torch.rand(n, m, generator=g)
    const[:, 0] = 3.0
    cases["constant_objective"] = const
    period = torch.rand(n, m, generator=g)
    period[:, m - 1] = (torch.arange(n) % 2048).float()  # (the sample takes every (n / 2048)-th row)
    cases["periodic"] = period
    hidden = torch.zeros(n, m)
    hidden[:, 0] = torch.rand(n, generator=g)
    seen = (torch.arange(2048) * n) // 2048  # the rows of the sample: the only ones that differ in the last objective
    hidden[seen, m - 1] = 1.0 + torch.rand(2048, generator=g)
    cases["crowd_hidden_from_the_sample"] = hidden
    for name, f in cases.items():
        say("stream_orders", m, name)
        with runtime.options(prefix_min_rows=4097, order_stream=0):
            want_state = {}
            want = _matrix_words(f.contiguous(), 0, want_state)
        for capacity in (16384, 700):
            with runtime.options(prefix_min_rows=4097, order_stream=1, order_stream_capacity=capacity):
                got_state = {}
                got = _matrix_words(f.contiguous(), 0, got_state)
            assert np.array_equal(got, want), (m, name, capacity, int((got != want).sum()))
            assert np.array_equal(got_state["count"], want_state["count"]), (m, name, capacity)
            assert np.array_equal(got_state["rank"], want_state["rank"]), (m, name, capacity)
        del want, got
    # the sorted pairs stay behind for the ordering of a large last front: a selection out of one front
    from oracle import c_oracle

    front = cases["uniform"] / cases["uniform"].sum(dim=1, keepdim=True)
    order, rank, dist, _ = c_oracle.select(as_np(front), n // 2)
    x = torch.arange(n, dtype=torch.int32, device=DEV)[:, None]
    for capacity in (16384, 700):
        with runtime.options(prefix_min_rows=4097, order_stream_capacity=capacity):
            xs, fs, rs, ds = nd_environmental_selection(x, front.to(DEV), n // 2)
        assert runtime.last_status()["error"] == 0
        assert np.array_equal(as_np(rs), rank[order])
        assert_dist_close(ds, dist[order], "stream orders")
        if m in (2, 3, 8):
            assert np.array_equal(as_np(xs)[:, 0].astype(np.int64), order)
    runtime.release_workspaces()


@pytest.mark.parametrize("m", [1, 2, 3, 4, 6, 8, 11, 16])
def test_dominance_arithmetic_form_corner_values(m):
    """A population of finite values takes the arithmetic form of the dominance test (signs of differences):
    denormal differences, differences that overflow, signed zeros, huge and tiny magnitudes, duplicates."""
    say("dominance_arith", m)
    g = torch.Generator("cpu").manual_seed(60 + m)
    tiny = torch.tensor([0.0, -0.0, 1.4e-45, -1.4e-45, 2.8e-45, 1.17549435e-38, 1.17549421e-38, -1.17549435e-38])
    huge = torch.tensor([3.4028235e38, -3.4028235e38, 3.4028233e38, 1e38, -1e38, 1.0, -1.0, 1.0000001])
    pool = torch.cat([tiny, huge])
    f = pool[torch.randint(0, pool.numel(), (700, m), generator=g)].contiguous()
    assert bool(torch.isfinite(f).all())
    n = f.size(0)
    fd = f.to(DEV)
    ws = runtime.workspace(n, m, fd.device)
    s = runtime.stream_handle(fd.device)
    want = as_np(er.pareto_dominance(f, f)).T
    for variant in (0, 1):
        _lib.call("evox_hip_stage_prepare", fd.data_ptr(), n, m, fd.stride(0), fd.stride(1), ws.data_ptr(), ws.numel(), s)
        _lib.call("evox_hip_stage_dominance", n, m, variant, ws.data_ptr(), ws.numel(), s)
        torch.cuda.synchronize()
        assert np.array_equal(unpack_bits(runtime.workspace_views(ws, n, m), n), want), (m, variant)
    assert np.array_equal(as_np(non_dominate_rank(fd)), as_np(er.ranks_by_peeling(f)))
    # one infinity anywhere switches the whole population to the compare form: same answers
    f2 = f.clone()
    f2[3, 0] = float("inf")
    f2[9, m - 1] = -float("inf")
    assert np.array_equal(as_np(non_dominate_rank(f2.to(DEV))), as_np(er.ranks_by_peeling(f2)))


def test_dominance_variants_agree_c3():
    say("dominance_variants_agree_c3")
    w = workloads.c3()
    fd = w.f.to(DEV)
    n, m = fd.shape
    ws = runtime.workspace(n, m, fd.device)
    s = runtime.stream_handle(fd.device)
    doms = []
    for variant in (0, 1, 2, 3):
        _lib.call("evox_hip_stage_prepare", fd.data_ptr(), n, m, fd.stride(0), fd.stride(1), ws.data_ptr(), ws.numel(), s)
        _lib.call("evox_hip_stage_dominance", n, m, variant, ws.data_ptr(), ws.numel(), s)
        v = runtime.workspace_views(ws, n, m)
        keep = torch.from_numpy(defined_words(n, v["nwords"])).to(DEV).bool()
        doms.append(torch.where(keep, v["dom"][:, : v["nwords"]], 0))
    assert torch.equal(doms[0], doms[1]) and torch.equal(doms[0], doms[2]) and torch.equal(doms[0], doms[3])
    # popcount of the whole matrix = dominated ordered pairs; 12.3% of N^2 (2^-3 for three independent uniform objectives)
    sample = doms[0][::50]  # every 50th slot
    dens = float(sum(bin(int(x) & (2**64 - 1)).count("1") for x in sample.flatten().tolist())) / (sample.size(0) * n)
    assert abs(dens - 0.125) < 0.02


# ---------------------------------------------------------------------- rank


@pytest.mark.parametrize("name,f,ks", EDGE, ids=IDS)
def test_rank_edge(name, f, ks):
    say("rank", name, tuple(f.shape))
    got = non_dominate_rank(f.to(DEV))
    assert got.dtype == torch.int32 and got.device.type == "cuda"
    assert np.array_equal(as_np(got), as_np(er.ranks_by_peeling(f)))
    assert runtime.last_status()["error"] == 0


def test_both_slot_sorts_on_small_and_mid_size_inputs(population_path):
    """Populations of at most 4096 rows are put in slot order by one kernel, larger ones by the bucket sort;
    here the bucket sort also gets the small inputs (every edge case, the tie-heavy layered configuration,
    two-part input), and both must give the ranks and the selection of the restatement."""
    if population_path != "pipeline":
        pytest.skip("about the bit-matrix pipeline")
    say("slot_sorts")
    cases = [(name, f) for name, f, _ in EDGE]
    cases.append(("c2", workloads.c2().f))
    cases.append(("uniform-4096x4", workloads.uniform_population(4096, 4, 0, 21)[0]))
    cases.append(("uniform-4097x2", workloads.uniform_population(4097, 2, 0, 22)[0]))
    cases.append(("wide-60x200", workloads.uniform_population(60, 200, 0, 23)[0]))   # keys near 2^40
    cases.append(("wide-40x300", workloads.uniform_population(40, 300, 0, 24)[0]))   # too wide for the one-kernel sort
    for small_sort in (0, 1):
        with runtime.options(small_sort=small_sort):
            for name, f in cases:
                want = er.ranks_by_peeling(f)
                assert np.array_equal(as_np(non_dominate_rank(f.to(DEV))), as_np(want)), (small_sort, name)
                assert runtime.last_status()["error"] == 0
                n = f.size(0)
                if n >= 2:
                    topk = max(1, n // 2)
                    picked, _, _, order = er.environmental_selection(f, f, topk, return_all=True)
                    h = n // 3
                    got = nd_environmental_selection_two_part(f[:h].to(DEV), f[:h].to(DEV), f[h:].to(DEV), f[h:].to(DEV), topk)
                    assert np.array_equal(as_np(got[0]), as_np(f)[as_np(order)], equal_nan=True), (small_sort, name)
                    assert np.array_equal(as_np(got[2]), as_np(picked[2])), (small_sort, name)


def test_rank_strided_and_half_inputs():
    say("rank_strided")
    g = torch.Generator("cpu").manual_seed(3)
    base = torch.rand(150, 7, generator=g)
    f = base[:, 1:6:2]  # non-contiguous view, M = 3
    assert np.array_equal(as_np(non_dominate_rank(f.to(DEV)[:, :])), as_np(er.ranks_by_peeling(f.contiguous())))
    fd = base.to(DEV)[:, 1:6:2]
    assert not fd.is_contiguous()
    assert np.array_equal(as_np(non_dominate_rank(fd)), as_np(er.ranks_by_peeling(f.contiguous())))
    ft = base.t().contiguous().t()[:, :4]  # column-major
    assert np.array_equal(as_np(non_dominate_rank(ft.to(DEV))), as_np(er.ranks_by_peeling(ft.contiguous())))
    h = base[:, :3].half()
    assert np.array_equal(as_np(non_dominate_rank(h.to(DEV))), as_np(er.ranks_by_peeling(h.float())))


@pytest.fixture(params=["lds", "witness-records", "witness-master", "sweep", "stepped"])
def peel_algorithm(request):
    """The peeling variants: matrix rows resident in LDS (default where the matrix fits), the three that rescan
    rows in memory: witness pass with the record protocol, witness pass with the master barrier and front
    bitmaps, and the popcount-decrement sweep (master barrier); and one launch per front by a kernel whose workgroups
    never wait for each other (with the last front of a selection ordered likewise)."""
    with runtime.options(peel_lds=1 if request.param == "lds" else 0, peel_witness=0 if request.param == "sweep" else 1,
                         peel_records=1 if request.param == "witness-records" else 0,
                         peel_stepped=1 if request.param == "stepped" else 0):
        yield request.param


@pytest.mark.parametrize("name", ["C1", "C2", "C2p", "C3"])
def test_rank_configs_golden(name, peel_algorithm):
    say("rank_config", name, peel_algorithm)
    w, g = golden_io.config(name)
    got = non_dominate_rank(w.f.to(DEV))
    assert np.array_equal(as_np(got), g["rank"])
    st = runtime.last_status()
    assert st["error"] == 0 and st.get("fronts", int(g["rank"].max()) + 1) == int(g["rank"].max()) + 1


def test_rank_batched_c4_and_vmap():
    say("rank_c4_first8")
    w, g = golden_io.c4_first8()
    fd = w.f[:8].to(DEV)
    assert np.array_equal(as_np(non_dominate_rank(fd[0])), g["rank"][0])
    got = torch.vmap(non_dominate_rank)(fd)
    assert np.array_equal(as_np(got), g["rank"])
    nested = torch.vmap(torch.vmap(non_dominate_rank))(fd.view(2, 4, *fd.shape[1:]))
    assert np.array_equal(as_np(nested).reshape(8, -1), g["rank"])


def test_rank_compile_vmap_consistency():
    """The reference's own test of this operator (unit_test/operators/test_non_dominate.py:9-26):
    eager == compile == compile(vmap) == compile(vmap(vmap))."""
    say("rank_compile_vmap")
    f = torch.randn(12, 3, generator=torch.Generator("cpu").manual_seed(5)).to(DEV)
    rank = non_dominate_rank(f)
    assert np.array_equal(as_np(rank), as_np(er.ranks_by_peeling(f.cpu())))
    assert torch.equal(torch.compile(non_dominate_rank, fullgraph=True)(f), rank)
    got = torch.compile(torch.vmap(non_dominate_rank))(torch.stack([f] * 5))
    assert torch.equal(got, torch.stack([rank] * 5))
    got = torch.compile(torch.vmap(torch.vmap(non_dominate_rank)))(torch.stack([torch.stack([f] * 5)] * 3))
    assert torch.equal(got, torch.stack([torch.stack([rank] * 5)] * 3))


def test_rank_medium_shapes_against_oracle(peel_algorithm):
    for n, m, seed in [(1000, 2, 1), (1500, 3, 2), (777, 5, 3), (2049, 4, 4), (640, 8, 5), (500, 10, 6)]:
        say("rank_medium", n, m)
        f = workloads.uniform_population(n, m, 0, seed)[0]
        assert np.array_equal(as_np(non_dominate_rank(f.to(DEV))), as_np(er.ranks_by_peeling(f)))
    chain = torch.arange(300, dtype=torch.float32)[:, None].repeat(1, 2)  # 300 fronts of one row
    assert as_np(non_dominate_rank(chain.to(DEV))).tolist() == list(range(300))
    assert runtime.last_status().get("fronts", 300) == 300


# ------------------------------------------------------------------ crowding


def _masks_for(n, seed):
    g = torch.Generator("cpu").manual_seed(seed)
    out = [torch.ones(n, dtype=torch.bool), torch.rand(n, generator=g) < 0.5, torch.rand(n, generator=g) < 0.15]
    one = torch.zeros(n, dtype=torch.bool)
    one[n // 2] = True
    out.append(one)
    return out


@pytest.fixture(scope="module")
def edge_golden():
    return golden_io.load("edge_cases.npz")


@pytest.mark.parametrize("name,f,ks", EDGE, ids=IDS)
def test_crowding_edge_golden(edge_golden, name, f, ks):
    say("crowding", name)
    fd = f.to(DEV)
    got = crowding_distance(fd, None)
    assert got.dtype == torch.float32 and got.device.type == "cuda"
    assert_dist_close(got, edge_golden[f"{name}/cd_none"], name)
    for t in range(4):
        mask = torch.from_numpy(edge_golden[f"{name}/mask{t}"])
        assert_dist_close(crowding_distance(fd, mask.to(DEV)), edge_golden[f"{name}/cd_mask{t}"], f"{name} mask{t}")
    empty = torch.zeros(f.size(0), dtype=torch.bool, device=DEV)
    assert np.isneginf(as_np(crowding_distance(fd, empty))).all()


def test_crowding_medium_against_oracle():
    for n, m, seed in [(3000, 3, 1), (5000, 2, 2), (1200, 8, 3), (999, 5, 4)]:
        say("crowding_medium", n, m)
        f = workloads.uniform_population(n, m, 0, seed)[0]
        for mask in _masks_for(n, seed):
            assert_dist_close(crowding_distance(f.to(DEV), mask.to(DEV)), er.crowding(f, mask), f"{n}x{m}")
    grid = workloads.layered_grid_population(20, 100, 7)  # heavy ties
    for mask in _masks_for(2000, 9):
        assert_dist_close(crowding_distance(grid.to(DEV), mask.to(DEV)), er.crowding(grid, mask), "grid")


def test_large_front_uses_radix_sort():
    """Fronts above 4096 rows are ordered by the segmented radix sort instead of counting: a
    many-objective population whose first front holds most rows, and the crowding distance of a
    whole 9000-row population with heavy ties."""
    say("large_front_radix")
    f = workloads.sphere_shell_population((9000,), 6, 0.05, seed=12)
    x = torch.arange(9000, dtype=torch.float32)[:, None].repeat(1, 3)
    (_, _, _, _), rank, dist, order = er.environmental_selection(x, f, 4500, return_all=True)
    assert int((rank == 0).sum()) > 4096  # the last admitted front is front 0 and it is large
    check_selection(f, x, 4500, as_np(rank), as_np(dist), as_np(order), "sphere 9000x6")
    assert runtime.last_status()["last_front_size"] > 4096
    g = torch.Generator("cpu").manual_seed(99)
    ties = (torch.randint(0, 50, (9000, 3), generator=g).float() / 50.0).contiguous()
    assert_dist_close(crowding_distance(ties.to(DEV), None), er.crowding(ties, None), "ties 9000x3")
    mask = torch.rand(9000, generator=g) < 0.7
    assert_dist_close(crowding_distance(ties.to(DEV), mask.to(DEV)), er.crowding(ties, mask), "ties masked")


def test_large_front_with_more_objectives_than_one_sort_launch_takes():
    """The radix path orders at most 16 objectives per launch: 17 to 70 objectives on 9000 rows, whole
    population and a masked part, and a selection whose last front is large."""
    say("large_front_many_objectives")
    g = torch.Generator("cpu").manual_seed(123)
    for m in (17, 24, 33, 70):
        f = (torch.randint(0, 200, (9000, m), generator=g).float() / 16.0).contiguous()
        assert_dist_close(crowding_distance(f.to(DEV), None), er.crowding(f, None), f"9000x{m}")
        mask = torch.rand(9000, generator=g) < 0.95
        assert_dist_close(crowding_distance(f.to(DEV), mask.to(DEV)), er.crowding(f, mask), f"9000x{m} masked")
    # a selection out of one large front.  The sum of 40 terms is associated differently from torch's (tolerance
    # 1e-5 on the distance), so rows whose distances nearly tie may swap: the order is checked through what defines it
    f = torch.rand(9000, 40, generator=g)
    x = torch.arange(9000, dtype=torch.float32)[:, None]
    (_, _, _, _), rank, dist, order = er.environmental_selection(x, f, 8500, return_all=True)
    xs, fs, rs, ds = nd_environmental_selection(x.to(DEV), f.to(DEV), 8500)
    assert runtime.last_status()["error"] == 0 and runtime.last_status()["last_front_size"] > 8192
    picked = as_np(xs)[:, 0].astype(np.int64)
    assert len(set(picked.tolist())) == 8500
    assert np.array_equal(as_np(rs), as_np(rank)[picked]) and np.array_equal(as_np(fs), as_np(f)[picked])
    assert_dist_close(ds, as_np(dist)[picked], "uniform 9000x40")
    got_d = as_np(ds).astype(np.float64)
    key = np.where(np.isnan(got_d), -np.inf, got_d)
    assert np.array_equal(picked, picked[np.lexsort((picked, -key, as_np(rs)))])  # rank, distance descending, index
    left_out = np.setdiff1d(np.arange(9000), picked)
    cut = as_np(dist)[picked].min()
    assert (as_np(dist)[left_out] <= cut * (1 + 1e-5)).all()  # nothing clearly better than the worst taken row is left out


def test_crowding_dtype_rule():
    with pytest.raises(RuntimeError):
        crowding_distance(torch.rand(8, 2, dtype=torch.float64, device=DEV), None)


# ----------------------------------------------------------------- selection


def check_selection(f, x, topk, want_rank, want_dist, want_order, what):
    xs, fs, rs, ds = nd_environmental_selection(x.to(DEV), f.to(DEV), topk)
    assert runtime.last_status()["error"] == 0
    assert xs.shape == (topk, *x.shape[1:]) and fs.shape == (topk, f.size(1)) and rs.dtype == torch.int32
    want_order = np.asarray(want_order).astype(np.int64)
    assert np.array_equal(as_np(rs), np.asarray(want_rank)[want_order]), what
    assert_dist_close(ds, np.asarray(want_dist)[want_order], what)
    assert np.array_equal(as_np(fs), as_np(f)[want_order], equal_nan=True), what
    assert np.array_equal(as_np(xs), as_np(x)[want_order], equal_nan=True), what


@pytest.mark.parametrize("name,f,ks", EDGE, ids=IDS)
def test_selection_edge_golden(edge_golden, name, f, ks):
    x = torch.arange(f.size(0), dtype=torch.float32)[:, None].repeat(1, 2)
    for k in ks:
        say("selection", name, "topk", k)
        check_selection(f, x, k, edge_golden[f"{name}/rank"], edge_golden[f"{name}/dist@{k}"],
                        edge_golden[f"{name}/order@{k}"], f"{name}@{k}")


@pytest.mark.parametrize("name", ["C1", "C2", "C2p", "C3"])
def test_selection_configs_golden(name, peel_algorithm):
    say("selection_config", name, peel_algorithm)
    w, g = golden_io.config(name)
    x = w.x if w.x is not None else torch.arange(w.f.size(0), dtype=torch.float32)[:, None].repeat(1, 5)
    check_selection(w.f, x, w.topk, g["rank"], g["dist"], g["order"], name)


def test_selection_c4_first8_vmap():
    say("selection_c4_first8")
    w, g = golden_io.c4_first8()
    fd = w.f[:8].to(DEV)
    xd = torch.arange(512, dtype=torch.int64, device=DEV)[None, :, None].repeat(8, 1, 3)
    xs, fs, rs, ds = torch.vmap(lambda x, f: nd_environmental_selection(x, f, w.topk))(xd, fd)
    for b in range(8):
        order = g["order"][b].astype(np.int64)
        assert np.array_equal(as_np(xs[b])[:, 0], order)
        assert np.array_equal(as_np(rs[b]), g["rank"][b][order])
        assert_dist_close(ds[b], g["dist"][b][order])
        assert np.array_equal(as_np(fs[b]), as_np(w.f[b])[order])


def test_c4_every_population_against_the_cpu_side():
    """All 1024 populations of the batched configuration in one call: the ranks of every population against the
    batched restatement of the reference's loop, and every population's selection against the plain-C checker."""
    from oracle import c_oracle

    say("c4_every_population")
    w = workloads.c4()
    fd = w.f.to(DEV)
    xd = torch.arange(512, dtype=torch.int32, device=DEV)[None, :, None].expand(1024, 512, 1).contiguous()
    ranks = as_np(non_dominate_rank(fd))
    xs, fs, rs, ds = (as_np(t) for t in nd_environmental_selection(xd, fd, w.topk))
    for lo in range(0, 1024, 64):  # (64 populations: 50 MB for each of the restatement's (B, N, N, M) temporaries)
        assert np.array_equal(ranks[lo: lo + 64], as_np(er.ranks_by_peeling_batched(w.f[lo: lo + 64]))), lo
    f_np = as_np(w.f)
    for b in range(1024):
        order, rank, dist, _ = c_oracle.select(f_np[b], w.topk)
        assert np.array_equal(rank, ranks[b]), b
        assert np.array_equal(xs[b][:, 0].astype(np.int64), order), b
        assert np.array_equal(rs[b], rank[order]), b
        assert_dist_close(ds[b], dist[order], f"population {b}")
        assert np.array_equal(fs[b], f_np[b][order]), b


def test_c4_full_batch_one_launch():
    """All 1024 populations of the batched configuration in one call: the first eight against the
    golden vectors, a sample of the others against the single-population pipeline."""
    say("c4_full_batch")
    w, g = golden_io.c4_first8()
    fd = w.f.to(DEV)
    xd = torch.arange(512, dtype=torch.float32, device=DEV)[None, :, None].expand(1024, 512, 4).contiguous()
    ranks = non_dominate_rank(fd)
    xs, fs, rs, ds = nd_environmental_selection(xd, fd, w.topk)
    assert ranks.shape == (1024, 512) and xs.shape == (1024, 256, 4) and fs.shape == (1024, 256, 3)
    assert np.array_equal(as_np(ranks[:8]), g["rank"])
    for b in range(8):
        order = g["order"][b].astype(np.int64)
        assert np.array_equal(as_np(xs[b])[:, 0].astype(np.int64), order)
        assert np.array_equal(as_np(rs[b]), g["rank"][b][order])
        assert_dist_close(ds[b], g["dist"][b][order])
    keep = runtime.use_small_population_kernel
    runtime.use_small_population_kernel = False
    try:
        for b in (8, 333, 1023):
            assert torch.equal(non_dominate_rank(fd[b]), ranks[b])
            one = nd_environmental_selection(xd[b], fd[b], w.topk)
            assert torch.equal(one[0], xs[b]) and torch.equal(one[2], rs[b])
            assert_dist_close(one[3], ds[b])
    finally:
        runtime.use_small_population_kernel = keep


@pytest.mark.parametrize("n,m", [(33, 1), (64, 2), (95, 3), (130, 4), (257, 5), (500, 6), (777, 7), (1024, 8), (1000, 3), (300, 9),
                                 (512, 12), (200, 13), (1024, 16)])
def test_batched_selection_shapes_layouts_and_row_units(n, m, population_path):
    """The one-workgroup kernel over ragged sizes, every objective count, packed and strided fitness (its
    dominator loads take different paths), non-finite values (the compare form) and rows of x whose size
    allows 16-byte, 4-byte or single-byte units; every population against the CPU restatement."""
    if population_path != "small-kernel":
        pytest.skip("about the one-workgroup kernel")
    say("batched_shapes", n, m)
    g = torch.Generator("cpu").manual_seed(100 * n + m)
    batch, topk = 3, max(1, n // 3)
    f = torch.rand(batch, n, m, generator=g)
    f[0, : n // 4] = (f[0, : n // 4] * 4).round() / 4        # ties and duplicate rows
    f[1, 1] = f[1, 0]
    f_strided = f.transpose(1, 2).contiguous().transpose(1, 2)  # same values, objective-major memory
    f_bad = f.clone()
    f_bad[2, 0, 0] = float("nan")
    f_bad[2, n - 1, m - 1] = float("inf")
    f_bad[1, n // 2, 0] = -float("inf")
    xs = [torch.rand(batch, n, 8, generator=g),                                  # 32-byte rows: 16-byte units
          torch.rand(batch, n, 5, generator=g),                                  # 20-byte rows: 4-byte units
          torch.randint(0, 255, (batch, n, 7), generator=g, dtype=torch.uint8),  # 7-byte rows: single bytes
          torch.rand(batch, n, 300, generator=g)]                                # several units per lane and row
    for fit in (f, f_strided, f_bad):
        assert m == 1 or fit.is_contiguous() == (fit is not f_strided)
        want = [er.environmental_selection(fit[b], fit[b], topk, return_all=True) for b in range(batch)]
        ranks = non_dominate_rank(fit.to(DEV))
        for b in range(batch):
            assert np.array_equal(as_np(ranks[b]), as_np(want[b][1])), b
        for x in xs:
            ox, of, orank, odist = nd_environmental_selection(x.to(DEV), fit.to(DEV), topk)
            for b in range(batch):
                order = as_np(want[b][3])
                assert np.array_equal(as_np(ox[b]), as_np(x[b])[order]), (b, tuple(x.shape))
                assert np.array_equal(as_np(of[b]), as_np(fit[b])[order], equal_nan=True), b
                assert np.array_equal(as_np(orank[b]), as_np(want[b][0][2])), b
                assert_dist_close(odist[b], as_np(want[b][0][3]))


@pytest.mark.parametrize("n,m,d,topk", [(200, 3, 30, 100), (5000, 3, 16, 2500)])
def test_selection_captured_in_a_graph_replays_correctly(n, m, d, topk, population_path):
    """The whole selection (no allocation by the library, no host synchronisation, state cleared by kernels)
    can be captured in a HIP graph; every replay, with eager calls in between, must equal the eager result."""
    if population_path == "small-kernel" and n > 1024:
        pytest.skip("population too large for the one-workgroup kernel")
    say("graph", n, m, population_path)
    g = torch.Generator("cpu").manual_seed(n)
    fs = [torch.rand(n, m, generator=g) for _ in range(3)]
    xs = [torch.rand(n, d, generator=g) for _ in range(3)]
    f_static, x_static = fs[0].to(DEV).clone(), xs[0].to(DEV).clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):  # warm-up on a side stream, as torch asks before a capture
        for _ in range(2):
            nd_environmental_selection(x_static, f_static, topk)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = nd_environmental_selection(x_static, f_static, topk)
    for rep in range(5):
        i = rep % 3
        f_static.copy_(fs[i].to(DEV))
        x_static.copy_(xs[i].to(DEV))
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in out]
        want = nd_environmental_selection(xs[i].to(DEV), fs[i].to(DEV), topk)  # eager work between the replays
        torch.cuda.synchronize()
        for a, b in zip(got, want):
            assert np.array_equal(as_np(a), as_np(b), equal_nan=a.dtype.is_floating_point), rep
    del graph
    runtime.release_workspaces()  # the workspace of the capture stream lives in the graph's private pool


def test_selection_x_dtypes_and_shapes():
    say("selection_x_dtypes")
    f = workloads.uniform_population(300, 3, 0, 8)[0]
    _, _, _, order = er.environmental_selection(f, f, 120, return_all=True)
    order = as_np(order)
    for x in (torch.arange(300, dtype=torch.int64), torch.rand(300, 7).double(), torch.rand(300, 3, 5),
              torch.arange(300, dtype=torch.uint8)[:, None].repeat(1, 3), torch.rand(300, 13).half(),
              torch.rand(300, 40)[:, ::2]):
        xs = nd_environmental_selection(x.to(DEV), f.to(DEV), 120)[0]
        assert xs.dtype == x.dtype and np.array_equal(as_np(xs), as_np(x)[order])


@pytest.mark.parametrize("name,f,ks", EDGE, ids=IDS)
def test_rank_of_other_dtypes_edge(name, f, ks):
    """float64 and integer fitness is ranked through per-objective dense ranks, which keep every
    `<=` and `<` of the original values (the reference ranks any dtype, non_dominate.py:172-195)."""
    from evox_amd.operators.selection import non_dominated_mask

    say("rank_f64", name)
    want = as_np(er.ranks_by_peeling(f.double()))
    assert np.array_equal(want, as_np(er.ranks_by_peeling(f)))  # widening float32 keeps the order
    assert np.array_equal(as_np(non_dominate_rank(f.double().to(DEV))), want)
    assert np.array_equal(as_np(non_dominated_mask(f.double().to(DEV))), want == 0)


def test_rank_of_other_dtypes_values_beyond_float32():
    say("rank_dtypes")
    g = torch.Generator("cpu").manual_seed(77)
    # float64 values that collapse when rounded to float32, and 64-bit integers beyond 2**24
    f64 = 1.0 + torch.randint(0, 50, (700, 3), generator=g).double() * 1e-12
    f64[5, 1] = float("nan")
    f64[6] = f64[7]
    f64[8, 0], f64[9, 0] = 0.0, -0.0
    i64 = (2**40 + torch.randint(0, 40, (500, 2), generator=g)).long()
    i32 = torch.randint(-5, 5, (400, 4), generator=g, dtype=torch.int32)
    for t in (f64, i64, i32):
        want = as_np(er.ranks_by_peeling(t))
        assert want.max() > 3
        assert np.array_equal(as_np(non_dominate_rank(t.to(DEV))), want), t.dtype
    assert not np.array_equal(as_np(er.ranks_by_peeling(f64.float())), as_np(er.ranks_by_peeling(f64)))
    stacked = torch.stack([f64, f64.flip(0)])
    assert np.array_equal(as_np(non_dominate_rank(stacked.to(DEV))), np.stack([as_np(er.ranks_by_peeling(x)) for x in stacked]))
    with pytest.raises(TypeError):
        non_dominate_rank(torch.zeros(4, 2, dtype=torch.bool, device=DEV))


def test_selection_errors():
    f = torch.rand(5, 2, device=DEV)
    with pytest.raises(RuntimeError):
        nd_environmental_selection(f, f, 6)
    with pytest.raises(IndexError):
        nd_environmental_selection(f, f, 0)
    with pytest.raises(RuntimeError):
        non_dominate_rank(torch.rand(5, 2))  # CPU tensors are refused: there is no fallback


def test_selection_compile():
    say("selection_compile")
    w, g = golden_io.config("C1")
    fn = torch.compile(lambda x, f: nd_environmental_selection(x, f, 100), fullgraph=True)
    xs, fs, rs, ds = fn(w.x.to(DEV), w.f.to(DEV))
    order = g["order"].astype(np.int64)
    assert np.array_equal(as_np(rs), g["rank"][order]) and np.array_equal(as_np(xs), as_np(w.x)[order])


# ------------------------------------------------------- size-independent


def test_properties_at_full_size_c3():
    """At the benchmark size: the selected set is rank-sorted, complete below the last front,
    distance-sorted inside it, and re-ranking the survivors alone reproduces their ranks'
    ordering (survivors of better fronts never become dominated by dropping rows)."""
    say("properties_c3")
    w = workloads.c3(seed=7)
    fd, xd = w.f.to(DEV), w.x.to(DEV)
    rank = non_dominate_rank(fd)
    xs, fs, rs, ds = nd_environmental_selection(xd, fd, w.topk)
    rank_np, rs_np, ds_np = as_np(rank), as_np(rs), as_np(ds)
    assert (np.diff(rs_np) >= 0).all()
    worst = rs_np[-1]
    assert (rs_np < worst).sum() == (rank_np < worst).sum()
    tail = ds_np[rs_np == worst]
    assert (tail[1:] <= tail[:-1]).all()
    assert np.isneginf(ds_np[rs_np < worst]).all()
    # every selected fitness row exists in the input, and rows of rank < worst are all selected
    sel = {tuple(r) for r in as_np(fs).tolist()}
    assert all(tuple(r) in sel for r in as_np(w.f)[rank_np < worst][:500].tolist())
    # idempotence of ranking on the better fronts: removing worse rows does not change their rank
    keep = rank < int(worst)
    again = non_dominate_rank(fd[keep])
    assert torch.equal(again, rank[keep])


def test_c5_full_size_against_c_checker(population_path):
    """The large-scale configuration (N = 200000, M = 8, 5 GB bit matrix): ranks, distances and the
    selected order against the plain-C checker (the dense restatement cannot allocate here)."""
    if population_path == "small-kernel":
        pytest.skip("one run is enough: populations of this size always take the pipeline")
    from oracle import c_oracle

    say("c5_full_size")
    w = workloads.c5()
    n = w.f.size(0)
    order, rank, dist, fronts = c_oracle.select(as_np(w.f), w.topk)
    say("c5 checker done", fronts, "fronts")
    fd = w.f.to(DEV)
    got_rank = non_dominate_rank(fd)
    assert np.array_equal(as_np(got_rank), rank)
    assert runtime.last_status()["fronts"] == fronts
    x = torch.arange(n, dtype=torch.int32, device=DEV)[:, None].repeat(1, 2)
    xs, fs, rs, ds = nd_environmental_selection(x, fd, w.topk)
    assert runtime.last_status()["error"] == 0
    assert np.array_equal(as_np(xs)[:, 0].astype(np.int64), order)
    assert np.array_equal(as_np(rs), rank[order])
    assert_dist_close(ds, dist[order], "C5")
    assert np.array_equal(as_np(fs), as_np(w.f)[order])
    runtime.release_workspaces()


def test_large_front_ordered_from_the_objective_orders_with_ties():
    """A population large enough for the order-based matrix, whose cut front is large: that front's per-objective
    order is read off the orders of the whole population.  Values on a coarse grid, so that every objective has long
    runs of equal values (which a stable sort keeps in index order) and duplicate rows; against the plain-C checker."""
    from oracle import c_oracle

    say("large_front_from_orders_ties")
    for n, m, scale, topk, seed in ((70000, 8, 32.0, 35000, 5), (70000, 4, 8.0, 60000, 6)):  # the second: 66806 duplicate rows
        f = (workloads.sphere_shell_population((n,), m, 0.05, seed=seed) * scale).round() / scale
        f = f.contiguous()
        order, rank, dist, fronts = c_oracle.select(as_np(f), topk)
        x = torch.arange(n, dtype=torch.int32, device=DEV)[:, None]
        xs, fs, rs, ds = nd_environmental_selection(x, f.to(DEV), topk)
        st = runtime.last_status()
        assert st["error"] == 0 and st["last_front_size"] > 8192, st
        assert np.array_equal(as_np(xs)[:, 0].astype(np.int64), order)
        assert np.array_equal(as_np(rs), rank[order])
        assert_dist_close(ds, dist[order], f"ties {n}x{m}")
        assert np.array_equal(as_np(fs), as_np(f)[order])
        runtime.release_workspaces()


def test_large_front_ordered_from_the_objective_orders_twelve_objectives():
    """The same with twelve objectives (tiles of four words, the lower row limit of the order-based matrix).  The
    distance is a sum of twelve terms, associated differently from the checker's (tolerance 1e-5), so rows whose
    distances nearly tie may swap: the order is checked through what defines it."""
    from oracle import c_oracle

    say("large_front_from_orders_m12")
    n, m, topk = 52000, 12, 30000
    f = ((workloads.sphere_shell_population((n,), m, 0.05, seed=8) * 64.0).round() / 64.0).contiguous()
    order, rank, dist, fronts = c_oracle.select(as_np(f), topk)
    x = torch.arange(n, dtype=torch.int32, device=DEV)[:, None]
    xs, fs, rs, ds = nd_environmental_selection(x, f.to(DEV), topk)
    st = runtime.last_status()
    assert st["error"] == 0 and st["last_front_size"] > 8192, st
    picked = as_np(xs)[:, 0].astype(np.int64)
    assert len(set(picked.tolist())) == topk
    assert np.array_equal(as_np(rs), rank[picked]) and np.array_equal(as_np(fs), as_np(f)[picked])
    assert_dist_close(ds, dist[picked], "ties 52000x12")
    got_d = as_np(ds).astype(np.float64)
    key = np.where(np.isnan(got_d), -np.inf, got_d)
    assert np.array_equal(picked, picked[np.lexsort((picked, -key, as_np(rs)))])  # rank, distance descending, index
    runtime.release_workspaces()


def test_stop_early_matches_full_ranking(peel_algorithm):
    say("stop_early", peel_algorithm)
    f = workloads.uniform_population(4000, 3, 0, 21)[0]
    fd = f.to(DEV)
    full = as_np(non_dominate_rank(fd))
    views, st = run_stages(fd, 2000)
    part = as_np(views["rank"])
    ranked = part != 0x7FFFFFFF
    assert np.array_equal(part[ranked], full[ranked])
    assert ranked.sum() >= 2000 and st["worst_rank"] == np.sort(full)[1999]
    perm = as_np(views["perm"])[: st["better_rows"] + st["last_front_size"]]
    assert np.array_equal(perm, np.lexsort((np.arange(4000), full))[: perm.size])


def test_barrier_timeout_is_reported_not_hung():
    """A spin limit of one poll makes the bounded device-side wait give up: the kernel must end and
    the status must carry the error."""
    say("barrier_timeout")
    f, x = workloads.uniform_population(3000, 3, 4, 5)
    f, x = f.to(DEV), x.to(DEV)
    want = as_np(er.ranks_by_peeling(f.cpu()))

    def failed():
        try:
            runtime.last_status()
        except _lib.EvoxHipError as e:
            assert e.code == _lib.E_BARRIER_TIMEOUT
            return True
        return False

    with runtime.options(spin_limit=1):
        # with one poll a wait may still succeed when the other blocks are already there: either the result is
        # right and the status clean, or the status carries the error and NO partial result is handed out --
        # every rank -1, every distance NaN, the rows all-ones bytes
        rank = non_dominate_rank(f)
        if failed():
            say("barrier_timeout: the ranking gave up")
            assert (as_np(rank) == -1).all()
        else:
            assert np.array_equal(as_np(rank), want)
        xs, fs, rs, ds = nd_environmental_selection(x, f, 1500)
        if failed():
            say("barrier_timeout: the selection gave up")
            assert (as_np(rs) == -1).all() and np.isnan(as_np(ds)).all() and np.isnan(as_np(fs)).all()
            assert np.isnan(as_np(xs)).all()
        else:
            assert np.array_equal(as_np(rs), np.sort(want)[:1500])
        dist = crowding_distance(f, None)
        if failed():
            assert np.isnan(as_np(dist)).all()
    assert np.array_equal(as_np(non_dominate_rank(f)), want)
    assert not failed()


def test_fronts_of_thousands_of_rows(peel_algorithm):
    """Every pass ranks about 3000 rows at once: with the record protocol most blocks then hold more
    rows than their record carries and publish through the front bitmaps, and the lister merges both
    sources.  Checked against the plain-C checker."""
    from oracle import c_oracle

    say("big_fronts", peel_algorithm)
    f = workloads.layered_grid_population(10, 3000, seed=3, permute=True)
    n = f.size(0)
    want_rank, fronts = c_oracle.nd_rank(as_np(f))
    assert fronts >= 10
    fd = f.to(DEV)
    assert np.array_equal(as_np(non_dominate_rank(fd)), want_rank)
    st = runtime.last_status()
    assert st["error"] == 0 and st["fronts"] == fronts
    x = torch.arange(n, dtype=torch.float32)[:, None].repeat(1, 2)
    for topk in (n // 2, 2999, n):
        order, rank, dist, _ = c_oracle.select(as_np(f), topk)
        xs, fs, rs, ds = nd_environmental_selection(x.to(DEV), fd, topk)
        assert np.array_equal(as_np(xs)[:, 0].astype(np.int64), order), topk
        assert np.array_equal(as_np(rs), rank[order])
        assert_dist_close(ds, dist[order], f"big fronts topk {topk}")


def test_large_fronts_between_small_ones_above_65534_rows(population_path):
    """70 000 rows of three objectives in layers that dominate one another: a front of 9000 rows (more than the
    records of the sweeping workgroups carry: it goes through the bitmaps in memory), then the thin fronts of 15 000
    uniform rows (records only: their bitmaps are never written and are not cleared either), a front of 12 000, thin
    fronts again, and so on.  Ranks and the selection against the plain-C checker."""
    if population_path != "pipeline":
        pytest.skip("single large populations always take the pipeline")
    from oracle import c_oracle

    say("large_and_small_fronts")
    g = torch.Generator("cpu").manual_seed(4242)

    def simplex(rows):
        u = torch.rand(rows, 3, generator=g)
        return u / u.sum(dim=1, keepdim=True)

    parts = [simplex(9000), 2.0 + torch.rand(15000, 3, generator=g), 10.0 + simplex(12000), 20.0 + torch.rand(14000, 3, generator=g),
             30.0 + simplex(8500), 40.0 + torch.rand(11500, 3, generator=g)]
    f = torch.cat(parts)[torch.randperm(70000, generator=g)].contiguous()
    n = f.size(0)
    want_rank, fronts = c_oracle.nd_rank(as_np(f))
    assert fronts > 40
    fd = f.to(DEV)
    assert np.array_equal(as_np(non_dominate_rank(fd)), want_rank)
    st = runtime.last_status()
    assert st["error"] == 0 and st["fronts"] == fronts
    x = torch.arange(n, dtype=torch.int32, device=DEV)[:, None]
    for topk in (30000, 69000):
        order, rank, dist, _ = c_oracle.select(as_np(f), topk)
        xs, fs, rs, ds = nd_environmental_selection(x, fd, topk)
        assert runtime.last_status()["error"] == 0
        assert np.array_equal(as_np(xs)[:, 0].astype(np.int64), order), topk
        assert np.array_equal(as_np(rs), rank[order])
        assert_dist_close(ds, dist[order], f"large and small fronts topk {topk}")
    runtime.release_workspaces()


def test_rank_at_the_protocol_boundary(population_path):
    """65534 rows is the largest population whose records hold three 16-bit slots a unit, 65535 the first one with
    two 24-bit slots: both against the plain-C checker."""
    if population_path != "pipeline":
        pytest.skip("single large populations always take the pipeline")
    from oracle import c_oracle

    f = workloads.uniform_population(65535, 3, 0, 77)[0]
    for n in (65534, 65535):
        say("protocol_boundary", n)
        want, fronts = c_oracle.nd_rank(as_np(f[:n]))
        got = non_dominate_rank(f[:n].to(DEV))
        assert np.array_equal(as_np(got), want)
        st = runtime.last_status()
        assert st["error"] == 0 and st["fronts"] == fronts
    runtime.release_workspaces()


def test_record_protocol_with_other_block_counts():
    """The number of sweeping blocks of the record protocol is a tunable; records need not fill the unit
    array (100 blocks x 8 units) and may be long (16 blocks x 64 units)."""
    say("record_blocks")
    f = workloads.uniform_population(6000, 3, 0, 12)[0]
    want = as_np(er.ranks_by_peeling(f))
    for blocks in (16, 37, 100, 128, 200):
        with runtime.options(peel_lds=0, peel_record_blocks=blocks):
            assert np.array_equal(as_np(non_dominate_rank(f.to(DEV))), want), blocks
            assert runtime.last_status()["error"] == 0


# ------------------------------------------------------------------ ranks up to the cut front only


@pytest.mark.parametrize("name,f,ks", EDGE, ids=IDS)
def test_rank_until_edge(name, f, ks, peel_algorithm):
    from evox_amd.operators.selection import non_dominate_rank_until

    for k in sorted(set(ks) | {1, f.size(0)}):
        say("rank_until", name, k, peel_algorithm)
        worst, keep, rank = er.front_cut(f, k)
        got = non_dominate_rank_until(f.to(DEV), k).cpu()
        # the caller's own statements on the truncated ranks (nsga3.py:170-171)
        assert torch.equal(torch.topk(got, k, largest=False)[0][-1], worst)
        assert torch.equal(got <= worst, keep)
        assert torch.equal(got[keep], rank[keep]) and bool((got[~keep] == 2**31 - 1).all())


def test_rank_until_c3_and_batch(peel_algorithm):
    from evox_amd.operators.selection import non_dominate_rank_until

    say("rank_until_c3", peel_algorithm)
    w, gold = golden_io.config("C3")
    rank = torch.from_numpy(gold["rank"])
    for k in (1, 31, 10001, 20000):
        worst = torch.topk(rank, k, largest=False)[0][-1]
        got = non_dominate_rank_until(w.f.to(DEV), k).cpu()
        assert torch.equal(got <= worst, rank <= worst) and torch.equal(got[rank <= worst], rank[rank <= worst])
        assert bool((got[rank > worst] == 2**31 - 1).all())
        assert runtime.last_status()["fronts"] == int(worst) + 1
    fb = torch.stack([workloads.uniform_population(500, 3, 0, 90 + b)[0] for b in range(3)])
    got = non_dominate_rank_until(fb.to(DEV), 100).cpu()
    for b in range(3):
        worst, keep, r = er.front_cut(fb[b], 100)
        assert torch.equal(got[b] <= worst, keep) and torch.equal(got[b][keep], r[keep])
    assert torch.equal(torch.vmap(lambda t: non_dominate_rank_until(t, 100))(fb.to(DEV)).cpu(), got)
    with pytest.raises(RuntimeError):
        non_dominate_rank_until(fb[0].to(DEV), 501)
    with pytest.raises(IndexError):
        non_dominate_rank_until(fb[0].to(DEV), 0)


# ------------------------------------------------------------------ first front only (rank == 0)


@pytest.mark.parametrize("name,f,ks", EDGE, ids=IDS)
def test_first_front_edge(name, f, ks, population_path):
    if population_path != "pipeline":
        pytest.skip("does not depend on the population path")
    from evox_amd.operators.selection import non_dominated_mask

    say("first_front", name, tuple(f.shape))
    got = non_dominated_mask(f.to(DEV))
    assert got.dtype == torch.bool and got.shape == (f.size(0),)
    assert np.array_equal(as_np(got), as_np(er.first_front_mask(f)))
    assert runtime.last_status()["error"] == 0


@pytest.mark.parametrize("m", [1, 2, 3, 4, 5, 6, 7, 8, 9, 12, 16, 17])
def test_first_front_all_m(m, population_path):
    if population_path != "pipeline":
        pytest.skip("does not depend on the population path")
    from evox_amd.operators.selection import non_dominated_mask

    say("first_front_all_m", m)
    g = torch.Generator("cpu").manual_seed(140 + m)
    for n in (333, 1500):
        f = (torch.randint(0, 3 + m, (n, m), generator=g).float() / 4.0).contiguous()
        f[::17] = f[1::17][: f[::17].size(0)]  # duplicate rows
        f[5, 0] = float("nan")
        assert np.array_equal(as_np(non_dominated_mask(f.to(DEV))), as_np(er.first_front_mask(f))), (m, n)
        ft = f.t().contiguous().t()  # column-major strides
        assert np.array_equal(as_np(non_dominated_mask(ft.to(DEV))), as_np(er.first_front_mask(f))), (m, n)


@pytest.mark.parametrize("name", ["C1", "C2", "C2p", "C3"])
def test_first_front_configs_golden(name, population_path):
    if population_path != "pipeline":
        pytest.skip("does not depend on the population path")
    from evox_amd.operators.selection import non_dominated_mask

    say("first_front_golden", name)
    w, gold = golden_io.config(name)
    got = as_np(non_dominated_mask(w.f.to(DEV)))
    assert np.array_equal(got, gold["rank"] == 0)


def test_first_front_large_history_and_batch(population_path):
    """The monitor's use: a long evaluation history.  200 000 rows x 3 objectives need 0.5 TB as a
    matrix; here the first front comes from the linear-memory entry point and is checked against the
    plain-C checker.  Then C5 (nearly everything non-dominated: the worst case, every wave scans all
    the slots below it) against the full ranking."""
    if population_path != "pipeline":
        pytest.skip("does not depend on the population path")
    from evox_amd.operators.selection import non_dominated_mask
    from oracle import c_oracle

    say("first_front_large")
    f = workloads.uniform_population(200000, 3, 0, 31)[0]
    got = as_np(non_dominated_mask(f.to(DEV)))
    want = c_oracle.first_front(as_np(f))
    assert np.array_equal(got, want)
    w = workloads.c5()
    fd = w.f.to(DEV)
    got5 = non_dominated_mask(fd)
    assert torch.equal(got5, non_dominate_rank(fd) == 0)
    runtime.release_workspaces()
    # leading batch dimensions and vmap
    fb = torch.stack([workloads.uniform_population(700, 3, 0, 50 + b)[0] for b in range(4)]).to(DEV)
    want_b = torch.stack([er.first_front_mask(fb[b].cpu()) for b in range(4)])
    assert torch.equal(non_dominated_mask(fb).cpu(), want_b)
    assert torch.equal(torch.vmap(non_dominated_mask)(fb).cpu(), want_b)
    assert torch.equal(torch.compile(non_dominated_mask, fullgraph=True)(fb[0]).cpu(), want_b[0])


# ------------------------------------------------------------------ parents + offspring given as two parts


@pytest.mark.parametrize("name", ["C1", "C2p", "C3"])
def test_two_part_selection_golden(name, population_path):
    if population_path != "pipeline":
        pytest.skip("the two-part entry always takes the pipeline")
    from evox_amd.operators.selection import nd_environmental_selection_two_part

    w, gold = golden_io.config(name)
    n = w.f.size(0)
    x = w.x if w.x is not None else torch.arange(n, dtype=torch.float32)[:, None].repeat(1, 3)
    fd, xd = w.f.to(DEV), x.to(DEV)
    order = gold["order"]
    for cut in (n // 2, 1, n - 1, 0, n, 129):
        say("two_part", name, cut)
        xs, fs, rs, ds = nd_environmental_selection_two_part(xd[:cut], fd[:cut], xd[cut:], fd[cut:], w.topk)
        assert np.array_equal(as_np(rs), gold["rank"][order])
        assert np.array_equal(as_np(fs), as_np(w.f)[order]) and np.array_equal(as_np(xs), as_np(x)[order])
        assert_dist_close(ds, gold["dist"][order], f"{name} cut {cut}")
    # parts with strides of their own: column-major fitness in one, padded rows of x in the other
    cut = n // 3
    fa = fd[:cut].t().contiguous().t()
    xb = torch.zeros(n - cut, x.size(1) + 5, device=DEV)[:, : x.size(1)]
    xb.copy_(xd[cut:])
    xs, fs, rs, ds = nd_environmental_selection_two_part(xd[:cut], fa, xb, fd[cut:], w.topk)
    assert np.array_equal(as_np(rs), gold["rank"][order]) and np.array_equal(as_np(xs), as_np(x)[order])


def test_two_part_selection_edge_and_errors(edge_golden, population_path):
    if population_path != "pipeline":
        pytest.skip("the two-part entry always takes the pipeline")
    from evox_amd.operators.selection import nd_environmental_selection_two_part

    for name, f, ks in EDGE:
        n = f.size(0)
        x = torch.arange(n, dtype=torch.float64)[:, None, None].repeat(1, 2, 2)  # any dtype, any row shape
        for k in ks:
            for cut in sorted({0, n // 2, n}):
                say("two_part_edge", name, k, cut)
                want, _, _, order = er.merged_selection(x[:cut], f[:cut], x[cut:], f[cut:], k, return_all=True)
                assert np.array_equal(as_np(order), edge_golden[f"{name}/order@{k}"])
                got = nd_environmental_selection_two_part(x[:cut].to(DEV), f[:cut].to(DEV), x[cut:].to(DEV), f[cut:].to(DEV), k)
                assert np.array_equal(as_np(got[0]), as_np(want[0])) and np.array_equal(as_np(got[2]), as_np(want[2]))
                assert np.array_equal(as_np(got[1]), as_np(want[1]), equal_nan=True)
                assert_dist_close(got[3], as_np(want[3]), f"{name}@{k}")
    f = torch.rand(6, 2, device=DEV)
    x = torch.rand(6, 4, device=DEV)
    with pytest.raises(RuntimeError):
        nd_environmental_selection_two_part(x[:3], f[:3], x[3:], f[3:], 7)
    with pytest.raises(IndexError):
        nd_environmental_selection_two_part(x[:3], f[:3], x[3:], f[3:], 0)
    with pytest.raises(ValueError):
        nd_environmental_selection_two_part(x[:3], f[:3], x[3:, :2], f[3:], 2)
    with pytest.raises(ValueError):
        nd_environmental_selection_two_part(x[:3], f[:3], x[3:], f[3:, :1], 2)
    compiled = torch.compile(nd_environmental_selection_two_part, fullgraph=True)
    a = compiled(x[:3], f[:3], x[3:], f[3:], 4)
    b = nd_environmental_selection(x, f, 4)
    assert all(torch.equal(p, q) for p, q in zip(a, b))


# ------------------------------------------------------------------ lexsort as a function of its own


def test_lexsort_matches_numpy_and_the_restatement(population_path):
    if population_path != "pipeline":
        pytest.skip("does not depend on the population path")
    from evox_amd.utils import lexsort

    g = torch.Generator("cpu").manual_seed(5)
    for n in (1, 2, 63, 64, 65, 1000, 4097, 8191, 8192, 8193, 12000, 24576, 32768, 32769, 70000):
        say("lexsort", n)
        k_f32 = torch.randint(0, 7, (n,), generator=g).float() / 2 - 1
        k_f32[torch.rand(n, generator=g) < 0.05] = float("nan")
        k_f32[torch.rand(n, generator=g) < 0.05] = -0.0
        k_f32[torch.rand(n, generator=g) < 0.05] = float("inf")
        k_f32[torch.rand(n, generator=g) < 0.05] = -float("inf")
        k_i32 = torch.randint(-3, 3, (n,), generator=g, dtype=torch.int32)
        k_i64 = torch.randint(-2, 2, (n,), generator=g) * (2**40) + torch.randint(0, 2, (n,), generator=g)
        k_f64 = 1.0 + torch.randint(0, 4, (n,), generator=g).double() * 1e-13
        k_f64[torch.rand(n, generator=g) < 0.05] = float("nan")
        k_u8 = torch.randint(0, 3, (n,), generator=g, dtype=torch.uint8)
        for keys in ([k_f32], [k_i32], [k_i64], [k_f64], [k_u8, k_f32], [k_f32, k_i32, k_u8], [k_f64, k_i64], [k_f32.half(), k_i32]):
            want = er.chained_stable_argsort([k.float() if k.dtype == torch.float16 else k for k in keys])
            got = lexsort([k.to(DEV) for k in keys])
            assert got.dtype == torch.int64 and torch.equal(got.cpu(), want), (n, [k.dtype for k in keys])
        # distinct values over a wide range, and the same with a crowd on one value (a distance that is -inf for most rows)
        k_wide = (torch.rand(n, generator=g) - 0.5) * 1e6
        k_crowd = torch.where(torch.rand(n, generator=g) < 0.7, torch.full((n,), -float("inf")), k_wide)
        for keys in ([k_wide], [k_crowd], [k_crowd, k_i32]):
            assert torch.equal(lexsort([k.to(DEV) for k in keys]).cpu(), er.chained_stable_argsort(keys)), (n, "wide")
        # numpy's lexsort on keys without NaN (same convention: last key primary, stable)
        assert np.array_equal(as_np(lexsort([k_i32.to(DEV), k_u8.to(DEV)])), np.lexsort((as_np(k_i32), as_np(k_u8))))
    # a strided key of a mid-sized sort, and the same sorts through the radix sort (the tunable that sends them there)
    base = torch.randint(0, 50, (40000,), generator=g).float()
    strided = base.to(DEV)[::2]
    assert strided.stride(0) == 2
    second = torch.randint(0, 5, (20000,), generator=g, dtype=torch.int32)
    want = er.chained_stable_argsort([base[::2], second])
    assert torch.equal(lexsort([strided, second.to(DEV)]).cpu(), want)
    with runtime.options(mid_argsort=0):
        assert torch.equal(lexsort([strided, second.to(DEV)]).cpu(), want)
    # along a dimension of a matrix, as the crowding distance uses it (non_dominate.py:221)
    c = torch.rand(300, 4, generator=g)
    m = (torch.rand(300, generator=g) < 0.5).float()[:, None].expand(-1, 4).contiguous()
    assert torch.equal(lexsort([c.to(DEV), m.to(DEV)], dim=0).cpu(), er.chained_stable_argsort([c, m], dim=0))
    assert torch.equal(lexsort([c.t().contiguous().to(DEV)], dim=-1).cpu(), er.chained_stable_argsort([c.t().contiguous()], dim=-1))


def test_lexsort_along_a_dimension_of_many_sorts(population_path):
    """Keys with more than one dimension (jit_fix_operator.py:246-250 with `dim`): every sort of the batch
    in the same launches for up to 16384 positions, one after the other above that."""
    if population_path != "pipeline":
        pytest.skip("does not depend on the population path")
    from evox_amd.utils import lexsort

    g = torch.Generator("cpu").manual_seed(15)
    shapes = [(5, 1), (4000, 2), (130, 3), (9, 64), (37, 200), (3, 256), (3, 257), (5, 300), (2, 1000), (4, 1024), (3, 1025),
              (2, 4096), (3, 4097), (9, 5000), (8, 8192), (2, 8192), (2, 8193), (2, 16384), (2, 16385), (3, 20000), (300, 2048), (0, 7), (6, 0)]
    for batch, n in shapes:
        say("lexsort rows", batch, n)
        k_f32 = torch.randint(0, 9, (batch, n), generator=g).float() / 4 - 1
        k_f32[torch.rand(batch, n, generator=g) < 0.03] = float("nan")
        k_f32[torch.rand(batch, n, generator=g) < 0.03] = -0.0
        k_i32 = torch.randint(-3, 3, (batch, n), generator=g, dtype=torch.int32)
        k_f64 = 1.0 + torch.randint(0, 4, (batch, n), generator=g).double() * 1e-13
        for keys in ([k_f32], [k_f32, k_i32], [k_f64, k_f32]):
            want = er.chained_stable_argsort(keys, dim=-1)
            got = lexsort([k.to(DEV) for k in keys], dim=-1)
            assert got.dtype == torch.int64 and got.shape == want.shape and torch.equal(got.cpu(), want), (batch, n)
    # a middle dimension, keys that are views, and the tournament's shape (tournament_selection.py:26)
    a = torch.randint(0, 5, (6, 50, 7), generator=g).float()
    b = torch.randint(0, 3, (6, 50, 7), generator=g, dtype=torch.int32)
    for dim in (0, 1, 2, -2):
        assert torch.equal(lexsort([a.to(DEV), b.to(DEV)], dim=dim).cpu(), er.chained_stable_argsort([a, b], dim=dim)), dim
    at = a.to(DEV).transpose(0, 2)
    assert torch.equal(lexsort([at, b.to(DEV).transpose(0, 2)], dim=1).cpu(),
                       er.chained_stable_argsort([a.transpose(0, 2), b.transpose(0, 2)], dim=1))
    wide = torch.rand(2, 8192, generator=g)[:, ::2]  # strided within the sort
    assert torch.equal(lexsort([wide.to(DEV)[:, :]], dim=1).cpu(), er.chained_stable_argsort([wide], dim=1))
    flipped = torch.rand(4, 33, generator=g)
    assert torch.equal(lexsort([flipped.to(DEV).flip(0)], dim=1).cpu(), er.chained_stable_argsort([flipped.flip(0)], dim=1))


def test_lexsort_gives_the_selection_order(population_path):
    """HypE's `lexsort([-dis, rank])[:pop_size]` (hype.py:143) and the selection's own final ordering
    (non_dominate.py:253) on the golden rank and distance of C3."""
    if population_path != "pipeline":
        pytest.skip("does not depend on the population path")
    from evox_amd.utils import lexsort

    w, gold = golden_io.config("C3")
    rank = torch.from_numpy(gold["rank"]).to(DEV)
    dist = torch.from_numpy(gold["dist"]).to(DEV)
    got = lexsort([-dist, rank])[: w.topk]
    assert np.array_equal(as_np(got), gold["order"])


# ------------------------------------------------------------------ hypervolume contributions (HypE)


def test_hv_contributions_against_oracle(population_path):
    """Tolerance 1e-5 relative: the per-point sums run over the samples in another order than torch's."""
    if population_path != "pipeline":
        pytest.skip("does not depend on the population path")
    from evox_amd import ops
    from evox_amd.hype import cal_hv, hv_alpha

    g = torch.Generator("cpu").manual_seed(19)
    for n, m, pop, ns in ((1, 2, 1, 100), (7, 2, 3, 333), (200, 3, 100, 10000), (1000, 5, 400, 5000), (64, 9, 64, 1025),
                          (50, 17, 20, 700)):
        say("hv", n, m, pop, ns)
        fit = torch.rand(n, m, generator=g)
        if n > 3:
            fit[1] = fit[0]
        ref = torch.full((m,), 1.2)
        u = torch.rand(ns, m, generator=g)
        want = er.hv_contributions(fit, ref, pop, u)
        f_min = fit.min(dim=0).values
        samples = u * (ref - f_min) + f_min  # the same float32 values as the restatement forms
        alpha = hv_alpha(n, pop, DEV)
        got = ops.hv_contributions(fit.to(DEV), samples.to(DEV), alpha, 1.0).cpu() * torch.prod(ref - f_min) / ns
        assert torch.allclose(got, want, rtol=1e-5, atol=1e-9), (n, m)
    # the function with the reference's signature draws its samples itself
    fit = torch.rand(300, 3, generator=g).to(DEV)
    ref = torch.full((3,), 1.1, device=DEV)
    torch.manual_seed(7)
    got = cal_hv(fit, ref, 150, 4000)
    torch.manual_seed(7)
    u = torch.rand(4000, 3, device=DEV)
    want = er.hv_contributions(fit.cpu(), ref.cpu(), 150, u.cpu())
    assert got.shape == (300,) and torch.allclose(got.cpu(), want, rtol=1e-5, atol=1e-9)


def test_hv_metric_against_oracle(population_path):
    """Counts are integers, so the estimate equals the restatement's bit for bit on the same samples."""
    if population_path != "pipeline":
        pytest.skip("does not depend on the population path")
    from evox_amd import ops
    from evox_amd.metrics import hv

    g = torch.Generator("cpu").manual_seed(23)
    for n, m, ns in ((1, 2, 100), (7, 2, 333), (200, 3, 10000), (1000, 5, 5000), (64, 9, 1025), (50, 17, 700), (3000, 3, 100000)):
        say("hv metric", n, m, ns)
        objs = torch.rand(n, m, generator=g)
        if n > 3:
            objs[1] = objs[0]
        if n == 1000:
            objs[5, 0] = float("nan")   # the bound, every sample and the estimate become NaN (torch.max propagates)
        ref = torch.full((m,), 1.2)
        u = torch.rand(ns, m, generator=g)
        want = er.hv_estimate(objs, ref, u)
        points = torch.abs(objs - ref)
        samples = u * points.max(dim=0).values
        covered = ops.hv_covered_count(points.to(DEV), samples.to(DEV))
        exact = int(torch.any(torch.all(samples.unsqueeze(1) < points.unsqueeze(0), dim=2), dim=1).sum()) if n * ns <= 5e6 else None
        if exact is not None:
            assert int(covered) == exact, (n, m)
        got = covered.cpu() / ns * torch.prod(points.max(dim=0).values)  # hv.py:19 on the CPU, like the restatement
        assert torch.equal(got, want) or (torch.isnan(got) and torch.isnan(want)), (n, m, float(got), float(want))
    # the count itself with non-finite points among finite samples (NaN compares false, +inf exceeds everything)
    points = torch.rand(500, 3, generator=g)
    points[::7, 0] = float("nan")
    points[::11, 1] = float("inf")
    points[::13, 2] = -float("inf")
    samples = torch.rand(4000, 3, generator=g) * 1.05
    samples[::17, 1] = float("nan")
    samples[::19, 2] = float("inf")
    exact = int(torch.any(torch.all(samples.unsqueeze(1) < points.unsqueeze(0), dim=2), dim=1).sum())
    assert 0 < exact < 4000 and int(ops.hv_covered_count(points.to(DEV), samples.to(DEV))) == exact
    # strictness: a sample on a face of the only box is outside
    points = torch.tensor([[1.0, 2.0]], device=DEV)
    samples = torch.tensor([[0.5, 1.0], [1.0, 1.0], [0.5, 2.0], [0.0, 0.0]], device=DEV)
    assert int(ops.hv_covered_count(points, samples)) == 2
    # the function with the reference's signature draws its samples itself, on the default device
    objs = torch.rand(300, 3, generator=g)
    ref = torch.full((3,), 1.1)
    torch.manual_seed(11)
    got = hv(objs.to(DEV), ref.to(DEV), 20000)
    torch.manual_seed(11)
    want = er.hv_estimate(objs, ref, torch.rand(20000, 3))
    # hv.py:19 runs on the GPU here: torch's division and product there may differ from the CPU's in the last bit
    assert got.shape == () and got.device.type == "cuda" and float(got) == pytest.approx(float(want), rel=1e-6)
    assert float(hv(objs.to(DEV), ref.to(DEV))) == pytest.approx(float(want), rel=0.02)  # default: 100000 samples


# ------------------------------------------------------------------ tournament (consumer of rank / distance)


def _tournament_case(seed, n_cand, n_round, tsize):
    g = torch.Generator("cpu").manual_seed(seed)
    rank = torch.randint(0, 3, (n_cand,), generator=g, dtype=torch.int32)
    dist = torch.randint(0, 4, (n_cand,), generator=g).float() / 2
    dist[torch.rand(n_cand, generator=g) < 0.15] = float("inf")
    dist[torch.rand(n_cand, generator=g) < 0.15] = -float("inf")
    dist[torch.rand(n_cand, generator=g) < 0.1] = float("nan")
    dist[torch.rand(n_cand, generator=g) < 0.1] = -0.0
    parents = torch.randint(0, n_cand, (n_round, tsize), generator=g)
    return parents, [-dist, rank]


@pytest.mark.parametrize("tsize", [1, 2, 3, 5])
def test_tournament_pick_against_oracle(tsize, population_path):
    if population_path != "pipeline":
        pytest.skip("does not depend on the population path")
    from evox_amd import ops

    for seed, n_cand, n_round in ((1, 1, 5), (2, 6, 64), (3, 50, 3000), (4, 10000, 100000)):
        say("tournament", tsize, seed, n_cand, n_round)
        parents, fits = _tournament_case(seed, n_cand, n_round, tsize)
        want = as_np(er.tournament_winners(parents, fits)).reshape(-1)
        table = torch.stack([k.to(DEV) for k in fits], dim=1)
        got = as_np(ops.tournament_pick(parents.to(DEV), table))
        assert np.array_equal(got, want), (tsize, seed)
        # a transposed (column-major) key table goes through the strides, not through a copy
        table_t = torch.stack([k.to(DEV).float() for k in fits], dim=0).t()
        assert n_cand == 1 or not table_t.is_contiguous()
        assert np.array_equal(as_np(ops.tournament_pick(parents.to(DEV), table_t)), want)


@pytest.mark.parametrize("tsize", [1, 2, 5])
def test_tournament_pick_on_a_list_of_keys(tsize, population_path):
    """The keys as the caller holds them (float32 distances, int32 ranks; strided views; one to four of them) give
    the winners of the stacked table."""
    if population_path != "pipeline":
        pytest.skip("does not depend on the population path")
    from evox_amd import ops

    for seed, n_cand, n_round in ((1, 1, 5), (2, 6, 64), (3, 50, 3000), (4, 10000, 100000)):
        say("tournament_keys", tsize, seed, n_cand, n_round)
        parents, fits = _tournament_case(seed, n_cand, n_round, tsize)
        want = as_np(er.tournament_winners(parents, fits)).reshape(-1)
        keys = [k.to(DEV) for k in fits]
        assert keys[0].dtype == torch.float32 and keys[1].dtype == torch.int32
        assert np.array_equal(as_np(ops.tournament_pick_keys(parents.to(DEV), keys)), want), (tsize, seed)
        # every second element of a longer vector: through the stride
        wide = [torch.stack([k, k + 1], dim=1).reshape(-1)[::2] for k in keys]
        assert n_cand == 1 or not wide[0].is_contiguous()
        assert np.array_equal(as_np(ops.tournament_pick_keys(parents.to(DEV), wide)), want)
        # one, three and four keys against the stacked table
        g = torch.Generator("cpu").manual_seed(seed)
        more = [torch.randint(0, 3, (n_cand,), generator=g).float().to(DEV) for _ in range(2)]
        for chosen in ([keys[1]], [more[0], keys[0], keys[1]], [more[1], more[0], keys[0], keys[1]]):
            table = torch.stack([k.float() for k in chosen], dim=1)
            assert torch.equal(ops.tournament_pick_keys(parents.to(DEV), chosen), ops.tournament_pick(parents.to(DEV), table))
    with pytest.raises(ValueError):
        ops.tournament_pick_keys(parents.to(DEV), [keys[0].double()])
    with pytest.raises(ValueError):
        ops.tournament_pick_keys(parents.to(DEV), [keys[0]] * 5)


def test_tournament_selection_multifit_follows_the_generator(population_path):
    """Same seed, same tournaments as the reference draws them (torch.randint on the fitness device),
    so the winners are those the restatement finds for that draw."""
    if population_path != "pipeline":
        pytest.skip("does not depend on the population path")
    from evox_amd.operators.selection import tournament_selection_multifit

    say("tournament_multifit")
    w = workloads.c1()
    xs, fs, rank, dist = nd_environmental_selection(w.x.to(DEV), w.f.to(DEV), w.topk)
    for n_round, tsize in ((100, 2), (1, 2), (37, 4)):
        torch.manual_seed(123)
        got = tournament_selection_multifit(n_round, [-dist, rank], tsize)
        torch.manual_seed(123)
        parents = torch.randint(0, rank.size(0), (n_round, tsize), device=DEV)
        want = er.tournament_winners(parents.cpu(), [-dist.cpu(), rank.cpu()])
        assert got.shape == want.shape and got.dtype == torch.int64 and got.device.type == "cuda"
        assert torch.equal(got.cpu(), want)
    compiled = torch.compile(lambda p, t: ops_tournament(p, t), fullgraph=True)
    parents = torch.randint(0, rank.size(0), (64, 2), device=DEV)
    table = torch.stack([-dist, rank], dim=1)
    assert torch.equal(compiled(parents, table), ops_tournament(parents, table))


def test_tournament_selection_single_fitness(population_path):
    if population_path != "pipeline":
        pytest.skip("does not depend on the population path")
    from evox_amd.operators.selection import tournament_selection

    say("tournament_single")
    g = torch.Generator("cpu").manual_seed(41)
    fit = torch.randint(0, 50, (500,), generator=g).float() / 4
    fit[torch.rand(500, generator=g) < 0.1] = float("nan")
    fit[torch.rand(500, generator=g) < 0.05] = -float("inf")
    fit[torch.rand(500, generator=g) < 0.05] = -0.0
    fd = fit.to(DEV)
    for n_round, tsize in ((1000, 2), (1, 2), (333, 5)):
        torch.manual_seed(77)
        got = tournament_selection(n_round, fd, tsize)
        torch.manual_seed(77)
        parents = torch.randint(0, 500, (n_round, tsize), device=DEV)
        want = er.tournament_winners_single(parents.cpu(), fit)
        assert got.shape == want.shape and got.dtype == torch.int64 and torch.equal(got.cpu(), want)


def ops_tournament(parents, table):
    from evox_amd import ops

    return ops.tournament_pick(parents, table)


def test_abi_symbols_resolve():
    handle = ctypes.CDLL(_lib.LIB_PATH)
    for name in _lib.EXPORTED_SYMBOLS:
        assert hasattr(handle, name)
