"""Many populations of one shape with more rows than the one-workgroup kernel takes: the stages of the pipeline run
once for several populations at a time (``evox_hip_many_*``).  Every population's result must equal what the
single-population entry points give for it alone, and the C checker's.  The reference reaches this through vmap
(src/evox/operators/selection/non_dominate.py:107-125, src/evox/utils/op_register.py:26-51)."""

import numpy as np
import pytest
import torch

from evox_amd import _lib, runtime
from evox_amd.operators.selection import nd_environmental_selection, non_dominate_rank, non_dominate_rank_until
from oracle import c_oracle
from tests.cases import as_np

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda", 0)


@pytest.fixture(autouse=True)
def through_the_pipeline():
    runtime.use_small_population_kernel = False
    yield
    runtime.use_small_population_kernel = None


def _populations(batch, n, m, seed, kind):
    g = torch.Generator("cpu").manual_seed(seed)
    f = torch.rand(batch, n, m, generator=g)
    if kind == "ties":  # ties in every objective, duplicate rows, a NaN row, an infinity, signed zeros
        f = (f * 12).round() / 12
        f[:, 5] = f[:, 6]
        f[0, 9, 0] = float("nan")
        f[batch - 1, 11, m - 1] = float("inf")
        f[batch // 2, 3, 0], f[batch // 2, 4, 0] = 0.0, -0.0
    elif kind == "fronts":  # population b has about b + 1 fronts of very different sizes
        for b in range(batch):
            f[b] = f[b] + torch.randint(0, b + 1, (n, 1), generator=g).float()
    elif kind == "one_front":
        f = f / f.sum(dim=-1, keepdim=True)
    x = torch.rand(batch, n, 5, generator=g)
    return f, x


def _per_launch(batch, n, m, stop):
    return int(_lib.lib().evox_hip_many_populations_per_launch(batch, n, m, stop))


SHAPES = [  # batch, n, m, kind
    (16, 4096, 3, "uniform"), (5, 2000, 2, "ties"), (7, 1500, 5, "fronts"), (30, 1100, 3, "uniform"), (2, 9000, 8, "uniform"),
    (4, 3000, 16, "ties"), (3, 1300, 17, "uniform"), (6, 2500, 3, "one_front"), (9, 5000, 4, "fronts"), (3, 20000, 3, "uniform"),
    (12, 1025, 1, "ties"), (2, 12000, 3, "one_front"),
    # two objectives above the rows of the one-workgroup kernel: alone they go through the chain of workgroups,
    # together through the kernels that they share
    (6, 5000, 2, "ties"), (3, 9000, 2, "fronts"),
]


@pytest.mark.parametrize("batch,n,m,kind", SHAPES, ids=[f"{b}x{n}x{m}-{k}" for b, n, m, k in SHAPES])
def test_ranks_of_many_populations(batch, n, m, kind):
    f, _ = _populations(batch, n, m, 100 + batch + n + m, kind)
    fd = f.to(DEV)
    got = non_dominate_rank(fd)
    status = runtime.last_status()
    assert status["error"] == 0
    assert got.shape == (batch, n) and got.dtype == torch.int32
    stop = n // 3
    until = non_dominate_rank_until(fd, stop)
    for b in range(batch):
        want, _fronts = c_oracle.nd_rank(f[b])
        assert np.array_equal(as_np(got[b]), as_np(want)), (b, "all ranks")
        alone = non_dominate_rank_until(fd[b], stop)
        assert torch.equal(until[b], alone), (b, "ranks up to the cut")


@pytest.mark.parametrize("batch,n,m,kind", SHAPES, ids=[f"{b}x{n}x{m}-{k}" for b, n, m, k in SHAPES])
def test_selection_of_many_populations(batch, n, m, kind):
    f, x = _populations(batch, n, m, 200 + batch + n + m, kind)
    fd, xd = f.to(DEV), x.to(DEV)
    for topk in (n // 2, 1, n):
        got = nd_environmental_selection(xd, fd, topk)
        assert runtime.last_status()["error"] == 0
        assert got[0].shape == (batch, topk, 5) and got[1].shape == (batch, topk, m)
        for b in range(batch):
            alone = nd_environmental_selection(xd[b], fd[b], topk)
            for part, (a, c) in enumerate(zip(got, alone)):
                assert np.array_equal(as_np(a[b]), as_np(c), equal_nan=True), (topk, b, part)
    # against the C checker: the order of the selected rows and their ranks
    topk = n // 2
    got = nd_environmental_selection(torch.arange(n, device=DEV, dtype=torch.float32)[None, :, None].repeat(batch, 1, 1), fd, topk)
    for b in range(0, batch, max(1, batch // 3)):
        order, rank, _dist, _fronts = c_oracle.select(f[b], topk)
        assert np.array_equal(as_np(got[0][b, :, 0]).astype(np.int64), as_np(order)[:topk]), b
        assert np.array_equal(as_np(got[2][b]), as_np(rank)[as_np(order)[:topk]]), b


def test_shares_and_passes():
    """How many populations share a launch: all of a small batch, even passes for a larger one, one at a time where
    a population needs the whole device (then the library runs them one after the other)."""
    assert _per_launch(16, 4096, 3, 2048) == 16
    assert _per_launch(30, 1100, 3, 550) in (15, 30)  # (30 where two workgroups of the peel share a compute unit)
    assert 2 <= _per_launch(500, 1100, 3, 550) <= 113
    assert _per_launch(3, 20000, 3, 10000) == 1
    assert _per_launch(1, 4096, 3, 2048) == 1
    with runtime.options(peel_stepped=1):
        assert _per_launch(16, 4096, 3, 2048) == 1
    with runtime.options(peel_lds=0):
        assert _per_launch(16, 4096, 3, 2048) == 1


def test_vmap_strides_and_dtypes():
    f, x = _populations(6, 2048, 3, 7, "ties")
    fd, xd = f.to(DEV), x.to(DEV)
    want = nd_environmental_selection(xd, fd, 1000)
    # populations along another dimension (strided batch), float16 decision vectors, no decision columns at all
    f_t = fd.permute(1, 0, 2).contiguous()  # (n, batch, m)
    x_t = xd.permute(1, 0, 2).contiguous()
    mapped = torch.vmap(lambda a, b: nd_environmental_selection(a, b, 1000), in_dims=(1, 1))(x_t, f_t)
    for a, c in zip(mapped, want):
        assert np.array_equal(as_np(a), as_np(c), equal_nan=True)
    ranks = torch.vmap(non_dominate_rank, in_dims=1)(f_t)
    assert torch.equal(ranks, non_dominate_rank(fd))
    half = nd_environmental_selection(xd.half(), fd, 1000)
    assert half[0].dtype == torch.float16 and torch.equal(half[0], want[0].half()) and torch.equal(half[2], want[2])
    none = nd_environmental_selection(xd[:, :, :0], fd, 1000)
    assert none[0].shape == (6, 1000, 0) and torch.equal(none[2], want[2])
    nested = torch.vmap(torch.vmap(non_dominate_rank))(fd.view(2, 3, 2048, 3))
    assert torch.equal(nested.view(6, 2048), ranks)


def test_a_wait_that_runs_out_poisons_every_population():
    f, x = _populations(8, 3000, 3, 9, "uniform")
    with runtime.options(spin_limit=1):
        rank = non_dominate_rank(f.to(DEV))
        with pytest.raises(_lib.EvoxHipError):
            runtime.last_status()
        got = nd_environmental_selection(x.to(DEV), f.to(DEV), 1500)
    torch.cuda.synchronize()
    bad = (as_np(rank) == -1).all(axis=1)
    assert bad.any()  # (a population whose workgroups never had to wait for each other may come through)
    for b in range(8):
        if not bad[b]:
            want, _fronts = c_oracle.nd_rank(f[b])
            assert np.array_equal(as_np(rank[b]), as_np(want))
    poisoned = (as_np(got[2]) == -1).all(axis=1)
    assert np.array_equal(np.isnan(as_np(got[3])).all(axis=1), poisoned)
    # with the status checked, the call is issued once more through the kernels that never wait
    runtime.CHECK_STATUS = True
    try:
        with runtime.options(spin_limit=1):
            again = non_dominate_rank(f.to(DEV))
    finally:
        runtime.CHECK_STATUS = False
    for b in range(8):
        want, _fronts = c_oracle.nd_rank(f[b])
        assert np.array_equal(as_np(again[b]), as_np(want))


@pytest.mark.parametrize("batch,n,m,kind", [(5, 3000, 3, "ties"), (12, 1500, 2, "uniform"), (3, 40000, 3, "uniform"),
                                            (4, 9000, 8, "one_front"), (2, 2000, 17, "ties"), (70, 1100, 3, "fronts")])
def test_first_front_and_crowding_of_many_populations(batch, n, m, kind):
    """The first-front mask and the crowding distances under leading batch dimensions: one set of launches for all
    populations, the same results as population by population."""
    from evox_amd.operators.selection import crowding_distance, non_dominated_mask
    from oracle import eager_restatement as er

    f, _ = _populations(batch, n, m, 300 + batch + n + m, kind)
    fd = f.to(DEV)
    first = non_dominated_mask(fd)
    assert first.shape == (batch, n) and first.dtype == torch.bool
    g = torch.Generator("cpu").manual_seed(batch)
    mask = torch.rand(batch, n, generator=g) < 0.3
    mask[0] = False  # an empty selection
    mask[batch - 1] = True
    maskd = mask.to(DEV)
    dist_all = crowding_distance(fd, None)
    dist_masked = crowding_distance(fd, maskd)
    dist_front = crowding_distance(fd, first)
    assert runtime.last_status()["error"] == 0
    for b in range(batch):
        assert torch.equal(first[b], non_dominated_mask(fd[b])), b
        for got, mk in ((dist_all, None), (dist_masked, maskd[b]), (dist_front, first[b])):
            assert np.array_equal(as_np(got[b]), as_np(crowding_distance(fd[b], mk)), equal_nan=True), b
    for b in range(0, batch, max(1, batch // 2)):
        want_first = as_np(c_oracle.nd_rank(f[b])[0]) == 0
        assert np.array_equal(as_np(first[b]), want_first), b
        want = as_np(er.crowding(f[b], mask[b]))
        got = as_np(dist_masked[b])
        fin = np.isfinite(want)
        assert np.array_equal(np.isfinite(got), fin) and np.array_equal(got[~fin], want[~fin], equal_nan=True), b
        np.testing.assert_allclose(got[fin], want[fin], rtol=1e-5)
    # a mask that is a strided view, populations along the second dimension
    mapped = torch.vmap(crowding_distance, in_dims=(1, 1))(fd.permute(1, 0, 2).contiguous(), maskd.t().contiguous())
    assert np.array_equal(as_np(mapped), as_np(dist_masked), equal_nan=True)


def test_chains_of_two_objective_populations_share_a_launch_and_report_a_wait_that_runs_out():
    """Two objectives above 4096 rows: every population is a chain of workgroups of its own, all chains in one launch."""
    assert _per_launch(16, 10000, 2, 5000) == 16 and _per_launch(300, 5000, 2, 5000) > 100
    f, x = _populations(5, 6000, 2, 11, "fronts")
    fd, xd = f.to(DEV), x.to(DEV)
    with runtime.options(spin_limit=1):
        rank = non_dominate_rank(fd)
        with pytest.raises(_lib.EvoxHipError):
            runtime.last_status()
        got = nd_environmental_selection(xd, fd, 3000)
    torch.cuda.synchronize()
    for b in range(5):
        r = as_np(rank[b])
        if not (r == -1).all():  # (a chain of two workgroups may come through: the second one's first load can succeed)
            assert np.array_equal(r, as_np(c_oracle.nd_rank(f[b])[0])), b
        assert (as_np(got[2][b]) == -1).all() == bool(np.isnan(as_np(got[3][b])).all()), b
    assert (as_np(rank) == -1).all(axis=1).any()
    with runtime.options(two_min_rows=0):  # the matrix kernels for the same batch
        other = nd_environmental_selection(xd, fd, 3000)
    good = nd_environmental_selection(xd, fd, 3000)
    for a, c in zip(good, other):
        assert np.array_equal(as_np(a), as_np(c), equal_nan=True)
