"""Two objectives ranked without a dominance matrix (rows sorted by (f1, f2, index); every front is the set of strict
prefix minima of f2 among the rows that remain; the minima handed from workgroup to workgroup) against the CPU
restatement, the C checker and the matrix path of the same library.  Reference semantics:
src/evox/operators/selection/non_dominate.py:6-26 (the relation), :161-195 (the fronts)."""

import numpy as np
import pytest
import torch

from evox_amd import runtime
from evox_amd.operators.selection import (nd_environmental_selection, nd_environmental_selection_two_part, non_dominate_rank,
                                          non_dominate_rank_until)
from oracle import c_oracle
from oracle import eager_restatement as er
from tests.cases import as_np, edge_cases

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda", 0)
TWO = [c for c in edge_cases() if c[1].size(1) == 2]


@pytest.fixture(autouse=True)
def through_the_pipeline():
    runtime.use_small_population_kernel = False
    yield
    runtime.use_small_population_kernel = None


@pytest.mark.parametrize("name,f,ks", TWO, ids=[c[0] for c in TWO])
def test_two_objective_edge_cases(name, f, ks):
    x = torch.arange(f.size(0), dtype=torch.float32)[:, None]
    with runtime.options(two_min_rows=1):
        assert np.array_equal(as_np(non_dominate_rank(f.to(DEV))), as_np(er.ranks_by_peeling(f))), name
        for k in ks:
            got = nd_environmental_selection(x.to(DEV), f.to(DEV), k)
            want = er.environmental_selection(x, f, k)
            assert torch.equal(got[0].cpu(), want[0]) and torch.equal(got[2].cpu(), want[2]), (name, k)
            assert np.array_equal(as_np(got[3]), as_np(want[3]), equal_nan=True) or np.allclose(
                as_np(got[3]), as_np(want[3]), rtol=1e-5, equal_nan=True), (name, k)
        assert runtime.last_status()["error"] == 0


def _populations():
    g = torch.Generator("cpu").manual_seed(2222)
    out = {}
    out["uniform_5000"] = torch.rand(5000, 2, generator=g)
    out["uniform_20000"] = torch.rand(20000, 2, generator=g)
    out["uniform_70000"] = torch.rand(70000, 2, generator=g)
    q = (torch.rand(30000, 2, generator=g) * 40).round() / 40  # heavy ties and thousands of identical rows
    q[::97, 0] = float("nan")
    q[5::211, 1] = float("inf")
    q[9::307, 0] = float("-inf")
    out["quantised_with_nan_and_inf_30000"] = q
    t = torch.arange(6000, dtype=torch.float32)
    out["chain_6000"] = torch.stack([t, t], dim=1)[torch.randperm(6000, generator=g)]  # as many fronts as rows
    u = torch.arange(9000, dtype=torch.float32)
    out["one_front_9000"] = torch.stack([u, -u], dim=1)[torch.randperm(9000, generator=g)]
    z = torch.zeros(8192, 2)
    z[::2, 0] = -0.0
    z[1::3, 1] = -0.0
    out["signed_zeros_all_equal_8192"] = z
    layered = []
    for layer in range(40):  # 40 layers of the line f1 + f2 = layer + 1, values on a grid of 1/64
        a = (torch.rand(250, generator=g) * (layer + 1) * 64).round() / 64
        layered.append(torch.stack([a, (layer + 1) - a], dim=1))
    out["layered_10000"] = torch.cat(layered)[torch.randperm(10000, generator=g)]
    return out


POPS = _populations()


@pytest.mark.parametrize("name", sorted(POPS))
def test_two_objective_populations_against_the_checker(name):
    f = POPS[name]
    n = f.size(0)
    want = c_oracle.nd_rank(f.numpy())[0]
    fd = f.to(DEV)
    got = as_np(non_dominate_rank(fd))
    assert runtime.last_status()["error"] == 0
    assert np.array_equal(got, want), name
    with runtime.options(two_min_rows=0):  # the matrix path of the same library
        assert np.array_equal(as_np(non_dominate_rank(fd)), want), name
    topk = n // 2
    order, rank, dist, _ = c_oracle.select(f.numpy(), topk)
    x = torch.arange(n, dtype=torch.int32)[:, None]
    with runtime.options(two_min_rows=1):  # (by default a population of up to 4096 rows takes the matrix, or the one-workgroup kernel)
        sel = nd_environmental_selection(x.to(DEV), fd, topk)
        until = as_np(non_dominate_rank_until(fd, topk + 1))
    assert np.array_equal(as_np(sel[2]), rank[order]), name
    gd, wd = as_np(sel[3]), dist[order]
    fin = np.isfinite(wd)
    assert np.array_equal(np.isfinite(gd), fin) and np.array_equal(np.isnan(gd), np.isnan(wd)), name
    np.testing.assert_allclose(gd[fin], wd[fin], rtol=1e-5, err_msg=name)
    if not np.array_equal(as_np(sel[0])[:, 0], order):
        # rows may only change places where their distances tie within rounding at the cut
        assert sorted(as_np(sel[0])[:, 0].tolist()) == sorted(order.tolist()) or np.allclose(np.sort(gd[fin]), np.sort(wd[fin]), rtol=1e-5), name
    worst = np.sort(want)[topk]
    assert np.array_equal(until, np.where(want <= worst, want, 2**31 - 1)), name


def test_two_objectives_in_two_parts_and_with_strides():
    g = torch.Generator("cpu").manual_seed(2223)
    f = (torch.rand(12000, 2, generator=g) * 500).round() / 500
    x = torch.rand(12000, 5, generator=g)
    want = er.environmental_selection(x, f, 5000)
    with runtime.options(two_min_rows=1):
        got = nd_environmental_selection_two_part(x[:7000].to(DEV), f[:7000].to(DEV), x[7000:].to(DEV), f[7000:].to(DEV), 5000)
    for a, b in zip(got[:3], want[:3]):
        assert torch.equal(a.cpu(), b)
    wide = torch.zeros(12000, 5)
    wide[:, 1:4:2] = f
    assert np.array_equal(as_np(non_dominate_rank(wide.to(DEV)[:, 1:4:2])), as_np(er.ranks_by_peeling(f)))


def _stop_cases():
    g = torch.Generator("cpu").manual_seed(2224)
    out = {}
    # the first workgroup holds a chain of 4096 rows (its own front each), the others two fronts: the fronts so far hold
    # the rows asked for after two rounds, while the first workgroup has thousands of rounds before it
    t = torch.arange(4096, dtype=torch.float32)
    chain = torch.stack([t * 1e-3, 100.0 + t], dim=1)
    a = torch.rand(12000, generator=g)
    rest = torch.stack([10.0 + a, 1.0 - a + (torch.rand(12000, generator=g) < 0.5).float() * 2.0], dim=1)
    out["chain_in_the_first_workgroup"] = torch.cat([chain, rest])
    # every row four times: only the first copy of a row counts while the peeling looks for its end, so it goes on
    # beyond the front that holds the rows asked for
    u = torch.rand(5000, 2, generator=g)
    out["every_row_four_times"] = u.repeat(4, 1)[torch.randperm(20000, generator=g)]
    # few fronts, all of them large: the cut falls into the first rounds of a chain of ten workgroups
    b = torch.rand(40000, generator=g)
    out["five_lines"] = torch.stack([b, 1.0 - b + torch.randint(0, 5, (40000,), generator=g).float()], dim=1)
    # more rounds than the ring of hand-over words holds, three times over
    c = torch.rand(9000, 2, generator=g)
    out["many_fronts"] = c + torch.arange(9000)[:, None].float().div(9).floor() * 0.01
    out["uniform_60000"] = torch.rand(60000, 2, generator=g)
    return out


STOPS = _stop_cases()


@pytest.mark.parametrize("name", sorted(STOPS))
def test_the_peeling_may_end_at_the_cut(name):
    """Selections and ranks up to a cut, where the chain of workgroups stops peeling once the fronts so far hold the rows
    asked for: every stop count gives the checker's ranks up to its cut front and the same selection as all ranks do."""
    f = STOPS[name]
    n = f.size(0)
    fd = f.to(DEV)
    want, _fronts = c_oracle.nd_rank(f)
    want = as_np(want)
    assert np.array_equal(as_np(non_dominate_rank(fd)), want), name
    x = torch.arange(n, dtype=torch.int32)[:, None].to(DEV)
    for topk in (1, 7, n // 10, n // 2, n - 1, n):
        until = as_np(non_dominate_rank_until(fd, topk))
        worst = np.sort(want)[topk - 1]
        assert np.array_equal(until, np.where(want <= worst, want, 2**31 - 1)), (name, topk)
        if n > 30000 and topk != n // 2:  # (the checker's selection of that many rows takes seconds)
            continue
        sel = nd_environmental_selection(x, fd, topk)
        status = runtime.last_status()
        assert status["error"] == 0 and status["fronts"] == worst + 1, (name, topk, status)
        order, rank, dist, _ = c_oracle.select(f.numpy(), topk)
        order, rank, dist = as_np(order)[:topk], as_np(rank), as_np(dist)
        assert np.array_equal(as_np(sel[2]), rank[order]), (name, topk)
        gd, wd = as_np(sel[3]), dist[order]
        fin = np.isfinite(wd)
        assert np.array_equal(np.isfinite(gd), fin), (name, topk)
        np.testing.assert_allclose(gd[fin], wd[fin], rtol=1e-5, err_msg=f"{name} {topk}")
        got_rows = as_np(sel[0])[:, 0]
        if not np.array_equal(got_rows, order):  # rows may only change places where their distances tie within rounding
            assert np.allclose(np.sort(gd[fin]), np.sort(wd[fin]), rtol=1e-5), (name, topk)
            assert np.array_equal(np.sort(got_rows[rank[got_rows] < worst]), np.sort(order[rank[order] < worst])), (name, topk)


def test_a_wait_that_runs_out_in_the_chain_is_reported():
    f = torch.rand(60000, 2, generator=torch.Generator("cpu").manual_seed(2225))
    fd = f.to(DEV)
    x = torch.arange(60000, dtype=torch.float32)[:, None].to(DEV)
    with runtime.options(spin_limit=1):
        rank = non_dominate_rank(fd)
        with pytest.raises(Exception):
            runtime.last_status()
        sel = nd_environmental_selection(x, fd, 30000)
    torch.cuda.synchronize()
    assert (as_np(rank) == -1).all() and (as_np(sel[2]) == -1).all() and np.isnan(as_np(sel[3])).all()
    # ... and with the status checked, the call comes through on the kernels that never wait
    runtime.CHECK_STATUS = True
    try:
        with runtime.options(spin_limit=1):
            again = non_dominate_rank(fd)
    finally:
        runtime.CHECK_STATUS = False
    assert np.array_equal(as_np(again), as_np(c_oracle.nd_rank(f)[0]))


def test_half_a_million_rows_on_a_grid():
    """The points (i, j) of a 707 x 707 grid: the rank of a point is i + j (1413 fronts, 131 workgroups in the chain,
    five rings of hand-over words), which no checker has to compute."""
    side = 707
    n = side * side
    i, j = np.divmod(np.arange(n), side)
    perm = np.random.default_rng(side).permutation(n)
    f = torch.from_numpy(np.stack([i, j], 1).astype(np.float32)[perm])
    want = (i + j)[perm]
    fd = f.to(DEV)
    assert np.array_equal(as_np(non_dominate_rank(fd)), want)
    assert runtime.last_status()["error"] == 0
    x = torch.arange(n, dtype=torch.float32, device=DEV)[:, None]
    for topk in (1000, n // 2):
        worst = np.sort(want)[topk - 1]
        assert np.array_equal(as_np(non_dominate_rank_until(fd, topk)), np.where(want <= worst, want, 2**31 - 1)), topk
        sel = nd_environmental_selection(x, fd, topk)
        status = runtime.last_status()
        assert status["error"] == 0 and status["fronts"] == worst + 1, status
        rows = as_np(sel[0])[:, 0].astype(np.int64)
        assert len(np.unique(rows)) == topk and np.array_equal(as_np(sel[2]), want[rows]), topk
        assert np.array_equal(np.sort(rows[want[rows] < worst]), np.flatnonzero(want < worst)), topk
