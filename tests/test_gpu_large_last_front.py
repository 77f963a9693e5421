"""Last fronts of more than 1024 rows in populations of at most 32 768 rows -- a converged population, where most
rows are non-dominated -- whose per-objective orders and distance order come from workgroups that sort in LDS: against
the plain-C checker, against the radix path (option ``mid_argsort`` off), and ``crowding_distance`` on masks of that
size.  Ties in an objective (equal costs keep their row order), duplicate rows, a NaN objective, the largest
population of the path and cuts that take one row, half and all of the front."""

import numpy as np
import pytest
import torch

from evox_amd import runtime
from evox_amd.operators.selection import crowding_distance, nd_environmental_selection
from oracle import c_oracle
from tests.cases import as_np

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda", 0)


def _simplex(n, m, g):
    f = torch.rand(n, m, generator=g)
    return f / f.sum(dim=1, keepdim=True)


def _cases():
    g = torch.Generator("cpu").manual_seed(1234)
    cases = {}
    cases["simplex_20000x3"] = (_simplex(20000, 3, g), [1, 10000, 20000])
    cases["simplex_24576x2"] = (_simplex(24576, 2, g), [12288])
    cases["simplex_32768x3"] = (_simplex(32768, 3, g), [16384])  # the largest population of the path
    most = _simplex(26000, 3, g)
    most[24000:] = most[24000:] * 1.5 + 0.1  # a population that gets the small tables, a front that would fit the large ones
    cases["front0_24000_of_26000x3"] = (most, [13000])
    cases["simplex_12000x5"] = (_simplex(12000, 5, g), [6000])
    mixed = _simplex(20000, 3, g)
    mixed[14000:] = mixed[14000:] * 1.5 + 0.1  # 30 % of the rows dominated: the cut falls into front 0 of 14 000 rows
    cases["front0_14000_of_20000x3"] = (mixed[torch.randperm(20000, generator=g)], [10000, 13999])
    ties = torch.randint(0, 200, (16000, 3), generator=g).float()
    ties[:, 2] = 400 - ties[:, 0] - ties[:, 1]  # one plane, many equal costs per objective, duplicate rows
    cases["ties_on_a_plane_16000x3"] = (ties, [8000])
    a = torch.rand(9000, generator=g)
    cases["two_objectives_9000_smallest_of_the_path"] = (torch.stack([a, -a], dim=1), [4500])
    wide = _simplex(9000, 16, g)
    cases["simplex_9000x16"] = (wide, [4500])
    cases["simplex_2000x3"] = (_simplex(2000, 3, g), [1, 1000, 2000])
    cases["simplex_5000x4"] = (_simplex(5000, 4, g), [2500])
    small = _simplex(3000, 3, g)
    small[1100:] = small[1100:] * 1.5 + 0.1  # a front of 1100 rows, just above the smallest that is sorted this way
    cases["front0_1100_of_3000x3"] = (small, [1000])
    # larger populations: the front goes to a launch of its own beside the one that holds the radix sort
    big = _simplex(40000, 3, g)
    big[9000:] = big[9000:] * 1.5 + 0.1  # front 0 of 9000 rows, ordered by objective and by distance in LDS
    cases["front0_9000_of_40000x3"] = (big[torch.randperm(40000, generator=g)], [5000])
    big2 = _simplex(40000, 4, g)
    big2[30000:] = big2[30000:] * 1.5 + 0.1  # front 0 of 30 000 rows
    cases["front0_30000_of_40000x4"] = (big2, [20000])
    big3 = _simplex(70000, 3, g)
    big3[20000:] = big3[20000:] * (1.5 + torch.rand(50000, 1, generator=g)) + 0.1  # (a population whose matrix comes from the objective orders)
    cases["front0_20000_of_70000x3"] = (big3, [12000])
    return cases


CASES = _cases()


def _check(f, k, got, name):
    order, rank, dist, _ = c_oracle.select(as_np(f), k)
    xs, fs, rs, ds = got
    assert np.array_equal(as_np(rs), rank[order]), (name, k)
    gd, wd = as_np(ds), dist[order]
    assert np.array_equal(np.isnan(gd), np.isnan(wd)) and np.array_equal(np.isinf(gd), np.isinf(wd)), (name, k)
    fin = np.isfinite(wd)
    np.testing.assert_allclose(gd[fin], wd[fin], rtol=1e-5)
    assert np.array_equal(as_np(xs)[:, 0].astype(np.int64), order), (name, k)


@pytest.mark.parametrize("name", sorted(CASES))
def test_large_last_front_against_the_c_checker_and_the_radix_path(name):
    f, ks = CASES[name]
    n, m = f.shape
    fd = f.to(DEV)
    x = torch.arange(n, dtype=torch.int32, device=DEV)[:, None]
    for k in ks:
        got = nd_environmental_selection(x, fd, k)
        st = runtime.last_status()
        assert st["error"] == 0 and st["last_front_size"] > 1024, st
        _check(f, k, got, name)
        with runtime.options(mid_argsort=0):
            old = nd_environmental_selection(x, fd, k)
            assert runtime.last_status()["error"] == 0
        for a, b in zip(got, old):
            assert torch.equal(a, b) or torch.equal(torch.nan_to_num(a.float(), nan=-7.0), torch.nan_to_num(b.float(), nan=-7.0)), (name, k)
    runtime.release_workspaces()


@pytest.mark.parametrize("n,m,keep", [(20000, 3, 1.0), (24576, 2, 0.6), (10000, 8, 0.9), (50000, 3, 0.4), (40000, 2, 1.0)])
def test_crowding_distance_of_a_large_mask(n, m, keep):
    g = torch.Generator("cpu").manual_seed(n + m)
    costs = torch.rand(n, m, generator=g)
    whole = n // 5 * 5
    costs[0:whole:5, 0] = costs[1:whole:5, 0]  # ties in an objective
    mask = torch.rand(n, generator=g) < keep
    want = c_oracle.crowding(as_np(costs), as_np(mask))
    got = as_np(crowding_distance(costs.to(DEV), mask.to(DEV)))
    with runtime.options(mid_argsort=0):
        old = as_np(crowding_distance(costs.to(DEV), mask.to(DEV)))
    assert np.array_equal(np.isinf(got), np.isinf(want))
    fin = np.isfinite(want)
    np.testing.assert_allclose(got[fin], want[fin], rtol=1e-5)
    assert np.array_equal(got, old)
    runtime.release_workspaces()
