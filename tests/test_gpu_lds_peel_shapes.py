"""Shapes chosen for the kernel that peels from LDS (populations whose dominance matrix fits the LDS of the device),
each against the plain-C checker: the largest populations that still fit, one front that holds every row (records
overflow into the bitmaps, the last front is too large for the kernel's own ordering), few large fronts, a single
objective (a front per distinct value), all rows equal, a chain, and selections whose cut falls into the first and
into the last front."""

import ctypes

import numpy as np
import pytest
import torch

from evox_amd import _lib, runtime
from evox_amd.operators.selection import nd_environmental_selection, non_dominate_rank
from oracle import c_oracle
from tests.cases import as_np

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda", 0)


def _peeled_from_lds(n, m):
    out = (ctypes.c_int64 * 3)()
    _lib.call("evox_hip_peel_plan", n, m, out)
    return bool(out[0])


def _cases():
    g = torch.Generator("cpu").manual_seed(99)
    cases = {}
    cases["uniform_23000x3"] = (torch.rand(23000, 3, generator=g), [1, 11500, 23000])
    cases["uniform_22500x4"] = (torch.rand(22500, 4, generator=g), [11250])
    a = torch.rand(20000, generator=g)
    cases["one_front_20000x2"] = (torch.stack([a, -a], dim=1), [1, 9999, 20000])
    cases["few_fronts_16000x2"] = (torch.stack([a[:16000], (-a[:16000] * 4).floor() + torch.randint(0, 3, (16000,), generator=g)], dim=1), [8000])
    cases["one_objective_12000"] = (torch.randint(0, 50, (12000, 1), generator=g).float(), [1, 6000, 12000])
    cases["all_equal_6000x3"] = (torch.full((6000, 3), 2.5), [1, 3000, 6000])
    chain = torch.arange(5000, dtype=torch.float32)[:, None].repeat(1, 2)
    cases["chain_5000x2"] = (chain[torch.randperm(5000, generator=g)], [1, 2500, 5000])
    dup = torch.rand(300, 3, generator=g)
    cases["duplicates_9000x3"] = (dup[torch.randint(0, 300, (9000,), generator=g)], [4500])
    nan = torch.rand(10000, 3, generator=g)
    nan[::17, 1] = float("nan")
    cases["nan_rows_10000x3"] = (nan, [5000])
    return cases


CASES = _cases()


@pytest.mark.parametrize("name", sorted(CASES))
def test_lds_peel_shapes_against_the_c_checker(name):
    f, ks = CASES[name]
    n, m = f.shape
    assert _peeled_from_lds(n, m), "the case is meant for the kernel that peels from LDS"
    fd = f.to(DEV)
    want_rank, fronts = c_oracle.nd_rank(as_np(f))
    got = non_dominate_rank(fd)
    st = runtime.last_status()
    assert st["error"] == 0 and st["fronts"] == fronts
    assert np.array_equal(as_np(got), want_rank)
    x = torch.arange(n, dtype=torch.int32, device=DEV)[:, None]
    for k in ks:
        order, rank, dist, _ = c_oracle.select(as_np(f), k)
        xs, fs, rs, ds = nd_environmental_selection(x, fd, k)
        assert runtime.last_status()["error"] == 0
        assert np.array_equal(as_np(rs), rank[order]), (name, k)
        gd, wd = as_np(ds), dist[order]
        assert np.array_equal(np.isnan(gd), np.isnan(wd)) and np.array_equal(np.isinf(gd), np.isinf(wd)), (name, k)
        fin = np.isfinite(wd)
        np.testing.assert_allclose(gd[fin], wd[fin], rtol=1e-5)
        assert np.array_equal(as_np(xs)[:, 0].astype(np.int64), order), (name, k)
    runtime.release_workspaces()
