"""Selections of randomly drawn shapes and kinds of population (uniform, on a simplex, partly converged, small
integers, many duplicates, a penalty value on a share of the rows, a few NaN), each against the plain-C checker: ranks,
order and crowding distances of the survivors.  The draws are seeded; the sizes cross the limits between the paths
(one workgroup, peeling from LDS, the sorters of the last front)."""

import numpy as np
import pytest
import torch

from evox_amd import runtime
from evox_amd.operators.selection import nd_environmental_selection
from oracle import c_oracle

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda", 0)
KINDS = ["uniform", "simplex", "partial", "ints", "dups", "penalty", "nan"]


def _population(n, m, kind, rng, g):
    f = torch.rand(n, m, generator=g)
    if kind == "simplex":
        f = f / f.sum(dim=1, keepdim=True)
    elif kind == "partial":
        f = f / f.sum(dim=1, keepdim=True)
        f = f * (1 + 0.05 * torch.randn(n, 1, generator=g).abs())
    elif kind == "ints":
        f = torch.randint(0, int(rng.integers(2, 60)), (n, m), generator=g).float()
    elif kind == "dups":
        k = int(rng.integers(1, max(2, n // 3)))
        f = torch.rand(k, m, generator=g)[torch.randint(0, k, (n,), generator=g)]
    elif kind == "penalty":
        f = f / f.sum(dim=1, keepdim=True)
        f[torch.rand(n, generator=g) < float(rng.uniform(0.1, 0.9))] = 1e10
    elif kind == "nan":
        f[torch.rand(n, generator=g) < 0.02, int(rng.integers(0, m))] = float("nan")
    return f


@pytest.mark.parametrize("seed", [11, 12, 13])
def test_random_shapes_against_the_c_checker(seed):
    rng = np.random.default_rng(seed)
    for case in range(25):
        n = int(rng.choice([rng.integers(2, 1200), rng.integers(1200, 9000), rng.integers(9000, 26000)]))
        m = int(rng.choice([1, 2, 3, 4, 5, 8, 11]))
        kind = str(rng.choice(KINDS))
        g = torch.Generator("cpu").manual_seed(int(rng.integers(1 << 30)))
        f = _population(n, m, kind, rng, g)
        k = int(rng.integers(1, n + 1))
        what = (seed, case, n, m, kind, k)
        print("random_shape", *what, flush=True)
        x = torch.arange(n, dtype=torch.int32, device=DEV)[:, None]
        order, rank, dist, _ = c_oracle.select(f.numpy(), k)
        xs, fs, rs, ds = nd_environmental_selection(x, f.to(DEV), k)
        assert runtime.last_status()["error"] == 0, what
        assert np.array_equal(rs.cpu().numpy(), rank[order]), what
        assert np.array_equal(xs.cpu().numpy()[:, 0].astype(np.int64), order), what
        got, want = ds.cpu().numpy(), dist[order]
        assert np.array_equal(np.isnan(got), np.isnan(want)) and np.array_equal(np.isinf(got), np.isinf(want)), what
        fin = np.isfinite(want)
        np.testing.assert_allclose(got[fin], want[fin], rtol=1e-5, err_msg=str(what))
    runtime.release_workspaces()


def test_more_fronts_than_a_record_tag_counts():
    """One objective, 71 099 distinct values: a front per row, more fronts than the 16-bit tags of the peel's records
    count before they wrap.  The rank of a row is the dense rank of its value; the selection is the stable sort."""
    g = torch.Generator("cpu").manual_seed(3)
    n = 71099
    f = torch.rand(n, 1, generator=g)
    fd = f.to(DEV)
    from evox_amd.operators.selection import non_dominate_rank

    rank = non_dominate_rank(fd)
    st = runtime.last_status()
    want = torch.unique(f[:, 0], return_inverse=True)[1]
    assert st["error"] == 0 and st["fronts"] == int(want.max()) + 1 > 65536
    assert torch.equal(rank.cpu().long(), want)
    x = torch.arange(n, dtype=torch.int32, device=DEV)[:, None]
    xs, _, rs, _ = nd_environmental_selection(x, fd, n // 2)
    order = torch.argsort(f[:, 0], stable=True)[: n // 2]
    assert torch.equal(xs[:, 0].cpu().long(), order) and torch.equal(rs.cpu().long(), want[order])
    runtime.release_workspaces()
