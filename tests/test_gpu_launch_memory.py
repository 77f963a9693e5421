"""The choice of launches after the peel follows what the last selection of the same shape found (a word of pinned
host memory that the last kernel of a selection writes).  Whatever it says, stale or not, the results are those of
the plain-C checker: selections with a small and with a large last front take turns here, so that every call meets
the word left by a call of the other kind, and a run of equal calls meets its own."""

import numpy as np
import pytest
import torch

from evox_amd import runtime
from evox_amd.operators.selection import nd_environmental_selection
from oracle import c_oracle
from tests.cases import as_np

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda", 0)


@pytest.fixture(autouse=True)
def through_the_pipeline():
    runtime.use_small_population_kernel = False  # (the one-workgroup kernels have no such choice to make)
    yield
    runtime.use_small_population_kernel = None


def _check(f, k, got):
    order, rank, dist, _ = c_oracle.select(as_np(f), k)
    xs, fs, rs, ds = got
    assert np.array_equal(as_np(xs)[:, 0].astype(np.int64), order)
    assert np.array_equal(as_np(rs), rank[order])
    gd, wd = as_np(ds), dist[order]
    assert np.array_equal(np.isinf(gd), np.isinf(wd))
    fin = np.isfinite(wd)
    np.testing.assert_allclose(gd[fin], wd[fin], rtol=1e-5)


@pytest.mark.parametrize("n,m", [(6000, 3), (3000, 2)])
def test_small_and_large_last_fronts_in_turn(n, m):
    g = torch.Generator("cpu").manual_seed(n + m)
    uniform = torch.rand(n, m, generator=g)  # many fronts, the last one small: the peel kernel orders it
    simplex = torch.rand(n, m, generator=g)
    simplex = simplex / simplex.sum(dim=1, keepdim=True)  # one front: the ordering kernels have it
    x = torch.arange(n, dtype=torch.int32, device=DEV)[:, None]
    sizes = []
    for f in (uniform, uniform, simplex, simplex, uniform, simplex, uniform, uniform):
        got = nd_environmental_selection(x, f.to(DEV), n // 2)
        st = runtime.last_status()
        assert st["error"] == 0
        sizes.append(st["last_front_size"])
        _check(f, n // 2, got)
    assert min(sizes) < 1024 < max(sizes), sizes  # both kinds of last front were met
    with runtime.options(launch_memory=0):
        for f in (simplex, uniform):
            _check(f, n // 2, nd_environmental_selection(x, f.to(DEV), n // 2))
    runtime.release_workspaces()


def test_counting_first_follows_what_front_0_held():
    """40 000 rows of eight objectives get their matrix from the per-objective orders.  After two selections that
    found every row they keep in front 0, the next one counts dominators first and builds the matrix only if front 0
    falls short: populations with a large and with a small front 0, and one with an infinity, take turns, so that
    every kind of call meets every state of the word."""
    n, m, k = 40000, 8, 5000
    g = torch.Generator("cpu").manual_seed(408)
    wide = torch.rand(n, m, generator=g)  # thousands of rows in front 0
    deep = torch.rand(n, m, generator=g) + (torch.arange(n) % 64)[:, None].float()  # a few hundred
    holed = wide.clone()
    holed[torch.randperm(n, generator=g)[:200], 3] = float("inf")
    want = {}
    x = torch.arange(n, dtype=torch.int32, device=DEV)[:, None]
    front0 = {}
    for name, f in (("wide", wide), ("deep", deep), ("holed", holed)):
        want[name] = c_oracle.select(as_np(f), k)
        front0[name] = int((want[name][1] == 0).sum())
    assert front0["wide"] >= k > front0["deep"], front0

    def run(name, f):
        print("count first:", name, flush=True)
        xs, fs, rs, ds = nd_environmental_selection(x, f.to(DEV), k)
        assert runtime.last_status()["error"] == 0
        order, rank, dist, _ = want[name]
        assert np.array_equal(as_np(xs)[:, 0].astype(np.int64), order), name
        assert np.array_equal(as_np(rs), rank[order]), name
        gd, wd = as_np(ds), dist[order]
        assert np.array_equal(np.isinf(gd), np.isinf(wd)), name
        fin = np.isfinite(wd)
        np.testing.assert_allclose(gd[fin], wd[fin], rtol=1e-4)

    turns = ["wide", "wide", "wide", "wide", "deep", "deep", "wide", "wide", "holed", "wide", "wide", "wide", "holed",
             "deep", "wide"]
    table = {"wide": wide, "deep": deep, "holed": holed}
    for name in turns:
        run(name, table[name])
    with runtime.options(prefix_count_first=0):
        for name in ("wide", "wide", "wide", "deep"):
            run(name, table[name])
    runtime.release_workspaces()


def test_a_graph_captured_while_counting_first_builds_the_matrix_when_a_replay_needs_it():
    """Captured after selections that found all they keep in front 0, a selection holds the launch for the row
    totals, the count stage and the guarded launch for the matrix: a replay on a population with a short front 0
    must build the matrix on the device's own decision (the host plays no part in a replay)."""
    n, m, k = 40000, 8, 5000
    g = torch.Generator("cpu").manual_seed(409)
    wide = torch.rand(n, m, generator=g)
    deep = torch.rand(n, m, generator=g) + (torch.arange(n) % 64)[:, None].float()
    want = {"wide": c_oracle.select(as_np(wide), k), "deep": c_oracle.select(as_np(deep), k)}
    assert int((want["wide"][1] == 0).sum()) >= k > int((want["deep"][1] == 0).sum())
    x = torch.arange(n, dtype=torch.int32, device=DEV)[:, None]
    f_static = wide.to(DEV).clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):  # the word of the launch memory says "twice in a row" from the second call on
            nd_environmental_selection(x, f_static, k)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = nd_environmental_selection(x, f_static, k)
    for name in ("wide", "deep", "deep", "wide", "deep"):
        print("replay:", name, flush=True)
        f_static.copy_((wide if name == "wide" else deep).to(DEV))
        graph.replay()
        torch.cuda.synchronize()
        xs, fs, rs, ds = [t.clone() for t in out]
        nd_environmental_selection(x, wide.to(DEV), k)  # eager work between the replays
        torch.cuda.synchronize()
        order, rank, dist, _ = want[name]
        assert np.array_equal(as_np(xs)[:, 0].astype(np.int64), order), name
        assert np.array_equal(as_np(rs), rank[order]), name
        gd, wd = as_np(ds), dist[order]
        assert np.array_equal(np.isinf(gd), np.isinf(wd)), name
        fin = np.isfinite(wd)
        np.testing.assert_allclose(gd[fin], wd[fin], rtol=1e-4)
    del graph
    runtime.release_workspaces()
