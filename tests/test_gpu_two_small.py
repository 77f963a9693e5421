"""Two objectives in the one-workgroup kernel that needs no dominance matrix (``two_small_kernel``: up to 4096 rows,
every front a prefix minimum, every ordering a radix sort in LDS) against the CPU restatement, the C checker and
the matrix kernels.  Reference: src/evox/operators/selection/non_dominate.py:172-254 for M = 2."""

import numpy as np
import pytest
import torch

from evox_amd import _lib, runtime, workloads
from evox_amd.operators.selection import (nd_environmental_selection, nd_environmental_selection_two_part, non_dominate_rank)
from oracle import c_oracle
from oracle import eager_restatement as er
from tests.cases import as_np

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda", 0)


def _same_selection(got, want, what):
    assert torch.equal(got[0].cpu(), want[0]), what
    assert np.array_equal(as_np(got[1]), as_np(want[1]), equal_nan=True), what
    assert torch.equal(got[2].cpu(), want[2]), what
    g, w = as_np(got[3]), as_np(want[3])
    fin = np.isfinite(w)
    assert np.array_equal(np.isfinite(g), fin) and np.array_equal(g[~fin], w[~fin], equal_nan=True), what
    np.testing.assert_allclose(g[fin], w[fin], rtol=1e-5, err_msg=str(what))


def _population(kind, n, seed):
    g = torch.Generator("cpu").manual_seed(seed)
    f = torch.rand(n, 2, generator=g)
    if kind == "grid":  # ties in both objectives, many duplicate rows
        f = (f * 9).floor() / 9
    elif kind == "line":  # one front: f2 = 1 - f1
        f[:, 1] = 1.0 - f[:, 0]
    elif kind == "chain":  # every row its own front
        f[:, 0] = torch.arange(n).float()
        f[:, 1] = torch.arange(n).float()
        f = f[torch.randperm(n, generator=g)]
    elif kind == "layers":  # about twenty fronts of equal size, as C2
        layer = torch.randint(0, 20, (n,), generator=g).float()
        a = torch.rand(n, generator=g)
        f = torch.stack([a + layer, (1.0 - a) + layer], dim=1)
    elif kind == "special":  # NaN rows, infinities, signed zeros, copies of all of them
        f = (f * 5).floor() / 5
        for i, (a, b) in enumerate([(float("nan"), 0.5), (0.5, float("nan")), (float("nan"), float("nan")), (float("inf"), 0.1),
                                    (0.1, float("inf")), (-float("inf"), 0.9), (0.0, -0.0), (-0.0, 0.0), (float("inf"), float("inf"))]):
            for rep in range(2):
                if 3 * i + rep < n:
                    f[(7 * i + 11 * rep) % n] = torch.tensor([a, b])
    elif kind == "equal":  # every row the same
        f[:] = 0.25
    x = torch.arange(n, dtype=torch.float32)[:, None].repeat(1, 3)
    return f, x


CASES = [("uniform", 1), ("uniform", 2), ("uniform", 63), ("uniform", 64), ("uniform", 65), ("uniform", 1000), ("uniform", 2000),
         ("uniform", 4096), ("grid", 300), ("grid", 2500), ("grid", 4096), ("line", 700), ("line", 1025), ("line", 3000), ("line", 4096),
         ("chain", 200), ("chain", 1500), ("layers", 2000), ("layers", 4095), ("special", 40), ("special", 1300), ("special", 4096),
         ("equal", 5), ("equal", 1100), ("equal", 4096)]


@pytest.mark.parametrize("kind,n", CASES, ids=[f"{k}-{n}" for k, n in CASES])
def test_against_the_restatement(kind, n):
    f, x = _population(kind, n, 1000 + n)
    fd, xd = f.to(DEV), x.to(DEV)
    assert runtime.small_population_kernel_fits(n, 2, 1)
    want_rank = er.ranks_by_peeling(f)
    assert np.array_equal(as_np(non_dominate_rank(fd)), as_np(want_rank)), "all ranks"
    for topk in sorted({1, max(1, n // 3), max(1, n // 2), n}):
        _same_selection(nd_environmental_selection(xd, fd, topk), er.environmental_selection(x, f, topk), (kind, n, topk))


def test_c2_goldens_and_the_matrix_kernels():
    w = workloads.c2()
    f, x = w.f, (w.x if w.x is not None else w.f)
    got = nd_environmental_selection(x.to(DEV), f.to(DEV), w.topk)
    _same_selection(got, er.environmental_selection(x, f, w.topk), "C2")
    with runtime.options(two_small_min_rows=0):
        assert not runtime.small_population_kernel_fits(2000, 2, 1) or runtime.use_small_population_kernel is True
        other = nd_environmental_selection(x.to(DEV), f.to(DEV), w.topk)
    for a, b in zip(got, other):
        assert np.array_equal(as_np(a), as_np(b), equal_nan=True)
    order, rank, _dist, _fronts = c_oracle.select(f, w.topk)
    assert np.array_equal(as_np(got[2]), as_np(rank)[as_np(order)[:w.topk]])


def test_batches_two_parts_and_strides():
    g = torch.Generator("cpu").manual_seed(5)
    f = torch.rand(9, 1800, 2, generator=g)
    f[3] = (f[3] * 7).floor() / 7
    f[5, :, 1] = 1.0 - f[5, :, 0]
    x = torch.rand(9, 1800, 6, generator=g)
    fd, xd = f.to(DEV), x.to(DEV)
    got = nd_environmental_selection(xd, fd, 900)
    ranks = non_dominate_rank(fd)
    for b in range(9):
        _same_selection([t[b] for t in got], er.environmental_selection(x[b], f[b], 900), b)
        assert np.array_equal(as_np(ranks[b]), as_np(er.ranks_by_peeling(f[b]))), b
    # populations along another dimension, fitness as a strided view, float64 decision vectors
    mapped = torch.vmap(lambda a, c: nd_environmental_selection(a, c, 900), in_dims=(1, 1))(xd.permute(1, 0, 2).contiguous().double(),
                                                                                            fd.permute(1, 0, 2).contiguous())
    assert torch.equal(mapped[0], got[0].double()) and torch.equal(mapped[2], got[2])
    wide = torch.rand(2500, 5, generator=g).to(DEV)
    view = wide[:, 1:4:2]  # columns 1 and 3
    _same_selection(nd_environmental_selection(torch.empty(2500, 0, device=DEV), view, 1200),
                    er.environmental_selection(torch.empty(2500, 0), view.cpu(), 1200), "strided")
    # parents and offspring in two tensors (1500 + 1500 rows: beyond the matrix kernel's 1024)
    fa, fb = torch.rand(1500, 2, generator=g), torch.rand(1500, 2, generator=g)
    xa, xb = torch.rand(1500, 4, generator=g), torch.rand(1500, 4, generator=g)
    two = nd_environmental_selection_two_part(xa.to(DEV), fa.to(DEV), xb.to(DEV), fb.to(DEV), 1500)
    _same_selection(two, er.environmental_selection(torch.cat([xa, xb]), torch.cat([fa, fb]), 1500), "two parts")


def test_limits_and_the_switch():
    lib = _lib.lib()
    assert int(lib.evox_hip_batched_max_rows(2)) == 4096 and int(lib.evox_hip_batched_max_rows(3)) == 1024
    with runtime.options(two_small_min_rows=0):
        assert int(lib.evox_hip_batched_max_rows(2)) == 1024
    f = torch.rand(4097, 2).to(DEV)
    assert not runtime.small_population_kernel_fits(4097, 2, 1)
    assert np.array_equal(as_np(non_dominate_rank(f)), as_np(er.ranks_by_peeling(f.cpu())))
