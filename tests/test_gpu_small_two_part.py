"""A small population given as parents and offspring goes through the one-workgroup kernel, which reads both tensors
where they lie: the results must be those of the selection on the concatenation -- through the same kernel, through
the pipeline, and by the plain-C checker -- whatever the sizes of the parts (a boundary inside a group of 8, 32 or
64 rows), the number of objectives, the width of a row of decision variables, ties, NaN and infinite objectives."""

import numpy as np
import pytest
import torch

from evox_amd import runtime
from evox_amd.operators.selection import nd_environmental_selection, nd_environmental_selection_two_part
from oracle import c_oracle
from tests.cases import as_np

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda", 0)

SHAPES = [  # n_a, n_b, m, row shape of x, dtype of x
    (100, 100, 3, (30,), torch.float32),
    (100, 100, 2, (12,), torch.float32),
    (1, 1, 2, (3,), torch.float32),
    (1, 200, 3, (5,), torch.float64),
    (63, 1, 1, (7,), torch.float32),
    (64, 64, 4, (16,), torch.float32),
    (33, 95, 8, (4, 3), torch.float32),
    (250, 250, 3, (10,), torch.float16),
    (96, 104, 5, (1,), torch.int8),
    (7, 300, 16, (9,), torch.float32),
    (50, 50, 3, (0,), torch.float32),
]


@pytest.mark.parametrize("n_a,n_b,m,row,dtype", SHAPES)
def test_small_two_part_equals_the_selection_on_the_concatenation(n_a, n_b, m, row, dtype):
    n = n_a + n_b
    g = torch.Generator("cpu").manual_seed(1000 * n_a + n_b + m)
    for kind in ("uniform", "ties", "special"):
        f = torch.rand(n, m, generator=g)
        if kind == "ties":
            f = torch.floor(f * 4)
        if kind == "special" and n > 4:
            f[n // 3, 0] = float("nan")
            f[n // 2, m - 1] = float("inf")
            f[n - 1, 0] = float("-inf")
        if dtype.is_floating_point:
            x = torch.rand(n, *row, generator=g).to(dtype)
        else:
            x = torch.randint(-100, 100, (n, *row), generator=g).to(dtype)
        fd, xd = f.to(DEV), x.to(DEV)
        for k in sorted({1, n // 2, n}):
            got = nd_environmental_selection_two_part(xd[:n_a], fd[:n_a], xd[n_a:], fd[n_a:], k)
            if runtime.small_population_kernel_fits(n, m, 1):  # (307 rows of 16 objectives are the pipeline's)
                assert runtime.last_status() == {"error": 0}  # the one-workgroup kernel has no control block
            whole = nd_environmental_selection(xd, fd, k)
            runtime.use_small_population_kernel = False
            try:
                piped = nd_environmental_selection_two_part(xd[:n_a], fd[:n_a], xd[n_a:], fd[n_a:], k)
            finally:
                runtime.use_small_population_kernel = None
            for a, b, c in zip(got, whole, piped):
                assert a.shape == b.shape and a.dtype == b.dtype
                assert torch.equal(torch.nan_to_num(a.double(), nan=-7.0), torch.nan_to_num(b.double(), nan=-7.0)), (kind, k)
                assert torch.equal(torch.nan_to_num(a.double(), nan=-7.0), torch.nan_to_num(c.double(), nan=-7.0)), (kind, k)
            order, rank, dist, _ = c_oracle.select(as_np(f), k)
            assert np.array_equal(as_np(got[2]), rank[order]), (kind, k)
            assert np.array_equal(as_np(got[1]), as_np(f)[order], equal_nan=True), (kind, k)
    runtime.release_workspaces()


def test_small_two_part_takes_other_strides_through_the_general_path():
    g = torch.Generator("cpu").manual_seed(3)
    f = torch.rand(120, 3, generator=g).to(DEV)
    x = torch.rand(120, 6, generator=g).to(DEV)
    fa, fb = f[:60], f[60:].t().contiguous().t()  # same values, other strides
    got = nd_environmental_selection_two_part(x[:60], fa, x[60:], fb, 60)
    want = nd_environmental_selection(x, f, 60)
    for a, b in zip(got, want):
        assert torch.equal(a, b)
