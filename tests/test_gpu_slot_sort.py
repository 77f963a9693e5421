"""The slot sort (rows relabelled by ascending (row key, original index)) against numpy, on the keys that the kernels
themselves report: key distributions with large buckets (one key held by thousands of rows, clusters next to
outliers), non-finite values, signed zeros, sizes around the limits of the one-workgroup-per-sixteen-rows kernel and
of the bucket sort's grid; and the fitness in layouts other than packed rows."""

import numpy as np
import pytest
import torch

from evox_amd import _lib, runtime
from tests.cases import as_np

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda", 0)


def _sorted_arrays(f, n_first=None):
    """Runs stage_prepare (keys, state reset, slot sort) and returns copies of what it leaves."""
    n, m = f.shape
    ws = runtime.workspace(n, m, f.device)
    s = runtime.stream_handle(f.device)
    _lib.call("evox_hip_stage_prepare", f.data_ptr(), n, m, f.stride(0), f.stride(1), ws.data_ptr(), ws.numel(), s)
    torch.cuda.synchronize()
    v = runtime.workspace_views(ws, n, m)
    return {k: as_np(v[k]).copy() for k in ("orig_of_padded", "key_sorted", "kid_sorted", "xs_sorted", "xs", "slot_of")}


def _cases():
    g = torch.Generator("cpu").manual_seed(4242)
    cases = {}
    cases["uniform_20000x3"] = torch.rand(20000, 3, generator=g)
    cases["uniform_4097x2"] = torch.rand(4097, 2, generator=g)
    cases["uniform_32768x3"] = torch.rand(32768, 3, generator=g)
    cases["uniform_32767x5"] = torch.rand(32767, 5, generator=g)
    cases["uniform_9000x16"] = torch.rand(9000, 16, generator=g)
    cases["uniform_5000x33"] = torch.rand(5000, 33, generator=g)
    cases["uniform_65536x2"] = torch.rand(65536, 2, generator=g)
    cases["uniform_50000x3"] = torch.rand(50000, 3, generator=g)
    cases["all_equal_20000x3"] = torch.full((20000, 3), 0.25)
    two = torch.rand(20000, 3, generator=g)
    two[:9000] = 0.5  # one key with 9000 rows among 11000 distinct ones
    cases["one_large_tie_group"] = two[torch.randperm(20000, generator=g)]
    cases["tie_group_in_the_first_rows"] = two.clone()  # whole waves of equal rows, then whole waves of distinct ones
    cases["all_equal_20001x2"] = torch.full((20001, 2), -3.0)  # (the padding behind the last row belongs to half a workgroup)
    ties = torch.randint(0, 3, (30000, 2), generator=g).float()  # five distinct keys
    cases["five_keys_30000x2"] = ties
    cl = torch.rand(25000, 3, generator=g) * 1e-6 + 0.5  # keys within a sliver of the range ...
    cl[0] = 1e30  # ... that one row stretches
    cl[1] = -1e30
    cases["cluster_and_outliers"] = cl
    two_cl = torch.cat([torch.rand(10000, 2, generator=g) * 1e-5, 1e20 + torch.rand(10000, 2, generator=g) * 1e15])
    cases["two_far_clusters"] = two_cl[torch.randperm(20000, generator=g)]
    nonfin = torch.rand(12000, 4, generator=g)
    nonfin[::7, 1] = float("nan")
    nonfin[3::11, 2] = float("inf")
    nonfin[5::13, 0] = float("-inf")
    cases["nan_and_infinities"] = nonfin
    z = torch.zeros(8000, 2)
    z[::2] = -0.0
    cases["signed_zeros"] = z
    simplex = torch.rand(20000, 3, generator=g)  # a converged front of normalised objectives: every row sums to one
    cases["simplex_20000x3"] = simplex / simplex.sum(dim=1, keepdim=True)
    return cases


@pytest.mark.parametrize("name", sorted(_cases()))
def test_slot_sort_orders_by_key_then_index(name):
    f_cpu = _cases()[name]
    f = f_cpu.to(DEV)
    n, m = f.shape
    try:
        got = _sorted_arrays(f)
    finally:
        runtime.release_workspaces()
    # ascending (key, original index); kid = first slot of the key; slot_of = the inverse table
    key = got["key_sorted"][:n].view(np.uint64)
    orig = got["orig_of_padded"][:n].astype(np.int64)
    assert np.array_equal(np.sort(orig), np.arange(n))
    assert np.array_equal(got["slot_of"][orig], np.arange(n))
    assert np.all((key[1:] > key[:-1]) | ((key[1:] == key[:-1]) & (orig[1:] > orig[:-1])))
    first = np.flatnonzero(np.concatenate([[True], key[1:] != key[:-1]]))
    assert np.array_equal(got["kid_sorted"][:n], np.repeat(first, np.diff(np.concatenate([first, [n]]))).astype(np.int32))
    # the keys are the weighted sums of the order-preserving integer images of the values (NaN largest, the zeros equal)
    u = as_np(f_cpu).view(np.uint32).astype(np.uint64)
    image = np.where(u >> 31 == 1, (~u) & 0xFFFFFFFF, u | 0x80000000)
    image = np.where(as_np(f_cpu) == 0, np.uint64(0x80000000), image)
    image = np.where(np.isnan(as_np(f_cpu)), np.uint64(0xFFFFFFFF), image)
    weights = (16 + (np.arange(m) & 7)).astype(np.uint64)  # unequal, so that rows on a plane sum(x) = const keep apart
    assert np.array_equal(key, (image * weights).sum(axis=1)[orig])
    # the fitness by slot (with -0.0 stored as +0.0) and by original index, NaN behind the n-th row
    want_sorted = (as_np(f_cpu)[orig] + np.float32(0.0)).T
    assert np.array_equal(got["xs_sorted"][:, :n].view(np.uint32), want_sorted.view(np.uint32))
    assert np.array_equal(got["xs"][:, :n].view(np.uint32), as_np(f_cpu).T.view(np.uint32))
    assert np.all(np.isnan(got["xs_sorted"][:, n:])) and np.all(got["orig_of_padded"][n:] == -1)


@pytest.mark.parametrize("layout", ["column_major", "row_gaps", "two_parts"])
def test_slot_sort_strides_and_two_parts(layout):
    from evox_amd.operators.selection import nd_environmental_selection, nd_environmental_selection_two_part

    g = torch.Generator("cpu").manual_seed(77)
    base = torch.rand(15000, 4, generator=g).to(DEV)
    x = torch.arange(15000, dtype=torch.int32, device=DEV)[:, None]
    want = nd_environmental_selection(x, base, 7000)
    if layout == "column_major":
        f = base.t().contiguous().t()
        assert f.stride() == (1, 15000)
        got = nd_environmental_selection(x, f, 7000)
    elif layout == "row_gaps":
        wide = torch.zeros(15000, 9, device=DEV)
        wide[:, 1:9:2] = base
        f = wide[:, 1:9:2]
        assert f.stride() == (9, 2)
        got = nd_environmental_selection(x, f, 7000)
    else:
        got = nd_environmental_selection_two_part(x[:6001].clone(), base[:6001].clone(), x[6001:].clone(), base[6001:].clone(), 7000)
    for a, b in zip(got, want):
        assert torch.equal(a, b)
