"""The selection path whose kernels never wait for each other (tunable ``peel_stepped``: one launch per front, the last
front ordered by argsort steps and element-wise kernels) against the CPU restatement and the C checker, and the way
into it: a call whose device-side wait ran out is issued once more through it when the status is checked, also while
another kernel keeps the device busy.  The reference's own loop is one short launch per front and always makes
progress (src/evox/operators/selection/non_dominate.py:161-169)."""

import numpy as np
import pytest
import torch

from evox_amd import _lib, runtime, workloads
from evox_amd.operators.selection import (nd_environmental_selection, nd_environmental_selection_two_part, non_dominate_rank,
                                          non_dominate_rank_until)
from oracle import c_oracle
from oracle import eager_restatement as er
from tests.cases import as_np

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda", 0)


@pytest.fixture(autouse=True)
def through_the_pipeline():
    runtime.use_small_population_kernel = False  # (the one-workgroup kernel waits for nobody either; not what is tested here)
    yield
    runtime.use_small_population_kernel = None


def _same_selection(got, want, what):
    assert torch.equal(got[0].cpu(), want[0]), what
    assert np.array_equal(as_np(got[1]), as_np(want[1]), equal_nan=True), what
    assert torch.equal(got[2].cpu(), want[2]), what
    g, w = as_np(got[3]), as_np(want[3])
    fin = np.isfinite(w)
    assert np.array_equal(np.isfinite(g), fin) and np.array_equal(g[~fin], w[~fin], equal_nan=True), what
    np.testing.assert_allclose(g[fin], w[fin], rtol=1e-5, err_msg=str(what))


@pytest.mark.parametrize("n,m,topk,seed", [(700, 3, 350, 1), (3000, 2, 1500, 2), (5000, 5, 100, 3), (9000, 3, 9000, 4),
                                            (2500, 8, 1200, 5), (1500, 1, 700, 6)])
def test_stepped_selection_equals_the_restatement(n, m, topk, seed):
    f, x = workloads.uniform_population(n, m, 6, seed)
    if seed % 2 == 0:  # ties, duplicate rows and a NaN row
        f = (f * 16).round() / 16
        f[7] = float("nan")
    with runtime.options(peel_stepped=1):
        got = nd_environmental_selection(x.to(DEV), f.to(DEV), topk)
        rank = non_dominate_rank(f.to(DEV))
        status = runtime.last_status()
    assert status["error"] == 0
    _same_selection(got, er.environmental_selection(x, f, topk), (n, m, topk))
    assert np.array_equal(as_np(rank), as_np(er.ranks_by_peeling(f)))


def test_stepped_two_part_and_rank_until():
    f, x = workloads.uniform_population(6000, 3, 5, 11)
    with runtime.options(peel_stepped=1):
        got = nd_environmental_selection_two_part(x[:2500].to(DEV), f[:2500].to(DEV), x[2500:].to(DEV), f[2500:].to(DEV), 3000)
        until = non_dominate_rank_until(f.to(DEV), 3001)
    _same_selection(got, er.environmental_selection(x, f, 3000), "two parts")
    full = as_np(er.ranks_by_peeling(f))
    worst = np.sort(full)[3000]
    assert np.array_equal(as_np(until), np.where(full <= worst, full, 2**31 - 1))


def test_stepped_selection_beyond_the_lds_sorters():
    """More than 32 768 rows: the argsort steps of the last front's ordering are the radix sort."""
    f, x = workloads.uniform_population(50000, 3, 2, 12)
    with runtime.options(peel_stepped=1):
        got = nd_environmental_selection(x.to(DEV), f.to(DEV), 20000)
        assert runtime.last_status()["error"] == 0
    order, rank, dist, _ = c_oracle.select(f.numpy(), 20000)
    assert np.array_equal(as_np(got[2]), rank[order])
    assert np.array_equal(as_np(got[0]), x.numpy()[order])


def test_a_wait_that_ran_out_is_issued_again_without_coresidency():
    """A long plain kernel on a second stream holds the device while a selection is issued whose waits give up after
    one poll (forced from the host, so that every kernel exits normally): with the status checked, the call is issued
    again through the stepped path and returns the restatement's result."""
    w = workloads.c2()
    f = w.f.to(DEV)
    x = torch.arange(f.size(0), dtype=torch.float32, device=DEV)[:, None].repeat(1, 4)
    want = er.environmental_selection(x.cpu(), w.f, w.topk)
    sink = torch.zeros(1, dtype=torch.float32, device=DEV)
    side = torch.cuda.Stream(device=DEV)
    checking = runtime.CHECK_STATUS
    runtime.CHECK_STATUS = True
    try:
        with torch.cuda.stream(side):  # about ten milliseconds of vector additions on every compute unit
            _lib.call("evox_hip_calibration_launch", 0, 4096, 20000, sink.data_ptr(), side.cuda_stream)
        with runtime.options(spin_limit=1):
            got = nd_environmental_selection(x, f, w.topk)
            rank = non_dominate_rank(f)
        side.synchronize()
        torch.cuda.synchronize()
    finally:
        runtime.CHECK_STATUS = checking
    _same_selection(got, want, "issued again")
    assert np.array_equal(as_np(rank), as_np(er.ranks_by_peeling(w.f)))
    # without the second issue the same call reports the wait that ran out (or, if every poll succeeded, is right)
    runtime.RETRY_WITHOUT_CORESIDENCY = False
    runtime.CHECK_STATUS = True
    try:
        with runtime.options(spin_limit=1):
            try:
                plain = nd_environmental_selection(x, f, w.topk)
                _same_selection(plain, want, "no wait ran out")
            except _lib.EvoxHipError as e:
                assert e.code == _lib.E_BARRIER_TIMEOUT
    finally:
        runtime.RETRY_WITHOUT_CORESIDENCY = True
        runtime.CHECK_STATUS = checking
