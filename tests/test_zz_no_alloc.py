"""The selection entry point that allocates nothing (its scratch memory is part of the library's device image)
against the entry point that takes a caller's workspace: same results, on two calls in a row, the second on a
smaller population, so that whatever the first call left in the shared buffer is seen not to matter."""

import numpy as np
import pytest
import torch

from evox_amd import _lib, runtime, workloads

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda", 0)


def _select(entry, f, x, topk, workspace):
    n, m = f.shape
    out_x = torch.empty(topk, x.size(1), dtype=x.dtype, device=DEV)
    out_f = torch.empty(topk, m, dtype=torch.float32, device=DEV)
    out_rank = torch.empty(topk, dtype=torch.int32, device=DEV)
    out_dist = torch.empty(topk, dtype=torch.float32, device=DEV)
    out_order = torch.empty(topk, dtype=torch.int32, device=DEV)
    s = runtime.stream_handle(DEV)
    head = (x.data_ptr(), x.size(1) * x.element_size(), x.stride(0) * x.element_size(), f.data_ptr(), n, m, f.stride(0),
            f.stride(1), topk, out_x.data_ptr(), out_f.data_ptr(), out_rank.data_ptr(), out_dist.data_ptr(),
            out_order.data_ptr())
    if workspace:
        ws = runtime.workspace(n, m, DEV)
        _lib.call(entry, *head, ws.data_ptr(), ws.numel(), s)
    else:
        _lib.call(entry, *head, s)
    torch.cuda.synchronize()
    return [t.cpu().numpy() for t in (out_x, out_f, out_rank, out_dist, out_order)]


def test_static_selection_equals_workspace_selection_on_two_calls_in_a_row():
    # the first population takes the bit-matrix pipeline with a last front ordered by the radix sort's buffers in
    # reach (n > 8192), the second is smaller: it finds the buffer as the first call left it
    for n, m, d, topk, seed in ((9000, 3, 24, 4500, 11), (1500, 2, 7, 700, 12)):
        print("static selection", n, m, d, topk, seed, flush=True)
        f, x = workloads.uniform_population(n, m, d, seed)
        f, x = f.to(DEV), x.to(DEV)
        want = _select("evox_hip_nd_environmental_selection", f, x, topk, workspace=True)
        got = _select("evox_hip_nd_environmental_selection_static", f, x, topk, workspace=False)
        for name, a, b in zip(("x", "f", "rank", "dist", "order"), got, want):
            # same kernels on the same input: the bytes agree, crowding distances (with their infinities) included
            assert np.array_equal(a.view(np.uint8), b.view(np.uint8)), (n, name)
        assert (np.diff(got[2]) >= 0).all() and len(set(got[4].tolist())) == topk


def test_static_selection_equals_the_reference_written_golden_of_c2():
    from oracle import eager_restatement as er

    w = workloads.c2()
    x = torch.arange(w.f.size(0), dtype=torch.float32)[:, None].repeat(1, 4)
    got = _select("evox_hip_nd_environmental_selection_static", w.f.to(DEV), x.to(DEV), w.topk, workspace=False)
    want = er.environmental_selection(x, w.f, w.topk)  # (pinned by the golden vectors of this workload on the CPU side)
    assert np.array_equal(got[0], want[0].numpy()) and np.array_equal(got[1], want[1].numpy())
    assert np.array_equal(got[2], want[2].numpy())
    fin = np.isfinite(want[3].numpy())
    assert np.array_equal(np.isfinite(got[3]), fin)
    np.testing.assert_allclose(got[3][fin], want[3].numpy()[fin], rtol=1e-5)


def test_static_selection_takes_no_device_memory_and_reports_its_status():
    import ctypes

    f, x = workloads.uniform_population(3000, 3, 8, 13)
    f, x = f.to(DEV), x.to(DEV)
    _select("evox_hip_nd_environmental_selection_static", f, x, 1500, workspace=False)  # (first call on the device done)
    outs = [torch.empty(1500 * 8, dtype=torch.float32, device=DEV) for _ in range(4)]
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info(DEV)[0]
    s = runtime.stream_handle(DEV)

    def call():
        _lib.call("evox_hip_nd_environmental_selection_static", x.data_ptr(), 32, 32, f.data_ptr(), 3000, 3, 3, 1, 1500,
                  outs[0].data_ptr(), outs[1].data_ptr(), outs[2].data_ptr(), outs[3].data_ptr(), None, s)

    call()
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info(DEV)[0] == free_before  # nothing allocated, nothing freed
    status = (ctypes.c_int32 * 8)()
    assert _lib.lib().evox_hip_read_status(None, s, status) == 0 and status[0] == 0 and status[4] >= 1
    # a device-side wait that runs out (forced from the host with a limit of one poll; every kernel still ends) is
    # reported there, and the outputs hold no partial result
    with runtime.options(spin_limit=1):
        call()
    code = _lib.lib().evox_hip_read_status(None, s, status)
    if code != 0:
        assert code == _lib.E_BARRIER_TIMEOUT and status[0] == _lib.E_BARRIER_TIMEOUT
        assert (outs[2][:1500].view(torch.int32) == -1).all() and torch.isnan(outs[3][:1500]).all()
    call()
    assert _lib.lib().evox_hip_read_status(None, s, status) == 0 and status[0] == 0


def test_static_selection_refuses_what_its_buffer_cannot_hold():
    n, m = 20000, 3
    assert int(_lib.lib().evox_hip_workspace_bytes(n, m)) > 32 * 2**20
    f = torch.rand(n, m, device=DEV)
    out = torch.empty(4 * n, dtype=torch.float32, device=DEV)
    with pytest.raises(_lib.EvoxHipError) as err:
        _lib.call("evox_hip_nd_environmental_selection_static", None, 0, 0, f.data_ptr(), n, m, m, 1, 100, None,
                  out.data_ptr(), out.data_ptr(), out.data_ptr(), None, runtime.stream_handle(DEV))
    assert err.value.code == _lib.E_STATIC_LIMIT
