"""Host-side plumbing between torch tensors and the C ABI: workspaces, streams, status."""

import contextlib
import ctypes
import threading
import os
from typing import Dict, Optional, Tuple

import torch

from . import _lib

_workspaces: Dict[Tuple[int, int], torch.Tensor] = {}
_last: Optional[Tuple[torch.Tensor, int]] = None  # (workspace, stream handle) of the latest call

CHECK_STATUS = os.environ.get("EVOX_AMD_CHECK_STATUS", "0") not in ("", "0")

# Populations of at most evox_hip_batched_max_rows(m) rows can run in the one-workgroup-per-population
# kernel, larger ones need the bit-matrix pipeline.  None = choose by size: a lone population is faster in
# the pipeline, which spreads it over the whole device, from a size on that shrinks as the objectives grow
# (measured, one-workgroup kernel against pipeline, in us: 3 objectives 48/75 at 704 rows and 86/81 at 960;
# 5 objectives 60/71 at 704, 94/80 at 960; 8 objectives 65/68 at 256, 85/76 at 384; 16 objectives 67/77 at 128,
# 119/101 at 256); two or three populations up to twice that size, and four or more always, take the
# one-workgroup kernel, which runs them side by side.  True / False force the choice where it is possible
# (tests use that to drive small inputs through both).
use_small_population_kernel = None


def _lone_population_limit(m: int) -> int:
    if m <= 3:
        return 896
    if m <= 5:
        return 768
    if m <= 8:
        return 288
    return 160


_batched_max_rows = {}  # objectives -> rows that the one-workgroup kernel takes (asked of the library once)


def small_population_kernel_fits(n: int, m: int, batch: int) -> bool:
    if use_small_population_kernel is False:
        return False
    if m == 2:
        # (two objectives have a one-workgroup kernel of their own, which takes up to 4096 rows and beats the pipeline
        # at every size; a tunable switches it off, so the library is asked every time)
        most = int(_lib.lib().evox_hip_batched_max_rows(m))
        return 1 <= n <= most and (most > 1024 or use_small_population_kernel is True or batch >= 4
                                   or n <= _lone_population_limit(m) * (1 if batch == 1 else 2))
    most = _batched_max_rows.get(m)
    if most is None:
        most = _batched_max_rows[m] = int(_lib.lib().evox_hip_batched_max_rows(m))
    if not 1 <= n <= most:
        return False
    if use_small_population_kernel is True:
        return True
    if batch >= 4:
        return True
    return n <= _lone_population_limit(m) * (1 if batch == 1 else 2)


def require_gpu_tensor(t: torch.Tensor, what: str) -> None:
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"{what} must be a torch.Tensor")
    if not t.is_cuda:
        raise RuntimeError(
            f"{what} is on {t.device}: evox_amd runs on an AMD GPU only (HIP kernels, no CPU fallback); "
            "move the tensors to the 'cuda' device"
        )


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def stream_handle(device: torch.device) -> int:
    """The hipStream_t of torch's current stream on ``device`` (asked of torch directly where it offers that: the
    Stream object costs 1.5 us more to build)."""
    if _raw_stream is not None and device.index is not None:
        return _raw_stream(device.index)
    return int(torch.cuda.current_stream(device).cuda_stream)


_workspace_need = {}  # (rows, objectives, with the matrix) -> bytes (asked of the library once per shape)


def workspace(n: int, m: int, device: torch.device, with_matrix: bool = True) -> torch.Tensor:
    """A uint8 tensor of at least evox_hip_workspace_bytes(n, m) bytes, cached per (device, stream):
    calls on one stream are ordered, so they can share it.  ``with_matrix=False`` asks only for the
    bytes that the entry points without a dominance matrix need."""
    need = _workspace_need.get((n, m, with_matrix))
    if need is None:
        query = _lib.lib().evox_hip_workspace_bytes if with_matrix else _lib.lib().evox_hip_first_front_workspace_bytes
        need = int(query(n, m))
        if need == 0:
            raise ValueError(f"unsupported population shape n={n}, m={m}")
        if len(_workspace_need) < 4096:
            _workspace_need[(n, m, with_matrix)] = need
    key = (device.index if device.index is not None else torch.cuda.current_device(), stream_handle(device))
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < need:
        _workspaces.pop(key, None)
        ws = None
        ws = torch.empty(need, dtype=torch.uint8, device=device)
        assert ws.data_ptr() % 256 == 0
        _workspaces[key] = ws
    return ws


def sort_workspace(n: int, device: torch.device) -> torch.Tensor:
    """Workspace of the standalone stable argsort; shares the per-(device, stream) buffer of `workspace`
    (every call initialises the parts it uses)."""
    need = int(_lib.lib().evox_hip_argsort_workspace_bytes(n))
    if need == 0:
        raise ValueError(f"unsupported sort length n={n}")
    key = (device.index if device.index is not None else torch.cuda.current_device(), stream_handle(device))
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < need:
        _workspaces.pop(key, None)
        ws = None
        ws = torch.empty(need, dtype=torch.uint8, device=device)
        _workspaces[key] = ws
    return ws


def wide_workspace(n: int, m: int, device: torch.device, copies: int = 1) -> torch.Tensor:
    """Workspace of the entry points for 8-byte fitness (`copies` of it, each rounded up to 256 bytes, for as many
    populations in the same launches); shares the per-(device, stream) buffer of `workspace`."""
    need = int(_lib.lib().evox_hip_wide_workspace_bytes(n, m))
    if need == 0:
        raise ValueError(f"unsupported population shape n={n}, m={m}")
    if copies > 1:
        need = ((need + 255) // 256 * 256) * copies
    key = (device.index if device.index is not None else torch.cuda.current_device(), stream_handle(device))
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < need:
        _workspaces.pop(key, None)
        ws = None
        ws = torch.empty(need, dtype=torch.uint8, device=device)
        _workspaces[key] = ws
    return ws


def sized_workspace(need: int, device: torch.device) -> torch.Tensor:
    """The per-(device, stream) buffer of `workspace`, at least `need` bytes."""
    if need <= 0:
        raise ValueError("unsupported population shape")
    key = (device.index if device.index is not None else torch.cuda.current_device(), stream_handle(device))
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < need:
        _workspaces.pop(key, None)
        ws = None
        ws = torch.empty(need, dtype=torch.uint8, device=device)
        assert ws.data_ptr() % 256 == 0
        _workspaces[key] = ws
    return ws


def many_workspace(batch: int, n: int, m: int, stop_count: int, device: torch.device):
    """Workspace of the entry points that take many populations of one shape: (tensor, populations per launch, bytes
    from one population's copy of the workspace to the next); shares the per-(device, stream) buffer of `workspace`.
    Asked anew at every call: the answer depends on the tunables in use."""
    lib = _lib.lib()
    need = int(lib.evox_hip_many_workspace_bytes(batch, n, m, stop_count))
    per_launch = int(lib.evox_hip_many_populations_per_launch(batch, n, m, stop_count))
    if need == 0 or per_launch < 1:
        raise ValueError(f"unsupported population shape n={n}, m={m}")
    key = (device.index if device.index is not None else torch.cuda.current_device(), stream_handle(device))
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < need:
        _workspaces.pop(key, None)
        ws = None
        ws = torch.empty(need, dtype=torch.uint8, device=device)
        assert ws.data_ptr() % 256 == 0
        _workspaces[key] = ws
    return ws, per_launch, need // per_launch


def release_workspaces() -> None:
    _workspaces.clear()


def note_call(ws: torch.Tensor, stream: int, copies: int = 1, step: int = 0) -> None:
    """copies, step: the call used that many copies of the workspace, `step` bytes apart, each with a control block."""
    global _last
    _last = (ws, stream, copies, step)
    if CHECK_STATUS:
        last_status()


# With status checking on, a ranking or selection whose device-side wait ran out (the persistent kernels need all
# their workgroups resident at once: another kernel may hold the compute units) is issued once more through the
# kernels that never wait for each other (tunable peel_stepped), instead of raising.
RETRY_WITHOUT_CORESIDENCY = True


def checked(issue) -> None:
    """``issue()`` enqueues one library call and notes it (``note_call``)."""
    try:
        issue()
    except _lib.EvoxHipError as e:
        if e.code != _lib.E_BARRIER_TIMEOUT or not RETRY_WITHOUT_CORESIDENCY or current_option("peel_stepped", 0):
            raise
        with options(peel_stepped=1):
            issue()


def note_small_kernel_call() -> None:
    """The one-workgroup-per-population kernel has no control block and no device-side waits."""
    global _last
    _last = None


def last_status() -> dict:
    """Waits for the latest call and returns its control block; raises if the device reported an error.
    Calls served by the small-population kernel have no control block: {"error": 0}."""
    if _last is None:
        return {"error": 0}
    ws, stream, copies, step = _last
    out = (ctypes.c_int32 * 8)()
    for b in reversed(range(copies)):  # (the control block reported is that of the first copy)
        code = _lib.lib().evox_hip_read_status(ws.data_ptr() + b * step, stream, out)
        if code != 0:
            raise _lib.EvoxHipError("evox_hip_read_status", code)
    keys = ("error", "fronts", "worst_rank", "better_rows", "last_front_size", "taken_from_last", "passes")
    return dict(zip(keys, list(out)[:7]))


_process_options: Dict[str, int] = {}  # what set_option has changed (the library holds the values themselves)


def set_option(name: str, value: int) -> None:
    """Changes a process-wide tunable (configuration at start-up; see ``options`` for a scoped change)."""
    _lib.call("evox_hip_set_option", name.encode(), int(value))
    _process_options[name] = int(value)


_options_in_use = threading.local()


def current_option(name: str, default: int) -> int:
    """The value of a tunable as the calls of this thread see it, where this module has set it (else ``default``,
    which must be the library's own default)."""
    stack = getattr(_options_in_use, "stack", None)
    if stack and name in stack[-1][1]:
        return stack[-1][1][name]
    return _process_options.get(name, default)


@contextlib.contextmanager
def options(**tunables):
    """Tunables for the library calls that this thread makes inside the ``with`` block (the process-wide ones,
    with the given changes); other threads and the process-wide values are left alone."""
    lib = _lib.lib()
    handle = lib.evox_hip_options_create()
    if not handle:
        raise MemoryError("evox_hip_options_create")
    stack = getattr(_options_in_use, "stack", None)
    if stack is None:
        stack = _options_in_use.stack = []
    try:
        if stack:  # start from the enclosing block's values, not from the process-wide ones
            for name, value in stack[-1][1].items():
                _lib.call("evox_hip_options_set", handle, name.encode(), int(value))
        merged = dict(stack[-1][1]) if stack else {}
        for name, value in tunables.items():
            _lib.call("evox_hip_options_set", handle, name.encode(), int(value))
            merged[name] = int(value)
        stack.append((handle, merged))
        _lib.call("evox_hip_options_use", handle)
        try:
            yield
        finally:
            stack.pop()
            _lib.call("evox_hip_options_use", stack[-1][0] if stack else None)
    finally:
        lib.evox_hip_options_destroy(handle)


def workspace_views(ws: torch.Tensor, n: int, m: int) -> dict:
    """Typed views of the workspace regions (for tests and tools)."""
    out = (ctypes.c_int64 * 11)()
    _lib.call("evox_hip_workspace_layout", n, m, out)
    dom_off, wstride, nwords, count, rank, dist, perm, fstart, order, ctrl, orig_of = list(out)

    def view(off, count_, dtype):
        size = torch.empty((), dtype=dtype).element_size()
        return ws[off: off + count_ * size].view(dtype)

    sort = (ctypes.c_int64 * 6)()
    _lib.call("evox_hip_slot_sort_layout", n, m, sort)
    npad = sort[4]
    return {
        "key_sorted": view(sort[0], npad, torch.int64),
        "kid_sorted": view(sort[1], npad, torch.int32),
        "xs_sorted": view(sort[2], m * npad, torch.float32).view(m, npad),
        "xs": view(sort[3], m * npad, torch.float32).view(m, npad),
        "slot_of": view(sort[5], n, torch.int32),
        "dom": view(dom_off, n * wstride, torch.int64).view(n, wstride),
        "nwords": nwords,
        "count": view(count, n, torch.int32),
        "rank": view(rank, n, torch.int32),
        "dist": view(dist, n, torch.float32),
        "perm": view(perm, n, torch.int32),
        "fstart": view(fstart, n + 2, torch.int32),
        "order": view(order, n, torch.int32),
        "ctrl": view(ctrl, 16, torch.int32),
        "orig_of": view(orig_of, n, torch.int32),
        "orig_of_padded": view(orig_of, npad, torch.int32),
    }
