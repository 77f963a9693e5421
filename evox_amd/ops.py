"""torch.library custom operators backed by the HIP kernels.

The reference wraps its peeling loop in a custom operator with a fake (shape-only) implementation
and vmap rules for two nesting levels (src/evox/utils/op_register.py:54-132, used at
src/evox/operators/selection/non_dominate.py:151-169).  The operators here follow the same pattern
in a namespace of their own (``evox_amd::``): each has a fake implementation so that it traces
under ``torch.compile(fullgraph=True)``, and a vmap rule that moves the mapped dimension to the
front; the operators themselves accept any number of leading batch dimensions, so nested vmaps
need no extra registrations.
"""

import ctypes
from typing import List, Optional, Tuple

import torch

from torch.utils._python_dispatch import _get_current_dispatch_mode

from . import _lib, runtime


def _batched_first(info, dims, tensors):
    """The tensors of a vmap rule with the mapped dimension in front; those that are not mapped are expanded."""
    out = []
    for t, d in zip(tensors, dims):
        if t is None:
            out.append(None)
        elif d is None:
            out.append(t.unsqueeze(0).expand(info.batch_size, *t.shape))
        else:
            out.append(t.movedim(d, 0))
    return out


def _as_f32(t: torch.Tensor, what: str) -> torch.Tensor:
    if t.dtype == torch.float32:
        return t
    if t.dtype in (torch.float16, torch.bfloat16):
        return t.float()  # exact and order preserving
    raise TypeError(f"{what} must be float32 (float16 / bfloat16 are widened exactly); got {t.dtype}")


def _order_preserving_f32(t: torch.Tensor, what: str) -> torch.Tensor:
    """A float32 tensor with the same `<=` / `<` relations inside every objective (column) as ``t``.

    Dominance only looks at the order of the values within one objective, so fitness of a dtype that
    the kernels do not read (float64, integers) is replaced, objective by objective, by the dense rank
    of each value among the values of that objective (a sort on the device: equal values get equal
    ranks, -0.0 and 0.0 tie, NaN stays NaN).  Dense ranks below 2**24 are exact in float32.
    Used for ranking only: crowding distances depend on the values themselves.
    """
    if t.dtype in (torch.float32, torch.float16, torch.bfloat16):
        return _as_f32(t, what)
    if t.is_complex() or t.dtype == torch.bool:
        raise TypeError(f"{what} must be a real numeric tensor; got {t.dtype}")
    if t.shape[-2] >= 2**24:
        raise ValueError(f"{what} of dtype {t.dtype} is limited to 2**24 rows per population")
    # one sort per objective column, all columns and populations in the same calls: in sorted order a value opens
    # a new rank when it differs from the value before it (-0.0 == 0.0; NaN, sorted last, is put back below)
    # (every objective as a contiguous row: torch's scan along any other dimension takes milliseconds for 20 000 rows)
    flat = t.reshape(-1, t.shape[-2], t.shape[-1]).transpose(1, 2).contiguous()
    values, index = torch.sort(flat, dim=2)
    if flat.dtype in (torch.float64, torch.int64) and flat.is_cuda:
        # the rest in one kernel: a value opens a new rank when it differs from the one before it, the ranks go back to
        # the rows that the values came from
        dense = torch.empty(flat.size(0), flat.size(2), flat.size(1), dtype=torch.float32, device=t.device)
        with torch.cuda.device(t.device):
            _lib.call("evox_hip_dense_rank_rows", values.data_ptr(), 0 if flat.dtype == torch.float64 else 1, index.data_ptr(),
                      flat.size(0), flat.size(2), flat.size(1), dense.data_ptr(), runtime.stream_handle(t.device))
        return dense.reshape(t.shape)
    opens = torch.zeros(flat.shape, dtype=torch.int32, device=t.device)
    opens[:, :, 1:] = values[:, :, 1:] != values[:, :, :-1]
    dense = torch.empty(flat.shape, dtype=torch.float32, device=t.device)
    dense.scatter_(2, index, opens.cumsum(dim=2, dtype=torch.int32).to(torch.float32))
    if flat.is_floating_point():
        dense = torch.where(torch.isnan(flat), torch.full_like(dense, float("nan")), dense)
    return dense.transpose(1, 2).reshape(t.shape)


def _passes(batch: int, per_launch: int):
    """(first population, populations) of the library calls that rank or select `batch` populations: one call for all
    of them -- the library then runs its launches for `per_launch` populations at a time -- unless the status of every
    call is checked, which looks at the control blocks of one pass."""
    if not runtime.CHECK_STATUS or per_launch >= batch:
        return [(0, batch)]
    return [(b0, min(per_launch, batch - b0)) for b0 in range(0, batch, per_launch)]


def _rank_many(flat_f: torch.Tensor, flat_out: torch.Tensor, count: int) -> None:
    """Ranks of (B, N, M) float32 fitness as far as the front that holds the count-th row, into (B, N) int32."""
    batch, n, m = flat_f.shape
    if batch == 1:
        ws = runtime.workspace(n, m, flat_f.device)
        stream = runtime.stream_handle(flat_f.device)

        def issue_one():
            _lib.call("evox_hip_non_dominate_rank_until", flat_f.data_ptr(), n, m, flat_f.stride(1), flat_f.stride(2), count,
                      flat_out.data_ptr(), ws.data_ptr(), ws.numel(), stream)
            runtime.note_call(ws, stream)

        runtime.checked(issue_one)
        return
    stream = runtime.stream_handle(flat_f.device)

    def issue():
        ws, per_launch, step = runtime.many_workspace(batch, n, m, count, flat_f.device)
        for b0, nb in _passes(batch, per_launch):
            _lib.call("evox_hip_many_non_dominate_rank_until", flat_f[b0].data_ptr(), nb, n, m, flat_f.stride(0), flat_f.stride(1),
                      flat_f.stride(2), count, flat_out[b0].data_ptr(), ws.data_ptr(), ws.numel(), stream)
            runtime.note_call(ws, stream, min(per_launch, nb), step)

    runtime.checked(issue)


@torch.library.custom_op("evox_amd::nd_rank", mutates_args=())
def nd_rank(f: torch.Tensor) -> torch.Tensor:
    """(..., N, M) fitness -> (..., N) int32 non-domination rank."""
    runtime.require_gpu_tensor(f, "fitness")
    if f.dim() < 2:
        raise ValueError("fitness must have shape (..., N, M)")
    f32 = _order_preserving_f32(f, "fitness") if f.shape[-2] > 0 and f.shape[-1] > 0 else f.float()
    n, m = f32.shape[-2:]
    out = torch.empty(f32.shape[:-1], dtype=torch.int32, device=f.device)
    if n == 0 or out.numel() == 0:
        return out
    if m == 0:
        return out.zero_()
    with torch.cuda.device(f.device):
        flat_f = f32.reshape(-1, n, m)
        flat_out = out.view(-1, n)
        if runtime.small_population_kernel_fits(n, m, flat_f.size(0)):
            _lib.call("evox_hip_batched_non_dominate_rank", flat_f.data_ptr(), flat_f.size(0), n, m, flat_f.stride(0),
                      flat_f.stride(1), flat_f.stride(2), flat_out.data_ptr(), runtime.stream_handle(f.device))
            runtime.note_small_kernel_call()
        else:
            _rank_many(flat_f, flat_out, n)
    return out


@nd_rank.register_fake
def _(f):
    return f.new_empty(f.shape[:-1], dtype=torch.int32)


def _nd_rank_vmap(info, in_dims, f):
    return nd_rank(f.movedim(in_dims[0], 0)), 0


torch.library.register_vmap(nd_rank, _nd_rank_vmap)


RANK_UNSET = 0x7FFFFFFF
def _argsort_waits(n: int) -> bool:
    """Whether a one-dimensional argsort step of n positions goes through the radix kernel, whose workgroups wait for
    each other and report a wait that ran out in a control block: sorts of more than 32 768 positions, and with the
    tunable ``mid_argsort`` switched off those of more than 8192."""
    return n > (32768 if runtime.current_option("mid_argsort", 1) else 8192)


_ROWS_ARGSORT_MAX = 16384  # longest sort of a batch that runs inside one workgroup


@torch.library.custom_op("evox_amd::nd_rank_until", mutates_args=())
def nd_rank_until(f: torch.Tensor, count: int) -> torch.Tensor:
    """(..., N, M) fitness -> (..., N) int32 rank, peeled only as far as the front that holds the
    count-th best row; rows of later fronts get RANK_UNSET."""
    runtime.require_gpu_tensor(f, "fitness")
    if f.dim() < 2:
        raise ValueError("fitness must have shape (..., N, M)")
    n, m = f.shape[-2:]
    if count > n:
        raise RuntimeError(f"selected index k out of range: count={count} exceeds the population size {n}")
    if count < 1:
        raise IndexError(f"count must be at least 1; got {count}")
    if m == 0:
        raise ValueError("fitness must have at least one objective")
    f32 = _order_preserving_f32(f, "fitness")
    out = torch.empty(f32.shape[:-1], dtype=torch.int32, device=f.device)
    if out.numel() == 0:
        return out
    with torch.cuda.device(f.device):
        _rank_many(f32.reshape(-1, n, m), out.view(-1, n), count)
    return out


@nd_rank_until.register_fake
def _(f, count):
    return f.new_empty(f.shape[:-1], dtype=torch.int32)


def _nd_rank_until_vmap(info, in_dims, f, count):
    return nd_rank_until(f.movedim(in_dims[0], 0), count), 0


torch.library.register_vmap(nd_rank_until, _nd_rank_until_vmap)


@torch.library.custom_op("evox_amd::nd_first_front", mutates_args=())
def nd_first_front(f: torch.Tensor) -> torch.Tensor:
    """(..., N, M) fitness -> (..., N) bool, True for the rows that no row dominates (rank 0)."""
    runtime.require_gpu_tensor(f, "fitness")
    if f.dim() < 2:
        raise ValueError("fitness must have shape (..., N, M)")
    f32 = _order_preserving_f32(f, "fitness") if f.shape[-2] > 0 and f.shape[-1] > 0 else f.float()
    n, m = f32.shape[-2:]
    out = torch.empty(f32.shape[:-1], dtype=torch.bool, device=f.device)
    if n == 0 or out.numel() == 0:
        return out
    if m == 0:
        return out.fill_(True)
    with torch.cuda.device(f.device):
        flat_f = f32.reshape(-1, n, m)
        flat_out = out.view(-1, n)
        stream = runtime.stream_handle(f.device)
        if flat_f.size(0) == 1:
            ws = runtime.workspace(n, m, f.device, with_matrix=False)
            _lib.call("evox_hip_first_front_mask", flat_f.data_ptr(), n, m, flat_f.stride(1), flat_f.stride(2), flat_out.data_ptr(),
                      ws.data_ptr(), ws.numel(), stream)
        else:
            ws = runtime.sized_workspace(int(_lib.lib().evox_hip_many_first_front_workspace_bytes(flat_f.size(0), n, m)), f.device)
            _lib.call("evox_hip_many_first_front_mask", flat_f.data_ptr(), flat_f.size(0), n, m, flat_f.stride(0), flat_f.stride(1),
                      flat_f.stride(2), flat_out.data_ptr(), ws.data_ptr(), ws.numel(), stream)
        runtime.note_call(ws, stream)
    return out


@nd_first_front.register_fake
def _(f):
    return f.new_empty(f.shape[:-1], dtype=torch.bool)


def _nd_first_front_vmap(info, in_dims, f):
    return nd_first_front(f.movedim(in_dims[0], 0)), 0


torch.library.register_vmap(nd_first_front, _nd_first_front_vmap)


@torch.library.custom_op("evox_amd::crowding", mutates_args=())
def crowding(costs: torch.Tensor, mask: Optional[torch.Tensor]) -> torch.Tensor:
    """(..., N, M) costs, optional (..., N) bool mask -> (..., N) float32 crowding distance."""
    runtime.require_gpu_tensor(costs, "costs")
    if costs.dim() < 2:
        raise ValueError("costs must have shape (..., N, M)")
    c32 = _as_f32(costs, "costs")
    n, m = c32.shape[-2:]
    out = torch.empty(c32.shape[:-1], dtype=torch.float32, device=costs.device)
    if mask is not None:
        runtime.require_gpu_tensor(mask, "mask")
        if mask.dtype != torch.bool:
            raise TypeError(f"mask must be a bool tensor; got {mask.dtype}")
        if mask.shape != out.shape:
            raise ValueError(f"mask shape {tuple(mask.shape)} does not match costs {tuple(costs.shape)}")
    if n == 0 or out.numel() == 0:
        return out
    if m == 0:
        raise ValueError("costs must have at least one objective")
    with torch.cuda.device(costs.device):
        flat_c = c32.reshape(-1, n, m)
        flat_out = out.view(-1, n)
        flat_mask = None if mask is None else mask.reshape(-1, n)
        stream = runtime.stream_handle(costs.device)
        if flat_c.size(0) == 1:
            ws = runtime.workspace(n, m, costs.device)
            _lib.call("evox_hip_crowding_distance", flat_c.data_ptr(), n, m, flat_c.stride(1), flat_c.stride(2),
                      None if flat_mask is None else flat_mask.data_ptr(), 0 if flat_mask is None else flat_mask.stride(1),
                      flat_out.data_ptr(), ws.data_ptr(), ws.numel(), stream)
        else:
            ws = runtime.sized_workspace(int(_lib.lib().evox_hip_many_crowding_workspace_bytes(flat_c.size(0), n, m)), costs.device)
            _lib.call("evox_hip_many_crowding_distance", flat_c.data_ptr(), flat_c.size(0), n, m, flat_c.stride(0), flat_c.stride(1),
                      flat_c.stride(2), None if flat_mask is None else flat_mask.data_ptr(),
                      0 if flat_mask is None else flat_mask.stride(0), 0 if flat_mask is None else flat_mask.stride(1),
                      flat_out.data_ptr(), ws.data_ptr(), ws.numel(), stream)
        runtime.note_call(ws, stream)
    return out


@crowding.register_fake
def _(costs, mask):
    return costs.new_empty(costs.shape[:-1], dtype=torch.float32)


def _crowding_vmap(info, in_dims, costs, mask):
    cd, md = in_dims
    costs = costs.movedim(cd, 0) if cd is not None else costs.unsqueeze(0).expand(info.batch_size, *costs.shape)
    if mask is not None:
        mask = mask.movedim(md, 0) if md is not None else mask.unsqueeze(0).expand(info.batch_size, *mask.shape)
    return crowding(costs, mask), 0


torch.library.register_vmap(crowding, _crowding_vmap)


def _wide_costs(t: torch.Tensor, what: str):
    """Costs of a dtype that the float32 kernels do not read, as the 8-byte elements that the wide kernels read:
    (tensor, kind of the C ABI, dtype of the distances)."""
    if t.dtype == torch.float64:
        return t, 0, torch.float64
    if t.is_floating_point() or t.is_complex() or t.dtype == torch.bool:
        raise TypeError(f"{what} must be float64 or an integer tensor here; got {t.dtype}")
    out_dtype = torch.get_default_dtype()  # integer differences are divided in the default float dtype
    if out_dtype not in (torch.float32, torch.float64):
        raise TypeError(f"integer {what} needs a default float dtype of float32 or float64; got {out_dtype}")
    return t.to(torch.int64), 1, out_dtype


@torch.library.custom_op("evox_amd::crowding_wide", mutates_args=())
def crowding_wide(costs: torch.Tensor, mask: Optional[torch.Tensor]) -> torch.Tensor:
    """(..., N, M) float64 or integer costs, optional (..., N) bool mask -> (..., N) crowding distance: float64 for
    float64 costs, torch's default float dtype for integer costs."""
    runtime.require_gpu_tensor(costs, "costs")
    if costs.dim() < 2:
        raise ValueError("costs must have shape (..., N, M)")
    wide, kind, out_dtype = _wide_costs(costs, "costs")
    n, m = wide.shape[-2:]
    out = torch.empty(wide.shape[:-1], dtype=out_dtype, device=costs.device)
    if mask is not None:
        runtime.require_gpu_tensor(mask, "mask")
        if mask.dtype != torch.bool:
            raise TypeError(f"mask must be a bool tensor; got {mask.dtype}")
        if mask.shape != out.shape:
            raise ValueError(f"mask shape {tuple(mask.shape)} does not match costs {tuple(costs.shape)}")
    if n == 0 or out.numel() == 0:
        return out
    if m == 0:
        raise ValueError("costs must have at least one objective")
    with torch.cuda.device(costs.device):
        flat_c = wide.reshape(-1, n, m)
        flat_out = out.view(-1, n)
        flat_mask = None if mask is None else mask.reshape(-1, n)
        stream = runtime.stream_handle(costs.device)
        ws = runtime.wide_workspace(n, m, costs.device)
        for b in range(flat_c.size(0)):
            c = flat_c[b]
            mk = None if flat_mask is None else flat_mask[b]
            _lib.call("evox_hip_crowding_distance_wide", c.data_ptr(), kind, n, m, c.stride(0), c.stride(1),
                      None if mk is None else mk.data_ptr(), 0 if mk is None else mk.stride(0), flat_out[b].data_ptr(),
                      0 if out_dtype == torch.float64 else 1, ws.data_ptr(), ws.numel(), stream)
        runtime.note_small_kernel_call()
    return out


@crowding_wide.register_fake
def _(costs, mask):
    return costs.new_empty(costs.shape[:-1], dtype=torch.float64 if costs.dtype == torch.float64 else torch.get_default_dtype())


def _crowding_wide_vmap(info, in_dims, costs, mask):
    costs, mask = _batched_first(info, in_dims, (costs, mask))
    return crowding_wide(costs, mask), 0


torch.library.register_vmap(crowding_wide, _crowding_wide_vmap)


@torch.library.custom_op("evox_amd::nd_select_wide", mutates_args=())
def nd_select_wide(x: torch.Tensor, f: torch.Tensor, topk: int) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """nd_select for float64 or integer fitness: x (..., N, *D), f (..., N, M), topk -> (x, f, rank, crowding distance)
    of the topk survivors, the distance in float64 for float64 fitness and in the default float dtype for integers."""
    runtime.require_gpu_tensor(f, "fitness")
    runtime.require_gpu_tensor(x, "decision vectors")
    if f.dim() < 2:
        raise ValueError("fitness must have shape (..., N, M)")
    bd = f.dim() - 2
    n, m = f.shape[-2:]
    if x.dim() < bd + 1 or x.shape[: bd + 1] != f.shape[: bd + 1]:
        raise ValueError(f"decision vectors {tuple(x.shape)} and fitness {tuple(f.shape)} disagree on the leading dimensions")
    if x.device != f.device:
        raise RuntimeError("decision vectors and fitness are on different devices")
    if topk > n:
        raise RuntimeError(f"selected index k out of range: topk={topk} exceeds the population size {n}")
    if topk < 1:
        raise IndexError(f"topk must be at least 1; got {topk}")
    if m == 0:
        raise ValueError("fitness must have at least one objective")
    wide, kind, out_dtype = _wide_costs(f, "fitness")
    batch = f.shape[:bd]
    out_x = torch.empty(*batch, topk, *x.shape[bd + 1:], dtype=x.dtype, device=x.device)
    out_f = torch.empty(*batch, topk, m, dtype=f.dtype, device=f.device)
    out_rank = torch.empty(*batch, topk, dtype=torch.int32, device=f.device)
    out_dist = torch.empty(*batch, topk, dtype=out_dtype, device=f.device)
    if out_rank.numel() == 0:
        return out_x, out_f, out_rank, out_dist
    # the ranks, as far as the front that holds the topk-th row, from the ranking kernels on a float32 image of the
    # fitness that keeps every comparison (the rows behind that front are marked unset)
    rank = nd_rank_until(f, topk)
    with torch.cuda.device(f.device):
        flat_w = wide.reshape(-1, n, m)
        flat_f = f.reshape(-1, n, m).contiguous()
        flat_x = x.reshape(flat_w.size(0), n, -1).contiguous()
        flat_rank = rank.reshape(-1, n)
        row_bytes = flat_x.size(-1) * flat_x.element_size()
        f_row_bytes = m * flat_f.element_size()
        has_x = row_bytes > 0
        fo_x = out_x.view(flat_w.size(0), topk, -1)
        fo_f, fo_r, fo_d = out_f.view(-1, topk, m), out_rank.view(-1, topk), out_dist.view(-1, topk)
        stream = runtime.stream_handle(f.device)
        count = flat_w.size(0)
        if count == 1:
            ws = runtime.wide_workspace(n, m, f.device)
            wb = flat_w[0]
            _lib.call("evox_hip_nd_environmental_selection_wide", flat_x.data_ptr() if has_x else None, row_bytes, row_bytes,
                      flat_f.data_ptr(), f_row_bytes, f_row_bytes, wb.data_ptr(), kind, n, m, wb.stride(0), wb.stride(1),
                      flat_rank.data_ptr(), topk, fo_x.data_ptr() if has_x else None, fo_f.data_ptr(), fo_r.data_ptr(),
                      fo_d.data_ptr(), 0 if out_dtype == torch.float64 else 1, ws.data_ptr(), ws.numel(), stream)
        else:
            # all populations in the same launches where the library can (it takes them one after the other otherwise);
            # at most 1 GiB of workspace copies at a time
            one = (int(_lib.lib().evox_hip_wide_workspace_bytes(n, m)) + 255) // 256 * 256
            per_call = max(1, min(count, (1 << 30) // max(one, 1)))
            flat_rank = flat_rank.contiguous()
            for b0 in range(0, count, per_call):
                nb = min(per_call, count - b0)
                ws = runtime.wide_workspace(n, m, f.device, nb)
                wb = flat_w[b0:b0 + nb]
                _lib.call("evox_hip_many_nd_environmental_selection_wide", flat_x[b0].data_ptr() if has_x else None, row_bytes, row_bytes,
                          n * row_bytes, flat_f[b0].data_ptr(), f_row_bytes, f_row_bytes, n * f_row_bytes, wb.data_ptr(), kind, nb, n, m,
                          wb.stride(0), wb.stride(1), wb.stride(2), flat_rank[b0].data_ptr(), topk,
                          fo_x[b0].data_ptr() if has_x else None, fo_f[b0].data_ptr(), fo_r[b0].data_ptr(), fo_d[b0].data_ptr(),
                          0 if out_dtype == torch.float64 else 1, ws.data_ptr(), ws.numel(), stream)
        runtime.note_small_kernel_call()
    return out_x, out_f, out_rank, out_dist


@nd_select_wide.register_fake
def _(x, f, topk):
    bd = f.dim() - 2
    batch = f.shape[:bd]
    return (
        x.new_empty(*batch, topk, *x.shape[bd + 1:]),
        f.new_empty(*batch, topk, f.shape[-1]),
        f.new_empty(*batch, topk, dtype=torch.int32),
        f.new_empty(*batch, topk, dtype=torch.float64 if f.dtype == torch.float64 else torch.get_default_dtype()),
    )


def _nd_select_wide_vmap(info, in_dims, x, f, topk):
    x, f = _batched_first(info, in_dims[:2], (x, f))
    return nd_select_wide(x, f, topk), (0, 0, 0, 0)


torch.library.register_vmap(nd_select_wide, _nd_select_wide_vmap)


@torch.library.custom_op("evox_amd::nd_select", mutates_args=())
def nd_select(x: torch.Tensor, f: torch.Tensor, topk: int) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """x (..., N, *D), f (..., N, M), topk -> (x, f, rank, crowding distance) of the topk survivors."""
    runtime.require_gpu_tensor(f, "fitness")
    runtime.require_gpu_tensor(x, "decision vectors")
    if f.dim() < 2:
        raise ValueError("fitness must have shape (..., N, M)")
    bd = f.dim() - 2
    n, m = f.shape[-2:]
    if x.dim() < bd + 1 or x.shape[: bd + 1] != f.shape[: bd + 1]:
        raise ValueError(f"decision vectors {tuple(x.shape)} and fitness {tuple(f.shape)} disagree on the leading dimensions")
    if x.device != f.device:
        raise RuntimeError("decision vectors and fitness are on different devices")
    if topk > n:
        raise RuntimeError(f"selected index k out of range: topk={topk} exceeds the population size {n}")
    if topk < 1:
        raise IndexError(f"topk must be at least 1; got {topk}")
    if m == 0:
        raise ValueError("fitness must have at least one objective")
    if bd == 0 and f.dtype is torch.float32 and x.is_contiguous() and f.device.index == torch.cuda.current_device():
        # One population of float32 fitness on the current device -- what an algorithm's step passes: the same call
        # without the views and the device guard of the general path below (a third of the time of a selection of
        # 200 rows is spent on this side of the C ABI).
        out_x = torch.empty((topk,) + tuple(x.shape[1:]), dtype=x.dtype, device=x.device)
        out_f = torch.empty((topk, m), dtype=torch.float32, device=f.device)
        out_rank = torch.empty((topk,), dtype=torch.int32, device=f.device)
        out_dist = torch.empty((topk,), dtype=torch.float32, device=f.device)
        es = x.element_size()
        row_bytes = (x.numel() // n) * es
        has_x = row_bytes > 0
        stream = runtime.stream_handle(f.device)
        if runtime.small_population_kernel_fits(n, m, 1):
            _lib.call("evox_hip_batched_nd_environmental_selection", x.data_ptr() if has_x else None, row_bytes, row_bytes,
                      n * row_bytes, f.data_ptr(), 1, n, m, n * f.stride(0), f.stride(0), f.stride(1), topk,
                      out_x.data_ptr() if has_x else None, out_f.data_ptr(), out_rank.data_ptr(), out_dist.data_ptr(), stream)
            runtime.note_small_kernel_call()
        else:
            ws = runtime.workspace(n, m, f.device)

            def issue():
                _lib.call("evox_hip_nd_environmental_selection", x.data_ptr() if has_x else None, row_bytes, row_bytes,
                          f.data_ptr(), n, m, f.stride(0), f.stride(1), topk, out_x.data_ptr() if has_x else None,
                          out_f.data_ptr(), out_rank.data_ptr(), out_dist.data_ptr(), None, ws.data_ptr(), ws.numel(), stream)
                runtime.note_call(ws, stream)

            runtime.checked(issue)
        return out_x, out_f, out_rank, out_dist
    f32 = _as_f32(f, "fitness")
    batch = f.shape[:bd]
    tail = x.shape[bd + 1:]
    out_x = torch.empty(*batch, topk, *tail, dtype=x.dtype, device=x.device)
    out_f = torch.empty(*batch, topk, m, dtype=torch.float32, device=f.device)
    out_rank = torch.empty(*batch, topk, dtype=torch.int32, device=f.device)
    out_dist = torch.empty(*batch, topk, dtype=torch.float32, device=f.device)
    if out_rank.numel() == 0:
        return out_x, out_f.to(f.dtype), out_rank, out_dist
    with torch.cuda.device(f.device):
        flat_f = f32.reshape(-1, n, m)
        flat_x = x.reshape(flat_f.size(0), n, -1)
        if flat_x.stride(-1) != 1 and flat_x.size(-1) > 1:
            flat_x = flat_x.contiguous()
        row_bytes = flat_x.size(-1) * flat_x.element_size()
        fo_x = out_x.view(flat_f.size(0), topk, -1)
        fo_f = out_f.view(-1, topk, m)
        fo_r = out_rank.view(-1, topk)
        fo_d = out_dist.view(-1, topk)
        stream = runtime.stream_handle(f.device)
        has_x = row_bytes > 0
        if runtime.small_population_kernel_fits(n, m, flat_f.size(0)):
            es = flat_x.element_size()
            _lib.call("evox_hip_batched_nd_environmental_selection", flat_x.data_ptr() if has_x else None, row_bytes,
                      flat_x.stride(1) * es, flat_x.stride(0) * es, flat_f.data_ptr(), flat_f.size(0), n, m, flat_f.stride(0),
                      flat_f.stride(1), flat_f.stride(2), topk, fo_x.data_ptr() if has_x else None, fo_f.data_ptr(),
                      fo_r.data_ptr(), fo_d.data_ptr(), stream)
            runtime.note_small_kernel_call()
            return out_x, out_f.to(f.dtype), out_rank, out_dist
        batch_count = flat_f.size(0)
        es = flat_x.element_size()

        def issue():
            ws, per_launch, step = runtime.many_workspace(batch_count, n, m, topk, f.device)
            for b0, nb in _passes(batch_count, per_launch):
                _lib.call("evox_hip_many_nd_environmental_selection", flat_x[b0].data_ptr() if has_x else None, row_bytes,
                          flat_x.stride(1) * es, flat_x.stride(0) * es, flat_f[b0].data_ptr(), nb, n, m, flat_f.stride(0),
                          flat_f.stride(1), flat_f.stride(2), topk, fo_x[b0].data_ptr() if has_x else None, fo_f[b0].data_ptr(),
                          fo_r[b0].data_ptr(), fo_d[b0].data_ptr(), ws.data_ptr(), ws.numel(), stream)
                runtime.note_call(ws, stream, min(per_launch, nb), step)

        runtime.checked(issue)
    return out_x, out_f.to(f.dtype), out_rank, out_dist


@nd_select.register_fake
def _(x, f, topk):
    bd = f.dim() - 2
    batch = f.shape[:bd]
    return (
        x.new_empty(*batch, topk, *x.shape[bd + 1:]),
        f.new_empty(*batch, topk, f.shape[-1]),
        f.new_empty(*batch, topk, dtype=torch.int32),
        f.new_empty(*batch, topk, dtype=torch.float32),
    )


def _nd_select_vmap(info, in_dims, x, f, topk):
    xd, fd, _ = in_dims
    x = x.movedim(xd, 0) if xd is not None else x.unsqueeze(0).expand(info.batch_size, *x.shape)
    f = f.movedim(fd, 0) if fd is not None else f.unsqueeze(0).expand(info.batch_size, *f.shape)
    return nd_select(x, f, topk), (0, 0, 0, 0)


torch.library.register_vmap(nd_select, _nd_select_vmap)


@torch.library.custom_op("evox_amd::nd_select_two_part", mutates_args=())
def nd_select_two_part(x_a: torch.Tensor, f_a: torch.Tensor, x_b: torch.Tensor, f_b: torch.Tensor,
                       topk: int) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """nd_select on the concatenation of (x_a, f_a) and (x_b, f_b) along the rows, without making it.
    x_* (N_*, *D), f_* (N_*, M); one population (no leading batch dimensions)."""
    for t, what in ((f_a, "fitness"), (f_b, "fitness"), (x_a, "decision vectors"), (x_b, "decision vectors")):
        runtime.require_gpu_tensor(t, what)
    if f_a.dim() != 2 or f_b.dim() != 2 or f_a.size(1) != f_b.size(1):
        raise ValueError(f"fitness parts must be (N_a, M) and (N_b, M); got {tuple(f_a.shape)} and {tuple(f_b.shape)}")
    if x_a.dim() < 1 or x_b.dim() < 1 or x_a.shape[1:] != x_b.shape[1:] or x_a.dtype != x_b.dtype:
        raise ValueError("the decision vectors of the two parts differ in row shape or dtype")
    if x_a.size(0) != f_a.size(0) or x_b.size(0) != f_b.size(0):
        raise ValueError("decision vectors and fitness disagree on the number of rows")
    if len({x_a.device, x_b.device, f_a.device, f_b.device}) != 1:
        raise RuntimeError("the parts are on different devices")
    if f_a.dtype != f_b.dtype:
        raise TypeError("the fitness parts differ in dtype")
    n_a, n_b, m = f_a.size(0), f_b.size(0), f_a.size(1)
    n = n_a + n_b
    if topk > n:
        raise RuntimeError(f"selected index k out of range: topk={topk} exceeds the population size {n}")
    if topk < 1:
        raise IndexError(f"topk must be at least 1; got {topk}")
    if m == 0:
        raise ValueError("fitness must have at least one objective")
    if (n_a > 0 and n_b > 0 and f_a.dtype is torch.float32 and f_a.stride() == f_b.stride() and x_a.is_contiguous()
            and x_b.is_contiguous() and f_a.device.index == torch.cuda.current_device()
            and runtime.small_population_kernel_fits(n, m, 1)):
        # parents and offspring of a run with a few hundred individuals: one launch of the one-workgroup kernel,
        # which reads both parts where they lie (the pipeline's four launches took half as long again)
        out_x = torch.empty((topk,) + tuple(x_a.shape[1:]), dtype=x_a.dtype, device=x_a.device)
        out_f = torch.empty((topk, m), dtype=torch.float32, device=f_a.device)
        out_rank = torch.empty((topk,), dtype=torch.int32, device=f_a.device)
        out_dist = torch.empty((topk,), dtype=torch.float32, device=f_a.device)
        row_bytes = (x_a.numel() // n_a) * x_a.element_size()
        has_x = row_bytes > 0
        _lib.call("evox_hip_small_nd_environmental_selection_two_part", x_a.data_ptr() if has_x else None,
                  x_b.data_ptr() if has_x else None, row_bytes, row_bytes, f_a.data_ptr(), n_a, f_b.data_ptr(), n_b, m,
                  f_a.stride(0), f_a.stride(1), topk, out_x.data_ptr() if has_x else None, out_f.data_ptr(),
                  out_rank.data_ptr(), out_dist.data_ptr(), runtime.stream_handle(f_a.device))
        runtime.note_small_kernel_call()
        return out_x, out_f, out_rank, out_dist
    fa32, fb32 = _as_f32(f_a, "fitness"), _as_f32(f_b, "fitness")
    tail = x_a.shape[1:]
    out_x = torch.empty(topk, *tail, dtype=x_a.dtype, device=x_a.device)
    out_f = torch.empty(topk, m, dtype=torch.float32, device=f_a.device)
    out_rank = torch.empty(topk, dtype=torch.int32, device=f_a.device)
    out_dist = torch.empty(topk, dtype=torch.float32, device=f_a.device)
    with torch.cuda.device(f_a.device):
        width = 1
        for d in tail:
            width *= d
        xa, xb = x_a.reshape(n_a, width), x_b.reshape(n_b, width)
        if xa.size(1) > 1 and xa.stride(1) != 1:
            xa = xa.contiguous()
        if xb.size(1) > 1 and xb.stride(1) != 1:
            xb = xb.contiguous()
        es = xa.element_size()
        row_bytes = xa.size(1) * es
        has_x = row_bytes > 0
        ws = runtime.workspace(n, m, f_a.device)
        stream = runtime.stream_handle(f_a.device)
        def issue():
            _lib.call("evox_hip_nd_environmental_selection_two_part", xa.data_ptr() if has_x else None, xa.stride(0) * es,
                      xb.data_ptr() if has_x else None, xb.stride(0) * es, row_bytes, fa32.data_ptr(), n_a, fa32.stride(0),
                      fa32.stride(1), fb32.data_ptr(), n_b, fb32.stride(0), fb32.stride(1), m, topk,
                      out_x.data_ptr() if has_x else None, out_f.data_ptr(), out_rank.data_ptr(), out_dist.data_ptr(), None,
                      ws.data_ptr(), ws.numel(), stream)
            runtime.note_call(ws, stream)

        runtime.checked(issue)
    return out_x, out_f.to(f_a.dtype), out_rank, out_dist


@nd_select_two_part.register_fake
def _(x_a, f_a, x_b, f_b, topk):
    return (
        x_a.new_empty(topk, *x_a.shape[1:]),
        f_a.new_empty(topk, f_a.shape[-1]),
        f_a.new_empty(topk, dtype=torch.int32),
        f_a.new_empty(topk, dtype=torch.float32),
    )


def _nd_select_two_part_vmap(info, in_dims, x_a, f_a, x_b, f_b, topk):
    # populations side by side: the concatenation is the definition of the result, and the batched operator
    # takes small populations through the one-workgroup kernel
    x_a, f_a, x_b, f_b = _batched_first(info, in_dims[:4], (x_a, f_a, x_b, f_b))
    return nd_select(torch.cat([x_a, x_b], dim=1), torch.cat([f_a, f_b], dim=1), topk), (0, 0, 0, 0)


torch.library.register_vmap(nd_select_two_part, _nd_select_two_part_vmap)


@torch.library.custom_op("evox_amd::stable_argsort_step", mutates_args=())
def stable_argsort_step(key: torch.Tensor, kind: int, prev: Optional[torch.Tensor]) -> torch.Tensor:
    """One step of lexsort on a 1-D key of 4-byte elements: ``prev`` (int32 order, or None for the
    identity) rearranged by a stable ascending sort of ``key[prev]``.  kind 0: float32, 1: int32,
    2: uint32 bit patterns held in an int32 tensor.  Returns an int32 order."""
    runtime.require_gpu_tensor(key, "key")
    if key.dim() != 1 or key.element_size() != 4 or kind not in (0, 1, 2):
        raise ValueError("key must be one-dimensional with 4-byte elements and kind 0, 1 or 2")
    if (kind == 0) != (key.dtype == torch.float32):
        raise TypeError(f"kind {kind} does not fit a key of dtype {key.dtype}")
    n = key.size(0)
    out = torch.empty(n, dtype=torch.int32, device=key.device)
    if n == 0:
        return out
    if prev is not None:
        runtime.require_gpu_tensor(prev, "prev")
        if prev.dtype != torch.int32 or prev.shape != (n,):
            raise ValueError("prev must be an int32 order of the same length as the key")
        prev = prev.contiguous()
    with torch.cuda.device(key.device):
        ws = runtime.sort_workspace(n, key.device)
        stream = runtime.stream_handle(key.device)
        _lib.call("evox_hip_stable_argsort_step", key.data_ptr(), kind, key.stride(0), n,
                  None if prev is None else prev.data_ptr(), out.data_ptr(), ws.data_ptr(), ws.numel(), stream)
        # only the radix sort of long keys waits on the device and keeps a control block
        if _argsort_waits(n):
            runtime.note_call(ws, stream)
        else:
            runtime.note_small_kernel_call()
    return out


@stable_argsort_step.register_fake
def _(key, kind, prev):
    return key.new_empty(key.shape, dtype=torch.int32)


@torch.library.custom_op("evox_amd::stable_argsort_rows", mutates_args=())
def stable_argsort_rows(key: torch.Tensor, kind: int, prev: Optional[torch.Tensor]) -> torch.Tensor:
    """``stable_argsort_step`` for every row of a 2-D key at once: ``prev`` (int32 orders, one per row, or
    None for the identity) rearranged, row by row, by a stable ascending sort of ``key[r, prev[r]]``.
    The key may have any strides; ``prev`` is made contiguous.  Returns int32 orders of the key's shape."""
    runtime.require_gpu_tensor(key, "key")
    if key.dim() != 2 or key.element_size() != 4 or kind not in (0, 1, 2):
        raise ValueError("key must be two-dimensional with 4-byte elements and kind 0, 1 or 2")
    if (kind == 0) != (key.dtype == torch.float32):
        raise TypeError(f"kind {kind} does not fit a key of dtype {key.dtype}")
    batch, n = key.shape
    out = torch.empty((batch, n), dtype=torch.int32, device=key.device)
    if batch == 0 or n == 0:
        return out
    if prev is not None:
        runtime.require_gpu_tensor(prev, "prev")
        if prev.dtype != torch.int32 or prev.shape != (batch, n):
            raise ValueError("prev must hold one int32 order per row of the key")
        prev = prev.contiguous()
    if key.stride(0) < 0 or key.stride(1) < 0:
        key = key.contiguous()
    with torch.cuda.device(key.device):
        ws = runtime.sort_workspace(n, key.device)
        stream = runtime.stream_handle(key.device)
        _lib.call("evox_hip_stable_argsort_step_batched", key.data_ptr(), kind, key.stride(0), key.stride(1), batch, n,
                  None if prev is None else prev.data_ptr(), out.data_ptr(), ws.data_ptr(), ws.numel(), stream)
        if _argsort_waits(n) and (batch < 2 or n > _ROWS_ARGSORT_MAX):
            runtime.note_call(ws, stream)
        else:
            runtime.note_small_kernel_call()
    return out


@stable_argsort_rows.register_fake
def _(key, kind, prev):
    return key.new_empty(key.shape, dtype=torch.int32)


def _stable_argsort_step_vmap(info, in_dims, key, kind, prev):
    key, prev = _batched_first(info, (in_dims[0], in_dims[2]), (key, prev))
    return stable_argsort_rows(key, kind, prev), 0  # one sort per row


def _stable_argsort_rows_vmap(info, in_dims, key, kind, prev):
    key, prev = _batched_first(info, (in_dims[0], in_dims[2]), (key, prev))
    flat_prev = None if prev is None else prev.reshape(-1, prev.shape[-1])
    return stable_argsort_rows(key.reshape(-1, key.shape[-1]), kind, flat_prev).view(key.shape), 0


torch.library.register_vmap(stable_argsort_step, _stable_argsort_step_vmap)
torch.library.register_vmap(stable_argsort_rows, _stable_argsort_rows_vmap)


@torch.library.custom_op("evox_amd::hv_contributions", mutates_args=())
def hv_contributions(fit: torch.Tensor, samples: torch.Tensor, alpha: torch.Tensor, scale: float) -> torch.Tensor:
    """fit (N, M), samples (S, M), alpha (N,) float32 -> (N,) float32:
    scale * sum over the samples s that point i covers of alpha[max(c_s - 1, 0)], c_s = points covering s."""
    for t, what in ((fit, "fitness"), (samples, "samples"), (alpha, "alpha")):
        runtime.require_gpu_tensor(t, what)
    if fit.dim() != 2 or samples.dim() != 2 or fit.size(1) != samples.size(1) or alpha.shape != (fit.size(0),):
        raise ValueError("expected fit (N, M), samples (S, M) and alpha (N,)")
    n, m = fit.shape
    n_sample = samples.size(0)
    out = torch.zeros(n, dtype=torch.float32, device=fit.device)
    if n == 0 or n_sample == 0 or m == 0:
        return out
    with torch.cuda.device(fit.device):
        fit_t = _as_f32(fit, "fitness").t().contiguous()
        samples_t = _as_f32(samples, "samples").t().contiguous()
        alpha32 = _as_f32(alpha, "alpha").contiguous()
        need = int(_lib.lib().evox_hip_hv_workspace_bytes(n, n_sample))
        ws = torch.empty(need, dtype=torch.uint8, device=fit.device)
        _lib.call("evox_hip_hv_contributions", fit_t.data_ptr(), samples_t.data_ptr(), alpha32.data_ptr(), n, m, n_sample,
                  float(scale), out.data_ptr(), ws.data_ptr(), ws.numel(), runtime.stream_handle(fit.device))
    return out


@hv_contributions.register_fake
def _(fit, samples, alpha, scale):
    return fit.new_empty(fit.shape[0], dtype=torch.float32)


def _hv_contributions_vmap(info, in_dims, fit, samples, alpha, scale):
    fit, samples, alpha = _batched_first(info, in_dims[:3], (fit, samples, alpha))
    return torch.stack([hv_contributions(fit[b], samples[b], alpha[b], scale) for b in range(info.batch_size)]), 0


torch.library.register_vmap(hv_contributions, _hv_contributions_vmap)


@torch.library.custom_op("evox_amd::hv_covered_count", mutates_args=())
def hv_covered_count(points: torch.Tensor, samples: torch.Tensor) -> torch.Tensor:
    """points (N, M), samples (S, M) float32 -> 0-d int64: the number of samples that some point exceeds
    strictly in every objective."""
    runtime.require_gpu_tensor(points, "points")
    runtime.require_gpu_tensor(samples, "samples")
    if points.dim() != 2 or samples.dim() != 2 or points.size(1) != samples.size(1):
        raise ValueError("expected points (N, M) and samples (S, M)")
    n, m = points.shape
    n_sample = samples.size(0)
    out = torch.zeros((), dtype=torch.int64, device=points.device)
    if n == 0 or n_sample == 0:
        return out
    if m == 0:  # an empty conjunction holds: every sample is covered (torch.all over an empty dimension)
        return out + n_sample
    with torch.cuda.device(points.device):
        points_t = _as_f32(points, "points").t().contiguous()
        samples_t = _as_f32(samples, "samples").t().contiguous()
        need = int(_lib.lib().evox_hip_hv_covered_workspace_bytes(n_sample))
        ws = torch.empty(need, dtype=torch.uint8, device=points.device)
        _lib.call("evox_hip_hv_covered_count", points_t.data_ptr(), samples_t.data_ptr(), n, m, n_sample, out.data_ptr(),
                  ws.data_ptr(), ws.numel(), runtime.stream_handle(points.device))
    return out


@hv_covered_count.register_fake
def _(points, samples):
    return points.new_empty((), dtype=torch.int64)


def _hv_covered_count_vmap(info, in_dims, points, samples):
    points, samples = _batched_first(info, in_dims, (points, samples))
    return torch.stack([hv_covered_count(points[b], samples[b]) for b in range(info.batch_size)]), 0


torch.library.register_vmap(hv_covered_count, _hv_covered_count_vmap)


@torch.library.custom_op("evox_amd::tournament_pick", mutates_args=())
def tournament_pick(parents: torch.Tensor, fitness: torch.Tensor) -> torch.Tensor:
    """parents (n_round, t) int64 candidate indices, fitness (candidates, keys) float32 -> (n_round,) int64 winners."""
    runtime.require_gpu_tensor(parents, "parents")
    runtime.require_gpu_tensor(fitness, "fitness")
    if parents.dim() != 2 or fitness.dim() != 2 or parents.dtype != torch.int64:
        raise ValueError("parents must be (n_round, tournament_size) int64 and fitness (candidates, keys)")
    # (keys of other dtypes -- float64 distances under a float64 default, integers -- as per-column dense ranks, which
    # keep every comparison)
    fit = _order_preserving_f32(fitness, "fitness") if fitness.numel() > 0 else fitness.float()
    par = parents.contiguous()
    out = torch.empty(par.size(0), dtype=torch.int64, device=parents.device)
    with torch.cuda.device(parents.device):
        _lib.call("evox_hip_tournament_pick", par.data_ptr(), par.size(0), par.size(1), fit.data_ptr(), fit.size(0), fit.size(1),
                  fit.stride(0), fit.stride(1), out.data_ptr(), runtime.stream_handle(parents.device))
    return out


@tournament_pick.register_fake
def _(parents, fitness):
    return parents.new_empty(parents.shape[0])


def _tournament_pick_vmap(info, in_dims, parents, fitness):
    # tournaments of all the mapped populations in one launch: population b's candidates are rows b * candidates ...
    parents, fitness = _batched_first(info, in_dims, (parents, fitness))
    batch, candidates = fitness.shape[0], fitness.shape[1]
    offset = (torch.arange(batch, device=parents.device, dtype=torch.int64) * candidates).view(batch, 1, 1)
    flat = tournament_pick((parents + offset).reshape(-1, parents.shape[-1]), fitness.reshape(batch * candidates, -1))
    return flat.view(batch, -1) - offset.view(batch, 1), 0


torch.library.register_vmap(tournament_pick, _tournament_pick_vmap)


def tournament_keys_fit(keys) -> bool:
    """Whether tournament_pick_keys takes this list of key tensors: one to four float32 or int32 vectors of one length
    on one GPU (anything else goes through the stacked copy and tournament_pick)."""
    if not 1 <= len(keys) <= 4:
        return False
    first = keys[0]
    return all(isinstance(t, torch.Tensor) and t.is_cuda and t.dim() == 1 and t.dtype in (torch.float32, torch.int32)
               and t.device == first.device and t.size(0) == first.size(0) for t in keys) and first.size(0) > 0


def plain_eager() -> bool:
    """True when no transform (vmap, grad), tracer (torch.compile, make_fx) or dispatch mode is looking at the call,
    so that an operator's implementation may be called as the Python function it is: the dispatcher's way to the same
    function costs about 10 us, a third of a host-bound call like a tournament selection."""
    try:
        return (not torch.compiler.is_compiling() and torch._C._functorch.peek_interpreter_stack() is None
                and _get_current_dispatch_mode() is None)
    except AttributeError:  # another torch: take the dispatcher
        return False


def tournament_pick_keys_direct(parents: torch.Tensor, keys: List[torch.Tensor]) -> torch.Tensor:
    """parents (n_round, t) int64 candidate indices, keys: one to four (candidates,) float32 or int32 vectors ->
    (n_round,) int64 winners, as tournament_pick on torch.stack(keys, dim=1) without making it."""
    runtime.require_gpu_tensor(parents, "parents")
    if parents.dim() != 2 or parents.dtype != torch.int64 or not tournament_keys_fit(keys):
        raise ValueError("parents must be (n_round, tournament_size) int64 and keys one to four float32 or int32 vectors")
    par = parents.contiguous()
    out = torch.empty(par.size(0), dtype=torch.int64, device=parents.device)
    count = len(keys)
    pointers = (ctypes.c_void_p * count)(*[t.data_ptr() for t in keys])
    kinds = (ctypes.c_int32 * count)(*[0 if t.dtype is torch.float32 else 1 for t in keys])
    strides = (ctypes.c_int64 * count)(*[t.stride(0) for t in keys])
    with torch.cuda.device(parents.device):
        _lib.call("evox_hip_tournament_pick_keys", par.data_ptr(), par.size(0), par.size(1), keys[0].size(0), count,
                  ctypes.addressof(pointers), ctypes.addressof(kinds), ctypes.addressof(strides), out.data_ptr(),
                  runtime.stream_handle(parents.device))
    return out


@torch.library.custom_op("evox_amd::tournament_pick_keys", mutates_args=())
def tournament_pick_keys(parents: torch.Tensor, keys: List[torch.Tensor]) -> torch.Tensor:
    """tournament_pick_keys_direct as an operator (traceable, with a batching rule)."""
    return tournament_pick_keys_direct(parents, keys)


@tournament_pick_keys.register_fake
def _(parents, keys):
    return parents.new_empty(parents.shape[0])


def _tournament_pick_keys_vmap(info, in_dims, parents, keys):
    # mapped populations: the stacked form, whose batching rule puts all tournaments into one launch
    parents_dim, keys_dims = in_dims
    size = info.batch_size
    moved = [k.movedim(d, 0) if d is not None else k.unsqueeze(0).expand(size, *k.shape) for k, d in zip(keys, keys_dims)]
    par = parents.movedim(parents_dim, 0) if parents_dim is not None else parents.unsqueeze(0).expand(size, *parents.shape)
    stacked = torch.stack([k.to(torch.float32) for k in moved], dim=-1)
    return _tournament_pick_vmap(info, (0, 0), par, stacked)


torch.library.register_vmap(tournament_pick_keys, _tournament_pick_keys_vmap)
