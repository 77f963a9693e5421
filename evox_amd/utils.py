"""Drop-in replacement for ``evox.utils.lexsort`` (src/evox/utils/jit_fix_operator.py:213-252) on the GPU.

The reference chains one stable ``torch.argsort`` per key; here every link of that chain is one stable
argsort step on the GPU (``evox_amd::stable_argsort_step`` for a one-dimensional sort: a counting kernel up
to 8192 positions, above that the segmented LSD radix sort that also orders large fronts inside the
selection path; ``evox_amd::stable_argsort_rows`` for many sorts along one dimension at once).
"""

from typing import List, Sequence, Tuple

import torch

from . import ops

_SIGN64 = -(2**63)


def _key_parts(key: torch.Tensor) -> List[Tuple[torch.Tensor, int]]:
    """A key as a list of (4-byte tensor, kind) sorted least significant part first."""
    if key.dtype == torch.float32:
        return [(key, 0)]
    if key.dtype in (torch.float16, torch.bfloat16):
        return [(key.float(), 0)]
    if key.dtype in (torch.int32,):
        return [(key, 1)]
    if key.dtype in (torch.int8, torch.int16, torch.uint8, torch.bool):
        return [(key.to(torch.int32), 1)]
    if key.dtype == torch.int64:
        return [((key & 0xFFFFFFFF).to(torch.int32), 2), ((key >> 32).to(torch.int32), 1)]
    if key.dtype == torch.float64:
        # order-preserving 64-bit pattern: -0.0 ties with 0.0, NaN after every number
        bits = (key + 0.0).view(torch.int64)
        ordered = torch.where(bits < 0, ~bits, bits | _SIGN64)
        ordered = torch.where(torch.isnan(key), torch.full_like(ordered, -1), ordered)
        return [((ordered & 0xFFFFFFFF).to(torch.int32), 2), ((ordered >> 32).to(torch.int32), 2)]
    raise TypeError(f"lexsort: unsupported key dtype {key.dtype}")


def lexsort(keys: Sequence[torch.Tensor], dim: int = -1) -> torch.Tensor:
    """Indices that sort by the LAST key, ties by the key before it, ..., ties by position.

    Same contract as the reference's ``lexsort`` (jit_fix_operator.py:213-252): every key has the same
    shape, the sort runs along ``dim``, NaN sorts after every number and the result is ``int64``.
    """
    keys = list(keys)
    if not keys:
        raise IndexError("lexsort needs at least one key")
    shape = keys[0].shape
    if any(k.shape != shape for k in keys):
        raise ValueError("lexsort: all keys must have the same shape")
    if keys[0].dim() == 0:
        raise IndexError("lexsort: keys must have at least one dimension")
    if keys[0].numel() == 0:
        keys[0].size(dim)  # an IndexError for a dimension the keys do not have
        return torch.empty(shape, dtype=torch.int64, device=keys[0].device)
    moved = [k.movedim(dim, -1) for k in keys]
    n = moved[0].shape[-1]
    rows = [m.reshape(-1, n) for m in moved]
    order = None
    if rows[0].size(0) == 1:
        for key_rows in rows:
            for part, kind in _key_parts(key_rows[0]):
                order = ops.stable_argsort_step(part, kind, order)
        out = order.to(torch.int64)
    else:  # every row in the same launches
        for key_rows in rows:
            for part, kind in _key_parts(key_rows):
                order = ops.stable_argsort_rows(part, kind, order)
        out = order.to(torch.int64)
    return out.reshape(moved[0].shape).movedim(-1, dim)
