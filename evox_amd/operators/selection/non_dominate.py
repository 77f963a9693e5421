"""Drop-in replacements for the three selection operators of
``evox.operators.selection.non_dominate`` (src/evox/operators/selection/non_dominate.py),
with the same names, positional arguments, return arity, dtypes and devices.  The work is done by
hand-written gfx950 kernels reached through the ``evox_amd::`` custom operators, for float32 fitness
(the kernels of the selection path) as for float64 and integer fitness (kernels that read 8-byte
values); there is no PyTorch or CPU implementation behind them.
"""

from typing import Optional, Tuple

import torch

from ... import ops


def _plain(op, *tensors):
    """``op`` itself, or -- for plain tensors with no transform, tracer or dispatch mode looking at the call
    (``ops.plain_eager``) -- the function that the custom operator wraps: what the operator would run after four
    layers of dispatch, a fifth of the time of a selection of 200 rows.  Tensor subclasses (fake tensors, functional
    wrappers) and tensors that require a gradient keep to the operator."""
    for t in tensors:
        if type(t) is not torch.Tensor or t.requires_grad:
            return op
    return getattr(op, "_init_fn", op) if ops.plain_eager() else op  # (another torch may not keep it there: the operator then)


def non_dominate_rank(x: torch.Tensor) -> torch.Tensor:
    """Non-domination rank of every row of ``x`` (minimisation).

    Same contract as the reference's ``non_dominate_rank`` (non_dominate.py:172-195):
    ``x`` is ``(N, M)``; the result is ``int32 (N,)`` on ``x.device``; rank 0 is the Pareto front,
    rank r + 1 the front of what remains after removing ranks 0..r.  Rows holding a NaN neither
    dominate nor are dominated (rank 0); identical rows do not dominate each other.  Any real dtype is
    accepted, as in the reference: float32 (and float16 / bfloat16, widened exactly) goes to the kernels
    as it is, other dtypes through per-objective dense ranks, which keep every comparison.
    """
    return _plain(ops.nd_rank, x)(x)


def non_dominate_rank_until(x: torch.Tensor, count: int) -> torch.Tensor:
    """``non_dominate_rank(x)`` peeled only as far as the front that holds the ``count``-th best row.

    Rows of that front and of the better ones get their rank; every other row gets ``2**31 - 1``.  Not a name
    of the reference; it serves its callers that rank a merged population only to cut it at a front --
    ``worst = torch.topk(rank, k, largest=False)[0][-1]; keep = rank <= worst`` in NSGA-III
    (src/evox/algorithms/mo/nsga3.py:169-171) and the argsort form of the same in HypE
    (src/evox/algorithms/mo/hype.py:135-138) -- which read the same ``worst`` and ``keep`` from the
    truncated ranks without the fronts behind the cut ever being peeled.
    """
    return _plain(ops.nd_rank_until, x)(x, int(count))


def non_dominated_mask(x: torch.Tensor) -> torch.Tensor:
    """``non_dominate_rank(x) == 0`` without ranking anything else: bool ``(N,)`` on ``x.device``.

    Not a name of the reference; it replaces the two statements with which ``EvalMonitor.get_pf_fitness``
    and ``get_pf`` (src/evox/workflows/eval_monitor.py:301-302, :333-335) rank the whole evaluation
    history only to keep the rows of rank 0.  No dominance matrix is built, so memory stays linear in
    ``N`` and a history of millions of rows can be filtered.
    """
    return _plain(ops.nd_first_front, x)(x)


def crowding_distance(costs: torch.Tensor, mask: Optional[torch.Tensor]) -> torch.Tensor:
    """Crowding distance of the rows selected by ``mask`` (all rows when ``mask`` is ``None``).

    Same contract as the reference's ``crowding_distance`` (non_dominate.py:198-231): per objective
    the selected rows are sorted by (cost, row index) with NaN last; the first and last row of any
    objective get ``+inf``; every other selected row gets the sum over objectives of
    ``(next - previous) / (last - first)``; unselected rows get ``-inf``.  The result has torch's
    default float dtype, and, as in the reference (its scatter at :224-225), ``costs`` must have that
    dtype too.  With the default dtype set to float64 the distances are computed in float64, and integer costs
    are subtracted exactly and divided in the default float dtype, by kernels that read 8-byte values.
    """
    if costs.is_floating_point() and costs.dtype != torch.get_default_dtype():
        raise RuntimeError(
            f"crowding_distance: expected costs.dtype to be the default dtype {torch.get_default_dtype()}, got {costs.dtype}"
        )
    if costs.dtype == torch.float64 or not costs.is_floating_point():
        return ops.crowding_wide(costs, mask)
    return _plain(ops.crowding, costs, *(() if mask is None else (mask,)))(costs, mask)


def nd_environmental_selection(x: torch.Tensor, f: torch.Tensor, topk: int) -> Tuple[torch.Tensor, ...]:
    """NSGA-II environmental selection of ``topk`` rows.

    Same contract as the reference's ``nd_environmental_selection`` (non_dominate.py:234-254):
    returns ``(x[order], f[order], rank[order], crowding_dis[order])`` where ``order`` sorts by rank
    ascending, then by the crowding distance within the last admitted front descending (NaN last),
    then by row index; the distance of rows in better fronts is ``-inf``.  ``topk > N`` raises
    ``RuntimeError`` and ``topk < 1`` raises ``IndexError`` as ``torch.topk`` / indexing do there.
    """
    if f.is_floating_point() and f.dtype not in (torch.float16, torch.bfloat16) and f.dtype != torch.get_default_dtype():
        # the reference fails in the scatter of its crowding distance (non_dominate.py:224-225)
        raise RuntimeError(
            f"nd_environmental_selection: expected f.dtype to be the default dtype {torch.get_default_dtype()}, got {f.dtype}"
        )
    if f.dtype == torch.float64 or not (f.is_floating_point() or f.is_complex() or f.dtype == torch.bool):
        return ops.nd_select_wide(x, f, int(topk))
    return _plain(ops.nd_select, x, f)(x, f, int(topk))


def nd_environmental_selection_two_part(
    x_a: torch.Tensor, f_a: torch.Tensor, x_b: torch.Tensor, f_b: torch.Tensor, topk: int
) -> Tuple[torch.Tensor, ...]:
    """``nd_environmental_selection(cat([x_a, x_b]), cat([f_a, f_b]), topk)`` without the two ``cat`` copies.

    Not a name of the reference; it replaces the merge step of its NSGA-II
    (src/evox/algorithms/mo/nsga2.py:99-102), where parents and offspring are concatenated only to be
    handed to the selection.  Same four results as ``nd_environmental_selection``.  Fitness that the two-part
    kernels do not read (float64, integers, parts of different dtypes) is concatenated after all, with
    ``torch.cat``'s promotion of the dtypes, and goes the way of ``nd_environmental_selection``.
    """
    narrow = (torch.float32, torch.float16, torch.bfloat16)
    if f_a.dtype != f_b.dtype or f_a.dtype not in narrow or x_a.dtype != x_b.dtype:
        return nd_environmental_selection(torch.cat([x_a, x_b], dim=0), torch.cat([f_a, f_b], dim=0), int(topk))
    return _plain(ops.nd_select_two_part, x_a, f_a, x_b, f_b)(x_a, f_a, x_b, f_b, int(topk))
