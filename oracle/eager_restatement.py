"""TEST INFRASTRUCTURE ONLY -- CPU restatement of the reference's eager selection path.

This module is the parity checker for the HIP kernels.  Only ``tests/``, ``__graft_entry__.smoke()``
and the ``cpu_baseline`` leg of ``bench.py`` may import it; the product package never does.

It restates, operation for operation and with the same dtypes, the eager (non-compiled) branch of
the reference's multi-objective environmental selection, on torch CPU tensors:

  pareto_dominance          <- src/evox/operators/selection/non_dominate.py:6-26
  peel_once                 <- src/evox/operators/selection/non_dominate.py:29-59
  ranks_by_peeling          <- src/evox/operators/selection/non_dominate.py:161-169, 172-195
  ranks_by_peeling_batched  <- src/evox/operators/selection/non_dominate.py:107-125
  chained_stable_argsort    <- src/evox/utils/jit_fix_operator.py:246-252
  crowding                  <- src/evox/operators/selection/non_dominate.py:198-231
  environmental_selection   <- src/evox/operators/selection/non_dominate.py:234-254
  tournament_winners        <- src/evox/operators/selection/tournament_selection.py:18-27
  first_front_mask          <- src/evox/workflows/eval_monitor.py:301-302 (= :333-334)
  merged_selection          <- src/evox/algorithms/mo/nsga2.py:99-102
  front_cut                 <- src/evox/algorithms/mo/nsga3.py:169-171 (hype.py:135-138 is the argsort form)
  hv_contributions          <- src/evox/algorithms/mo/hype.py:12-39 (cal_hv, with the uniform draws handed in)

How each function is pinned (tests/test_oracle.py):
  * dominance / ranks: tiny-input brute force, longest-dominator-chain definition, Deb's fast
    non-dominated sort, closed forms (chain, all-equal, M=1 dense rank, layered construction).
  * chained_stable_argsort: numpy.lexsort on the same keys.
  * first_front_mask: the independent definition "no row dominates it" (brute_force.dominates_matrix).
  * tournament_winners: explicit tuple comparison and numpy.lexsort per tournament.
  * hv_contributions: an explicit loop over samples and points (brute_force.hv_contributions_brute) and the
    closed form for a single point (its contribution is the whole sampled box).
  * crowding / environmental_selection: independent numpy brute force, hand-worked examples, and
    the golden vectors under tests/golden/ (written once from the reference itself).
"""

from typing import List, Optional

import torch


def pareto_dominance(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """bool (n1, n2): entry (i, j) says a_i dominates b_j (minimisation).  non_dominate.py:6-26."""
    lhs = a[:, None, :]
    rhs = b[None, :, :]
    no_worse = (lhs <= rhs).all(dim=2)
    better_somewhere = (lhs < rhs).any(dim=2)
    return no_worse & better_somewhere


def peel_once(dom: torch.Tensor, count: torch.Tensor, front: torch.Tensor, rank: torch.Tensor, level: int):
    """One pass of non_dominate.py:29-59: stamp the front, subtract what it dominates, retire it."""
    rank = torch.where(front, level, rank)
    released = torch.sum(front.unsqueeze(-1) * dom, dim=-2)
    count = count - released
    count = count - front.int()
    return rank, count


def ranks_by_peeling(f: torch.Tensor) -> torch.Tensor:
    """int32 (N,) non-domination rank.  non_dominate.py:172-195 with the eager loop of :161-169."""
    n = f.size(0)
    dom = pareto_dominance(f, f)
    count = dom.sum(dim=0)  # int64: how many rows dominate column j
    rank = torch.zeros(n, dtype=torch.int32, device=f.device)
    front = count == 0
    level = 0
    while bool(front.any()):
        rank, count = peel_once(dom, count, front, rank, level)
        level += 1
        front = count == 0
    return rank


def ranks_by_peeling_batched(f: torch.Tensor) -> torch.Tensor:
    """(B, N, M) -> int32 (B, N).  Batched loop of non_dominate.py:107-125: the loop runs while any
    population still has a front; a population whose front is empty keeps its (empty) front."""
    b, n, _ = f.shape
    lhs = f[:, :, None, :]
    rhs = f[:, None, :, :]
    dom = (lhs <= rhs).all(dim=-1) & (lhs < rhs).any(dim=-1)
    count = dom.sum(dim=-2)
    rank = torch.zeros(b, n, dtype=torch.int32, device=f.device)
    front = count == 0
    level = 0
    while bool(front.any()):
        rank, count = peel_once(dom, count, front, rank, level)
        level += 1
        nxt = count == 0
        front = torch.where(front.any(dim=-1, keepdim=True), nxt, front)
    return rank


def chained_stable_argsort(keys: List[torch.Tensor], dim: int = -1) -> torch.Tensor:
    """Last key is primary; ties fall to earlier keys, then to index.  jit_fix_operator.py:246-252."""
    order = torch.argsort(keys[0], dim=dim, stable=True)
    for key in keys[1:]:
        moved = key.gather(dim, order)
        step = torch.argsort(moved, dim=dim, stable=True)
        order = order.gather(dim, step)
    return order


def crowding(costs: torch.Tensor, mask: Optional[torch.Tensor]) -> torch.Tensor:
    """Crowding distance of the masked rows; -inf elsewhere.  non_dominate.py:198-231.

    Kept quirks: the scratch buffer has torch's default dtype (:224), its rows at sorted position
    0 and N-1 are never written by the scatter (:225) and only matter through the two +inf row
    assignments (:226-227); a zero objective range divides 0 by 0."""
    n = costs.size(0)
    if mask is None:
        n_valid = n
        mask = torch.ones(n, dtype=torch.bool)
    else:
        n_valid = mask.sum()
    outside = (~mask).unsqueeze(1).expand(-1, costs.size(1)).to(costs.dtype)
    order = chained_stable_argsort([costs, outside], dim=0)
    sorted_costs = torch.gather(costs, dim=0, index=order)
    span = sorted_costs[n_valid - 1] - sorted_costs[0]
    per_objective = torch.empty(sorted_costs.size(), device=costs.device)
    per_objective = per_objective.scatter(0, order[1:-1], (sorted_costs[2:] - sorted_costs[:-2]) / span)
    per_objective[order[0], :] = torch.inf
    per_objective[order[n_valid - 1], :] = torch.inf
    per_objective = torch.where(mask.unsqueeze(1), per_objective, -torch.inf)
    return torch.sum(per_objective, dim=1)


def environmental_selection(x: torch.Tensor, f: torch.Tensor, topk: int, return_all: bool = False):
    """NSGA-II survivor selection.  non_dominate.py:234-254.

    With ``return_all`` the full-length rank, crowding distance and the selected order are
    returned as well (they are intermediates of the reference, used by the parity tests)."""
    rank = ranks_by_peeling(f)
    worst = torch.topk(rank, topk, largest=False)[0][-1]
    last_front = rank == worst
    dist = crowding(f, last_front)
    order = chained_stable_argsort([-dist, rank])[:topk]
    picked = (x[order], f[order], rank[order], dist[order])
    if return_all:
        return picked, rank, dist, order
    return picked


def tournament_winners(parents: torch.Tensor, fitnesses: List[torch.Tensor]) -> torch.Tensor:
    """Winner of each row of ``parents`` (n_round, t): tournament_selection.py:18-27 without the random
    draw (:21), which the caller supplies so that the checker and the GPU path see the same tournaments."""
    table = torch.stack(fitnesses, dim=1)
    keys = table[parents]
    ordering = chained_stable_argsort(keys.unbind(-1))
    return torch.gather(parents, 1, ordering[:, 0].unsqueeze(1)).squeeze()


def tournament_winners_single(parents: torch.Tensor, fitness: torch.Tensor) -> torch.Tensor:
    """Winner of each row of ``parents`` (n_round, t) on one fitness tensor: tournament_selection.py:48-54
    without the random draw (:47)."""
    candidates_fitness = fitness[parents]
    winner_indices = torch.argmin(candidates_fitness, dim=1)
    return torch.gather(parents, 1, winner_indices.unsqueeze(1)).squeeze()


def first_front_mask(f: torch.Tensor) -> torch.Tensor:
    """bool (N,): the rows that EvalMonitor.get_pf_fitness / get_pf keep (eval_monitor.py:301-302, :333-335):
    the whole history is ranked and only ``rank == 0`` is used."""
    return ranks_by_peeling(f) == 0


def merged_selection(x_a, f_a, x_b, f_b, topk: int, return_all: bool = False):
    """The merge step of NSGA-II, nsga2.py:99-102: concatenate parents and offspring, then select."""
    return environmental_selection(torch.cat([x_a, x_b], dim=0), torch.cat([f_a, f_b], dim=0), topk, return_all)


def front_cut(f: torch.Tensor, count: int):
    """(worst_rank, keep mask, rank) of nsga3.py:169-171: rank everything, find the rank of the count-th
    best row, keep the rows up to that front."""
    rank = ranks_by_peeling(f)
    worst = torch.topk(rank, count, largest=False)[0][-1]
    return worst, rank <= worst, rank


def hv_contributions(fit: torch.Tensor, ref: torch.Tensor, pop_size, uniform: torch.Tensor) -> torch.Tensor:
    """cal_hv of hype.py:12-39 with the draws of its torch.rand (:28) supplied as ``uniform`` (n_sample, m)."""
    n, m = fit.size()
    n_sample = uniform.size(0)
    alpha = torch.cumprod(
        torch.cat([torch.ones(1), (pop_size - torch.arange(1, n)) / (n - torch.arange(1, n))]), dim=0
    ) / torch.arange(1, n + 1)
    alpha = torch.nan_to_num(alpha)
    f_min = torch.min(fit, dim=0).values
    samples = uniform * (ref - f_min) + f_min
    ds = torch.zeros(n_sample, dtype=torch.int64)
    pds = (fit.unsqueeze(0).expand(n_sample, -1, -1) - samples.unsqueeze(1).expand(-1, n, -1) <= 0).all(dim=2)
    ds = torch.sum(torch.where(pds, ds.unsqueeze(1) + 1, ds.unsqueeze(1)), dim=1)
    ds = torch.where(ds == 0, ds, ds - 1)
    temp = torch.where(pds.T, ds.unsqueeze(0), -1)
    value = torch.where(temp != -1, alpha[temp], torch.tensor(0, dtype=torch.float32))
    f = torch.sum(value, dim=1)
    return f * torch.prod(ref - f_min) / n_sample


def hv_estimate(objs: torch.Tensor, ref: torch.Tensor, uniform: torch.Tensor) -> torch.Tensor:
    """hv of metrics/hv.py:13-20 with the draws of its torch.rand (:17) supplied as ``uniform`` (num_sample, m)."""
    points = torch.abs(objs - ref)
    bound = torch.max(points, dim=0).values
    max_vol = torch.prod(bound)
    samples = uniform * bound
    in_hypercube = torch.any(torch.all(samples.unsqueeze(1) < points.unsqueeze(0), dim=2), dim=1)
    return in_hypercube.sum() / uniform.size(0) * max_vol
