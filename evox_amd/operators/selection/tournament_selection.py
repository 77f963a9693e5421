"""Drop-in replacements for ``evox.operators.selection.tournament_selection_multifit``
(src/evox/operators/selection/tournament_selection.py:8-29), the consumer of the rank and crowding
distance that ``nd_environmental_selection`` returns (src/evox/algorithms/mo/nsga2.py:94), and for its
single-fitness sibling ``tournament_selection`` (tournament_selection.py:32-54).
"""

from typing import List

import torch

from ... import ops


def tournament_selection_multifit(n_round: int, fitnesses: List[torch.Tensor], tournament_size: int = 2) -> torch.Tensor:
    """Indices of the winners of ``n_round`` random tournaments of ``tournament_size`` candidates.

    Same contract as the reference: candidates are drawn with ``torch.randint`` on the fitness
    device (so a seeded generator gives the same tournaments as the reference), and each tournament
    is won by the candidate that sorts first by the LAST tensor of ``fitnesses``, ties by the one
    before it, ..., ties by position in the tournament (NaN last).  The result is squeezed, as there.
    """
    if ops.tournament_keys_fit(fitnesses):
        # float32 and int32 vectors -- the crowding distances and ranks that NSGA-II passes: read where they lie
        # (the stacked copy with its type promotion is two or three more launches than the tournaments themselves)
        parents = torch.randint(0, fitnesses[0].size(0), (n_round, tournament_size), device=fitnesses[0].device)
        pick = ops.tournament_pick_keys_direct if ops.plain_eager() else ops.tournament_pick_keys
        return pick(parents, list(fitnesses)).squeeze()
    fitness_tensor = torch.stack(fitnesses, dim=1)
    num_candidates = fitness_tensor.size(0)
    parents = torch.randint(0, num_candidates, (n_round, tournament_size), device=fitnesses[0].device)
    return ops.tournament_pick(parents, fitness_tensor).squeeze()


def tournament_selection(n_round: int, fitness: torch.Tensor, tournament_size: int = 2) -> torch.Tensor:
    """Indices of the winners of ``n_round`` random tournaments on one fitness tensor: the candidate of
    least fitness, the first of them on ties, and -- as ``torch.argmin`` has it (tournament_selection.py:50) --
    a NaN before every number.  Candidates are drawn as the reference draws them (:47)."""
    num_candidates = fitness.size(0)
    parents = torch.randint(0, num_candidates, (n_round, tournament_size), device=fitness.device)
    # the kernel orders by the last column first and puts NaN last: "is a number" as the last column puts NaN first
    keys = torch.stack([fitness, (~torch.isnan(fitness)).to(fitness.dtype)], dim=1)
    return ops.tournament_pick(parents, keys).squeeze()
