__all__ = [
    "crowding_distance",
    "nd_environmental_selection",
    "nd_environmental_selection_two_part",
    "non_dominate_rank",
    "non_dominate_rank_until",
    "non_dominated_mask",
    "tournament_selection",
    "tournament_selection_multifit",
]

from .non_dominate import (
    crowding_distance,
    nd_environmental_selection,
    nd_environmental_selection_two_part,
    non_dominate_rank,
    non_dominate_rank_until,
    non_dominated_mask,
)
from .tournament_selection import tournament_selection, tournament_selection_multifit
