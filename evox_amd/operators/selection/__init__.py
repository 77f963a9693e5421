__all__ = ["crowding_distance", "nd_environmental_selection", "non_dominate_rank", "tournament_selection_multifit"]

from .non_dominate import crowding_distance, nd_environmental_selection, non_dominate_rank
from .tournament_selection import tournament_selection_multifit
