__all__ = ["crowding_distance", "nd_environmental_selection", "non_dominate_rank"]

from .non_dominate import crowding_distance, nd_environmental_selection, non_dominate_rank
