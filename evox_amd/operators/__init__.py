__all__ = ["selection", "crowding_distance", "non_dominate_rank"]

from . import selection
from .selection import crowding_distance, non_dominate_rank
