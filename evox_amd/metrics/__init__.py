__all__ = ["hv"]

from .hv import hv
