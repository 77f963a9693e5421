"""Rebinding helper for users who run the real EvoX next to this package.

EvoX's algorithms bind the selection operators as module globals at import time
(src/evox/algorithms/mo/nsga2.py:8, nsga3.py:10, hype.py:8, rveaa.py:10,
src/evox/workflows/eval_monitor.py:12), before its extension loader runs
(src/evox/__init__.py:25-31), so a plugin cannot swap them; this helper rebinds those names.
"""

import importlib

from .hype import cal_hv
from .metrics.hv import hv
from .operators.selection import (
    crowding_distance,
    nd_environmental_selection,
    non_dominate_rank,
    tournament_selection,
    tournament_selection_multifit,
)

_TARGETS = (
    "evox.operators.selection.non_dominate",
    "evox.operators.selection.tournament_selection",
    "evox.operators.selection",
    "evox.operators",
    "evox.algorithms.mo.nsga2",
    "evox.algorithms.mo.nsga3",
    "evox.algorithms.mo.hype",
    "evox.algorithms.mo.rveaa",
    "evox.workflows.eval_monitor",
    "evox.metrics.hv",
    "evox.metrics",
)
_FUNCS = {
    "non_dominate_rank": non_dominate_rank,
    "crowding_distance": crowding_distance,
    "nd_environmental_selection": nd_environmental_selection,
    "tournament_selection_multifit": tournament_selection_multifit,
    "tournament_selection": tournament_selection,
    "cal_hv": cal_hv,  # only evox.algorithms.mo.hype holds this name
    "hv": hv,  # the function that evox.metrics and evox.metrics.hv hold (src/evox/metrics/__init__.py:4), not the module
}


def install_into_evox() -> list:
    """Replaces EvoX's selection operators (and HypE's ``cal_hv``, and the ``hv`` metric), wherever a module
    already holds them, by the HIP-backed ones.  Returns the list of ``module.name`` bindings that were changed."""
    changed = []
    for target in _TARGETS:
        try:
            module = importlib.import_module(target)
        except ImportError:
            continue
        for name, fn in _FUNCS.items():
            if callable(getattr(module, name, None)):
                setattr(module, name, fn)
                changed.append(f"{target}.{name}")
    return changed
