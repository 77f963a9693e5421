"""The rebinding helper, against a stand-in package laid out like EvoX's modules (no GPU needed: the
functions are only rebound, not called)."""

import sys
import types

import evox_amd
from evox_amd.operators import selection as hip_selection


def _fake_evox():
    names = [
        "evox", "evox.operators", "evox.operators.selection", "evox.operators.selection.non_dominate",
        "evox.operators.selection.tournament_selection", "evox.algorithms", "evox.algorithms.mo",
        "evox.algorithms.mo.nsga2", "evox.algorithms.mo.nsga3", "evox.algorithms.mo.hype", "evox.algorithms.mo.rveaa",
        "evox.workflows", "evox.workflows.eval_monitor", "evox.metrics", "evox.metrics.hv", "evox.metrics.igd",
    ]
    mods = {n: types.ModuleType(n) for n in names}
    for n, m in mods.items():
        m.__path__ = []  # packages, so that importlib finds the sub-modules in sys.modules
        parent, _, leaf = n.rpartition(".")
        if parent:
            setattr(mods[parent], leaf, m)

    def original(*a, **k):
        raise AssertionError("the original binding is still in place")

    # the early-bound module globals of the reference (nsga2.py:8, nsga3.py:10, hype.py:8-9, rveaa.py:10, eval_monitor.py:12)
    for n in ("evox.operators.selection.non_dominate", "evox.operators.selection"):
        for f in ("non_dominate_rank", "crowding_distance", "nd_environmental_selection"):
            setattr(mods[n], f, original)
    mods["evox.operators.selection.tournament_selection"].tournament_selection_multifit = original
    mods["evox.operators.selection.tournament_selection"].tournament_selection = original
    mods["evox.operators.selection"].tournament_selection_multifit = original
    mods["evox.operators.selection"].tournament_selection = original  # the function shadows the sub-module (__init__.py:14)
    mods["evox.operators"].non_dominate_rank = original
    mods["evox.operators"].crowding_distance = original
    mods["evox.algorithms.mo.nsga2"].nd_environmental_selection = original
    mods["evox.algorithms.mo.nsga2"].tournament_selection_multifit = original
    mods["evox.algorithms.mo.nsga3"].non_dominate_rank = original
    mods["evox.algorithms.mo.hype"].non_dominate_rank = original
    mods["evox.algorithms.mo.hype"].cal_hv = original
    mods["evox.algorithms.mo.rveaa"].non_dominate_rank = original
    mods["evox.workflows.eval_monitor"].non_dominate_rank = original
    mods["evox.workflows.eval_monitor"].unrelated = original
    mods["evox.metrics.hv"].hv = original
    mods["evox.metrics"].hv = original  # the package's `from .hv import hv` shadows the sub-module (metrics/__init__.py:4)
    return mods, original


def test_install_rebinds_every_early_bound_name(monkeypatch):
    mods, original = _fake_evox()
    for n, m in mods.items():
        monkeypatch.setitem(sys.modules, n, m)
    changed = evox_amd.install_into_evox()
    assert mods["evox.algorithms.mo.nsga2"].nd_environmental_selection is hip_selection.nd_environmental_selection
    assert mods["evox.algorithms.mo.nsga2"].tournament_selection_multifit is hip_selection.tournament_selection_multifit
    for n in ("evox.algorithms.mo.nsga3", "evox.algorithms.mo.hype", "evox.algorithms.mo.rveaa", "evox.workflows.eval_monitor",
              "evox.operators", "evox.operators.selection", "evox.operators.selection.non_dominate"):
        assert mods[n].non_dominate_rank is hip_selection.non_dominate_rank, n
    assert mods["evox.operators.selection"].crowding_distance is hip_selection.crowding_distance
    assert mods["evox.algorithms.mo.hype"].cal_hv is evox_amd.hype.cal_hv
    assert mods["evox.operators.selection"].tournament_selection is hip_selection.tournament_selection
    assert mods["evox.workflows.eval_monitor"].unrelated is original  # nothing else is touched
    assert mods["evox.metrics"].hv is evox_amd.metrics.hv and mods["evox.metrics.hv"].hv is evox_amd.metrics.hv
    assert isinstance(mods["evox.metrics"].igd, types.ModuleType)  # sub-modules stay what they are
    assert "evox.algorithms.mo.nsga2.nd_environmental_selection" in changed and len(changed) == 21


def test_install_without_evox_changes_nothing():
    assert "evox" not in sys.modules
    assert evox_amd.install_into_evox() == []
