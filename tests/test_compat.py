"""The rebinding helper (no GPU needed: on CPU tensors the installed dispatchers hand every call back to the
binding they found).

Two sources: a stand-in package laid out like EvoX's modules, and `golden/evox_bindings.json`, which
`golden/make_binding_fixture.py` wrote by running the helper against the imported reference in the build container
(which modules hold the functions, what the helper changed there, and that the package's own CPU callers --
`EvalMonitor.get_pf_fitness` / `get_pf` on the default CPU history, an NSGA-II workflow -- give the same results
after the install)."""

import json
import os
import sys
import types

import pytest
import torch

import evox_amd
from evox_amd import compat

FIXTURE = json.load(open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "evox_bindings.json")))


def _fake_evox():
    """Modules and module globals as the reference holds them (the `holders` of the fixture)."""
    mods = {}

    def module(name):
        if name not in mods:
            mods[name] = types.ModuleType(name)
            mods[name].__path__ = []  # a package, so that importlib finds sub-modules in sys.modules
            parent, _, leaf = name.rpartition(".")
            if parent:
                setattr(module(parent), leaf, mods[name])
        return mods[name]

    originals = {}

    def original_for(name):
        if name not in originals:
            def original(*args, **kwargs):
                return ("original", name)
            originals[name] = original
        return originals[name]

    # sub-modules first: on two packages a function shadows the sub-module of the same name
    # (operators/selection/__init__.py:14, metrics/__init__.py:4)
    for leaf in ("evox.operators.selection.non_dominate", "evox.operators.selection.tournament_selection", "evox.metrics.hv",
                 "evox.metrics.igd", "evox.utils.jit_fix_operator", "evox.algorithms.mo.nsga2", "evox.algorithms.mo.nsga3", "evox.algorithms.mo.hype",
                 "evox.algorithms.mo.rveaa", "evox.workflows.eval_monitor"):
        module(leaf)
    for holder in FIXTURE["holders"]:
        mod_name, _, name = holder.rpartition(".")
        if mod_name not in mods:  # "evox.metrics.hv.hv": the module evox.metrics.hv
            module(mod_name)
        setattr(mods[mod_name], name, original_for(name))
    mods["evox.workflows.eval_monitor"].unrelated = original_for("unrelated")
    return mods, originals


@pytest.fixture
def fake_evox(monkeypatch):
    mods, originals = _fake_evox()
    for n, m in mods.items():
        monkeypatch.setitem(sys.modules, n, m)
    yield mods, originals
    compat.uninstall_from_evox()


def test_targets_cover_every_module_that_holds_the_functions_in_the_real_package():
    reachable = {f"{target}.{name}" for target in compat._TARGETS for name in compat._FUNCS}
    assert set(FIXTURE["holders"]) <= reachable
    # run against the imported reference, the helper changed exactly those bindings, once
    assert sorted(FIXTURE["changed_by_install"]) == sorted(FIXTURE["holders"]) and len(FIXTURE["holders"]) == 28
    assert FIXTURE["changed_by_second_install"] == []
    assert FIXTURE["cpu_workflow_and_monitor_unchanged_after_install"] is True
    assert FIXTURE["cpu_workflow_and_monitor_unchanged_after_patch_callers"] is True
    assert sorted(FIXTURE["holders_after_uninstall"]) == sorted(FIXTURE["holders"])
    assert len(FIXTURE["changed_by_patch_callers"]) == 5


def test_install_routes_every_early_bound_name_and_keeps_what_it_found(fake_evox):
    mods, originals = fake_evox
    changed = evox_amd.install_into_evox()
    assert sorted(changed) == sorted(FIXTURE["holders"])
    cpu = torch.rand(6, 3)
    for holder in FIXTURE["holders"]:
        mod_name, _, name = holder.rpartition(".")
        bound = getattr(mods[mod_name], name)
        assert bound is not originals[name] and bound.__evox_amd_original__ is originals[name], holder
        assert bound.__name__ == name
        # a CPU tensor (bare, in a list, or by keyword) still reaches the function that was bound there
        assert bound(cpu) == ("original", name) and bound(4, [cpu, cpu]) == ("original", name)
        assert bound(x=cpu) == ("original", name)
    # one dispatcher per original, wherever it is bound
    assert mods["evox.algorithms.mo.nsga3"].non_dominate_rank is mods["evox.operators.selection"].non_dominate_rank
    assert mods["evox.workflows.eval_monitor"].unrelated is originals["unrelated"]  # nothing else is touched
    assert isinstance(mods["evox.metrics"].igd, types.ModuleType)  # sub-modules stay what they are
    assert evox_amd.install_into_evox() == []  # nothing is wrapped twice
    assert sorted(compat.uninstall_from_evox()) == sorted(FIXTURE["holders"])
    for holder in FIXTURE["holders"]:
        mod_name, _, name = holder.rpartition(".")
        assert getattr(mods[mod_name], name) is originals[name]


def test_gpu_tensors_would_go_to_the_hip_functions(fake_evox, monkeypatch):
    mods, _ = fake_evox
    evox_amd.install_into_evox()
    monkeypatch.setattr(compat, "_on_gpu", lambda args, kwargs: True)
    with pytest.raises(RuntimeError, match="AMD GPU only"):  # the HIP function itself: it refuses the CPU tensor
        mods["evox.algorithms.mo.nsga3"].non_dominate_rank(torch.rand(5, 2))


class _Algo:
    """The attribute protocol of the reference's NSGA2 / NSGA3 / HypE as far as the patched steps use it."""

    def __init__(self):
        self.pop_size = 4
        self.pop = torch.rand(4, 2)
        self.calls = []

    def step(self):
        self.calls.append(("original step", compat._rank_until))
        return "stepped"


def test_patch_callers_on_cpu_populations_runs_the_original_methods(fake_evox):
    mods, _ = fake_evox

    class NSGA2(_Algo):
        pass

    class NSGA3(_Algo):
        pass

    class HypE(_Algo):
        pass

    class EvalMonitor:
        multi_obj = True
        fitness_history = [torch.rand(3, 2)]

        def get_pf_fitness(self, deduplicate=True):
            return "original pf fitness"

        def get_pf(self, deduplicate=True):
            return "original pf"

    for cls in (NSGA2, NSGA3, HypE, EvalMonitor):
        cls.__module__ = {"NSGA2": "evox.algorithms.mo.nsga2", "NSGA3": "evox.algorithms.mo.nsga3",
                          "HypE": "evox.algorithms.mo.hype", "EvalMonitor": "evox.workflows.eval_monitor"}[cls.__name__]
        setattr(mods[cls.__module__], cls.__name__, cls)
    changed = evox_amd.install_into_evox(patch_callers=True)
    assert changed[-5:] == FIXTURE["changed_by_patch_callers"]
    a2, a3, hy, mon = NSGA2(), NSGA3(), HypE(), EvalMonitor()
    assert a2.step() == "stepped" and a2.calls == [("original step", None)]  # a CPU population: the reference's own step
    assert a3.step() == "stepped" and a3.calls == [("original step", 5)]  # topk(rank, pop_size + 1), nsga3.py:170
    assert hy.step() == "stepped" and hy.calls == [("original step", 4)]  # rank[order[pop_size - 1]], hype.py:137
    assert compat._rank_until is None
    assert mon.get_pf_fitness() == "original pf fitness" and mon.get_pf(False) == "original pf"  # CPU history
    assert evox_amd.install_into_evox(patch_callers=True) == []
    compat.uninstall_from_evox()
    assert NSGA3().step.__func__ is _Algo.step and "__evox_amd_original__" not in vars(EvalMonitor.get_pf)


def test_install_without_evox_changes_nothing():
    assert "evox" not in sys.modules
    assert evox_amd.install_into_evox(patch_callers=True) == []
