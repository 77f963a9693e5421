"""Rebinding helper for users who run the real EvoX next to this package.

EvoX's algorithms bind the selection operators as module globals at import time
(src/evox/algorithms/mo/nsga2.py:8, nsga3.py:10, hype.py:8, rveaa.py:10,
src/evox/workflows/eval_monitor.py:12), before its extension loader runs
(src/evox/__init__.py:25-31), so a plugin cannot swap them; this helper rebinds those names.

What it installs is not the HIP function itself but a dispatcher that keeps the binding it found: tensors on the
GPU go to the HIP kernels, everything else goes to EvoX's own function as before.  EvoX calls these operators on
CPU tensors too -- ``EvalMonitor`` keeps its history on the CPU unless told otherwise
(src/evox/workflows/eval_monitor.py:124) and ranks it in ``get_pf_fitness`` / ``get_pf`` (:301, :333) -- and this
package has no CPU path of its own.

``install_into_evox(patch_callers=True)`` also changes the four callers that can do less work than a rebound name
allows them to: NSGA-II's merge (nsga2.py:99-102) hands parents and offspring to the selection as they lie,
NSGA-III and HypE (nsga3.py:169-171, hype.py:135-138) rank their merged population only as far as the front they cut
it at, and ``EvalMonitor.get_pf_fitness`` / ``get_pf`` take the first front of a history on the GPU without ranking
the rest.
"""

import contextlib
import functools
import importlib

import torch

from .hype import cal_hv
from .metrics.hv import hv
from .utils import lexsort
from .operators.selection import (
    crowding_distance,
    nd_environmental_selection,
    nd_environmental_selection_two_part,
    non_dominate_rank,
    non_dominate_rank_until,
    non_dominated_mask,
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
    "evox.utils.jit_fix_operator",
    "evox.utils",
)
_FUNCS = {
    "non_dominate_rank": non_dominate_rank,
    "crowding_distance": crowding_distance,
    "nd_environmental_selection": nd_environmental_selection,
    "tournament_selection_multifit": tournament_selection_multifit,
    "tournament_selection": tournament_selection,
    "cal_hv": cal_hv,  # only evox.algorithms.mo.hype holds this name
    "hv": hv,  # the function that evox.metrics and evox.metrics.hv hold (src/evox/metrics/__init__.py:4), not the module
    # src/evox/utils/jit_fix_operator.py:213-252, held by HypE (hype.py:9, used at :143) and the two selection modules
    "lexsort": lexsort,
}

_installed = {}  # "module.name" -> the binding that was found there
_patched = []  # (class, attribute, original) of the callers changed by patch_callers
_dispatchers = {}  # (name, id(original)) -> dispatcher, so that one original gets one dispatcher wherever it is bound
_rank_until = None  # stop count for the ranking inside a patched NSGA-III / HypE step (a plain global: the steps of
                    # one process run one at a time, and a compiled step reads it while it is traced)


def _first_tensor(values):
    for v in values:
        if isinstance(v, torch.Tensor):
            return v
        if isinstance(v, (list, tuple)):
            t = _first_tensor(v)
            if t is not None:
                return t
    return None


def _on_gpu(args, kwargs) -> bool:
    t = _first_tensor(list(args) + list(kwargs.values()))
    return t is not None and t.is_cuda


def _dispatcher(name, hip_fn, original):
    key = (name, id(original))
    found = _dispatchers.get(key)
    if found is not None:
        return found

    @functools.wraps(hip_fn)
    def dispatch(*args, **kwargs):
        if _on_gpu(args, kwargs):
            if name == "non_dominate_rank" and _rank_until is not None:
                return non_dominate_rank_until(args[0], min(_rank_until, args[0].shape[-2]))
            return hip_fn(*args, **kwargs)
        return original(*args, **kwargs)

    dispatch.__evox_amd_original__ = original
    _dispatchers[key] = dispatch
    return dispatch


@contextlib.contextmanager
def _rank_only_until(count: int):
    global _rank_until
    before = _rank_until
    _rank_until = int(count)
    try:
        yield
    finally:
        _rank_until = before


def _patch(cls, attribute, make):
    original = getattr(cls, attribute)
    if getattr(original, "__evox_amd_original__", None) is not None:
        return None
    replacement = make(original)
    replacement.__evox_amd_original__ = original
    setattr(cls, attribute, replacement)
    _patched.append((cls, attribute, original))
    return f"{cls.__module__}.{cls.__name__}.{attribute}"


def _nsga2_step(module):
    """NSGA2.step (nsga2.py:92-102) with the merge left out: parents and offspring go to the selection in two
    parts.  Everything before the merge is the reference's sequence of calls, through the names its module holds."""

    def make(original):
        @functools.wraps(original)
        def step(self):
            if not self.pop.is_cuda:
                return original(self)
            mating_pool = self.selection(self.pop_size, [-self.dis, self.rank])
            crossovered = self.crossover(self.pop[mating_pool])
            offspring = self.mutation(crossovered, self.lb, self.ub)
            offspring = module.clamp(offspring, self.lb, self.ub)
            off_fit = self.evaluate(offspring)
            self.pop, self.fit, self.rank, self.dis = nd_environmental_selection_two_part(
                self.pop, self.fit, offspring, off_fit, self.pop_size
            )

        return step

    return make


def _step_with_rank_cut(extra: int):
    """A step whose one ranking of the merged population stops at the front that holds row pop_size + extra: the
    rows behind it get the largest int32, under which `topk(rank, k, largest=False)[0][-1]`, `rank <= worst`
    (nsga3.py:170-171) and `rank[argsort(rank)[k - 1]]` (hype.py:136-137) read what they read from full ranks."""

    def make(original):
        @functools.wraps(original)
        def step(self):
            with _rank_only_until(self.pop_size + extra):
                return original(self)

        return step

    return make


def _monitor_front(module, with_solutions: bool):
    """EvalMonitor.get_pf_fitness / get_pf (eval_monitor.py:290-303, :314-337) for a history kept on the GPU: the
    rows of rank 0 from the first-front kernel instead of a ranking of the whole history."""

    def make(original):
        @functools.wraps(original)
        def get(self, deduplicate=True):
            history = self.fitness_history
            if not self.multi_obj or len(history) == 0 or not history[0].is_cuda:
                return original(self, deduplicate)
            all_fitness = torch.cat(history, dim=0)
            opt_dir = self.opt_direction.to(self.history_device)
            if not with_solutions:
                if deduplicate:
                    all_fitness = torch.unique(all_fitness, dim=0)
                return all_fitness[non_dominated_mask(all_fitness)] * opt_dir
            all_solutions = torch.cat(self.get_solution_history(), dim=0)
            if deduplicate:
                _, unique_index, _, _ = module.unique(all_solutions)
                all_solutions = all_solutions[unique_index]
                all_fitness = all_fitness[unique_index]
            front = non_dominated_mask(all_fitness)
            return all_solutions[front], all_fitness[front] * opt_dir

        return get

    return make


def _patch_callers() -> list:
    changed = []

    def module_of(name):
        try:
            return importlib.import_module(name)
        except ImportError:
            return None

    nsga2 = module_of("evox.algorithms.mo.nsga2")
    if nsga2 is not None and hasattr(nsga2, "NSGA2"):
        changed.append(_patch(nsga2.NSGA2, "step", _nsga2_step(nsga2)))
    nsga3 = module_of("evox.algorithms.mo.nsga3")
    if nsga3 is not None and hasattr(nsga3, "NSGA3"):
        changed.append(_patch(nsga3.NSGA3, "step", _step_with_rank_cut(1)))  # topk(rank, pop_size + 1), nsga3.py:170
    hype = module_of("evox.algorithms.mo.hype")
    if hype is not None and hasattr(hype, "HypE"):
        changed.append(_patch(hype.HypE, "step", _step_with_rank_cut(0)))  # rank[order[pop_size - 1]], hype.py:137
    monitor = module_of("evox.workflows.eval_monitor")
    if monitor is not None and hasattr(monitor, "EvalMonitor"):
        changed.append(_patch(monitor.EvalMonitor, "get_pf_fitness", _monitor_front(monitor, False)))
        changed.append(_patch(monitor.EvalMonitor, "get_pf", _monitor_front(monitor, True)))
    return [c for c in changed if c is not None]


def install_into_evox(patch_callers: bool = False) -> list:
    """Routes EvoX's selection operators (and ``lexsort``, HypE's ``cal_hv`` and the ``hv`` metric), wherever a module already
    holds them, to the HIP-backed ones for tensors on the GPU; tensors elsewhere keep going to the function that
    was bound there.  With ``patch_callers`` the four callers named in the module docstring are changed as well.
    Returns the list of ``module.name`` bindings (and ``module.Class.method`` callers) that were changed; a second
    call changes nothing more."""
    changed = []
    for target in _TARGETS:
        try:
            module = importlib.import_module(target)
        except ImportError:
            continue
        for name, fn in _FUNCS.items():
            found = getattr(module, name, None)
            if not callable(found) or getattr(found, "__evox_amd_original__", None) is not None:
                continue
            setattr(module, name, _dispatcher(name, fn, found))
            _installed[f"{target}.{name}"] = found
            changed.append(f"{target}.{name}")
    if patch_callers:
        changed.extend(_patch_callers())
    return changed


def uninstall_from_evox() -> list:
    """Puts back every binding and method that ``install_into_evox`` changed; returns their names."""
    restored = []
    for qualified, original in list(_installed.items()):
        target, _, name = qualified.rpartition(".")
        try:
            setattr(importlib.import_module(target), name, original)
            restored.append(qualified)
        except ImportError:
            pass
        del _installed[qualified]
    while _patched:
        cls, attribute, original = _patched.pop()
        setattr(cls, attribute, original)
        restored.append(f"{cls.__module__}.{cls.__name__}.{attribute}")
    _dispatchers.clear()
    return restored
