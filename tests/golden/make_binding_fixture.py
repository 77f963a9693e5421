"""Writes tests/golden/evox_bindings.json by importing the reference itself, once, in the build container:

    PYTHONPATH=/root/reference/src python tests/golden/make_binding_fixture.py

What is stored is data only: which modules of the imported package hold, as module globals, the functions that
`evox_amd.compat.install_into_evox` routes to the HIP kernels (the early-bound names that a plugin cannot reach),
what the helper reports when it is run against the real package, and whether the package's own callers still work on
CPU tensors afterwards (`EvalMonitor.get_pf_fitness` / `get_pf` on its default CPU history, an NSGA-II workflow).
`tests/test_compat.py` checks the helper's target list against this file; nothing of the reference travels."""

import json
import os
import sys

import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)

import evox  # noqa: E402
from evox.algorithms import NSGA2  # noqa: E402
from evox.problems.numerical import DTLZ2  # noqa: E402
from evox.workflows import EvalMonitor, StdWorkflow  # noqa: E402

import evox_amd  # noqa: E402
from evox_amd import compat  # noqa: E402

NAMES = ("non_dominate_rank", "crowding_distance", "nd_environmental_selection", "tournament_selection_multifit",
         "tournament_selection", "cal_hv", "hv", "lexsort")


def holders():
    """module.name for every loaded evox module that holds one of the functions as a module global."""
    import importlib

    # (through sys.modules: on the packages, the functions `hv` and `tournament_selection` shadow their sub-modules)
    hype_module = importlib.import_module("evox.algorithms.mo.hype")
    hv_module = importlib.import_module("evox.metrics.hv")
    nd_module = importlib.import_module("evox.operators.selection.non_dominate")
    ts_module = importlib.import_module("evox.operators.selection.tournament_selection")

    canonical = {
        "non_dominate_rank": nd_module.non_dominate_rank,
        "crowding_distance": nd_module.crowding_distance,
        "nd_environmental_selection": nd_module.nd_environmental_selection,
        "tournament_selection_multifit": ts_module.tournament_selection_multifit,
        "tournament_selection": ts_module.tournament_selection,
        "cal_hv": hype_module.cal_hv,
        "hv": hv_module.hv,
        "lexsort": importlib.import_module("evox.utils.jit_fix_operator").lexsort,
    }
    found = []
    for mod_name, module in sorted(sys.modules.items()):
        if module is None or not (mod_name == "evox" or mod_name.startswith("evox.")):
            continue
        for name, fn in canonical.items():
            if getattr(module, name, None) is fn:
                found.append(f"{mod_name}.{name}")
    return found


def run_workflow(seed: int):
    torch.manual_seed(seed)
    monitor = EvalMonitor(multi_obj=True, full_fit_history=True, full_sol_history=True)
    algo = NSGA2(pop_size=20, n_objs=3, lb=-torch.ones(10), ub=torch.ones(10))
    workflow = StdWorkflow(algo, DTLZ2(m=3), monitor)
    workflow.init_step()
    for _ in range(3):
        workflow.step()
    sols, fit = monitor.get_pf()
    return monitor.get_pf_fitness(), sols, fit


def main():
    torch.set_default_device("cpu")
    out = {"evox_version": getattr(evox, "__version__", "unknown"), "torch": torch.__version__}
    out["holders"] = holders()
    before = run_workflow(7)
    out["changed_by_install"] = evox_amd.install_into_evox()
    out["changed_by_second_install"] = evox_amd.install_into_evox()
    after = run_workflow(7)
    out["cpu_workflow_and_monitor_unchanged_after_install"] = all(torch.equal(a, b) for a, b in zip(before, after))
    out["changed_by_patch_callers"] = evox_amd.install_into_evox(patch_callers=True)
    patched = run_workflow(7)
    out["cpu_workflow_and_monitor_unchanged_after_patch_callers"] = all(torch.equal(a, b) for a, b in zip(before, patched))
    out["restored_by_uninstall"] = sorted(compat.uninstall_from_evox())
    out["holders_after_uninstall"] = holders()
    with open(os.path.join(HERE, "evox_bindings.json"), "w") as fh:
        json.dump(out, fh, indent=1, sort_keys=True)
        fh.write("\n")
    print(json.dumps(out, indent=1, sort_keys=True))


if __name__ == "__main__":
    main()
