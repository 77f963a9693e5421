"""MI355X-native multi-objective environmental selection with EvoX's operator signatures.

    from evox_amd.operators.selection import non_dominate_rank, crowding_distance, nd_environmental_selection

The package holds only this hot path: HIP kernels for gfx950 behind a C ABI (``csrc/``,
``include/evox_hip.h``), the ``evox_amd::`` torch custom operators and the Python functions around them
(``operators.selection``, ``utils.lexsort``).
"""

__all__ = ["hype", "metrics", "operators", "ops", "runtime", "utils", "workloads", "install_into_evox", "uninstall_from_evox"]

from . import hype, metrics, operators, ops, runtime, utils, workloads
from .compat import install_into_evox, uninstall_from_evox
