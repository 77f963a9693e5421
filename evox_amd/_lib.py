"""ctypes binding of libevox_hip.so (the C ABI declared in include/evox_hip.h).

There is no fallback: if the library is missing or a call fails, an exception is raised."""

import ctypes
import os
from ctypes import c_float, c_char_p, c_int, c_int64, c_size_t, c_void_p

from .build import LIB_PATH

E_BAD_ARG = -1
E_WORKSPACE = -2
E_BARRIER_TIMEOUT = -3
E_STATIC_LIMIT = -4

_MESSAGES = {
    E_BAD_ARG: "invalid argument",
    E_WORKSPACE: "workspace too small or misaligned",
    E_BARRIER_TIMEOUT: "a device-side wait ran out of polls (grid barrier timeout)",
    E_STATIC_LIMIT: "the population needs more scratch memory than the library's own buffer holds",
}

_SIGNATURES = {
    "evox_hip_abi_version": (c_int, []),
    "evox_hip_workspace_bytes": (c_size_t, [c_int64, c_int64]),
    "evox_hip_non_dominate_rank": (c_int, [c_void_p, c_int64, c_int64, c_int64, c_int64, c_void_p, c_void_p, c_size_t, c_void_p]),
    "evox_hip_non_dominate_rank_until": (c_int, [c_void_p, c_int64, c_int64, c_int64, c_int64, c_int64, c_void_p, c_void_p, c_size_t,
                                                 c_void_p]),
    "evox_hip_first_front_workspace_bytes": (c_size_t, [c_int64, c_int64]),
    "evox_hip_first_front_mask": (c_int, [c_void_p, c_int64, c_int64, c_int64, c_int64, c_void_p, c_void_p, c_size_t, c_void_p]),
    "evox_hip_crowding_distance": (c_int, [c_void_p, c_int64, c_int64, c_int64, c_int64, c_void_p, c_int64, c_void_p, c_void_p,
                                           c_size_t, c_void_p]),
    "evox_hip_wide_workspace_bytes": (c_size_t, [c_int64, c_int64]),
    "evox_hip_crowding_distance_wide": (c_int, [c_void_p, c_int, c_int64, c_int64, c_int64, c_int64, c_void_p, c_int64, c_void_p,
                                                c_int, c_void_p, c_size_t, c_void_p]),
    "evox_hip_many_nd_environmental_selection_wide": (c_int, [c_void_p, c_int64, c_int64, c_int64, c_void_p, c_int64, c_int64, c_int64,
                                                              c_void_p, c_int, c_int64, c_int64, c_int64, c_int64, c_int64, c_int64,
                                                              c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_int,
                                                              c_void_p, c_size_t, c_void_p]),
    "evox_hip_dense_rank_rows": (c_int, [c_void_p, c_int, c_void_p, c_int64, c_int64, c_int64, c_void_p, c_void_p]),
    "evox_hip_nd_environmental_selection_wide": (c_int, [c_void_p, c_int64, c_int64, c_void_p, c_int64, c_int64, c_void_p, c_int,
                                                         c_int64, c_int64, c_int64, c_int64, c_void_p, c_int64, c_void_p, c_void_p,
                                                         c_void_p, c_void_p, c_int, c_void_p, c_size_t, c_void_p]),
    "evox_hip_nd_environmental_selection": (c_int, [c_void_p, c_int64, c_int64, c_void_p, c_int64, c_int64, c_int64, c_int64,
                                                    c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                                    c_size_t, c_void_p]),
    "evox_hip_nd_environmental_selection_two_part": (c_int, [c_void_p, c_int64, c_void_p, c_int64, c_int64, c_void_p, c_int64,
                                                             c_int64, c_int64, c_void_p, c_int64, c_int64, c_int64, c_int64,
                                                             c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                                             c_void_p, c_size_t, c_void_p]),
    "evox_hip_nd_environmental_selection_static": (c_int, [c_void_p, c_int64, c_int64, c_void_p, c_int64, c_int64, c_int64, c_int64,
                                                           c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]),
    "evox_hip_batched_max_rows": (c_int64, [c_int64]),
    "evox_hip_batched_non_dominate_rank": (c_int, [c_void_p, c_int64, c_int64, c_int64, c_int64, c_int64, c_int64, c_void_p,
                                                   c_void_p]),
    "evox_hip_batched_nd_environmental_selection": (c_int, [c_void_p, c_int64, c_int64, c_int64, c_void_p, c_int64, c_int64,
                                                            c_int64, c_int64, c_int64, c_int64, c_int64, c_void_p, c_void_p,
                                                            c_void_p, c_void_p, c_void_p]),
    "evox_hip_many_first_front_workspace_bytes": (c_size_t, [c_int64, c_int64, c_int64]),
    "evox_hip_many_first_front_mask": (c_int, [c_void_p, c_int64, c_int64, c_int64, c_int64, c_int64, c_int64, c_void_p, c_void_p,
                                               c_size_t, c_void_p]),
    "evox_hip_many_crowding_workspace_bytes": (c_size_t, [c_int64, c_int64, c_int64]),
    "evox_hip_many_crowding_distance": (c_int, [c_void_p, c_int64, c_int64, c_int64, c_int64, c_int64, c_int64, c_void_p, c_int64,
                                                c_int64, c_void_p, c_void_p, c_size_t, c_void_p]),
    "evox_hip_many_workspace_bytes": (c_size_t, [c_int64, c_int64, c_int64, c_int64]),
    "evox_hip_many_populations_per_launch": (c_int64, [c_int64, c_int64, c_int64, c_int64]),
    "evox_hip_many_non_dominate_rank_until": (c_int, [c_void_p, c_int64, c_int64, c_int64, c_int64, c_int64, c_int64, c_int64,
                                                      c_void_p, c_void_p, c_size_t, c_void_p]),
    "evox_hip_many_nd_environmental_selection": (c_int, [c_void_p, c_int64, c_int64, c_int64, c_void_p, c_int64, c_int64,
                                                         c_int64, c_int64, c_int64, c_int64, c_int64, c_void_p, c_void_p,
                                                         c_void_p, c_void_p, c_void_p, c_size_t, c_void_p]),
    "evox_hip_tournament_pick_keys": (c_int, [c_void_p, c_int64, c_int64, c_int64, c_int64, c_void_p, c_void_p, c_void_p, c_void_p,
                                              c_void_p]),
    "evox_hip_small_nd_environmental_selection_two_part": (c_int, [c_void_p, c_void_p, c_int64, c_int64, c_void_p, c_int64,
                                                                   c_void_p, c_int64, c_int64, c_int64, c_int64, c_int64,
                                                                   c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]),
    "evox_hip_tournament_pick": (c_int, [c_void_p, c_int64, c_int64, c_void_p, c_int64, c_int64, c_int64, c_int64, c_void_p,
                                         c_void_p]),
    "evox_hip_argsort_workspace_bytes": (c_size_t, [c_int64]),
    "evox_hip_stable_argsort_step": (c_int, [c_void_p, c_int, c_int64, c_int64, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p]),
    "evox_hip_stable_argsort_step_batched": (c_int, [c_void_p, c_int, c_int64, c_int64, c_int64, c_int64, c_void_p, c_void_p,
                                                     c_void_p, c_size_t, c_void_p]),
    "evox_hip_hv_workspace_bytes": (c_size_t, [c_int64, c_int64]),
    "evox_hip_hv_contributions": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_float, c_void_p, c_void_p,
                                          c_size_t, c_void_p]),
    "evox_hip_hv_covered_workspace_bytes": (c_size_t, [c_int64]),
    "evox_hip_hv_covered_count": (c_int, [c_void_p, c_void_p, c_int64, c_int64, c_int64, c_void_p, c_void_p, c_size_t, c_void_p]),
    "evox_hip_calibration_launch": (c_int, [c_int, c_int64, c_int64, c_void_p, c_void_p]),
    "evox_hip_stage_prepare": (c_int, [c_void_p, c_int64, c_int64, c_int64, c_int64, c_void_p, c_size_t, c_void_p]),
    "evox_hip_stage_dominance": (c_int, [c_int64, c_int64, c_int, c_void_p, c_size_t, c_void_p]),
    "evox_hip_stage_count": (c_int, [c_int64, c_int64, c_void_p, c_size_t, c_void_p]),
    "evox_hip_stage_peel": (c_int, [c_int64, c_int64, c_int64, c_void_p, c_void_p, c_size_t, c_void_p]),
    "evox_hip_stage_crowding": (c_int, [c_int64, c_int64, c_void_p, c_size_t, c_void_p]),
    "evox_hip_stage_order": (c_int, [c_int64, c_int64, c_void_p, c_size_t, c_void_p]),
    "evox_hip_workspace_layout": (c_int, [c_int64, c_int64, c_void_p]),
    "evox_hip_slot_sort_layout": (c_int, [c_int64, c_int64, c_void_p]),
    "evox_hip_peel_plan": (c_int, [c_int64, c_int64, c_void_p]),
    "evox_hip_dominance_plan": (c_int, [c_int64, c_int64, c_void_p]),
    "evox_hip_read_status": (c_int, [c_void_p, c_void_p, c_void_p]),
    "evox_hip_set_option": (c_int, [c_char_p, c_int64]),
    "evox_hip_options_create": (c_void_p, []),
    "evox_hip_options_destroy": (None, [c_void_p]),
    "evox_hip_options_set": (c_int, [c_void_p, c_char_p, c_int64]),
    "evox_hip_options_use": (c_int, [c_void_p]),
}

EXPORTED_SYMBOLS = tuple(_SIGNATURES)

_lib = None


class EvoxHipError(RuntimeError):
    def __init__(self, fn: str, code: int):
        what = _MESSAGES.get(code, f"hipError_t {code}" if code > 0 else f"error {code}")
        super().__init__(f"{fn} failed: {what}")
        self.code = code


def lib() -> ctypes.CDLL:
    """The loaded library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python -m evox_amd.build` (needs hipcc). "
                "evox_amd has no CPU or PyTorch fallback."
            )
        handle = ctypes.CDLL(LIB_PATH)
        for name, (restype, argtypes) in _SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = restype
            fn.argtypes = argtypes
        if handle.evox_hip_abi_version() != 1:
            raise RuntimeError("libevox_hip.so has an unexpected ABI version; rebuild it")
        _lib = handle
    return _lib


def call(name: str, *args) -> None:
    code = getattr(lib(), name)(*args)
    if code != 0:
        raise EvoxHipError(name, code)
