"""CPU-side checks of the C ABI: the library builds, loads and exports every symbol that
include/evox_hip.h declares; argument validation works without a GPU."""

import ctypes
import os
import re

import pytest

from evox_amd import _lib
from evox_amd.build import LIB_PATH, build_library

HEADER = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "include", "evox_hip.h")


@pytest.fixture(scope="module")
def handle():
    if not os.path.exists(LIB_PATH):
        build_library()
    return _lib.lib()


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(evox_hip_\w+)\s*\(", text)))


def test_header_and_binding_agree():
    assert declared_symbols() == sorted(_lib.EXPORTED_SYMBOLS)


def test_every_declared_symbol_is_exported(handle):
    raw = ctypes.CDLL(LIB_PATH)
    for name in declared_symbols():
        assert hasattr(raw, name), name
    assert handle.evox_hip_abi_version() == 1


def test_workspace_size_and_layout(handle):
    assert handle.evox_hip_workspace_bytes(0, 3) == 0
    assert handle.evox_hip_workspace_bytes(10, 0) == 0
    b = handle.evox_hip_workspace_bytes(20000, 3)
    # dominated by the bit matrix: 20000 rows x 320 words (313 rounded up to a 128-byte multiple)
    # (plus the state arrays, the buffers of the last front's sorts and those of the stepped path's ordering)
    assert 20000 * 320 * 8 <= b <= 20000 * 320 * 8 + 12 * 2**20
    b5 = handle.evox_hip_workspace_bytes(200000, 8)
    assert 5.0e9 < b5 < 5.3e9
    # the first-front entry builds no matrix: a few arrays of n entries
    assert handle.evox_hip_first_front_workspace_bytes(0, 3) == 0
    assert 0 < handle.evox_hip_first_front_workspace_bytes(20000, 3) < 8 * 2**20
    # (behind the matrix lie the buffers of the stepped path's ordering of the last front: a few arrays of n * m entries)
    assert 0 < b5 - 200000 * 3136 * 8 - handle.evox_hip_first_front_workspace_bytes(200000, 8) < 64 * 2**20
    out = (ctypes.c_int64 * 11)()
    assert handle.evox_hip_workspace_layout(20000, 3, out) == 0
    assert out[1] == 320 and out[2] == 314 and out[0] % 256 == 0 and out[9] == 0


def test_argument_validation_without_gpu(handle):
    # null / misaligned / short workspaces and bad sizes are rejected before anything is launched
    assert handle.evox_hip_non_dominate_rank(None, 10, 3, 3, 1, None, None, 0, None) == _lib.E_BAD_ARG
    buf = ctypes.create_string_buffer(64)
    p = ctypes.addressof(buf)
    assert handle.evox_hip_non_dominate_rank(p, 10, 3, 3, 1, p, None, 0, None) == _lib.E_WORKSPACE
    assert handle.evox_hip_non_dominate_rank(p, 10, 3, 3, 1, p, p, 64, None) == _lib.E_WORKSPACE
    assert handle.evox_hip_non_dominate_rank(p, 0, 3, 3, 1, p, p, 64, None) == _lib.E_BAD_ARG
    assert handle.evox_hip_nd_environmental_selection(None, 0, 0, p, 10, 3, 3, 1, 11, None, p, p, p, None, p, 64, None) == _lib.E_BAD_ARG
    assert handle.evox_hip_non_dominate_rank_until(p, 10, 3, 3, 1, 11, p, p, 64, None) == _lib.E_BAD_ARG
    assert handle.evox_hip_non_dominate_rank_until(p, 10, 3, 3, 1, 0, p, p, 64, None) == _lib.E_BAD_ARG
    assert handle.evox_hip_non_dominate_rank_until(p, 10, 3, 3, 1, 5, p, p, 64, None) == _lib.E_WORKSPACE
    assert handle.evox_hip_argsort_workspace_bytes(0) == 0 and handle.evox_hip_argsort_workspace_bytes(1000) > 16000
    assert handle.evox_hip_stable_argsort_step(p, 3, 1, 10, None, p, p, 64, None) == _lib.E_BAD_ARG
    assert handle.evox_hip_stable_argsort_step(p, 0, 1, 10, None, p, p, 64, None) == _lib.E_WORKSPACE
    assert handle.evox_hip_stable_argsort_step_batched(p, 0, 10, 1, 0, 10, None, p, p, 1 << 20, None) == _lib.E_BAD_ARG
    assert handle.evox_hip_stable_argsort_step_batched(p, 0, 10, 1, 4, 10, None, p, p, 64, None) == _lib.E_WORKSPACE
    assert handle.evox_hip_hv_workspace_bytes(0, 10) == 0 and handle.evox_hip_hv_workspace_bytes(100, 5000) >= 4 * (5000 + 5 * 100)
    assert handle.evox_hip_hv_contributions(p, p, p, 10, 0, 100, 1.0, p, p, 64, None) == _lib.E_BAD_ARG
    assert handle.evox_hip_hv_contributions(p, p, p, 10, 3, 100, 1.0, p, p, 64, None) == _lib.E_WORKSPACE
    assert handle.evox_hip_hv_covered_workspace_bytes(0) == 0 and handle.evox_hip_hv_covered_workspace_bytes(100000) >= 4 * 391
    assert handle.evox_hip_hv_covered_count(p, p, 10, 0, 100, p, p, 1 << 20, None) == _lib.E_BAD_ARG
    assert handle.evox_hip_hv_covered_count(p, p, 10, 3, 100000, p, p, 64, None) == _lib.E_WORKSPACE
    assert handle.evox_hip_first_front_mask(p, 10, 3, 3, 1, None, p, 64, None) == _lib.E_BAD_ARG
    assert handle.evox_hip_first_front_mask(p, 10, 3, 3, 1, p, p, 64, None) == _lib.E_WORKSPACE
    assert handle.evox_hip_tournament_pick(None, 4, 2, p, 10, 2, 2, 1, p, None) == _lib.E_BAD_ARG
    assert handle.evox_hip_tournament_pick(p, 4, 0, p, 10, 2, 2, 1, p, None) == _lib.E_BAD_ARG
    assert handle.evox_hip_nd_environmental_selection_two_part(None, 0, None, 0, 0, p, 5, 3, 1, p, 5, 3, 1, 3, 11, None, p, p, p,
                                                               None, p, 64, None) == _lib.E_BAD_ARG  # topk > n_a + n_b
    assert handle.evox_hip_nd_environmental_selection_two_part(None, 0, None, 0, 0, p, 5, 3, 1, None, 5, 3, 1, 3, 4, None, p, p,
                                                               p, None, p, 64, None) == _lib.E_BAD_ARG  # missing part
    assert handle.evox_hip_nd_environmental_selection_two_part(None, 0, None, 0, 0, p, 5, 3, 1, p, 5, 3, 1, 3, 4, None, p, p, p,
                                                               None, p, 64, None) == _lib.E_WORKSPACE
    three = (ctypes.c_void_p * 3)(p, p, None)
    kinds = (ctypes.c_int32 * 3)(0, 1, 0)
    strides = (ctypes.c_int64 * 3)(1, 1, 1)
    by_keys = handle.evox_hip_tournament_pick_keys
    assert by_keys(p, 4, 2, 10, 5, ctypes.addressof(three), ctypes.addressof(kinds), ctypes.addressof(strides), p, None) == _lib.E_BAD_ARG  # five keys
    assert by_keys(p, 4, 2, 10, 3, ctypes.addressof(three), ctypes.addressof(kinds), ctypes.addressof(strides), p, None) == _lib.E_BAD_ARG  # a null key
    kinds[1] = 7
    assert by_keys(p, 4, 2, 10, 2, ctypes.addressof(three), ctypes.addressof(kinds), ctypes.addressof(strides), p, None) == _lib.E_BAD_ARG  # unknown kind
    assert by_keys(p, 4, 0, 10, 1, ctypes.addressof(three), ctypes.addressof(kinds), ctypes.addressof(strides), p, None) == _lib.E_BAD_ARG
    small = handle.evox_hip_small_nd_environmental_selection_two_part
    assert small(None, None, 0, 0, p, 5, p, 5, 3, 3, 1, 11, None, p, p, p, None) == _lib.E_BAD_ARG  # topk > n_a + n_b
    assert small(None, None, 0, 0, p, 5, None, 5, 3, 3, 1, 4, None, p, p, p, None) == _lib.E_BAD_ARG  # missing part
    assert small(None, None, 0, 0, p, 5, p, 0, 3, 3, 1, 4, None, p, p, p, None) == _lib.E_BAD_ARG  # a part without rows
    assert small(None, None, 0, 0, p, 1000, p, 25, 3, 3, 1, 4, None, p, p, p, None) == _lib.E_BAD_ARG  # more than 1024 rows
    assert handle.evox_hip_set_option(b"no_such_option", 1) == _lib.E_BAD_ARG
    assert handle.evox_hip_set_option(b"launch_memory", 1) == 0
    assert handle.evox_hip_set_option(b"peel_blocks_per_cu", 2) == 0
    # tunables for the calls of one thread: created from the process-wide ones, set by name, handed over and taken back
    opts = handle.evox_hip_options_create()
    assert opts
    assert handle.evox_hip_options_set(opts, b"spin_limit", 5) == 0
    assert handle.evox_hip_options_set(opts, b"spin_limit", 0) == _lib.E_BAD_ARG
    assert handle.evox_hip_options_set(opts, b"no_such_option", 1) == _lib.E_BAD_ARG
    assert handle.evox_hip_options_set(None, b"spin_limit", 5) == _lib.E_BAD_ARG
    assert handle.evox_hip_options_use(opts) == 0 and handle.evox_hip_options_use(None) == 0
    assert handle.evox_hip_options_use(opts) == 0
    handle.evox_hip_options_destroy(opts)  # (the set in use: the thread falls back to the process-wide tunables)
    handle.evox_hip_options_destroy(None)


def test_scoped_options_nest_and_restore():
    from evox_amd import runtime

    with runtime.options(spin_limit=7):
        with runtime.options(peel_witness=0):
            assert [d for _, d in runtime._options_in_use.stack] == [{"spin_limit": 7}, {"spin_limit": 7, "peel_witness": 0}]
        assert len(runtime._options_in_use.stack) == 1
        with pytest.raises(_lib.EvoxHipError):
            with runtime.options(no_such_option=1):
                pass
        assert len(runtime._options_in_use.stack) == 1
    assert runtime._options_in_use.stack == []
