"""What the compiler made of the kernels, read from the metadata of the built library (the gfx950 code object inside
libevox_hip.so; no GPU needed): every kernel is wave64, none uses accumulation registers (no kernel here has matrix
instructions, so a count above zero would mean vector registers spilled into them), and the kernel that ranks two
objectives by a chain of workgroups, whose rounds are bound by instruction issue, spills nothing.
"""

import os
import struct

import msgpack
import pytest

from evox_amd.build import LIB_PATH, build_library

MAGIC = b"__CLANG_OFFLOAD_BUNDLE__"


def _gfx950_code_object(blob: bytes) -> bytes:
    start = blob.find(MAGIC)
    assert start >= 0, "no offload bundle in the library"
    (entries,) = struct.unpack_from("<Q", blob, start + len(MAGIC))
    at = start + len(MAGIC) + 8
    for _ in range(entries):
        offset, size, triple_size = struct.unpack_from("<QQQ", blob, at)
        at += 24
        triple = blob[at:at + triple_size].decode()
        at += triple_size
        if "gfx950" in triple:
            return blob[start + offset:start + offset + size]
    raise AssertionError("no gfx950 code object in the library")


def _kernels(elf: bytes):
    assert elf[:4] == b"\x7fELF"
    (section_table,) = struct.unpack_from("<Q", elf, 0x28)
    entry_size, count, _names = struct.unpack_from("<HHH", elf, 0x3A)
    for s in range(count):
        _name, kind, _flags, _addr, offset, size = struct.unpack_from("<IIQQQQ", elf, section_table + s * entry_size)
        if kind != 7:  # SHT_NOTE
            continue
        at, end = offset, offset + size
        while at < end:
            name_size, desc_size, note_type = struct.unpack_from("<III", elf, at)
            at += 12 + ((name_size + 3) & ~3)
            desc = elf[at:at + desc_size]
            at += (desc_size + 3) & ~3
            if note_type == 32:  # NT_AMDGPU_METADATA
                return msgpack.unpackb(desc, raw=False)["amdhsa.kernels"]
    raise AssertionError("no kernel metadata in the code object")


@pytest.fixture(scope="module")
def kernels():
    if not os.path.exists(LIB_PATH):
        build_library()
    with open(LIB_PATH, "rb") as fh:
        return _kernels(_gfx950_code_object(fh.read()))


def test_no_kernel_uses_accumulation_registers(kernels):
    assert {k[".name"]: k[".agpr_count"] for k in kernels if k.get(".agpr_count", 0)} == {}


def test_the_chain_kernel_spills_nothing(kernels):
    chain = next(k for k in kernels if "two_peel_kernel" in k[".name"])
    assert chain[".private_segment_fixed_size"] == 0
    assert chain[".max_flat_workgroup_size"] == 1024


def test_the_one_workgroup_kernels_spill_nothing(kernels):
    """Their registers are capped for eight waves per SIMD up to twelve objectives; a path added to them must fit."""
    small = [k for k in kernels if "batched_kernel" in k[".name"] or "two_small_kernel" in k[".name"]]
    assert len(small) == 17
    assert {k[".name"]: k[".private_segment_fixed_size"] for k in small if k[".private_segment_fixed_size"]} == {}


def test_every_kernel_is_built_for_wave64(kernels):
    assert len(kernels) > 100
    assert all(k[".wavefront_size"] == 64 for k in kernels)
