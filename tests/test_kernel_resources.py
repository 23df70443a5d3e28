"""Register allocation of the shipped kernels, read from the built library (no GPU needed).

A kernel that spills keeps part of its working set in scratch memory; for the tile GEMM kernels that has cost up to a
tenth of the run time without failing any result check, so the library's own code-object metadata is checked here:
no kernel of the library may use scratch at all.
"""
import os
import struct

import msgpack
import pytest

LIB = os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", "pto-isa-mirror_amd", "lib", "libptoamd.so")
MAGIC = b"__CLANG_OFFLOAD_BUNDLE__"


def _code_objects(blob):
    """Yield the gfx950 ELF images of every offload bundle in the shared library."""
    pos = blob.find(MAGIC)
    while pos >= 0:
        (count,) = struct.unpack_from("<Q", blob, pos + len(MAGIC))
        off = pos + len(MAGIC) + 8
        for _ in range(count):
            start, size, tlen = struct.unpack_from("<QQQ", blob, off)
            triple = blob[off + 24:off + 24 + tlen].decode()
            off += 24 + tlen
            if "amdgcn" in triple and size:
                assert triple.endswith("gfx950"), triple
                yield blob[pos + start:pos + start + size]
        pos = blob.find(MAGIC, pos + 1)


def _kernels(elf):
    """The amdhsa.kernels records of one code object (its NT_AMDGPU_METADATA note is a msgpack map)."""
    assert elf[:4] == b"\x7fELF" and elf[4] == 2, "64-bit ELF expected"
    shoff, = struct.unpack_from("<Q", elf, 0x28)
    shentsize, shnum = struct.unpack_from("<HH", elf, 0x3A)
    for i in range(shnum):
        sh_type, = struct.unpack_from("<I", elf, shoff + i * shentsize + 4)
        if sh_type != 7:  # SHT_NOTE
            continue
        off, size = struct.unpack_from("<QQ", elf, shoff + i * shentsize + 0x18)
        p, end = off, off + size
        while p + 12 <= end:
            namesz, descsz, ntype = struct.unpack_from("<III", elf, p)
            name = elf[p + 12:p + 12 + namesz].rstrip(b"\0")
            desc_at = p + 12 + (namesz + 3) // 4 * 4
            if name == b"AMDGPU" and ntype == 32:
                meta = msgpack.unpackb(elf[desc_at:desc_at + descsz], raw=False, strict_map_key=False)
                yield from meta.get("amdhsa.kernels", [])
            p = desc_at + (descsz + 3) // 4 * 4


@pytest.fixture(scope="module")
def kernels():
    if not os.path.exists(LIB):
        pytest.skip("libptoamd.so is not built")
    with open(LIB, "rb") as f:
        blob = f.read()
    ks = [k for elf in _code_objects(blob) for k in _kernels(elf)]
    assert ks, "no kernel metadata found in the library"
    return ks


def test_no_kernel_uses_scratch(kernels):
    names = [k[".name"] for k in kernels]
    for tag in ("gemm_tile_dtl_kernel", "gemm_tile_kernel", "gemv_mxfp4_splitk", "tquant_", "tdequant"):
        assert any(tag in n for n in names), (tag, names)
    spilled = {k[".name"]: k[".private_segment_fixed_size"] for k in kernels if k[".private_segment_fixed_size"]}
    assert not spilled, spilled


def test_large_tiles_keep_two_waves_per_simd(kernels):
    """The 8-wave 256 x 256 DMA tiles run two waves per SIMD: at most 256 vector registers, and an LDS budget set at
    launch (no static LDS)."""
    big = [k for k in kernels if "gemm_tile_dtl_kernel" in k[".name"] and "Li256ELi256ELi2ELi4" in k[".name"]]
    assert len(big) >= 8, [k[".name"] for k in kernels if "dtl" in k[".name"]]
    for k in big:
        assert k[".vgpr_count"] + k.get(".agpr_count", 0) <= 256, (k[".name"], k[".vgpr_count"], k.get(".agpr_count"))
        assert k[".max_flat_workgroup_size"] == 512
