"""The C-ABI library loads and exports every symbol include/ptoamd.h declares (no GPU, no compute calls)."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "ptoamd.h")
LIB = os.path.join(ROOT, "pto-isa-mirror_amd", "lib", "libptoamd.so")


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ptoamd_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_surface():
    names = declared_symbols()
    for must in ("ptoamd_init", "ptoamd_malloc", "ptoamd_memcpy", "ptoamd_stream_synchronize", "ptoamd_gemm",
                 "ptoamd_gemm_w8a8", "ptoamd_gemm_mx", "ptoamd_gemv_mxfp4", "ptoamd_tquant_mx", "ptoamd_tquant_int8",
                 "ptoamd_tdequant", "ptoamd_mx_scale_relayout"):
        assert must in names


def test_library_exports_every_declared_symbol():
    assert os.path.exists(LIB), "build the library first: make -C pto-isa-mirror_amd -j8"
    lib = ctypes.CDLL(LIB)
    missing = [s for s in declared_symbols() if not hasattr(lib, s)]
    assert not missing, missing


def test_python_binding_lists_the_same_symbols():
    import __graft_entry__ as ge

    pa = ge.load_package()
    assert sorted(pa.EXPORTS) == declared_symbols()


def test_argument_errors_are_reported_without_a_gpu():
    lib = ctypes.CDLL(LIB)
    lib.ptoamd_last_error.restype = ctypes.c_char_p
    rc = lib.ptoamd_gemm(None, 0, None, None, 1, None, 4, 4, 4, 4, 4, 4, 1, 0, None)
    assert rc == -1 and b"null operand" in lib.ptoamd_last_error()
    buf = ctypes.create_string_buffer(64)
    rc = lib.ptoamd_gemm(buf, 0, buf, buf, 1, None, 0, 4, 4, 4, 4, 4, 1, 0, None)
    assert rc == -1 and b"positive" in lib.ptoamd_last_error()
    rc = lib.ptoamd_gemm(buf, 3, buf, buf, 2, None, 4, 4, 4, 4, 4, 4, 1, 0, None)  # bf16 operands, int32 result
    assert rc == -2
    rc = lib.ptoamd_gemm_mx(buf, 0, buf, buf, 6, 8, buf, buf, 1, 5, None, 16, 16, 64, 64, 64, 16, 1, None)
    assert rc == -2 and b"both" in lib.ptoamd_last_error()  # fp8 x fp4 is not a TMATMUL_MX combination
    rc = lib.ptoamd_gemm_mx(buf, 0, buf, buf, 6, 6, buf, buf, 1, 5, None, 16, 16, 96, 96, 96, 16, 1, None)
    assert rc == -1 and b"multiple of 64" in lib.ptoamd_last_error()
    rc = lib.ptoamd_gemv_mxfp4(buf, 0, buf, buf, buf, 17, 32, 256, 256, 256, 32, None)
    assert rc == -2
    lib.ptoamd_gemm_mx_workspace_bytes.restype = ctypes.c_size_t
    assert lib.ptoamd_gemm_mx_workspace_bytes(64, 48, 256, 0, 3) == 64 * 8 + 48 * 8  # ZZ / NN: both scale arrays re-laid
    assert lib.ptoamd_gemm_mx_workspace_bytes(64, 48, 256, 1, 5) == 0                # the natural layouts need none
