"""The header boundary, checked from the reference's side: its own PTO kernel sources for the matmul path are parsed and
type-checked, unchanged and where they lie, against pto-isa-mirror_amd/include (device pass of hipcc, -fsyntax-only, so no
GPU is needed).  Runs only where the reference tree is mounted; nothing is copied out of it.

PTO_AMD_CHECK_REFERENCE_SOURCE lifts the 160 KiB LDS budget for this check (those kernels TASSIGN the NPU's 512 KiB L1
addresses) and lets the host-side launch wrappers in the same files name the core functions.
"""
import os
import shutil
import subprocess

import pytest

REF = "/root/reference/tests/cpu/st/testcase"
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SOURCES = ["tmatmul/tmatmul_kernel.cpp", "tmatmul_mx/tmatmul_mx_kernel.cpp", "tmatmul_mx_nddn/tmatmul_mx_nddn_kernel.cpp",
           "tdequant/tdequant_kernel.cpp", "tstore_quant/tstore_quant_kernel.cpp"]


@pytest.mark.parametrize("source", SOURCES)
def test_reference_kernel_source_compiles_against_the_header_layer(source):
    path = os.path.join(REF, source)
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(path):
        pytest.skip("reference tree not mounted")
    if not os.path.exists(hipcc):
        pytest.skip("hipcc not installed")
    cmd = [hipcc, "-std=c++17", "-O1", "--offload-arch=gfx950", "-x", "hip", "--cuda-device-only", "-fsyntax-only",
           "-DPTO_AMD_CHECK_REFERENCE_SOURCE", "-DPTO_AMD_L1_BYTES=524288", "-DPTO_AMD_L0A_BYTES=65536",
           "-DPTO_AMD_L0B_BYTES=65536", "-DPTO_AMD_UB_BYTES=262144", "-DPTO_AMD_L0S_BYTES=16384",
           "-I" + os.path.join(ROOT, "pto-isa-mirror_amd", "include"), path]
    res = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    assert res.returncode == 0, res.stderr[-4000:]
