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


# The reference's hand-tuned kernels for this path are written in the same tile ISA.  Their core programs -- everything
# but one statement -- are checked the same way.  The statement is the CANN launch configuration
# `<<<blockDim, nullptr, stream>>>` (block count, an L2 control pointer, a stream), which is not HIP's
# `<<<grid, block, shared bytes, stream>>>`: it is taken out of a temporary copy (the kernel is then named as an ordinary
# function call, which instantiates the whole core program for the shape the file launches), nothing else is touched and
# the copy lives in pytest's temporary directory only.
MANUAL = "/root/reference/kernels/manual"
MANUAL_SOURCES = ["a2a3/gemm_performance/gemm_performance_kernel.cpp", "a5/matmul_mxfp8_performance/mxmatmul_performance_kernel.cpp",
                  "a5/matmul_mxfp4_performance/mxmatmul_performance_kernel.cpp"]
CANN_LAUNCH = "<<<blockDim, nullptr, stream>>>"


@pytest.mark.parametrize("source", MANUAL_SOURCES)
def test_reference_performance_kernel_core_program_compiles_against_the_header_layer(source, tmp_path):
    path = os.path.join(MANUAL, source)
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(path):
        pytest.skip("reference tree not mounted")
    if not os.path.exists(hipcc):
        pytest.skip("hipcc not installed")
    text = open(path).read()
    assert text.count(CANN_LAUNCH) == 1, "the file's one launch statement"
    copy = tmp_path / os.path.basename(source)
    copy.write_text(text.replace(CANN_LAUNCH, ""))
    cmd = [hipcc, "-std=c++17", "-O1", "--offload-arch=gfx950", "-x", "hip", "--cuda-device-only", "-fsyntax-only",
           "-DPTO_AMD_CHECK_REFERENCE_SOURCE", "-DPTO_AMD_L1_BYTES=524288", "-DPTO_AMD_L0A_BYTES=65536",
           "-DPTO_AMD_L0B_BYTES=65536", "-DPTO_AMD_UB_BYTES=262144", "-DPTO_AMD_L0S_BYTES=16384",
           "-I" + os.path.join(ROOT, "pto-isa-mirror_amd", "include"), str(copy)]
    res = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    assert res.returncode == 0, res.stderr[-4000:]

