"""The GEMM written in the PTO tile ISA (pto-isa-mirror_amd/kernels/gemm_performance.hip: double-buffered TLOAD of K
panels, TEXTRACT, TMATMUL / TMATMUL_ACC, one TSTORE per core) against the oracle, through its extern "C" launcher.

The kernels run on the header layer's fast forms -- LDS-DMA TLOAD, Left / Right windows, register-blocked TMATMUL, staged
TSTORE -- so these are also the parity tests of those forms at full size.  The bars are the ones the C-ABI launcher of
the same product is held to (tests/test_gpu_parity.py::test_config2_bf16_4096_cubed).
"""
import ctypes as C
import os

import numpy as np
import pytest
import torch

import __graft_entry__ as ge
from oracle import binding as ob
from test_gpu_parity import DEV, bf16_to_f32, check_f32_drain, host, pa, relerr, sel  # noqa: F401  (pa: the package fixture)

pytestmark = pytest.mark.gpu

LIB = os.path.join(ge.PKG_DIR, "lib", "libpto_gemm_performance.so")


@pytest.fixture(scope="module")
def perf():
    assert os.path.exists(LIB), "build first: make -C pto-isa-mirror_amd"
    lib = C.CDLL(LIB)

    def run(case, out, a, b):
        rc = lib.pto_gemm_performance(case, C.c_void_p(out.data_ptr()), C.c_void_p(a.data_ptr()), C.c_void_p(b.data_ptr()),
                                      C.c_void_p(torch.cuda.current_stream().cuda_stream))
        assert rc == 0, f"launch failed with HIP error {rc}"
        torch.cuda.synchronize()
        assert lib.pto_gemm_performance_status() == 0
        return out

    return run


def test_f16_1024x1024x512_whole_matrix(pa, oracle, perf):
    """Case 2: fp16 inputs uniform in [-1, 1], fp32 result, 16 cores of 256 x 256; every output against the oracle."""
    m, n, k = 1024, 1024, 512
    r = np.random.default_rng(77)
    a = r.uniform(-1, 1, (m, k)).astype(np.float16)
    b = r.uniform(-1, 1, (n, k)).astype(np.float16)   # [N][K]: the DN view of B
    out = perf(2, torch.full((m, n), float("nan"), dtype=torch.float32, device=DEV), torch.from_numpy(a).to(DEV),
               torch.from_numpy(b).to(DEV))
    ref = oracle.matmul_f16(a.view(np.uint16), b.view(np.uint16), b_dn=True)
    absdot = np.abs(a.astype(np.float64)) @ np.abs(b.astype(np.float64)).T
    check_f32_drain(host(out), ref, absdot, k, "PTO-style GEMM f16 1024x1024x512")


def test_bf16_4096_cubed(pa, oracle, perf):
    """Cases 0 and 1: configs[1] (bf16 4096^3, A row-major, B column-major, N(0,1) * 0.02) written in the tile ISA.  The
    fp32 drain is held to both error bars on 4096 sampled outputs and two whole 256 x 256 tiles; the bf16 drain must be
    the rounding of the fp32 drain bit for bit, everywhere; every output element must have been written."""
    m = n = k = 4096
    gen = torch.Generator(device=DEV).manual_seed(2)
    a = (torch.randn((m, k), generator=gen, device=DEV) * 0.02).to(torch.bfloat16)
    b = (torch.randn((n, k), generator=gen, device=DEV) * 0.02).to(torch.bfloat16)
    f = perf(1, torch.full((m, n), float("nan"), dtype=torch.float32, device=DEV), a, b)
    out = perf(0, torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=DEV), a, b)
    f_h, out_h = host(f), host(out)
    assert not np.isnan(f_h).any()
    assert np.array_equal(out_h, oracle.store_f32(f_h, ob.ST_BF16))
    rows = np.unique(np.concatenate([[0, 1, 255, 256, 2047, 2048, 4095], np.arange(5, 4096, 72)]))[:64]
    cols = np.arange(0, 4096, 64) + np.arange(64) % 64
    blocks = [("samples", rows, cols), ("tile (0, 0)", np.arange(256), np.arange(256)),
              ("tile (15, 15)", np.arange(3840, 4096), np.arange(3840, 4096)),
              ("tile (7, 3)", np.arange(1792, 2048), np.arange(768, 1024))]
    for label, rr, cc in blocks:
        ar, bc = host(sel(a, rr)), host(sel(b, cc))
        ref = oracle.matmul_bf16(ar, bc, b_dn=True)
        absdot = np.abs(bf16_to_f32(ar).astype(np.float64)) @ np.abs(bf16_to_f32(bc).astype(np.float64)).T
        check_f32_drain(f_h[np.ix_(rr, cc)], ref, absdot, k, f"PTO-style GEMM bf16 4096^3, {label}")
        assert relerr(bf16_to_f32(out_h[np.ix_(rr, cc)]), ref) <= 1e-2
    # the same product through the C-ABI launcher: both run k ascending in 16-wide MFMA steps per output element
    assert relerr(f_h, host(pa.gemm(a, b, pa.BF16, pa.F32, pa.B_DN))) <= 1e-5


TILED_LIB = os.path.join(ge.PKG_DIR, "lib", "libpto_gemm_tiled.so")


@pytest.mark.parametrize("case", [0, 1])
def test_configs0_tiled_gemm_in_the_tile_isa(pa, oracle, case):
    """configs[0] written in the tile ISA (kernels/gemm_tiled.hip): fp16 512^3 -> fp32, A and B row-major, K slabs of 64,
    128 x 128 (case 0) or 64 x 64 (case 1) tiles of C per core.  B's slab is transposed by the TMOV into the Right tile.
    Every output against the oracle's sequential fp32 sum."""
    lib = C.CDLL(TILED_LIB)
    r = np.random.default_rng(1234)
    a = r.uniform(-1, 1, (512, 512)).astype(np.float16)
    b = r.uniform(-1, 1, (512, 512)).astype(np.float16)   # [K][N]
    da, db = torch.from_numpy(a).to(DEV), torch.from_numpy(b).to(DEV)
    out = torch.full((512, 512), float("nan"), dtype=torch.float32, device=DEV)
    rc = lib.pto_gemm_tiled(case, C.c_void_p(out.data_ptr()), C.c_void_p(da.data_ptr()), C.c_void_p(db.data_ptr()),
                            C.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == 0
    torch.cuda.synchronize()
    assert lib.pto_gemm_tiled_status() == 0
    ref = oracle.matmul_f16(a.view(np.uint16), b.view(np.uint16), b_dn=False)
    absdot = np.abs(a.astype(np.float64)) @ np.abs(b.astype(np.float64))
    check_f32_drain(host(out), ref, absdot, 512, f"PTO-style tiled GEMM f16 512^3, case {case}")


# ---- the block-scaled GEMM written in the tile ISA (kernels/mxmatmul_performance.hip) ------------------------------------
MX_LIB = os.path.join(ge.PKG_DIR, "lib", "libpto_mxmatmul_performance.so")


@pytest.fixture(scope="module")
def mxperf():
    assert os.path.exists(MX_LIB), "build first: make -C pto-isa-mirror_amd"
    lib = C.CDLL(MX_LIB)

    def run(case, out, a, b, sa, sb):
        rc = lib.pto_mxmatmul_performance(case, *(C.c_void_p(t.data_ptr()) for t in (out, a, b, sa, sb)),
                                          C.c_void_p(torch.cuda.current_stream().cuda_stream))
        assert rc == 0, f"launch failed with HIP error {rc}"
        torch.cuda.synchronize()
        assert lib.pto_mxmatmul_performance_status() == 0
        return out

    return run


def test_mxfp8_512x768x1024_whole_matrix(pa, oracle, mxperf):
    """Case 2: E4M3 codes over the whole finite range, scales 2^-8 .. 2^7, six cores; every output against the oracle (the
    bar of fp8 data that spans all codes: 2^-11 sum|a||b| element-wise, 1e-3 normalised), and bit for bit against the
    C-ABI launcher, which issues the same scaled MFMAs in the same k order."""
    m, n, k = 512, 768, 1024
    r = np.random.default_rng(123)
    a = r.integers(0, 256, (m, k)).astype(np.uint8)
    b = r.integers(0, 256, (n, k)).astype(np.uint8)
    a[(a & 0x7F) == 0x7F] = 0x12
    b[(b & 0x7F) == 0x7F] = 0x12
    sa = r.integers(119, 135, (m, k // 32)).astype(np.uint8)
    sb = r.integers(119, 135, (n, k // 32)).astype(np.uint8)
    d = [torch.from_numpy(x).to(DEV) for x in (a, b, sa, sb)]
    out = mxperf(2, torch.full((m, n), float("nan"), dtype=torch.float32, device=DEV), *d)
    got = host(out)
    ref = oracle.matmul_mx(a, b, sa, sb, m, k, n, ob.E4M3, ob.E4M3)
    table = oracle.mx_decode_table(ob.E4M3)
    wa = np.abs(table[a]) * np.repeat(2.0 ** (sa.astype(np.float64) - 127), 32, 1)
    wb = np.abs(table[b]) * np.repeat(2.0 ** (sb.astype(np.float64) - 127), 32, 1)
    check_f32_drain(got, ref, wa @ wb.T, k, "PTO-style MXFP8 512x768x1024", max_rel=1e-3, eps=2.0 ** -11)
    launcher = pa.gemm_mx(d[0], d[1], d[2], d[3], m, n, k, pa.E4M3, pa.E4M3, pa.F32)
    assert torch.equal(out, launcher)


def test_mxfp8_config3_full_size(pa, oracle, mxperf):
    """Cases 0 and 1: configs[3] (E4M3 4096 x 14336 x 4096, operands quantised from N(0,1) by TQUANT<MXFP8>) written in
    the tile ISA: the fp32 drain equals the launcher's bit for bit (itself held to the oracle in test_gpu_parity), the bf16
    drain is its rounding, every output is written, and a sample is checked against the oracle directly."""
    m, n, k = 4096, 14336, 4096
    gen = torch.Generator(device=DEV).manual_seed(4)
    a, sa = pa.tquant_mx(torch.randn((m, k), generator=gen, device=DEV), pa.OCP_MXFP8, want_aux=False)
    b, sb = pa.tquant_mx(torch.randn((n, k), generator=gen, device=DEV), pa.OCP_MXFP8, want_aux=False)
    f = mxperf(1, torch.full((m, n), float("nan"), dtype=torch.float32, device=DEV), a, b, sa, sb)
    out = mxperf(0, torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=DEV), a, b, sa, sb)
    assert not bool(torch.isnan(f).any())
    launcher = pa.gemm_mx(a, b, sa, sb, m, n, k, pa.E4M3, pa.E4M3, pa.F32)
    assert torch.equal(f, launcher)
    del launcher
    assert torch.equal(out, f.to(torch.bfloat16))
    rows = np.unique(np.concatenate([[0, 255, 256, 2049, 4095], np.arange(7, m, 131)]))[:32]
    cols = np.arange(0, n, 448) + np.arange(32) % 448
    ar, bc, sar, sbc = host(sel(a, rows)), host(sel(b, cols)), host(sel(sa, rows)), host(sel(sb, cols))
    ref = oracle.matmul_mx(ar, bc, sar, sbc, len(rows), k, len(cols), ob.E4M3, ob.E4M3)
    table = oracle.mx_decode_table(ob.E4M3)
    wa = np.abs(table[ar]) * np.repeat(2.0 ** (sar.astype(np.float64) - 127), 32, 1)
    wb = np.abs(table[bc]) * np.repeat(2.0 ** (sbc.astype(np.float64) - 127), 32, 1)
    check_f32_drain(host(f)[np.ix_(rows, cols)], ref, wa @ wb.T, k, "PTO-style MXFP8 configs[3], samples")


def test_mxfp4_512x768x1024_whole_matrix(pa, oracle, mxperf):
    """Case 5: packed E2M1 codes over all 16 values, scales 2^-8 .. 2^7: the same program with fp4 operand tiles (Mat
    tiles of packed codes stored as lines along K, loaded by LDS-DMA from an ND A and a DN B; Left / Right windows; the
    register-blocked TMATMUL_MX with one 16-byte fragment per block and k-step).  Every output against the oracle with the
    plain fp32 bars, and bit for bit against the C-ABI launcher."""
    m, n, k = 512, 768, 1024
    r = np.random.default_rng(321)
    a = r.integers(0, 256, (m, k // 2)).astype(np.uint8)
    b = r.integers(0, 256, (n, k // 2)).astype(np.uint8)
    sa = r.integers(119, 135, (m, k // 32)).astype(np.uint8)
    sb = r.integers(119, 135, (n, k // 32)).astype(np.uint8)
    d = [torch.from_numpy(x).to(DEV) for x in (a, b, sa, sb)]
    out = mxperf(5, torch.full((m, n), float("nan"), dtype=torch.float32, device=DEV), *d)
    got = host(out)
    ref = oracle.matmul_mx(a, b, sa, sb, m, k, n, ob.E2M1, ob.E2M1)
    table = oracle.mx_decode_table(ob.E2M1)
    unpack = lambda x: np.stack([table[x & 0xF], table[x >> 4]], -1).reshape(x.shape[0], -1)
    wa = np.abs(unpack(a)) * np.repeat(2.0 ** (sa.astype(np.float64) - 127), 32, 1)
    wb = np.abs(unpack(b)) * np.repeat(2.0 ** (sb.astype(np.float64) - 127), 32, 1)
    check_f32_drain(got, ref, wa @ wb.T, k, "PTO-style MXFP4 512x768x1024")
    launcher = pa.gemm_mx(d[0], d[1], d[2], d[3], m, n, k, pa.E2M1, pa.E2M1, pa.F32)
    assert torch.equal(out, launcher)


def test_mxfp4_2048x8192x8192_against_the_launcher(pa, mxperf):
    """Case 4: MXFP4 2048 x 8192 (K) x 8192, operands quantised from N(0,1) by TQUANT<MXFP4> -> bf16: every output written
    and equal to the launcher's (held to the oracle in test_gpu_parity)."""
    m, n, k = 2048, 8192, 8192
    gen = torch.Generator(device=DEV).manual_seed(44)
    a, sa = pa.tquant_mx(torch.randn((m, k), generator=gen, device=DEV), pa.OCP_MXFP4, want_aux=False)
    b, sb = pa.tquant_mx(torch.randn((n, k), generator=gen, device=DEV), pa.OCP_MXFP4, want_aux=False)
    out = mxperf(4, torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=DEV), a, b, sa, sb)
    assert not bool(torch.isnan(out).any())
    launcher = pa.gemm_mx(a, b, sa, sb, m, n, k, pa.E2M1, pa.E2M1, pa.BF16)
    assert torch.equal(out, launcher)

