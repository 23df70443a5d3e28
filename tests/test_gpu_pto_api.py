"""Parity of PTO-style kernel sources compiled against the gfx950 header layer (pto-isa-mirror_amd/include/pto).

tests/pto_kernels/matmul_kernels.hip holds kernels written the way the reference's test kernels are (TASSIGN / TLOAD /
TMOV / TMATMUL(_ACC|_BIAS) / TGEMV / TSTORE on Tile<> and GlobalTensor<>); its extern "C" launcher is called here with
device pointers and the results are compared with the oracle.  Case ids and shapes follow the reference's tmatmul test
list (tests/cpu/st/testcase/tmatmul/main.cpp:96-252); inputs use its own distribution (small integers: every partial
sum is exact, so the MFMA result must equal the simulator's bit for bit) and a float distribution (tolerance 1e-2 /
2e-2 as for every MFMA path).
"""
import ctypes
import os
import subprocess

import numpy as np
import pytest
import torch

from oracle import binding as ob

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(HERE, "pto_kernels", "build", "libptokernels.so")
DEMO = os.path.join(HERE, "pto_kernels", "build", "gemm_demo")
DEV = "cuda:0"


@pytest.fixture(scope="module")
def kernels():
    if not os.path.exists(LIB):
        raise RuntimeError(f"{LIB} is missing: run __graft_entry__.build() (make -C tests/pto_kernels)")
    lib = ctypes.CDLL(LIB)
    lib.pto_kernels_launch.argtypes = [ctypes.c_int] + [ctypes.c_void_p] * 5
    lib.pto_kernels_launch.restype = ctypes.c_int
    lib.pto_kernels_status.restype = ctypes.c_int
    torch.zeros(1, device=DEV)
    return lib


def run(lib, case, out, a, b, bias=None):
    da, db = torch.from_numpy(np.ascontiguousarray(a)).to(DEV), torch.from_numpy(np.ascontiguousarray(b)).to(DEV)
    dbias = torch.from_numpy(np.ascontiguousarray(bias)).to(DEV) if bias is not None else None
    dout = torch.zeros(out[0], dtype=out[1], device=DEV)
    stream = torch.cuda.current_stream().cuda_stream
    rc = lib.pto_kernels_launch(case, dout.data_ptr(), da.data_ptr(), db.data_ptr(),
                                dbias.data_ptr() if dbias is not None else None, stream)
    assert rc == 0, f"launch of case {case} failed with HIP error {rc}"
    torch.cuda.synchronize()
    assert lib.pto_kernels_status() == 0
    return dout


def relerr(got, ref):
    return float(np.abs(got.astype(np.float64) - ref.astype(np.float64)).max() / max(np.abs(ref).max(), 1e-30))


def f16_bits(x):
    return np.asarray(x, np.float32).astype(np.float16).view(np.uint16)


def bf16_bits(x):
    return torch.from_numpy(np.ascontiguousarray(x, np.float32)).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)


# case id -> (element kind, M, K, N, has bias)
SINGLE_TILE = {1: ("f16", 40, 50, 60, False), 4: ("f32", 56, 110, 40, False), 5: ("f16", 1, 110, 50, False),
               6: ("f32", 1, 128, 48, False), 7: ("bf16", 40, 50, 60, False), 11: ("f16", 26, 100, 94, True),
               13: ("f16", 1, 64, 96, True)}


@pytest.mark.parametrize("case", sorted(SINGLE_TILE))
@pytest.mark.parametrize("dist", ["ints", "floats"])
def test_single_tile_matmul(kernels, oracle, case, dist):
    kind, m, k, n, has_bias = SINGLE_TILE[case]
    r = np.random.default_rng(100 * case + (dist == "ints"))
    if dist == "ints":
        a, b = r.integers(1, 5, (m, k)).astype(np.float32), r.integers(1, 5, (k, n)).astype(np.float32)
        bias = r.integers(1, 5, (1, n)).astype(np.float32)
    else:
        a, b = r.uniform(-1, 1, (m, k)).astype(np.float32), r.uniform(-1, 1, (k, n)).astype(np.float32)
        bias = r.uniform(-1, 1, (1, n)).astype(np.float32)
    bias_arg = bias if has_bias else None
    if kind == "f16":
        ab, bb = f16_bits(a), f16_bits(b)
        ref = oracle.matmul_f16(ab, bb, bias=bias_arg)
    elif kind == "bf16":
        ab, bb = bf16_bits(a), bf16_bits(b)
        ref = oracle.matmul_bf16(ab, bb, bias=bias_arg)
    else:
        ab, bb = a, b
        ref = oracle.matmul_f32(ab, bb, bias=bias_arg)
    got = run(kernels, case, ((m, n), torch.float32), ab, bb, bias_arg).cpu().numpy()
    if dist == "ints":
        assert np.array_equal(got, ref)
    else:
        assert relerr(got, ref) <= 1e-2


@pytest.mark.parametrize("case,m,k,n,has_bias", [(2, 6, 7, 8, False), (12, 8, 7, 6, True)])
def test_single_tile_int8_bit_exact(kernels, oracle, case, m, k, n, has_bias):
    r = np.random.default_rng(case)
    a, b = r.integers(-128, 128, (m, k)).astype(np.int8), r.integers(-128, 128, (k, n)).astype(np.int8)
    bias = r.integers(-1000, 1000, (1, n)).astype(np.int32) if has_bias else None
    got = run(kernels, case, ((m, n), torch.int32), a, b, bias).cpu().numpy()
    assert np.array_equal(got, oracle.matmul_i8(a, b, bias=bias))


def test_single_tile_fp8(kernels, oracle):
    r = np.random.default_rng(8)
    m, k, n = 33, 64, 70
    a, b = r.integers(0, 256, (m, k)).astype(np.uint8), r.integers(0, 256, (k, n)).astype(np.uint8)
    a[(a & 0x7F) == 0x7F] = 0x3C  # no NaN codes
    b[(b & 0x7F) == 0x7F] = 0x3C
    got = run(kernels, 8, ((m, n), torch.float32), a, b).cpu().numpy()
    assert relerr(got, oracle.matmul_fp8(a, b)) <= 2e-2


# MX case id -> (A type, B type, M, K, N, A-scale layout, B-scale layout, bias)
MX_CASES = {1: (ob.E4M3, ob.E4M3, 32, 128, 48, ob.MX_A_ZZ, ob.MX_B_NN, False),
            2: (ob.E5M2, ob.E4M3, 33, 192, 70, ob.MX_A_ND, ob.MX_B_DN, True),
            3: (ob.E4M3, ob.E5M2, 16, 64, 32, ob.MX_A_DN, ob.MX_B_ND, False),
            4: (ob.E2M1, ob.E2M1, 40, 128, 60, ob.MX_A_ND, ob.MX_B_DN, False),   # packed fp4, two codes per byte
            5: (ob.E2M1, ob.E2M1, 32, 256, 64, ob.MX_A_ZZ, ob.MX_B_NN, True)}


def _codes(r, typ, shape):
    if typ == ob.E2M1:  # every nibble is a finite value; pairs run along the last axis
        return r.integers(0, 256, (shape[0], shape[1] // 2)).astype(np.uint8)
    c = r.integers(0, 256, shape).astype(np.uint8)
    if typ == ob.E4M3:
        c[(c & 0x7F) == 0x7F] = 0x38  # NaN codes -> 1.0
    else:
        c[(c & 0x7F) >= 0x7C] = 0x3C  # inf / NaN codes -> 1.0
    return c


@pytest.mark.parametrize("case", sorted(MX_CASES))
def test_tmatmul_mx_with_scale_tiles(kernels, oracle, case):
    """TLOAD of the E8M0 scale matrices from their GM layouts, TMOV into the Left / Right scale tiles, TMATMUL_MX."""
    ta, tb, m, k, n, la, lb, has_bias = MX_CASES[case]
    r = np.random.default_rng(40 + case)
    a, b = _codes(r, ta, (m, k)), _codes(r, tb, (k, n))
    kg = k // 32
    sa_log, sb_log = r.integers(120, 134, (m, kg)).astype(np.uint8), r.integers(120, 134, (kg, n)).astype(np.uint8)
    sa, sb = np.zeros(m * kg, np.uint8), np.zeros(kg * n, np.uint8)
    sa[oracle.mx_scale_offsets(la, m, kg)] = sa_log
    sb[oracle.mx_scale_offsets(lb, kg, n)] = sb_log
    bias = r.uniform(-1, 1, (1, n)).astype(np.float32) if has_bias else None
    ref = oracle.matmul_mx(a, b, sa, sb, m, k, n, ta, tb, sa_layout=la, sb_layout=lb, b_dn=False, bias=bias)

    kernels.pto_kernels_launch_mx.argtypes = [ctypes.c_int] + [ctypes.c_void_p] * 7
    kernels.pto_kernels_launch_mx.restype = ctypes.c_int
    d = [torch.from_numpy(x).to(DEV) for x in (a, b, sa, sb)]
    dbias = torch.from_numpy(bias).to(DEV) if has_bias else None
    out = torch.zeros((m, n), dtype=torch.float32, device=DEV)
    rc = kernels.pto_kernels_launch_mx(case, out.data_ptr(), d[0].data_ptr(), d[1].data_ptr(), d[2].data_ptr(), d[3].data_ptr(),
                                       dbias.data_ptr() if has_bias else None, torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    torch.cuda.synchronize()
    assert kernels.pto_kernels_status() == 0
    assert relerr(out.cpu().numpy(), ref) <= 2e-2


def test_nz_global_layout_and_acc_to_vec_move(kernels, oracle):
    """TLOAD from an NZ GlobalTensor; TMOV Acc -> Vec (f32 -> f16, round to nearest even); TSTORE of the Vec tile."""
    m, k, n, c0 = 32, 64, 48, 16
    r = np.random.default_rng(20)
    a, b = r.uniform(-1, 1, (m, k)).astype(np.float32), r.uniform(-1, 1, (k, n)).astype(np.float32)
    ab, bb = f16_bits(a), f16_bits(b)
    a_nz = np.ascontiguousarray(ab.reshape(m, k // c0, c0).transpose(1, 0, 2))  # [k / C0][m][C0]
    out = run(kernels, 20, ((m, n), torch.float16), a_nz, bb)
    got = out.cpu().numpy()
    ref32 = oracle.matmul_f16(ab, bb)
    assert relerr(got.astype(np.float32), ref32) <= 1e-2
    with_int = r.integers(1, 5, (m, k)).astype(np.float32), r.integers(1, 5, (k, n)).astype(np.float32)
    ab, bb = f16_bits(with_int[0]), f16_bits(with_int[1])
    a_nz = np.ascontiguousarray(ab.reshape(m, k // c0, c0).transpose(1, 0, 2))
    got = run(kernels, 20, ((m, n), torch.float16), a_nz, bb).cpu().numpy()
    assert np.array_equal(got.view(np.uint16), oracle.store_f32(oracle.matmul_f16(ab, bb), ob.ST_F16))


def test_split_k_accumulates_in_the_accumulator_tile(kernels, oracle):
    """TMATMUL then four TMATMUL_ACC over five K-slabs of a 128 x 128 x 64 tile (reference case 3)."""
    r = np.random.default_rng(3)
    m, k, n, reps = 128, 128, 64, 5
    a, b = r.integers(1, 5, (reps, m, k)).astype(np.float32), r.integers(1, 5, (reps, k, n)).astype(np.float32)
    got = run(kernels, 3, ((m, n), torch.float32), f16_bits(a), f16_bits(b)).cpu().numpy()
    ref = np.zeros((m, n), np.float32)
    for i in range(reps):
        ref = oracle.matmul_f16(f16_bits(a[i]), f16_bits(b[i]), cin=ref)
    assert np.array_equal(got, ref)
    a, b = r.uniform(-1, 1, (reps, m, k)).astype(np.float32), r.uniform(-1, 1, (reps, k, n)).astype(np.float32)
    got = run(kernels, 3, ((m, n), torch.float32), f16_bits(a), f16_bits(b)).cpu().numpy()
    ref = np.zeros((m, n), np.float32)
    for i in range(reps):
        ref = oracle.matmul_f16(f16_bits(a[i]), f16_bits(b[i]), cin=ref)
    assert relerr(got, ref) <= 1e-2


def test_tiled_gemm_512_cubed_f16(kernels, oracle):
    """configs[0] as a PTO program: 16 cores, 128 x 128 output tiles, K walked by 64."""
    r = np.random.default_rng(1234)
    a, b = r.uniform(-1, 1, (512, 512)).astype(np.float32), r.uniform(-1, 1, (512, 512)).astype(np.float32)
    got = run(kernels, 100, ((512, 512), torch.float32), f16_bits(a), f16_bits(b)).cpu().numpy()
    assert relerr(got, oracle.matmul_f16(f16_bits(a), f16_bits(b))) <= 1e-2


def test_tiled_gemm_bf16_column_major_b_bf16_out(kernels, oracle):
    """The configs[1] pipeline at 512^3: B as a DN GlobalTensor, TSTORE converting the fp32 accumulator to bf16."""
    r = np.random.default_rng(77)
    a, bt = (r.standard_normal((512, 512)) * 0.02).astype(np.float32), (r.standard_normal((512, 512)) * 0.02).astype(np.float32)
    ab, bb = bf16_bits(a), bf16_bits(bt)  # bt is [N][K]
    out = run(kernels, 101, ((512, 512), torch.bfloat16), ab, bb)
    got = (out.view(torch.int16).cpu().numpy().view(np.uint16).astype(np.uint32) << 16).view(np.float32)
    assert relerr(got, oracle.matmul_bf16(ab, bb, b_dn=True)) <= 1e-2


def test_host_demo_program():
    """The C++ host program (aclrt* runtime names over the C ABI + a Launch function) runs and checks itself."""
    if not os.path.exists(DEMO):
        raise RuntimeError(f"{DEMO} is missing: run __graft_entry__.build()")
    res = subprocess.run([DEMO], capture_output=True, text=True, timeout=120)
    assert res.returncode == 0, res.stdout + res.stderr
    assert "max_abs_diff=" in res.stdout and "status=0" in res.stdout


# ------------------------------------------------------------------------------------------- TQUANT / TDEQUANT tiles
def _eq_f32(a, b):
    return np.array_equal(a.view(np.uint32) & 0xFFBFFFFF, b.view(np.uint32) & 0xFFBFFFFF)  # NaN quiet bit aside


def _quant_launch(lib, case, dst, exp, mx, sc, src, scale=None, offset=None):
    lib.pto_kernels_launch_quant.argtypes = [ctypes.c_int] + [ctypes.c_void_p] * 8
    lib.pto_kernels_launch_quant.restype = ctypes.c_int
    p = lambda t: t.data_ptr() if t is not None else None
    rc = lib.pto_kernels_launch_quant(case, p(dst), p(exp), p(mx), p(sc), p(src), p(scale), p(offset),
                                      torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    torch.cuda.synchronize()
    assert lib.pto_kernels_status() == 0


# case -> (rows, cols, algorithm id, source dtype, oracle source kind)
QUANT_MX = {1: (16, 64, ob.OCP_FP8, torch.float32, ob.SRC_F32), 2: (16, 64, ob.NV_FP8, torch.float32, ob.SRC_F32),
            3: (16, 64, ob.OCP_FP4, torch.float32, ob.SRC_F32), 4: (16, 64, ob.NV_FP4, torch.float32, ob.SRC_F32),
            5: (8, 128, ob.OCP_FP4, torch.bfloat16, ob.SRC_BF16), 6: (8, 128, ob.OCP_FP8, torch.float16, ob.SRC_F16)}


@pytest.mark.parametrize("case", sorted(QUANT_MX))
def test_tquant_mx_tile_instruction_bit_exact(kernels, oracle, case):
    rows, cols, alg, dtype, kind = QUANT_MX[case]
    r = np.random.default_rng(case)
    x = (r.standard_normal((rows, cols)) * 10 ** r.uniform(-3, 3, (rows, 1))).astype(np.float32)
    x[0, :32] = 0                      # an all-zero group
    x[1, 3] = np.inf                   # the reference tests' edge inputs: infinity, NaN, the E4M3 boundary
    x[2, 40] = np.nan
    x[3, 0], x[3, 1] = 448.0, np.nextafter(np.float32(448.0), np.float32(np.inf))
    src = torch.from_numpy(x).to(dtype)
    fp4 = alg in (ob.OCP_FP4, ob.NV_FP4)
    g = rows * cols // 32
    dst = torch.zeros(rows * cols // (2 if fp4 else 1), dtype=torch.uint8, device=DEV)
    exp = torch.zeros(g, dtype=torch.uint8, device=DEV)
    mx, sc = torch.zeros(g, dtype=torch.float32, device=DEV), torch.zeros(g, dtype=torch.float32, device=DEV)
    _quant_launch(kernels, case, dst, exp, mx, sc, src.to(DEV))
    rc, re, rm, rs = oracle.tquant_mx(src.float().numpy(), alg, 1, kind)
    assert np.array_equal(exp.cpu().numpy(), re.ravel())
    assert np.array_equal(dst.cpu().numpy(), rc.ravel())
    assert _eq_f32(mx.cpu().numpy(), rm.ravel()) and _eq_f32(sc.cpu().numpy(), rs.ravel())


@pytest.mark.parametrize("case,alg", [(7, ob.OCP_FP8), (8, ob.NV_FP4)])
def test_tquant_mx_column_groups_bit_exact(kernels, oracle, case, alg):
    """TQUANT<0, alg>: 32 consecutive rows of a column share the exponent (the reference's tquant_dn form)."""
    rows, cols = 64, 16
    r = np.random.default_rng(case)
    x = (r.standard_normal((rows, cols)) * 10 ** r.uniform(-3, 3, (1, cols))).astype(np.float32)
    x[:32, 0] = 0
    x[5, 1] = np.inf
    fp4 = alg in (ob.OCP_FP4, ob.NV_FP4)
    g = rows // 32 * cols
    dst = torch.zeros(rows * cols // (2 if fp4 else 1), dtype=torch.uint8, device=DEV)
    exp = torch.zeros(g, dtype=torch.uint8, device=DEV)
    mx, sc = torch.zeros(g, dtype=torch.float32, device=DEV), torch.zeros(g, dtype=torch.float32, device=DEV)
    _quant_launch(kernels, case, dst, exp, mx, sc, torch.from_numpy(x).to(DEV))
    rc, re, rm, rs = oracle.tquant_mx(x, alg, 0, ob.SRC_F32)
    assert np.array_equal(exp.cpu().numpy(), re.ravel())
    assert np.array_equal(dst.cpu().numpy(), rc.ravel())
    assert _eq_f32(mx.cpu().numpy(), rm.ravel()) and _eq_f32(sc.cpu().numpy(), rs.ravel())


def test_tquant_mx_nz_store_mode_reorders_exponents(kernels, oracle):
    """TQUANT<MXFP8, VecStoreMode::NZ>: codes and row-major exponents as in ND mode, plus the exponents in 16-row x
    2-group boxes (reference: cpu/TQuant.hpp:254-278 ReorderExponentZZ)."""
    rows, cols = 16, 128
    r = np.random.default_rng(9)
    x = (r.standard_normal((rows, cols)) * 10 ** r.uniform(-2, 2, (rows, cols // 32)).repeat(32, axis=1)).astype(np.float16)
    g = rows * cols // 32
    dst = torch.zeros(rows * cols, dtype=torch.uint8, device=DEV)
    exp = torch.zeros(g, dtype=torch.uint8, device=DEV)
    zz = torch.zeros(g, dtype=torch.float32, device=DEV)  # the launcher's `max` slot carries exp_zz's bytes here
    sc = torch.zeros(g, dtype=torch.float32, device=DEV)
    _quant_launch(kernels, 9, dst, exp, zz, sc, torch.from_numpy(x).to(DEV))
    rc, re, _, rs = oracle.tquant_mx(x.astype(np.float32), ob.OCP_FP8, 1, ob.SRC_F16)
    assert np.array_equal(dst.cpu().numpy(), rc.ravel())
    assert np.array_equal(exp.cpu().numpy(), re.ravel())
    assert _eq_f32(sc.cpu().numpy(), rs.ravel())
    gc = cols // 32
    want = re.reshape(rows // 16, 16, gc // 2, 2).transpose(0, 2, 1, 3).ravel()
    assert len(set(re.ravel().tolist())) > 4  # the permutation is visible in the data
    assert np.array_equal(zz.cpu().numpy().view(np.uint8)[:g], want)


def test_tquant_int8_and_tdequant_tile_instructions_bit_exact(kernels, oracle):
    r = np.random.default_rng(21)
    src = (r.standard_normal((16, 64)) * 60).astype(np.float32)
    scale, off = r.uniform(0.2, 3, 16).astype(np.float32), r.uniform(0, 200, 16).astype(np.float32)
    d = lambda a: torch.from_numpy(a).to(DEV)
    for case, offset in ((10, None), (11, off)):
        dst = torch.zeros((16, 64), dtype=torch.uint8, device=DEV)
        _quant_launch(kernels, case, dst, None, None, None, d(src), d(scale), d(off))
        ref = oracle.tquant_int8(src, scale, offset)
        assert np.array_equal(dst.cpu().numpy(), ref.view(np.uint8))
    for case, shape, dt in ((20, (16, 64), np.int8), (21, (8, 32), np.int32)):
        q = r.integers(-120, 120, shape).astype(dt) if dt == np.int8 else r.integers(-10 ** 6, 10 ** 6, shape).astype(dt)
        s, o = r.uniform(0.01, 2, shape[0]).astype(np.float32), r.uniform(-5, 5, shape[0]).astype(np.float32)
        out = torch.zeros(shape, dtype=torch.float32, device=DEV)
        _quant_launch(kernels, case, out, None, None, None, d(q), d(s), d(o))
        assert np.array_equal(out.cpu().numpy().view(np.uint32), oracle.tdequant(q, s, o).view(np.uint32))


# ------------------------------------------------------------------------------------------- TSTORE with quantisation
def _word(scale, offset=0, signed=True, vector=False):
    bits = int(np.float32(scale).view(np.uint32))
    if vector:
        bits &= 0xFFFFE000  # 19-bit (1, 8, 10) float at bits 13..31
    return np.uint64(bits | (offset << 37) | (int(signed) << 46))


# case -> (input kind, M, K, N, per-column words, relu, oracle destination kind, numpy output dtype, signed 8-bit target)
STORE_QUANT = {1: ("f16", 40, 50, 60, False, False, ob.ST_I8, np.int8, True),
               2: ("f16", 33, 64, 70, True, True, ob.ST_U8, np.uint8, False),
               3: ("i8", 24, 96, 40, True, False, ob.ST_F16, np.uint16, True),
               4: ("i8", 24, 96, 40, False, False, ob.ST_I8, np.int8, True),
               5: ("f16", 40, 50, 60, False, False, ob.ST_BF16, np.uint16, True),
               6: ("i8", 24, 96, 40, True, True, ob.ST_BF16, np.uint16, True),
               7: ("i8", 24, 96, 40, False, False, ob.ST_I16, np.int16, True),
               8: ("i8", 24, 96, 40, True, True, ob.ST_I16, np.int16, True)}


@pytest.mark.parametrize("case", sorted(STORE_QUANT))
def test_tstore_fix_pipe_quantisation(kernels, oracle, case):
    """Accumulators are exact here (integer-valued inputs), so the quantised stores must match the simulator bit for bit."""
    kind, m, k, n, vector, relu, dst_kind, out_dt, signed = STORE_QUANT[case]
    r = np.random.default_rng(60 + case)
    if kind == "f16":
        a, b = r.integers(-4, 5, (m, k)).astype(np.float32), r.integers(-4, 5, (k, n)).astype(np.float32)
        acc = oracle.matmul_f16(f16_bits(a), f16_bits(b))
        da, db = f16_bits(a), f16_bits(b)
    else:
        da, db = r.integers(-128, 128, (m, k)).astype(np.int8), r.integers(-128, 128, (k, n)).astype(np.int8)
        acc = oracle.matmul_i8(da, db)
    span = float(np.abs(acc).max())
    to_byte = dst_kind in (ob.ST_I8, ob.ST_U8)
    scales = r.uniform(0.5, 1.5, n) * (100.0 / span if to_byte else 1.0 / 64)
    words = np.array([_word(s, offset=(3 if to_byte else 0), signed=signed, vector=vector) for s in scales], np.uint64)
    if dst_kind == ob.ST_I16:  # shift mode: the count sits in bits 32..35
        words = words & np.uint64(0xFFFFFFFF) | (r.integers(0, 12, n).astype(np.uint64) << np.uint64(32))
    if not vector:
        words = words[:1]
    ref = oracle.store_quant(acc, dst_kind, words, per_column=vector, relu=relu)

    kernels.pto_kernels_launch_store_quant.argtypes = [ctypes.c_int] + [ctypes.c_void_p] * 5
    kernels.pto_kernels_launch_store_quant.restype = ctypes.c_int
    t = [torch.from_numpy(np.ascontiguousarray(x)).to(DEV) for x in (da, db)]
    dw = torch.from_numpy(words.view(np.int64)).to(DEV)
    out = torch.zeros(m * n * np.dtype(out_dt).itemsize, dtype=torch.uint8, device=DEV)
    rc = kernels.pto_kernels_launch_store_quant(case, out.data_ptr(), t[0].data_ptr(), t[1].data_ptr(), dw.data_ptr(),
                                                torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    torch.cuda.synchronize()
    assert kernels.pto_kernels_status() == 0
    got = out.cpu().numpy().view(out_dt).reshape(m, n)
    assert np.array_equal(got, ref.view(out_dt))
    assert len(np.unique(got)) > 8  # the case exercises the quantiser, not a saturated constant


# ------------------------------------------------------------------------------- framework-free runner + launch trace
RUNNER = os.path.join(HERE, "pto_kernels", "build", "case_runner")


def test_case_runner_and_launch_trace(tmp_path):
    """The C++ test main (aclrt* calls, Launch, host golden, ResultCmp) passes its cases, exits non-zero otherwise, and
    with PTOAMD_TRACE_DIR set every C-ABI launch leaves one JSON record."""
    import json

    if not os.path.exists(RUNNER):
        raise RuntimeError(f"{RUNNER} is missing: run __graft_entry__.build()")
    env = dict(os.environ, PTOAMD_TRACE_DIR=str(tmp_path))
    for case in ("tmatmul", "tmatmul_i8", "tmatmul_mx", "gemm", "gemm_mx", "quant_gemm"):
        res = subprocess.run([RUNNER, case], capture_output=True, text=True, timeout=120, env=env)
        assert res.returncode == 0, case + "\n" + res.stdout + res.stderr
        assert f"{case}: PASS" in res.stdout and "err count: 0," in res.stdout, res.stdout
    assert subprocess.run([RUNNER, "no_such_case"], capture_output=True, timeout=60, env=env).returncode == 2
    records = []
    for name in sorted(os.listdir(tmp_path)):
        assert name.startswith("ptoamd_trace_") and name.endswith(".jsonl")
        with open(tmp_path / name) as f:
            records.append([json.loads(line) for line in f])
    by_len = sorted(records, key=len)
    # the three C-ABI cases: one, one and three launches (PTO-kernel cases launch no C-ABI kernel and write no file)
    assert [len(r) for r in by_len] == [1, 1, 3]
    ops = sorted(r[0]["opcode"] for r in by_len[:2])
    assert ops == ["TMATMUL", "TMATMUL_MX"]
    for recs in by_len:
        for i, rec in enumerate(recs):
            assert rec["sequence_id"] == i and rec["kernel"] and rec["pipeline"] in ("cube", "vector")
            assert all({"address", "shape", "layout", "dtype"} <= set(t) for t in rec["input_tiles"] + rec["output_tiles"])
    gemm = next(r[0] for r in by_len[:2] if r[0]["opcode"] == "TMATMUL")
    assert (gemm["m"], gemm["n"], gemm["k"]) == (256, 384, 512) and gemm["kernel"].startswith("tile")
    assert [t["dtype"] for t in gemm["input_tiles"]] == ["bf16", "bf16"] and gemm["input_tiles"][1]["layout"] == "DN"
    assert gemm["output_tiles"][0]["dtype"] == "f32" and gemm["output_tiles"][0]["shape"] == [256, 384]
    quant = by_len[2]
    assert [r["opcode"] for r in quant] == ["TQUANT_MXFP8", "TQUANT_MXFP8", "TMATMUL_MX"]
    assert quant[0]["pipeline"] == "vector" and quant[0]["kernel"] == "tquant_mx_rows"
    assert [t["layout"] for t in quant[2]["input_tiles"][2:4]] == ["MX_A_ND", "MX_B_DN"]


def test_instruction_trace_of_a_pto_kernel(tmp_path, monkeypatch):
    """A kernel source compiled with -DPTO_AMD_TRACE leaves one record per executed tile instruction, in execution order,
    with the operands' place, shape and dtype: the single-tile matmul of case 1 is TLOAD, TLOAD, TMOV, TMOV, TMATMUL,
    TSTORE; the split-K program of case 3 repeats its body five times, with TMATMUL first and TMATMUL_ACC after."""
    import json

    path = os.path.join(HERE, "pto_kernels", "build", "libptokernels_trace.so")
    if not os.path.exists(path):
        raise RuntimeError(f"{path} is missing: run __graft_entry__.build() (make -C tests/pto_kernels)")
    lib = ctypes.CDLL(path)
    lib.pto_kernels_launch.argtypes = [ctypes.c_int] + [ctypes.c_void_p] * 5
    lib.pto_kernels_launch.restype = ctypes.c_int
    lib.pto_kernels_status.restype = ctypes.c_int
    monkeypatch.setenv("PTOAMD_TRACE_DIR", str(tmp_path))
    r = np.random.default_rng(3)
    a = r.integers(1, 5, (40, 50)).astype(np.float16)
    b = r.integers(1, 5, (50, 60)).astype(np.float16)
    out = run(lib, 1, ((40, 60), torch.float32), a, b)
    assert np.array_equal(out.cpu().numpy(), a.astype(np.float32) @ b.astype(np.float32))  # the traced build computes the same
    files = sorted(os.listdir(tmp_path))
    assert len(files) == 1 and files[0].startswith("ptoamd_instr_trace_") and files[0].endswith(".jsonl")
    with open(tmp_path / files[0]) as f:
        recs = [json.loads(line) for line in f]
    assert [x["opcode"] for x in recs] == ["TLOAD", "TLOAD", "TMOV", "TMOV", "TMATMUL", "TSTORE"]
    assert [x["sequence_id"] for x in recs] == list(range(6)) and all(x["block_idx"] == 0 for x in recs)
    assert recs[0]["output_tiles"] == [{"address": 0, "shape": [40, 50], "layout": "Mat", "dtype": "float16"}]
    assert recs[0]["input_tiles"][0]["layout"] == "ND" and recs[0]["input_tiles"][0]["shape"] == [40, 50]
    assert recs[1]["output_tiles"][0]["address"] == 0x8000 and recs[1]["output_tiles"][0]["shape"] == [50, 60]
    assert [t["layout"] for t in recs[4]["output_tiles"] + recs[4]["input_tiles"]] == ["Acc", "Left", "Right"]
    assert recs[4]["output_tiles"][0] == {"address": 0, "shape": [40, 60], "layout": "Acc", "dtype": "float32"}
    assert recs[5]["output_tiles"][0]["layout"] == "ND" and recs[5]["output_tiles"][0]["dtype"] == "float32"
    assert recs[5]["input_tiles"][0]["layout"] == "Acc"
    # a loop is recorded as executed: five K slabs
    os.remove(tmp_path / files[0])
    a5 = r.integers(1, 5, (5 * 128, 128)).astype(np.float16)
    b5 = r.integers(1, 5, (5 * 128, 64)).astype(np.float16)
    run(lib, 3, ((128, 64), torch.float32), a5, b5)
    with open(tmp_path / sorted(os.listdir(tmp_path))[0]) as f:
        ops = [json.loads(line)["opcode"] for line in f]
    body = ["TLOAD", "TLOAD", "TMOV", "TMOV"]
    assert ops == body + ["TMATMUL"] + (body + ["TMATMUL_ACC"]) * 4 + ["TSTORE"]


def _expand_runner_cases(tmp_path):
    """tests/golden/runner_cases.npz -> <tmp>/<suite>/<case>/<name>.bin, the files the runner reads."""
    data = np.load(os.path.join(HERE, "golden", "runner_cases.npz"), allow_pickle=False)
    for key in data.files:
        suite, case, name = key.split("/")
        os.makedirs(tmp_path / suite / case, exist_ok=True)
        data[key].tofile(tmp_path / suite / case / f"{name}.bin")
    return os.path.join(HERE, "golden", "runner_cases.txt")


def test_case_runner_reference_case_lists(tmp_path):
    """The framework-free runner over the reference's own case lists (tmatmul case1-4 / gemm / bias, tmatmul_mx case1-19,
    tstore_acc2gm, tstore_quant ND_1 ... ND_10 as tile-ISA kernels, tquant, tdequant): inputs and goldens come from files (goldens made by the oracle), every case runs through the
    C ABI, those with a compiled PTO kernel through that too, and the comparison is the reference's ResultCmp.  -l lists,
    -t selects a suite or a case, an unknown selection is exit status 2."""
    if not os.path.exists(RUNNER):
        raise RuntimeError(f"{RUNNER} is missing: run __graft_entry__.build()")
    manifest = _expand_runner_cases(tmp_path)
    base = [RUNNER, "--data", str(tmp_path), "--manifest", manifest]
    listed = subprocess.run(base + ["-l"], capture_output=True, text=True, timeout=60)
    names = listed.stdout.split()
    assert listed.returncode == 0 and len(names) == 93
    assert {"tmatmul.case1", "tmatmul.case_bias_5", "tmatmul_mx.case19", "tstore_acc2gm.case_relu_21", "tdequant.case2",
            "tstore_quant.DN_9", "tquant.MxFp4E2M1NVBf16NdMixed", "tquant.Int8Asym"} <= set(names)
    res = subprocess.run(base, capture_output=True, text=True, timeout=300)
    assert res.returncode == 0, res.stdout[-4000:] + res.stderr[-2000:]
    assert "93 cases run, 0 failed" in res.stdout
    for name in names:
        assert f"{name}: PASS" in res.stdout, name
    # tmatmul case1, 2, 3, gemm_1, bf16_1, bias_1 also ran as tile-ISA kernels; the ten tstore_quant cases only so
    assert res.stdout.count("[pto kernel]") == 16
    one = subprocess.run(base + ["-t", "tmatmul_mx.case2"], capture_output=True, text=True, timeout=60)
    assert one.returncode == 0 and "1 cases run, 0 failed" in one.stdout
    suite = subprocess.run(base + ["-t", "tdequant"], capture_output=True, text=True, timeout=60)
    assert suite.returncode == 0 and "2 cases run, 0 failed" in suite.stdout
    assert subprocess.run(base + ["-t", "no_such_suite"], capture_output=True, timeout=60).returncode == 2
    # a wrong golden is a failure, not a pass: flip one case's golden and run it alone
    path = tmp_path / "tmatmul" / "case1" / "golden.bin"
    g = np.fromfile(path, np.float32)
    (g + 1.0).astype(np.float32).tofile(path)
    bad = subprocess.run(base + ["-t", "tmatmul.case1"], capture_output=True, text=True, timeout=60)
    assert bad.returncode == 1 and "tmatmul.case1: FAIL" in bad.stdout
