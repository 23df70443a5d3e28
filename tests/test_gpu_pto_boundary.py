"""Parity of the header-layer instructions around the matmul path: tests/pto_kernels/boundary_kernels.hip.

Block-scaled matmul programs shaped like the reference's own (tests/cpu/st/testcase/tmatmul_mx/tmatmul_mx_kernel.cpp:63-209
and :365-472) at its case shapes with K not a multiple of 64 (main.cpp case2 127x72x64, case3 128x110x63, case6 128x118x64),
E1M2 operands, TGEMV_MX; TCVT; TFILLPAD; TEXTRACT at nonzero offsets; TSTORE<AtomicAdd>; 5-D ND / DN global tensors; the
fix-pipe forms of TMOV / TEXTRACT; TRESHAPE; the TASSIGN status word.  Everything is compared with the oracle (bit for bit
where the arithmetic is exact) and, for the block-scaled products, also with a float64 closed form.
"""
import ctypes
import os

import numpy as np
import pytest
import torch

from oracle import binding as ob

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(HERE, "pto_kernels", "build", "libptoboundary.so")
DEV = "cuda:0"
VP = ctypes.c_void_p


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(LIB):
        raise RuntimeError(f"{LIB} is missing: run __graft_entry__.build() (make -C tests/pto_kernels)")
    L = ctypes.CDLL(LIB)
    L.pto_boundary_launch_mx.argtypes = [ctypes.c_int] + [VP] * 7
    L.pto_boundary_launch_cvt.argtypes = [ctypes.c_int, VP, VP, ctypes.c_int, ctypes.c_int, VP]
    L.pto_boundary_launch.argtypes = [ctypes.c_int, VP, VP, VP, VP, ctypes.c_uint, VP]
    torch.zeros(1, device=DEV)
    return L


def dev(x):
    return None if x is None else torch.from_numpy(np.ascontiguousarray(x)).to(DEV)


def ptr(t):
    return None if t is None else t.data_ptr()


def stream():
    return torch.cuda.current_stream().cuda_stream


def launch(lib, case, out, src0=None, src1=None, src2=None, arg=0, status=0):
    rc = lib.pto_boundary_launch(case, ptr(out), ptr(src0), ptr(src1), ptr(src2), arg, stream())
    assert rc == 0, f"launch of case {case} failed with HIP error {rc}"
    torch.cuda.synchronize()
    assert lib.pto_boundary_status() == status
    return out


def f16_bits(x):
    return np.asarray(x, np.float32).astype(np.float16).view(np.uint16)


def assert_sum_close(got, ref, absdot, k, what="", rel=1e-2, eps=None):
    """|got - ref| <= rel |ref| + eps sum|a||b| element by element (eps = 8 k 2^-24 unless given); prints the worst error."""
    err = np.abs(got.astype(np.float64) - ref.astype(np.float64))
    bound = rel * np.abs(ref.astype(np.float64)) + (8 * k * 2.0 ** -24 if eps is None else eps) * absdot
    worst = float((err / np.maximum(bound, 1e-300)).max())
    print(f"{what}: max|got-ref| = {err.max():.3e}, max|ref| = {np.abs(ref).max():.3e}, worst error / bound = {worst:.3e}, "
          f"max error / sum|a||b| = {float((err / np.maximum(absdot, 1e-300)).max()):.3e}")
    assert (err <= bound).all()


# ------------------------------------------------------------------------------------------ block-scaled matmul
FP4 = (ob.E2M1, ob.E1M2)
# case -> (A type, B type, M, K, N, bias)
MX_TILE = {2: (ob.E4M3, ob.E4M3, 127, 72, 64, False), 3: (ob.E4M3, ob.E5M2, 128, 110, 63, False),
           5: (ob.E1M2, ob.E2M1, 117, 64, 60, False), 6: (ob.E2M1, ob.E1M2, 128, 118, 64, False),
           15: (ob.E2M1, ob.E1M2, 35, 128, 56, True)}
# case -> (A type, B type, K, N, B-scale layout)
MX_GEMV = {11: (ob.E1M2, ob.E1M2, 128, 62, ob.MX_B_ND), 12: (ob.E4M3, ob.E5M2, 256, 20, ob.MX_B_ND),
           21: (ob.E2M1, ob.E2M1, 192, 40, ob.MX_B_DN)}


def _values_to_codes(oracle, typ, vals):
    """Nearest code of each value (round to nearest even), one code per array element."""
    if typ in FP4:
        table = oracle.mx_decode_table(typ)[:16]
        return np.abs(vals[..., None] - table).argmin(-1).astype(np.uint8)
    return np.vectorize(lambda v: oracle.lib.pto_fp8_encode_round(typ, float(v), 1, 0), otypes=[np.uint8])(vals)


def _mx_operand(oracle, r, typ, shape, dist):
    """(one code per element, decoded float64 values) of an operand matrix."""
    if dist == "ints":  # the reference generator's ranges (tmatmul_mx/gen_data.py:109-121)
        lo, hi = {ob.E2M1: (-6, 6), ob.E1M2: (-1, 2)}.get(typ, (-10, 10))
        codes = _values_to_codes(oracle, typ, r.integers(lo, hi, shape).astype(np.float64))
    elif typ in FP4:
        codes = r.integers(0, 16, shape).astype(np.uint8)
    else:
        codes = r.integers(0, 256, shape).astype(np.uint8)
        bad = (codes & 0x7F) == 0x7F if typ == ob.E4M3 else (codes & 0x7F) >= 0x7C
        codes[bad] = 0x38
    return codes, oracle.mx_decode_table(typ)[codes]


def _pack(codes, typ):
    """Global-memory bytes of a code matrix: fp4 packs pairs along the last axis, even element in the low nibble."""
    if typ in FP4:
        return (codes[..., 0::2] | (codes[..., 1::2] << 4)).astype(np.uint8)
    return codes


def _pad_k(codes, k_align, axis):
    pad = [(0, 0), (0, 0)]
    pad[axis] = (0, k_align - codes.shape[axis])
    return np.pad(codes, pad)


def _mx_problem(oracle, r, ta, tb, m, k, n, dist):
    k_align = (k + 63) // 64 * 64
    kg = k_align // 32
    a, av = _mx_operand(oracle, r, ta, (m, k), dist)
    b, bv = _mx_operand(oracle, r, tb, (k, n), dist)
    lo, hi = (127, 130) if dist == "ints" else (118, 136)
    sa, sb = r.integers(lo, hi, (m, kg)).astype(np.uint8), r.integers(lo, hi, (kg, n)).astype(np.uint8)
    wa = av * np.repeat(2.0 ** (sa.astype(np.float64) - 127), 32, 1)[:, :k]
    wb = bv * np.repeat(2.0 ** (sb.astype(np.float64) - 127), 32, 0)[:k, :]
    # the oracle walks the K the tiles are padded to: zero codes there (what TFILLPAD / the zero fill of TMOV leave)
    ref = oracle.matmul_mx(_pack(_pad_k(a, k_align, 1), ta), _pack(_pad_k(b, k_align, 0), tb), sa, np.ascontiguousarray(sb.T),
                           m, k_align, n, ta, tb, sa_layout=ob.MX_A_ND, sb_layout=ob.MX_B_DN, b_dn=False)
    return a, b, sa, sb, ref, wa @ wb, np.abs(wa) @ np.abs(wb), kg


def _mx_bound(ta):
    """Error bound of a block-scaled product on operands drawn from the whole code range, relative to sum|a||b|.
    FP4 products accumulate like fp32 sums.  The FP8 form of the scaled MFMA aligns the 64 products of one instruction
    to their largest exponent before adding them and keeps about 13 bits below it (measured: 2.4e-4 sum|a||b| at worst
    on codes spanning 2^-9 .. 448 with scales 2^-9 .. 2^8), so the bound is 2^-11 sum|a||b| with no relative term; on
    the reference's own test distribution the result is exact (the "ints" cases)."""
    return {} if ta in FP4 else {"rel": 0.0, "eps": 2.0 ** -11}


@pytest.mark.parametrize("dist", ["ints", "codes"])
@pytest.mark.parametrize("case", sorted(MX_TILE))
def test_tmatmul_mx_unaligned_k_with_tfillpad(lib, oracle, case, dist):
    ta, tb, m, k, n, has_bias = MX_TILE[case]
    r = np.random.default_rng(1000 + case)
    a, b, sa, sb, ref, exact, absdot, kg = _mx_problem(oracle, r, ta, tb, m, k, n, dist)
    mp, np_ = (m + 15) // 16 * 16, (n + (63 if ta in FP4 else 31)) // (64 if ta in FP4 else 32) * (64 if ta in FP4 else 32)
    sa_gm, sb_gm = np.zeros(mp * kg, np.uint8), np.zeros(kg * np_, np.uint8)
    sa_gm[oracle.mx_scale_offsets(ob.MX_A_ZZ, mp, kg)[:m]] = sa
    sb_gm[oracle.mx_scale_offsets(ob.MX_B_NN, kg, np_)[:, :n]] = sb
    bias = r.integers(1, 10, (1, n)).astype(np.float32) if has_bias else None
    out = torch.full((m, n), float("nan"), dtype=torch.float32, device=DEV)
    d = [dev(x) for x in (_pack(a, ta), _pack(b, tb), sa_gm, sb_gm, bias)]
    rc = lib.pto_boundary_launch_mx(case, ptr(out), ptr(d[0]), ptr(d[1]), ptr(d[2]), ptr(d[3]), ptr(d[4]), stream())
    assert rc == 0
    torch.cuda.synchronize()
    assert lib.pto_boundary_status() == 0
    got = out.cpu().numpy()
    if has_bias:
        ref, exact = ref + bias, exact + bias
    if dist == "ints":
        # every product and partial sum is a small integer times 2^(0..4): fp32 accumulation is exact in any order
        assert np.array_equal(got, exact.astype(np.float32))
        assert np.array_equal(got, ref)
    else:
        assert_sum_close(got, ref, absdot, k, f"mx case {case}", **_mx_bound(ta))
        assert_sum_close(got, exact, absdot, k, f"mx case {case} vs float64", **_mx_bound(ta))


@pytest.mark.parametrize("dist", ["powers", "normal"])
def test_quantise_then_matmul_mx_in_one_kernel(lib, oracle, dist):
    """f32 A -> TQUANT<MXFP8> in Vec tiles -> TMOV codes ND -> NZ Mat tile, exponents -> scale Mat tile -> TMATMUL_MX.
    The kernel's result is compared with the oracle's TMATMUL_MX of the oracle's own quantisation of A: a wrong code
    layout, exponent row or scale pairing after the TMOVs shows as a gross error.  'powers': A holds signed powers of
    two and B small integers, so codes, scales and sums are all exact and the match must be bit for bit."""
    m, k, n = 32, 128, 64
    kg = k // 32
    r = np.random.default_rng(70 + len(dist))
    if dist == "powers":
        # a different binade per 64 elements (one MFMA's worth, so that nothing is shifted out inside the instruction),
        # narrow enough that every partial sum fits 24 bits and the order of the additions cannot matter
        e = np.repeat(r.integers(-2, 3, (m, k // 64)), 64, 1) + r.integers(-3, 1, (m, k))
        a = (np.ldexp(1.0, e) * r.choice([-1.0, 1.0], (m, k))).astype(np.float32)
        b, bv = _mx_operand(oracle, r, ob.E4M3, (k, n), "ints")
        sb = r.integers(125, 130, (kg, n)).astype(np.uint8)
    else:
        a = (r.standard_normal((m, k)) * np.exp(r.uniform(-3, 3, (m, 1)))).astype(np.float32)
        b, bv = _mx_operand(oracle, r, ob.E4M3, (k, n), "codes")
        sb = r.integers(118, 136, (kg, n)).astype(np.uint8)
    codes, exp, _, _ = oracle.tquant_mx(a, ob.OCP_FP8, 1)
    ref = oracle.matmul_mx(codes, b, exp, np.ascontiguousarray(sb.T), m, k, n, ob.E4M3, ob.E4M3,
                           sa_layout=ob.MX_A_ND, sb_layout=ob.MX_B_DN, b_dn=False)
    sb_gm = np.zeros(kg * n, np.uint8)
    sb_gm[oracle.mx_scale_offsets(ob.MX_B_NN, kg, n)] = sb
    out = torch.full((m, n), float("nan"), dtype=torch.float32, device=DEV)
    launch(lib, 70, out, dev(a), dev(b), dev(sb_gm))
    got = out.cpu().numpy()
    wa = oracle.mx_decode_table(ob.E4M3)[codes] * np.repeat(2.0 ** (exp.astype(np.float64) - 127), 32, 1)
    wb = bv * np.repeat(2.0 ** (sb.astype(np.float64) - 127), 32, 0)
    assert np.abs(ref).max() > 0 and len(np.unique(exp)) > 3
    assert_sum_close(got, ref, np.abs(wa) @ np.abs(wb), k, "quantise-then-matmul " + dist, **_mx_bound(ob.E4M3))
    if dist == "powers":
        assert np.array_equal(got, ref)


@pytest.mark.parametrize("dist", ["ints", "codes"])
@pytest.mark.parametrize("case", sorted(MX_GEMV))
def test_tgemv_mx(lib, oracle, case, dist):
    ta, tb, k, n, lb = MX_GEMV[case]
    r = np.random.default_rng(2000 + case)
    a, b, sa, sb, ref, exact, absdot, kg = _mx_problem(oracle, r, ta, tb, 1, k, n, dist)
    sb_gm = np.zeros(kg * n, np.uint8)
    sb_gm[oracle.mx_scale_offsets(lb, kg, n)] = sb
    out = torch.full((1, n), float("nan"), dtype=torch.float32, device=DEV)
    d = [dev(x) for x in (_pack(a, ta), _pack(b, tb), sa.reshape(-1), sb_gm)]
    rc = lib.pto_boundary_launch_mx(case, ptr(out), ptr(d[0]), ptr(d[1]), ptr(d[2]), ptr(d[3]), None, stream())
    assert rc == 0
    torch.cuda.synchronize()
    assert lib.pto_boundary_status() == 0
    got = out.cpu().numpy()
    if dist == "ints":
        assert np.array_equal(got, exact.astype(np.float32))
        assert np.array_equal(got, ref)
    else:
        assert_sum_close(got, ref, absdot, k, f"gemv mx case {case}", **_mx_bound(ta))


@pytest.mark.parametrize("dist", ["ints", "codes"])
@pytest.mark.parametrize("case", [30, 31, 32, 33])
def test_fp4_operands_from_nd_and_dn_global_tensors(lib, oracle, case, dist):
    """Packed fp4 codes pair along the unit-stride direction of the global tensor (a row of ND, a column of DN), and in
    a boxed Mat tile along its lines (rows on the A side, columns on the B side).  All four combinations through the
    element-wise TLOAD (tiles with a ragged valid region): bytes move where the directions agree, and are built from two
    source nibbles where they do not.  Case 30 + (A is DN) + 2 (B is DN)."""
    m, k, n = 30, 128, 60
    r = np.random.default_rng(3000 + case)
    a, b, sa, sb, ref, exact, absdot, kg = _mx_problem(oracle, r, ob.E2M1, ob.E2M1, m, k, n, dist)
    a_dn, b_dn = (case - 30) & 1, (case - 30) & 2
    a_gm = _pack(np.ascontiguousarray(a.T), ob.E2M1) if a_dn else _pack(a, ob.E2M1)
    b_gm = _pack(np.ascontiguousarray(b.T), ob.E2M1) if b_dn else _pack(b, ob.E2M1)
    out = torch.full((m, n), float("nan"), dtype=torch.float32, device=DEV)
    d = [dev(x) for x in (a_gm, b_gm, sa.reshape(-1), np.ascontiguousarray(sb.T).reshape(-1))]
    rc = lib.pto_boundary_launch_mx(case, ptr(out), ptr(d[0]), ptr(d[1]), ptr(d[2]), ptr(d[3]), None, stream())
    assert rc == 0
    torch.cuda.synchronize()
    assert lib.pto_boundary_status() == 0
    got = out.cpu().numpy()
    if dist == "ints":
        assert np.array_equal(got, exact.astype(np.float32))
        assert np.array_equal(got, ref)
    else:
        assert_sum_close(got, ref, absdot, k, f"fp4 layouts case {case}", **_mx_bound(ob.E2M1))


# ------------------------------------------------------------------------------------------------------- TCVT
R, C, V = 16, 72, 70
RINT, ROUND, FLOOR, CEIL, TRUNC, ODD = 1, 2, 3, 4, 5, 6
SAT_ON, SAT_OFF = 0, 1


def _cvt(lib, case, src, dst_dtype, mode, sat):
    out = torch.zeros((R, V), dtype=dst_dtype, device=DEV)
    d = dev(src)
    rc = lib.pto_boundary_launch_cvt(case, ptr(out), ptr(d), mode, sat, stream())
    assert rc == 0
    torch.cuda.synchronize()
    assert lib.pto_boundary_status() == 0
    return out.cpu().numpy()


def _cvt_source(r):
    x = (r.standard_normal((R, V)) * 10.0 ** r.uniform(-3, 3, (R, 1))).astype(np.float32)
    x[0, :12] = [0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 3.5, -3.5, 0.0, -0.0, 126.5, -127.5]  # ties
    x[1, :6] = [300.0, -300.0, 70000.0, -70000.0, 3e9, -3e9]                              # beyond int8 / half / int32
    return x


def _round_int(x, mode):
    x = x.astype(np.float64)
    if mode == RINT:
        return np.rint(x)
    if mode == ROUND:
        return np.sign(x) * np.floor(np.abs(x) + 0.5)
    if mode == FLOOR:
        return np.floor(x)
    if mode == CEIL:
        return np.ceil(x)
    if mode == TRUNC:
        return np.trunc(x)
    f = np.floor(x)  # ODD: nearest, a tie to the odd neighbour
    frac = x - f
    return np.where(frac > 0.5, f + 1, np.where(frac < 0.5, f, np.where(f.astype(np.int64) & 1, f, f + 1)))


@pytest.mark.parametrize("mode", [RINT, ROUND, FLOOR, CEIL, TRUNC, ODD])
def test_tcvt_float_to_integer_round_modes(lib, mode):
    """cpu/TCvt.hpp:80-113 (the rounding) and :207-230 (saturation ON clamps to the destination range first)."""
    x = _cvt_source(np.random.default_rng(mode))
    want = _round_int(np.clip(x, -2.0 ** 31, 2.0 ** 31 - 1), mode)
    got = _cvt(lib, 3, x, torch.int32, mode, SAT_ON)
    ok = np.abs(x) < 2.0 ** 31 - 256  # float(2^31 - 1) rounds up to 2^31: leave the top edge to the dedicated values
    assert np.array_equal(got[ok], want[ok].astype(np.int32))
    got8 = _cvt(lib, 4, x, torch.int8, mode, SAT_ON)
    assert np.array_equal(got8, _round_int(np.clip(x, -128, 127), mode).astype(np.int8))
    gotu8 = _cvt(lib, 5, x, torch.uint8, mode, SAT_ON)
    assert np.array_equal(gotu8, _round_int(np.clip(x, 0, 255), mode).astype(np.uint8))
    small = np.clip(x, -100, 100)  # in range: saturation OFF and the overload without a mode agree with ON
    assert np.array_equal(_cvt(lib, 4, small, torch.int8, mode, SAT_OFF), _round_int(small, mode).astype(np.int8))
    assert np.array_equal(_cvt(lib, 4, small, torch.int8, mode, -1), _round_int(small, mode).astype(np.int8))


def test_tcvt_float_to_half_and_bf16(lib, oracle):
    x = _cvt_source(np.random.default_rng(11))
    x[1, :6] = [65504.0, 65519.9, 65520.0, -65520.0, 1e-8, 6e-8]  # the half overflow boundary and subnormals
    want16 = np.vectorize(lambda v: oracle.lib.pto_f32_to_f16(float(v)), otypes=[np.uint16])(x)
    got16 = _cvt(lib, 1, x, torch.float16, RINT, SAT_OFF).view(np.uint16)
    assert np.array_equal(got16, want16)
    assert np.array_equal(got16, x.astype(np.float16).view(np.uint16))
    sat = _cvt(lib, 1, x, torch.float16, RINT, SAT_ON).view(np.uint16)
    assert np.array_equal(sat, np.clip(x, -65504, 65504).astype(np.float16).view(np.uint16))
    wantbf = np.vectorize(lambda v: oracle.lib.pto_f32_to_bf16(float(v)), otypes=[np.uint16])(x)
    out = torch.zeros((R, V), dtype=torch.bfloat16, device=DEV)  # (numpy has no bf16: read the bits back)
    assert lib.pto_boundary_launch_cvt(2, ptr(out), ptr(dev(x)), RINT, SAT_OFF, stream()) == 0
    torch.cuda.synchronize()
    assert np.array_equal(out.view(torch.int16).cpu().numpy().view(np.uint16), wantbf)


@pytest.mark.parametrize("case,typ", [(6, ob.E4M3), (7, ob.E5M2)])
@pytest.mark.parametrize("sat", [SAT_ON, SAT_OFF])
@pytest.mark.parametrize("mode", [RINT, ROUND, FLOOR, CEIL, TRUNC, ODD])
def test_tcvt_float_to_fp8_round_modes(lib, oracle, case, typ, sat, mode):
    """The rounding constructor of the FP8 types (cpu/MXTypes.hpp:95-170), which the oracle restates and the compiled
    reference pins (tests/golden encode_round_fp8)."""
    r = np.random.default_rng(100 * case + 10 * mode + sat)
    x = _cvt_source(r)
    x[2, :10] = [448.0, 464.0, 465.0, 480.0, -449.0, 57344.0, 61440.0, 65536.0, 2.0 ** -9, 2.0 ** -10 * 1.5]
    x[3, :4] = [np.inf, -np.inf, np.nan, 2.0 ** -17]
    # oracle saturation flag: 1 = saturate (golden axis order (0, 1) = (off, on))
    want = np.vectorize(lambda v: oracle.lib.pto_fp8_encode_round(typ, float(v), mode, int(sat == SAT_ON)),
                        otypes=[np.uint8])(x.astype(np.float64))
    out = torch.zeros((R, V), dtype=torch.uint8, device=DEV)
    assert lib.pto_boundary_launch_cvt(case, ptr(out), ptr(dev(x)), mode, sat, stream()) == 0
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    nan = np.isnan(x)
    assert np.array_equal(got[~nan], want[~nan])
    assert ((got[nan] & 0x7F) >= (0x7F if typ == ob.E4M3 else 0x7D)).all()


def test_tcvt_widening_and_integer_sources(lib, oracle):
    r = np.random.default_rng(12)
    h = (r.standard_normal((R, V)) * 100).astype(np.float16)
    assert np.array_equal(_cvt(lib, 8, h, torch.float32, RINT, SAT_OFF), h.astype(np.float32))
    i = r.integers(-2 ** 31, 2 ** 31, (R, V)).astype(np.int32)
    assert np.array_equal(_cvt(lib, 9, i, torch.float32, RINT, SAT_OFF), i.astype(np.float32))
    assert np.array_equal(_cvt(lib, 10, h, torch.int16, FLOOR, SAT_ON), np.floor(h.astype(np.float64)).astype(np.int16))
    codes = r.integers(0, 256, (R, V)).astype(np.uint8)
    codes[(codes & 0x7F) == 0x7F] = 0x12
    out = torch.zeros((R, V), dtype=torch.float32, device=DEV)
    assert lib.pto_boundary_launch_cvt(11, ptr(out), ptr(dev(codes)), RINT, SAT_OFF, stream()) == 0
    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().numpy(), oracle.mx_decode_table(ob.E4M3)[codes].astype(np.float32))
    want = np.vectorize(lambda v: oracle.lib.pto_fp8_encode_round(ob.E4M3, float(v), RINT, 1), otypes=[np.uint8])(h.astype(np.float64))
    out8 = torch.zeros((R, V), dtype=torch.uint8, device=DEV)
    assert lib.pto_boundary_launch_cvt(12, ptr(out8), ptr(dev(h)), RINT, SAT_ON, stream()) == 0
    torch.cuda.synchronize()
    assert np.array_equal(out8.cpu().numpy(), want)


# ---------------------------------------------------------------------------------------------------- TFILLPAD
@pytest.mark.parametrize("case,dtype,pad", [(1, np.float32, np.inf), (2, np.float16, -np.inf), (3, np.int32, 0)])
def test_tfillpad_vec_tile(lib, case, dtype, pad):
    """cpu/TFillPad.hpp:22-64: the source's valid 13 x 50 region, the destination tile's pad value around it."""
    r = np.random.default_rng(case)
    src = (r.standard_normal((13, 50)) * 50).astype(dtype)
    out = launch(lib, case, torch.zeros((16, 64), dtype=getattr(torch, np.dtype(dtype).name), device=DEV), dev(src)).cpu().numpy()
    want = np.full((16, 64), pad, dtype)
    want[:13, :50] = src
    assert np.array_equal(out, want)


@pytest.mark.parametrize("case,vr,vc,dtype", [(4, 27, 40, np.float16), (5, 32, 33, np.uint8)])
def test_tfillpad_mat_tile_in_place_clears_stale_storage(lib, case, vr, vc, dtype):
    r = np.random.default_rng(case)
    junk = r.integers(1, 120, (32, 64)).astype(dtype)
    src = r.integers(1, 120, (vr, vc)).astype(dtype)
    tdt = torch.float16 if dtype == np.float16 else torch.uint8
    out = launch(lib, case, torch.zeros((32, 64), dtype=tdt, device=DEV), dev(src), dev(junk)).cpu().numpy()
    want = np.zeros((32, 64), dtype)
    want[:vr, :vc] = src
    assert np.array_equal(out, want)


# ------------------------------------------------------------------------------------- TEXTRACT / TSTORE / TLOAD
def test_textract_sub_blocks_of_mat_tiles(lib, oracle):
    r = np.random.default_rng(10)
    a, b = r.uniform(-1, 1, (64, 128)).astype(np.float32), r.uniform(-1, 1, (128, 64)).astype(np.float32)
    ab, bb = f16_bits(a), f16_bits(b)
    got = launch(lib, 10, torch.zeros((32, 32), dtype=torch.float32, device=DEV), dev(ab), dev(bb)).cpu().numpy()
    sa, sb = np.ascontiguousarray(ab[32:64, 64:128]), np.ascontiguousarray(bb[64:128, 32:64])
    ref = oracle.matmul_f16(sa, sb)
    absdot = np.abs(sa.view(np.float16).astype(np.float64)) @ np.abs(sb.view(np.float16).astype(np.float64))
    assert_sum_close(got, ref, absdot, 64, "textract f16")
    ai, bi = r.integers(-128, 128, (32, 128)).astype(np.int8), r.integers(-128, 128, (128, 64)).astype(np.int8)
    got = launch(lib, 11, torch.zeros((16, 32), dtype=torch.int32, device=DEV), dev(ai), dev(bi)).cpu().numpy()
    assert np.array_equal(got, oracle.matmul_i8(np.ascontiguousarray(ai[16:32, 32:96]), np.ascontiguousarray(bi[32:96, 32:64])))


def test_tstore_atomic_add_accumulates_across_cores(lib, oracle):
    r = np.random.default_rng(20)
    m, k, n, cores = 40, 50, 60, 3
    a, b = r.integers(1, 5, (cores, m, k)).astype(np.float32), r.integers(1, 5, (k, n)).astype(np.float32)
    init = r.integers(-100, 100, (m, n)).astype(np.float32)
    got = launch(lib, 20, dev(init.copy()), dev(f16_bits(a)), dev(f16_bits(b))).cpu().numpy()
    want = init.copy()
    for c in range(cores):  # integers: exact in any order
        want += oracle.matmul_f16(f16_bits(a[c]), f16_bits(b))
    assert np.array_equal(got, want)
    m, k, n, cores = 24, 64, 40, 2
    ai, bi = r.integers(-128, 128, (cores, m, k)).astype(np.int8), r.integers(-128, 128, (k, n)).astype(np.int8)
    init = r.integers(-2 ** 31, 2 ** 31, (m, n)).astype(np.int32)  # wraps mod 2^32 like the accumulator
    got = launch(lib, 21, dev(init.copy()), dev(ai), dev(bi)).cpu().numpy()
    want = init.astype(np.int64) + sum(oracle.matmul_i8(ai[c], bi).astype(np.int64) for c in range(cores))
    assert np.array_equal(got, (want & 0xFFFFFFFF).astype(np.uint32).view(np.int32))


@pytest.mark.parametrize("case,which,dtype", [(30, 0, np.float16), (31, 1, np.float16), (32, 0, np.float32)])
def test_global_tensor_5d(lib, oracle, golden, case, which, dtype):
    """Shape<2,3,4,8,16> with padded strides, every outer dimension above 1: TLOAD gathers the logical matrix through
    the same offset map the compiled reference produced (tests/golden global_offset_*), TSTORE scatters it back."""
    offs = golden[f"global_offset_{which}"]
    sh, st = golden[f"global_shape_{which}"], golden[f"global_stride_{which}"]
    layout = ob.ND if which == 0 else ob.DN
    assert np.array_equal(offs, oracle.global_offsets(layout, sh, st, *offs.shape))
    size = int(offs.max()) + 1
    r = np.random.default_rng(case)
    src = r.integers(-1000, 1000, size).astype(dtype)
    tdt = torch.float16 if dtype == np.float16 else torch.float32
    packed = torch.zeros(offs.shape, dtype=tdt, device=DEV)
    scattered = torch.full((size,), -7.0, dtype=tdt, device=DEV)
    launch(lib, case, packed, dev(src), scattered)
    assert np.array_equal(packed.cpu().numpy(), src[offs])
    want = np.full(size, -7.0, dtype)
    want[offs] = src[offs]
    assert np.array_equal(scattered.cpu().numpy(), want)


def _word_scalar(scale, offset=0, sign=1):
    return int(np.float32(scale).view(np.uint32)) | (offset << 37) | (sign << 46)


def _word_vector(scale, offset=0, sign=1):
    bits = int(np.float32(scale).view(np.uint32))
    m1 = ((bits >> 31) << 18) | (((bits >> 23) & 0xFF) << 10) | ((bits >> 13) & 0x3FF)
    return (m1 << 13) | (offset << 37) | (sign << 46)


def test_tmov_and_textract_fixpipe_forms(lib, oracle):
    """Accumulator -> Vec tile with relu, with a scalar quantisation word, with per-column words, and the sub-block forms
    (cpu/TMov.hpp, cpu/TExtract.hpp:21-46, cpu/common.hpp:117-185)."""
    r = np.random.default_rng(40)
    m, k, n = 48, 64, 96
    a, b = r.integers(-4, 5, (m, k)).astype(np.float32), r.integers(-4, 5, (k, n)).astype(np.float32)
    ab, bb = f16_bits(a), f16_bits(b)
    acc = oracle.matmul_f16(ab, bb)  # integers: the accumulator is exact
    da, db = dev(ab), dev(bb)
    got = launch(lib, 40, torch.zeros((m, n), dtype=torch.float16, device=DEV), da, db).cpu().numpy()
    assert np.array_equal(got.view(np.uint16), oracle.store_f32(acc, ob.ST_F16, relu=True))
    word = np.array([_word_scalar(0.37, offset=3)] * n, np.uint64)
    got = launch(lib, 41, torch.zeros((m, n), dtype=torch.int8, device=DEV), da, db, dev(word.view(np.int64))).cpu().numpy()
    assert np.array_equal(got, oracle.store_quant(acc, ob.ST_I8, word[:1], per_column=False))
    words = np.array([_word_vector(s) for s in r.uniform(0.01, 0.5, n)], np.uint64)
    got = launch(lib, 42, torch.zeros((m, n), dtype=torch.float16, device=DEV), da, db, dev(words.view(np.int64))).cpu().numpy()
    assert np.array_equal(got.view(np.uint16), oracle.store_quant(acc, ob.ST_F16, words, per_column=True, relu=True))
    got = launch(lib, 43, torch.zeros((m - 16, n - 32), dtype=torch.int8, device=DEV), da, db, dev(word.view(np.int64))).cpu().numpy()
    assert np.array_equal(got, oracle.store_quant(acc, ob.ST_I8, word[:1], per_column=False)[16:, 32:])
    got = launch(lib, 44, torch.zeros((m - 16, n - 32), dtype=torch.float32, device=DEV), da, db).cpu().numpy()
    assert np.array_equal(got, acc[16:, 32:])
    ai, bi = r.integers(-128, 128, (m, k)).astype(np.int8), r.integers(-128, 128, (k, n)).astype(np.int8)
    word = np.array([_word_scalar(2.0 ** -9, offset=5)], np.uint64)
    got = launch(lib, 45, torch.zeros((m, n), dtype=torch.int8, device=DEV), dev(ai), dev(bi), dev(word.view(np.int64))).cpu().numpy()
    assert np.array_equal(got, oracle.store_quant(oracle.matmul_i8(ai, bi), ob.ST_I8, word, per_column=False))


def test_tmov_and_textract_into_an_accumulator_tile(lib, oracle):
    """The start value of an accumulator comes from a Vec tile (TMOV), from an offset of a larger Vec tile with relu
    (TEXTRACT), or from another accumulator (reference: cpu/TMov.hpp:21-35 moves between any two tile kinds); the
    product is then added onto it by TMATMUL_ACC, so the result is the oracle's matmul with that start value."""
    r = np.random.default_rng(46)
    m, k, n = 40, 50, 60
    # small integers: every partial sum is exact, so the MFMA's order of additions cannot show
    a, b = f16_bits(r.integers(-4, 5, (m, k))), f16_bits(r.integers(-4, 5, (k, n)))
    c0 = r.integers(-100, 100, (m, n)).astype(np.float32)
    got = launch(lib, 46, torch.zeros((m, n), dtype=torch.float32, device=DEV), dev(a), dev(b), dev(c0)).cpu().numpy()
    assert np.array_equal(got.view(np.uint32), oracle.matmul_f16(a, b, cin=c0).view(np.uint32))
    big = r.integers(-100, 100, (m + 8, n + 16)).astype(np.float32)
    got = launch(lib, 47, torch.zeros((m, n), dtype=torch.float32, device=DEV), dev(a), dev(b), dev(big)).cpu().numpy()
    start = np.maximum(big[8:, 16:], 0).astype(np.float32)
    assert np.array_equal(got.view(np.uint32), oracle.matmul_f16(a, b, cin=np.ascontiguousarray(start)).view(np.uint32))
    got = launch(lib, 48, torch.zeros((m, n), dtype=torch.float32, device=DEV), dev(a), dev(b), dev(c0)).cpu().numpy()
    assert np.array_equal(got.view(np.uint32), oracle.matmul_f16(a, b, cin=oracle.matmul_f16(a, b)).view(np.uint32))
    m, k, n = 24, 64, 40
    ai, bi = r.integers(-128, 128, (m, k)).astype(np.int8), r.integers(-128, 128, (k, n)).astype(np.int8)
    ci = r.integers(-10 ** 6, 10 ** 6, (m, n)).astype(np.int32)
    got = launch(lib, 49, torch.zeros((m, n), dtype=torch.int32, device=DEV), dev(ai), dev(bi), dev(ci)).cpu().numpy()
    assert np.array_equal(got, oracle.matmul_i8(ai, bi, cin=ci))


def test_treshape_aliases_the_storage(lib):
    src = np.arange(1024, dtype=np.float32).reshape(16, 64)
    got = launch(lib, 50, torch.zeros((8, 128), dtype=torch.float32, device=DEV), dev(src)).cpu().numpy()
    assert np.array_equal(got, src.reshape(8, 128))


def test_tassign_outside_the_region_sets_the_status_word(lib):
    """An address past the tile's region, or one that is not 16-byte aligned, leaves status 1 behind (sticky until it is
    reset); the core itself carries on at offset 0, so the copy still completes."""
    src = np.arange(256, dtype=np.float32).reshape(8, 32)
    for addr in (40 * 1024, 40 * 1024 - 512, 8):  # past the end; end of the tile past the end; misaligned
        assert lib.pto_boundary_reset_status() == 0
        got = launch(lib, 60, torch.zeros((8, 32), dtype=torch.float32, device=DEV), dev(src), arg=addr, status=1).cpu().numpy()
        assert np.array_equal(got, src)
    assert lib.pto_boundary_reset_status() == 0
    got = launch(lib, 60, torch.zeros((8, 32), dtype=torch.float32, device=DEV), dev(src), arg=40 * 1024 - 1024, status=0).cpu().numpy()
    assert np.array_equal(got, src)
