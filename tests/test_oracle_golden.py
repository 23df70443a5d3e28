"""The plain-C oracle against (1) fixtures the compiled reference produced (tests/golden/pto_golden.npz),
(2) the reference tests' own known answers, restated, and (3) what the mathematics fixes independently
(IEEE conversions of numpy/torch, exact integer identities, closed forms).  No GPU, no reference tree needed."""
import numpy as np
import pytest
import torch

from oracle import binding as ob


def bits(x):
    return np.ascontiguousarray(x).view(np.uint32)


# ---------------------------------------------------------------- conversions
def test_f16_conversion_matches_ieee(oracle):
    allh = np.arange(65536, dtype=np.uint16)
    f = allh.view(np.float16).astype(np.float32)
    got = np.array([oracle.lib.pto_f16_to_f32(int(h)) for h in allh], np.float32)
    ok = (bits(got) == bits(f)) | (np.isnan(got) & np.isnan(f))
    assert ok.all()
    # every rounding boundary between adjacent halves, and the values just beside it
    fin = allh[(allh & 0x7C00) != 0x7C00]
    v = np.sort(fin.view(np.float16).astype(np.float64))
    mids = ((v[:-1] + v[1:]) / 2).astype(np.float32)
    r = np.random.default_rng(0)
    probe = np.concatenate([mids, np.nextafter(mids, np.float32(-1e30)), np.nextafter(mids, np.float32(1e30)),
                            (r.standard_normal(20000) * 10 ** r.uniform(-9, 6, 20000)).astype(np.float32),
                            np.array([65504, 65519.99, 65520, 1e9, -1e9, np.inf, -np.inf, 0.0, -0.0, 2 ** -25,
                                      2 ** -24, 1e-45], np.float32)])
    with np.errstate(over="ignore"):
        want = probe.astype(np.float16).view(np.uint16)
    assert np.array_equal(oracle.f32_to_f16(probe), want)
    assert oracle.lib.pto_f32_to_f16(float("nan")) & 0x7C00 == 0x7C00 and oracle.lib.pto_f32_to_f16(float("nan")) & 0x3FF


def test_bf16_conversion_matches_torch(oracle):
    r = np.random.default_rng(1)
    probe = np.concatenate([(r.standard_normal(30000) * 10 ** r.uniform(-20, 20, 30000)).astype(np.float32),
                            np.array([0.0, -0.0, np.inf, -np.inf, 1.0, 1.00390625, 1.01171875, 3.3895314e38, 3.4e38],
                                     np.float32)])
    # exact ties on the 16th mantissa bit
    base = (r.integers(0, 2 ** 15, 5000).astype(np.uint32) << 16) | 0x8000
    probe = np.concatenate([probe, base.view(np.float32)])
    probe = probe[np.isfinite(probe) | np.isinf(probe)]
    want = torch.from_numpy(probe.copy()).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(oracle.f32_to_bf16(probe), want)
    nan = oracle.lib.pto_f32_to_bf16(float("nan"))
    assert (nan & 0x7F80) == 0x7F80 and (nan & 0x7F)


def test_e4m3_decode_is_the_ocp_table(oracle, golden):
    dec = oracle.mx_decode_table(ob.E4M3)
    for code in range(256):
        e, m, s = (code >> 3) & 15, code & 7, -1.0 if code & 0x80 else 1.0
        if (code & 0x7F) == 0x7F:
            assert np.isnan(dec[code])
        else:
            want = s * (m / 8 * 2.0 ** -6 if e == 0 else (1 + m / 8) * 2.0 ** (e - 7))
            assert dec[code] == want
    assert dec[0x7E] == 448.0
    e2m1 = oracle.mx_decode_table(ob.E2M1)[:16]
    assert list(e2m1[:8]) == [0, 0.5, 1, 1.5, 2, 3, 4, 6] and list(e2m1[9:]) == [-0.5, -1, -1.5, -2, -3, -4, -6]
    assert e2m1[8] == 0 and not np.signbit(e2m1[8])  # the reference decodes fp4 "-0" to +0
    e8 = oracle.mx_decode_table(ob.E8M0)
    assert e8[127] == 1.0 and e8[0] == 2.0 ** -127 and e8[255] == 2.0 ** 128 and e8[130] == 8.0
    for typ, nm in enumerate(("e4m3", "e5m2", "e2m1", "e1m2", "e8m0")):
        want = golden[f"decode_{nm}"]
        got = oracle.mx_decode_table(typ)[: len(want)]
        assert np.array_equal(np.isnan(want), np.isnan(got))
        assert np.array_equal(np.nan_to_num(want), np.nan_to_num(got))
        assert np.array_equal(np.signbit(want), np.signbit(got))


def test_encode_fixtures(oracle, golden):
    vals = golden["encode_vals"]
    for t in range(5):
        got = [oracle.lib.pto_mx_encode_trunc(t, float(v)) for v in vals]
        assert np.array_equal(golden["encode_trunc"][t], np.array(got, np.uint8)), t
    for ti, t in enumerate((0, 1)):
        for mode in range(7):
            for sat in (0, 1):
                got = [oracle.lib.pto_fp8_encode_round(t, float(v), mode, sat) for v in vals]
                assert np.array_equal(golden["encode_round_fp8"][ti, mode, sat], np.array(got, np.uint8))
    for ti, t in enumerate((2, 3)):
        for mode in range(7):
            got = [oracle.lib.pto_fp4_encode_round(t, float(v), mode) for v in vals]
            assert np.array_equal(golden["encode_round_fp4"][ti, mode], np.array(got, np.uint8))


def test_fp8_rint_encode_is_nearest_even(oracle):
    """RINT + saturation must pick the nearest representable value (ties to even mantissa)."""
    dec = oracle.mx_decode_table(ob.E4M3)[:0x7F]
    r = np.random.default_rng(2)
    for v in np.concatenate([r.uniform(-460, 460, 3000), r.standard_normal(3000) * 0.01]):
        code = oracle.lib.pto_fp8_encode_round(ob.E4M3, float(v), ob_mode_rint := 1, 1)
        d = np.abs(dec - abs(v))
        assert d[code & 0x7F] == d.min(), (v, code)


# ---------------------------------------------------------------- addressing
TILE_KINDS = {0: (64, 128, 0, 1, 512, 2, 0), 1: (64, 128, 1, 2, 512, 2, 0), 2: (64, 128, 0, 1, 512, 2, 0),
              3: (64, 128, 1, 2, 512, 2, 0), 4: (64, 128, 0, 1, 1024, 4, 0), 5: (64, 128, 0, 1, 512, 1, 0),
              6: (64, 128, 0, 1, 512, 1, 1), 7: (64, 8, 1, 1, 32, 1, 0), 8: (8, 64, 0, 2, 32, 1, 0),
              9: (64, 128, 1, 0, 512, 4, 0), 10: (64, 128, 0, 0, 512, 4, 0), 11: (64, 128, 0, 1, 512, 4, 0)}


@pytest.mark.parametrize("kind", sorted(TILE_KINDS))
def test_tile_offset_fixtures(oracle, golden, kind):
    assert np.array_equal(golden[f"tile_offset_{kind}"], oracle.tile_offsets(*TILE_KINDS[kind]))


def test_nz_offset_closed_form(oracle):
    """Mat NZ for fp16: 16x16 fractals, fractal columns outermost: (c/16)*rows*16 + r*16 + c%16."""
    got = oracle.tile_offsets(64, 128, 0, 1, 512, 2, 0)
    r, c = np.meshgrid(np.arange(64), np.arange(128), indexing="ij")
    assert np.array_equal(got, (c // 16) * 64 * 16 + r * 16 + c % 16)


def test_mx_scale_layout_fixtures(oracle, golden):
    for lid, layout in enumerate((ob.MX_A_ZZ, ob.MX_A_ND, ob.MX_A_DN, ob.MX_B_NN, ob.MX_B_ND, ob.MX_B_DN)):
        rows, cols = (32, 8) if lid < 3 else (8, 32)
        assert np.array_equal(golden[f"mx_scale_offset_{lid}"], oracle.mx_scale_offsets(layout, rows, cols))
    # the two "natural" layouts are plain row-major [M][K/32] and [N][K/32]
    assert np.array_equal(oracle.mx_scale_offsets(ob.MX_A_ND, 32, 8), np.arange(256).reshape(32, 8))
    assert np.array_equal(oracle.mx_scale_offsets(ob.MX_B_DN, 8, 32), np.arange(256).reshape(32, 8).T)


# ---------------------------------------------------------------- TMATMUL
GLOBAL_CASES = {0: (ob.ND, 2 * 3 * 4 * 8, 16), 1: (ob.DN, 8, 2 * 3 * 4 * 16), 2: (ob.NZ, 48, 32)}


@pytest.mark.parametrize("which", sorted(GLOBAL_CASES))
def test_global_offset_fixtures(oracle, golden, which):
    """5-D GlobalTensors with every outer dimension above 1 and padded strides, as the compiled reference maps them."""
    layout, rows, cols = GLOBAL_CASES[which]
    sh, st = golden[f"global_shape_{which}"], golden[f"global_stride_{which}"]
    got = oracle.global_offsets(layout, sh, st, rows, cols)
    assert np.array_equal(golden[f"global_offset_{which}"], got)
    assert len(np.unique(got)) == got.size


def test_global_offset_nd_is_numpy_strides(oracle):
    """ND: the logical row runs over dims 0..3 in C order, so the map is numpy's own strided view."""
    sh, st = np.array([2, 3, 4, 8, 16]), np.array([2000, 650, 160, 20, 1])
    buf = np.arange(2 * 2000)
    view = np.lib.stride_tricks.as_strided(buf, sh, st * buf.itemsize).reshape(-1, 16)
    assert np.array_equal(view, oracle.global_offsets(ob.ND, sh, st, 2 * 3 * 4 * 8, 16))
    # DN: rows are dim 3, columns run over dims 0, 1, 2, 4
    st = np.array([2000, 650, 160, 1, 10])
    view = np.lib.stride_tricks.as_strided(buf, sh, st * buf.itemsize).transpose(3, 0, 1, 2, 4).reshape(8, -1)
    assert np.array_equal(view, oracle.global_offsets(ob.DN, sh, st, 8, 2 * 3 * 4 * 16))


def test_layout_2d_fixtures(oracle, golden):
    for lay in (ob.ND, ob.DN, ob.NZ):
        for rows, cols in ((32, 64), (48, 16)):
            sh, st = oracle.layout_2d(lay, rows, cols, c0=8)  # 32-byte C0 of float
            assert np.array_equal(golden[f"layout2d_{lay}_{rows}x{cols}"], np.stack([sh, st])), (lay, rows, cols)
            offs = oracle.global_offsets(lay, sh, st, rows, cols)
            assert sorted(offs.ravel().tolist()) == list(range(rows * cols))


def test_reorder_exp_zz_fixture_and_layout_identity(oracle, golden):
    assert np.array_equal(golden["zz_reordered"], oracle.reorder_exp_zz(golden["zz_exp"]))
    # the reordered stream is the MX_A_ZZ global layout of the same [rows][groups] matrix
    e = golden["zz_exp"]
    offs = oracle.mx_scale_offsets(ob.MX_A_ZZ, *e.shape)
    assert np.array_equal(oracle.reorder_exp_zz(e)[offs], e)


def test_matmul_reference_test_distribution_is_exact(oracle, golden):
    """tests/cpu/st/testcase/tmatmul/gen_data.py draws randint(1,5): every partial sum is an exact integer."""
    for name in ("case1", "case3_splitk", "gemv"):
        a, b = golden[f"mm_f16_int_{name}_a"], golden[f"mm_f16_int_{name}_b"]
        exact = a.view(np.float16).astype(np.int64) @ b.view(np.float16).astype(np.int64)
        got = oracle.matmul_f16(a, b)
        assert np.array_equal(got, exact.astype(np.float32))
        assert np.array_equal(golden[f"mm_f16_int_{name}_out"], got)


def test_matmul_fixtures(oracle, golden):
    g = golden
    assert np.array_equal(bits(g["mm_f16_out"]), bits(oracle.matmul_f16(g["mm_f16_a"], g["mm_f16_bt"], b_dn=True)))
    assert np.array_equal(bits(g["mm_f16_out_acc"]),
                          bits(oracle.matmul_f16(g["mm_f16_a"], g["mm_f16_bt"], cin=g["mm_f16_cin"], b_dn=True)))
    acc = oracle.matmul_f16(g["mm_f16_a"], g["mm_f16_bt"], b_dn=True)
    assert np.array_equal(g["mm_f16_out_f16"], oracle.store_f32(acc, ob.ST_F16))
    assert np.array_equal(g["mm_f16_out_f16_relu"], oracle.store_f32(acc, ob.ST_F16, relu=True))
    assert np.array_equal(bits(g["mm_f32_out"]), bits(oracle.matmul_f32(g["mm_f32_a"], g["mm_f32_b"])))
    assert np.array_equal(g["mm_i8_out"], oracle.matmul_i8(g["mm_i8_a"], g["mm_i8_bt"], b_dn=True))
    assert np.array_equal(g["mm_i8_out_acc"],
                          oracle.matmul_i8(g["mm_i8_a"], g["mm_i8_bt"], cin=g["mm_i8_cin"], b_dn=True))
    assert np.array_equal(bits(g["mm_e4m3_out"]), bits(oracle.matmul_fp8(g["mm_e4m3_a"], g["mm_e4m3_b"])))


def test_matmul_bf16_equals_f32_path_on_bf16_values(oracle, golden):
    a, bt = golden["mm_bf16rep_a"], golden["mm_bf16rep_bt"]
    a16 = (bits(a) >> 16).astype(np.uint16)
    b16 = (bits(bt) >> 16).astype(np.uint16)
    got = oracle.matmul_bf16(a16, b16, b_dn=True)
    assert np.array_equal(bits(golden["mm_bf16rep_out"]), bits(got))
    f64 = a.astype(np.float64) @ bt.astype(np.float64).T
    assert np.abs(got - f64).max() <= 1e-5 * np.abs(f64).max() + 1e-7


def test_matmul_accumulates_in_k_order_fused(oracle):
    """tmatmul_layout 'AccumulatesFromExistingFp32Value': accIn = 1e8, sixteen fused += 1*1 leave 1e8 exactly."""
    ones = np.ones((16, 16), np.float32)
    out = oracle.matmul_f32(ones, ones, cin=np.full((16, 16), 1e8, np.float32))
    assert (out == np.float32(1e8)).all()  # dot-then-add would give 100000016
    a = np.array([[1.0 + 2.0 ** -12]], np.float32)
    got = oracle.matmul_f32(a, a, cin=np.array([[-1.0]], np.float32))
    assert got[0, 0] == np.float32(2.0 ** -11 + 2.0 ** -24)  # only a fused multiply-add keeps the 2^-24 term


def test_matmul_i8_wraps_mod_2_32(oracle):
    r = np.random.default_rng(3)
    a = r.integers(-128, 128, (9, 700)).astype(np.int8)
    b = r.integers(-128, 128, (700, 11)).astype(np.int8)
    cin = np.full((9, 11), 2 ** 31 - 5, np.int32)
    want = (a.astype(np.int64) @ b.astype(np.int64) + cin).astype(np.uint64).astype(np.uint32).view(np.int32)
    want = ((a.astype(np.int64) @ b.astype(np.int64) + cin) & 0xFFFFFFFF).astype(np.uint32).view(np.int32)
    assert np.array_equal(oracle.matmul_i8(a, b, cin=cin), want)


def test_bias_is_added_after_the_k_loop(oracle):
    a = np.full((2, 3), 1e8, np.float32)
    b = np.full((3, 2), 1.0, np.float32)
    bias = np.array([1.0, 16.0], np.float32)
    out = oracle.matmul_f32(a, b, bias=bias)
    assert out[0, 0] == np.float32(3e8) + np.float32(1.0) and out[0, 1] == np.float32(np.float32(3e8) + 16.0)


# ---------------------------------------------------------------- TMATMUL_MX
@pytest.mark.parametrize("tname,typ", [("e4m3", ob.E4M3), ("e5m2", ob.E5M2), ("e2m1", ob.E2M1), ("e1m2", ob.E1M2)])
def test_matmul_mx_fixtures(oracle, golden, tname, typ):
    g = golden
    m, k, n = 48, 192, 80
    a, bt, sa, sb = (g[f"mx_{tname}_{x}"] for x in ("a", "bt", "sa", "sb"))
    for fmt, (la, lb) in enumerate(((ob.MX_A_ZZ, ob.MX_B_NN), (ob.MX_A_ND, ob.MX_B_ND), (ob.MX_A_DN, ob.MX_B_DN))):
        got = oracle.matmul_mx(a, bt, sa, sb, m, k, n, typ, typ, la, lb, b_dn=True)
        assert np.array_equal(bits(g[f"mx_{tname}_out_fmt{fmt}"]), bits(got)), fmt
    got = oracle.matmul_mx(a, bt, sa, sb, m, k, n, typ, typ, ob.MX_A_DN, ob.MX_B_DN, b_dn=True,
                           cin=g[f"mx_{tname}_cin"])
    assert np.array_equal(bits(g[f"mx_{tname}_out_acc_fmt2"]), bits(got))


def _unpack(codes, typ, rows, cols, oracle):
    tab = oracle.mx_decode_table(typ)
    if typ in (ob.E2M1, ob.E1M2):
        lo, hi = codes & 0xF, codes >> 4
        full = np.stack([lo, hi], -1).reshape(rows, cols)
        return tab[full]
    return tab[codes]


@pytest.mark.parametrize("typ", [ob.E4M3, ob.E2M1])
def test_matmul_mx_closed_form(oracle, typ):
    """tmatmul_mx/gen_data.py: golden = matmul(x1 * 2^(s1-127), x2 * 2^(s2-127)) in float64, eps 1e-3."""
    r = np.random.default_rng(4)
    m, k, n = 32, 128, 48
    packed = typ == ob.E2M1
    a = r.integers(0, 256, (m, k // 2 if packed else k)).astype(np.uint8)
    bt = r.integers(0, 256, (n, k // 2 if packed else k)).astype(np.uint8)
    if not packed:
        a[(a & 0x7F) == 0x7F] = 0
        bt[(bt & 0x7F) == 0x7F] = 0
    sa = r.integers(125, 130, (m, k // 32)).astype(np.uint8)
    sb = r.integers(125, 130, (n, k // 32)).astype(np.uint8)
    av = _unpack(a, typ, m, k, oracle) * np.repeat(2.0 ** (sa.astype(np.float64) - 127), 32, 1)
    bv = _unpack(bt, typ, n, k, oracle) * np.repeat(2.0 ** (sb.astype(np.float64) - 127), 32, 1)
    want = av @ bv.T
    got = oracle.matmul_mx(a, bt, sa, sb, m, k, n, typ, typ)
    assert np.abs(got - want).max() <= 1e-3 * np.abs(want).max()
    # all scales = 127 and E4M3 operands: block scaling drops out and the plain fp8 TMATMUL must agree
    if typ == ob.E4M3:
        one = np.full_like(sa, 127)
        plain = oracle.matmul_fp8(a, bt, b_dn=True)
        mx1 = oracle.matmul_mx(a, bt, one, np.full_like(sb, 127), m, k, n, typ, typ)
        assert np.abs(plain - mx1).max() <= 1e-5 * np.abs(plain).max()


# ---------------------------------------------------------------- fix-pipe stores
def test_quant_word_known_answers(oracle):
    """tquantmode/main.cpp: unit tensor word = (127 << 10) << 13; scalar 0.5 * 2.0 = 1.0; saturation to 65504."""
    unit = (127 << 10) << 13
    assert oracle.lib.pto_quant_word_scale(unit, 1) == 1.0
    half_word = int(np.float32(0.5).view(np.uint32))
    assert oracle.lib.pto_quant_word_scale(half_word, 0) == 0.5
    out = oracle.store_quant(np.array([[3.0]], np.float32), ob.ST_F16, np.array([unit], np.uint64), 1)
    assert out.view(np.float16)[0, 0] == 3.0
    out = oracle.store_quant(np.array([[2.0]], np.float32), ob.ST_F16, np.array([half_word], np.uint64), 0)
    assert out.view(np.float16)[0, 0] == 1.0
    out = oracle.store_quant(np.array([[1e9]], np.float32), ob.ST_F16, np.array([unit], np.uint64), 1, saturate_inf=1)
    assert out.view(np.float16)[0, 0] == 65504.0
    out = oracle.store_quant(np.array([[1e9]], np.float32), ob.ST_F16, np.array([unit], np.uint64), 1, saturate_inf=0)
    assert out.view(np.float16)[0, 0] == 65504.0  # finite input is clamped in either mode
    out = oracle.store_quant(np.array([[1 << 20]], np.int32), ob.ST_F16, np.array([unit], np.uint64), 1)
    assert out.view(np.float16)[0, 0] == 65504.0


def test_store_quant_fixtures(oracle, golden):
    g = golden
    for per_col in (0, 1):
        for relu in (0, 1):
            k = f"{per_col}_{relu}"
            assert np.array_equal(g["st_f32_i8_" + k], oracle.store_quant(g["st_accf"], ob.ST_I8, g[f"st_w8_{per_col}"], per_col, relu))
            assert np.array_equal(g["st_f32_u8_" + k], oracle.store_quant(g["st_accf"], ob.ST_U8, g[f"st_wu_{per_col}"], per_col, relu))
            assert np.array_equal(g["st_i32_i8_" + k], oracle.store_quant(g["st_acci"], ob.ST_I8, g[f"st_wi_{per_col}"], per_col, relu))
            assert np.array_equal(g["st_f32_f16_" + k], oracle.store_quant(g["st_accf"], ob.ST_F16, g[f"st_wh_{per_col}"], per_col, relu))
            assert np.array_equal(g["st_i32_f16_" + k], oracle.store_quant(g["st_acci"], ob.ST_F16, g[f"st_wh_{per_col}"], per_col, relu))


# ---------------------------------------------------------------- TQUANT / TDEQUANT
def test_tquant_edge_known_answers(oracle):
    """tquant/main.cpp 'MxFpNvExponentScalingEdges' / 'MxFpOcpExponentScalingInfEdges'."""
    L = oracle.lib
    inf, nan = float("inf"), float("nan")
    assert L.pto_shared_exponent(ob.NV_FP4, inf) == 0xFE and L.pto_group_scaling(ob.NV_FP4, inf, 0xFE) == 2.0 ** -127
    assert L.pto_shared_exponent(ob.NV_FP4, 0.0) == 0 and L.pto_group_scaling(ob.NV_FP4, 0.0, 0) == 2.0 ** 127
    assert L.pto_shared_exponent(ob.NV_FP4, nan) == 0xFF and np.isnan(L.pto_group_scaling(ob.NV_FP4, nan, 0xFF))
    assert L.pto_shared_exponent(ob.NV_FP8, inf) == 0xFE and L.pto_group_scaling(ob.NV_FP8, inf, 0xFE) == 2.0 ** -127
    assert L.pto_shared_exponent(ob.OCP_FP4, inf) == 0xFD and L.pto_group_scaling(ob.OCP_FP4, inf, 0xFD) == 2.0 ** -126
    assert L.pto_encode_e2m1_magic(inf) == 0x7 and L.pto_encode_e2m1_magic(-inf) == 0xF
    assert L.pto_shared_exponent(ob.OCP_FP4, nan) == 0xFF and np.isnan(L.pto_group_scaling(ob.OCP_FP4, nan, 0xFF))
    assert L.pto_shared_exponent(ob.OCP_FP8, inf) == 0xF7 and L.pto_group_scaling(ob.OCP_FP8, inf, 0xF7) == 2.0 ** -120
    assert L.pto_shared_exponent(ob.OCP_FP8, nan) == 0xFF and np.isnan(L.pto_group_scaling(ob.OCP_FP8, nan, 0xFF))


def test_e4m3_encode_is_exhaustive_nearest(oracle):
    """tquant/main.cpp's in-test encoder: nearest of the 254 finite codes, ties to the even code, then lower code."""
    dec = np.array([oracle.lib.pto_mx_decode(ob.E4M3, c) for c in range(256)], np.float32)
    finite = np.array([c for c in range(256) if (c & 0x7F) != 0x7F])
    r = np.random.default_rng(5)
    pos = dec[:0x7F]
    mids = ((pos[:-1].astype(np.float64) + pos[1:]) / 2).astype(np.float32)
    probe = np.concatenate([r.uniform(-500, 500, 4000).astype(np.float32), (r.standard_normal(4000) * 0.02).astype(np.float32),
                            mids, -mids, pos, -pos, np.array([0.0, -0.0, 1e-30, -1e-30], np.float32)])
    for v in probe:
        clipped = np.clip(v, np.float32(-448), np.float32(448))
        dist = np.abs(dec[finite] - clipped)
        cand = finite[dist == dist.min()]
        even = cand[cand % 2 == 0]
        want = int((even if len(even) else cand).min())
        assert oracle.lib.pto_encode_e4m3fn(float(v), 0) == want, v


def test_e2m1_magic_is_round_to_nearest_even_on_the_grid(oracle):
    grid = np.array([0, 0.5, 1, 1.5, 2, 3, 4, 6], np.float32)
    r = np.random.default_rng(6)
    for v in np.concatenate([r.uniform(-7, 7, 5000).astype(np.float32), grid, -grid, (grid[:-1] + grid[1:]) / 2]):
        a = min(abs(float(v)), 6.0)
        d = np.abs(grid - a)
        cand = np.flatnonzero(d == d.min())
        want = int(cand[cand % 2 == 0][0] if len(cand) > 1 else cand[0])
        got = oracle.lib.pto_encode_e2m1_magic(float(v))
        assert (got & 7) == want and bool(got & 8) == bool(np.signbit(v)), v


def test_tquant_fixtures(oracle, golden):
    g = golden
    for sid in (2, 5):
        for si in range(3):
            src = g[f"tq_src_{sid}_{si}"]
            for alg in range(4):
                for axis in ((1, 0) if sid == 5 else (1,)):
                    key = f"tq_{sid}_{si}_{alg}_{axis}"
                    codes, exp, mx, sc = oracle.tquant_mx(src, alg, axis)
                    assert np.array_equal(g[key + "_codes"], codes), key
                    assert np.array_equal(g[key + "_exp"], exp), key
                    for want, got in ((g[key + "_max"], mx), (g[key + "_scaling"], sc)):
                        assert np.array_equal(bits(want) & 0xFFBFFFFF, bits(got) & 0xFFBFFFFF), key
    assert np.array_equal(g["q8_sym"], oracle.tquant_int8(g["q8_src"], g["q8_scale"]))
    assert np.array_equal(g["q8_asym"], oracle.tquant_int8(g["q8_src"], g["q8_scale"], g["q8_off"]))
    for nm in ("i8", "i16", "i32"):
        got = oracle.tdequant(g[f"dq_src_{nm}"], g["q8_scale"], g["q8_off"])
        assert np.array_equal(bits(g[f"dq_out_{nm}"]), bits(got))


@pytest.mark.parametrize("alg", [ob.OCP_FP8, ob.NV_FP8, ob.OCP_FP4, ob.NV_FP4])
def test_tquant_bf16_source_equals_f32_source_on_bf16_values(oracle, alg):
    """The bf16 source path may differ from fp32 only through rounding to bf16 (group maximum taken on bf16 bits,
    scaled value re-rounded): on inputs that already are bf16 values, scaled by a power of two, nothing rounds."""
    r = np.random.default_rng(31)
    src = (r.standard_normal((32, 256)) * 10.0 ** r.uniform(-2, 2, (32, 1))).astype(np.float32)
    src = (src.view(np.uint32) & 0xFFFF0000).view(np.float32)
    a = oracle.tquant_mx(src, alg, 1, ob.SRC_F32)
    b = oracle.tquant_mx(src, alg, 1, ob.SRC_BF16)
    for x, y in zip(a, b):
        assert np.array_equal(bits(x) if x.dtype == np.float32 else x, bits(y) if y.dtype == np.float32 else y)


def test_tquant_round_trip_error_bound(oracle):
    """Quantise -> dequantise stays within half a grid step of the source (OCP FP8, finite data)."""
    r = np.random.default_rng(7)
    src = r.standard_normal((8, 256)).astype(np.float32)
    codes, exp, _, _ = oracle.tquant_mx(src, ob.OCP_FP8)
    dec = oracle.mx_decode_table(ob.E4M3)[codes] * np.repeat(2.0 ** (exp.astype(np.float64) - 127), 32, 1)
    sc = np.repeat(2.0 ** (exp.astype(np.float64) - 127), 32, 1)
    # three mantissa bits: half an ulp is 2^-4 relative in the normal range, 2^-10 (scaled) below it; the OCP
    # exponent (floor(log2 max) - 8) lets scaled values in (448, 512) saturate to 448, at most 12.5 % off
    scaled = np.abs(src) / sc
    bound = np.where(scaled > 448, np.abs(src) * 0.125, np.maximum(np.abs(src) * 2.0 ** -4, sc * 2.0 ** -10))
    assert (np.abs(dec - src) <= bound + 1e-12).all()
    # int8 symmetric: |q / s - x| <= 0.5 / s inside the clamp range
    scale = np.full(8, 20.0, np.float32)
    q = oracle.tquant_int8(src, scale)
    assert (np.abs(q / 20.0 - src)[np.abs(src) < 6] <= 0.5 / 20 + 1e-6).all()


def test_tdequant_closed_form(oracle):
    """tdequant/gen_data.py: (x - offset[i]) * scale[i] per row, in float32."""
    r = np.random.default_rng(8)
    q = r.integers(-128, 128, (16, 64)).astype(np.int8)
    scale = r.uniform(0.1, 2, 16).astype(np.float32)
    off = r.uniform(-5, 5, 16).astype(np.float32)
    want = (q.astype(np.float32) - off[:, None]) * scale[:, None]
    assert np.array_equal(bits(want), bits(oracle.tdequant(q, scale, off)))


def test_parameter_tile_fixtures(oracle, golden):
    """Parameter tiles as the reference reads them: TDEQUANT clamps the column, TQUANT INT8 reads column 0 and clamps
    the row (vectors from the compiled reference); plus the numpy closed form, which a swapped clamp would fail."""
    g = golden
    for pc in (1, 3, 8):
        got = oracle.tdequant_para(g["dqp_src"], g[f"dqp_scale_{pc}"], g[f"dqp_off_{pc}"])
        assert np.array_equal(bits(got), bits(g[f"dqp_out_{pc}"])), pc
        col = np.minimum(np.arange(64), pc - 1)
        want = (g["dqp_src"].astype(np.float32) - g[f"dqp_off_{pc}"][:, col]) * g[f"dqp_scale_{pc}"][:, col]
        assert np.array_equal(bits(got), bits(want))
    for pr in (1, 5, 16):
        sc, of = g[f"q8p_scale_{pr}"], g[f"q8p_off_{pr}"]
        assert np.array_equal(oracle.tquant_int8_para(g["q8p_src"], sc), g[f"q8p_sym_{pr}"]), pr
        assert np.array_equal(oracle.tquant_int8_para(g["q8p_src"], sc, of), g[f"q8p_asym_{pr}"]), pr
        row = np.minimum(np.arange(16), pr - 1)
        want = np.clip(np.rint(g["q8p_src"] * sc[row][:, None]), -128, 127).astype(np.int8)
        assert np.array_equal(g[f"q8p_sym_{pr}"], want)


def test_store_int16_shift_mode(oracle, golden):
    """SHIFTS322S16: (int16)(acc >> (bits 32..35 + 1)), narrowed before the clamp (so it wraps), then relu: the
    compiled reference's outputs and the closed form."""
    g = golden
    acc, words = g["s16_acc"], g["s16_words"]
    for per_col in (0, 1):
        w = words if per_col else words[:1]
        shift = ((w >> np.uint64(32)) & np.uint64(15)).astype(np.int64) + 1
        want = (acc.astype(np.int64) >> (shift[None, :] if per_col else shift[0])).astype(np.int16)
        for relu in (0, 1):
            got = oracle.store_quant(acc, ob.ST_I16, w, per_col, relu)
            assert np.array_equal(got, g[f"s16_out_{per_col}_{relu}"]), (per_col, relu)
            assert np.array_equal(got, np.maximum(want, 0) if relu else want)
    assert (g["s16_out_0_0"] < 0).any() and len(np.unique(g["s16_out_1_0"])) > 100


def test_store_quant_bf16_target_against_torch(oracle):
    """QF322BF16_PRE / QS322BF16_PRE: the product acc * scale rounded to bfloat16 (the compiled reference cannot pin
    this target: its bfloat16_t is a half in this build), checked against float32 multiply + torch's bf16 rounding."""
    import torch
    r = np.random.default_rng(12)
    accf = (r.standard_normal((24, 40)) * 300).astype(np.float32)
    acci = r.integers(-2 ** 24, 2 ** 24, (24, 40)).astype(np.int32)
    scales = r.uniform(0.001, 3.0, 40).astype(np.float32)
    words = np.array([int(s.view(np.uint32)) for s in scales], np.uint64)
    for acc in (accf, acci):
        for relu in (False, True):
            prod = acc.astype(np.float32) * scales[0]
            prod = np.maximum(prod, 0) if relu else prod
            want = torch.from_numpy(prod).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
            assert np.array_equal(oracle.store_quant(acc, ob.ST_BF16, words[:1], False, relu), want)


# ---------------------------------------------------------------- the CPU-simulator-shaped baseline walk
def test_sim_tiled_equals_one_shot(oracle):
    r = np.random.default_rng(9)
    a = r.uniform(-1, 1, (256, 192)).astype(np.float16).view(np.uint16)
    b = r.uniform(-1, 1, (192, 128)).astype(np.float16).view(np.uint16)
    out, threads = oracle.sim_gemm_tiled(a, b, 0, ob.ST_F32, b_dn=False)
    assert threads >= 1
    assert np.array_equal(bits(out), bits(oracle.matmul_f16(a, b)))
    bt = np.ascontiguousarray(b.T)
    out2, _ = oracle.sim_gemm_tiled(a, bt, 0, ob.ST_F32, b_dn=True, max_threads=2)
    assert np.array_equal(bits(out2), bits(out))
    ai = r.integers(-127, 128, (130, 200)).astype(np.int8)
    bi = r.integers(-127, 128, (70, 200)).astype(np.int8)
    outi, _ = oracle.sim_gemm_tiled(ai, bi, 2, ob.ST_I32, b_dn=True)
    assert np.array_equal(outi, oracle.matmul_i8(ai, bi, b_dn=True))
    a8 = r.integers(0, 120, (128, 128)).astype(np.uint8)
    b8 = r.integers(0, 120, (128, 128)).astype(np.uint8)
    sa = r.integers(120, 134, (128, 4)).astype(np.uint8)
    sb = r.integers(120, 134, (128, 4)).astype(np.uint8)
    outm, _ = oracle.sim_gemm_mx_tiled(a8, b8, sa, sb, 128, 128, 128, ob.E4M3, ob.E4M3, ob.ST_F32)
    assert np.array_equal(bits(outm), bits(oracle.matmul_mx(a8, b8, sa, sb, 128, 128, 128, ob.E4M3, ob.E4M3)))
