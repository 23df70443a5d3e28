"""The plain-C oracle against the compiled reference CPU simulator, bit for bit.

Runs only where oracle/_ref/libptoref.so exists (it is built from the reference's own headers where the reference
tree is mounted).  The same comparisons are frozen as fixtures in tests/golden/ so they also run without it.
"""
import numpy as np
import pytest

from oracle import binding as ob


def _rng(seed):
    return np.random.default_rng(seed)


def _f16(x):
    return np.asarray(x, np.float32).astype(np.float16).view(np.uint16)


@pytest.mark.parametrize("m,k,n,b_dn,kstep", [(40, 50, 60, False, 0), (128, 320, 64, False, 64), (6, 7, 8, True, 0),
                                              (1, 110, 50, False, 0), (33, 129, 47, True, 48)])
def test_matmul_f16(oracle, reflib, m, k, n, b_dn, kstep):
    r = _rng(m * 1000 + k)
    a = _f16(r.uniform(-1, 1, (m, k)))
    b = _f16(r.uniform(-1, 1, (n, k) if b_dn else (k, n)))
    ref = reflib.gemm("f16", a, b, b_dn=b_dn, kstep=kstep)
    got = oracle.matmul_f16(a, b, b_dn=b_dn)
    assert np.array_equal(ref.view(np.uint32), got.view(np.uint32))


def test_matmul_f16_with_acc_in(oracle, reflib):
    r = _rng(5)
    a = _f16(r.uniform(-1, 1, (32, 64)))
    b = _f16(r.uniform(-1, 1, (64, 48)))
    cin = r.uniform(-5, 5, (32, 48)).astype(np.float32)
    ref = reflib.gemm("f16", a, b, cin=cin)
    got = oracle.matmul_f16(a, b, cin=cin)
    assert np.array_equal(ref.view(np.uint32), got.view(np.uint32))


@pytest.mark.parametrize("m,k,n,b_dn", [(120, 110, 50, False), (1, 128, 64, False), (17, 33, 9, True)])
def test_matmul_f32_is_fused(oracle, reflib, m, k, n, b_dn):
    r = _rng(k)
    a = r.standard_normal((m, k)).astype(np.float32)
    b = r.standard_normal((n, k) if b_dn else (k, n)).astype(np.float32)
    ref = reflib.gemm("f32", a, b, b_dn=b_dn)
    got = oracle.matmul_f32(a, b, b_dn=b_dn)
    assert np.array_equal(ref.view(np.uint32), got.view(np.uint32))


@pytest.mark.parametrize("m,k,n,b_dn", [(6, 7, 8, False), (64, 512, 96, True), (130, 257, 33, False)])
def test_matmul_i8(oracle, reflib, m, k, n, b_dn):
    r = _rng(n)
    a = r.integers(-128, 128, (m, k)).astype(np.int8)
    b = r.integers(-128, 128, (n, k) if b_dn else (k, n)).astype(np.int8)
    cin = r.integers(-2**31, 2**31, (m, n)).astype(np.int32)
    for c in (None, cin):
        ref = reflib.gemm("i8", a, b, cin=c, b_dn=b_dn)
        got = oracle.matmul_i8(a, b, cin=c, b_dn=b_dn)
        assert np.array_equal(ref, got)


@pytest.mark.parametrize("kind,typ", [("e4m3", ob.E4M3), ("e5m2", ob.E5M2)])
def test_matmul_fp8(oracle, reflib, kind, typ):
    r = _rng(11)
    a = r.integers(0, 256, (48, 96)).astype(np.uint8)
    b = r.integers(0, 256, (96, 40)).astype(np.uint8)
    nan_inf = (lambda x: (x & 0x7F) == 0x7F) if typ == ob.E4M3 else (lambda x: (x & 0x7F) >= 0x7C)
    a[nan_inf(a)] = 0x3A
    b[nan_inf(b)] = 0x45
    ref = reflib.gemm(kind, a, b)
    got = oracle.matmul_fp8(a, b, a_type=typ, b_type=typ)
    assert np.array_equal(ref.view(np.uint32), got.view(np.uint32))


def _mx_codes(r, typ, rows, cols):
    if typ in (ob.E2M1, ob.E1M2):
        return r.integers(0, 256, (rows, cols // 2)).astype(np.uint8)
    x = r.integers(0, 256, (rows, cols)).astype(np.uint8)
    bad = (x & 0x7F) == 0x7F if typ == ob.E4M3 else (x & 0x7F) >= 0x7C
    x[bad] = 0x31
    return x


@pytest.mark.parametrize("typ", [ob.E4M3, ob.E5M2, ob.E2M1, ob.E1M2])
@pytest.mark.parametrize("fmt", [0, 1, 2])
@pytest.mark.parametrize("b_dn", [False, True])
def test_matmul_mx(oracle, reflib, typ, fmt, b_dn):
    r = _rng(typ * 10 + fmt)
    m, k, n = 32, 128, 64
    a = _mx_codes(r, typ, m, k)
    b = _mx_codes(r, typ, n, k) if b_dn else _mx_codes(r, typ, k, n)
    sa = r.integers(118, 136, m * k // 32).astype(np.uint8)
    sb = r.integers(118, 136, n * k // 32).astype(np.uint8)
    cin = r.standard_normal((m, n)).astype(np.float32)
    la = [ob.MX_A_ZZ, ob.MX_A_ND, ob.MX_A_DN][fmt]
    lb = [ob.MX_B_NN, ob.MX_B_ND, ob.MX_B_DN][fmt]
    for c in (None, cin):
        ref = reflib.gemm_mx(a, b, sa, sb, m, k, n, typ, fmt, b_dn, cin=c)
        got = oracle.matmul_mx(a, b, sa, sb, m, k, n, typ, typ, la, lb, b_dn=b_dn, cin=c)
        assert np.array_equal(ref.view(np.uint32), got.view(np.uint32))


def test_mx_decode_all_codes(oracle, reflib):
    for typ in range(5):
        for code in range(256 if typ in (0, 1, 4) else 16):
            a = reflib.lib.ref_mx_decode(typ, code)
            b = oracle.lib.pto_mx_decode(typ, code)
            assert (np.isnan(a) and np.isnan(b)) or (a == b and np.signbit(a) == np.signbit(b)), (typ, code, a, b)


def test_mx_encode(oracle, reflib):
    r = _rng(3)
    vals = np.concatenate([r.standard_normal(4000) * 10 ** r.uniform(-6, 5, 4000), [0.0, -0.0, np.inf, -np.inf],
                           np.ldexp(1.0, np.arange(-30, 20)), -np.ldexp(1.5, np.arange(-30, 20)),
                           np.arange(-8, 8, 0.125)])
    for typ in range(5):
        for v in vals:
            assert reflib.lib.ref_mx_encode_trunc(typ, float(v)) == oracle.lib.pto_mx_encode_trunc(typ, float(v)), \
                (typ, v)
    for typ in (0, 1):
        for mode in range(7):
            for sat in (0, 1):
                for v in list(vals) + [float("nan")]:
                    assert reflib.lib.ref_mx_encode_round(typ, float(v), mode, sat) == \
                        oracle.lib.pto_fp8_encode_round(typ, float(v), mode, sat), (typ, mode, sat, v)
    for typ in (2, 3):
        for mode in range(7):
            for v in vals:
                assert reflib.lib.ref_mx_encode_round(typ, float(v), mode, 0) == \
                    oracle.lib.pto_fp4_encode_round(typ, float(v), mode), (typ, mode, v)


TILE_KINDS = {  # ref kind -> (rows, cols, row_major, sfractal, sfractal_size, elem_bytes, packed2)
    0: (64, 128, 0, 1, 512, 2, 0), 1: (64, 128, 1, 2, 512, 2, 0), 2: (64, 128, 0, 1, 512, 2, 0),
    3: (64, 128, 1, 2, 512, 2, 0), 4: (64, 128, 0, 1, 1024, 4, 0), 5: (64, 128, 0, 1, 512, 1, 0),
    6: (64, 128, 0, 1, 512, 1, 1), 7: (64, 8, 1, 1, 32, 1, 0), 8: (8, 64, 0, 2, 32, 1, 0),
    9: (64, 128, 1, 0, 512, 4, 0), 10: (64, 128, 0, 0, 512, 4, 0), 11: (64, 128, 0, 1, 512, 4, 0),
}


@pytest.mark.parametrize("kind", sorted(TILE_KINDS))
def test_tile_offsets(oracle, reflib, kind):
    rows, cols = TILE_KINDS[kind][:2]
    got = oracle.tile_offsets(*TILE_KINDS[kind])
    ref = np.array([[reflib.lib.ref_tile_offset(kind, r, c) for c in range(cols)] for r in range(rows)])
    assert np.array_equal(ref, got)
    assert sorted(got.ravel().tolist()) == list(range(rows * cols))  # a layout is a bijection


@pytest.mark.parametrize("layout,ref_id", [(ob.MX_A_ZZ, 0), (ob.MX_A_ND, 1), (ob.MX_A_DN, 2), (ob.MX_B_NN, 3),
                                           (ob.MX_B_ND, 4), (ob.MX_B_DN, 5)])
def test_mx_scale_layouts(oracle, reflib, layout, ref_id):
    rows, cols = (32, 8) if ref_id < 3 else (8, 32)
    got = oracle.mx_scale_offsets(layout, rows, cols)
    ref = np.array([[reflib.lib.ref_mx_scale_offset(ref_id, rows, cols, r, c) for c in range(cols)]
                    for r in range(rows)])
    assert np.array_equal(ref, got)
    assert sorted(got.ravel().tolist()) == list(range(rows * cols))


@pytest.mark.parametrize("which,layout,rows,cols", [(0, ob.ND, 192, 16), (1, ob.DN, 8, 384), (2, ob.NZ, 48, 32)])
def test_global_offsets_5d(oracle, reflib, which, layout, rows, cols):
    ref, sh, st = reflib.global_offsets(which, rows, cols)
    assert np.array_equal(ref, oracle.global_offsets(layout, sh, st, rows, cols))


@pytest.mark.parametrize("layout", [ob.ND, ob.DN, ob.NZ])
@pytest.mark.parametrize("rows,cols", [(32, 64), (48, 16), (16, 8)])
def test_layout_2d(oracle, reflib, layout, rows, cols):
    want = reflib.layout_2d(layout, rows, cols)
    got = oracle.layout_2d(layout, rows, cols, c0=8)
    assert np.array_equal(want[0], got[0]) and np.array_equal(want[1], got[1])


def test_reorder_exp_zz(oracle, reflib):
    e = np.random.default_rng(3).integers(0, 256, (64, 10)).astype(np.uint8)
    assert np.array_equal(reflib.reorder_exp_zz(e), oracle.reorder_exp_zz(e))


def _word_scalar(scale, offset=0, sign=1):
    return int(np.float32(scale).view(np.uint32)) | (offset << 37) | (sign << 46)


def _word_vector(scale, offset=0, sign=1):
    bits = int(np.float32(scale).view(np.uint32))
    m1 = ((bits >> 31) << 18) | (((bits >> 23) & 0xFF) << 10) | ((bits >> 13) & 0x3FF)
    return (m1 << 13) | (offset << 37) | (sign << 46)


@pytest.mark.parametrize("per_col", [0, 1])
@pytest.mark.parametrize("relu", [False, True])
def test_store_quant(oracle, reflib, per_col, relu):
    r = _rng(17 + per_col)
    m, n = 24, 40
    accf = (r.standard_normal((m, n)) * 300).astype(np.float32)
    acci = r.integers(-40000, 40000, (m, n)).astype(np.int32)
    mk = _word_vector if per_col else _word_scalar
    for sign, dst, kind in ((1, "i8", ob.ST_I8), (0, "u8", ob.ST_U8)):
        words = np.array([mk(r.uniform(0.05, 1.0), int(r.integers(0, 20)), sign) for _ in range(n)], np.uint64)
        assert np.array_equal(reflib.store_quant(accf, dst, words, per_col, relu),
                              oracle.store_quant(accf, kind, words, per_col, relu))
    words = np.array([mk(r.uniform(0.0005, 0.01), 0, 1) for _ in range(n)], np.uint64)
    assert np.array_equal(reflib.store_quant(acci, "i8", words, per_col, relu),
                          oracle.store_quant(acci, ob.ST_I8, words, per_col, relu))
    words = np.array([mk(r.uniform(0.5, 400.0)) for _ in range(n)], np.uint64)
    assert np.array_equal(reflib.store_quant(accf, "f16", words, per_col, relu),
                          oracle.store_quant(accf, ob.ST_F16, words, per_col, relu))
    assert np.array_equal(reflib.store_quant(acci, "f16", words, per_col, relu),
                          oracle.store_quant(acci, ob.ST_F16, words, per_col, relu))


def test_store_int16_shift_mode(oracle, reflib):
    r = _rng(23)
    acc = r.integers(-2 ** 31, 2 ** 31, (24, 40)).astype(np.int32)
    words = (r.integers(0, 16, 40).astype(np.uint64) << np.uint64(32)) | r.integers(0, 2 ** 32, 40).astype(np.uint64)
    for per_col in (0, 1):
        for relu in (False, True):
            assert np.array_equal(reflib.store_quant(acc, "i16", words, per_col, relu),
                                  oracle.store_quant(acc, ob.ST_I16, words, per_col, relu))


def test_parameter_tiles(oracle, reflib):
    r = _rng(29)
    src8 = r.integers(-128, 128, (16, 64)).astype(np.int8)
    for pc in (1, 3, 8):
        sc = r.uniform(0.25, 2.0, (16, pc)).astype(np.float32)
        of = r.uniform(-20, 20, (16, pc)).astype(np.float32)
        assert np.array_equal(reflib.tdequant_para(src8, sc, of).view(np.uint32), oracle.tdequant_para(src8, sc, of).view(np.uint32))
    srcf = (r.standard_normal((16, 64)) * 40).astype(np.float32)
    for pr in (1, 5, 16):
        sc = r.uniform(0.5, 4.0, pr).astype(np.float32)
        of = r.uniform(0, 200, pr).astype(np.float32)
        assert np.array_equal(reflib.tquant_int8_para(srcf, sc), oracle.tquant_int8_para(srcf, sc))
        assert np.array_equal(reflib.tquant_int8_para(srcf, sc, of), oracle.tquant_int8_para(srcf, sc, of))


def test_store_f32_to_f16(oracle, reflib):
    r = _rng(23)
    a = _f16(r.uniform(-4, 4, (40, 64)))
    b = _f16(r.uniform(-4, 4, (64, 56)))
    for relu in (False, True):
        ref = reflib.gemm_f16_out_f16(a, b, relu=relu)
        got = oracle.store_f32(oracle.matmul_f16(a, b), ob.ST_F16, relu=relu)
        assert np.array_equal(ref, got)


def _quant_sources(r, rows, cols):
    yield (r.standard_normal((rows, cols)) * 10 ** r.uniform(-3, 3, (rows, 1))).astype(np.float32)
    x = (r.standard_normal((rows, cols)) * 5).astype(np.float32)
    x.ravel()[::7] = 0.0
    x.ravel()[3::11] *= 1e-30
    x.ravel()[5::13] *= 1e30
    yield x
    pattern = np.array([0.0, -0.0, 1e-45, -1e-45, 2.0 ** -130, -2.0 ** -130, np.nextafter(np.float32(448), 0), 448.0,
                        -448.0, np.nextafter(np.float32(448), np.inf), 896.0, np.inf, -np.inf, np.nan, 6.0, 0.75],
                       np.float32)
    yield np.resize(pattern, (rows, cols)).astype(np.float32)
    # NaNs of either sign inside otherwise finite groups (the pattern above always has an infinity in a NaN's group, which
    # hides how a NaN element itself is encoded)
    x = (r.standard_normal((rows, cols)) * 3).astype(np.float32)
    xb = x.view(np.uint32).ravel()
    xb[5::37] = 0x7FC00000
    xb[11::41] = 0xFFC00000
    xb[17::53] = 0xFF800001  # a negative signalling NaN
    yield x


@pytest.mark.parametrize("shape_id", [0, 1, 2, 3, 4, 5, 6])
@pytest.mark.parametrize("alg", [ob.OCP_FP8, ob.NV_FP8, ob.OCP_FP4, ob.NV_FP4])
@pytest.mark.parametrize("axis", [1, 0])
def test_tquant_mx(oracle, reflib, shape_id, alg, axis):
    rows, cols = reflib.shape(shape_id)
    if axis == 0 and shape_id not in (5, 6):
        pytest.skip("column grouping is compiled for shapes 5 and 6 only")
    if alg in (ob.OCP_FP4, ob.NV_FP4) and cols % 64:
        pytest.skip("packed fp4 rows must be 32-byte aligned")
    r = _rng(shape_id * 8 + alg)
    for src in _quant_sources(r, rows, cols):
        for f16 in (False, True):
            s = src.astype(np.float16).astype(np.float32) if f16 else src
            ref = reflib.tquant_mx(shape_id, s, alg, axis, src_f16=f16)
            got = oracle.tquant_mx(s, alg, axis, ob.SRC_F16 if f16 else ob.SRC_F32)
            for x, y, name in zip(ref, got, ("codes", "exp", "max", "scaling")):
                if x.dtype == np.float32:  # bit for bit; the quiet bit of a NaN may differ where both are NaN
                    xb, yb = x.view(np.uint32).copy(), y.view(np.uint32).copy()
                    both_nan = np.isnan(x) & np.isnan(y)
                    xb[both_nan] &= 0xFFBFFFFF
                    yb[both_nan] &= 0xFFBFFFFF
                    assert np.array_equal(xb, yb), name
                else:
                    assert np.array_equal(x, y), name


@pytest.mark.parametrize("shape_id", [0, 3, 6])
def test_tquant_int8_and_dequant(oracle, reflib, shape_id):
    rows, cols = reflib.shape(shape_id)
    r = _rng(shape_id)
    src = (r.standard_normal((rows, cols)) * 40).astype(np.float32)
    src.ravel()[::5] = np.round(src.ravel()[::5]) + 0.5  # exact ties
    scale = r.uniform(0.5, 4.0, rows).astype(np.float32)
    off = r.uniform(0, 200, rows).astype(np.float32)
    assert np.array_equal(reflib.tquant_int8(shape_id, src, scale).view(np.int8), oracle.tquant_int8(src, scale))
    assert np.array_equal(reflib.tquant_int8(shape_id, src, scale, off), oracle.tquant_int8(src, scale, off))
    for dt, lo, hi in ((np.int8, -128, 128), (np.int16, -30000, 30000), (np.int32, -2**31, 2**31)):
        q = r.integers(lo, hi, (rows, cols)).astype(dt)
        ref = reflib.tdequant(shape_id, q, scale, off)
        got = oracle.tdequant(q, scale, off)
        assert np.array_equal(ref.view(np.uint32), got.view(np.uint32))


def test_scalar_quant_helpers(oracle, reflib):
    r = _rng(29)
    vals = np.concatenate([(r.standard_normal(20000) * 10 ** r.uniform(-5, 3, 20000)).astype(np.float32),
                           np.array([0, -0.0, np.inf, -np.inf, np.nan, 448, 449, 464, 480, 2 ** -10, -2 ** -10, 2 ** -9,
                                     2 ** -11, -2 ** -11, 1e-40, -1e-40], np.float32)])
    dec = np.array([oracle.lib.pto_mx_decode(0, c) for c in range(0x7F)])
    mids = ((dec[:-1] + dec[1:]) / 2).astype(np.float32)  # every rounding boundary of E4M3
    vals = np.concatenate([vals, mids, -mids, np.nextafter(mids, np.float32(0)), np.nextafter(mids, np.float32(1e9))])
    for v in vals:
        for nv in (0, 1):
            assert reflib.lib.ref_encode_e4m3fn(float(v), nv) == oracle.lib.pto_encode_e4m3fn(float(v), nv), (v, nv)
        assert reflib.lib.ref_encode_e2m1_magic(float(v)) == oracle.lib.pto_encode_e2m1_magic(float(v)), v
    grid = np.array([0, .25, .5, .75, 1, 1.25, 1.5, 1.75, 2, 2.5, 3, 3.5, 4, 5, 6, 7, 100], np.float32)
    for v in np.concatenate([grid, -grid, np.nextafter(grid, np.float32(0)), np.nextafter(grid, np.float32(1e9))]):
        assert reflib.lib.ref_encode_e2m1_magic(float(v)) == oracle.lib.pto_encode_e2m1_magic(float(v)), v
    maxes = np.concatenate([np.abs(vals[:3000]), np.ldexp(np.float32(1), np.arange(-149, 128)).astype(np.float32),
                            np.ldexp(np.float32(1.5), np.arange(-126, 127)).astype(np.float32)])
    for alg in range(4):
        for mx in maxes:
            e = reflib.lib.ref_shared_exponent(alg, float(mx))
            assert e == oracle.lib.pto_shared_exponent(alg, float(mx)), (alg, mx)
            a = reflib.lib.ref_group_scaling(alg, float(mx), e)
            b = oracle.lib.pto_group_scaling(alg, float(mx), e)
            assert (np.isnan(a) and np.isnan(b)) or a == b, (alg, mx)
    for word in [int(x) for x in r.integers(0, 2 ** 63, 2000)]:
        for vm in (0, 1):
            a = reflib.lib.ref_extract_m1(word, vm)
            b = oracle.lib.pto_quant_word_scale(word, vm)
            assert (np.isnan(a) and np.isnan(b)) or a == b, (word, vm)


def test_hif8_decode_all_codes(oracle, reflib):
    """HiFloat8: all 256 codes, the oracle's arithmetic decode against the compiled reference's table (cpu/Hifloat8.hpp)."""
    want, got = reflib.hif8_table(), oracle.hif8_table()
    assert np.array_equal(np.isnan(want), np.isnan(got))
    assert np.array_equal(np.nan_to_num(want, nan=0.0).view(np.uint64), np.nan_to_num(got, nan=0.0).view(np.uint64))
    assert np.array_equal(np.signbit(want), np.signbit(got))
    assert np.array_equal(want[~np.isnan(want)].astype(np.float32).astype(np.float64), want[~np.isnan(want)])  # exact in f32


@pytest.mark.parametrize("per_col", [0, 1])
@pytest.mark.parametrize("relu", [False, True])
def test_store_quant_saturate_inf(oracle, reflib, per_col, relu):
    """The fix-pipe's saturation control (task cookie bit 48, cpu/common.hpp:146,157-164) on non-finite and overflowing
    products of a float accumulator, half target: off, they pass through; on, NaN becomes 0 and the rest is clamped."""
    r = _rng(31 + per_col)
    m, n = 16, 24
    acc = (r.standard_normal((m, n)) * 3000).astype(np.float32)
    acc[0, :4] = [np.inf, -np.inf, np.nan, 1e30]
    acc[3, 5:9] = [-1e30, 7e4, -7e4, np.nan]
    acc.ravel()[11::17] = np.inf
    mk = _word_vector if per_col else _word_scalar
    words = np.array([mk(r.uniform(0.5, 40.0)) for _ in range(n)], np.uint64)
    for sat in (0, 1):
        want = reflib.store_quant(acc, "f16", words, per_col, relu, saturate_inf=sat)
        got = oracle.store_quant(acc, ob.ST_F16, words, per_col, relu, saturate_inf=sat)
        both_nan = ((want & 0x7FFF) > 0x7C00) & ((got & 0x7FFF) > 0x7C00)
        assert np.array_equal(np.where(both_nan, 0, want), np.where(both_nan, 0, got)), sat
    assert not np.array_equal(reflib.store_quant(acc, "f16", words, per_col, relu, saturate_inf=0),
                              reflib.store_quant(acc, "f16", words, per_col, relu, saturate_inf=1))
