"""Writes tests/golden/pto_golden.npz: inputs and the outputs the *compiled reference CPU simulator*
(oracle/_ref/libptoref.so, built from the reference's own headers) produced for them.

Run where the reference tree is mounted:   make -C oracle && python tests/golden/gen_golden.py
The fixture is data only (seeded inputs + expected outputs); tests/test_oracle_golden.py and the GPU parity
tests replay it without the reference.
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import binding as ob  # noqa: E402


def f16(x):
    return np.asarray(x, np.float32).astype(np.float16).view(np.uint16)


def mx_codes(r, typ, rows, cols):
    if typ in (ob.E2M1, ob.E1M2):
        return r.integers(0, 256, (rows, cols // 2)).astype(np.uint8)
    x = r.integers(0, 256, (rows, cols)).astype(np.uint8)
    bad = (x & 0x7F) == 0x7F if typ == ob.E4M3 else (x & 0x7F) >= 0x7C
    x[bad] = 0x31
    return x


def main():
    ref = ob.RefLib()
    r = np.random.default_rng(20250101)
    g = {}

    # --- TMATMUL family -------------------------------------------------------------------
    # the reference tests' own input distribution: small integers, so every result is an exact integer
    for name, (m, k, n) in {"case1": (40, 50, 60), "case3_splitk": (128, 320, 64), "gemv": (1, 110, 50)}.items():
        a = f16(r.integers(1, 5, (m, k)))
        b = f16(r.integers(1, 5, (k, n)))
        g[f"mm_f16_int_{name}_a"], g[f"mm_f16_int_{name}_b"] = a, b
        g[f"mm_f16_int_{name}_out"] = ref.gemm("f16", a, b, kstep=64 if "splitk" in name else 0)
    a = f16(r.uniform(-1, 1, (96, 192)))
    b = f16(r.uniform(-1, 1, (80, 192)))  # column-major B ([n][k])
    cin = r.standard_normal((96, 80)).astype(np.float32)
    g["mm_f16_a"], g["mm_f16_bt"], g["mm_f16_cin"] = a, b, cin
    g["mm_f16_out"] = ref.gemm("f16", a, b, b_dn=True, kstep=64)
    g["mm_f16_out_acc"] = ref.gemm("f16", a, b, cin=cin, b_dn=True)
    g["mm_f16_out_f16"] = ref.gemm_f16_out_f16(a, b, b_dn=True)
    g["mm_f16_out_f16_relu"] = ref.gemm_f16_out_f16(a, b, b_dn=True, relu=True)
    a = r.standard_normal((50, 70)).astype(np.float32)
    b = r.standard_normal((70, 30)).astype(np.float32)
    g["mm_f32_a"], g["mm_f32_b"] = a, b
    g["mm_f32_out"] = ref.gemm("f32", a, b)
    # bf16-representable fp32 inputs: the fp32 path is then the bf16 path (products exact in fp32)
    a = (r.standard_normal((64, 160)) * 0.02).astype(np.float32).view(np.uint32) & 0xFFFF0000
    b = (r.standard_normal((48, 160)) * 0.02).astype(np.float32).view(np.uint32) & 0xFFFF0000
    g["mm_bf16rep_a"], g["mm_bf16rep_bt"] = a.view(np.float32), b.view(np.float32)
    g["mm_bf16rep_out"] = ref.gemm("f32", a.view(np.float32), b.view(np.float32), b_dn=True)
    a = r.integers(-128, 128, (72, 384)).astype(np.int8)
    b = r.integers(-128, 128, (56, 384)).astype(np.int8)
    cin = r.integers(-2 ** 31, 2 ** 31, (72, 56)).astype(np.int32)
    g["mm_i8_a"], g["mm_i8_bt"], g["mm_i8_cin"] = a, b, cin
    g["mm_i8_out"] = ref.gemm("i8", a, b, b_dn=True)
    g["mm_i8_out_acc"] = ref.gemm("i8", a, b, cin=cin, b_dn=True)
    a = mx_codes(r, ob.E4M3, 40, 96)
    b = mx_codes(r, ob.E4M3, 96, 24)
    g["mm_e4m3_a"], g["mm_e4m3_b"] = a, b
    g["mm_e4m3_out"] = ref.gemm("e4m3", a, b)

    # --- TMATMUL_MX -----------------------------------------------------------------------
    m, k, n = 48, 192, 80
    for tname, typ in (("e4m3", ob.E4M3), ("e5m2", ob.E5M2), ("e2m1", ob.E2M1), ("e1m2", ob.E1M2)):
        a = mx_codes(r, typ, m, k)
        bt = mx_codes(r, typ, n, k)
        sa = r.integers(115, 140, m * k // 32).astype(np.uint8)
        sb = r.integers(115, 140, n * k // 32).astype(np.uint8)
        cin = r.standard_normal((m, n)).astype(np.float32)
        g[f"mx_{tname}_a"], g[f"mx_{tname}_bt"], g[f"mx_{tname}_sa"], g[f"mx_{tname}_sb"] = a, bt, sa, sb
        g[f"mx_{tname}_cin"] = cin
        for fmt in (0, 1, 2):
            g[f"mx_{tname}_out_fmt{fmt}"] = ref.gemm_mx(a, bt, sa, sb, m, k, n, typ, fmt, True)
        g[f"mx_{tname}_out_acc_fmt2"] = ref.gemm_mx(a, bt, sa, sb, m, k, n, typ, 2, True, cin=cin)

    # --- element types ---------------------------------------------------------------------
    for typ, nm in enumerate(("e4m3", "e5m2", "e2m1", "e1m2", "e8m0")):
        ncodes = 16 if typ in (2, 3) else 256
        g[f"decode_{nm}"] = np.array([ref.lib.ref_mx_decode(typ, c) for c in range(ncodes)], np.float64)
    vals = np.concatenate([r.standard_normal(600) * 10 ** r.uniform(-5, 4, 600), np.arange(-8, 8, 0.125),
                           np.ldexp(1.0, np.arange(-20, 18)), [np.inf, -np.inf, 0.0]]).astype(np.float64)
    g["encode_vals"] = vals
    g["encode_trunc"] = np.array([[ref.lib.ref_mx_encode_trunc(t, float(v)) for v in vals] for t in range(5)],
                                 np.uint8)
    g["encode_round_fp8"] = np.array([[[[ref.lib.ref_mx_encode_round(t, float(v), mode, sat) for v in vals]
                                        for sat in (0, 1)] for mode in range(7)] for t in (0, 1)], np.uint8)
    g["encode_round_fp4"] = np.array([[[ref.lib.ref_mx_encode_round(t, float(v), mode, 0) for v in vals]
                                       for mode in range(7)] for t in (2, 3)], np.uint8)

    # --- addressing ------------------------------------------------------------------------
    shapes = {0: (64, 128), 1: (64, 128), 2: (64, 128), 3: (64, 128), 4: (64, 128), 5: (64, 128), 6: (64, 128),
              7: (64, 8), 8: (8, 64), 9: (64, 128), 10: (64, 128), 11: (64, 128)}
    for kind, (rows, cols) in shapes.items():
        g[f"tile_offset_{kind}"] = np.array([[ref.lib.ref_tile_offset(kind, rr, cc) for cc in range(cols)]
                                             for rr in range(rows)], np.int32)
    for lid in range(6):
        rows, cols = (32, 8) if lid < 3 else (8, 32)
        g[f"mx_scale_offset_{lid}"] = np.array([[ref.lib.ref_mx_scale_offset(lid, rows, cols, rr, cc)
                                                 for cc in range(cols)] for rr in range(rows)], np.int32)

    # --- fix-pipe stores -------------------------------------------------------------------
    accf = (r.standard_normal((24, 40)) * 300).astype(np.float32)
    acci = r.integers(-40000, 40000, (24, 40)).astype(np.int32)
    g["st_accf"], g["st_acci"] = accf, acci

    def sword(scale, off=0, sign=1):
        return int(np.float32(scale).view(np.uint32)) | (off << 37) | (sign << 46)

    def vword(scale, off=0, sign=1):
        bits = int(np.float32(scale).view(np.uint32))
        m1 = ((bits >> 31) << 18) | (((bits >> 23) & 0xFF) << 10) | ((bits >> 13) & 0x3FF)
        return (m1 << 13) | (off << 37) | (sign << 46)

    for per_col, mk in ((0, sword), (1, vword)):
        w8 = np.array([mk(r.uniform(0.05, 1.0), int(r.integers(0, 20)), 1) for _ in range(40)], np.uint64)
        wu = np.array([mk(r.uniform(0.05, 1.0), int(r.integers(0, 20)), 0) for _ in range(40)], np.uint64)
        wi = np.array([mk(r.uniform(0.0005, 0.01)) for _ in range(40)], np.uint64)
        wh = np.array([mk(r.uniform(0.5, 400.0)) for _ in range(40)], np.uint64)
        g[f"st_w8_{per_col}"], g[f"st_wu_{per_col}"], g[f"st_wi_{per_col}"], g[f"st_wh_{per_col}"] = w8, wu, wi, wh
        for relu in (0, 1):
            g[f"st_f32_i8_{per_col}_{relu}"] = ref.store_quant(accf, "i8", w8, per_col, relu)
            g[f"st_f32_u8_{per_col}_{relu}"] = ref.store_quant(accf, "u8", wu, per_col, relu)
            g[f"st_i32_i8_{per_col}_{relu}"] = ref.store_quant(acci, "i8", wi, per_col, relu)
            g[f"st_f32_f16_{per_col}_{relu}"] = ref.store_quant(accf, "f16", wh, per_col, relu)
            g[f"st_i32_f16_{per_col}_{relu}"] = ref.store_quant(acci, "f16", wh, per_col, relu)

    # --- TQUANT / TDEQUANT -----------------------------------------------------------------
    pattern = np.array([0.0, -0.0, 1e-45, -1e-45, 2.0 ** -130, -2.0 ** -130, np.nextafter(np.float32(448), 0), 448.0,
                        -448.0, np.nextafter(np.float32(448), np.inf), 896.0, np.inf, -np.inf, np.nan, 6.0, 0.75],
                       np.float32)
    for sid in (2, 5):
        rows, cols = ref.shape(sid)
        srcs = [(r.standard_normal((rows, cols)) * 10 ** r.uniform(-3, 3, (rows, 1))).astype(np.float32),
                np.resize(pattern, (rows, cols)).astype(np.float32)]
        mixed = (r.standard_normal((rows, cols)) * 5).astype(np.float32)
        mixed.ravel()[::7] = 0.0
        mixed.ravel()[3::11] *= 1e-30
        mixed.ravel()[5::13] *= 1e30
        srcs.append(mixed)
        for si, src in enumerate(srcs):
            g[f"tq_src_{sid}_{si}"] = src
            for alg in range(4):
                for axis in ((1, 0) if sid == 5 else (1,)):
                    codes, exp, mx, sc = ref.tquant_mx(sid, src, alg, axis)
                    key = f"tq_{sid}_{si}_{alg}_{axis}"
                    g[key + "_codes"], g[key + "_exp"], g[key + "_max"], g[key + "_scaling"] = codes, exp, mx, sc
    rows, cols = ref.shape(3)
    src = (r.standard_normal((rows, cols)) * 40).astype(np.float32)
    src.ravel()[::5] = np.round(src.ravel()[::5]) + 0.5
    scale = r.uniform(0.5, 4.0, rows).astype(np.float32)
    off = r.uniform(0, 200, rows).astype(np.float32)
    g["q8_src"], g["q8_scale"], g["q8_off"] = src, scale, off
    g["q8_sym"] = ref.tquant_int8(3, src, scale).view(np.int8)
    g["q8_asym"] = ref.tquant_int8(3, src, scale, off)
    for nm, dt, lo, hi in (("i8", np.int8, -128, 128), ("i16", np.int16, -30000, 30000),
                           ("i32", np.int32, -2 ** 31, 2 ** 31)):
        q = r.integers(lo, hi, (rows, cols)).astype(dt)
        g[f"dq_src_{nm}"] = q
        g[f"dq_out_{nm}"] = ref.tdequant(3, q, scale, off)

    # --- 5-D global tensors, whole-matrix shape helpers, ZZ exponent reorder (appended: earlier draws unchanged) ---
    for which, (rows, cols) in enumerate(((2 * 3 * 4 * 8, 16), (8, 2 * 3 * 4 * 16), (48, 32))):
        offs, sh, st = ref.global_offsets(which, rows, cols)
        g[f"global_offset_{which}"], g[f"global_shape_{which}"], g[f"global_stride_{which}"] = offs, sh, st
    for lay in range(3):
        for rows, cols in ((32, 64), (48, 16)):
            sh, st = ref.layout_2d(lay, rows, cols)
            g[f"layout2d_{lay}_{rows}x{cols}"] = np.stack([sh, st])
    e = r.integers(0, 256, (48, 6)).astype(np.uint8)
    g["zz_exp"], g["zz_reordered"] = e, ref.reorder_exp_zz(e)

    # --- parameter tiles wider / shorter than the data tile; the int16 shift mode of the requantising store ---
    src8 = r.integers(-128, 128, (16, 64)).astype(np.int8)
    g["dqp_src"] = src8
    for pc in (1, 3, 8):
        sc = r.uniform(0.25, 2.0, (16, pc)).astype(np.float32)
        of = r.uniform(-20, 20, (16, pc)).astype(np.float32)
        g[f"dqp_scale_{pc}"], g[f"dqp_off_{pc}"] = sc, of
        g[f"dqp_out_{pc}"] = ref.tdequant_para(src8, sc, of)
    srcf = (r.standard_normal((16, 64)) * 40).astype(np.float32)
    g["q8p_src"] = srcf
    for pr in (1, 5, 16):
        sc = r.uniform(0.5, 4.0, pr).astype(np.float32)
        of = r.uniform(0, 200, pr).astype(np.float32)
        g[f"q8p_scale_{pr}"], g[f"q8p_off_{pr}"] = sc, of
        g[f"q8p_sym_{pr}"] = ref.tquant_int8_para(srcf, sc)
        g[f"q8p_asym_{pr}"] = ref.tquant_int8_para(srcf, sc, of)
    acc = r.integers(-2 ** 31, 2 ** 31, (24, 40)).astype(np.int32)
    acc[0, :8] = [0, 1, -1, 65535, 65536, -65536, 2 ** 31 - 1, -2 ** 31]
    wsh = (r.integers(0, 16, 40).astype(np.uint64) << np.uint64(32)) | r.integers(0, 2 ** 32, 40).astype(np.uint64)
    g["s16_acc"], g["s16_words"] = acc, wsh
    for per_col in (0, 1):
        for relu in (0, 1):
            g[f"s16_out_{per_col}_{relu}"] = ref.store_quant(acc, "i16", wsh, per_col, relu=bool(relu))

    out = os.path.join(ROOT, "tests", "golden", "pto_golden.npz")
    np.savez_compressed(out, **g)
    print(f"wrote {out}: {len(g)} arrays, {os.path.getsize(out)} bytes")


if __name__ == "__main__":
    main()
