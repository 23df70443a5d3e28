"""Writes the data of the framework-free case runner (tests/pto_kernels/case_runner.hip): inputs and goldens of the
reference's own test lists for the matmul path -- tests/cpu/st/testcase/tmatmul/main.cpp:96-252 (case1-4, gemm_1/2, bf16_1,
bias_1/2/5/gemm, bf16_bias_1), tmatmul_mx/main.cpp:151-330 (case1-19), tstore_acc2gm/main.cpp:220-247 (nz2nd and scalar
quantisation cases), tstore_quant/main.cpp:112-130 (ND_1 ... ND_10), tquant/main.cpp:161-777, tdequant/gen_data.py:69-72 -- with shapes, element types and value distributions taken from those
files and their gen_data.py, the inputs drawn from this script's own seeds, and every golden computed by the oracle
(oracle/pto_oracle.c), not by the runner.

    python tests/golden/gen_runner_cases.py        # rewrites tests/golden/runner_cases.npz and runner_cases.txt

runner_cases.txt is the manifest the runner reads (one case per line); runner_cases.npz holds the arrays, which the test
expands into <dir>/<suite>/<case>/<name>.bin files named as the reference names them (x1_gm.bin, x2_gm.bin, bias_gm.bin,
x1_mx_gm.bin, x2_mx_gm.bin, golden.bin).  Data only.
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import binding as ob  # noqa: E402

orc = ob.Oracle()
rng = np.random.default_rng(20251)
arrays, manifest = {}, []

F16 = lambda x: np.asarray(x, np.float32).astype(np.float16).view(np.uint16)  # noqa: E731
BF16 = lambda x: (np.asarray(x, np.float32).view(np.uint32) >> 16).astype(np.uint16)  # noqa: E731  (exact for small integers)


def put(suite, case, **files):
    for name, arr in files.items():
        arrays[f"{suite}/{case}/{name}"] = np.ascontiguousarray(arr)


def line(suite, case, op, m, k, n, at, bt, ct, extra=0, eps=0.001, pto="-"):
    manifest.append(f"{suite} {case} {op} {m} {k} {n} {at} {bt} {ct} {extra} {eps} {pto}")


# ---- tmatmul (integers 1..4 as tmatmul/gen_data.py:43-49; int8 full range) -------------------------------------------------
def ints(shape, lo=1, hi=5):
    return rng.integers(lo, hi, shape)


def tmatmul(case, kind, m, k, n, bias=False, repeats=1, pto="-"):
    if kind == "i8":
        a, b = ints((repeats * m, k), -128, 128).astype(np.int8), ints((repeats * k, n), -128, 128).astype(np.int8)
        mm, ct, bias_v = orc.matmul_i8, "i32", ints(n, -1000, 1000).astype(np.int32)
    else:
        conv = {"f16": F16, "bf16": BF16, "f32": lambda x: np.asarray(x, np.float32)}[kind]
        a, b = conv(ints((repeats * m, k))), conv(ints((repeats * k, n)))
        mm, ct = {"f16": orc.matmul_f16, "bf16": orc.matmul_bf16, "f32": orc.matmul_f32}[kind], "f32"
        bias_v = ints(n, 1, 10).astype(np.float32)
    acc = None
    for r in range(repeats):
        acc = mm(a[r * m:(r + 1) * m], b[r * k:(r + 1) * k], cin=acc, bias=bias_v if (bias and r == repeats - 1) else None)
    files = dict(x1_gm=a, x2_gm=b, golden=acc)
    if bias:
        files["bias_gm"] = bias_v
    put("tmatmul", case, **files)
    op = "gemm_bias" if bias else ("gemm_splitk" if repeats > 1 else "gemm")
    line("tmatmul", case, op, m, k, n, kind, kind, ct, repeats, 0.001, pto)


tmatmul("case1", "f16", 40, 50, 60, pto="k1")
tmatmul("case2", "i8", 6, 7, 8, pto="k2")
tmatmul("case3", "f16", 128, 128, 64, repeats=5, pto="k3")
tmatmul("case4", "f32", 120, 110, 50)
tmatmul("case_gemm_1", "f16", 1, 110, 50, pto="k5")
tmatmul("case_gemm_2", "f32", 1, 128, 64)
tmatmul("case_bf16_1", "bf16", 40, 50, 60, pto="k7")
tmatmul("case_bias_1", "i8", 8, 7, 6, bias=True, pto="k12")
tmatmul("case_bias_2", "f16", 16, 15, 16, bias=True)
tmatmul("case_bias_5", "f32", 127, 128, 63, bias=True)
tmatmul("case_bias_gemm", "f16", 1, 110, 50, bias=True)
tmatmul("case_bf16_bias_1", "bf16", 16, 15, 16, bias=True)

# ---- tmatmul_mx (tmatmul_mx/gen_data.py:227-259: scales 127..129; K padded to a multiple of 64 with zero codes) ---------------
E4, E5, E2, E1 = ob.E4M3, ob.E5M2, ob.E2M1, ob.E1M2
TNAME = {E4: "e4m3", E5: "e5m2", E2: "e2m1", E1: "e1m2"}


def codes(typ, shape):
    if typ in (E2, E1):
        return rng.integers(0, 16, shape).astype(np.uint8)
    table = orc.mx_decode_table(typ)
    ok = np.array([c for c in range(256) if np.isfinite(table[c]) and abs(table[c]) <= 16 and float(table[c]).is_integer()], np.uint8)
    return ok[rng.integers(0, len(ok), shape)]


def pack4(c):  # [rows][cols] codes -> [rows][cols / 2] bytes, even element in the low nibble
    return (c[:, 0::2] | (c[:, 1::2] << 4)).astype(np.uint8)


def tmatmul_mx(case, ta, tb, m, k, n, bias=False, sfmt=("zz", "nn"), pto="-"):
    kp = (k + 63) // 64 * 64
    fp4 = ta in (E2, E1)
    mp = (m + 15) // 16 * 16 if sfmt[0] == "zz" else m
    npad = (n + 15) // 16 * 16 if sfmt[1] == "nn" else n
    a = np.zeros((mp, kp), np.uint8)
    b = np.zeros((npad, kp), np.uint8)          # B as [N][K]: the DN view
    a[:m, :k], b[:n, :k] = codes(ta, (m, k)), codes(tb, (n, k))
    kg = kp // 32
    sa, sb = rng.integers(127, 130, (mp, kg)).astype(np.uint8), rng.integers(127, 130, (npad, kg)).astype(np.uint8)
    a_bin, b_bin = (pack4(a), pack4(b)) if fp4 else (a, b)
    bias_v = ints(npad, 1, 10).astype(np.float32) if bias else None
    ref = orc.matmul_mx(a_bin, b_bin, sa, sb, mp, kp, npad, ta, tb, bias=bias_v)   # plain [M][K/32], [N][K/32] scales
    # the scale files in the layout the case names (zz / nn boxes, or plain rows)
    la = ob.MX_A_ZZ if sfmt[0] == "zz" else ob.MX_A_ND
    lb = ob.MX_B_NN if sfmt[1] == "nn" else ob.MX_B_DN
    sa_file, sb_file = np.zeros(mp * kg, np.uint8), np.zeros(npad * kg, np.uint8)
    sa_file[orc.mx_scale_offsets(la, mp, kg).ravel()] = sa.ravel()
    sb_file[orc.mx_scale_offsets(lb, kg, npad).ravel()] = np.ascontiguousarray(sb.T).ravel()
    files = dict(x1_gm=a_bin, x2_gm=b_bin, x1_mx_gm=sa_file, x2_mx_gm=sb_file, golden=ref[:m, :n])
    if bias:
        files["bias_gm"] = bias_v
    put("tmatmul_mx", case, **files)
    # extra: valid m, k, n packed as m * 2^40 + k * 2^20 + n; the m / k / n columns are the padded extents the launch uses
    line("tmatmul_mx", case, "mx_bias" if bias else "mx", mp, kp, npad, TNAME[ta], TNAME[tb], "f32",
         f"{m}:{k}:{n}:{sfmt[0]}:{sfmt[1]}", 0.001, pto)


MX_CASES = [(E5, E5, 128, 64, 64), (E4, E4, 127, 72, 64), (E4, E5, 128, 110, 63), (E2, E2, 128, 64, 64), (E1, E2, 117, 64, 60),
            (E2, E1, 128, 118, 64), (E2, E1, 115, 64, 30), (E4, E4, 16, 32, 16), (E4, E5, 10, 50, 54), (E2, E2, 4, 30, 8)]
for i, (ta, tb, m, k, n) in enumerate(MX_CASES):
    tmatmul_mx(f"case{i + 1}", ta, tb, m, k, n)
tmatmul_mx("case11", E1, E1, 1, 128, 62, sfmt=("nd", "nd"))
tmatmul_mx("case12", E4, E5, 1, 256, 20, sfmt=("nd", "nd"))
for i, (ta, tb, m, k, n) in enumerate([(E5, E4, 115, 64, 30), (E4, E4, 200, 192, 95), (E2, E1, 35, 128, 56), (E1, E1, 47, 128, 62),
                                       (E4, E5, 64, 192, 64), (E1, E1, 1, 64, 62)]):
    tmatmul_mx(f"case{i + 13}", ta, tb, m, k, n, bias=True)
tmatmul_mx("case19", E1, E1, 1, 2048, 64, bias=True, sfmt=("nd", "nn"))

# ---- tstore_acc2gm: matmul, then the accumulator leaves through TSTORE (tstore_acc2gm/gen_data.py:102-131, 259-283) -----------
ST = {"f32": ob.ST_F32, "f16": ob.ST_F16, "bf16": ob.ST_BF16, "i32": ob.ST_I32, "i8": ob.ST_I8, "u8": ob.ST_U8}


def acc2gm(case, dst, src, m, k, n, relu=False, scalar=None):
    if src == "i8":
        lo, hi = (-1, 2) if dst == "i8" else (-5, 6)
        a, b = ints((m, k), lo, hi).astype(np.int8), ints((k, n), lo, hi).astype(np.int8)
        acc = orc.matmul_i8(a, b)
    else:
        conv, mm = {"f16": (F16, orc.matmul_f16), "bf16": (BF16, orc.matmul_bf16), "f32": (lambda x: np.asarray(x, np.float32), orc.matmul_f32)}[src]
        a, b = conv(ints((m, k), -5, 6)), conv(ints((k, n), -5, 6))
        acc = mm(a, b)
    if scalar is None:
        golden = acc if dst in ("f32", "i32") else orc.store_f32(acc, ST[dst], relu=relu)
        if dst in ("f32", "i32") and relu:
            golden = np.maximum(acc, 0)
        op, extra = "store", int(relu)
    else:
        word = int(np.float32(scalar).view(np.uint32)) | ((1 << 46) if dst == "i8" else 0)
        golden = orc.store_quant(acc, ST[dst], np.array([word], np.uint64), 0, relu=relu)
        op, extra = "store_q", f"{word}:{int(relu)}"
    put("tstore_acc2gm", case, x1_gm=a, x2_gm=b, golden=golden)
    line("tstore_acc2gm", case, op, m, k, n, src, src, dst, extra, 0.001)


acc2gm("case0", "f32", "f32", 128, 128, 32)
acc2gm("case1", "f32", "f32", 128, 128, 16)
acc2gm("case2", "f32", "f32", 31, 32, 15)
acc2gm("case3", "f32", "f16", 65, 128, 96)
acc2gm("case4", "f16", "f16", 73, 64, 32)
acc2gm("case5", "f32", "bf16", 13, 32, 25)
acc2gm("case6", "bf16", "bf16", 100, 222, 60)
acc2gm("case13", "i32", "i8", 44, 128, 27)
acc2gm("case16", "f16", "i8", 64, 64, 64, scalar=5)
acc2gm("case17", "i8", "i8", 31, 32, 26, scalar=2)
acc2gm("case18", "u8", "i8", 16, 32, 17, scalar=2)
acc2gm("case24", "i8", "f16", 25, 35, 32, scalar=2)
acc2gm("case25", "u8", "f32", 16, 20, 25, scalar=1)
acc2gm("case26", "f16", "f16", 49, 65, 37, scalar=3)
acc2gm("case27", "bf16", "f16", 160, 79, 51, scalar=3)
acc2gm("case_relu_1", "f32", "f32", 117, 97, 71, relu=True)
acc2gm("case_relu_21", "i8", "f16", 77, 34, 81, relu=True, scalar=2)

# ---- tdequant (tdequant/gen_data.py:51-53, 69-72: int8 and int16 sources, one scale and offset per row) ----------------------
for case, dt, rows, cols in (("case1", np.int8, 64, 64), ("case2", np.int16, 32, 128)):
    src = rng.integers(np.iinfo(dt).min, np.iinfo(dt).max + 1, (rows, cols)).astype(dt)
    scale, off = rng.uniform(0.01, 2.0, rows).astype(np.float32), rng.uniform(-20, 20, rows).astype(np.float32)
    put("tdequant", case, x1_gm=src, x2_gm=scale, bias_gm=off, golden=orc.tdequant(src, scale, off))
    line("tdequant", case, "dequant", rows, 0, cols, "i8" if dt == np.int8 else "i16", "f32", "f32", 0, 0.001)

# ---- tstore_quant (tstore_quant/main.cpp:112-130, tstore_quant/gen_data.py:46-64,170-186): a Vec tile of float / int32
# integers in [-5, 5) leaves through the quantising TSTORE; ND cases are [g0 g1 g2 g3][g4] row-major, DN cases
# [g3][g0 g1 g2 g4] stored column by column.  Words: scale in [0, 5), offset in [0, 512), a shift count, bit 46 for int8.
def quant_words(dst, count):
    out = []
    for _ in range(count):
        bits = int(np.float32(rng.uniform(0.0, 5.0)).view(np.uint32))
        out.append((int(rng.integers(0, 16)) << 32) | ((1 << 46) if dst == "i8" else 0) | (int(rng.integers(0, 512)) << 37) | bits)
    return np.array(out, np.uint64)


ST["i16"] = ob.ST_I16
for cid, (fmt, src, dst, g, vq, sat, relu) in enumerate([
        ("ND", "f32", "i8", (1, 1, 1, 2, 128), True, True, True), ("ND", "i32", "i16", (1, 2, 1, 23, 121), True, True, False),
        ("ND", "i32", "i8", (2, 2, 3, 23, 47), True, False, True), ("DN", "f32", "f16", (1, 1, 1, 4, 21), False, True, True),
        ("DN", "f32", "f16", (3, 1, 1, 1, 124), False, False, False), ("DN", "i32", "i8", (2, 1, 2, 32, 32), False, True, False),
        ("DN", "f32", "f16", (1, 1, 1, 16, 8), False, False, True), ("DN", "i32", "i16", (2, 2, 2, 16, 16), False, False, False),
        ("DN", "i32", "i8", (1, 2, 1, 16, 32), True, True, True), ("ND", "f32", "f16", (1, 1, 1, 16, 16), True, False, False)], 1):
    rows, cols = (g[0] * g[1] * g[2] * g[3], g[4]) if fmt == "ND" else (g[3], g[0] * g[1] * g[2] * g[4])
    x = rng.integers(-5, 5, (rows, cols)).astype(np.float32 if src == "f32" else np.int32)
    words = quant_words(dst, cols if vq else 1)
    golden = orc.store_quant(x, ST[dst], words, int(vq), relu=relu, saturate_inf=int(sat))
    if fmt == "DN":  # memory holds the matrix column by column
        x, golden = np.ascontiguousarray(x.T), np.ascontiguousarray(golden.T)
    case = f"{fmt}_{cid}"
    put("tstore_quant", case, input=x, quant=words, golden=golden)
    line("tstore_quant", case, "storeq_tile", rows, 0, cols, src, src, dst, f"{cid}:{int(sat)}", 0, f"q{cid}")


# ---- tquant (tquant/main.cpp:161-777: INT8 sym / asym, MXFP8 OCP / NV from f32, f16 and bf16 sources, the 2 x 256
# boundary patterns, the MXFP4 pattern families from f16 and bf16 sources, the NZ re-ordering of the exponents).  The
# value patterns are this script's own renderings of what the case names say; the goldens are the oracle's.
SRC = {"f32": ob.SRC_F32, "f16": ob.SRC_F16, "bf16": ob.SRC_BF16}


def as_source(x, kind):
    """The f32 values a source of that precision holds, and the array the kernel reads."""
    x = np.asarray(x, np.float32)
    if kind == "f16":
        with np.errstate(over="ignore"):
            h = x.astype(np.float16)
        return h.astype(np.float32), h.view(np.uint16)
    if kind == "bf16":
        bits = x.view(np.uint32)
        rounded = ((bits.astype(np.uint64) + 0x7FFF + ((bits >> 16) & 1)) >> 16).astype(np.uint16)
        rounded = np.where(np.isnan(x), np.uint16(0x7FC0), rounded)
        return (rounded.astype(np.uint32) << 16).view(np.float32), rounded
    return x, x


def tquant_case(case, x, kind, alg, nz=False):
    vals, stored = as_source(x, kind)
    codes, exp, _, _ = orc.tquant_mx(vals, alg, axis=1, src_kind=SRC[kind])
    rows, cols = vals.shape
    put("tquant", case, input=stored, golden=codes, golden_exp=orc.reorder_exp_zz(exp) if nz else exp)
    line("tquant", case, "tquant_mx", rows, 0, cols, kind, kind, "u8", f"{alg}:{int(nz)}", 0)


def pattern(name, rows, cols, fp4):
    top = 6.0 if fp4 else 448.0
    if name == "special":
        base = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, top, -top, top * 2, 1.0, -1.0, 0.5, 3.0], np.float32)
        return np.resize(base, (rows, cols)).astype(np.float32)
    if name == "subnormal":
        return (rng.standard_normal((rows, cols)) * 2.0 ** rng.integers(-149, -120, (rows, cols // 32)).repeat(32, 1)).astype(np.float32)
    if name == "rounding":  # values on and next to the ties between neighbouring codes of the group's binade
        steps = np.arange(rows * cols, dtype=np.float32).reshape(rows, cols) % 64
        x = (steps * 0.125 + 0.0625).astype(np.float32)
        x[:, ::3] = np.nextafter(x[:, ::3], np.float32(np.inf))
        x[:, 1::3] = -x[:, 1::3]
        return x
    if name in ("exp_a", "exp_b"):
        lo, hi = (-30, 30) if name == "exp_a" else (-126, 127)
        return (rng.uniform(1, 2, (rows, cols)) * 2.0 ** rng.integers(lo, hi, (rows, cols)) * rng.choice([-1, 1], (rows, cols))).astype(np.float32)
    x = (rng.standard_normal((rows, cols)) * 5).astype(np.float32)  # mixed
    x.ravel()[::7] = 0.0
    x.ravel()[3::11] *= np.float32(1e-30)
    x.ravel()[5::13] *= np.float32(1e30)
    x.ravel()[17::97] = np.nan
    x.ravel()[29::101] = -np.inf
    return x


q8 = (rng.standard_normal((64, 128)) * 40).astype(np.float32)
q8.ravel()[::5] = np.round(q8.ravel()[::5]) + 0.5
q8_scale, q8_off = rng.uniform(0.5, 4.0, 64).astype(np.float32), rng.uniform(0, 200, 64).astype(np.float32)
put("tquant", "Int8Sym", input=q8, scale=q8_scale, golden=orc.tquant_int8(q8, q8_scale))
line("tquant", "Int8Sym", "tquant_i8", 64, 0, 128, "f32", "f32", "i8", 0, 0)
put("tquant", "Int8Asym", input=q8, scale=q8_scale, offset=q8_off, golden=orc.tquant_int8(q8, q8_scale, q8_off))
line("tquant", "Int8Asym", "tquant_i8", 64, 0, 128, "f32", "f32", "u8", 1, 0)
for kind, tag in (("f32", ""), ("f16", "FP16"), ("bf16", "BF16")):
    tquant_case(f"MxFp8{tag}Nd", (rng.standard_normal((32, 128)) * 10 ** rng.uniform(-3, 3, (32, 1))).astype(np.float32), kind, 0)
    tquant_case(f"MxFp8{tag}Nz", (rng.standard_normal((32, 128)) * 10 ** rng.uniform(-3, 3, (32, 1))).astype(np.float32), kind, 0, nz=True)
tquant_case("MxFp8NvNd", (rng.standard_normal((32, 128)) * 10 ** rng.uniform(-3, 3, (32, 1))).astype(np.float32), "f32", 1)
edges = np.array([0.0, -0.0, 1e-45, 2.0 ** -130, np.nextafter(np.float32(448), 0), 448.0, -448.0, np.nextafter(np.float32(448), np.inf),
                  896.0, np.inf, -np.inf, np.nan, 6.0, 0.75, 2.0 ** 127, -2.0 ** -126], np.float32)
for kind, alg, tag in (("f32", 0, "OcpFp32"), ("f32", 1, "NvFp32"), ("f16", 1, "NvFp16"), ("bf16", 1, "NvBf16")):
    tquant_case(f"MxFp8{tag}Boundary2x256", np.resize(edges, (2, 256)).astype(np.float32), kind, alg)
for kind, tag in (("f16", "Fp16"), ("bf16", "Bf16")):
    for name, label in (("special", "Special"), ("subnormal", "Subnormal"), ("rounding", "Rounding"), ("exp_a", "ExpRandomA"),
                        ("exp_b", "ExpRandomB"), ("mixed", "Mixed")):
        tquant_case(f"MxFp4E2M1{tag}Nd{label}", pattern(name, 2, 256, True), kind, 2)
    tquant_case(f"MxFp4E2M1{tag}NdMixed32x1024", pattern("mixed", 32, 1024, True), kind, 2)
    for name, label in (("special", "Special"), ("rounding", "Rounding"), ("mixed", "Mixed")):
        tquant_case(f"MxFp4E2M1NV{tag}Nd{label}", pattern(name, 2, 256, True), kind, 3)

np.savez_compressed(os.path.join(HERE, "runner_cases.npz"), **arrays)
with open(os.path.join(HERE, "runner_cases.txt"), "w") as f:
    f.write("# suite case op m k n a_type b_type c_type extra eps pto_kernel   (written by gen_runner_cases.py)\n")
    f.write("\n".join(manifest) + "\n")
print(len(manifest), "cases,", sum(a.nbytes for a in arrays.values()), "bytes of arrays")
