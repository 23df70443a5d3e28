"""Throughput of the PTO tile-matmul hot path on one MI355X, with roofline fraction and a CPU baseline.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--settle-ms T] [--no-cpu] [--no-extra] [--only N] [--published] [--calibrate-copy]

A "step" is one TLOAD -> TMATMUL_ACC -> TSTORE pass over one synthetic batch.  The headline workload is
BASELINE.json configs[1] (bf16 GEMM, M = N = K = 4096, A row-major, B column-major, N(0,1) * 0.02, fp32 accumulate,
bf16 output); inputs are resident in HBM before the timed region.  The other configs are measured once each after the
headline and reported under "per_config" (the metric is "per GEMM config").  One JSON line goes to stdout.
"""
import argparse
import json
import os
import sys
import time

import numpy as np
import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
import __graft_entry__ as ge  # noqa: E402

METRIC = "TFLOP/s (or GB/s) + % of MI355X roofline per GEMM config, 1 GPU"
PEAK_TFLOPS = {"bf16": 2500.0, "f16": 2500.0, "int8": 5000.0, "fp8": 5000.0, "fp4": 10100.0}
PEAK_HBM_GBPS = 8000.0
DEV = "cuda:0"

# HBM bytes per launch of the headline kernel from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (scaled by a copy kernel of
# known size: FETCH_SIZE x 2.000, WRITE_SIZE x 1.000), see profiles/gemm_tile_dtl_256x256_bf16_4096cubed.md.
HEADLINE_TRAFFIC_BYTES = 235_224_064


class Events:
    """HIP events recorded on torch's current stream through the library's C ABI."""

    def __init__(self, pa):
        import ctypes as C
        self.C, self.lib = C, pa.lib()
        self.e0, self.e1 = C.c_void_p(), C.c_void_p()
        assert self.lib.ptoamd_event_create(C.byref(self.e0)) == 0 and self.lib.ptoamd_event_create(C.byref(self.e1)) == 0

    def _stream(self):
        return self.C.c_void_p(torch.cuda.current_stream().cuda_stream)

    def start(self):
        assert self.lib.ptoamd_event_record(self.e0, self._stream()) == 0

    def stop_ms(self):
        assert self.lib.ptoamd_event_record(self.e1, self._stream()) == 0
        assert self.lib.ptoamd_event_synchronize(self.e1) == 0
        ms = self.C.c_float()
        assert self.lib.ptoamd_event_elapsed_ms(self.C.byref(ms), self.e0, self.e1) == 0
        return float(ms.value)


# Untimed run-in before the warmup steps.  The clock governor of this part takes some 30 ms of continuous load to settle
# (the first 50 launches of the headline kernel average 132 us, launches 250+ a steady 111 us); a measurement taken
# during that ramp reports the governor, not the kernel.
SETTLE_MS = 100.0


def time_launches(ev, fn, steps, warmup):
    t_end = time.perf_counter() + SETTLE_MS / 1e3
    while SETTLE_MS > 0 and time.perf_counter() < t_end:
        for _ in range(20):
            fn()
        torch.cuda.synchronize()
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    ev.start()
    for _ in range(steps):
        fn()
    kernel_ms = ev.stop_ms() / steps
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    return wall_ms, kernel_ms


def randn_bf16(shape, gen, scale=1.0):
    return (torch.randn(shape, generator=gen, device=DEV) * scale).to(torch.bfloat16)


def config1(pa, ev, gen, steps, warmup):
    a = (torch.rand((512, 512), generator=gen, device=DEV) * 2 - 1).to(torch.float16)
    b = (torch.rand((512, 512), generator=gen, device=DEV) * 2 - 1).to(torch.float16)
    out = torch.empty((512, 512), dtype=torch.float32, device=DEV)
    wall, ker = time_launches(ev, lambda: pa.gemm(a, b, pa.F16, pa.F32, pa.B_ND, out=out), steps, warmup)
    flops = 2 * 512 ** 3
    return dict(config="configs[0] fp16 512^3 -> fp32, B row-major", kernel=pa.last_kernel(), ms=ker, wall_ms=wall,
                tflops=flops / ker / 1e9, bound="latency", frac_of_peak=flops / ker / 1e9 / PEAK_TFLOPS["f16"],
                cpu="config1")


def config3(pa, ev, gen, steps, warmup):
    m, n, k = 2048, 8192, 8192
    a = torch.randint(-127, 128, (m, k), generator=gen, device=DEV, dtype=torch.int8)
    b = torch.randint(-127, 128, (n, k), generator=gen, device=DEV, dtype=torch.int8)
    sa = torch.rand(m, generator=gen, device=DEV) * 0.01 + 0.001
    sb = torch.rand(n, generator=gen, device=DEV) * 0.01 + 0.001
    out = torch.empty((m, n), dtype=torch.bfloat16, device=DEV)
    wall, ker = time_launches(ev, lambda: pa.gemm_w8a8(a, b, sa, sb, out=out), steps, warmup)
    ops = 2 * m * n * k
    return dict(config="configs[2] W8A8 int8 2048x8192x8192 -> bf16, fused dequant", kernel=pa.last_kernel(), ms=ker,
                wall_ms=wall, tflops=ops / ker / 1e9, bound="mfma", frac_of_peak=ops / ker / 1e9 / PEAK_TFLOPS["int8"],
                cpu="config3")


def config4(pa, ev, gen, steps, warmup):
    m, n, k = 4096, 14336, 4096
    a, sa = pa.tquant_mx(torch.randn((m, k), generator=gen, device=DEV), pa.OCP_MXFP8, want_aux=False)
    b, sb = pa.tquant_mx(torch.randn((n, k), generator=gen, device=DEV), pa.OCP_MXFP8, want_aux=False)
    out = torch.empty((m, n), dtype=torch.bfloat16, device=DEV)
    wall, ker = time_launches(ev, lambda: pa.gemm_mx(a, b, sa, sb, m, n, k, pa.E4M3, pa.E4M3, pa.BF16, out=out), steps,
                              warmup)
    flops = 2 * m * n * k
    return dict(config="configs[3] MXFP8 E4M3 4096x14336x4096 -> bf16", kernel=pa.last_kernel(), ms=ker, wall_ms=wall,
                tflops=flops / ker / 1e9, bound="mfma", frac_of_peak=flops / ker / 1e9 / PEAK_TFLOPS["fp8"], cpu="config4")


def config5(pa, ev, gen, steps, warmup):
    m, n, k = 16, 28672, 8192
    a = randn_bf16((m, k), gen)
    # four weight copies (4 x 125 MB) rotated between launches so every launch streams from HBM, not the 256 MB MALL
    copies = []
    for _ in range(4):
        w, sw = pa.tquant_mx(torch.randn((n, k), generator=gen, device=DEV), pa.OCP_MXFP4, want_aux=False)
        copies.append((w, sw))
    out = torch.empty((m, n), dtype=torch.bfloat16, device=DEV)
    state = {"i": 0}

    def step():
        w, sw = copies[state["i"] % 4]
        state["i"] += 1
        pa.gemv_mxfp4(a, w, sw, n, k, pa.BF16, out=out)

    wall, ker = time_launches(ev, step, steps, warmup)
    nbytes = n * k // 2 + n * k // 32 + m * k * 2 + m * n * 2
    return dict(config="configs[4] MXFP4 decode GEMV 16x28672x8192 -> bf16 (weights rotated over 4 copies)",
                kernel=pa.last_kernel(), ms=ker, wall_ms=wall, gbps=nbytes / ker / 1e6, bound="hbm",
                frac_of_peak=nbytes / ker / 1e6 / PEAK_HBM_GBPS, cpu="config5")


def config5_packed(pa, ev, gen, steps, warmup):
    """configs[4] with the weights packed ahead of time into the kernel's stage order (same sums, same bits)."""
    m, n, k = 16, 28672, 8192
    a = randn_bf16((m, k), gen)
    copies = []
    for _ in range(4):
        w, sw = pa.tquant_mx(torch.randn((n, k), generator=gen, device=DEV), pa.OCP_MXFP4, want_aux=False)
        copies.append(pa.gemv_mxfp4_pack(w, sw, n, k))
    ref = pa.gemv_mxfp4(a, w, sw, n, k, pa.BF16)
    out = torch.empty((m, n), dtype=torch.bfloat16, device=DEV)
    pa.gemv_mxfp4_packed(a, copies[3], n, k, pa.BF16, out=out)
    if not torch.equal(out, ref):
        raise RuntimeError("the packed GEMV does not reproduce the plain one")
    del w, sw
    state = {"i": 0}

    def step():
        packed = copies[state["i"] % 4]
        state["i"] += 1
        pa.gemv_mxfp4_packed(a, packed, n, k, pa.BF16, out=out)

    wall, ker = time_launches(ev, step, steps, warmup)
    nbytes = n * k // 2 + n * k // 32 + m * k * 2 + m * n * 2
    return dict(config="configs[4] MXFP4 decode GEMV 16x28672x8192 -> bf16, weights pre-packed by ptoamd_gemv_mxfp4_pack "
                       "(rotated over 4 copies)",
                kernel=pa.last_kernel(), ms=ker, wall_ms=wall, gbps=nbytes / ker / 1e6, bound="hbm",
                frac_of_peak=nbytes / ker / 1e6 / PEAK_HBM_GBPS, cpu="config5")


def _pto_lib(name):
    """A library of kernels written in the PTO tile ISA against the header layer (pto-isa-mirror_amd/kernels/<name>.hip)."""
    import ctypes as C
    path = os.path.join(ge.PKG_DIR, "lib", f"libpto_{name}.so")
    if not os.path.exists(path):
        raise RuntimeError(f"{path} is missing: build it with `make -C pto-isa-mirror_amd`")
    return C, C.CDLL(path)


def pto_api_bf16(pa, ev, gen, steps, warmup):
    """configs[1] through the reference's own programming interface: the GEMM of kernels/gemm_performance.hip is a core
    program of TASSIGN / TLOAD / TEXTRACT / TMATMUL(_ACC) / TSTORE calls, compiled against include/pto."""
    C, lib = _pto_lib("gemm_performance")
    m = n = k = 4096
    a = randn_bf16((m, k), gen, 0.02)
    b = randn_bf16((n, k), gen, 0.02)
    out = torch.empty((m, n), dtype=torch.bfloat16, device=DEV)

    def step():
        rc = lib.pto_gemm_performance(0, C.c_void_p(out.data_ptr()), C.c_void_p(a.data_ptr()), C.c_void_p(b.data_ptr()),
                                      C.c_void_p(torch.cuda.current_stream().cuda_stream))
        assert rc == 0, rc

    wall, ker = time_launches(ev, step, steps, warmup)
    ref = pa.gemm(a, b, pa.BF16, pa.BF16, pa.B_DN)
    torch.cuda.synchronize()
    assert lib.pto_gemm_performance_status() == 0 and torch.equal(out, ref), "the PTO-style GEMM and the launcher disagree"
    flops = 2 * m * n * k
    return dict(config="configs[1] bf16 4096^3 -> bf16 written in the PTO tile ISA (TLOAD / TEXTRACT / TMATMUL_ACC / TSTORE, "
                       "256 x 256 tiles, K panels of 64)", kernel="GemmPerformance<bf16, 256, 256, 64> (header layer)", ms=ker,
                wall_ms=wall, tflops=flops / ker / 1e9, bound="mfma", frac_of_peak=flops / ker / 1e9 / PEAK_TFLOPS["bf16"],
                cpu="headline")


def pto_api_mxfp8(pa, ev, gen, steps, warmup):
    """configs[3] through the reference's own programming interface: kernels/mxmatmul_performance.hip is a core program of
    TLOAD / TEXTRACT / TMATMUL_MX / TSTORE calls (operand panels and E8M0 scale tiles double-buffered in L1)."""
    C, lib = _pto_lib("mxmatmul_performance")
    m, n, k = 4096, 14336, 4096
    a, sa = pa.tquant_mx(torch.randn((m, k), generator=gen, device=DEV), pa.OCP_MXFP8, want_aux=False)
    b, sb = pa.tquant_mx(torch.randn((n, k), generator=gen, device=DEV), pa.OCP_MXFP8, want_aux=False)
    out = torch.empty((m, n), dtype=torch.bfloat16, device=DEV)

    def step():
        rc = lib.pto_mxmatmul_performance(0, *(C.c_void_p(t.data_ptr()) for t in (out, a, b, sa, sb)),
                                          C.c_void_p(torch.cuda.current_stream().cuda_stream))
        assert rc == 0, rc

    wall, ker = time_launches(ev, step, steps, warmup)
    ref = pa.gemm_mx(a, b, sa, sb, m, n, k, pa.E4M3, pa.E4M3, pa.BF16)
    torch.cuda.synchronize()
    assert lib.pto_mxmatmul_performance_status() == 0 and torch.equal(out, ref), "the PTO-style MX GEMM and the launcher disagree"
    flops = 2 * m * n * k
    return dict(config="configs[3] MXFP8 E4M3 4096x14336x4096 -> bf16 written in the PTO tile ISA (TLOAD / TEXTRACT / TMATMUL_MX / "
                       "TSTORE, 256 x 256 tiles, K panels of 128, scale tiles of 16 K-groups)",
                kernel="MxMatmulPerformance<e4m3, 256, 256, 128> (header layer)", ms=ker, wall_ms=wall, tflops=flops / ker / 1e9,
                bound="mfma", frac_of_peak=flops / ker / 1e9 / PEAK_TFLOPS["fp8"], cpu="config4")


def pto_api_mxfp4(pa, ev, gen, steps, warmup):
    """MXFP4 2048 x 8192 (K) x 8192 -> bf16 (a shape the reference publishes a time for) through the same core program as
    pto_api_mxfp8, on packed E2M1 operand tiles."""
    C, lib = _pto_lib("mxmatmul_performance")
    m, n, k = 2048, 8192, 8192
    a, sa = pa.tquant_mx(torch.randn((m, k), generator=gen, device=DEV), pa.OCP_MXFP4, want_aux=False)
    b, sb = pa.tquant_mx(torch.randn((n, k), generator=gen, device=DEV), pa.OCP_MXFP4, want_aux=False)
    out = torch.empty((m, n), dtype=torch.bfloat16, device=DEV)

    def step():
        rc = lib.pto_mxmatmul_performance(4, *(C.c_void_p(t.data_ptr()) for t in (out, a, b, sa, sb)),
                                          C.c_void_p(torch.cuda.current_stream().cuda_stream))
        assert rc == 0, rc

    wall, ker = time_launches(ev, step, steps, warmup)
    ref = pa.gemm_mx(a, b, sa, sb, m, n, k, pa.E2M1, pa.E2M1, pa.BF16)
    launcher = pa.last_kernel()
    torch.cuda.synchronize()
    assert lib.pto_mxmatmul_performance_status() == 0 and torch.equal(out, ref), "the PTO-style MXFP4 GEMM and the launcher disagree"
    lwall, lker = time_launches(ev, lambda: pa.gemm_mx(a, b, sa, sb, m, n, k, pa.E2M1, pa.E2M1, pa.BF16, out=out), steps, warmup)
    flops = 2 * m * n * k
    return dict(config="MXFP4 E2M1 2048x8192x8192 (m, k, n) -> bf16 written in the PTO tile ISA (TLOAD / TEXTRACT / TMATMUL_MX / TSTORE, "
                       "256 x 256 tiles, K panels of 256 codes, scale tiles of 16 K-groups)",
                kernel="MxMatmulPerformance<e2m1, 256, 256, 256> (header layer)", ms=ker, wall_ms=wall, tflops=flops / ker / 1e9,
                bound="mfma", frac_of_peak=flops / ker / 1e9 / PEAK_TFLOPS["fp4"], launcher_kernel=launcher, launcher_ms=lker,
                cpu=None)


def pto_api_config1(pa, ev, gen, steps, warmup):
    """configs[0] through the tile ISA (kernels/gemm_tiled.hip): 128 x 128 tiles as BASELINE.json words it, and 64 x 64."""
    C, lib = _pto_lib("gemm_tiled")
    a = (torch.rand((512, 512), generator=gen, device=DEV) * 2 - 1).to(torch.float16)
    b = (torch.rand((512, 512), generator=gen, device=DEV) * 2 - 1).to(torch.float16)
    out = torch.empty((512, 512), dtype=torch.float32, device=DEV)
    res = {}
    for case in (0, 1):
        def step():
            rc = lib.pto_gemm_tiled(case, C.c_void_p(out.data_ptr()), C.c_void_p(a.data_ptr()), C.c_void_p(b.data_ptr()),
                                    C.c_void_p(torch.cuda.current_stream().cuda_stream))
            assert rc == 0, rc
        res[case] = time_launches(ev, step, steps, warmup)
    flops = 2 * 512 ** 3
    wall, ker = res[0]
    return dict(config="configs[0] fp16 512^3 -> fp32, B row-major, written in the PTO tile ISA (TLOAD / TMOV / TMATMUL_ACC / "
                       "TSTORE, 128 x 128 tiles, K slabs of 64, 16 cores)", kernel="RunTiledGemm<f16, 128, 128, 64> (header layer)",
                ms=ker, wall_ms=wall, tflops=flops / ker / 1e9, bound="latency",
                frac_of_peak=flops / ker / 1e9 / PEAK_TFLOPS["f16"], ms_with_64x64_tiles=res[1][1], cpu="config1")


def _elementwise(name, kernel, nbytes, wall, ker, cpu):
    return dict(config=name, kernel=kernel, ms=ker, wall_ms=wall, gbps=nbytes / ker / 1e6, bound="hbm",
                frac_of_peak=nbytes / ker / 1e6 / PEAK_HBM_GBPS, algorithmic_bytes=nbytes, cpu=cpu)


def _rotating(make, copies):
    """`copies` instances of an input, used in turn, so that every launch reads from HBM and not from the 256 MB MALL."""
    items = [make() for _ in range(copies)]
    state = {"i": 0}

    def nxt():
        state["i"] += 1
        return items[state["i"] % copies]
    return nxt


def quant_mxfp8(pa, ev, gen, steps, warmup):
    rows, cols = 14336, 4096  # the weight matrix of configs[3]
    src = _rotating(lambda: randn_bf16((rows, cols), gen), 4)
    out = (torch.empty((rows, cols), dtype=torch.uint8, device=DEV), torch.empty((rows, cols // 32), dtype=torch.uint8, device=DEV))
    wall, ker = time_launches(ev, lambda: pa.tquant_mx(src(), pa.OCP_MXFP8, want_aux=False, out=out), steps, warmup)
    return _elementwise("TQUANT OCP-MXFP8, bf16 14336x4096 -> E4M3 codes + E8M0 exponents", "tquant_mx_rows",
                        rows * cols * 2 + rows * cols + rows * cols // 32, wall, ker, "quant:mxfp8")


def quant_mxfp4(pa, ev, gen, steps, warmup):
    rows, cols = 28672, 8192  # the weight matrix of configs[4]; 470 MB of bf16, larger than the MALL
    src = randn_bf16((rows, cols), gen)
    out = (torch.empty((rows, cols // 2), dtype=torch.uint8, device=DEV), torch.empty((rows, cols // 32), dtype=torch.uint8, device=DEV))
    wall, ker = time_launches(ev, lambda: pa.tquant_mx(src, pa.OCP_MXFP4, want_aux=False, out=out), steps, warmup)
    return _elementwise("TQUANT OCP-MXFP4, bf16 28672x8192 -> E2M1 codes + E8M0 exponents", "tquant_mx_rows",
                        rows * cols * 2 + rows * cols // 2 + rows * cols // 32, wall, ker, "quant:mxfp4")


def quant_int8(pa, ev, gen, steps, warmup):
    rows, cols = 2048, 8192  # the activation matrix of configs[2]
    src = _rotating(lambda: torch.randn((rows, cols), generator=gen, device=DEV), 8)
    scale = torch.rand(rows, generator=gen, device=DEV) * 20 + 1
    out = torch.empty((rows, cols), dtype=torch.int8, device=DEV)
    wall, ker = time_launches(ev, lambda: pa.tquant_int8(src(), scale, out=out), steps, warmup)
    return _elementwise("TQUANT INT8_SYM, f32 2048x8192 -> int8", "tquant_int8", rows * cols * 5 + rows * 4, wall, ker,
                        "quant:int8")


def dequant_int8(pa, ev, gen, steps, warmup):
    rows, cols = 2048, 8192
    src = _rotating(lambda: torch.randint(-128, 128, (rows, cols), generator=gen, device=DEV, dtype=torch.int8), 8)
    scale = torch.rand(rows, generator=gen, device=DEV) + 0.5
    offset = torch.rand(rows, generator=gen, device=DEV) * 10
    out = torch.empty((rows, cols), dtype=torch.float32, device=DEV)
    wall, ker = time_launches(ev, lambda: pa.tdequant(src(), scale, offset, out=out), steps, warmup)
    return _elementwise("TDEQUANT int8 2048x8192 -> f32", "tdequant", rows * cols * 5 + rows * 8, wall, ker, "quant:dequant")


# Shapes the reference publishes wall times for, on its own hardware (Ascend A3 / A5 NPUs: other silicon, so context and
# not a baseline).  kernels/manual/a2a3/gemm_performance/README.md:83-86, kernels/manual/a5/matmul_mxfp8_performance/
# README.md:95-98 and kernels/manual/a5/matmul_mxfp4_performance/README.md:95-100 of the reference.
PUBLISHED = [
    ("f16", 1536, 1536, 1536, 0.0388, "Ascend A3, 24 cores"), ("f16", 3072, 3072, 3072, 0.2067, "Ascend A3, 24 cores"),
    ("f16", 6144, 6144, 6144, 1.5060, "Ascend A3, 24 cores"), ("f16", 7680, 7680, 7680, 3.1680, "Ascend A3, 24 cores"),
    ("mxfp8", 2048, 2048, 2048, 0.0383, "Ascend A5, 32 cores"), ("mxfp8", 4096, 4096, 4096, 0.1879, "Ascend A5, 32 cores"),
    ("mxfp8", 6144, 6144, 6144, 0.6020, "Ascend A5, 32 cores"), ("mxfp8", 8192, 8192, 8192, 1.4749, "Ascend A5, 32 cores"),
    ("mxfp4", 2048, 2048, 2048, 0.0425, "Ascend A5, 32 cores"), ("mxfp4", 2048, 4096, 4096, 0.1003, "Ascend A5, 32 cores"),
    ("mxfp4", 4096, 1024, 8192, 0.1226, "Ascend A5, 32 cores"), ("mxfp4", 1024, 12288, 4096, 0.1377, "Ascend A5, 32 cores"),
    ("mxfp4", 2048, 8192, 8192, 0.3489, "Ascend A5, 32 cores"), ("mxfp4", 2040, 8192, 8100, 0.3773, "Ascend A5, 32 cores"),
]


def _finite_fp8(shape, gen, exp_mask):
    """Random fp8 codes with no inf / NaN pattern (the all-ones exponent field is cleared to a finite one)."""
    x = torch.randint(0, 256, shape, generator=gen, device=DEV, dtype=torch.uint8)
    return torch.where((x & exp_mask) == exp_mask, x & 0xBF, x)


def published_shapes(pa, ev, gen, steps, warmup):
    """The reference's own published benchmark shapes (m, k, n) on this GPU: fp16 -> fp32 GEMM, MXFP8 (E5M2) -> bf16 and
    MXFP4 (E2M1) -> bf16, each with the operand layouts of its README (A row-major, B column-major, scales per 32 K)."""
    rows = []
    for kind, m, k, n, ref_ms, hw in PUBLISHED:
        if kind == "f16":
            a = (torch.randn((m, k), generator=gen, device=DEV) * 0.05).to(torch.float16)
            b = (torch.randn((n, k), generator=gen, device=DEV) * 0.05).to(torch.float16)
            out = torch.empty((m, n), dtype=torch.float32, device=DEV)
            fn = lambda: pa.gemm(a, b, pa.F16, pa.F32, pa.B_DN, out=out)
            peak, name = PEAK_TFLOPS["f16"], "fp16 -> fp32 GEMM"
        else:
            fp4 = kind == "mxfp4"
            kb = k // 2 if fp4 else k
            a = torch.randint(0, 256, (m, kb), generator=gen, device=DEV, dtype=torch.uint8) if fp4 else \
                _finite_fp8((m, kb), gen, 0x7C)
            b = torch.randint(0, 256, (n, kb), generator=gen, device=DEV, dtype=torch.uint8) if fp4 else \
                _finite_fp8((n, kb), gen, 0x7C)
            sa = torch.randint(124, 131, (m, k // 32), generator=gen, device=DEV, dtype=torch.uint8)
            sb = torch.randint(124, 131, (n, k // 32), generator=gen, device=DEV, dtype=torch.uint8)
            out = torch.empty((m, n), dtype=torch.bfloat16, device=DEV)
            et = pa.E2M1 if fp4 else pa.E5M2
            fn = lambda: pa.gemm_mx(a, b, sa, sb, m, n, k, et, et, pa.BF16, out=out)
            peak, name = PEAK_TFLOPS["fp4" if fp4 else "fp8"], "MXFP4 E2M1 -> bf16" if fp4 else "MXFP8 E5M2 -> bf16"
        wall, ker = time_launches(ev, fn, steps, warmup)
        flops = 2.0 * m * n * k
        rows.append(dict(shape=f"{name} (m, k, n) = ({m}, {k}, {n})", kernel=pa.last_kernel(), ms=ker, wall_ms=wall,
                         tflops=flops / ker / 1e9, frac_of_peak=flops / ker / 1e9 / peak, reference_ms=ref_ms,
                         reference_hardware=hw))
        del a, b, out
        torch.cuda.empty_cache()
    return rows


class CpuSide:
    """The CPU leg: the reference CPU simulator itself where its compiled form is present (oracle/_ref, built from the
    reference's headers: TLOAD / TMOV / TMATMUL(_ACC) / TSTORE on tiles of up to 256 x 256, K walked in slabs), else the
    plain-C port of it (oracle/pto_oracle.c: per-element fractal addressing, per-TMATMUL thread fan-out).  Every figure
    says whether the whole shape was run ("measured") or a slab of its output tiles ("extrapolated": output tiles are
    independent and equal, so the full-shape time is the slab's time times the tile count)."""

    def __init__(self):
        from oracle import binding as ob
        self.ob = ob
        self.ref = ob.RefLib() if ob.RefLib.available() else None
        self.orc = ob.Oracle()
        self.threads = min(os.cpu_count() or 1, 16)
        self.kind = "reference" if self.ref is not None else "port"
        self.rng = np.random.default_rng(0)

    def _entry(self, work, dt, unit, sample, extent, full_s):
        return {"value": work / dt / 1e12, "unit": unit, "cores": self.threads, "kind": self.kind, "extent": extent,
                "full_shape_s": full_s, "sample": sample}

    def _f16(self, shape, scale=1.0):
        return (self.rng.standard_normal(shape) * scale).astype(np.float16).view(np.uint16)

    def _bf16(self, shape, scale=1.0):
        return ((self.rng.standard_normal(shape) * scale).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)

    def _bf16_values(self, shape):
        return (self._bf16(shape).astype(np.uint32) << 16).view(np.float32)

    def _bounded(self, run_tile, budget_s, at_least):
        tiles, t0 = 0, time.perf_counter()
        while tiles < at_least or time.perf_counter() - t0 < budget_s:
            run_tile(tiles)
            tiles += 1
        return tiles, time.perf_counter() - t0

    def headline(self):
        """configs[1]: 96 of the 256 output tiles of 256 x 256 x 4096 (one A row panel against 96 B column panels)."""
        k = 4096
        if self.ref is not None:
            # the simulator's bfloat16_t degrades to _Float16 without <stdfloat>: same loops and fp32 fma on fp16 inputs
            m, n, cols = 256, 256, 96
            a = self._f16((m, k), 0.02)
            b = self._f16((cols * n, k), 0.02)
            t0 = time.perf_counter()
            for j in range(cols):
                self.ref.gemm("f16", a, b[j * n:(j + 1) * n], b_dn=True, kstep=512)
            dt = time.perf_counter() - t0
            flop = 2.0 * m * n * cols * k
            return self._entry(flop, dt, "TFLOP/s",
                               f"{cols} independent 256 x 256 x 4096 output tiles of the workload (one A row panel against "
                               f"{cols} B column panels), fp16 stand-in for bf16 ({flop / 1e9:.1f} GFLOP) in {dt:.1f} s; the "
                               f"full 4096^3 is 256 such tiles and extrapolates to {dt * 256 / cols:.0f} s",
                               "extrapolated", dt * 256 / cols)
        m, n = 256, 4096
        a, b = self._bf16((m, k), 0.02), self._bf16((n, k), 0.02)
        t0 = time.perf_counter()
        _, self.threads = self.orc.sim_gemm_tiled(a, b, 1, self.ob.ST_BF16, b_dn=True, max_threads=16)
        dt = time.perf_counter() - t0
        return self._entry(2.0 * m * n * k, dt, "TFLOP/s",
                           f"256 of 4096 output rows x N=4096 x K=4096 (8.6 GFLOP) in {dt:.1f} s; full 4096^3 extrapolates "
                           f"to {dt * 16:.0f} s", "extrapolated", dt * 16)

    def config1(self):
        """configs[0] in full: fp16 512^3 -> fp32, B row-major, 128 x 128 output tiles, K walked in slabs of 64."""
        a = (self.rng.random((512, 512)) * 2 - 1).astype(np.float16).view(np.uint16)
        b = (self.rng.random((512, 512)) * 2 - 1).astype(np.float16).view(np.uint16)
        bcols = [np.ascontiguousarray(b[:, j:j + 128]) for j in range(0, 512, 128)]
        times = []
        for _ in range(4):  # one warm-up, then the median of three
            t0 = time.perf_counter()
            if self.ref is not None:
                for i in range(0, 512, 128):
                    for bj in bcols:
                        self.ref.gemm("f16", a[i:i + 128], bj, b_dn=False, kstep=64)
            else:
                _, self.threads = self.orc.sim_gemm_tiled(a, b, 0, self.ob.ST_F32, b_dn=False, max_threads=16)
            times.append(time.perf_counter() - t0)
        dt = float(np.median(times[1:]))
        return self._entry(2.0 * 512 ** 3, dt, "TFLOP/s",
                           f"the whole 512^3 as 16 tiles of 128 x 128 with K slabs of 64: median of 3 runs after one warm-up, "
                           f"{dt:.3f} s", "measured", dt)

    def config3(self, budget_s=4.0):
        """configs[2]: the int32 accumulators of 256 x 256 x 8192 tiles.  The dequantising drain is left out: one multiply
        per output element against 8192 multiply-adds."""
        m, n, k = 2048, 8192, 8192
        a = self.rng.integers(-127, 128, (256, k), dtype=np.int8)
        b = self.rng.integers(-127, 128, (256, k), dtype=np.int8)

        def tile(_):
            if self.ref is not None:
                self.ref.gemm("i8", a, b, b_dn=True, kstep=512)
            else:
                _, self.threads = self.orc.sim_gemm_tiled(a, b, 2, self.ob.ST_I32, b_dn=True, max_threads=16)
        tiles, dt = self._bounded(tile, budget_s, 2)
        total = (m // 256) * (n // 256)
        return self._entry(2.0 * 256 * 256 * k * tiles, dt, "TOP/s",
                           f"{tiles} of the {total} output tiles of 256 x 256 x 8192 (int8 -> int32 accumulators) in "
                           f"{dt:.1f} s", "extrapolated", dt * total / tiles)

    def config4(self, budget_s=4.0):
        """configs[3]: TMATMUL_MX on 256 x 256 tiles; K = 4096 is eight accumulating calls of 512 in the reference."""
        m, n, k = 4096, 14336, 4096
        a = self.rng.integers(0, 0x7F, (256, k), dtype=np.uint8)  # finite E4M3 codes
        b = self.rng.integers(0, 0x7F, (256, k), dtype=np.uint8)
        sa = self.rng.integers(125, 130, (256, k // 32), dtype=np.uint8)
        sb = self.rng.integers(125, 130, (256, k // 32), dtype=np.uint8)
        slabs = [(np.ascontiguousarray(a[:, k0:k0 + 512]), np.ascontiguousarray(b[:, k0:k0 + 512]),
                  np.ascontiguousarray(sa[:, k0 // 32:k0 // 32 + 16]), np.ascontiguousarray(sb[:, k0 // 32:k0 // 32 + 16]))
                 for k0 in range(0, k, 512)]

        def tile(_):
            if self.ref is not None:
                acc = None
                for sl in slabs:  # scale layouts MX_A_DN / MX_B_DN, B column-major
                    acc = self.ref.gemm_mx(sl[0], sl[1], sl[2], sl[3], 256, 512, 256, 0, 2, True, cin=acc)
            else:
                _, self.threads = self.orc.sim_gemm_mx_tiled(a, b, sa, sb, 256, k, 256, self.ob.E4M3, self.ob.E4M3,
                                                             self.ob.ST_BF16, max_threads=16)
        tiles, dt = self._bounded(tile, budget_s, 1)
        total = (m // 256) * (n // 256)
        return self._entry(2.0 * 256 * 256 * k * tiles, dt, "TFLOP/s",
                           f"{tiles} of the {total} output tiles of 256 x 256 x 4096 (E4M3 codes, E8M0 scales per 32 K) in "
                           f"{dt:.1f} s", "extrapolated", dt * total / tiles)

    def config5(self):
        """configs[4] in full: 16 x 28672 x 8192.  The reference has no matmul of bf16 activations by MXFP4 weights; its
        CPU form of this product is TMATMUL on the weights already expanded to 16-bit floats (every E2M1 x 2^e value is
        exact there), so that is what is timed; the expansion itself is left out."""
        m, n, k = 16, 28672, 8192
        a = self._f16((m, k))
        w = self._f16((256, k))
        t0 = time.perf_counter()
        if self.ref is not None:
            for _ in range(n // 256):
                self.ref.gemm("f16", a, w, b_dn=True, kstep=512)
        else:
            for _ in range(n // 256):
                _, self.threads = self.orc.sim_gemm_tiled(a, w, 1, self.ob.ST_BF16, b_dn=True, max_threads=16)
        dt = time.perf_counter() - t0
        nbytes = n * k // 2 + n * k // 32 + m * k * 2 + m * n * 2
        e = self._entry(nbytes * 1e3, dt, "GB/s",
                        f"the whole 16 x 28672 x 8192 as {n // 256} column blocks of 256 weight rows, K slabs of 512, weights "
                        f"expanded to 16-bit floats beforehand: {dt:.1f} s ({2.0 * m * n * k / dt / 1e9:.2f} GFLOP/s); GB/s "
                        f"counts the same algorithmic bytes as the GPU figure", "measured", dt)
        return e

    def quant(self, what):
        """The elementwise kernels on a slab of rows through the port (the compiled reference holds TQUANT / TDEQUANT for
        a few fixed tile shapes only)."""
        ob, r = self.ob, self.rng
        if what == "mxfp8":
            rows, cols, full = 512, 4096, 14336
            src = self._bf16_values((rows, cols))
            fn = lambda: self.orc.tquant_mx(src, 0, axis=1, src_kind=ob.SRC_BF16)
            per_row = cols * 2 + cols + cols // 32
        elif what == "mxfp4":
            rows, cols, full = 256, 8192, 28672
            src = self._bf16_values((rows, cols))
            fn = lambda: self.orc.tquant_mx(src, 2, axis=1, src_kind=ob.SRC_BF16)
            per_row = cols * 2 + cols // 2 + cols // 32
        elif what == "int8":
            rows, cols, full = 2048, 8192, 2048
            src = r.standard_normal((rows, cols)).astype(np.float32)
            scale = (r.random(rows) * 20 + 1).astype(np.float32)
            fn = lambda: self.orc.tquant_int8(src, scale)
            per_row = cols * 5 + 4
        else:
            rows, cols, full = 2048, 8192, 2048
            src = r.integers(-128, 128, (rows, cols), dtype=np.int8)
            scale = (r.random(rows) + 0.5).astype(np.float32)
            offset = (r.random(rows) * 10).astype(np.float32)
            fn = lambda: self.orc.tdequant(src, scale, offset)
            per_row = cols * 5 + 8
        fn()
        times = []
        for _ in range(3):
            t0 = time.perf_counter()
            fn()
            times.append(time.perf_counter() - t0)
        dt = float(np.median(times))
        return {"value": rows * per_row / dt / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
                "extent": "measured" if rows == full else "extrapolated", "full_shape_s": dt * full / rows,
                "sample": f"{rows} of {full} rows x {cols} columns, scalar C restatement, median of 3 runs: {dt:.3f} s"}


def main():
    global SETTLE_MS
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--settle-ms", type=float, default=SETTLE_MS,
                    help="untimed run-in of the same launches before the warmup steps, for the GPU clock to settle")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extra", action="store_true", help="skip the per-config measurements after the headline")
    ap.add_argument("--only", type=int, choices=[0, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13], default=None,
                    help="measure just BASELINE.json configs[N] (a per_config entry) and print it: for profiling one kernel; "
                         "5-8 are the elementwise kernels (TQUANT MXFP8, TQUANT MXFP4, TQUANT INT8, TDEQUANT), 9, 10 and 11 "
                         "configs[1], configs[0] and configs[3] written in the PTO tile ISA, 12 configs[4] on pre-packed weights, 13 an MXFP4 GEMM in the tile ISA")
    ap.add_argument("--published", action="store_true",
                    help="measure only the shapes the reference publishes wall times for and print those rows")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one plain 256 MiB device copy (a kernel of known traffic, to scale rocprofv3 "
                         "FETCH_SIZE / WRITE_SIZE readings)")
    args = ap.parse_args()
    SETTLE_MS = args.settle_ms
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: every box of this build has one MI355X and the path needs no second "
                 "(output tiles are independent, so M or N shards need no exchange). Run with --gpus 1.")

    pa = ge.load_package()
    pa.init(0)
    ev = Events(pa)
    if args.calibrate_copy:
        src = torch.ones(64 * 1024 * 1024, dtype=torch.float32, device=DEV)  # 256 MiB read + 256 MiB written
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    gen = torch.Generator(device=DEV).manual_seed(1)
    if args.published:
        print(json.dumps(published_shapes(pa, ev, gen, args.steps, args.warmup)))
        return
    if args.only is not None:
        fn = {0: config1, 2: config3, 3: config4, 4: config5, 5: quant_mxfp8, 6: quant_mxfp4, 7: quant_int8,
              8: dequant_int8, 9: pto_api_bf16, 10: pto_api_config1, 11: pto_api_mxfp8, 12: config5_packed, 13: pto_api_mxfp4}[args.only]
        entry = fn(pa, ev, gen, args.steps, args.warmup)
        entry.pop("cpu", None)
        print(json.dumps(entry))
        return

    m = n = k = 4096
    a = randn_bf16((m, k), gen, 0.02)
    b = randn_bf16((n, k), gen, 0.02)
    out = torch.empty((m, n), dtype=torch.bfloat16, device=DEV)
    wall_ms, kernel_ms = time_launches(ev, lambda: pa.gemm(a, b, pa.BF16, pa.BF16, pa.B_DN, out=out), args.steps,
                                       args.warmup)
    kernel = pa.last_kernel()
    flops = 2 * m * n * k
    value = flops / wall_ms / 1e9
    achieved = flops / kernel_ms / 1e9
    line = {
        "metric": METRIC, "value": value, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": wall_ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "configs[1]: bf16 GEMM M=N=K=4096, A row-major, B column-major, N(0,1)*0.02, "
                               "fp32 accumulate, bf16 output", "kernel": kernel, "clock_settle_ms": SETTLE_MS},
        "roofline": {"bound": "mfma", "achieved": achieved, "peak": PEAK_TFLOPS["bf16"], "unit": "TFLOP/s",
                     "frac": achieved / PEAK_TFLOPS["bf16"], "traffic": HEADLINE_TRAFFIC_BYTES,
                     "kernel_ms": kernel_ms, "algorithmic_flops_per_launch": flops},
    }
    if not args.no_extra:
        per = []
        for fn in (config1, config3, config4, config5, config5_packed, pto_api_bf16, pto_api_config1, pto_api_mxfp8, pto_api_mxfp4, quant_mxfp8, quant_mxfp4, quant_int8,
                   dequant_int8):
            per.append(fn(pa, ev, gen, 50, 5))
            torch.cuda.empty_cache()
        line["per_config"] = per
        line["published_shapes"] = published_shapes(pa, ev, gen, 20, 3)
    if not args.no_cpu:
        cpu, memo = CpuSide(), {}

        def leg(tag):
            if tag not in memo:
                memo[tag] = cpu.quant(tag[6:]) if tag.startswith("quant:") else getattr(cpu, tag)()
            return memo[tag]
        line["cpu_baseline"] = leg("headline")
        for entry in line.get("per_config", []):
            tag = entry.pop("cpu")
            if tag is not None:  # (entries outside BASELINE.json's configs carry no CPU leg)
                entry["cpu_baseline"] = leg(tag)
    for entry in line.get("per_config", []):
        entry.pop("cpu", None)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
