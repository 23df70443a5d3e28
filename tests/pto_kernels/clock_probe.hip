// Per-workgroup timestamps of the direct-to-LDS 256 x 256 tile GEMM kernel on one problem (default 4096^3).
// -DPROBE_KIND=0 bf16 (default), 1 int8 -> i32, 2 MXFP8 (E4M3 x E4M3, unit block scales) -> bf16, 3 W8A8 (int8 -> bf16
// through per-row and per-column float scales), 4 MXFP4 (E2M1 x E2M1, unit block scales, k given in operand bytes) -> bf16.
//
// Compiled with -DPTOAMD_CLOCK_PROBE the kernel writes, per workgroup, eight 64-bit words through p.acc_out:
// [0] core clocks spent in the K loop, [1] wall clock (100 MHz) at entry, [2] at the start of the K loop, [3] at its end,
// [4] at exit.  This program runs the launch back to back until the clocks have settled, then prints the phases of the
// last launch (mean / max over the workgroups) and the K loop per XCD (workgroup id mod 8).  Timing tool only: it checks
// no results.  Build: make -C tests/pto_kernels build/clock_probe   (not part of the default target; under a minute;
//                     build/clock_probe_i8 and build/clock_probe_fp8 are the other two kinds; build/clock_probe_nodma and
//                     build/clock_probe_halfdma leave out all / half of the slab DMAs to show what the copy-in costs)
//        run:   tests/pto_kernels/build/clock_probe [m n k [zeros]]   (a fourth argument fills the operands with zeros:
//               the same instruction stream at the lowest switching power)
#define PTOAMD_CLOCK_PROBE 1
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "../../pto-isa-mirror_amd/csrc/gemm_tile_dtl.hpp"

using namespace ptoamd;
#ifndef PROBE_KIND
#define PROBE_KIND 0
#endif
#ifndef PROBE_BLK
#define PROBE_BLK 16  // MFMA block edge of the bf16 / int8 kinds: 16 (the shipped tile) or 32
#endif
#if PROBE_KIND == 0 && PROBE_BLK == 16
using ProbeOp = OpBF16x16;
constexpr int ESZ = 2, CSZ = 2, OUT = OUT_BF16;
constexpr const char* KIND = "bf16 (16x16x32)";
#elif PROBE_KIND == 1 && PROBE_BLK == 16
using ProbeOp = OpI8x16;
constexpr int ESZ = 1, CSZ = 4, OUT = OUT_I32;
constexpr const char* KIND = "int8 (16x16x64)";
#elif PROBE_KIND == 4
using ProbeOp = OpFP4;   // k counts operand BYTES here (two E2M1 codes each)
constexpr int ESZ = 1, CSZ = 2, OUT = OUT_BF16;
constexpr const char* KIND = "MXFP4 (k in bytes)";
#elif PROBE_KIND == 3
using ProbeOp = OpI8x16;
constexpr int ESZ = 1, CSZ = 2, OUT = OUT_W8A8_BF16;
constexpr const char* KIND = "W8A8 int8 (16x16x64) -> bf16 with row and column scales";
#elif PROBE_KIND == 0
using ProbeOp = OpBF16;
constexpr int ESZ = 2, CSZ = 2, OUT = OUT_BF16;
constexpr const char* KIND = "bf16";
#elif PROBE_KIND == 1
using ProbeOp = OpI8;
constexpr int ESZ = 1, CSZ = 4, OUT = OUT_I32;
constexpr const char* KIND = "int8";
#else
using ProbeOp = OpFP8<0, 0>;
constexpr int ESZ = 1, CSZ = 2, OUT = OUT_BF16;
constexpr const char* KIND = "MXFP8";
#endif
#ifndef PROBE_WAVES_N
#define PROBE_WAVES_N 4  // 4: eight waves with 128 x 64 wave tiles (the default tile); 2: four waves with 128 x 128 wave tiles
#endif
#ifndef PROBE_BN
#define PROBE_BN 256  // tile width: 256, or 128 (with PROBE_WAVES_N=2: the four-wave 256 x 128 tile)
#endif
#ifndef PROBE_WAVES_M
#define PROBE_WAVES_M 2
#endif
using Cfg = TileCfg<256, PROBE_BN, PROBE_WAVES_M, PROBE_WAVES_N, ProbeOp>;

#define CK(x)                                                                          \
    do {                                                                               \
        hipError_t e_ = (x);                                                           \
        if (e_ != hipSuccess) {                                                        \
            printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__);      \
            return 1;                                                                  \
        }                                                                              \
    } while (0)

constexpr int GROUP_BYTES = ProbeOp::SCALED ? 128 / ProbeOp::GROUPS_PER_SLAB : 32;  // operand bytes per MX group

int main(int argc, char** argv)
{
    const int m = argc > 1 ? atoi(argv[1]) : 4096, n = argc > 2 ? atoi(argv[2]) : 4096, k = argc > 3 ? atoi(argv[3]) : 4096;
    if (m <= 0 || n <= 0 || k <= 0 || m % 256 || n % 256 || k % 512) {
        printf("m and n must be multiples of 256, k a multiple of 512\n");
        return 2;
    }
    const size_t kb = (size_t)k * ESZ;
    // row pitch of A and B: the K extent plus PTOAMD_PROBE_PITCH_PAD bytes (a multiple of 16; default 0 = contiguous rows)
    const size_t pitch = kb + (getenv("PTOAMD_PROBE_PITCH_PAD") ? atoi(getenv("PTOAMD_PROBE_PITCH_PAD")) : 0);
    if ((size_t)(std::max(m, n) - 1) * pitch + kb > 0xffffffffull || pitch % 16) {
        printf("operands must stay below 4 GiB (32-bit DMA offsets)\n");
        return 2;
    }
    // operand bytes: 16-bit patterns 0x3c00 + 10 random bits with a random sign are bf16 values of magnitude 1 - 2; as
    // byte pairs they are ordinary int8 values and, with bit 3 of each byte cleared, finite E4M3 codes
    std::vector<uint16_t> ha((size_t)m * pitch / 2), hb((size_t)n * pitch / 2);
    srand(1);
    for (auto& v : ha) v = (uint16_t)(0x3c00 + (rand() & 0x3ff) - ((rand() & 1) << 15));
    for (auto& v : hb) v = (uint16_t)(0x3c00 + (rand() & 0x3ff) - ((rand() & 1) << 15));
    if (argc > 4) {
        std::fill(ha.begin(), ha.end(), 0);
        std::fill(hb.begin(), hb.end(), 0);
    }
    if (ProbeOp::SCALED) {
        for (auto& v : ha) v &= 0xf7f7;
        for (auto& v : hb) v &= 0xf7f7;
    }
    uint8_t *a, *b, *sa = nullptr, *sb = nullptr;
    void* c;
    long* stamps;
    const int tiles = (m / Cfg::BM) * (n / Cfg::BN);
    CK(hipMalloc(&a, ha.size() * 2));
    CK(hipMalloc(&b, hb.size() * 2));
    CK(hipMalloc(&c, (size_t)m * n * CSZ));
    CK(hipMalloc(&stamps, (size_t)tiles * 64));
    CK(hipMemcpy(a, ha.data(), ha.size() * 2, hipMemcpyHostToDevice));
    CK(hipMemcpy(b, hb.data(), hb.size() * 2, hipMemcpyHostToDevice));
    CK(hipMemset(stamps, 0, (size_t)tiles * 64));
    if (ProbeOp::SCALED) {
        CK(hipMalloc(&sa, (size_t)m * (kb / GROUP_BYTES)));
        CK(hipMalloc(&sb, (size_t)n * (kb / GROUP_BYTES)));
        CK(hipMemset(sa, 127, (size_t)m * (kb / GROUP_BYTES)));
        CK(hipMemset(sb, 127, (size_t)n * (kb / GROUP_BYTES)));
    }

    TileGemmParams p{};
    if (OUT == OUT_W8A8_BF16) {
        float *rs, *cs;
        std::vector<float> hs(std::max(m, n), 0.001f);
        CK(hipMalloc(&rs, (size_t)m * 4));
        CK(hipMalloc(&cs, (size_t)n * 4));
        CK(hipMemcpy(rs, hs.data(), (size_t)m * 4, hipMemcpyHostToDevice));
        CK(hipMemcpy(cs, hs.data(), (size_t)n * 4, hipMemcpyHostToDevice));
        p.row_scale = rs;
        p.col_scale = cs;
    }
    p.a = a;
    p.b = b;
    p.c = c;
    p.m = m;
    p.n = n;
    p.k_bytes = (int)kb;
    p.lda_bytes = (long)pitch;
    p.ldb_bytes = (long)pitch;
    p.ldc = n;
    p.out_kind = OUT;
    p.group_m = getenv("PTOAMD_PROBE_GROUP_M") ? atoi(getenv("PTOAMD_PROBE_GROUP_M")) : 4;  // tile rows walked together (the library's value)
    p.sa = sa;
    p.sb = sb;
    p.scale_ld = (int)(kb / GROUP_BYTES);
    p.acc_out = (int32_t*)stamps;
    auto kernel = gemm_tile_dtl_kernel<Cfg>;
    CK(hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, Cfg::LDS_BYTES));

    hipEvent_t e0, e1;
    CK(hipEventCreate(&e0));
    CK(hipEventCreate(&e1));
    for (int i = 0; i < 300; ++i) hipLaunchKernelGGL(kernel, dim3(tiles), dim3(Cfg::THREADS), Cfg::LDS_BYTES, 0, p);
    CK(hipEventRecord(e0));
    for (int i = 0; i < 100; ++i) hipLaunchKernelGGL(kernel, dim3(tiles), dim3(Cfg::THREADS), Cfg::LDS_BYTES, 0, p);
    CK(hipEventRecord(e1));
    CK(hipEventSynchronize(e1));
    float ms;
    CK(hipEventElapsedTime(&ms, e0, e1));
    printf("%d x %d x %d %s%s, %d workgroups: %.2f us per launch with the stamps compiled in\n", m, n, k, KIND, argc > 4 ? " (zero operands)" : "", tiles, ms * 10.f);

    std::vector<long> h((size_t)tiles * 8);
    CK(hipMemcpy(h.data(), stamps, (size_t)tiles * 64, hipMemcpyDeviceToHost));
    long first = h[1], last = 0;
    for (int t = 0; t < tiles; ++t) {
        first = std::min(first, h[8 * t + 1]);
        last = std::max(last, h[8 * t + 4]);
    }
    double sum[4] = {0, 0, 0, 0}, mx[4] = {0, 0, 0, 0}, clocks = 0;
    double xcd_loop[8] = {0}, xcd_clk[8] = {0}, xcd_max[8] = {0};
    int xcd_cnt[8] = {0};
    for (int t = 0; t < tiles; ++t) {
        const long* o = &h[8 * t];
        const double ph[4] = {double(o[1] - first), double(o[2] - o[1]), double(o[3] - o[2]), double(o[4] - o[3])};
        for (int i = 0; i < 4; ++i) {
            sum[i] += ph[i];
            mx[i] = std::max(mx[i], ph[i]);
        }
        clocks += o[0];
        xcd_loop[t % 8] += ph[2];
        xcd_clk[t % 8] += o[0];
        xcd_max[t % 8] = std::max(xcd_max[t % 8], ph[2]);
        ++xcd_cnt[t % 8];
    }
    const char* names[4] = {"entry after the first workgroup's", "prologue", "K loop", "TSTORE"};
    for (int i = 0; i < 4; ++i) printf("%-34s mean %7.2f us  max %7.2f us\n", names[i], sum[i] / tiles / 100, mx[i] / 100);
    printf("K loop: %.0f core clocks per workgroup = %.0f per 128-byte slab, %.3f GHz\n", clocks / tiles,
           clocks / tiles / (kb / 128.0), clocks / sum[2] / 10.0);
    printf("first entry -> last exit %.2f us\n", (last - first) / 100.0);
    if (tiles > 256) {  // more workgroups than CUs: when each round of the chip starts and ends
        std::vector<long> entry(tiles), exit_(tiles);
        for (int t = 0; t < tiles; ++t) {
            entry[t] = h[8 * t + 1] - first;
            exit_[t] = h[8 * t + 4] - first;
        }
        std::sort(entry.begin(), entry.end());
        std::sort(exit_.begin(), exit_.end());
        for (int r = 0; r * 256 < tiles; ++r) {
            const int lo = r * 256, hi = std::min(tiles, lo + 256) - 1;
            printf("  workgroups %4d-%4d by start: entries %.2f .. %.2f us; by end: exits %.2f .. %.2f us\n", lo, hi,
                   entry[lo] / 100.0, entry[hi] / 100.0, exit_[lo] / 100.0, exit_[hi] / 100.0);
        }
    }
    for (int x = 0; x < 8; ++x)
        if (xcd_cnt[x])
            printf("  XCD %d: K loop mean %.2f us, max %.2f us, %.3f GHz\n", x, xcd_loop[x] / xcd_cnt[x] / 100, xcd_max[x] / 100,
                   xcd_clk[x] / xcd_loop[x] / 10.0);
    return 0;
}
