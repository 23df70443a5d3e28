// What the matrix pipe sustains on its own: a loop of nothing but MFMAs on register operands, one workgroup per CU.
// Under sustained load on random data this part is power-limited, so the figure that bounds a GEMM's K loop is
// (sustained clock) x (issue rate), and it differs between the instruction shapes of one operand type.
//
//   kind 0  v_mfma_f32_32x32x16_bf16            kind 1  v_mfma_f32_16x16x32_bf16
//   kind 2  v_mfma_i32_32x32x32_i8              kind 3  v_mfma_i32_16x16x64_i8
//   kind 4  v_mfma_scale_f32_32x32x64_f8f6f4    kind 5  v_mfma_scale_f32_16x16x128_f8f6f4   (E4M3 x E4M3, unit scales)
//
// Each wave keeps two sets of A and B fragments (a 128 x 64 wave tile's worth) and walks its accumulator blocks in the
// order a tile kernel does (consecutive MFMAs share one operand).  Operands: the clock probe's 16-bit patterns (bf16
// values of magnitude 1 - 2 with random signs and mantissas; as bytes ordinary int8 values, and finite E4M3 codes with
// bit 3 cleared), or zeros (no switching in the multipliers: the clock then stays at its ceiling).
// Timing tool only.  Build: make -C tests/pto_kernels build/mfma_power      (not part of the default target)
//        run:   tests/pto_kernels/build/mfma_power <kind> [zeros(0/1) [iterations [threads per workgroup: 256 or 512]]]
// With 512 threads the SIMD's two waves run one after the other (the issue arbiter prefers the older wave), so the
// per-wave stamps of workgroup 0 printed at the end show two groups; the launch time covers both.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <vector>

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(16))) int i32x16;
typedef __attribute__((ext_vector_type(4))) int i32x4;
typedef __attribute__((ext_vector_type(8))) int i32x8;

#define CK(x)                                                                          \
    do {                                                                               \
        hipError_t e_ = (x);                                                           \
        if (e_ != hipSuccess) {                                                        \
            printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__);      \
            return 1;                                                                  \
        }                                                                              \
    } while (0)

template <int KIND>
struct Shape;
template <> struct Shape<0> { using Frag = bf16x8; using Acc = f32x16; static constexpr int NA = 4, NB = 2, REGS = 16; };
template <> struct Shape<1> { using Frag = bf16x8; using Acc = f32x4; static constexpr int NA = 8, NB = 4, REGS = 4; };
template <> struct Shape<2> { using Frag = i32x4; using Acc = i32x16; static constexpr int NA = 4, NB = 2, REGS = 16; };
template <> struct Shape<3> { using Frag = i32x4; using Acc = i32x4; static constexpr int NA = 8, NB = 4, REGS = 4; };
template <> struct Shape<4> { using Frag = i32x8; using Acc = f32x16; static constexpr int NA = 4, NB = 2, REGS = 16; };
// (32-byte fragments: a 64 x 32 wave tile's worth keeps the two fragment sets inside the register file)
template <> struct Shape<5> { using Frag = i32x8; using Acc = f32x4; static constexpr int NA = 4, NB = 2, REGS = 4; };

template <int KIND, class Frag, class Acc>
__device__ __forceinline__ Acc mma(const Frag& b, const Frag& a, const Acc& c)
{
    constexpr int unit = 0x7f7f7f7f;  // E8M0 127 in every byte
    if constexpr (KIND == 0) return __builtin_amdgcn_mfma_f32_32x32x16_bf16(b, a, c, 0, 0, 0);
    else if constexpr (KIND == 1) return __builtin_amdgcn_mfma_f32_16x16x32_bf16(b, a, c, 0, 0, 0);
    else if constexpr (KIND == 2) return __builtin_amdgcn_mfma_i32_32x32x32_i8(b, a, c, 0, 0, 0);
    else if constexpr (KIND == 3) return __builtin_amdgcn_mfma_i32_16x16x64_i8(b, a, c, 0, 0, 0);
    else if constexpr (KIND == 4) return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(b, a, c, 0, 0, 0, unit, 0, unit);
    else return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(b, a, c, 0, 0, 0, unit, 0, unit);
}

template <int KIND>
__global__ __launch_bounds__(512) void mfma_loop(const uint4* __restrict__ src, float* __restrict__ out, int iters,
                                                 unsigned long long* stamps)
{
    using S = Shape<KIND>;
    using Frag = typename S::Frag;
    using Acc = typename S::Acc;
    constexpr int NA = S::NA, NB = S::NB, PIECES = sizeof(Frag) / 16;
    const int gid = blockIdx.x * blockDim.x + threadIdx.x;
    Frag a[2][NA], b[2][NB];
    // 32 sixteen-byte pieces per lane; fragments of 32 bytes take two (re-using pieces across fragments is harmless)
    auto load = [&](int piece) __attribute__((always_inline)) {
        Frag f;
        uint4 v[2];
        for (int h = 0; h < PIECES; ++h) {
            v[h] = src[(size_t)gid * 32 + ((piece + 5 * h) & 31)];
            if (KIND >= 4) {  // finite E4M3 codes
                v[h].x &= 0xf7f7f7f7u; v[h].y &= 0xf7f7f7f7u; v[h].z &= 0xf7f7f7f7u; v[h].w &= 0xf7f7f7f7u;
            }
        }
        __builtin_memcpy(&f, v, sizeof(Frag));
        return f;
    };
    for (int s = 0; s < 2; ++s) {
        for (int i = 0; i < NA; ++i) a[s][i] = load(s * 16 + i);
        for (int j = 0; j < NB; ++j) b[s][j] = load(s * 16 + 8 + j);
    }
    Acc acc[NA][NB] = {};
    const unsigned long long t0 = clock64(), w0 = wall_clock64();
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int s = 0; s < 2; ++s)
#pragma unroll
            for (int i = 0; i < NA; ++i)
#pragma unroll
                for (int j = 0; j < NB; ++j) acc[i][j] = mma<KIND>(b[s][j], a[s][i], acc[i][j]);
    }
    float r = 0;
    for (int i = 0; i < NA; ++i)
        for (int j = 0; j < NB; ++j)
            for (int e = 0; e < S::REGS; ++e) r += (float)acc[i][j][e];
    out[gid] = r;
    const unsigned long long t1 = clock64(), w1 = wall_clock64();
    if ((threadIdx.x & 63) == 0) {
        unsigned long long* o = stamps + (blockIdx.x * 8 + (threadIdx.x >> 6)) * 4;
        o[0] = t1 - t0; o[1] = w1 - w0; o[2] = w0; o[3] = w1;
    }
}

int main(int argc, char** argv)
{
    const int kind = argc > 1 ? atoi(argv[1]) : 0;
    const int zeros = argc > 2 ? atoi(argv[2]) : 0;
    const int iters = argc > 3 ? atoi(argv[3]) : 2000;
    const int thr = argc > 4 ? atoi(argv[4]) : 256;
    if (kind < 0 || kind > 5 || iters <= 0 || (thr != 256 && thr != 512)) {
        printf("usage: mfma_power <kind 0-5> [zeros 0/1 [iterations [256 | 512]]]\n");
        return 2;
    }
    hipDeviceProp_t prop;
    CK(hipGetDeviceProperties(&prop, 0));
    const int wgs = prop.multiProcessorCount, nw = thr / 64;
    const size_t pieces = (size_t)wgs * thr * 32;
    std::vector<uint16_t> h(pieces * 8);
    srand(1);
    for (auto& v : h) v = zeros ? 0 : (uint16_t)(0x3c00 + (rand() & 0x3ff) - ((rand() & 1) << 15));
    uint4* d;
    float* out;
    unsigned long long* stamps;
    CK(hipMalloc(&d, pieces * 16));
    CK(hipMalloc(&out, (size_t)wgs * thr * 4));
    CK(hipMalloc(&stamps, (size_t)wgs * 8 * 32));
    CK(hipMemset(stamps, 0, (size_t)wgs * 8 * 32));
    CK(hipMemcpy(d, h.data(), pieces * 16, hipMemcpyHostToDevice));
    hipEvent_t e0, e1;
    CK(hipEventCreate(&e0));
    CK(hipEventCreate(&e1));
    static const char* names[] = {"bf16 32x32x16", "bf16 16x16x32", "i8 32x32x32", "i8 16x16x64", "fp8 scaled 32x32x64", "fp8 scaled 16x16x128"};
    static const double flop_per_mfma[] = {2.0 * 32 * 32 * 16, 2.0 * 16 * 16 * 32, 2.0 * 32 * 32 * 32, 2.0 * 16 * 16 * 64, 2.0 * 32 * 32 * 64, 2.0 * 16 * 16 * 128};
    static const int mfmas_per_iter[] = {16, 64, 16, 64, 16, 16};  // 2 fragment sets x NA x NB
    const double peak = kind < 2 ? 2.5 : 5.0;                       // PFLOP/s (POP/s), dense
    const double flop = (double)wgs * nw * iters * mfmas_per_iter[kind] * flop_per_mfma[kind];
    for (int rep = 0; rep < 3; ++rep) {
        const int launches = 100;
        CK(hipEventRecord(e0));
        for (int l = 0; l < launches; ++l) {
            switch (kind) {
                case 0: hipLaunchKernelGGL(mfma_loop<0>, dim3(wgs), dim3(thr), 0, 0, d, out, iters, stamps); break;
                case 1: hipLaunchKernelGGL(mfma_loop<1>, dim3(wgs), dim3(thr), 0, 0, d, out, iters, stamps); break;
                case 2: hipLaunchKernelGGL(mfma_loop<2>, dim3(wgs), dim3(thr), 0, 0, d, out, iters, stamps); break;
                case 3: hipLaunchKernelGGL(mfma_loop<3>, dim3(wgs), dim3(thr), 0, 0, d, out, iters, stamps); break;
                case 4: hipLaunchKernelGGL(mfma_loop<4>, dim3(wgs), dim3(thr), 0, 0, d, out, iters, stamps); break;
                default: hipLaunchKernelGGL(mfma_loop<5>, dim3(wgs), dim3(thr), 0, 0, d, out, iters, stamps); break;
            }
        }
        CK(hipGetLastError());
        CK(hipEventRecord(e1));
        CK(hipEventSynchronize(e1));
        float ms;
        CK(hipEventElapsedTime(&ms, e0, e1));
        std::vector<unsigned long long> hc((size_t)wgs * 8 * 4);
        CK(hipMemcpy(hc.data(), stamps, hc.size() * 8, hipMemcpyDeviceToHost));
        double cs = 0, ws = 0;
        for (int i = 0; i < wgs * 8; ++i) {
            if ((i & 7) >= nw) continue;
            cs += (double)hc[4 * i];
            ws += (double)hc[4 * i + 1];
        }
        const double us = ms * 1000 / launches;
        printf("%s, %s operands, %d waves per CU: %.1f us per launch, %.3f PFLOP/s (%.1f %% of %.1f), sustained clock %.3f GHz, "
               "%.1f clocks per MFMA per SIMD\n",
               names[kind], zeros ? "zero" : "random", nw, us, flop / us * 1e-9, flop / us * 1e-9 / peak * 100, peak, cs / ws * 0.1,
               us * 1e3 * (cs / ws * 0.1) / ((double)iters * mfmas_per_iter[kind] * (nw / 4)));
        if (rep == 2) {
            printf("  workgroup 0, per wave (start, end in us after the wave's first stamp):");
            for (int w = 0; w < nw; ++w) printf(" [%.1f %.1f]", (hc[4 * w + 2] - hc[2]) * 0.01, (hc[4 * w + 3] - hc[2]) * 0.01);
            printf("\n");
        }
        fflush(stdout);
    }
    return 0;
}
