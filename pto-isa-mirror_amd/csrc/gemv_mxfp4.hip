// Decode-shaped weight-only MXFP4 GEMV/GEMM (m <= 16): out[m][n] = sum_k A[m][k] * (e2m1 W[n][k] * 2^(sw[n][k/32]-127)).
//
// The shape is HBM-bound (every weight byte is read once, ~60 FLOP per byte), so the kernel is built around keeping
// enough weight bytes in flight:
//   * a workgroup owns WAVES x 16 weight rows over the full K; each wave streams its 16 rows in 512-k chunks, four
//     16-byte loads (32 fp4 = one MX group each) plus one 16-byte scale load per lane per chunk, with DEPTH chunks of
//     loads outstanding per wave (registers are cheap here: the accumulator is 4 VGPRs);
//   * the bf16 activations (the Left operand, shared by every wave) are staged per chunk into a double-buffered LDS
//     strip already laid out as MFMA operand fragments, so a ds_read_b128 per MFMA is conflict-free;
//   * dequantisation happens in registers (v_cvt_scalef32_pk_bf16_fp4: fp4 pair * 2^e -> bf16 pair, exact), the
//     product runs on v_mfma_f32_16x16x32_bf16 with fp32 accumulation, and each wave stores its own 16 x 16 result
//     (TSTORE f32 -> f32 | bf16): no cross-wave reduction, one barrier per chunk for the activation strip.
// Operand k-slots are assigned so that a lane's 32 consecutive k (one MX group, one scale byte) feed 4 MFMAs.
#include "common_host.hpp"
#include "device_types.hpp"

#include <stdlib.h>

namespace ptoamd {

typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;

struct GemvParams {
    const uint16_t* a;  // bf16 [m][lda]
    const uint8_t* w;   // e2m1 packed [n][ldw_bytes]
    const uint8_t* sw;  // e8m0 [n][k/32]
    void* out;
    int m, n, k;
    long lda, ldw_bytes;
    int ldc;
    int out_bf16;
    int n_groups;       // ceil(n / 16)
};

constexpr int GEMV_CHUNK = 512;  // k per chunk
constexpr int GEMV_DEPTH = 4;    // chunks of weight loads in flight per wave

// 8 packed fp4 (one dword) times 2^(e-127) -> 8 bf16, exact.  HW: one v_cvt_scalef32_pk_bf16_fp4 per byte.
template <bool HW_CVT>
__device__ __forceinline__ uint4 dequant8(uint32_t x, float scale)
{
    uint4 r;
    if constexpr (HW_CVT) {
        r.x = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(x, scale, 0));
        r.y = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(x, scale, 1));
        r.z = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(x, scale, 2));
        r.w = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(x, scale, 3));
    } else {
        uint32_t h[8];
#pragma unroll
        for (int i = 0; i < 8; ++i)
            h[i] = f2u(__fmul_rn(e2m1_to_f32((x >> (4 * i)) & 0xFu), scale)) >> 16;  // exact, so truncation is exact
        r.x = h[0] | (h[1] << 16);
        r.y = h[2] | (h[3] << 16);
        r.z = h[4] | (h[5] << 16);
        r.w = h[6] | (h[7] << 16);
    }
    return r;
}

// LDS strip of one activation chunk: [4 sub-chunks of 128 k][4 MFMAs][64 lanes] x 16 bytes = 16 KiB.  Lane (row l16,
// quarter g) of MFMA j of sub-chunk c holds A[l16][128 c + 32 g + 8 j .. + 7].
template <bool HW_CVT, int WAVES>
__global__ void __launch_bounds__(WAVES * 64) gemv_mxfp4_kernel(const GemvParams p)
{
    constexpr int NT = WAVES * 64;
    __shared__ uint4 astrip[2][16 * 64];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l16 = lane & 15, g = lane >> 4;
    const int chunks = p.k / GEMV_CHUNK;
    const int row = min((blockIdx.x * WAVES + wave) * 16 + l16, p.n - 1);
    const uint8_t* wp = p.w + (long)row * p.ldw_bytes + g * 16;   // + chunk * 256 + c * 64
    const uint8_t* sp = p.sw + (long)row * (p.k / 32);            // + chunk * 16

    // activation chunk -> registers -> LDS (fragment-major); 1024 pieces of 16 bytes per chunk
    constexpr int APIECES = (1024 + NT - 1) / NT;
    // The activation pieces of chunk kc are fetched together with the weights of chunk kc (DEPTH chunks ahead), not one
    // chunk ahead: vmcnt retires loads in issue order, so waiting for a young activation load would also wait for
    // every older weight prefetch and collapse the prefetch depth to one chunk.
    uint4 areg[GEMV_DEPTH][APIECES];
    auto a_fetch = [&](int stage, int kc) {
#pragma unroll
        for (int x = 0; x < APIECES; ++x) {
            const int piece = tid + x * NT;            // m = piece % 16, q = piece / 16 (q-th group of 8 k)
            const int m = piece & 15, q = piece >> 4;
            areg[stage][x] = make_uint4(0, 0, 0, 0);
            if (piece < 1024 && m < p.m)
                areg[stage][x] = *reinterpret_cast<const uint4*>(p.a + (long)m * p.lda + kc * GEMV_CHUNK + q * 8);
        }
    };
    auto a_stage = [&](int stage, int buf) {
#pragma unroll
        for (int x = 0; x < APIECES; ++x) {
            const int piece = tid + x * NT;
            const int m = piece & 15, q = piece >> 4;  // q = 16 c + 4 g + j; 16 rows of one q are contiguous in LDS
            if (piece < 1024)
                astrip[buf][((q >> 4) * 4 + (q & 3)) * 64 + ((q >> 2) & 3) * 16 + m] = areg[stage][x];
        }
    };

    uint4 wreg[GEMV_DEPTH][4], sreg[GEMV_DEPTH];
    auto w_fetch = [&](int stage, int kc) {
#pragma unroll
        for (int c = 0; c < 4; ++c)
            wreg[stage][c] = *reinterpret_cast<const uint4*>(wp + (long)kc * (GEMV_CHUNK / 2) + c * 64);
        sreg[stage] = *reinterpret_cast<const uint4*>(sp + kc * (GEMV_CHUNK / 32));
    };

    f32x4 acc = {0, 0, 0, 0};
#pragma unroll
    for (int d = 0; d < GEMV_DEPTH; ++d)
        if (d < chunks) {
            a_fetch(d, d);
            w_fetch(d, d);
        }
    a_stage(0, 0);
    __syncthreads();

    for (int kc0 = 0; kc0 < chunks; kc0 += GEMV_DEPTH) {
#pragma unroll
        for (int d = 0; d < GEMV_DEPTH; ++d) {
            const int kc = kc0 + d;
            if (kc < chunks) {
                const int buf = kc & 1;
                const uint32_t sw4[4] = {sreg[d].x, sreg[d].y, sreg[d].z, sreg[d].w};
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    const float scale = e8m0_to_f32((sw4[c] >> (8 * g)) & 0xFFu);  // MX group 4 c + g of the chunk
                    const uint32_t xs[4] = {wreg[d][c].x, wreg[d][c].y, wreg[d][c].z, wreg[d][c].w};
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const uint4 wv = dequant8<HW_CVT>(xs[j], scale);
                        const uint4 av = astrip[buf][(c * 4 + j) * 64 + lane];
                        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, av),
                                                                     __builtin_bit_cast(bf16x8, wv), acc, 0, 0, 0);
                    }
                }
                if (kc + 1 < chunks)
                    a_stage((d + 1) % GEMV_DEPTH, buf ^ 1);  // chunk kc + 1's activations, fetched DEPTH - 1 chunks ago
                if (kc + GEMV_DEPTH < chunks) {  // refill this stage: DEPTH chunks of loads stay in flight
                    a_fetch(d, kc + GEMV_DEPTH);
                    w_fetch(d, kc + GEMV_DEPTH);
                }
                __syncthreads();
            }
        }
    }

    const int n0 = (blockIdx.x * WAVES + wave) * 16;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int gi = 4 * g + r, gj = n0 + l16;
        if (gi < p.m && gj < p.n) {
            if (p.out_bf16)
                reinterpret_cast<uint16_t*>(p.out)[(long)gi * p.ldc + gj] = f32_to_bf16_bits(acc[r]);
            else
                reinterpret_cast<float*>(p.out)[(long)gi * p.ldc + gj] = acc[r];
        }
    }
}

// Generic form for shapes the streaming kernel does not take: one thread per output, k ascending, fp32 fma
// (the same order as the reference TMATMUL on the dequantised bf16 weights).
__global__ void gemv_mxfp4_generic_kernel(const GemvParams p)
{
    const int gj = blockIdx.x * blockDim.x + threadIdx.x;
    const int gi = blockIdx.y;
    if (gj >= p.n || gi >= p.m)
        return;
    float acc = 0.0f;
    for (int kk = 0; kk < p.k; ++kk) {
        const uint32_t code = (p.w[(long)gj * p.ldw_bytes + (kk >> 1)] >> ((kk & 1) * 4)) & 0xFu;
        const float wv = __fmul_rn(e2m1_to_f32(code), e8m0_to_f32(p.sw[(long)gj * (p.k / 32) + kk / 32]));
        acc = __fmaf_rn(bf16_bits_to_f32(p.a[(long)gi * p.lda + kk]), wv, acc);
    }
    if (p.out_bf16)
        reinterpret_cast<uint16_t*>(p.out)[(long)gi * p.ldc + gj] = f32_to_bf16_bits(acc);
    else
        reinterpret_cast<float*>(p.out)[(long)gi * p.ldc + gj] = acc;
}

}  // namespace ptoamd

using namespace ptoamd;

extern "C" int ptoamd_gemv_mxfp4(void* out, int c_type, const void* a_bf16, const uint8_t* w, const uint8_t* sw, int m,
                                 int n, int k, int lda, int ldw, int ldc, void* stream_)
{
    hipStream_t stream = as_stream(stream_);
    PTOAMD_REQUIRE(out && a_bf16 && w && sw, PTOAMD_E_INVALID, "ptoamd_gemv_mxfp4: null operand");
    PTOAMD_REQUIRE(m > 0 && n > 0 && k > 0, PTOAMD_E_INVALID, "ptoamd_gemv_mxfp4: m, n, k must be positive");
    PTOAMD_REQUIRE(m <= 16, PTOAMD_E_UNSUPPORTED, "ptoamd_gemv_mxfp4: m = %d exceeds the decode batch of 16 (use ptoamd_gemm_mx)", m);
    PTOAMD_REQUIRE(k % 32 == 0, PTOAMD_E_INVALID, "ptoamd_gemv_mxfp4: k = %d must be a multiple of the MX block of 32", k);
    PTOAMD_REQUIRE(c_type == PTOAMD_F32 || c_type == PTOAMD_BF16, PTOAMD_E_UNSUPPORTED, "ptoamd_gemv_mxfp4: output is f32 or bf16");
    PTOAMD_REQUIRE(lda >= k && ldw >= k && ldc >= n && ldw % 2 == 0, PTOAMD_E_INVALID,
                   "ptoamd_gemv_mxfp4: leading dimension smaller than the row length (or odd ldw)");
    GemvParams p{};
    p.a = reinterpret_cast<const uint16_t*>(a_bf16);
    p.w = w; p.sw = sw; p.out = out;
    p.m = m; p.n = n; p.k = k; p.lda = lda; p.ldw_bytes = ldw / 2; p.ldc = ldc;
    p.out_bf16 = c_type == PTOAMD_BF16;
    p.n_groups = (n + 15) / 16;
    const char* fg = getenv("PTOAMD_FORCE_GENERIC");
    const bool stream_ok = !(fg && fg[0] == '1') && k % GEMV_CHUNK == 0 && (reinterpret_cast<uintptr_t>(a_bf16) & 15u) == 0 &&
                           (reinterpret_cast<uintptr_t>(w) & 15u) == 0 && (reinterpret_cast<uintptr_t>(sw) & 15u) == 0 &&
                           (lda % 8) == 0 && (p.ldw_bytes % 16) == 0;
    if (!stream_ok) {
        dim3 block(128), grid((n + 127) / 128, m);
        hipLaunchKernelGGL(gemv_mxfp4_generic_kernel, grid, block, 0, stream, p);
        PTOAMD_HIP_CHECK(hipGetLastError());
        set_last_kernel("gemv_mxfp4_generic");
        return PTOAMD_OK;
    }
    // 16 rows per wave; 7 waves per workgroup when that tiles the row groups more evenly over the CUs than 8
    // (N = 28672: 1792 groups = 256 workgroups of 7), else 8
    int dev = 0, cus = 256;
    PTOAMD_HIP_CHECK(hipGetDevice(&dev));
    PTOAMD_HIP_CHECK(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    const int g7 = (p.n_groups + 6) / 7, g8 = (p.n_groups + 7) / 8;
    const auto rounds = [&](int blocks) { return (blocks + cus - 1) / cus; };
    const bool use7 = rounds(g7) * 7 < rounds(g8) * 8;
    const char* sw_cvt = getenv("PTOAMD_GEMV_SW_CVT");
    const bool swc = sw_cvt && sw_cvt[0] == '1';
    if (use7) {
        if (swc)
            hipLaunchKernelGGL((gemv_mxfp4_kernel<false, 7>), dim3(g7), dim3(7 * 64), 0, stream, p);
        else
            hipLaunchKernelGGL((gemv_mxfp4_kernel<true, 7>), dim3(g7), dim3(7 * 64), 0, stream, p);
    } else {
        if (swc)
            hipLaunchKernelGGL((gemv_mxfp4_kernel<false, 8>), dim3(g8), dim3(8 * 64), 0, stream, p);
        else
            hipLaunchKernelGGL((gemv_mxfp4_kernel<true, 8>), dim3(g8), dim3(8 * 64), 0, stream, p);
    }
    set_last_kernel(swc ? "gemv_mxfp4_stream_swcvt" : "gemv_mxfp4_stream");
    PTOAMD_HIP_CHECK(hipGetLastError());
    return PTOAMD_OK;
}
