// Decode-shaped weight-only MXFP4 GEMV/GEMM (m <= 16): out[m][n] = sum_k A[m][k] * (e2m1 W[n][k] * 2^(sw[n][k/32]-127)).
//
// The shape is HBM-bound (every weight byte is read once, ~60 FLOP per byte), so the kernel is built around the
// weight stream:
//   * the K range is split over the 8 waves of a workgroup; each wave keeps its [16][K/8] slice of the bf16
//     activations in registers for the whole kernel (the TLOAD of the Left operand happens once per workgroup);
//   * a workgroup walks groups of 16 weight rows; each lane streams 16-byte pieces (32 fp4 = one MX group) with the
//     loads of the next row group in flight while the current one is multiplied;
//   * dequantisation happens in registers (v_cvt_scalef32_pk_bf16_fp4: fp4 pair * 2^e -> bf16 pair, exact), the
//     product runs on v_mfma_f32_16x16x32_bf16 with fp32 accumulation, and the 8 partial 16x16 tiles are summed
//     through LDS in a fixed order before the store (TSTORE f32 -> f32 | bf16).
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

constexpr int GEMV_WAVES = 8;
constexpr int GEMV_MAX_CHUNKS = 8;  // 128-k chunks per wave: K <= 8 * 8 * 128 = 8192

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

template <bool HW_CVT>
__global__ void __launch_bounds__(GEMV_WAVES * 64) gemv_mxfp4_kernel(const GemvParams p)
{
    __shared__ float red[GEMV_WAVES][64][4];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int l16 = lane & 15, g = lane >> 4;
    const int ks = p.k / GEMV_WAVES;  // this wave's K slice, a multiple of 128
    const int chunks = ks / 128;
    const int k0 = wave * ks;

    // Left operand slice -> registers: lane (row l16, quarter g) holds k0 + 128c + 32g .. +31 of its row, per chunk c
    uint4 areg[GEMV_MAX_CHUNKS][4];
#pragma unroll
    for (int c = 0; c < GEMV_MAX_CHUNKS; ++c) {
#pragma unroll
        for (int j = 0; j < 4; ++j)
            areg[c][j] = make_uint4(0, 0, 0, 0);
        if (c < chunks && l16 < p.m) {
            const uint4* src = reinterpret_cast<const uint4*>(p.a + (long)l16 * p.lda + k0 + c * 128 + g * 32);
#pragma unroll
            for (int j = 0; j < 4; ++j)
                areg[c][j] = src[j];
        }
    }

    uint4 wreg[GEMV_MAX_CHUNKS];
    uint32_t sreg[GEMV_MAX_CHUNKS];
    auto load_group = [&](int ng) {
        const int row = min(ng * 16 + l16, p.n - 1);
        const uint8_t* wp = p.w + (long)row * p.ldw_bytes + (k0 + g * 32) / 2;
        const uint8_t* sp = p.sw + (long)row * (p.k / 32) + k0 / 32 + g;
#pragma unroll
        for (int c = 0; c < GEMV_MAX_CHUNKS; ++c)
            if (c < chunks) {
                wreg[c] = *reinterpret_cast<const uint4*>(wp + c * 64);
                sreg[c] = sp[c * 4];
            }
    };

    int ng = blockIdx.x;
    if (ng < p.n_groups)
        load_group(ng);
    for (; ng < p.n_groups; ng += gridDim.x) {
        uint4 wcur[GEMV_MAX_CHUNKS];
        uint32_t scur[GEMV_MAX_CHUNKS];
#pragma unroll
        for (int c = 0; c < GEMV_MAX_CHUNKS; ++c) {
            wcur[c] = wreg[c];
            scur[c] = sreg[c];
        }
        if (ng + (int)gridDim.x < p.n_groups)
            load_group(ng + gridDim.x);  // next row group's weights are in flight during the multiply

        f32x4 acc = {0, 0, 0, 0};
#pragma unroll
        for (int c = 0; c < GEMV_MAX_CHUNKS; ++c)
            if (c < chunks) {
                const float scale = e8m0_to_f32(scur[c]);
                const uint32_t xs[4] = {wcur[c].x, wcur[c].y, wcur[c].z, wcur[c].w};
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const uint4 wv = dequant8<HW_CVT>(xs[j], scale);
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, areg[c][j]),
                                                                 __builtin_bit_cast(bf16x8, wv), acc, 0, 0, 0);
                }
            }
        // sum the 8 K-slice partials in wave order (deterministic), then TSTORE
#pragma unroll
        for (int r = 0; r < 4; ++r)
            red[wave][lane][r] = acc[r];
        __syncthreads();
        if (threadIdx.x < 256) {
            const int ol = threadIdx.x >> 2, r = threadIdx.x & 3;
            float s = 0.0f;
#pragma unroll
            for (int w8 = 0; w8 < GEMV_WAVES; ++w8)
                s += red[w8][ol][r];
            const int gi = 4 * (ol >> 4) + r, gj = ng * 16 + (ol & 15);
            if (gi < p.m && gj < p.n) {
                if (p.out_bf16)
                    reinterpret_cast<uint16_t*>(p.out)[(long)gi * p.ldc + gj] = f32_to_bf16_bits(s);
                else
                    reinterpret_cast<float*>(p.out)[(long)gi * p.ldc + gj] = s;
            }
        }
        __syncthreads();
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
    const bool stream_ok = !(fg && fg[0] == '1') && k % (GEMV_WAVES * 128) == 0 && k <= GEMV_WAVES * GEMV_MAX_CHUNKS * 128 &&
                           (reinterpret_cast<uintptr_t>(a_bf16) & 15u) == 0 && (reinterpret_cast<uintptr_t>(w) & 15u) == 0 &&
                           (lda % 8) == 0 && (p.ldw_bytes % 16) == 0;
    if (!stream_ok) {
        dim3 block(128), grid((n + 127) / 128, m);
        hipLaunchKernelGGL(gemv_mxfp4_generic_kernel, grid, block, 0, stream, p);
        PTOAMD_HIP_CHECK(hipGetLastError());
        set_last_kernel("gemv_mxfp4_generic");
        return PTOAMD_OK;
    }
    int dev = 0, cus = 256;
    PTOAMD_HIP_CHECK(hipGetDevice(&dev));
    PTOAMD_HIP_CHECK(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    // one workgroup per CU walks its share of the row groups; a grid that divides the groups evenly avoids a tail
    int grid = p.n_groups < cus ? p.n_groups : cus;
    const char* sw_cvt = getenv("PTOAMD_GEMV_SW_CVT");
    if (sw_cvt && sw_cvt[0] == '1') {
        hipLaunchKernelGGL(gemv_mxfp4_kernel<false>, dim3(grid), dim3(GEMV_WAVES * 64), 0, stream, p);
        set_last_kernel("gemv_mxfp4_stream_swcvt");
    } else {
        hipLaunchKernelGGL(gemv_mxfp4_kernel<true>, dim3(grid), dim3(GEMV_WAVES * 64), 0, stream, p);
        set_last_kernel("gemv_mxfp4_stream");
    }
    PTOAMD_HIP_CHECK(hipGetLastError());
    return PTOAMD_OK;
}
