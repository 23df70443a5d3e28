// TQUANT (INT8 symmetric / asymmetric, MXFP8, MXFP4) and TDEQUANT as HBM-streaming gfx950 kernels.
// Arithmetic follows the reference CPU simulator step for step (include/pto/cpu/TQuant.hpp, cpu/TDeQuant.hpp) so the
// codes, shared exponents, group maxima and scalings are bit-identical; citations are given per function.
#include "common_host.hpp"
#include "device_types.hpp"
#include "lds_dma.hpp"
#include "../include/pto/amd/quant_math.hpp"

namespace ptoamd {

typedef short short2v __attribute__((ext_vector_type(2)));

static_assert(PTOAMD_OCP_MXFP8 == MX_OCP_FP8 && PTOAMD_NV_MXFP8 == MX_NV_FP8 && PTOAMD_OCP_MXFP4 == MX_OCP_FP4 &&
                  PTOAMD_NV_MXFP4 == MX_NV_FP4,
              "the C ABI's algorithm ids are the kernels' template arguments");

// ---- axis 1: 32-element groups along a row.  A lane owns one 16-byte piece of the source (4 f32 or 8 half / bf16
// elements), so a group is 8 or 4 neighbouring lanes and a wave reads 1 KiB per load instruction; every thread handles
// UNITS such pieces, one block-wide span apart, with all its loads in flight before the first is used.
// FP4 codes come from the packed hardware conversion (v_cvt_scalef32_pk_fp4_f32, round to nearest even, saturating): on
// finite and infinite input it is EncodeE2M1Magic (TQuant.hpp:155-176) -- the magic-number add there is a
// round-to-nearest-even onto the same grid with the same clamp; NaN elements are given that function's code (0x7) in
// software after the conversion, and the two cases where the code does not depend on the value alone (an infinite or
// NaN scaling) are resolved per group last.  The bf16 source's re-rounding of
// the scaled value (TQuant.hpp:68-76) is the identity here: the scaling is a power of two, so the product of a bf16
// value is a bf16 value again unless it is subnormal, and then it is far below the smallest code either way.
template <int ALG, typename T, bool SRC_BF16>
__global__ void __launch_bounds__(256) tquant_mx_rows_kernel(uint8_t* dst, uint8_t* exp, float* mx, float* scaling, const T* src, long units)
{
    constexpr bool FP4 = ALG == PTOAMD_OCP_MXFP4 || ALG == PTOAMD_NV_MXFP4;
    constexpr int EPL = 16 / (int)sizeof(T), LPG = 32 / EPL, UNITS = 4;
    const long first = (long)blockIdx.x * (UNITS * 256) + threadIdx.x;
    uint4 raw[UNITS];
#pragma unroll
    for (int u = 0; u < UNITS; ++u) {
        const long unit = first + u * 256;
        raw[u] = unit < units ? reinterpret_cast<const uint4*>(src)[unit] : make_uint4(0, 0, 0, 0);
    }
#pragma unroll
    for (int u = 0; u < UNITS; ++u) {
        const long unit = first + u * 256;
        const bool live = unit < units;  // (a block's span starts on a group boundary: all lanes of a group agree)
        float v[EPL];
        const uint32_t w[4] = {raw[u].x, raw[u].y, raw[u].z, raw[u].w};
#pragma unroll
        for (int i = 0; i < EPL; ++i) {
            if constexpr (sizeof(T) == 4) {
                v[i] = u2f(w[i]);
            } else {
                T t;
                t.b = (uint16_t)(w[i >> 1] >> (16 * (i & 1)));
                v[i] = widen<T>(t);
            }
        }
        uint32_t run = 0;
#pragma unroll
        for (int i = 0; i < EPL; ++i)
            run = max_step<ALG>(run, v[i], (int)(threadIdx.x & (LPG - 1)) * EPL + i);
#pragma unroll
        for (int off = 1; off < LPG; off <<= 1)
            run = max_merge<ALG>(run, (uint32_t)__shfl_xor((int)run, off, LPG));
        const float maxabs = max_value<ALG>(run);
        const uint32_t e = shared_exponent<ALG>(maxabs);
        const float sc = group_scaling<ALG>(maxabs, e);
        const long g = unit / LPG;
        if (live && (threadIdx.x & (LPG - 1)) == 0) {
            exp[g] = (uint8_t)e;
            if (mx)
                mx[g] = maxabs;
            if (scaling)
                scaling[g] = sc;
        }
        if (FP4) {
            uint32_t packed = 0;
            static_for<EPL / 2>([&](auto ic) {
                constexpr int i = decltype(ic)::value;
                packed = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(packed, __fmul_rn(v[2 * i], sc), __fmul_rn(v[2 * i + 1], sc), 1.0f, i);
            });
            // a NaN element encodes as +6 (0x7) whatever its sign (TQuant.hpp:157-159); what the packed conversion makes
            // of a NaN is not relied on
            uint32_t nan_nibbles = 0;
#pragma unroll
            for (int i = 0; i < EPL; ++i)
                nan_nibbles |= (v[i] != v[i]) ? (0xFu << (4 * i)) : 0u;
            packed = (packed & ~nan_nibbles) | (0x77777777u & nan_nibbles);
            const uint32_t sb = f2u(sc);  // StoreMxEncodedValue's two special scalings (TQuant.hpp:349-372)
            if ((sb & 0x7FFFFFFFu) == 0x7F800000u)
                packed = (sb >> 31) ? 0xFFFFFFFFu : 0x77777777u;
            else if ((sb & 0x7FFFFFFFu) > 0x7F800000u)
                packed = 0x77777777u;
            if (live) {
                if (EPL == 8)
                    reinterpret_cast<uint32_t*>(dst)[unit] = packed;
                else
                    reinterpret_cast<uint16_t*>(dst)[unit] = (uint16_t)packed;
            }
        } else {
            uint32_t words[EPL / 4];
            // The hardware conversion rounds every finite value inside +-448 exactly as EncodeE4M3Fn does (all 2^32
            // float patterns compared); it differs beyond 448 (NaN code instead of saturation), on NaN (0xFF instead
            // of 0x7F) and on negative values that round to zero (0x80 instead of 0x00).  So a lane whose own elements
            // hold no NaN (the group maximum ignores NaNs, so it cannot tell) clamps, converts in pairs and clears
            // the sign of zero codes; a lane with a NaN takes the software encoder.  Both give the same codes wherever
            // both apply, so the lanes of a group need not agree.
            uint32_t largest = 0;
#pragma unroll
            for (int i = 0; i < EPL; ++i)
                largest = max(largest, f2u(v[i]) & 0x7FFFFFFFu);
            const bool fast = ALG == PTOAMD_OCP_MXFP8 && largest <= 0x7F800000u && (f2u(sc) & 0x7F800000u) != 0x7F800000u;
            if (fast) {
                static_for<EPL / 4>([&](auto wc) {
                    constexpr int w = decltype(wc)::value;
                    float t[4];
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        t[i] = __builtin_amdgcn_fmed3f(__fmul_rn(v[4 * w + i], sc), -448.0f, 448.0f);
                    short2v pk = {0, 0};
                    pk = __builtin_amdgcn_cvt_scalef32_pk_fp8_f32(pk, t[0], t[1], 1.0f, false);
                    pk = __builtin_amdgcn_cvt_scalef32_pk_fp8_f32(pk, t[2], t[3], 1.0f, true);
                    const uint32_t x = __builtin_bit_cast(uint32_t, pk);
                    const uint32_t nonzero = ((x & 0x7F7F7F7Fu) + 0x7F7F7F7Fu) & 0x80808080u;  // bit 7 of bytes whose magnitude is not 0
                    words[w] = x & (nonzero | 0x7F7F7F7Fu);
                });
            } else {
                uint32_t c[EPL];
#pragma unroll
                for (int i = 0; i < EPL; ++i)
                    c[i] = encode_mx<ALG, SRC_BF16>(v[i], sc);
#pragma unroll
                for (int w = 0; w < EPL / 4; ++w)
                    words[w] = c[4 * w] | (c[4 * w + 1] << 8) | (c[4 * w + 2] << 16) | (c[4 * w + 3] << 24);
            }
            if (live) {
                if constexpr (EPL == 8)
                    reinterpret_cast<uint2*>(dst)[unit] = make_uint2(words[0], words[1]);
                else
                    reinterpret_cast<uint32_t*>(dst)[unit] = words[0];
            }
        }
    }
}

// ---- axis 0: 32-element groups along a column.  One thread owns two adjacent columns of one group. -----------
template <int ALG, typename T, bool SRC_BF16>
__global__ void tquant_mx_cols_kernel(uint8_t* dst, uint8_t* exp, float* mx, float* scaling, const T* src, int rows,
                                      int cols)
{
    constexpr bool FP4 = ALG == PTOAMD_OCP_MXFP4 || ALG == PTOAMD_NV_MXFP4;
    const int cp = blockIdx.x * blockDim.x + threadIdx.x;  // column pair
    const int g = blockIdx.y;
    if (cp * 2 >= cols)
        return;
    const T* p = src + (long)g * 32 * cols + cp * 2;
    uint32_t run[2] = {0, 0};
    for (int r = 0; r < 32; ++r) {
        run[0] = max_step<ALG>(run[0], widen<T>(p[(long)r * cols]), r);
        run[1] = max_step<ALG>(run[1], widen<T>(p[(long)r * cols + 1]), r);
    }
    float sc[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const float maxabs = max_value<ALG>(run[j]);
        const uint32_t e = shared_exponent<ALG>(maxabs);
        sc[j] = group_scaling<ALG>(maxabs, e);
        const long gi = (long)g * cols + cp * 2 + j;
        exp[gi] = (uint8_t)e;
        if (mx)
            mx[gi] = maxabs;
        if (scaling)
            scaling[gi] = sc[j];
    }
    for (int r = 0; r < 32; ++r) {
        const uint32_t c0 = encode_mx<ALG, SRC_BF16>(widen<T>(p[(long)r * cols]), sc[0]);
        const uint32_t c1 = encode_mx<ALG, SRC_BF16>(widen<T>(p[(long)r * cols + 1]), sc[1]);
        const long idx = ((long)g * 32 + r) * cols + cp * 2;
        if (FP4)
            dst[idx >> 1] = (uint8_t)(c0 | (c1 << 4));
        else
            reinterpret_cast<uint16_t*>(dst)[idx >> 1] = (uint16_t)(c0 | (c1 << 8));
    }
}

// ---- TQUANT INT8 (TQuant.hpp:86-96, 496-522): the "scale" operand multiplies -----------------------------------
template <bool ASYM>
__global__ void tquant_int8_kernel(uint8_t* dst, const float* src, const float* scale, const float* offset, int rows,
                                   int cols, int para_rows, int para_ld)
{
    const long idx4 = ((long)blockIdx.x * blockDim.x + threadIdx.x) * 4;
    const long total = (long)rows * cols;
    if (idx4 >= total)
        return;
    uint32_t packed = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const long idx = idx4 + i;
        if (idx >= total)
            break;
        // GetParamValue (TQuant.hpp:78-84): column 0 of the parameter tile, the row clamped to its last valid one
        const long pr = (long)min((int)(idx / cols), para_rows - 1) * para_ld;
        float v = __fmul_rn(src[idx], scale[pr]);
        if (ASYM)
            v = __fadd_rn(v, offset[pr]);
        v = rintf(v);
        const float lo = ASYM ? 0.0f : -128.0f, hi = ASYM ? 255.0f : 127.0f;
        v = v < lo ? lo : (v > hi ? hi : v);
        const int q = (int)v;
        packed |= ((uint32_t)q & 0xFFu) << (8 * i);
    }
    if (idx4 + 4 <= total && (total & 3) == 0) {
        reinterpret_cast<uint32_t*>(dst)[idx4 >> 2] = packed;
    } else {
        for (int i = 0; i < 4 && idx4 + i < total; ++i)
            dst[idx4 + i] = (uint8_t)(packed >> (8 * i));
    }
}

// Row-parallel forms for matrices whose rows are whole 4-element pieces: blockIdx.y is the row (no division to find the
// per-row scale), a lane moves four elements per piece -- 16 bytes of f32 in, one dword out -- and UNITS pieces per thread.
template <bool ASYM>
__global__ void __launch_bounds__(256) tquant_int8_rows_kernel(uint8_t* dst, const float* src, const float* scale, const float* offset, int cols)
{
    constexpr int UNITS = 2;
    const int r = blockIdx.y;
    const float s = scale[r], o = ASYM ? offset[r] : 0.0f;
    const float4* in = reinterpret_cast<const float4*>(src + (long)r * cols);
    uint32_t* out = reinterpret_cast<uint32_t*>(dst + (long)r * cols);
    const int pieces = cols >> 2, first = blockIdx.x * (UNITS * 256) + threadIdx.x;
    float4 v[UNITS];
#pragma unroll
    for (int u = 0; u < UNITS; ++u)
        v[u] = first + u * 256 < pieces ? in[first + u * 256] : make_float4(0, 0, 0, 0);
#pragma unroll
    for (int u = 0; u < UNITS; ++u) {
        const float x[4] = {v[u].x, v[u].y, v[u].z, v[u].w};
        uint32_t packed = 0;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            float q = __fmul_rn(x[i], s);
            if (ASYM)
                q = __fadd_rn(q, o);
            q = rintf(q);
            const float lo = ASYM ? 0.0f : -128.0f, hi = ASYM ? 255.0f : 127.0f;
            q = q < lo ? lo : (q > hi ? hi : q);
            packed |= ((uint32_t)(int)q & 0xFFu) << (8 * i);
        }
        if (first + u * 256 < pieces)
            out[first + u * 256] = packed;
    }
}

template <typename T>
__global__ void __launch_bounds__(256) tdequant_rows_kernel(float* dst, const T* src, const float* scale, const float* offset, int cols)
{
    constexpr int UNITS = 2;
    const int r = blockIdx.y;
    const float s = scale[r], o = offset[r];
    struct alignas(4 * sizeof(T)) Piece { T e[4]; };
    const Piece* in = reinterpret_cast<const Piece*>(src + (long)r * cols);
    float4* out = reinterpret_cast<float4*>(dst + (long)r * cols);
    const int pieces = cols >> 2, first = blockIdx.x * (UNITS * 256) + threadIdx.x;
    Piece v[UNITS];
#pragma unroll
    for (int u = 0; u < UNITS; ++u)
        if (first + u * 256 < pieces)
            v[u] = in[first + u * 256];
#pragma unroll
    for (int u = 0; u < UNITS; ++u)
        if (first + u * 256 < pieces)
            out[first + u * 256] = make_float4(__fmul_rn(__fsub_rn((float)v[u].e[0], o), s), __fmul_rn(__fsub_rn((float)v[u].e[1], o), s),
                                               __fmul_rn(__fsub_rn((float)v[u].e[2], o), s), __fmul_rn(__fsub_rn((float)v[u].e[3], o), s));
}

// ---- TDEQUANT (TDeQuant.hpp:18-37) ---------------------------------------------------------------------------
template <typename T>
__global__ void tdequant_kernel(float* dst, const T* src, const float* scale, const float* offset, int rows, int cols,
                                int para_cols, int para_ld)
{
    const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (long)rows * cols)
        return;
    const int r = (int)(idx / cols), c = (int)(idx - (long)r * cols);
    const long pi = (long)r * para_ld + min(c, para_cols - 1);  // TDeQuant.hpp:24-30: the parameter column is clamped
    dst[idx] = __fmul_rn(__fsub_rn((float)src[idx], offset[pi]), scale[pi]);
}

template <int ALG, typename T, bool SRC_BF16>
static int launch_tquant_mx(uint8_t* dst, uint8_t* exp, float* mx, float* scaling, const void* src, int rows, int cols,
                            int axis, hipStream_t stream)
{
    const T* s = reinterpret_cast<const T*>(src);
    if (axis == 1) {
        const long units = (long)rows * cols * (long)sizeof(T) / 16;  // 16-byte pieces; a row is a whole number of them
        hipLaunchKernelGGL((tquant_mx_rows_kernel<ALG, T, SRC_BF16>), dim3((unsigned)((units + 1023) / 1024)), dim3(256),
                           0, stream, dst, exp, mx, scaling, s, units);
    } else {
        dim3 block(128), grid((cols / 2 + 127) / 128, rows / 32);
        hipLaunchKernelGGL((tquant_mx_cols_kernel<ALG, T, SRC_BF16>), grid, block, 0, stream, dst, exp, mx, scaling, s,
                           rows, cols);
    }
    PTOAMD_HIP_CHECK(hipGetLastError());
    set_last_kernel(axis == 1 ? "tquant_mx_rows" : "tquant_mx_cols");
    return PTOAMD_OK;
}

template <int ALG>
static int dispatch_src(uint8_t* dst, uint8_t* exp, float* mx, float* scaling, const void* src, int src_type, int rows,
                        int cols, int axis, hipStream_t stream)
{
    switch (src_type) {
        case PTOAMD_F32: return launch_tquant_mx<ALG, float, false>(dst, exp, mx, scaling, src, rows, cols, axis, stream);
        case PTOAMD_F16: return launch_tquant_mx<ALG, half_bits, false>(dst, exp, mx, scaling, src, rows, cols, axis, stream);
        default: return launch_tquant_mx<ALG, bf16_bits, true>(dst, exp, mx, scaling, src, rows, cols, axis, stream);
    }
}

}  // namespace ptoamd

using namespace ptoamd;

extern "C" {

int ptoamd_tquant_int8(void* dst, const float* src, const float* scale, const float* offset, int rows, int cols,
                       void* stream)
{
    return ptoamd_tquant_int8_para(dst, src, scale, offset, rows, cols, rows, 1, stream);
}

int ptoamd_tquant_int8_para(void* dst, const float* src, const float* scale, const float* offset, int rows, int cols,
                            int para_rows, int para_ld, void* stream)
{
    TraceScope trace(offset ? "TQUANT_INT8_ASYM" : "TQUANT_INT8_SYM", "vector", rows, cols, 0);
    trace.in(src, rows, cols, "ND", PTOAMD_F32).in(scale, para_rows, 1, "ND", PTOAMD_F32).in(offset, para_rows, 1, "ND", PTOAMD_F32)
        .out(dst, rows, cols, "ND", offset ? PTOAMD_U8 : PTOAMD_I8);
    PTOAMD_REQUIRE(dst && src && scale, PTOAMD_E_INVALID, "ptoamd_tquant_int8: null operand");
    PTOAMD_REQUIRE(rows > 0 && cols > 0, PTOAMD_E_INVALID, "ptoamd_tquant_int8: rows and cols must be positive");
    PTOAMD_REQUIRE(para_rows > 0 && para_ld > 0, PTOAMD_E_INVALID,
                   "ptoamd_tquant_int8: the parameter tile needs at least one row and a positive row pitch");
    const long total = (long)rows * cols;
    if (para_rows >= rows && para_ld == 1 && (cols & 3) == 0 && rows <= 65535 && (reinterpret_cast<uintptr_t>(src) & 15u) == 0 && (reinterpret_cast<uintptr_t>(dst) & 3u) == 0) {
        const dim3 grid((unsigned)((cols / 4 + 511) / 512), (unsigned)rows);
        if (offset)
            hipLaunchKernelGGL(tquant_int8_rows_kernel<true>, grid, dim3(256), 0, as_stream(stream),
                               reinterpret_cast<uint8_t*>(dst), src, scale, offset, cols);
        else
            hipLaunchKernelGGL(tquant_int8_rows_kernel<false>, grid, dim3(256), 0, as_stream(stream),
                               reinterpret_cast<uint8_t*>(dst), src, scale, offset, cols);
        PTOAMD_HIP_CHECK(hipGetLastError());
        set_last_kernel("tquant_int8_rows");
        return PTOAMD_OK;
    }
    const unsigned blocks = (unsigned)((total / 4 + 256) / 256);
    if (offset)
        hipLaunchKernelGGL(tquant_int8_kernel<true>, dim3(blocks), dim3(256), 0, as_stream(stream),
                           reinterpret_cast<uint8_t*>(dst), src, scale, offset, rows, cols, para_rows, para_ld);
    else
        hipLaunchKernelGGL(tquant_int8_kernel<false>, dim3(blocks), dim3(256), 0, as_stream(stream),
                           reinterpret_cast<uint8_t*>(dst), src, scale, offset, rows, cols, para_rows, para_ld);
    PTOAMD_HIP_CHECK(hipGetLastError());
    set_last_kernel("tquant_int8");
    return PTOAMD_OK;
}

int ptoamd_tquant_mx(uint8_t* dst, uint8_t* exp, float* max, float* scaling, const void* src, int src_type, int rows,
                     int cols, int alg, int axis, void* stream)
{
    const bool fp4 = alg == PTOAMD_OCP_MXFP4 || alg == PTOAMD_NV_MXFP4;
    TraceScope trace(fp4 ? "TQUANT_MXFP4" : "TQUANT_MXFP8", "vector", rows, cols, 0);
    trace.in(src, rows, cols, "ND", src_type).out(dst, rows, cols, "ND", fp4 ? PTOAMD_E2M1 : PTOAMD_E4M3)
        .out(exp, axis == 1 ? rows : rows / 32, axis == 1 ? cols / 32 : cols, "ND", 100)
        .out(max, axis == 1 ? rows : rows / 32, axis == 1 ? cols / 32 : cols, "ND", PTOAMD_F32)
        .out(scaling, axis == 1 ? rows : rows / 32, axis == 1 ? cols / 32 : cols, "ND", PTOAMD_F32);
    PTOAMD_REQUIRE(dst && exp && src, PTOAMD_E_INVALID, "ptoamd_tquant_mx: null operand");
    PTOAMD_REQUIRE(rows > 0 && cols > 0, PTOAMD_E_INVALID, "ptoamd_tquant_mx: rows and cols must be positive");
    PTOAMD_REQUIRE(axis == 0 || axis == 1, PTOAMD_E_INVALID, "ptoamd_tquant_mx: axis must be 0 or 1");
    PTOAMD_REQUIRE(src_type == PTOAMD_F32 || src_type == PTOAMD_F16 || src_type == PTOAMD_BF16, PTOAMD_E_UNSUPPORTED,
                   "ptoamd_tquant_mx: the source must be f32, f16 or bf16");
    PTOAMD_REQUIRE(axis == 1 ? cols % 32 == 0 : rows % 32 == 0, PTOAMD_E_INVALID,
                   "ptoamd_tquant_mx: the grouped axis must be a multiple of 32 (rows %d, cols %d, axis %d)", rows, cols, axis);
    PTOAMD_REQUIRE(cols % 2 == 0, PTOAMD_E_INVALID, "ptoamd_tquant_mx: cols must be even");
    PTOAMD_REQUIRE((reinterpret_cast<uintptr_t>(dst) & 7u) == 0 && (reinterpret_cast<uintptr_t>(src) & 15u) == 0,
                   PTOAMD_E_ALIGNMENT, "ptoamd_tquant_mx: dst must be 8-byte and src 16-byte aligned");
    hipStream_t s = as_stream(stream);
    switch (alg) {
        case PTOAMD_OCP_MXFP8: return dispatch_src<PTOAMD_OCP_MXFP8>(dst, exp, max, scaling, src, src_type, rows, cols, axis, s);
        case PTOAMD_NV_MXFP8: return dispatch_src<PTOAMD_NV_MXFP8>(dst, exp, max, scaling, src, src_type, rows, cols, axis, s);
        case PTOAMD_OCP_MXFP4: return dispatch_src<PTOAMD_OCP_MXFP4>(dst, exp, max, scaling, src, src_type, rows, cols, axis, s);
        case PTOAMD_NV_MXFP4: return dispatch_src<PTOAMD_NV_MXFP4>(dst, exp, max, scaling, src, src_type, rows, cols, axis, s);
        default: set_error("ptoamd_tquant_mx: unknown algorithm %d", alg); return PTOAMD_E_INVALID;
    }
}

int ptoamd_tdequant(float* dst, const void* src, int src_type, const float* scale, const float* offset, int rows,
                    int cols, void* stream)
{
    return ptoamd_tdequant_para(dst, src, src_type, scale, offset, rows, cols, 1, 1, stream);
}

int ptoamd_tdequant_para(float* dst, const void* src, int src_type, const float* scale, const float* offset, int rows,
                         int cols, int para_cols, int para_ld, void* stream)
{
    TraceScope trace("TDEQUANT", "vector", rows, cols, 0);
    trace.in(src, rows, cols, "ND", src_type).in(scale, rows, para_cols, "ND", PTOAMD_F32).in(offset, rows, para_cols, "ND", PTOAMD_F32)
        .out(dst, rows, cols, "ND", PTOAMD_F32);
    PTOAMD_REQUIRE(dst && src && scale && offset, PTOAMD_E_INVALID, "ptoamd_tdequant: null operand");
    PTOAMD_REQUIRE(rows > 0 && cols > 0, PTOAMD_E_INVALID, "ptoamd_tdequant: rows and cols must be positive");
    PTOAMD_REQUIRE(para_cols > 0 && para_ld >= para_cols, PTOAMD_E_INVALID,
                   "ptoamd_tdequant: the parameter tile needs at least one column and a row pitch that holds its columns");
    const long total = (long)rows * cols;
    const dim3 grid((unsigned)((total + 255) / 256)), block(256);
    hipStream_t s = as_stream(stream);
    if (para_cols == 1 && para_ld == 1 && (cols & 3) == 0 && rows <= 65535 && (reinterpret_cast<uintptr_t>(src) & 15u) == 0 && (reinterpret_cast<uintptr_t>(dst) & 15u) == 0) {
        const dim3 rgrid((unsigned)((cols / 4 + 511) / 512), (unsigned)rows);
        switch (src_type) {
            case PTOAMD_I8:
                hipLaunchKernelGGL(tdequant_rows_kernel<int8_t>, rgrid, block, 0, s, dst, reinterpret_cast<const int8_t*>(src), scale, offset, cols);
                break;
            case PTOAMD_I16:
                hipLaunchKernelGGL(tdequant_rows_kernel<int16_t>, rgrid, block, 0, s, dst, reinterpret_cast<const int16_t*>(src), scale, offset, cols);
                break;
            case PTOAMD_I32:
                hipLaunchKernelGGL(tdequant_rows_kernel<int32_t>, rgrid, block, 0, s, dst, reinterpret_cast<const int32_t*>(src), scale, offset, cols);
                break;
            default: set_error("ptoamd_tdequant: source type %d is not int8, int16 or int32", src_type); return PTOAMD_E_UNSUPPORTED;
        }
        PTOAMD_HIP_CHECK(hipGetLastError());
        set_last_kernel("tdequant_rows");
        return PTOAMD_OK;
    }
    switch (src_type) {
        case PTOAMD_I8:
            hipLaunchKernelGGL(tdequant_kernel<int8_t>, grid, block, 0, s, dst, reinterpret_cast<const int8_t*>(src), scale, offset, rows, cols, para_cols, para_ld);
            break;
        case PTOAMD_I16:
            hipLaunchKernelGGL(tdequant_kernel<int16_t>, grid, block, 0, s, dst, reinterpret_cast<const int16_t*>(src), scale, offset, rows, cols, para_cols, para_ld);
            break;
        case PTOAMD_I32:
            hipLaunchKernelGGL(tdequant_kernel<int32_t>, grid, block, 0, s, dst, reinterpret_cast<const int32_t*>(src), scale, offset, rows, cols, para_cols, para_ld);
            break;
        default: set_error("ptoamd_tdequant: source type %d is not int8, int16 or int32", src_type); return PTOAMD_E_UNSUPPORTED;
    }
    PTOAMD_HIP_CHECK(hipGetLastError());
    set_last_kernel("tdequant");
    return PTOAMD_OK;
}

}  // extern "C"
