/*
 * TEST INFRASTRUCTURE ONLY — parity checker and "port" CPU baseline, never part of the product path.
 *
 * Plain-C restatement of the PTO CPU simulator's tile-matmul hot path.  Citations are relative to the
 * reference tree (include/pto/...).
 *
 * Pinning status (what proves each function equals the reference):
 *   pto_f32_to_f16 / pto_f16_to_f32        numpy float16 conversion (independent IEEE implementation), all 65536
 *                                          half codes and rounding boundaries.
 *   pto_f32_to_bf16                        torch float32->bfloat16 (independent RNE) and the bit formula's
 *                                          boundary cases.
 *   pto_mx_decode / encode_*               compiled reference (oracle/_ref) over all codes / dense value sweeps,
 *                                          frozen in tests/golden; E4M3 decode also against the OCP value table.
 *   pto_tile_offset / pto_global_offset    compiled reference over whole tiles and over 5-D ND / DN / NZ tensors with
 *   / pto_layout_2d                        every outer dimension above 1 and padded strides, frozen in tests/golden;
 *                                          bijection property; ND / DN equal numpy's strided views.
 *   pto_reorder_exp_zz                     compiled reference, frozen in tests/golden; equals the MX_A_ZZ offset map.
 *   pto_matmul_*                           compiled reference bit for bit; exact integer identities on the
 *                                          reference tests' own input distribution (randint(1,5)); the
 *                                          accIn = 1e8 K-order case of tmatmul_layout; int64 reference mod 2^32.
 *   pto_matmul_mx                          compiled reference bit for bit (all four element types, three scale
 *                                          layouts); float64 closed form of tmatmul_mx/gen_data.py to 1e-3.
 *   pto_store_* / pto_quant_word_scale     compiled reference bit for bit; tquantmode KATs (unit scale word,
 *                                          0.5 * 2.0, saturation to 65504).
 *   pto_tquant_* / pto_tdequant            compiled reference bit for bit on the tquant/tquant_dn test patterns;
 *                                          tquant/main.cpp edge KATs (inf/zero/NaN exponents); exhaustive
 *                                          nearest-code property for E4M3.
 *   pto_sim_gemm_*_tiled                   equality with pto_matmul_* (same arithmetic, tiled walk).
 * bf16 inputs cannot be driven through the compiled reference (its bfloat16_t degrades to _Float16 without
 * <stdfloat>); pto_matmul_bf16 is pinned through pto_matmul_f32 on bf16-representable inputs, where fp32 fma of
 * exact products is the same operation.
 */
#include "pto_oracle.h"

#include <math.h>
#include <pthread.h>
#include <stdlib.h>
#include <string.h>
#include <unistd.h>

static inline uint32_t f2u(float f)
{
    uint32_t u;
    memcpy(&u, &f, 4);
    return u;
}
static inline float u2f(uint32_t u)
{
    float f;
    memcpy(&f, &u, 4);
    return f;
}
static inline uint64_t d2u(double d)
{
    uint64_t u;
    memcpy(&u, &d, 8);
    return u;
}
static inline double u2d(uint64_t u)
{
    double d;
    memcpy(&d, &u, 8);
    return d;
}

/* ============================== half / bfloat16 ============================================ */

float pto_f16_to_f32(uint16_t h)
{
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    const uint32_t e = (h >> 10) & 0x1Fu;
    const uint32_t m = h & 0x3FFu;
    if (e == 0) {
        if (m == 0)
            return u2f(sign);
        return (sign ? -1.0f : 1.0f) * ldexpf((float)m, -24);
    }
    if (e == 31)
        return u2f(sign | 0x7F800000u | (m << 13));
    return u2f(sign | ((e + 112u) << 23) | (m << 13));
}

uint16_t pto_f32_to_f16(float f)
{
    const uint32_t x = f2u(f);
    const uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    const uint32_t a = x & 0x7FFFFFFFu;
    if (a >= 0x7F800000u) {
        if (a > 0x7F800000u)
            return (uint16_t)(sign | 0x7E00u | ((a >> 13) & 0x3FFu));
        return (uint16_t)(sign | 0x7C00u);
    }
    if (a >= 0x477FF000u) /* >= 65520 rounds to infinity */
        return (uint16_t)(sign | 0x7C00u);
    if (a < 0x38800000u) { /* below the smallest normal half, 2^-14 */
        if (a <= 0x33000000u) /* <= 2^-25: nearest (ties to even) is zero */
            return sign;
        const uint32_t e = a >> 23;
        const uint32_t m = (a & 0x7FFFFFu) | 0x800000u;
        const uint32_t shift = 126u - e; /* 14 .. 24 */
        uint32_t hm = m >> shift;
        const uint32_t rem = m & ((1u << shift) - 1u);
        const uint32_t halfway = 1u << (shift - 1u);
        if (rem > halfway || (rem == halfway && (hm & 1u)))
            hm++;
        return (uint16_t)(sign | hm);
    }
    uint32_t h = (((a >> 23) - 112u) << 10) | ((a & 0x7FFFFFu) >> 13);
    const uint32_t rem = a & 0x1FFFu;
    if (rem > 0x1000u || (rem == 0x1000u && (h & 1u)))
        h++;
    return (uint16_t)(sign | h);
}

float pto_bf16_to_f32(uint16_t h) { return u2f((uint32_t)h << 16); }

/* cpu/TQuant.hpp:49-55 (FloatToBf16BitsRound); NaN keeps a quiet payload instead of carrying into the sign */
uint16_t pto_f32_to_bf16(float f)
{
    const uint32_t bits = f2u(f);
    if ((bits & 0x7FFFFFFFu) > 0x7F800000u)
        return (uint16_t)((bits >> 16) | 0x0040u);
    const uint32_t lsb = (bits >> 16) & 1u;
    return (uint16_t)((bits + 0x7FFFu + lsb) >> 16);
}

/* ============================== MX element types (cpu/MXTypes.hpp) ========================== */

static void mx_params(int type, int* exp_sz, int* man_sz, int* bias)
{
    switch (type) {
        case PTO_E4M3: *exp_sz = 4; *man_sz = 3; *bias = 7; break;
        case PTO_E5M2: *exp_sz = 5; *man_sz = 2; *bias = 15; break;
        case PTO_E2M1: *exp_sz = 2; *man_sz = 1; *bias = 1; break;
        case PTO_E1M2: *exp_sz = 1; *man_sz = 2; *bias = 1; break;
        default: *exp_sz = 8; *man_sz = 0; *bias = 127; break;
    }
}

/* MXTypes.hpp:232-274 (operator double) */
double pto_mx_decode(int type, unsigned raw)
{
    int es, ms, bias;
    mx_params(type, &es, &ms, &bias);
    const unsigned data = raw & 0xFFu;
    const uint64_t mant = data & ((1u << ms) - 1u);
    const uint64_t expo = (data >> ms) & ((1u << es) - 1u);
    const uint64_t sign = (data >> (ms + es)) & 1u;
    if (type == PTO_E4M3 || type == PTO_E5M2) {
        const unsigned mag = data & 0x7Fu;
        if ((type == PTO_E4M3 && mag == 0x7Fu) || (type == PTO_E5M2 && mag > 0x7Cu))
            return copysign(NAN, sign ? -1.0 : 1.0);
        if (type == PTO_E5M2 && mag == 0x7Cu)
            return sign ? -INFINITY : INFINITY;
        if (mag == 0)
            return sign ? -0.0 : 0.0;
        const double v = expo == 0 ? ldexp((double)mant, 1 - bias - ms)
                                   : ldexp((double)((1u << ms) + mant), (int)expo - bias - ms);
        return sign ? -v : v;
    }
    if (expo > 0 || ms == 0)
        return u2d((sign << 63) | ((expo + 1023u - (unsigned)bias) << 52) | (mant << (52 - ms)));
    if (data == 0 || data == (1u << (ms + es)))
        return 0.0; /* the generic path decodes the "negative zero" code to +0 */
    int i = ms - 1;
    while (i >= 0 && !((mant >> i) & 1u))
        i--;
    return u2d((sign << 63) | ((uint64_t)(1023 - bias + 1 + (i - ms)) << 52) |
               ((mant & ((1ull << i) - 1ull)) << (52 - i)));
}

/* MXTypes.hpp:47-93: the plain MXType(double) constructor truncates the mantissa, no rounding, no saturation */
unsigned pto_mx_encode_trunc(int type, double v)
{
    int es, ms, bias;
    mx_params(type, &es, &ms, &bias);
    if (v == 0.0)
        return 0;
    const uint64_t bits = d2u(v);
    const uint64_t sign = bits >> 63;
    const int64_t dexp = (int64_t)((bits >> 52) & 0x7FFu);
    const uint64_t dman = bits & ((1ull << 52) - 1ull);
    if (dexp <= 0)
        return 0; /* double subnormals collapse to zero */
    uint64_t oman = dman >> (52 - ms);
    int64_t oexp = dexp + bias - 1023;
    if (oexp < 0) {
        const int64_t sh = 1 - oexp;
        oman = sh >= 64 ? 0 : ((oman | (1ull << ms)) >> sh);
        oexp = 0;
    }
    return (unsigned)(((sign << (ms + es)) | (((uint64_t)oexp & ((1ull << es) - 1ull)) << ms) |
                       (oman & ((1ull << ms) - 1ull))) & 0xFFu);
}

/* MXTypes.hpp:95-170: rounding constructor for E4M3 / E5M2 (used by TCVT) */
unsigned pto_fp8_encode_round(int type, double v, int mode, int sat_on)
{
    const int e4 = (type == PTO_E4M3);
    const int ms = e4 ? 3 : 2, bias = e4 ? 7 : 15;
    const unsigned max_code = e4 ? 0x7Eu : 0x7Bu, overflow_code = e4 ? 0x7Fu : 0x7Cu;
    const int max_exponent = e4 ? 8 : 15;
    const double max_value = e4 ? 448.0 : 57344.0;
    const unsigned sign = signbit(v) ? 0x80u : 0u;
    const double mag = fabs(v);
    if (isnan(v))
        return sign | 0x7Fu;
    if (sat_on && mag >= max_value)
        return sign | max_code;
    if (isinf(v))
        return sign | overflow_code;
    if (mag == 0)
        return sign;
    const int toward_zero = mode == PTO_CAST_TRUNC || (mode == PTO_CAST_FLOOR && !sign) ||
                            (mode == PTO_CAST_CEIL && sign);
    if (mag >= ldexp(1.0, max_exponent + 1))
        return sign | ((!e4 && toward_zero) ? max_code : overflow_code);
    int exponent;
    (void)frexp(mag, &exponent);
    exponent = exponent - 1 > 1 - bias ? exponent - 1 : 1 - bias;
    const double scaled = ldexp(mag, ms - exponent);
    unsigned sig = (unsigned)scaled;
    const double rem = scaled - sig;
    switch (mode) {
        case PTO_CAST_ROUND: sig += rem >= 0.5; break;
        case PTO_CAST_FLOOR: sig += sign && rem != 0; break;
        case PTO_CAST_CEIL: sig += !sign && rem != 0; break;
        case PTO_CAST_TRUNC: break;
        default: sig += rem > 0.5 || (rem == 0.5 && (sig & 1u)); break;
    }
    if (sig == (2u << ms)) {
        sig >>= 1;
        ++exponent;
    }
    unsigned code = sig < (1u << ms) ? sig : (((unsigned)(exponent + bias) << ms) + sig - (1u << ms));
    if (code > max_code)
        code = (sat_on || (!e4 && toward_zero)) ? max_code : overflow_code;
    return sign | code;
}

/* MXTypes.hpp:172-230: rounding constructor for E2M1 / E1M2 by grid search */
unsigned pto_fp4_encode_round(int type, double val, int mode)
{
    static const float grid_e1m2[8] = {0.0f, 0.25f, 0.5f, 0.75f, 1.0f, 1.25f, 1.5f, 1.75f};
    static const float grid_e2m1[8] = {0.0f, 0.5f, 1.0f, 1.5f, 2.0f, 3.0f, 4.0f, 6.0f};
    const float* grid = type == PTO_E1M2 ? grid_e1m2 : grid_e2m1;
    const unsigned sign = (val < 0.0) ? 8u : 0u;
    val = fabs(val);
    if (val >= grid[7])
        return sign | 7u;
    int upper = 0;
    while (upper < 8 && !(val < (double)grid[upper])) /* std::upper_bound */
        upper++;
    const int lower = upper - 1;
    const float midpoint = (grid[lower] + grid[upper]) / 2.0f;
    const int is_tie = fabs(val - (double)midpoint) <= (double)1e-8f;
    const int tie_bit = mode == PTO_CAST_ODD;
    int code = lower;
    switch (mode) {
        case PTO_CAST_FLOOR: code = sign == 0 ? lower : upper; break;
        case PTO_CAST_CEIL: code = sign == 0 ? upper : lower; break;
        case PTO_CAST_TRUNC: code = lower; break;
        default:
            if (is_tie) {
                if (lower % 2 == tie_bit)
                    code = lower;
                else if (upper % 2 == tie_bit)
                    code = upper;
            } else {
                code = (val < (double)midpoint) ? lower : upper;
            }
            break;
    }
    return sign | (unsigned)code;
}

/* ============================== addressing (cpu/tile_offsets.hpp) ========================== */

/* common/pto_tile.hpp:1460-1486 (getInnerRow / getInnerCol) */
void pto_tile_layout_init(pto_tile_layout* t, int rows, int cols, int row_major, int sfractal, int sfractal_size,
                          int elem_bytes, int packed2)
{
    t->rows = rows;
    t->cols = cols;
    t->row_major = row_major;
    t->sfractal = sfractal;
    const int inner_rm = sfractal == 1;
    const int c0 = (packed2 ? 2 : 1) * 32 / elem_bytes;
    if (sfractal == 0) {
        t->inner_rows = t->inner_cols = 1;
    } else if (sfractal_size == 1024) {
        t->inner_rows = t->inner_cols = 16;
    } else if (sfractal_size == 32) {
        t->inner_rows = inner_rm ? 16 : 2;
        t->inner_cols = inner_rm ? 2 : 16;
    } else {
        t->inner_rows = inner_rm ? 16 : c0;
        t->inner_cols = inner_rm ? c0 : 16;
    }
}

/* cpu/tile_offsets.hpp:41-87 */
int64_t pto_tile_offset(const pto_tile_layout* t, int r, int c)
{
    if (t->sfractal == 0)
        return t->row_major ? (int64_t)r * t->cols + c : (int64_t)c * t->rows + r;
    const int64_t ir = t->inner_rows, ic = t->inner_cols, numel = ir * ic;
    const int64_t sr = r / ir, inr = r % ir, sc = c / ic, inc = c % ic;
    if (!t->row_major && t->sfractal == 1) /* Nz */
        return sc * t->rows * ic + sr * numel + inr * ic + inc;
    if (t->row_major && t->sfractal == 2) /* Zn */
        return sr * t->cols * ir + sc * numel + inc * ir + inr;
    if (t->row_major && t->sfractal == 1) /* Zz */
        return sr * t->cols * ir + sc * numel + inr * ic + inc;
    return sc * t->rows * ic + sr * numel + inc * ir + inr; /* Nn */
}

/* cpu/tile_offsets.hpp:181-277 (MapTileIndicesToGlobalOffset) */
int64_t pto_global_offset(int layout, int64_t r, int64_t c, const int64_t shape[5], const int64_t stride[5])
{
    int64_t i0 = 0, i1 = 0, i2 = 0, i3 = 0, i4 = 0;
    switch (layout) {
        case PTO_ND:
            i4 = c;
            i3 = r % shape[3];
            i2 = (r / shape[3]) % shape[2];
            i1 = (r / (shape[3] * shape[2])) % shape[1];
            i0 = r / (shape[1] * shape[2] * shape[3]);
            break;
        case PTO_DN:
            i3 = r;
            i4 = c % shape[4];
            i2 = (c / shape[4]) % shape[2];
            i1 = (c / (shape[4] * shape[2])) % shape[1];
            i0 = c / (shape[1] * shape[2] * shape[4]);
            break;
        case PTO_NZ: {
            const int64_t outer = c / shape[4];
            i0 = outer / shape[1];
            i1 = outer % shape[1];
            i2 = r / shape[3];
            i3 = r % shape[3];
            i4 = c % shape[4];
            break;
        }
        case PTO_MX_A_ZZ: i1 = r / 16; i2 = c / 2; i3 = r % 16; i4 = c % 2; break;
        case PTO_MX_B_NN: i1 = c / 16; i2 = r / 2; i3 = c % 16; i4 = r % 2; break;
        case PTO_MX_A_ND: i2 = r; i3 = c / 2; i4 = c % 2; break;
        case PTO_MX_A_DN: i2 = c / 2; i3 = r; i4 = c % 2; break;
        case PTO_MX_B_ND: i2 = r / 2; i3 = c; i4 = r % 2; break;
        case PTO_MX_B_DN: i2 = c; i3 = r / 2; i4 = r % 2; break;
        default: return -1;
    }
    return i0 * stride[0] + i1 * stride[1] + i2 * stride[2] + i3 * stride[3] + i4 * stride[4];
}

/* common/pto_tile.hpp:664-1102 (TileShape2D / BaseShape2D for a whole [rows, cols] matrix) */
int pto_layout_2d(int layout, int64_t rows, int64_t cols, int c0, int64_t sh[5], int64_t st[5])
{
    const int64_t all = rows * cols;
    switch (layout) {
        case PTO_ND:
            sh[0] = sh[1] = sh[2] = 1; sh[3] = rows; sh[4] = cols;
            st[0] = st[1] = st[2] = all; st[3] = cols; st[4] = 1;
            return 0;
        case PTO_DN:
            sh[0] = sh[1] = sh[2] = 1; sh[3] = rows; sh[4] = cols;
            st[0] = st[1] = st[2] = all; st[3] = 1; st[4] = rows;
            return 0;
        case PTO_NZ:
            sh[0] = 1; sh[1] = cols / c0; sh[2] = rows / 16; sh[3] = 16; sh[4] = c0;
            st[0] = all; st[1] = rows * c0; st[2] = 16 * c0; st[3] = c0; st[4] = 1;
            return 0;
        case PTO_MX_A_ZZ:
            sh[0] = 1; sh[1] = rows / 16; sh[2] = cols / 2; sh[3] = 16; sh[4] = 2;
            st[0] = all; st[1] = cols * 16; st[2] = 32; st[3] = 2; st[4] = 1;
            return 0;
        case PTO_MX_A_ND:
            sh[0] = sh[1] = 1; sh[2] = rows; sh[3] = cols / 2; sh[4] = 2;
            st[0] = st[1] = all; st[2] = cols; st[3] = 2; st[4] = 1;
            return 0;
        case PTO_MX_A_DN:
            sh[0] = sh[1] = 1; sh[2] = cols / 2; sh[3] = rows; sh[4] = 2;
            st[0] = st[1] = all; st[2] = rows * 2; st[3] = 2; st[4] = 1;
            return 0;
        case PTO_MX_B_NN:
            sh[0] = 1; sh[1] = cols / 16; sh[2] = rows / 2; sh[3] = 16; sh[4] = 2;
            st[0] = all; st[1] = rows * 16; st[2] = 32; st[3] = 2; st[4] = 1;
            return 0;
        case PTO_MX_B_ND:
            sh[0] = sh[1] = 1; sh[2] = rows / 2; sh[3] = cols; sh[4] = 2;
            st[0] = st[1] = all; st[2] = cols * 2; st[3] = 2; st[4] = 1;
            return 0;
        case PTO_MX_B_DN:
            sh[0] = sh[1] = 1; sh[2] = cols; sh[3] = rows / 2; sh[4] = 2;
            st[0] = st[1] = all; st[2] = rows; st[3] = 2; st[4] = 1;
            return 0;
        default: return -1;
    }
}

int64_t pto_mx_scale_offset(int layout, int rows, int cols, int r, int c)
{
    int64_t sh[5], st[5];
    if (pto_layout_2d(layout, rows, cols, 2, sh, st) != 0)
        return -1;
    return pto_global_offset(layout, r, c, sh, st);
}

/* ============================== TMATMUL (cpu/TMatmul.hpp:77-113, 207-230) =================== */

#define B_AT(b, kk, j, ldb, b_dn) ((b_dn) ? (b)[(size_t)(j) * (ldb) + (kk)] : (b)[(size_t)(kk) * (ldb) + (j)])

typedef float (*pto_widen_fn)(const void* p, size_t idx);
static float widen_f16(const void* p, size_t i) { return pto_f16_to_f32(((const uint16_t*)p)[i]); }
static float widen_bf16(const void* p, size_t i) { return pto_bf16_to_f32(((const uint16_t*)p)[i]); }
static float widen_f32(const void* p, size_t i) { return ((const float*)p)[i]; }
static float widen_e4m3(const void* p, size_t i) { return (float)pto_mx_decode(PTO_E4M3, ((const uint8_t*)p)[i]); }
static float widen_e5m2(const void* p, size_t i) { return (float)pto_mx_decode(PTO_E5M2, ((const uint8_t*)p)[i]); }

/* acc = accIn or 0; for k ascending: acc = fma(a, b, acc); bias added after the K loop */
static void matmul_float(float* out, const void* a, const void* b, const float* cin, const float* bias, int m, int k,
                         int n, int lda, int ldb, int ldc, int b_dn, pto_widen_fn wa, pto_widen_fn wb)
{
    float* arow = (float*)malloc(sizeof(float) * (size_t)k);
    float* bcol = (float*)malloc(sizeof(float) * (size_t)k * (size_t)n);
    for (int j = 0; j < n; ++j)
        for (int kk = 0; kk < k; ++kk)
            bcol[(size_t)j * k + kk] = wb(b, b_dn ? (size_t)j * ldb + kk : (size_t)kk * ldb + j);
    for (int i = 0; i < m; ++i) {
        for (int kk = 0; kk < k; ++kk)
            arow[kk] = wa(a, (size_t)i * lda + kk);
        for (int j = 0; j < n; ++j) {
            float acc = cin ? cin[(size_t)i * ldc + j] : 0.0f;
            const float* bc = bcol + (size_t)j * k;
            for (int kk = 0; kk < k; ++kk)
                acc = fmaf(arow[kk], bc[kk], acc);
            if (bias)
                acc += bias[j];
            out[(size_t)i * ldc + j] = acc;
        }
    }
    free(arow);
    free(bcol);
}

void pto_matmul_f16(float* out, const uint16_t* a, const uint16_t* b, const float* cin, const float* bias, int m,
                    int k, int n, int lda, int ldb, int ldc, int b_dn)
{
    matmul_float(out, a, b, cin, bias, m, k, n, lda, ldb, ldc, b_dn, widen_f16, widen_f16);
}
void pto_matmul_bf16(float* out, const uint16_t* a, const uint16_t* b, const float* cin, const float* bias, int m,
                     int k, int n, int lda, int ldb, int ldc, int b_dn)
{
    matmul_float(out, a, b, cin, bias, m, k, n, lda, ldb, ldc, b_dn, widen_bf16, widen_bf16);
}
void pto_matmul_f32(float* out, const float* a, const float* b, const float* cin, const float* bias, int m, int k,
                    int n, int lda, int ldb, int ldc, int b_dn)
{
    matmul_float(out, a, b, cin, bias, m, k, n, lda, ldb, ldc, b_dn, widen_f32, widen_f32);
}
void pto_matmul_fp8(float* out, const uint8_t* a, const uint8_t* b, const float* cin, const float* bias, int m, int k,
                    int n, int lda, int ldb, int ldc, int b_dn, int a_type, int b_type)
{
    matmul_float(out, a, b, cin, bias, m, k, n, lda, ldb, ldc, b_dn, a_type == PTO_E4M3 ? widen_e4m3 : widen_e5m2,
                 b_type == PTO_E4M3 ? widen_e4m3 : widen_e5m2);
}

/* int8 x int8 -> int32 with two's-complement wrap (cpu/TMatmul.hpp:106) */
void pto_matmul_i8(int32_t* out, const int8_t* a, const int8_t* b, const int32_t* cin, const int32_t* bias, int m,
                   int k, int n, int lda, int ldb, int ldc, int b_dn)
{
    for (int i = 0; i < m; ++i) {
        for (int j = 0; j < n; ++j) {
            uint32_t acc = cin ? (uint32_t)cin[(size_t)i * ldc + j] : 0u;
            for (int kk = 0; kk < k; ++kk)
                acc += (uint32_t)((int32_t)a[(size_t)i * lda + kk] * (int32_t)B_AT(b, kk, j, ldb, b_dn));
            if (bias)
                acc += (uint32_t)bias[j];
            out[(size_t)i * ldc + j] = (int32_t)acc;
        }
    }
}

/* ============================== TMATMUL_MX (cpu/TMatmul.hpp:169-205) ======================== */

static inline unsigned mx_code_at(const uint8_t* p, size_t elem, int packed)
{
    if (!packed)
        return p[elem];
    return (p[elem >> 1] >> ((elem & 1u) ? 4 : 0)) & 0xFu; /* MXTypes.hpp:350-372 */
}

void pto_matmul_mx(float* out, const uint8_t* a, const uint8_t* b, const uint8_t* sa, const uint8_t* sb,
                   const float* cin, const float* bias, int m, int k, int n, int lda, int ldb, int ldc, int b_dn,
                   int a_type, int b_type, int sa_layout, int sb_layout)
{
    const int pa = (a_type == PTO_E2M1 || a_type == PTO_E1M2);
    const int pb = (b_type == PTO_E2M1 || b_type == PTO_E1M2);
    const int kg = k / 32;
    double lut_a[256], lut_b[256], lut_s[256];
    for (unsigned c = 0; c < 256; ++c) {
        lut_a[c] = pto_mx_decode(a_type, c);
        lut_b[c] = pto_mx_decode(b_type, c);
        lut_s[c] = pto_mx_decode(PTO_E8M0, c);
    }
    double* arow = (double*)malloc(sizeof(double) * (size_t)k);
    double* sarow = (double*)malloc(sizeof(double) * (size_t)(kg > 0 ? kg : 1));
    for (int i = 0; i < m; ++i) {
        for (int kk = 0; kk < k; ++kk)
            arow[kk] = lut_a[mx_code_at(a, (size_t)i * lda + kk, pa)];
        for (int g = 0; g < kg; ++g)
            sarow[g] = lut_s[sa[pto_mx_scale_offset(sa_layout, m, kg, i, g)]];
        for (int j = 0; j < n; ++j) {
            float acc = cin ? cin[(size_t)i * ldc + j] : 0.0f;
            for (int kk = 0; kk < k; ++kk) {
                const double sf = sarow[kk / 32] * lut_s[sb[pto_mx_scale_offset(sb_layout, kg, n, kk / 32, j)]];
                const double bv = lut_b[mx_code_at(b, b_dn ? (size_t)j * ldb + kk : (size_t)kk * ldb + j, pb)];
                /* float accumulator, double addend: one double add, then one rounding to float per k */
                acc = (float)((double)acc + arow[kk] * bv * sf);
            }
            if (bias)
                acc += bias[j];
            out[(size_t)i * ldc + j] = acc;
        }
    }
    free(arow);
    free(sarow);
}

/* ============================== TSTORE conversion (cpu/common.hpp, cpu/TStore.hpp) ========== */

static void put_converted(void* out, int dst_kind, size_t idx, float v)
{
    switch (dst_kind) {
        case PTO_ST_F32: ((float*)out)[idx] = v; break;
        case PTO_ST_F16: ((uint16_t*)out)[idx] = pto_f32_to_f16(v); break;
        case PTO_ST_BF16: ((uint16_t*)out)[idx] = pto_f32_to_bf16(v); break;
        case PTO_ST_I32: ((int32_t*)out)[idx] = (int32_t)v; break;
        case PTO_ST_I8: ((int8_t*)out)[idx] = (int8_t)v; break;
        case PTO_ST_I16: ((int16_t*)out)[idx] = (int16_t)v; break;
        default: ((uint8_t*)out)[idx] = (uint8_t)v; break;
    }
}

/* common.hpp:187-198: optional ReLU then static_cast */
void pto_store_f32(void* out, int dst_kind, const float* acc, int m, int n, int ldacc, int ldout, int relu)
{
    for (int i = 0; i < m; ++i)
        for (int j = 0; j < n; ++j) {
            float v = acc[(size_t)i * ldacc + j];
            if (relu)
                v = v > 0 ? v : 0;
            put_converted(out, dst_kind, (size_t)i * ldout + j, v);
        }
}

/* common.hpp:117-137 (extract_m1_from_quant) */
float pto_quant_word_scale(uint64_t word, int vector_mode)
{
    if (!vector_mode)
        return u2f((uint32_t)(word & 0xFFFFFFFFu));
    const uint32_t m1 = (uint32_t)((word >> 13) & 0x7FFFFu);
    const uint32_t s = (m1 >> 18) & 1u, e = (m1 >> 10) & 0xFFu, mant = m1 & 0x3FFu;
    if (e == 0 && mant == 0)
        return 0.0f;
    const float sv = s ? -1.0f : 1.0f;
    const float mv = 1.0f + ((float)mant / 1024.0f);
    const float ev = powf(2.0f, (float)e - 127.0f);
    return sv * mv * ev;
}

/* common.hpp:139-185 (quantize_element) for the 8-bit, f16, bf16 and (int32 source only) int16 targets; isrc is the
 * integer accumulator when src_is_int */
static float quant_core(float src, int32_t isrc, uint64_t word, int vector_mode, int dst_kind, int src_is_int,
                        int saturate_inf)
{
    const float f_scale = pto_quant_word_scale(word, vector_mode);
    const uint32_t offset = (uint32_t)((word >> 37) & 0x1FFu);
    const uint32_t sign = (uint32_t)((word >> 46) & 1u);
    float r = src * f_scale;
    if (dst_kind == PTO_ST_I8 || dst_kind == PTO_ST_U8) {
        const float rounded = rintf(r + (float)offset);
        const float lo = sign ? -128.0f : 0.0f, hi = sign ? 127.0f : 255.0f;
        r = rounded < lo ? lo : (rounded > hi ? hi : rounded); /* std::clamp; NaN passes through */
    } else if (dst_kind == PTO_ST_F16) {
        if (src_is_int) { /* DEQF16 / VDEQF16 */
            r = r < -65504.0f ? -65504.0f : (r > 65504.0f ? 65504.0f : r);
        } else if (isnan(r) && saturate_inf) {
            r = 0.0f;
        } else if (isfinite(r) || saturate_inf) {
            r = r < -65504.0f ? -65504.0f : (r > 65504.0f ? 65504.0f : r);
        }
    } else if (dst_kind == PTO_ST_BF16) {
        if (isnan(r) && saturate_inf)
            r = 0.0f;
        else if (isfinite(r) || saturate_inf)
            r = r < -3.402823466e38f ? -3.402823466e38f : (r > 3.402823466e38f ? 3.402823466e38f : r);
    } else if (dst_kind == PTO_ST_I16 && src_is_int) {
        /* SHIFTS322S16 / VSHIFTS322S16 (common.hpp:174-180): arithmetic shift by bits 32..35 of the word plus one; the
         * value is narrowed to int16 BEFORE the clamp, so it wraps and the clamp never acts */
        const int shift = (int)((word >> 32) & 0xFu) + 1;
        r = (float)(int16_t)(isrc >> shift);
    }
    return r;
}

void pto_store_quant_f32(void* out, int dst_kind, const float* acc, int m, int n, const uint64_t* words,
                         int per_column, int relu, int saturate_inf)
{
    for (int i = 0; i < m; ++i)
        for (int j = 0; j < n; ++j) {
            float r = quant_core(acc[(size_t)i * n + j], 0, words[per_column ? j : 0], per_column, dst_kind, 0,
                                 saturate_inf);
            if (relu)
                r = r > 0 ? r : 0;
            put_converted(out, dst_kind, (size_t)i * n + j, r);
        }
}

void pto_store_quant_i32(void* out, int dst_kind, const int32_t* acc, int m, int n, const uint64_t* words,
                         int per_column, int relu)
{
    for (int i = 0; i < m; ++i)
        for (int j = 0; j < n; ++j) {
            const int32_t a = acc[(size_t)i * n + j];
            float r = quant_core((float)a, a, words[per_column ? j : 0], per_column, dst_kind, 1, 0);
            if (relu)
                r = r > 0 ? r : 0;
            put_converted(out, dst_kind, (size_t)i * n + j, r);
        }
}

/* ============================== TQUANT (cpu/TQuant.hpp) ===================================== */

static inline float clampf(float v, float lo, float hi) { return v < lo ? lo : (v > hi ? hi : v); }

/* TQuant.hpp:86-96, 496-522.  The "scale" operand is multiplied (it is the inverse scale). */
/* GetParamValue (TQuant.hpp:78-84) as TQUANT INT8 calls it: column 0 of a [para_rows][para_ld] parameter tile, the
 * row clamped to para_rows - 1.  offset == NULL: symmetric (int8 codes in dst), else asymmetric (uint8 codes). */
void pto_tquant_int8_para(uint8_t* dst, const float* src, const float* scale, const float* offset, int rows, int cols,
                          int para_rows, int para_ld)
{
    for (int r = 0; r < rows; ++r) {
        const size_t pr = (size_t)(r < para_rows - 1 ? r : para_rows - 1) * para_ld;
        for (int c = 0; c < cols; ++c) {
            const float prod = src[(size_t)r * cols + c] * scale[pr];
            if (offset) {
                const float v = prod + offset[pr]; /* two roundings: multiply, then add */
                dst[(size_t)r * cols + c] = (uint8_t)clampf(nearbyintf(v), 0.0f, 255.0f);
            } else {
                dst[(size_t)r * cols + c] = (uint8_t)(int8_t)clampf(nearbyintf(prod), -128.0f, 127.0f);
            }
        }
    }
}

void pto_tquant_int8_sym(int8_t* dst, const float* src, const float* scale, int rows, int cols)
{
    pto_tquant_int8_para((uint8_t*)dst, src, scale, NULL, rows, cols, rows, 1);
}

void pto_tquant_int8_asym(uint8_t* dst, const float* src, const float* scale, const float* offset, int rows, int cols)
{
    pto_tquant_int8_para(dst, src, scale, offset, rows, cols, rows, 1);
}

static float e4m3_pos_value(unsigned code) /* TQuant.hpp:98-116 for codes 0..0x7E */
{
    const int e = (code >> 3) & 0xF, mant = code & 7;
    if (e == 0)
        return ldexpf((float)mant, -9);
    return ldexpf(1.0f + (float)mant / 8.0f, e - 7);
}

/* TQuant.hpp:118-153: nearest of the 254 finite codes to clamp(v, +-448); ties go to the even code, then to the
 * lower code (so both signs of a value that rounds to zero give code 0x00). */
unsigned pto_encode_e4m3fn(float v, int nv)
{
    if (isnan(v))
        return 0x7Fu;
    if (nv && fabsf(v) < 0.0009765625f)
        return signbit(v) ? 0x80u : 0x00u;
    const float clipped = clampf(v, -448.0f, 448.0f);
    const float a = fabsf(clipped);
    unsigned lo = 0, hi = 0x7Eu; /* positive codes are monotone in value */
    while (hi - lo > 1) {
        const unsigned mid = (lo + hi) / 2;
        if (e4m3_pos_value(mid) <= a)
            lo = mid;
        else
            hi = mid;
    }
    const float dlo = a - e4m3_pos_value(lo), dhi = e4m3_pos_value(hi) - a;
    unsigned code;
    if (dlo < dhi)
        code = lo;
    else if (dhi < dlo)
        code = hi;
    else
        code = (lo & 1u) ? hi : lo;
    if (code == 0)
        return 0;
    return (clipped < 0 ? 0x80u : 0u) | code;
}

/* TQuant.hpp:155-176 */
unsigned pto_encode_e2m1_magic(float value)
{
    if (isnan(value))
        return 0x7u;
    const uint32_t vb = f2u(value);
    const unsigned sign = (vb >> 28) & 0x8u;
    const float av = fabsf(value);
    if (isinf(av))
        return sign | 0x7u;
    const uint32_t ab = f2u(av);
    uint32_t be = (ab & 0x7F800000u) >> 23;
    be = be < 127u ? 127u : (be > 129u ? 129u : be);
    const uint32_t magic = (be + 22u) << 23;
    const uint32_t q = f2u(av + u2f(magic)) - magic;
    const uint32_t base = (be - 127u) << 1;
    const uint32_t mag = q + base < 7u ? q + base : 7u;
    return sign | mag;
}

/* TQuant.hpp:178-222, 308-334 */
unsigned pto_shared_exponent(int alg, float maxabs)
{
    const uint32_t bits = f2u(maxabs);
    if (alg == PTO_OCP_FP8 || alg == PTO_OCP_FP4) {
        const uint32_t e = (bits & 0x7F800000u) >> 23, mant = bits & 0x7FFFFFu;
        const uint32_t sub = alg == PTO_OCP_FP8 ? 8u : 2u;
        if (e == 0xFFu && mant != 0)
            return 0xFFu;
        if (e <= sub)
            return 0;
        return e - sub;
    }
    if (maxabs == 0.0f)
        return 0;
    const float descale = maxabs * (alg == PTO_NV_FP8 ? (1.0f / 448.0f) : (1.0f / 6.0f));
    const uint32_t db = f2u(descale);
    const uint32_t e = (db & 0x7F800000u) >> 23, mant = db & 0x7FFFFFu;
    if (e == 0xFFu)
        return mant == 0 ? 0xFEu : 0xFFu;
    const int round_up = mant > 0 && e != 0xFEu && !(e == 0 && mant <= 0x00400000u);
    return (e + (round_up ? 1u : 0u)) & 0xFFu;
}

/* cpu/Hifloat8.hpp:65-135 (decodeHiF8Mathematically): sign, a prefix code giving the number of exponent bits (4, 3, 2, 1
 * or 0, sign-magnitude with an implicit leading one) and mantissa bits (1, 2, 3, 3, 3); payloads 1..7 are 2^(p - 23);
 * 0x00 is zero, 0x80 NaN, 0x6F / 0xEF the infinities. */
double pto_hif8_to_f64(unsigned code)
{
    const double sign = (code & 0x80u) ? -1.0 : 1.0;
    const unsigned p = code & 0x7Fu;
    if ((p >> 3) == 0) {
        if ((p & 7u) == 0)
            return (code & 0x80u) ? (double)NAN : 0.0;
        return sign * ldexp(1.0, (int)(p & 7u) - 23);
    }
    int ebits, rest_bits;
    unsigned rest;
    if ((p >> 5) == 3) { ebits = 4; rest = p & 0x1Fu; rest_bits = 5; }
    else if ((p >> 5) == 2) { ebits = 3; rest = p & 0x1Fu; rest_bits = 5; }
    else if ((p >> 5) == 1) { ebits = 2; rest = p & 0x1Fu; rest_bits = 5; }
    else if ((p >> 4) == 1) { ebits = 1; rest = p & 0x0Fu; rest_bits = 4; }
    else { ebits = 0; rest = p & 0x07u; rest_bits = 3; }
    const int mbits = rest_bits - ebits;
    const unsigned raw_e = rest >> mbits, raw_m = rest & ((1u << mbits) - 1u);
    double e = 0.0;
    if (ebits > 0) {
        const unsigned sbit = raw_e & (1u << (ebits - 1));
        const double mag = (double)((1u << (ebits - 1)) | (raw_e - sbit));
        e = sbit ? -mag : mag;
    }
    if (ebits == 4 && e == 15.0 && raw_m == 1)
        return sign * (double)INFINITY;
    return sign * ldexp(1.0 + (double)raw_m / (double)(1u << mbits), (int)e);
}

/* TQuant.hpp:226-252, 336-347 */
float pto_group_scaling(int alg, float maxabs, unsigned e8m0)
{
    if (e8m0 == 0xFFu)
        return maxabs;
    if ((alg == PTO_NV_FP8 || alg == PTO_NV_FP4) && e8m0 == 0xFEu)
        return ldexpf(1.0f, -127);
    float s = u2f((254u - e8m0) << 23);
    if (s == 0.0f)
        s = ldexpf(1.0f, -127);
    return s;
}

/* A half source reaches the quantiser through the half -> float conversion (TQuant.hpp:291: `const float value =
 * src.data()[...]`), which quietens a signalling NaN; sources passed here as float already are widened by the caller,
 * so that step is restated for PTO_SRC_F16 (bf16 -> float is a shift and keeps the payload). */
static float mx_source_value(float v, int src_kind)
{
    if (src_kind == PTO_SRC_F16 && isnan(v))
        return u2f(f2u(v) | 0x00400000u);
    return v;
}

/* TQuant.hpp:280-306 */
static float mx_group_max(const float* src, int rows, int cols, int alg, int axis, int line, int group, int src_kind)
{
    (void)rows;
    float mx = 0.0f;
    uint16_t mx_bits = 0;
    for (int inner = 0; inner < 32; ++inner) {
        const int r = axis == 1 ? line : group * 32 + inner;
        const int c = axis == 1 ? group * 32 + inner : line;
        const float v = mx_source_value(src[(size_t)r * cols + c], src_kind);
        if (alg == PTO_OCP_FP4) {
            const uint16_t b = (uint16_t)((f2u(v) >> 16) & 0x7FFFu); /* truncated bf16 magnitude bits */
            if (b > mx_bits)
                mx_bits = b;
        } else {
            if (alg == PTO_NV_FP4 && isnan(v))
                return v;
            const float av = fabsf(v);
            mx = mx < av ? av : mx; /* std::max(maxAbs, fabs(v)): NaN is never taken */
        }
    }
    if (alg == PTO_OCP_FP4)
        mx = u2f((uint32_t)mx_bits << 16);
    return mx;
}

/* TQuant.hpp:349-372, 461-493 */
void pto_tquant_mx(uint8_t* dst, uint8_t* exp, float* mxo, float* scaling, const float* src, int rows, int cols,
                   int alg, int axis, int src_kind)
{
    const int fp4 = (alg == PTO_OCP_FP4 || alg == PTO_NV_FP4);
    const int groups = axis == 1 ? cols / 32 : rows / 32;
    const int lines = axis == 1 ? rows : cols;
    if (fp4)
        memset(dst, 0, (size_t)rows * cols / 2);
    for (int line = 0; line < lines; ++line) {
        for (int g = 0; g < groups; ++g) {
            const int flat = axis == 1 ? line * groups + g : g * lines + line;
            const float mx = mx_group_max(src, rows, cols, alg, axis, line, g, src_kind);
            const unsigned e = pto_shared_exponent(alg, mx);
            const float sc = pto_group_scaling(alg, mx, e);
            mxo[flat] = mx;
            exp[flat] = (uint8_t)e;
            scaling[flat] = sc;
            for (int inner = 0; inner < 32; ++inner) {
                const int r = axis == 1 ? line : g * 32 + inner;
                const int c = axis == 1 ? g * 32 + inner : line;
                const float v = mx_source_value(src[(size_t)r * cols + c], src_kind);
                const size_t idx = (size_t)r * cols + c;
                if (!fp4) {
                    dst[idx] = (uint8_t)pto_encode_e4m3fn(v * sc, alg == PTO_NV_FP8);
                } else {
                    unsigned code = 0x7u;
                    if (isinf(sc)) {
                        code = sc > 0 ? 0x7u : 0xFu;
                    } else if (!isnan(sc)) {
                        float scaled = v * sc;
                        if (src_kind == PTO_SRC_BF16) /* bf16 sources re-round the scaled value (TQuant.hpp:68-76) */
                            scaled = pto_bf16_to_f32(pto_f32_to_bf16(scaled));
                        code = pto_encode_e2m1_magic(scaled);
                    }
                    const int sh = (idx & 1u) ? 4 : 0;
                    dst[idx >> 1] = (uint8_t)((dst[idx >> 1] & ~(0xFu << sh)) | ((code & 0xFu) << sh));
                }
            }
        }
    }
}

/* TQuant.hpp:254-278 */
void pto_reorder_exp_zz(uint8_t* dst, const uint8_t* exp, int rows, int group_cols)
{
    size_t o = 0;
    for (int rb = 0; rb < rows / 16; ++rb)
        for (int gb = 0; gb < group_cols / 2; ++gb)
            for (int ir = 0; ir < 16; ++ir)
                for (int ig = 0; ig < 2; ++ig)
                    dst[o++] = exp[(size_t)(rb * 16 + ir) * group_cols + gb * 2 + ig];
}

/* cpu/TDeQuant.hpp:18-37 with a single scale/offset column */
/* TDeQuant.hpp:18-37.  scale / offset are [rows][para_ld] with para_cols valid columns; element (r, c) reads
 * parameter column min(c, para_cols - 1) (TDeQuant.hpp:24-30). */
void pto_tdequant_para(float* dst, const void* src, int src_kind, const float* scale, const float* offset, int rows,
                       int cols, int para_cols, int para_ld)
{
    for (int r = 0; r < rows; ++r)
        for (int c = 0; c < cols; ++c) {
            const size_t i = (size_t)r * cols + c;
            const size_t pi = (size_t)r * para_ld + (c < para_cols - 1 ? c : para_cols - 1);
            const float s = src_kind == 0 ? (float)((const int8_t*)src)[i]
                                          : (src_kind == 1 ? (float)((const int16_t*)src)[i]
                                                           : (float)((const int32_t*)src)[i]);
            const float d = s - offset[pi];
            dst[i] = d * scale[pi];
        }
}

void pto_tdequant(float* dst, const void* src, int src_kind, const float* scale, const float* offset, int rows,
                  int cols)
{
    pto_tdequant_para(dst, src, src_kind, scale, offset, rows, cols, 1, 1);
}

/* ============================== CPU-simulator-shaped tiled GEMM ============================ */
/*
 * Mirrors how the reference executes configs[0]-style kernels: per output tile, per K step,
 *   TLOAD  : element-by-element copy GM -> Mat tile through the NZ/ZN fractal offset map
 *            (cpu/TLoad.hpp:313-318), single-threaded;
 *   TMOV   : element-by-element copy Mat -> Left/Right (cpu/TMov.hpp:29-33);
 *   TMATMUL: rows fanned out over freshly created threads when m*n*k >= 16384
 *            (cpu/parallel.hpp:53-95), every operand read through the fractal offset map;
 *   TSTORE : per-element convert + strided write (cpu/TStore.hpp:64-78).
 */
#define SIM_BM 128
#define SIM_BN 128
#define SIM_BK 64

typedef struct {
    int dtype; /* 0 f16, 1 bf16, 2 i8, 3 e4m3 */
    const void* left;
    const void* right;
    void* acc;
    int m, k, n, first;
    pto_tile_layout la, lb, lc;
    int row_begin, row_end;
} sim_mm_job;

static float sim_widen(int dtype, const void* p, size_t i)
{
    switch (dtype) {
        case 0: return widen_f16(p, i);
        case 1: return widen_bf16(p, i);
        default: return widen_e4m3(p, i);
    }
}

static void* sim_mm_rows(void* arg)
{
    sim_mm_job* jb = (sim_mm_job*)arg;
    for (int i = jb->row_begin; i < jb->row_end; ++i) {
        for (int j = 0; j < jb->n; ++j) {
            const int64_t co = pto_tile_offset(&jb->lc, i, j);
            if (jb->dtype == 2) {
                uint32_t acc = jb->first ? 0u : (uint32_t)((int32_t*)jb->acc)[co];
                for (int kk = 0; kk < jb->k; ++kk)
                    acc += (uint32_t)((int32_t)((const int8_t*)jb->left)[pto_tile_offset(&jb->la, i, kk)] *
                                      (int32_t)((const int8_t*)jb->right)[pto_tile_offset(&jb->lb, kk, j)]);
                ((int32_t*)jb->acc)[co] = (int32_t)acc;
            } else {
                float acc = jb->first ? 0.0f : ((float*)jb->acc)[co];
                for (int kk = 0; kk < jb->k; ++kk)
                    acc = fmaf(sim_widen(jb->dtype, jb->left, (size_t)pto_tile_offset(&jb->la, i, kk)),
                               sim_widen(jb->dtype, jb->right, (size_t)pto_tile_offset(&jb->lb, kk, j)), acc);
                ((float*)jb->acc)[co] = acc;
            }
        }
    }
    return NULL;
}

static int sim_thread_count(int max_threads)
{
    long hw = sysconf(_SC_NPROCESSORS_ONLN);
    if (hw < 1)
        hw = 1;
    if (max_threads > 0 && hw > max_threads)
        hw = max_threads;
    return (int)hw;
}

static int sim_tmatmul(sim_mm_job* proto, int max_threads)
{
    const size_t work = (size_t)proto->m * proto->n * proto->k;
    int threads = sim_thread_count(max_threads);
    if (threads > proto->m)
        threads = proto->m;
    if (work < 16384u || proto->m < 2 || threads <= 1) {
        proto->row_begin = 0;
        proto->row_end = proto->m;
        sim_mm_rows(proto);
        return 1;
    }
    const int chunk = (proto->m + threads - 1) / threads;
    pthread_t tid[256];
    sim_mm_job jobs[256];
    if (threads > 256)
        threads = 256;
    int started = 0;
    for (int t = 0; t < threads; ++t) {
        const int b = t * chunk, e = b + chunk < proto->m ? b + chunk : proto->m;
        if (b >= e)
            break;
        jobs[t] = *proto;
        jobs[t].row_begin = b;
        jobs[t].row_end = e;
        pthread_create(&tid[t], NULL, sim_mm_rows, &jobs[t]);
        started++;
    }
    for (int t = 0; t < started; ++t)
        pthread_join(tid[t], NULL);
    return started;
}

int pto_sim_gemm_tiled(void* out, const void* a, const void* b, int m, int k, int n, int b_dn, int dtype,
                       int out_kind, int max_threads)
{
    const int eb = (dtype == 0 || dtype == 1) ? 2 : 1;
    const int ab = dtype == 2 ? 4 : 4; /* accumulator bytes */
    (void)ab;
    pto_tile_layout mat_a, mat_b, left, right, accl;
    pto_tile_layout_init(&mat_a, SIM_BM, SIM_BK, 0, 1, 512, eb, 0);                   /* Mat NZ */
    pto_tile_layout_init(&mat_b, SIM_BK, SIM_BN, b_dn ? 1 : 0, b_dn ? 2 : 1, 512, eb, 0); /* Mat ZN or NZ */
    pto_tile_layout_init(&left, SIM_BM, SIM_BK, 0, 1, 512, eb, 0);                    /* TileLeft  */
    pto_tile_layout_init(&right, SIM_BK, SIM_BN, 1, 2, 512, eb, 0);                   /* TileRight */
    pto_tile_layout_init(&accl, SIM_BM, SIM_BN, 0, 1, 1024, 4, 0);                    /* TileAcc   */
    uint8_t* ta = (uint8_t*)calloc((size_t)SIM_BM * SIM_BK, eb);
    uint8_t* tb = (uint8_t*)calloc((size_t)SIM_BK * SIM_BN, eb);
    uint8_t* tl = (uint8_t*)calloc((size_t)SIM_BM * SIM_BK, eb);
    uint8_t* tr = (uint8_t*)calloc((size_t)SIM_BK * SIM_BN, eb);
    uint8_t* tc = (uint8_t*)calloc((size_t)SIM_BM * SIM_BN, 4);
    int used = 1;
    for (int i0 = 0; i0 < m; i0 += SIM_BM) {
        const int mc = m - i0 < SIM_BM ? m - i0 : SIM_BM;
        for (int j0 = 0; j0 < n; j0 += SIM_BN) {
            const int nc = n - j0 < SIM_BN ? n - j0 : SIM_BN;
            for (int k0 = 0; k0 < k; k0 += SIM_BK) {
                const int kc = k - k0 < SIM_BK ? k - k0 : SIM_BK;
                /* TLOAD A (ND -> NZ) and B (ND -> NZ, or DN -> ZN) */
                for (int r = 0; r < mc; ++r)
                    for (int c = 0; c < kc; ++c)
                        memcpy(ta + (size_t)pto_tile_offset(&mat_a, r, c) * eb,
                               (const uint8_t*)a + ((size_t)(i0 + r) * k + k0 + c) * eb, eb);
                for (int r = 0; r < kc; ++r)
                    for (int c = 0; c < nc; ++c) {
                        const size_t g = b_dn ? (size_t)(j0 + c) * k + k0 + r : (size_t)(k0 + r) * n + j0 + c;
                        memcpy(tb + (size_t)pto_tile_offset(&mat_b, r, c) * eb, (const uint8_t*)b + g * eb, eb);
                    }
                /* TMOV Mat -> Left / Right */
                for (int c = 0; c < kc; ++c)
                    for (int r = 0; r < mc; ++r)
                        memcpy(tl + (size_t)pto_tile_offset(&left, r, c) * eb,
                               ta + (size_t)pto_tile_offset(&mat_a, r, c) * eb, eb);
                for (int c = 0; c < nc; ++c)
                    for (int r = 0; r < kc; ++r)
                        memcpy(tr + (size_t)pto_tile_offset(&right, r, c) * eb,
                               tb + (size_t)pto_tile_offset(&mat_b, r, c) * eb, eb);
                sim_mm_job jb;
                memset(&jb, 0, sizeof jb);
                jb.dtype = dtype;
                jb.left = tl;
                jb.right = tr;
                jb.acc = tc;
                jb.m = mc;
                jb.k = kc;
                jb.n = nc;
                jb.first = (k0 == 0);
                jb.la = left;
                jb.lb = right;
                jb.lc = accl;
                const int t = sim_tmatmul(&jb, max_threads);
                if (t > used)
                    used = t;
            }
            /* TSTORE */
            for (int r = 0; r < mc; ++r)
                for (int c = 0; c < nc; ++c) {
                    const size_t o = (size_t)(i0 + r) * n + j0 + c;
                    const int64_t co = pto_tile_offset(&accl, r, c);
                    if (dtype == 2)
                        ((int32_t*)out)[o] = ((int32_t*)tc)[co];
                    else
                        put_converted(out, out_kind, o, ((float*)tc)[co]);
                }
        }
    }
    free(ta);
    free(tb);
    free(tl);
    free(tr);
    free(tc);
    return used;
}

typedef struct {
    const uint8_t *a, *b, *sa, *sb;
    float* acc;
    int m, k, n, first, pa, pb, a_type, b_type;
    int lda, ldb, kg_total, ldsa_rows, ldsb_cols, g0, i0, j0, m_total, n_total;
    const double *lut_a, *lut_b, *lut_s;
    int row_begin, row_end;
} sim_mx_job;

static void* sim_mx_rows(void* arg)
{
    sim_mx_job* jb = (sim_mx_job*)arg;
    for (int i = jb->row_begin; i < jb->row_end; ++i)
        for (int j = 0; j < jb->n; ++j) {
            float acc = jb->first ? 0.0f : jb->acc[(size_t)i * SIM_BN + j];
            for (int kk = 0; kk < jb->k; ++kk) {
                const int g = jb->g0 + kk / 32;
                const double sf = jb->lut_s[jb->sa[(size_t)(jb->i0 + i) * jb->kg_total + g]] *
                                  jb->lut_s[jb->sb[(size_t)(jb->j0 + j) * jb->kg_total + g]];
                const double av = jb->lut_a[mx_code_at(jb->a, (size_t)(jb->i0 + i) * jb->lda + jb->g0 * 32 + kk, jb->pa)];
                const double bv = jb->lut_b[mx_code_at(jb->b, (size_t)(jb->j0 + j) * jb->ldb + jb->g0 * 32 + kk, jb->pb)];
                acc = (float)((double)acc + av * bv * sf);
            }
            jb->acc[(size_t)i * SIM_BN + j] = acc;
        }
    return NULL;
}

/* A [m, k] row-major codes, B column-major ([n][k]), scales MX_A_ND ([m][k/32]) and MX_B_DN ([n][k/32]) */
int pto_sim_gemm_mx_tiled(void* out, int out_kind, const uint8_t* a, const uint8_t* b, const uint8_t* sa,
                          const uint8_t* sb, int m, int k, int n, int a_type, int b_type, int max_threads)
{
    double lut_a[256], lut_b[256], lut_s[256];
    for (unsigned c = 0; c < 256; ++c) {
        lut_a[c] = pto_mx_decode(a_type, c);
        lut_b[c] = pto_mx_decode(b_type, c);
        lut_s[c] = pto_mx_decode(PTO_E8M0, c);
    }
    float* tc = (float*)calloc((size_t)SIM_BM * SIM_BN, sizeof(float));
    int used = 1;
    for (int i0 = 0; i0 < m; i0 += SIM_BM) {
        const int mc = m - i0 < SIM_BM ? m - i0 : SIM_BM;
        for (int j0 = 0; j0 < n; j0 += SIM_BN) {
            const int nc = n - j0 < SIM_BN ? n - j0 : SIM_BN;
            for (int k0 = 0; k0 < k; k0 += SIM_BK) {
                const int kc = k - k0 < SIM_BK ? k - k0 : SIM_BK;
                sim_mx_job p;
                memset(&p, 0, sizeof p);
                p.a = a; p.b = b; p.sa = sa; p.sb = sb; p.acc = tc;
                p.m = mc; p.k = kc; p.n = nc; p.first = (k0 == 0);
                p.pa = (a_type == PTO_E2M1 || a_type == PTO_E1M2);
                p.pb = (b_type == PTO_E2M1 || b_type == PTO_E1M2);
                p.lda = k; p.ldb = k; p.kg_total = k / 32; p.g0 = k0 / 32; p.i0 = i0; p.j0 = j0;
                p.lut_a = lut_a; p.lut_b = lut_b; p.lut_s = lut_s;
                int threads = sim_thread_count(max_threads);
                if (threads > mc)
                    threads = mc;
                if ((size_t)mc * nc * kc < 16384u || threads <= 1) {
                    p.row_begin = 0; p.row_end = mc;
                    sim_mx_rows(&p);
                } else {
                    pthread_t tid[256];
                    sim_mx_job jobs[256];
                    if (threads > 256)
                        threads = 256;
                    const int chunk = (mc + threads - 1) / threads;
                    int started = 0;
                    for (int t = 0; t < threads; ++t) {
                        const int bgn = t * chunk, end = bgn + chunk < mc ? bgn + chunk : mc;
                        if (bgn >= end)
                            break;
                        jobs[t] = p;
                        jobs[t].row_begin = bgn;
                        jobs[t].row_end = end;
                        pthread_create(&tid[t], NULL, sim_mx_rows, &jobs[t]);
                        started++;
                    }
                    for (int t = 0; t < started; ++t)
                        pthread_join(tid[t], NULL);
                    if (started > used)
                        used = started;
                }
            }
            for (int r = 0; r < mc; ++r)
                for (int c = 0; c < nc; ++c)
                    put_converted(out, out_kind, (size_t)(i0 + r) * n + j0 + c, tc[(size_t)r * SIM_BN + c]);
        }
    }
    free(tc);
    return used;
}
