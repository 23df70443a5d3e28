/*
 * TEST INFRASTRUCTURE ONLY.
 *
 * CPU restatement (plain C) of the PTO tile-matmul hot path as the reference CPU simulator
 * computes it.  It is the parity checker for the HIP backend and the "port" CPU baseline of
 * bench.py; the product library never links, loads or calls anything declared here.
 * Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may use it.
 *
 * All citations are relative to the reference tree (include/pto/...).
 * Pinning status of every function is listed at the top of pto_oracle.c.
 */
#ifndef PTO_ORACLE_H
#define PTO_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- element types ----------------------------------------------------------------------- */
enum pto_mx_type { PTO_E4M3 = 0, PTO_E5M2 = 1, PTO_E2M1 = 2, PTO_E1M2 = 3, PTO_E8M0 = 4 };
enum pto_round_mode {
    PTO_CAST_NONE = 0, PTO_CAST_RINT = 1, PTO_CAST_ROUND = 2, PTO_CAST_FLOOR = 3,
    PTO_CAST_CEIL = 4, PTO_CAST_TRUNC = 5, PTO_CAST_ODD = 6
};

float pto_f16_to_f32(uint16_t h);
uint16_t pto_f32_to_f16(float f);  /* round to nearest even, as static_cast<_Float16> */
float pto_bf16_to_f32(uint16_t h);
uint16_t pto_f32_to_bf16(float f); /* round to nearest even */

double pto_mx_decode(int type, unsigned raw);
unsigned pto_mx_encode_trunc(int type, double v);
unsigned pto_fp8_encode_round(int type, double v, int round_mode, int sat_on);
unsigned pto_fp4_encode_round(int type, double v, int round_mode);

/* ---- tile / global addressing ------------------------------------------------------------ */
typedef struct {
    int rows, cols;       /* static tile shape */
    int row_major;        /* BLayout::RowMajor ? 1 : 0 */
    int sfractal;         /* 0 NoneBox, 1 RowMajor, 2 ColMajor */
    int inner_rows, inner_cols;
} pto_tile_layout;

/* Fills inner_rows/inner_cols the way Tile<> derives them. elem_bytes = sizeof(DType), packed2 = fp4 twin type */
void pto_tile_layout_init(pto_tile_layout* t, int rows, int cols, int row_major, int sfractal, int sfractal_size,
                          int elem_bytes, int packed2);
int64_t pto_tile_offset(const pto_tile_layout* t, int r, int c);

enum pto_layout {
    PTO_ND = 0, PTO_DN = 1, PTO_NZ = 2, PTO_MX_A_ZZ = 3, PTO_MX_A_ND = 4, PTO_MX_A_DN = 5,
    PTO_MX_B_NN = 6, PTO_MX_B_ND = 7, PTO_MX_B_DN = 8
};
int64_t pto_global_offset(int layout, int64_t r, int64_t c, const int64_t shape[5], const int64_t stride[5]);
/* shape/stride of a whole [rows, cols] logical matrix in the given layout (TileShape2D / BaseShape2D) */
int pto_layout_2d(int layout, int64_t rows, int64_t cols, int c0, int64_t shape[5], int64_t stride[5]);
int64_t pto_mx_scale_offset(int layout, int rows, int cols, int r, int c);

/* ---- TMATMUL / TMATMUL_ACC / TMATMUL_BIAS ------------------------------------------------- */
/* A is [m, k] row-major (lda); B is [k, n] row-major (ldb) or, with b_dn, column-major (element (kk, j) at
 * b[j * ldb + kk]); cin (may be NULL) and out are [m, n] row-major (ldc); bias (may be NULL) is [n]. */
void pto_matmul_f16(float* out, const uint16_t* a, const uint16_t* b, const float* cin, const float* bias, int m,
                    int k, int n, int lda, int ldb, int ldc, int b_dn);
void pto_matmul_bf16(float* out, const uint16_t* a, const uint16_t* b, const float* cin, const float* bias, int m,
                     int k, int n, int lda, int ldb, int ldc, int b_dn);
void pto_matmul_f32(float* out, const float* a, const float* b, const float* cin, const float* bias, int m, int k,
                    int n, int lda, int ldb, int ldc, int b_dn);
void pto_matmul_i8(int32_t* out, const int8_t* a, const int8_t* b, const int32_t* cin, const int32_t* bias, int m,
                   int k, int n, int lda, int ldb, int ldc, int b_dn);
void pto_matmul_fp8(float* out, const uint8_t* a, const uint8_t* b, const float* cin, const float* bias, int m, int k,
                    int n, int lda, int ldb, int ldc, int b_dn, int a_type, int b_type);

/* ---- TMATMUL_MX --------------------------------------------------------------------------- */
/* a/b hold element codes: one byte per element for fp8, two elements per byte for fp4 (even element in the low
 * nibble, leading dimensions counted in elements).  sa(i, g) is read at sa[pto_mx_scale_offset(sa_layout, m, k/32,
 * i, g)], sb(g, j) at sb[pto_mx_scale_offset(sb_layout, k/32, n, g, j)]. */
void pto_matmul_mx(float* out, const uint8_t* a, const uint8_t* b, const uint8_t* sa, const uint8_t* sb,
                   const float* cin, const float* bias, int m, int k, int n, int lda, int ldb, int ldc, int b_dn,
                   int a_type, int b_type, int sa_layout, int sb_layout);

/* ---- TSTORE value conversion (Acc -> GM), incl. fix-pipe requantisation ------------------- */
enum pto_store_dst { PTO_ST_F32 = 0, PTO_ST_F16 = 1, PTO_ST_BF16 = 2, PTO_ST_I32 = 3, PTO_ST_I8 = 4, PTO_ST_U8 = 5, PTO_ST_I16 = 6 };
/* no-quant path: optional relu then static_cast */
void pto_store_f32(void* out, int dst_kind, const float* acc, int m, int n, int ldacc, int ldout, int relu);
/* quant path: words[j] per column when per_column, else words[0] */
float pto_quant_word_scale(uint64_t word, int vector_mode);
void pto_store_quant_f32(void* out, int dst_kind, const float* acc, int m, int n, const uint64_t* words,
                         int per_column, int relu, int saturate_inf);
void pto_store_quant_i32(void* out, int dst_kind, const int32_t* acc, int m, int n, const uint64_t* words,
                         int per_column, int relu);

/* ---- TQUANT / TDEQUANT -------------------------------------------------------------------- */
void pto_tquant_int8_sym(int8_t* dst, const float* src, const float* scale, int rows, int cols);
void pto_tquant_int8_asym(uint8_t* dst, const float* src, const float* scale, const float* offset, int rows, int cols);
void pto_tquant_int8_para(uint8_t* dst, const float* src, const float* scale, const float* offset, int rows, int cols,
                          int para_rows, int para_ld);

enum pto_mx_alg { PTO_OCP_FP8 = 0, PTO_NV_FP8 = 1, PTO_OCP_FP4 = 2, PTO_NV_FP4 = 3 };
enum pto_src_kind { PTO_SRC_F32 = 0, PTO_SRC_F16 = 1, PTO_SRC_BF16 = 2 };
unsigned pto_encode_e4m3fn(float v, int nv);
unsigned pto_encode_e2m1_magic(float v);
unsigned pto_shared_exponent(int alg, float maxabs);
float pto_group_scaling(int alg, float maxabs, unsigned e8m0);
double pto_hif8_to_f64(unsigned code); /* cpu/Hifloat8.hpp:65-135 */
/* src is [rows, cols] row-major, already widened to float from src_kind (which only matters for the fp4 bf16
 * re-rounding).  axis 1: groups of 32 along a row; exp/max/scaling are [rows][cols/32].  axis 0: groups of 32
 * along a column; exp/max/scaling are [rows/32][cols].  dst: bytes (fp8) or packed nibbles, row-major (fp4). */
void pto_tquant_mx(uint8_t* dst, uint8_t* exp, float* mx, float* scaling, const float* src, int rows, int cols,
                   int alg, int axis, int src_kind);
void pto_reorder_exp_zz(uint8_t* dst, const uint8_t* exp, int rows, int group_cols);

/* dst(r, c) = (float(src(r, c)) - offset[r]) * scale[r];  src_kind: 0 int8, 1 int16, 2 int32 */
void pto_tdequant(float* dst, const void* src, int src_kind, const float* scale, const float* offset, int rows,
                  int cols);
void pto_tdequant_para(float* dst, const void* src, int src_kind, const float* scale, const float* offset, int rows,
                       int cols, int para_cols, int para_ld);

/* ---- CPU-simulator-shaped tiled GEMM (the "port" CPU baseline) ---------------------------- */
/* Walks 128x128 output tiles with a K step of 64 the way the reference demo does: TLOAD copies into a private
 * tile buffer with per-element fractal addressing, TMATMUL(_ACC) fans rows out over freshly created threads
 * when m*n*k >= 16384, TSTORE converts per element.  dtype: 0 f16, 1 bf16, 2 i8 (out i32), 3 fp8 e4m3.
 * Returns the number of threads each TMATMUL used. */
int pto_sim_gemm_tiled(void* out, const void* a, const void* b, int m, int k, int n, int b_dn, int dtype,
                       int out_kind, int max_threads);
int pto_sim_gemm_mx_tiled(void* out, int out_kind, const uint8_t* a, const uint8_t* b, const uint8_t* sa,
                          const uint8_t* sb, int m, int k, int n, int a_type, int b_type, int max_threads);

#ifdef __cplusplus
}
#endif
#endif
