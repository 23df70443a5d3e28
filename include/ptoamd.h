/*
 * ptoamd — C ABI of the MI355X (gfx950) backend for the PTO tile-matmul hot path.
 *
 * Everything below is `extern "C"`, plain pointers and sizes.  Device pointers are ordinary HIP device
 * addresses (from ptoamd_malloc, hipMalloc or a framework allocator); `stream` is a hipStream_t passed as
 * void* (NULL = the default stream).  Every function returns 0 on success and a negative PTOAMD_E_* code on
 * failure; ptoamd_last_error() gives the text.  Launches are asynchronous on `stream`.
 *
 * Two groups of entry points:
 *   1. the host runtime the reference's tests and demos reach through `aclrt*`
 *      (reference: include/pto/common/cpu_stub.hpp:73-120, 524-555);
 *   2. whole-kernel launchers, the counterpart of the reference's per-kernel
 *      `Launch...(uint8_t* out, uint8_t* src..., void* stream)` host functions
 *      (reference: tests/cpu/st/testcase/tmatmul/tmatmul_kernel.cpp:175-203,
 *       kernels/manual/a5/matmul_mxfp8_performance/mxmatmul_performance_kernel.cpp:360-380),
 *      each of which runs one TLOAD -> TMATMUL/TMATMUL_ACC -> TSTORE pipeline (or one TQUANT / TDEQUANT pass)
 *      over whole matrices in HBM.
 */
#ifndef PTOAMD_H
#define PTOAMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- error codes ---------------------------------------------------------------------------------------- */
#define PTOAMD_OK 0
#define PTOAMD_E_INVALID (-1)     /* bad argument (null pointer, non-positive size, unknown enum) */
#define PTOAMD_E_UNSUPPORTED (-2) /* combination the backend has no kernel for */
#define PTOAMD_E_ALIGNMENT (-3)   /* pointer / leading dimension not aligned as the kernel needs */
#define PTOAMD_E_HIP (-4)         /* a HIP runtime call failed */
#define PTOAMD_E_NODEVICE (-5)    /* no gfx950 device */

/* ---- enums ---------------------------------------------------------------------------------------------- */
/* element types of GEMM operands / results */
enum {
    PTOAMD_F32 = 0,
    PTOAMD_F16 = 1,
    PTOAMD_BF16 = 2,
    PTOAMD_I32 = 3,
    PTOAMD_I8 = 4,
    PTOAMD_U8 = 5,
    PTOAMD_E4M3 = 6, /* float8_e4m3_t (OCP E4M3FN)        reference: include/pto/cpu/MXTypes.hpp:344 */
    PTOAMD_E5M2 = 7, /* float8_e5m2_t                      reference: MXTypes.hpp:345 */
    PTOAMD_E2M1 = 8, /* float4_e2m1x2_t, two per byte, even element in the low nibble   MXTypes.hpp:341,350-372 */
    PTOAMD_E1M2 = 9, /* float4_e1m2x2_t                    MXTypes.hpp:342 */
    PTOAMD_I16 = 10,
    PTOAMD_HIF8 = 11 /* hifloat8_t, one byte per element     reference: include/pto/cpu/Hifloat8.hpp:138-215 */
};

/* memory layout of the B operand ([K, N] logical) — reference Layout::ND / Layout::DN (common/type.hpp:163-165) */
enum {
    PTOAMD_B_ND = 0, /* row-major [K][N], element (k, n) at b[k * ldb + n] */
    PTOAMD_B_DN = 1  /* column-major, i.e. [N][K] in memory, element (k, n) at b[n * ldb + k] */
};

/* GM layouts of E8M0 block scales — reference Layout::MX_* (common/type.hpp:167-172, cpu/tile_offsets.hpp:233-268) */
enum {
    PTOAMD_MX_A_ZZ = 0,
    PTOAMD_MX_A_ND = 1, /* [M][K/32] */
    PTOAMD_MX_A_DN = 2,
    PTOAMD_MX_B_NN = 3,
    PTOAMD_MX_B_ND = 4, /* [K/64][N][2] */
    PTOAMD_MX_B_DN = 5  /* [N][K/32] */
};

/* TQUANT algorithms — reference MxQuantAlg (common/type.hpp:213-219) */
enum { PTOAMD_OCP_MXFP8 = 0, PTOAMD_NV_MXFP8 = 1, PTOAMD_OCP_MXFP4 = 2, PTOAMD_NV_MXFP4 = 3 };

/* aclrtMemcpy kinds (cpu_stub.hpp) */
enum { PTOAMD_MEMCPY_H2H = 0, PTOAMD_MEMCPY_H2D = 1, PTOAMD_MEMCPY_D2H = 2, PTOAMD_MEMCPY_D2D = 3 };

/* =========================================================================================================
 * 1. Host runtime  (replaces the fake aclrt* runtime, include/pto/common/cpu_stub.hpp:73-120, 524-555)
 * ========================================================================================================= */
/* aclInit + aclrtSetDevice: selects the device and checks it is gfx950.  It also does, for that device, everything a
 * first launch would otherwise do lazily (launch attributes of every kernel, the device address of the static scratch
 * array): after ptoamd_init(device) the entry points below issue kernel launches and nothing else, which is what a
 * caller that captures them into a HIP graph needs.  Without it the first call per kernel and device sets up lazily. */
int ptoamd_init(int device);
int ptoamd_finalize(void);                      /* aclrtResetDevice + aclFinalize */
/* The dispatchers' environment switches (PTOAMD_TILE, PTOAMD_NO_TAIL_SPLIT, PTOAMD_MX_16X16, PTOAMD_FORCE_GENERIC,
 * PTOAMD_B_ND_TRANSPOSE, PTOAMD_GEMV_*) are read once per process; this reads them again.  No counterpart in the
 * reference (its simulator reads PTO_CPU_MAX_THREADS and the buffer sizes once too, cpu/NPUMemoryModel.hpp:128-135). */
int ptoamd_reload_options(void);
const char* ptoamd_last_error(void);            /* text of the calling thread's last failure */
int ptoamd_device_info(int* compute_units, int* clock_khz, size_t* hbm_bytes, char* arch, size_t arch_len);

int ptoamd_malloc(void** dev_ptr, size_t bytes);      /* aclrtMalloc */
int ptoamd_free(void* dev_ptr);                       /* aclrtFree */
int ptoamd_malloc_host(void** host_ptr, size_t bytes); /* aclrtMallocHost (pinned) */
int ptoamd_free_host(void* host_ptr);                 /* aclrtFreeHost */
int ptoamd_memcpy(void* dst, size_t dst_bytes, const void* src, size_t count, int kind); /* aclrtMemcpy (blocking) */
int ptoamd_memcpy_async(void* dst, size_t dst_bytes, const void* src, size_t count, int kind, void* stream);
int ptoamd_memset(void* dev_ptr, size_t dst_bytes, int value, size_t count);             /* aclrtMemset */

int ptoamd_stream_create(void** stream);        /* aclrtCreateStream (default priority) */
int ptoamd_stream_destroy(void* stream);        /* aclrtDestroyStream */
int ptoamd_stream_synchronize(void* stream);    /* aclrtSynchronizeStream */

/* HIP events on a stream, for timing a launch region */
int ptoamd_event_create(void** event);
int ptoamd_event_destroy(void* event);
int ptoamd_event_record(void* event, void* stream);
int ptoamd_event_synchronize(void* event);
int ptoamd_event_elapsed_ms(float* ms, void* start, void* stop);

/* =========================================================================================================
 * 2. Kernel launchers
 * ========================================================================================================= */

/*
 * C[M, N] = A[M, K] * B[K, N] (+ Cin) : the TLOAD -> TMATMUL / TMATMUL_ACC -> TSTORE pipeline.
 * reference: include/pto/cpu/TMatmul.hpp:77-113, 207-217 (arithmetic), cpu/TLoad.hpp:287-321, cpu/TStore.hpp:41-79.
 *   ab_type : PTOAMD_F16 | PTOAMD_BF16 | PTOAMD_F32 | PTOAMD_I8 | PTOAMD_E4M3 | PTOAMD_E5M2  (A and B alike)
 *   c_type  : PTOAMD_F32 | PTOAMD_F16 | PTOAMD_BF16 for float inputs (TSTORE's static_cast, round to nearest even);
 *             PTOAMD_I32 for int8 (raw accumulators, bit-exact)
 *   a       : row-major, leading dimension lda (elements)
 *   b       : b_layout PTOAMD_B_ND ([K][N], ldb >= N) or PTOAMD_B_DN ([N][K], ldb >= K)
 *   c_in    : optional accumulator input (TMATMUL_ACC), same type as the accumulator (f32 / i32), ld = ldc; may be NULL
 *   relu    : flags: PTOAMD_RELU (1) = TSTORE's ReluPreMode::NormalRelu; PTOAMD_SATURATE_INF (2), quantising drains only
 * No alignment is asked of a, b or the leading dimensions beyond that of an element: rows of 16 bytes or more run on the
 * MFMA tiles whatever their alignment: the LDS-DMA tiles when rows start on 4-byte boundaries (bf16 / f16 / int8: any K
 * longer than 128 bytes; fp8: K a whole number of 128-byte slabs), the register-staged tiles otherwise; a row-major B is
 * transposed on its way into LDS by the latter.  Rows of C need no alignment either.
 * PTOAMD_F32 and PTOAMD_HIF8 operands (hif8 x hif8 only, cpu/TMatmul.hpp:38) run on the order-exact kernel: one thread
 * per output, k ascending, fmaf -- the simulator's arithmetic bit for bit.  No entry point of this group allocates.
 */
#define PTOAMD_RELU 1
#define PTOAMD_SATURATE_INF 2 /* bit 48 of the reference's task cookie (cpu/common.hpp:146): see ptoamd_gemm_requant */
int ptoamd_gemm(void* c, int c_type, const void* a, const void* b, int ab_type, const void* c_in, int m, int n, int k,
                int lda, int ldb, int ldc, int b_layout, int relu, void* stream);

/*
 * The same pipeline with TMATMUL_BIAS: C = A * B (+ Cin) + bias, the bias row added to every row of C after the K loop
 * and before TSTORE's relu / conversion.
 * reference: include/pto/cpu/TMatmul.hpp:219-230 (TMATMUL_BIAS_IMPL), common/pto_instr.hpp (TMATMUL_BIAS).
 *   bias    : [N] of the accumulator type (f32 for float inputs, i32 for int8); NULL = ptoamd_gemm
 */
int ptoamd_gemm_bias(void* c, int c_type, const void* a, const void* b, int ab_type, const void* c_in, const void* bias,
                     int m, int n, int k, int lda, int ldb, int ldc, int b_layout, int relu, void* stream);

/*
 * ptoamd_gemm_bias with a caller-owned workspace for a row-major B (PTOAMD_B_ND): B is re-ordered into the workspace once
 * ([N][K] with rows padded to 16 bytes, ptoamd_gemm_workspace_bytes(n, k, ab_type, b_layout) bytes, 256-byte aligned) and the product then runs on the
 * fastest tiles, where ptoamd_gemm transposes B inside the loader of the register-staged tiles for every tile row of C --
 * the better choice for small M, the slower one for large M.  workspace == NULL is ptoamd_gemm_bias.  No counterpart in
 * the reference (its TLOAD re-orders an ND panel into L1 per tile, cpu/TLoad.hpp:287-321).
 */
size_t ptoamd_gemm_workspace_bytes(int n, int k, int ab_type, int b_layout);
int ptoamd_gemm_ws(void* c, int c_type, const void* a, const void* b, int ab_type, const void* c_in, const void* bias, int m, int n,
                   int k, int lda, int ldb, int ldc, int b_layout, int relu, void* workspace, size_t workspace_bytes, void* stream);

/* TMATMUL / _ACC / _BIAS on a mixed fp8 pair (cpu/TMatmul.hpp:31-49 admits all four E4M3 / E5M2 pairings of Left and Right):
 * as ptoamd_gemm_bias with separate operand types; bias may be NULL. */
int ptoamd_gemm_fp8(void* c, int c_type, const void* a, int a_type, const void* b, int b_type, const void* c_in, const void* bias,
                    int m, int n, int k, int lda, int ldb, int ldc, int b_layout, int relu, void* stream);

/*
 * The same pipeline drained through the fix-pipe quantiser: TSTORE of the accumulator tile with a scalar quantisation
 * word (TSTORE(dst, src, preQuantScalar)) or one word per column (TSTORE_FP with a Scaling tile):
 *   r = acc(i, j) * scale(word);  s8 / u8: clamp(rint(r + offset(word)), byte range chosen by the word's sign bit);
 *   f16: clamp to +-65504 (finite values only for float accumulators);  bf16: the product rounded to bfloat16;
 *   with PTOAMD_SATURATE_INF in `relu` (the fix-pipe's saturation control, cpu/common.hpp:146,157-171) the f16 and bf16
 *   targets of a float accumulator turn a NaN product into 0 and clamp an infinite one like a finite one
 *   (+-65504 / +-FLT_MAX);
 *   s16 (int32 accumulators only, the SHIFTS322S16 mode): (int16)(acc >> (bits 32..35 of the word + 1)), wrapping as
 *   the reference does;  then relu, then the store.
 * Cin and bias are added to the accumulator before the quantisation.
 * reference: include/pto/cpu/common.hpp:117-185 (extract_m1_from_quant, quantize_element), cpu/TStore.hpp:118-181,
 *            common/pto_instr.hpp:439-490; test shapes tests/cpu/st/testcase/tstore_acc2gm, tstore_quant.
 *   c_type      : PTOAMD_I8 | PTOAMD_U8 | PTOAMD_F16 | PTOAMD_BF16 | PTOAMD_I16 (the byte's signedness comes from bit 46 of the word, as in the
 *                 reference: it must agree with c_type)
 *   quant_words : device memory, 8-byte aligned; one uint64 (per_column == 0) or N of them (per_column != 0).  Scalar
 *                 words hold an fp32 scale in bits 0..31; per-column words a 19-bit (1, 8, 10) float in bits 13..31;
 *                 both the offset in bits 37..45 and the sign bit 46
 *   ab_type     : as ptoamd_gemm (float inputs accumulate in f32, int8 in i32: the DEQF16 / REQ8 forms)
 */
int ptoamd_gemm_requant(void* c, int c_type, const void* a, const void* b, int ab_type, const void* c_in, const void* bias,
                        const uint64_t* quant_words, int per_column, int m, int n, int k, int lda, int ldb, int ldc,
                        int b_layout, int relu, void* stream);

/*
 * The same pipeline drained with TSTORE<AtomicAdd>: C(i, j) += (A * B)(i, j), one atomic add per element, so that
 * several launches (K split over calls or streams) may accumulate into one C.  c_type: PTOAMD_F32 (float inputs) or
 * PTOAMD_I32 (int8 inputs).  The order of the additions between concurrent launches is not defined; float sums may
 * therefore differ in the last bits from run to run, integer sums do not.
 * reference: include/pto/cpu/TStore.hpp:64-78 (AtomicType::AtomicAdd), common/pto_instr.hpp (TSTORE<..., AtomicAdd>).
 */
int ptoamd_gemm_atomic_add(void* c, int c_type, const void* a, const void* b, int ab_type, int m, int n, int k, int lda, int ldb,
                           int ldc, int b_layout, void* stream);

/*
 * W8A8: int8 x int8 -> int32 accumulate, then the dequantising drain fused in registers:
 *   out(i, j) = bf16( (float(acc(i, j)) * scale_a[i]) * scale_b[j] )
 * i.e. TMATMUL (cpu/TMatmul.hpp:106) -> TDEQUANT with offset 0 (cpu/TDeQuant.hpp:31-34) -> per-column multiply
 * (cpu/TColExpandOp.hpp:57-63) -> TCVT f32->bf16 RINT.  acc_out (optional, may be NULL) receives the raw int32
 * accumulators so parity can be checked bit for bit.
 */
int ptoamd_gemm_w8a8(void* out_bf16, int32_t* acc_out, const int8_t* a, const int8_t* b, const float* scale_a,
                     const float* scale_b, int m, int n, int k, int lda, int ldb, int ldc, int b_layout, void* stream);

/*
 * Block-scaled matmul, TMATMUL_MX (cpu/TMatmul.hpp:169-205, 254-292):
 *   C(i, j) = sum_k A(i, k) * B(k, j) * 2^(sa(i, k/32) - 127) * 2^(sb(k/32, j) - 127)   (+ Cin)
 *   a_type / b_type : both fp8 (PTOAMD_E4M3 | PTOAMD_E5M2) or both fp4 (PTOAMD_E2M1 | PTOAMD_E1M2).  A product with an
 *                     E1M2 operand runs on the E4M3 x E4M3 scaled MFMA, both operands' nibbles widened exactly to E4M3
 *                     bytes by the loader (b in PTOAMD_B_DN, K a multiple of 128, 8-byte aligned rows); other E1M2
 *                     shapes take the order-exact generic kernel.
 *   Numerics of the MFMA kernels: the scaled MFMA aligns the 64 products of a k-step to the largest exponent among
 *   them and keeps about 13 bits below it before adding, where the reference adds one product at a time in fp32
 *   (double add, one rounding per k).  Element-wise |C - C_ref| <= 2^-11 * sum_k |a||b| on fp8 data spanning all codes
 *   (<= 1e-3 of max|C|), within the fp32-sum bound on data of one magnitude; the generic kernel
 *   (PTOAMD_FORCE_GENERIC=1) reproduces the reference bit for bit.
 *   a  : [M][K] codes row-major (fp4: K/2 bytes per row);  b : PTOAMD_B_DN ([N][K]) or PTOAMD_B_ND ([K][N])
 *   sa : E8M0 bytes in sa_layout (PTOAMD_MX_A_*), logical [M][K/32];  sb : sb_layout (PTOAMD_MX_B_*), [K/32][N]
 *   c_type : PTOAMD_F32 | PTOAMD_BF16 | PTOAMD_F16
 * lda / ldb are in elements.  K must be a multiple of 64 (CheckMadMxValid, TMatmul.hpp:121-142).
 */
int ptoamd_gemm_mx(void* c, int c_type, const void* a, const void* b, int a_type, int b_type, const uint8_t* sa,
                   const uint8_t* sb, int sa_layout, int sb_layout, const float* c_in, int m, int n, int k, int lda,
                   int ldb, int ldc, int b_layout, void* stream);

/*
 * TMATMUL_MX with a bias row: C = A * B (+ Cin) + bias, bias [N] f32 added to every row after the K loop.
 * reference: include/pto/cpu/TMatmul.hpp:273-292 (TMATMUL_MX_IMPL with a bias tile), common/pto_instr.hpp (TMATMUL_MX).
 */
int ptoamd_gemm_mx_bias(void* c, int c_type, const void* a, const void* b, int a_type, int b_type, const uint8_t* sa,
                        const uint8_t* sb, int sa_layout, int sb_layout, const float* c_in, const float* bias, int m, int n,
                        int k, int lda, int ldb, int ldc, int b_layout, void* stream);

/*
 * ptoamd_gemm_mx with a caller-provided device workspace for what the kernels need beyond inputs and outputs: the MFMA
 * kernels stream scales as [M][K/32] (MX_A_ND) and [N][K/32] (MX_B_DN), and scales that arrive in another GM layout
 * (the TLOAD + TMOV of a scale tile, cpu/TLoad.hpp:287-321 with the MX_* maps of cpu/tile_offsets.hpp:233-268) are
 * re-laid into the workspace first, and the fastest (direct-to-LDS) kernels run.  ptoamd_gemm_mx reads such scales where
 * they lie instead, with the register-staged kernels; neither form allocates.  workspace: 256-byte aligned, at least ptoamd_gemm_mx_workspace_bytes(...) bytes (0 for the
 * two natural layouts: workspace may then be NULL).  A row-major B (PTOAMD_B_ND) of fp8 codes is transposed inside the
 * register-staged kernels' loader, every element once per row tile; a workspace of
 * ptoamd_gemm_mx_workspace_bytes_b_nd(...) bytes (the scales' part, rounded up to 256 bytes, plus a [N][K] copy of B with
 * rows padded to 16 bytes) lets the call transpose B once and run the direct-to-LDS kernels instead (M above 128; a
 * smaller workspace keeps the in-loader form).  Packed fp4 codes are never transposed.
 */
int ptoamd_gemm_mx_ws(void* c, int c_type, const void* a, const void* b, int a_type, int b_type, const uint8_t* sa,
                      const uint8_t* sb, int sa_layout, int sb_layout, const float* c_in, int m, int n, int k, int lda,
                      int ldb, int ldc, int b_layout, void* workspace, size_t workspace_bytes, void* stream);
size_t ptoamd_gemm_mx_workspace_bytes(int m, int n, int k, int sa_layout, int sb_layout);
size_t ptoamd_gemm_mx_workspace_bytes_b_nd(int m, int n, int k, int sa_layout, int sb_layout, int b_type);

/*
 * ptoamd_gemm_mx_ws with the workspace inside the library: a static device array of PTOAMD_STATIC_SCRATCH_BYTES, one
 * copy per GPU, held until the process ends.  It has no counterpart in the reference; it is for callers that cannot
 * allocate device memory around a call: code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc.  The call allocates nothing (no hipMalloc / hipFree, no stream-ordered allocation).  Scale sets whose
 * re-laid form (ptoamd_gemm_mx_workspace_bytes) exceeds the array are rejected with PTOAMD_E_UNSUPPORTED.  All calls on
 * one GPU share the one array: calls that overlap in time on the same GPU (two streams, two threads) race on it --
 * serialise them, or give each stream its own workspace through ptoamd_gemm_mx_ws.
 */
#define PTOAMD_STATIC_SCRATCH_BYTES (4 * 1024 * 1024)
int ptoamd_gemm_mx_static(void* c, int c_type, const void* a, const void* b, int a_type, int b_type, const uint8_t* sa,
                          const uint8_t* sb, int sa_layout, int sb_layout, const float* c_in, int m, int n, int k, int lda,
                          int ldb, int ldc, int b_layout, void* stream);

/*
 * Decode-shaped weight-only MXFP4 GEMV/GEMM (m <= 16):
 *   out(i, j) = sum_k bf16 A(i, k) * ( e2m1 W(j, k) * 2^(sw(j, k/32) - 127) )      fp32 accumulate
 * The dequantised weight is exact in bf16, so this is TMATMUL on bf16 operands (cpu/TMatmul.hpp:77-113) fed by the
 * MX decode of cpu/MXTypes.hpp:232-274, with the dequantisation done in registers.
 *   a : bf16 [m][k] (lda elements);  w : packed e2m1 [n][k/2] bytes (ldw elements);  sw : E8M0 [n][k/32]
 *   c_type : PTOAMD_F32 | PTOAMD_BF16
 */
int ptoamd_gemv_mxfp4(void* out, int c_type, const void* a_bf16, const uint8_t* w, const uint8_t* sw, int m, int n,
                      int k, int lda, int ldw, int ldc, void* stream);

/*
 * The same product with the weights stored once in the order the kernel consumes them (k a multiple of 2048): per
 * 16 rows x 2048 k one 16 KiB block of codes -- the 16 row pieces, their 16-byte chunks at the LDS positions the kernel
 * reads them from -- and, in a second region behind all code blocks, one 1 KiB block of the 16 x 64 scale bytes, so that
 * a stage is two contiguous runs of memory.  Same arithmetic in the same order as ptoamd_gemv_mxfp4 on the loader-wave
 * kernel (bit-identical outputs), 4 - 5 % faster on 16 x 28672 x 8192.  It is to this kernel what the NZ / fractal GM layouts are to the reference's cube unit
 * (include/pto/cpu/tile_offsets.hpp: data laid out in the consumer's order, once, ahead of time); the packed buffer is
 * only meaningful to ptoamd_gemv_mxfp4_packed.
 *   ptoamd_gemv_mxfp4_packed_bytes : size of the packed buffer (0 when k is not a multiple of 2048)
 *   ptoamd_gemv_mxfp4_pack         : w [n][ldw / 2] bytes (16-byte aligned rows), sw [n][k / 32] -> packed
 */
size_t ptoamd_gemv_mxfp4_packed_bytes(int n, int k);
int ptoamd_gemv_mxfp4_pack(void* packed, const uint8_t* w, const uint8_t* sw, int n, int k, int ldw, void* stream);
int ptoamd_gemv_mxfp4_packed(void* out, int c_type, const void* a_bf16, const void* packed, int m, int n, int k, int lda,
                             int ldc, void* stream);

/* TQUANT<INT8_SYM / INT8_ASYM> (cpu/TQuant.hpp:496-522): dst = clamp(nearbyint(src * scale[row] (+ offset[row]))).
 * offset == NULL selects the symmetric form (int8 output); otherwise the output is uint8.  src is [rows][cols] f32. */
int ptoamd_tquant_int8(void* dst, const float* src, const float* scale, const float* offset, int rows, int cols,
                       void* stream);
/* The same with the parameter tiles described as the reference's GetParamValue reads them (cpu/TQuant.hpp:78-84):
 * scale / offset are [para_rows][para_ld] f32, column 0 is used and the row index is clamped to para_rows - 1 (a
 * parameter tile with fewer valid rows than src repeats its last row). */
int ptoamd_tquant_int8_para(void* dst, const float* src, const float* scale, const float* offset, int rows, int cols,
                            int para_rows, int para_ld, void* stream);

/* TQUANT<MXFP8 | MXFP4_E2M1> (cpu/TQuant.hpp:461-493, 524-547).  src [rows][cols] of src_type (F32 | F16 | BF16);
 * axis 1 groups 32 elements along a row (exp / max / scaling are [rows][cols/32]), axis 0 along a column
 * ([rows/32][cols]).  dst: one byte per element (fp8) or packed nibbles (fp4).  max / scaling may be NULL. */
int ptoamd_tquant_mx(uint8_t* dst, uint8_t* exp, float* max, float* scaling, const void* src, int src_type, int rows,
                     int cols, int alg, int axis, void* stream);

/* TDEQUANT (cpu/TDeQuant.hpp:18-37): dst(r, c) = (float(src(r, c)) - offset[r]) * scale[r];
 * src_type PTOAMD_I8 | PTOAMD_I16 | PTOAMD_I32. */
int ptoamd_tdequant(float* dst, const void* src, int src_type, const float* scale, const float* offset, int rows,
                    int cols, void* stream);
/* The same with parameter tiles wider than one column (cpu/TDeQuant.hpp:24-30): scale / offset are [rows][para_ld] f32
 * with para_cols valid columns, and element (r, c) uses parameter column min(c, para_cols - 1). */
int ptoamd_tdequant_para(float* dst, const void* src, int src_type, const float* scale, const float* offset, int rows,
                         int cols, int para_cols, int para_ld, void* stream);

/* Copies an E8M0 scale matrix between GM layouts (the TLOAD + TMOV of a scale tile, cpu/tile_offsets.hpp:233-268):
 * rows x cols is the logical extent ([M][K/32] for the A side, [K/32][N] for the B side). */
int ptoamd_mx_scale_relayout(uint8_t* dst, int dst_layout, const uint8_t* src, int src_layout, int rows, int cols,
                             void* stream);

/* Names the kernel the last ptoamd_gemm* / ptoamd_gemv* call on this thread dispatched to ("tile256x256_bf16", ...,
 * "generic"): lets tests assert that the MFMA path, not the order-exact generic kernel, produced a result. */
const char* ptoamd_last_kernel(void);

#ifdef __cplusplus
}
#endif
#endif /* PTOAMD_H */
