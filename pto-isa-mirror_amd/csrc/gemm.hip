// C-ABI launchers of the matmul family (ptoamd_gemm, ptoamd_gemm_w8a8, ptoamd_gemm_mx) and the kernels around the
// tiled MFMA kernel: an order-exact generic kernel for shapes/layouts the tiled kernel does not take, the B-operand
// transpose (Layout::ND -> the K-contiguous form the MFMA path reads) and the MX scale re-layout.
#include "common_host.hpp"
#include "gemm_tile.hpp"

#include <stdlib.h>
#include <string.h>

#include <algorithm>
#include <mutex>

namespace ptoamd {

hipError_t launch_gemm_tile_bf16(int, const TileGemmParams&, hipStream_t);
hipError_t launch_gemm_tile_f16(int, const TileGemmParams&, hipStream_t);
hipError_t launch_gemm_tile_i8(int, const TileGemmParams&, hipStream_t);
hipError_t launch_gemm_tile_fp8_e4e4(int, const TileGemmParams&, hipStream_t);
hipError_t launch_gemm_tile_fp8_e5e5(int, const TileGemmParams&, hipStream_t);
hipError_t launch_gemm_tile_fp8_e4e5(int, const TileGemmParams&, hipStream_t);
hipError_t launch_gemm_tile_fp8_e5e4(int, const TileGemmParams&, hipStream_t);
hipError_t launch_gemm_tile_fp4(int, const TileGemmParams&, hipStream_t);

hipError_t launch_gemm_tile(int tile, int op, const TileGemmParams& p, hipStream_t stream)
{
    switch (op) {
        case TOP_BF16: return launch_gemm_tile_bf16(tile, p, stream);
        case TOP_F16: return launch_gemm_tile_f16(tile, p, stream);
        case TOP_I8: return launch_gemm_tile_i8(tile, p, stream);
        case TOP_FP8_E4E4: return launch_gemm_tile_fp8_e4e4(tile, p, stream);
        case TOP_FP8_E5E5: return launch_gemm_tile_fp8_e5e5(tile, p, stream);
        case TOP_FP8_E4E5: return launch_gemm_tile_fp8_e4e5(tile, p, stream);
        case TOP_FP8_E5E4: return launch_gemm_tile_fp8_e5e4(tile, p, stream);
        case TOP_FP4: return launch_gemm_tile_fp4(tile, p, stream);
        default: return hipErrorInvalidValue;
    }
}

void tile_shape(int tile, int* bm, int* bn)
{
    static const int bms[8] = {256, 128, 64, 256, 256, 128, 256, 256};
    static const int bns[8] = {256, 128, 64, 256, 256, 128, 128, 128};
    const int t = tile < 0 || tile > 7 ? 2 : tile;
    *bm = bms[t];
    *bn = bns[t];
}

// ---- MX scale GM layouts (reference: cpu/tile_offsets.hpp:233-268 with the strides of pto_tile.hpp:849-1102) ----
__host__ __device__ inline long mx_scale_offset(int layout, int rows, int cols, int r, int c)
{
    switch (layout) {
        case PTOAMD_MX_A_ZZ: return (long)(r / 16) * cols * 16 + (c / 2) * 32 + (r % 16) * 2 + c % 2;
        case PTOAMD_MX_A_ND: return (long)r * cols + c;
        case PTOAMD_MX_A_DN: return (long)(c / 2) * rows * 2 + r * 2 + c % 2;
        case PTOAMD_MX_B_NN: return (long)(c / 16) * rows * 16 + (r / 2) * 32 + (c % 16) * 2 + r % 2;
        case PTOAMD_MX_B_ND: return (long)(r / 2) * cols * 2 + c * 2 + r % 2;
        default: return (long)c * rows + r;  // PTOAMD_MX_B_DN
    }
}

__global__ void mx_scale_relayout_kernel(uint8_t* dst, int dst_layout, const uint8_t* src, int src_layout, int rows,
                                         int cols)
{
    const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (long)rows * cols)
        return;
    const int r = (int)(idx / cols), c = (int)(idx % cols);
    dst[mx_scale_offset(dst_layout, rows, cols, r, c)] = src[mx_scale_offset(src_layout, rows, cols, r, c)];
}

// ---- B operand: [K][N] row-major -> [N][K] so both operands are read K-contiguous -----------------------------
template <typename T>
__global__ void transpose_kernel(T* dst, const T* src, int rows, int cols, long ld_src, long ld_dst)
{
    __shared__ T tile[32][33];
    const int c0 = blockIdx.x * 32, r0 = blockIdx.y * 32;
    for (int i = threadIdx.y; i < 32; i += blockDim.y) {
        const int r = r0 + i, c = c0 + threadIdx.x;
        if (r < rows && c < cols)
            tile[i][threadIdx.x] = src[(long)r * ld_src + c];
    }
    __syncthreads();
    for (int i = threadIdx.y; i < 32; i += blockDim.y) {
        const int c = c0 + i, r = r0 + threadIdx.x;
        if (r < rows && c < cols)
            dst[(long)c * ld_dst + r] = tile[threadIdx.x][i];
    }
}

// ---- order-exact generic kernel -------------------------------------------------------------------------------
// One thread per output element, k ascending, one rounding per step exactly as the reference CPU simulator does
// (cpu/TMatmul.hpp:96-110 and :191-200).  Slow; it serves the shapes, layouts and element types the MFMA kernel
// does not take, and matches the simulator bit for bit on every type.
struct GenericParams {
    const void* a;
    const void* b;
    void* c;
    const void* c_in;
    const void* bias;  // [n] of the accumulator type, added after the K loop (TMATMUL_BIAS)
    int32_t* acc_out;
    const uint8_t* sa;
    const uint8_t* sb;
    const float* row_scale;
    const float* col_scale;
    int m, n, k;
    long lda, sbk, sbn;  // element strides: A row pitch; B(k, j) = b[k * sbk + j * sbn]
    int ldc;
    int a_type, b_type, out_kind, relu;  // relu: bit 0 relu, bit 1 saturate-inf (as TileGemmParams)
    int sa_layout, sb_layout, mx;
    const uint64_t* qwords;  // OUT_Q8 / OUT_QF16: fix-pipe quantisation words
    int q_per_column;
    int atomic_add;          // OUT_F32 / OUT_I32: C += result (TSTORE<AtomicAdd>)
};

__device__ __forceinline__ float load_elem_f32(const void* p, long idx, int type)
{
    switch (type) {
        case PTOAMD_F32: return reinterpret_cast<const float*>(p)[idx];
        case PTOAMD_F16: return f16_bits_to_f32(reinterpret_cast<const uint16_t*>(p)[idx]);
        case PTOAMD_BF16: return bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(p)[idx]);
        case PTOAMD_E4M3: return e4m3_to_f32(reinterpret_cast<const uint8_t*>(p)[idx]);
        case PTOAMD_E5M2: return e5m2_to_f32(reinterpret_cast<const uint8_t*>(p)[idx]);
        case PTOAMD_E2M1: return e2m1_to_f32((reinterpret_cast<const uint8_t*>(p)[idx >> 1] >> ((idx & 1) * 4)) & 0xFu);
        case PTOAMD_E1M2: return e1m2_to_f32((reinterpret_cast<const uint8_t*>(p)[idx >> 1] >> ((idx & 1) * 4)) & 0xFu);
        case PTOAMD_HIF8: return hif8_to_f32(reinterpret_cast<const uint8_t*>(p)[idx]);
        default: return (float)reinterpret_cast<const int8_t*>(p)[idx];
    }
}

// the quantising drains: word -> scale / offset / range, relu after the quantisation
template <bool SRC_INT>
__device__ __forceinline__ void store_quant(const GenericParams& p, long o, float acc, int gj)
{
    const uint64_t w = p.qwords[p.q_per_column ? gj : 0];
    const bool sat_inf = !SRC_INT && (p.relu & 2) != 0;
    if (p.out_kind == OUT_QBF16) {
        float r = __fmul_rn(acc, p.q_per_column ? fixpipe_word_scale<true>(w) : fixpipe_word_scale<false>(w));
        if (sat_inf)
            r = fixpipe_saturate_inf<false>(r);
        if (p.relu & 1)
            r = r > 0 ? r : 0;
        reinterpret_cast<uint16_t*>(p.c)[o] = f32_to_bf16_bits(r);
        return;
    }
    const bool byte = p.out_kind == OUT_Q8;
    float r;
    if (byte)
        r = p.q_per_column ? fixpipe_quantize<true, true, SRC_INT>(acc, w) : fixpipe_quantize<false, true, SRC_INT>(acc, w);
    else
        r = p.q_per_column ? fixpipe_quantize<true, false, SRC_INT>(acc, w) : fixpipe_quantize<false, false, SRC_INT>(acc, w);
    if (!byte && sat_inf)
        r = fixpipe_saturate_inf<true>(r);
    if (p.relu & 1)
        r = r > 0 ? r : 0;
    if (byte)
        reinterpret_cast<uint8_t*>(p.c)[o] = (uint8_t)(int32_t)r;
    else
        reinterpret_cast<uint16_t*>(p.c)[o] = f32_to_f16_bits(r);
}

__device__ __forceinline__ void store_out(const GenericParams& p, long o, float v, int gi, int gj)
{
    if (p.out_kind == OUT_Q8 || p.out_kind == OUT_QF16 || p.out_kind == OUT_QBF16) {
        store_quant<false>(p, o, v, gj);
        return;
    }
    if (p.relu & 1)
        v = v > 0 ? v : 0;
    switch (p.out_kind) {
        case OUT_F32:
            if (p.atomic_add)
                atomicAdd(reinterpret_cast<float*>(p.c) + o, v);
            else
                reinterpret_cast<float*>(p.c)[o] = v;
            break;
        case OUT_F16: reinterpret_cast<uint16_t*>(p.c)[o] = f32_to_f16_bits(v); break;
        default: reinterpret_cast<uint16_t*>(p.c)[o] = f32_to_bf16_bits(v); break;
    }
    (void)gi;
    (void)gj;
}

__global__ void gemm_generic_kernel(const GenericParams p)
{
    const int gj = blockIdx.x * blockDim.x + threadIdx.x;
    const int gi = blockIdx.y * blockDim.y + threadIdx.y;
    if (gi >= p.m || gj >= p.n)
        return;
    const long o = (long)gi * p.ldc + gj;
    if (p.a_type == PTOAMD_I8 && !p.mx) {
        uint32_t acc = p.c_in ? (uint32_t) reinterpret_cast<const int32_t*>(p.c_in)[o] : 0u;
        const int8_t* a = reinterpret_cast<const int8_t*>(p.a) + (long)gi * p.lda;
        const int8_t* b = reinterpret_cast<const int8_t*>(p.b) + (long)gj * p.sbn;
        for (int kk = 0; kk < p.k; ++kk)
            acc += (uint32_t)((int32_t)a[kk] * (int32_t)b[(long)kk * p.sbk]);
        if (p.bias)
            acc += (uint32_t) reinterpret_cast<const int32_t*>(p.bias)[gj];
        int32_t v = (int32_t)acc;
        if (p.out_kind == OUT_QS16) {
            int32_t r = fixpipe_shift_s16(v, p.qwords[p.q_per_column ? gj : 0]);
            if (p.relu & 1)
                r = r > 0 ? r : 0;
            reinterpret_cast<int16_t*>(p.c)[o] = (int16_t)r;
            return;
        }
        if (p.out_kind == OUT_Q8 || p.out_kind == OUT_QF16 || p.out_kind == OUT_QBF16) {
            store_quant<true>(p, o, (float)v, gj);
            return;
        }
        if (p.relu & 1)
            v = v > 0 ? v : 0;
        if (p.out_kind == OUT_I32) {
            if (p.atomic_add)
                atomicAdd(reinterpret_cast<int*>(p.c) + o, v);
            else
                reinterpret_cast<int32_t*>(p.c)[o] = v;
        } else {
            if (p.acc_out)
                p.acc_out[o] = v;
            const float t = __fmul_rn((float)v, p.row_scale[gi]);
            reinterpret_cast<uint16_t*>(p.c)[o] = f32_to_bf16_bits(__fmul_rn(t, p.col_scale[gj]));
        }
        return;
    }
    float acc = p.c_in ? reinterpret_cast<const float*>(p.c_in)[o] : 0.0f;
    if (!p.mx) {
        for (int kk = 0; kk < p.k; ++kk) {
            const float av = load_elem_f32(p.a, (long)gi * p.lda + kk, p.a_type);
            const float bv = load_elem_f32(p.b, (long)kk * p.sbk + (long)gj * p.sbn, p.b_type);
            acc = __fmaf_rn(av, bv, acc);
        }
    } else {
        const int kg = p.k / 32;
        for (int kk = 0; kk < p.k; ++kk) {
            const double sf = e8m0_to_f64(p.sa[mx_scale_offset(p.sa_layout, p.m, kg, gi, kk / 32)]) *
                              e8m0_to_f64(p.sb[mx_scale_offset(p.sb_layout, kg, p.n, kk / 32, gj)]);
            const double av = (double)load_elem_f32(p.a, (long)gi * p.lda + kk, p.a_type);
            const double bv = (double)load_elem_f32(p.b, (long)kk * p.sbk + (long)gj * p.sbn, p.b_type);
            acc = (float)((double)acc + av * bv * sf);  // double add, then one rounding to float per k
        }
    }
    if (p.bias)
        acc = __fadd_rn(acc, reinterpret_cast<const float*>(p.bias)[gj]);
    store_out(p, o, acc, gi, gj);
}

static int launch_generic(const GenericParams& p, hipStream_t stream)
{
    dim3 block(32, 8), grid((p.n + 31) / 32, (p.m + 7) / 8);
    hipLaunchKernelGGL(gemm_generic_kernel, grid, block, 0, stream, p);
    PTOAMD_HIP_CHECK(hipGetLastError());
    set_last_kernel("generic");
    return PTOAMD_OK;
}

static int elem_bits(int type)
{
    switch (type) {
        case PTOAMD_F32: case PTOAMD_I32: return 32;
        case PTOAMD_F16: case PTOAMD_BF16: case PTOAMD_I16: return 16;
        case PTOAMD_E2M1: case PTOAMD_E1M2: return 4;
        default: return 8;
    }
}

static bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
static long ws_row_bytes(long k_bytes) { return (k_bytes + 15) / 16 * 16; }  // row pitch of a transposed B in a workspace
static bool aligned4(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 3u) == 0; }

// Which tile shape to run: the largest whose grid still fills most of the 256 CUs.  PTOAMD_TILE=0|1|2 overrides,
// PTOAMD_FORCE_GENERIC=1 sends everything to the order-exact kernel (used by the parity tests).
// Tiles 0-2 stage slabs through registers (any K); tiles 3-7 DMA slabs straight into LDS and need K to be a whole
// number of 128-byte slabs (7: the 256 x 128 tile with a ring of three slabs, block-scaled types only -- for the other
// types the id selects tile 6).  Measured on MI355X: the 8-wave 256x256 DMA tile (4) is the
// fastest for every operand type once the grid fills the chip (the block-scaled types included: their scales come
// through LDS, which leaves the 32-byte fp8 fragments just enough registers); smaller grids take the 128x128 DMA tile.
// The DMA tiles address an operand as a wave-uniform 64-bit base plus a 32-bit per-lane byte offset: the last row's offset
// plus the K extent must fit 32 bits, or the tile has to take the register-staged form (64-bit addresses per lane).
static bool dma_offsets_fit(int m, int n, long lda_bytes, long ldb_bytes, long k_bytes)
{
    const long last = std::max((long)(m - 1) * lda_bytes, (long)(n - 1) * ldb_bytes) + k_bytes;
    return last <= (long)UINT32_MAX;
}

// dma_ok: what the DMA tiles need besides whole slabs -- 16-byte aligned operand rows, 32-bit lane offsets, and for the
// block-scaled types scale rows they can stream.
// The plain types' tiles 4 and 5 also take a K that is not a whole number of slabs (at least one slab long).
// (ragged_k_ok: the operand type has them -- bf16, f16, int8)
static int pick_tile(int m, int n, long k_bytes, bool scaled, bool fp4 = false, bool dma_ok = true, bool ragged_k_ok = false)
{
    const bool ragged_k = (k_bytes % 128) != 0;
    const bool dtl_ok = dma_ok && (!ragged_k || (ragged_k_ok && k_bytes > 128));
    if (options().tile >= 0) {
        int t = options().tile;
        if (ragged_k && t > 5)  // tiles 6 and 7 exist for whole slabs only
            t = 5;
        if (t == 0)  // nor is the register-staged 256 x 256 tile (it spilled: 315 against 176 us for the 128 x 128 one on
            t = 1;   // bf16 4096 x 4096 x 4104)
        if (t < 3 || dtl_ok)
            return t;
        return 1;
    }
    const long t256 = (long)((m + 255) / 256) * ((n + 255) / 256);
    const long t128 = (long)((m + 127) / 128) * ((n + 127) / 128);
    const long t256x128 = (long)((m + 255) / 256) * ((n + 127) / 128);
    const int cus = device_compute_units();
    // Block-scaled types between half and three quarters of a round of 256 x 256 tiles: the 256 x 128 tile with the
    // three-slab ring puts a workgroup on (nearly) every CU (MXFP4 2048 x 4096 x 4096: 22.5 against 24.9 us)
    if (scaled && dtl_ok && t256 >= cus / 2 && t256 < 3 * cus / 4 && t256x128 <= cus)
        return 7;
    if (scaled && dtl_ok && t256 >= cus / 2)
        return 4;  // half the copy-in bytes per MFMA of the 128x128 tile
    if (scaled)
        return t128 >= 3 * cus / 8 ? (dtl_ok ? 5 : 1) : 2;
    if (t256 >= cus / 2)
        return dtl_ok ? 4 : 1;
    if (t128 >= 3 * cus / 8)
        return dtl_ok ? 5 : 1;
    return 2;
}

// Launch on the chosen tile.  When the 256x256 grid is some (nearly) whole rounds of the CUs plus at most half a round,
// the columns of that remainder run as smaller tiles in a second launch on the same stream: 256x128 tiles (at most
// one workgroup per CU, same wave tile as the large form) or 128x128 tiles (two workgroups per CU); a tile of the tail
// then costs a half or a quarter of a 256x256 tile's time instead of a whole round (MXFP8 4096 x 14336 x 4096, 3.5
// rounds of 256 CUs).  PTOAMD_TILE (an explicit tile) and PTOAMD_NO_TAIL_SPLIT=1 switch the split off;
// PTOAMD_TAIL_TILE=5|6|7 picks the tail's tile (default: 7 for the block-scaled types, 5 otherwise).
static hipError_t launch_tiles_as(int tile, int op, const TileGemmParams& p, hipStream_t stream)
{
    if ((tile == 4 || tile == 3) && options().tile < 0 && !options().no_tail_split) {
        const int cus = device_compute_units();
        const int tiles_m = (p.m + 255) / 256, tiles_n = (p.n + 255) / 256;
        // `whole`: the most tile columns whose tiles make (nearly) whole rounds -- at most a sixteenth of a round idle --
        // with at most half a round's worth of tiles left over.  Looked for only when the grid's own last round is at most
        // five eighths full (a fuller one is better left alone).
        const long all = (long)tiles_m * tiles_n;
        const long last_fill = all - (all - 1) / cus * cus;
        int whole = 0;
        if (last_fill <= 5 * cus / 8) {
            for (int w = tiles_n - 1; w > 0 && (long)tiles_m * (tiles_n - w) <= cus / 2; --w) {
                const long head_tiles = (long)tiles_m * w;
                if ((head_tiles + cus - 1) / cus * cus - head_tiles <= cus / 16) {
                    whole = w;
                    break;
                }
            }
        }
        if (whole > 0) {
            const int n1 = whole * 256;
            TileGemmParams head = p;
            head.n = n1;
            const hipError_t e = launch_gemm_tile(tile, op, head, stream);
            if (e != hipSuccess)
                return e;
            TileGemmParams tail = p;
            const size_t esz = (p.out_kind == OUT_F32 || p.out_kind == OUT_I32) ? 4 : (p.out_kind == OUT_Q8 ? 1 : 2);
            tail.n = p.n - n1;
            tail.b = p.b + (long)n1 * p.ldb_bytes;
            tail.c = static_cast<uint8_t*>(p.c) + (size_t)n1 * esz;
            if (p.c_in)
                tail.c_in = static_cast<const uint8_t*>(p.c_in) + (size_t)n1 * 4;
            if (p.bias)
                tail.bias = static_cast<const uint8_t*>(p.bias) + (size_t)n1 * 4;
            if (p.acc_out)
                tail.acc_out = p.acc_out + n1;
            if (p.sb)
                tail.sb = p.sb + (long)n1 * p.scale_ld;
            if (p.col_scale)
                tail.col_scale = p.col_scale + n1;
            if (p.qwords && p.q_per_column)
                tail.qwords = p.qwords + n1;
            // block-scaled types: the 256 x 128 tile with the three-slab ring unless a tail tile was asked for
            const bool scaled_op = op >= TOP_FP8_E4E4;
            return launch_gemm_tile(options().tail_tile > 0 ? options().tail_tile : (scaled_op ? 7 : 5), op, tail, stream);
        }
    }
    return launch_gemm_tile(tile, op, p, stream);
}

static hipError_t launch_tiles(int tile, int op, const TileGemmParams& p, hipStream_t stream)
{
    // tile id 3: the 16x16x128 form of the block-scaled fp8 types' large tile (the other types have one form, under both
    // ids).  Same results bit for bit and, on MXFP8 4096 x 14336 x 4096, the same time: 2 718 clocks per slab at 1.71 GHz
    // against 2 500 at 1.58 GHz on one box -- what the part sustains under this kernel is a rate of matrix work, not a
    // clock.  The 32x32x64 form also takes ragged edges and stays the default; PTOAMD_MX_16X16=1 selects the other.
    const int big = options().mx_16x16 ? 3 : 4;
    if (tile == 4)
        return launch_tiles_as(big, op, p, stream);
    return launch_tiles_as(tile, op, p, stream);
}

static bool force_generic() { return options().force_generic; }

// the tile id a launch of `tile` ends up on (the block-scaled fp8 types' large tile has two forms, see launch_tiles)
static int tile_as_launched(int tile, int op, int m, int n)
{
    const bool fp8 = op >= TOP_FP8_E4E4 && op != TOP_FP4;
    if (fp8 && m % 256 == 0 && n % 256 == 0 && ((tile == 4 && options().mx_16x16) || tile == 3))
        return 3;
    return tile == 3 ? 4 : tile;
}

static const char* tile_kernel_name(int tile, int op)
{
    static const char* ops[TOP_COUNT] = {"bf16", "f16", "i8", "fp8_e4m3_e4m3", "fp8_e5m2_e5m2", "fp8_e4m3_e5m2",
                                         "fp8_e5m2_e4m3", "fp4_e2m1"};
    static const char* tiles[8] = {"tile256x256", "tile128x128", "tile64x64", "tile256x256w8x16_dtl", "tile256x256w8_dtl",
                                   "tile128x128_dtl", "tile256x128_dtl", "tile256x128r3_dtl"};
    static thread_local char buf[64];
    snprintf(buf, sizeof buf, "%s_%s", tiles[tile], ops[op]);
    return buf;
}

template <typename T>
static int transpose_b(void* dst, const void* src, int k, int n, long ldb, long ld_dst, hipStream_t stream)
{
    dim3 block(32, 8), grid((n + 31) / 32, (k + 31) / 32);
    hipLaunchKernelGGL(transpose_kernel<T>, grid, block, 0, stream, reinterpret_cast<T*>(dst),
                       reinterpret_cast<const T*>(src), k, n, ldb, ld_dst);
    PTOAMD_HIP_CHECK(hipGetLastError());
    return PTOAMD_OK;
}

// ---- the library's own scratch memory ---------------------------------------------------------------------------
// ptoamd_gemm_mx_static re-lays scales into this array instead of a caller workspace or an allocation.  Each GPU the
// library runs on holds its own copy at its own address until the process ends.  In host code the name `scratch` is
// only a handle for hipGetSymbolAddress: the device address it yields (once per device, with that device current) is
// what kernels and copies are given.
static __device__ __align__(256) uint8_t scratch[PTOAMD_STATIC_SCRATCH_BYTES];

constexpr int MAX_DEVICES = 64;
static uint8_t* g_scratch_ptr[MAX_DEVICES];   // device address of `scratch`, per device; written once under g_scratch_mu
static std::mutex g_scratch_mu;

static int static_scratch(uint8_t** ptr)
{
    int dev = 0;
    PTOAMD_HIP_CHECK(hipGetDevice(&dev));
    PTOAMD_REQUIRE(dev >= 0 && dev < MAX_DEVICES, PTOAMD_E_UNSUPPORTED, "ptoamd_gemm_mx_static: device ordinal %d out of range", dev);
    std::lock_guard<std::mutex> lock(g_scratch_mu);
    if (g_scratch_ptr[dev] == nullptr) {
        void* p = nullptr;
        PTOAMD_HIP_CHECK(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        PTOAMD_REQUIRE(p != nullptr, PTOAMD_E_HIP, "ptoamd_gemm_mx_static: the scratch array has no device address");
        g_scratch_ptr[dev] = reinterpret_cast<uint8_t*>(p);
    }
    *ptr = g_scratch_ptr[dev];
    return PTOAMD_OK;
}

int prepare_gemm_kernels()
{
    for (int op : {TOP_BF16, TOP_F16, TOP_I8, TOP_FP8_E4E4, TOP_FP8_E5E5, TOP_FP8_E4E5, TOP_FP8_E5E4, TOP_FP4})
        PTOAMD_HIP_CHECK(launch_gemm_tile(TILE_PREPARE_ALL, op, TileGemmParams{}, nullptr));
    uint8_t* unused = nullptr;
    return static_scratch(&unused);
}

}  // namespace ptoamd

using namespace ptoamd;

extern "C" {

int ptoamd_mx_scale_relayout(uint8_t* dst, int dst_layout, const uint8_t* src, int src_layout, int rows, int cols,
                             void* stream)
{
    static const char* const names[] = {"MX_A_ZZ", "MX_A_ND", "MX_A_DN", "MX_B_NN", "MX_B_ND", "MX_B_DN"};
    TraceScope trace("TMOV", "vector", rows, cols, 0);
    trace.in(src, rows, cols, src_layout >= 0 && src_layout <= 5 ? names[src_layout] : "?", 100)
        .out(dst, rows, cols, dst_layout >= 0 && dst_layout <= 5 ? names[dst_layout] : "?", 100);
    PTOAMD_REQUIRE(dst && src && rows > 0 && cols > 0, PTOAMD_E_INVALID, "ptoamd_mx_scale_relayout: bad argument");
    PTOAMD_REQUIRE(dst_layout >= 0 && dst_layout <= 5 && src_layout >= 0 && src_layout <= 5, PTOAMD_E_INVALID,
                   "ptoamd_mx_scale_relayout: unknown layout");
    const bool a_side = src_layout <= PTOAMD_MX_A_DN;
    PTOAMD_REQUIRE(a_side == (dst_layout <= PTOAMD_MX_A_DN), PTOAMD_E_INVALID,
                   "ptoamd_mx_scale_relayout: source and destination must both be A-side or both B-side layouts");
    const int pair_dim = a_side ? cols : rows;   // the K/32 axis is stored in pairs
    const int box_dim = a_side ? rows : cols;    // ZZ / NN box the other axis by 16
    PTOAMD_REQUIRE(pair_dim % 2 == 0, PTOAMD_E_INVALID, "ptoamd_mx_scale_relayout: K/32 must be even");
    const bool boxed = src_layout == PTOAMD_MX_A_ZZ || dst_layout == PTOAMD_MX_A_ZZ || src_layout == PTOAMD_MX_B_NN ||
                       dst_layout == PTOAMD_MX_B_NN;
    PTOAMD_REQUIRE(!boxed || box_dim % 16 == 0, PTOAMD_E_INVALID,
                   "ptoamd_mx_scale_relayout: ZZ/NN layouts need the row (A) / column (B) count to be a multiple of 16");
    const long total = (long)rows * cols;
    hipLaunchKernelGGL(mx_scale_relayout_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, as_stream(stream),
                       dst, dst_layout, src, src_layout, rows, cols);
    PTOAMD_HIP_CHECK(hipGetLastError());
    set_last_kernel("mx_scale_relayout");
    return PTOAMD_OK;
}

int ptoamd_gemm(void* c, int c_type, const void* a, const void* b, int ab_type, const void* c_in, int m, int n, int k,
                int lda, int ldb, int ldc, int b_layout, int relu, void* stream_)
{
    return ptoamd_gemm_bias(c, c_type, a, b, ab_type, c_in, nullptr, m, n, k, lda, ldb, ldc, b_layout, relu, stream_);
}

static int gemm_common(void* c, int c_type, const void* a, const void* b, int ab_type, const void* c_in, const void* bias,
                       const uint64_t* qwords, int q_per_column, int m, int n, int k, int lda, int ldb, int ldc, int b_layout,
                       int relu, void* stream_, int atomic_add = 0, int b_type = -1, void* ws = nullptr, size_t ws_bytes = 0);

int ptoamd_gemm_bias(void* c, int c_type, const void* a, const void* b, int ab_type, const void* c_in, const void* bias,
                     int m, int n, int k, int lda, int ldb, int ldc, int b_layout, int relu, void* stream_)
{
    return gemm_common(c, c_type, a, b, ab_type, c_in, bias, nullptr, 0, m, n, k, lda, ldb, ldc, b_layout, relu, stream_);
}

size_t ptoamd_gemm_workspace_bytes(int n, int k, int ab_type, int b_layout)
{
    if (n <= 0 || k <= 0 || b_layout != PTOAMD_B_ND)
        return 0;
    return (size_t)n * (size_t)ws_row_bytes((long)k * (elem_bits(ab_type) / 8));
}

int ptoamd_gemm_ws(void* c, int c_type, const void* a, const void* b, int ab_type, const void* c_in, const void* bias, int m, int n,
                   int k, int lda, int ldb, int ldc, int b_layout, int relu, void* workspace, size_t workspace_bytes, void* stream_)
{
    PTOAMD_REQUIRE(workspace == nullptr || (reinterpret_cast<uintptr_t>(workspace) & 255u) == 0, PTOAMD_E_ALIGNMENT,
                   "ptoamd_gemm_ws: the workspace must be 256-byte aligned");
    return gemm_common(c, c_type, a, b, ab_type, c_in, bias, nullptr, 0, m, n, k, lda, ldb, ldc, b_layout, relu, stream_, 0, -1,
                       workspace, workspace ? workspace_bytes : 0);
}

int ptoamd_gemm_fp8(void* c, int c_type, const void* a, int a_type, const void* b, int b_type, const void* c_in, const void* bias,
                    int m, int n, int k, int lda, int ldb, int ldc, int b_layout, int relu, void* stream_)
{
    const bool a8 = a_type == PTOAMD_E4M3 || a_type == PTOAMD_E5M2, b8 = b_type == PTOAMD_E4M3 || b_type == PTOAMD_E5M2;
    PTOAMD_REQUIRE(a8 && b8, PTOAMD_E_UNSUPPORTED, "ptoamd_gemm_fp8: both operand types must be e4m3 or e5m2 (got %d, %d)", a_type, b_type);
    return gemm_common(c, c_type, a, b, a_type, c_in, bias, nullptr, 0, m, n, k, lda, ldb, ldc, b_layout, relu, stream_, 0, b_type);
}

int ptoamd_gemm_requant(void* c, int c_type, const void* a, const void* b, int ab_type, const void* c_in, const void* bias,
                        const uint64_t* quant_words, int per_column, int m, int n, int k, int lda, int ldb, int ldc,
                        int b_layout, int relu, void* stream_)
{
    PTOAMD_REQUIRE(quant_words != nullptr, PTOAMD_E_INVALID, "ptoamd_gemm_requant: null quantisation words");
    PTOAMD_REQUIRE(c_type == PTOAMD_I8 || c_type == PTOAMD_U8 || c_type == PTOAMD_F16 || c_type == PTOAMD_BF16 || c_type == PTOAMD_I16,
                   PTOAMD_E_UNSUPPORTED, "ptoamd_gemm_requant: the fix-pipe quantiser stores s8, u8, f16, bf16 or s16 (got type %d)", c_type);
    PTOAMD_REQUIRE((reinterpret_cast<uintptr_t>(quant_words) & 7u) == 0, PTOAMD_E_ALIGNMENT,
                   "ptoamd_gemm_requant: quantisation words must be 8-byte aligned");
    return gemm_common(c, c_type, a, b, ab_type, c_in, bias, quant_words, per_column ? 1 : 0, m, n, k, lda, ldb, ldc, b_layout,
                       relu, stream_);
}

int ptoamd_gemm_atomic_add(void* c, int c_type, const void* a, const void* b, int ab_type, int m, int n, int k, int lda, int ldb,
                           int ldc, int b_layout, void* stream_)
{
    PTOAMD_REQUIRE(c_type == PTOAMD_F32 || c_type == PTOAMD_I32, PTOAMD_E_UNSUPPORTED,
                   "ptoamd_gemm_atomic_add: atomic adds target f32 or i32 (got type %d)", c_type);
    return gemm_common(c, c_type, a, b, ab_type, nullptr, nullptr, nullptr, 0, m, n, k, lda, ldb, ldc, b_layout, 0, stream_, 1);
}

static int gemm_common(void* c, int c_type, const void* a, const void* b, int ab_type, const void* c_in, const void* bias,
                       const uint64_t* qwords, int q_per_column, int m, int n, int k, int lda, int ldb, int ldc, int b_layout,
                       int relu, void* stream_, int atomic_add, int b_type, void* ws, size_t ws_bytes)
{
    // b_type: -1 = as ab_type; otherwise the second type of a mixed fp8 pair (ab_type is then A's)
    if (b_type < 0)
        b_type = ab_type;
    hipStream_t stream = as_stream(stream_);
    TraceScope trace(atomic_add ? "TMATMUL+TSTORE_ATOMIC_ADD"
                                : (qwords ? "TMATMUL+TSTORE_FP" : (bias ? "TMATMUL_BIAS" : (c_in ? "TMATMUL_ACC" : "TMATMUL"))),
                     "cube", m, n, k);
    trace.in(a, m, k, "ND", ab_type).in(b, k, n, b_layout == PTOAMD_B_DN ? "DN" : "ND", b_type)
        .in(c_in, m, n, "ND", ab_type == PTOAMD_I8 ? PTOAMD_I32 : PTOAMD_F32).in(bias, 1, n, "ND", ab_type == PTOAMD_I8 ? PTOAMD_I32 : PTOAMD_F32)
        .in(qwords, 1, q_per_column ? n : 1, "ND", 101).out(c, m, n, "ND", c_type);
    PTOAMD_REQUIRE(c && a && b, PTOAMD_E_INVALID, "ptoamd_gemm: null operand");
    PTOAMD_REQUIRE(m > 0 && n > 0 && k > 0, PTOAMD_E_INVALID, "ptoamd_gemm: m, n, k must be positive (%d, %d, %d)", m, n, k);
    PTOAMD_REQUIRE(b_layout == PTOAMD_B_ND || b_layout == PTOAMD_B_DN, PTOAMD_E_INVALID, "ptoamd_gemm: unknown b_layout");
    PTOAMD_REQUIRE(lda >= k && ldc >= n && ldb >= (b_layout == PTOAMD_B_DN ? k : n), PTOAMD_E_INVALID,
                   "ptoamd_gemm: leading dimension smaller than the row length");
    PTOAMD_REQUIRE((relu & ~(PTOAMD_RELU | PTOAMD_SATURATE_INF)) == 0, PTOAMD_E_INVALID, "ptoamd_gemm: unknown bits in the relu / flags argument");
    const bool is_int = ab_type == PTOAMD_I8;
    const bool is_float = ab_type == PTOAMD_F16 || ab_type == PTOAMD_BF16 || ab_type == PTOAMD_F32 ||
                          ab_type == PTOAMD_E4M3 || ab_type == PTOAMD_E5M2 || ab_type == PTOAMD_HIF8;
    PTOAMD_REQUIRE(is_int || is_float, PTOAMD_E_UNSUPPORTED,
                   "ptoamd_gemm: operand type %d is not a TMATMUL input type (s8, f16, bf16, f32, e4m3, e5m2, hif8)", ab_type);
    PTOAMD_REQUIRE((ab_type == PTOAMD_HIF8) == (b_type == PTOAMD_HIF8), PTOAMD_E_UNSUPPORTED,
                   "ptoamd_gemm: hif8 pairs with hif8 only");
    int out_kind;
    if (qwords != nullptr) {
        PTOAMD_REQUIRE(c_type != PTOAMD_I16 || is_int, PTOAMD_E_UNSUPPORTED,
                       "ptoamd_gemm_requant: the int16 shift mode takes int32 accumulators (int8 operands)");
        out_kind = c_type == PTOAMD_F16 ? OUT_QF16 : (c_type == PTOAMD_BF16 ? OUT_QBF16 : (c_type == PTOAMD_I16 ? OUT_QS16 : OUT_Q8));
    } else if (is_int) {
        PTOAMD_REQUIRE(c_type == PTOAMD_I32, PTOAMD_E_UNSUPPORTED, "ptoamd_gemm: int8 operands accumulate to int32 only");
        out_kind = OUT_I32;
    } else {
        PTOAMD_REQUIRE(c_type == PTOAMD_F32 || c_type == PTOAMD_F16 || c_type == PTOAMD_BF16, PTOAMD_E_UNSUPPORTED,
                       "ptoamd_gemm: float accumulators store as f32, f16 or bf16");
        out_kind = c_type == PTOAMD_F32 ? OUT_F32 : (c_type == PTOAMD_F16 ? OUT_F16 : OUT_BF16);
    }
    const int ebytes = elem_bits(ab_type) / 8;
    const long k_bytes = (long)k * ebytes, lda_b = (long)lda * ebytes, ldb_b = (long)ldb * ebytes;
    const uintptr_t emask = (uintptr_t)ebytes - 1;
    // The register-staged MFMA tiles take rows at any alignment and of any length from 16 bytes up (the row's last chunk
    // is masked), so only f32 / hif8 operands, rows shorter than 16 bytes and misaligned elements go to the order-exact
    // kernel.  B row-major: with a workspace it is re-ordered there once and the fastest tiles run; without one the
    // register-staged tiles transpose it on its way into LDS.  Nothing is allocated either way.
    const bool mfma_type = ab_type != PTOAMD_F32 && ab_type != PTOAMD_HIF8;
    const bool elems_ok = (reinterpret_cast<uintptr_t>(a) & emask) == 0 && (reinterpret_cast<uintptr_t>(b) & emask) == 0;
    const size_t ws_need = b_layout == PTOAMD_B_ND ? (size_t)n * (size_t)ws_row_bytes(k_bytes) : 0;
    const bool b_via_ws = b_layout == PTOAMD_B_ND && ws != nullptr && (ebytes == 1 || ebytes == 2) && !options().b_nd_in_loader;
    PTOAMD_REQUIRE(!b_via_ws || ws_need <= ws_bytes, PTOAMD_E_INVALID,
                   "ptoamd_gemm_ws: re-ordering B needs %zu bytes of workspace, %zu available", ws_need, ws_bytes);
    const bool b_in_kernel = b_layout == PTOAMD_B_ND && !b_via_ws && (ebytes == 1 || ebytes == 2) && (long)n * ebytes >= 16;
    const bool tile_ok = !force_generic() && mfma_type && elems_ok && k_bytes >= 16 &&
                         (b_layout == PTOAMD_B_DN || b_via_ws || b_in_kernel);
    if (!tile_ok) {
        GenericParams g{};
        g.a = a; g.b = b; g.c = c; g.c_in = c_in; g.bias = bias;
        g.m = m; g.n = n; g.k = k; g.lda = lda; g.ldc = ldc;
        g.sbk = b_layout == PTOAMD_B_DN ? 1 : ldb;
        g.sbn = b_layout == PTOAMD_B_DN ? ldb : 1;
        g.a_type = ab_type; g.b_type = b_type; g.out_kind = out_kind; g.relu = relu;
        g.qwords = qwords; g.q_per_column = q_per_column; g.atomic_add = atomic_add;
        return launch_generic(g, stream);
    }
    const uint8_t* b_kmajor = reinterpret_cast<const uint8_t*>(b);
    long ldb_kmajor = ldb_b;
    if (b_via_ws) {  // TLOAD of an ND B panel: re-order once so the MFMA path reads K-contiguous rows
        // rows of the re-ordered copy start on 16-byte boundaries whatever K is
        const long pitch = ws_row_bytes(k_bytes);
        const int rc = ebytes == 2 ? transpose_b<uint16_t>(ws, b, k, n, ldb, pitch / 2, stream)
                                   : transpose_b<uint8_t>(ws, b, k, n, ldb, pitch, stream);
        if (rc != PTOAMD_OK)
            return rc;
        b_kmajor = reinterpret_cast<const uint8_t*>(ws);
        ldb_kmajor = pitch;
    }
    TileGemmParams p{};
    p.a = reinterpret_cast<const uint8_t*>(a);
    p.b = b_kmajor;
    p.c = c; p.c_in = c_in; p.bias = bias;
    p.m = m; p.n = n; p.k_bytes = (int)k_bytes;
    p.lda_bytes = lda_b; p.ldb_bytes = ldb_kmajor; p.ldc = ldc;
    p.relu = relu; p.out_kind = out_kind; p.group_m = 4;
    p.qwords = qwords; p.q_per_column = q_per_column; p.atomic_add = atomic_add;
    const int op = ab_type == PTOAMD_BF16 ? TOP_BF16
                   : ab_type == PTOAMD_F16 ? TOP_F16
                   : ab_type == PTOAMD_I8 ? TOP_I8
                   : ab_type == PTOAMD_E4M3 ? (b_type == PTOAMD_E4M3 ? TOP_FP8_E4E4 : TOP_FP8_E4E5)
                                            : (b_type == PTOAMD_E5M2 ? TOP_FP8_E5E5 : TOP_FP8_E5E4);
    p.b_nd = b_in_kernel; p.b_esz = ebytes;
    // (LDS-DMA needs dword-aligned global addresses, no more: rows at 4-byte alignment run 114 against 100 us on bf16 4096^3)
    const bool dma_ok = !b_in_kernel && aligned4(a) && aligned4(b_kmajor) && (lda_b % 4) == 0 && (ldb_kmajor % 4) == 0 &&
                        dma_offsets_fit(m, n, lda_b, ldb_kmajor, k_bytes);
    const int tile = pick_tile(m, n, k_bytes, false, false, dma_ok, op == TOP_BF16 || op == TOP_F16 || op == TOP_I8);
    PTOAMD_HIP_CHECK(launch_tiles(tile, op, p, stream));
    set_last_kernel(tile_kernel_name(tile_as_launched(tile, op, m, n), op));
    return PTOAMD_OK;
}

int ptoamd_gemm_w8a8(void* out_bf16, int32_t* acc_out, const int8_t* a, const int8_t* b, const float* scale_a,
                     const float* scale_b, int m, int n, int k, int lda, int ldb, int ldc, int b_layout, void* stream_)
{
    hipStream_t stream = as_stream(stream_);
    TraceScope trace("TMATMUL+TDEQUANT", "cube", m, n, k);
    trace.in(a, m, k, "ND", PTOAMD_I8).in(b, k, n, b_layout == PTOAMD_B_DN ? "DN" : "ND", PTOAMD_I8).in(scale_a, m, 1, "ND", PTOAMD_F32)
        .in(scale_b, 1, n, "ND", PTOAMD_F32).out(out_bf16, m, n, "ND", PTOAMD_BF16).out(acc_out, m, n, "ND", PTOAMD_I32);
    PTOAMD_REQUIRE(out_bf16 && a && b && scale_a && scale_b, PTOAMD_E_INVALID, "ptoamd_gemm_w8a8: null operand");
    PTOAMD_REQUIRE(m > 0 && n > 0 && k > 0, PTOAMD_E_INVALID, "ptoamd_gemm_w8a8: m, n, k must be positive");
    PTOAMD_REQUIRE(b_layout == PTOAMD_B_ND || b_layout == PTOAMD_B_DN, PTOAMD_E_INVALID, "ptoamd_gemm_w8a8: unknown b_layout");
    PTOAMD_REQUIRE(lda >= k && ldc >= n && ldb >= (b_layout == PTOAMD_B_DN ? k : n), PTOAMD_E_INVALID,
                   "ptoamd_gemm_w8a8: leading dimension smaller than the row length");
    // (rows at any alignment, any K from 16 up: see ptoamd_gemm; a row-major B is transposed by the register-staged loader)
    const bool b_in_kernel = b_layout == PTOAMD_B_ND && n >= 16;
    const bool tile_ok = !force_generic() && k >= 16 && (b_layout == PTOAMD_B_DN || b_in_kernel);
    if (!tile_ok) {
        GenericParams g{};
        g.a = a; g.b = b; g.c = out_bf16; g.acc_out = acc_out; g.row_scale = scale_a; g.col_scale = scale_b;
        g.m = m; g.n = n; g.k = k; g.lda = lda; g.ldc = ldc;
        g.sbk = b_layout == PTOAMD_B_DN ? 1 : ldb;
        g.sbn = b_layout == PTOAMD_B_DN ? ldb : 1;
        g.a_type = g.b_type = PTOAMD_I8; g.out_kind = OUT_W8A8_BF16;
        return launch_generic(g, stream);
    }
    TileGemmParams p{};
    p.a = reinterpret_cast<const uint8_t*>(a);
    p.b = reinterpret_cast<const uint8_t*>(b);
    p.c = out_bf16; p.acc_out = acc_out; p.row_scale = scale_a; p.col_scale = scale_b;
    p.m = m; p.n = n; p.k_bytes = k; p.lda_bytes = lda; p.ldb_bytes = ldb; p.ldc = ldc;
    p.out_kind = OUT_W8A8_BF16; p.group_m = 4;
    p.b_nd = b_in_kernel; p.b_esz = 1;
    const bool dma_ok = !b_in_kernel && aligned4(a) && aligned4(b) && (lda % 4) == 0 && (ldb % 4) == 0 && dma_offsets_fit(m, n, lda, ldb, k);
    const int tile = pick_tile(m, n, k, false, false, dma_ok, true);
    PTOAMD_HIP_CHECK(launch_tiles(tile, TOP_I8, p, stream));
    set_last_kernel(tile_kernel_name(tile, TOP_I8));
    return PTOAMD_OK;
}

// Shared body of the TMATMUL_MX entry points.  The DMA tiles stream scales as [M][K/32] and [N][K/32] rows; other GM
// layouts are re-laid into `ws` (ws_bytes; the caller's workspace or the library's static array) when one is given, and
// addressed in place by the register-staged tiles when not.
static int gemm_mx_common(const char* who, void* c, int c_type, const void* a, const void* b, int a_type, int b_type,
                          const uint8_t* sa, const uint8_t* sb, int sa_layout, int sb_layout, const float* c_in, int m, int n,
                          int k, int lda, int ldb, int ldc, int b_layout, uint8_t* ws, size_t ws_bytes, void* stream_,
                          const float* bias = nullptr)
{
    hipStream_t stream = as_stream(stream_);
    static const char* const mx_layouts[] = {"MX_A_ZZ", "MX_A_ND", "MX_A_DN", "MX_B_NN", "MX_B_ND", "MX_B_DN"};
    TraceScope trace(bias ? "TMATMUL_MX_BIAS" : (c_in ? "TMATMUL_MX_ACC" : "TMATMUL_MX"), "cube", m, n, k);
    trace.in(a, m, k, "ND", a_type).in(b, k, n, b_layout == PTOAMD_B_DN ? "DN" : "ND", b_type)
        .in(sa, m, k / 32, sa_layout >= 0 && sa_layout < 6 ? mx_layouts[sa_layout] : "?", 100)
        .in(sb, k / 32, n, sb_layout >= 0 && sb_layout < 6 ? mx_layouts[sb_layout] : "?", 100).in(c_in, m, n, "ND", PTOAMD_F32)
        .in(bias, 1, n, "ND", PTOAMD_F32).out(c, m, n, "ND", c_type);
    PTOAMD_REQUIRE(c && a && b && sa && sb, PTOAMD_E_INVALID, "%s: null operand", who);
    PTOAMD_REQUIRE(m > 0 && n > 0 && k > 0, PTOAMD_E_INVALID, "%s: m, n, k must be positive", who);
    PTOAMD_REQUIRE(k % 64 == 0, PTOAMD_E_INVALID, "%s: k = %d must be a multiple of 64", who, k);
    PTOAMD_REQUIRE(b_layout == PTOAMD_B_ND || b_layout == PTOAMD_B_DN, PTOAMD_E_INVALID, "%s: unknown b_layout", who);
    PTOAMD_REQUIRE(sa_layout >= PTOAMD_MX_A_ZZ && sa_layout <= PTOAMD_MX_A_DN && sb_layout >= PTOAMD_MX_B_NN &&
                       sb_layout <= PTOAMD_MX_B_DN,
                   PTOAMD_E_INVALID, "%s: sa_layout must be an MX_A_* and sb_layout an MX_B_* layout", who);
    const bool a8 = a_type == PTOAMD_E4M3 || a_type == PTOAMD_E5M2, b8 = b_type == PTOAMD_E4M3 || b_type == PTOAMD_E5M2;
    const bool a4 = a_type == PTOAMD_E2M1 || a_type == PTOAMD_E1M2, b4 = b_type == PTOAMD_E2M1 || b_type == PTOAMD_E1M2;
    PTOAMD_REQUIRE((a8 && b8) || (a4 && b4), PTOAMD_E_UNSUPPORTED,
                   "%s: operands must both be fp8 (e4m3/e5m2) or both fp4 (e2m1/e1m2)", who);
    PTOAMD_REQUIRE(c_type == PTOAMD_F32 || c_type == PTOAMD_F16 || c_type == PTOAMD_BF16, PTOAMD_E_UNSUPPORTED,
                   "%s: the accumulator stores as f32, f16 or bf16", who);
    PTOAMD_REQUIRE(lda >= k && ldc >= n && ldb >= (b_layout == PTOAMD_B_DN ? k : n), PTOAMD_E_INVALID,
                   "%s: leading dimension smaller than the row length", who);
    PTOAMD_REQUIRE(sa_layout != PTOAMD_MX_A_ZZ || m % 16 == 0, PTOAMD_E_INVALID, "%s: MX_A_ZZ needs m %% 16 == 0", who);
    PTOAMD_REQUIRE(sb_layout != PTOAMD_MX_B_NN || n % 16 == 0, PTOAMD_E_INVALID, "%s: MX_B_NN needs n %% 16 == 0", who);
    if (a4)
        PTOAMD_REQUIRE(lda % 2 == 0 && ldb % 2 == 0, PTOAMD_E_ALIGNMENT, "%s: fp4 leading dimensions must be even", who);
    const int out_kind = c_type == PTOAMD_F32 ? OUT_F32 : (c_type == PTOAMD_F16 ? OUT_F16 : OUT_BF16);
    const int bits = a8 ? 8 : 4;
    const long k_bytes = (long)k * bits / 8, lda_b = (long)lda * bits / 8;
    long ldb_b = (long)ldb * bits / 8;
    // The scaled MFMA has no E1M2 operand format, but every E1M2 (and E2M1) value is an E4M3 value: a product with an
    // E1M2 operand runs on the E4M3 x E4M3 instruction, the register-staged loader expanding both operands' packed
    // nibbles to E4M3 bytes on their way into LDS (the block scales are per 32 elements in either form).
    const bool e1m2 = a_type == PTOAMD_E1M2 || b_type == PTOAMD_E1M2;
    const bool expand_ok = e1m2 && b_layout == PTOAMD_B_DN && (k % 128) == 0 && (reinterpret_cast<uintptr_t>(a) & 7u) == 0 &&
                           (reinterpret_cast<uintptr_t>(b) & 7u) == 0 && (lda_b % 8) == 0 && (ldb_b % 8) == 0;
    // Workspace layout: [M][K/32] scales of A (when they need re-laying), rounded up to 256 bytes, the [N][K/32] scales of
    // B likewise, then -- when B is row-major fp8 and the room is there -- a [N][K] copy of B, rows padded to 16 bytes.
    const int kg = k / 32;
    int sa_mode = sa_layout == PTOAMD_MX_A_ND ? 0 : (sa_layout == PTOAMD_MX_A_ZZ ? 1 : 2);
    int sb_mode = sb_layout == PTOAMD_MX_B_DN ? 0 : (sb_layout == PTOAMD_MX_B_NN ? 1 : 2);
    const size_t need_a = sa_mode != 0 ? (((size_t)m * kg + 255) & ~(size_t)255) : 0;
    const size_t need_b = sb_mode != 0 ? (size_t)n * kg : 0;
    const size_t bt_at = (need_a + need_b + 255) & ~(size_t)255;
    const long bt_pitch = ws_row_bytes(k_bytes);
    // A row-major B of one-byte codes: with room in the workspace it is transposed there first and the DMA tiles run (a
    // large product: every B element would otherwise be scattered into LDS once per row tile); without, the
    // register-staged tiles transpose it on its way into LDS.  Packed fp4 has neither.
    const bool b_via_ws = b_layout == PTOAMD_B_ND && a8 && ws != nullptr && !force_generic() && m > 128 &&
                          ws_bytes >= bt_at + (size_t)n * (size_t)bt_pitch && (k_bytes % 128) == 0;
    if (b_via_ws) {  // from here on B is the column-major copy
        const int rc = transpose_b<uint8_t>(ws + bt_at, b, k, n, ldb_b, bt_pitch, stream);
        if (rc != PTOAMD_OK)
            return rc;
        b = ws + bt_at;
        b_layout = PTOAMD_B_DN;
        ldb = (int)bt_pitch;
        ldb_b = bt_pitch;
        ws_bytes = bt_at;
    }
    const bool b_in_kernel = b_layout == PTOAMD_B_ND && a8 && (n % 16) == 0;
    const bool tile_ok = !force_generic() &&
                         (e1m2 ? expand_ok
                               : ((b_layout == PTOAMD_B_DN || b_in_kernel) && aligned16(a) && aligned16(b) && (lda_b % 16) == 0 &&
                                  (ldb_b % 16) == 0 && (k_bytes % 128) == 0));
    if (!tile_ok) {
        GenericParams g{};
        g.a = a; g.b = b; g.c = c; g.c_in = c_in; g.sa = sa; g.sb = sb; g.bias = bias;
        g.m = m; g.n = n; g.k = k; g.lda = lda; g.ldc = ldc;
        g.sbk = b_layout == PTOAMD_B_DN ? 1 : ldb;
        g.sbn = b_layout == PTOAMD_B_DN ? ldb : 1;
        g.a_type = a_type; g.b_type = b_type; g.out_kind = out_kind; g.mx = 1;
        g.sa_layout = sa_layout; g.sb_layout = sb_layout;
        return launch_generic(g, stream);
    }
    // Scales that are not plain [M][K/32] / [N][K/32] rows: with a workspace they are re-laid into it and the DMA tiles run
    // (the fastest form for a large product); without one the register-staged tiles address the pairs of the caller's
    // layout directly.  Nothing is allocated either way.
    const uint8_t* sa_use = sa;
    const uint8_t* sb_use = sb;
    if (ws != nullptr && need_a + need_b > 0) {
        PTOAMD_REQUIRE(need_a + need_b <= ws_bytes, PTOAMD_E_INVALID,
                       "%s: the scale layouts need %zu bytes of workspace, %zu available", who, need_a + need_b, ws_bytes);
        if (sa_mode != 0) {
            const int rc = ptoamd_mx_scale_relayout(ws, PTOAMD_MX_A_ND, sa, sa_layout, m, kg, stream_);
            if (rc != PTOAMD_OK)
                return rc;
            sa_use = ws;
            sa_mode = 0;
        }
        if (sb_mode != 0) {
            const int rc = ptoamd_mx_scale_relayout(ws + need_a, PTOAMD_MX_B_DN, sb, sb_layout, kg, n, stream_);
            if (rc != PTOAMD_OK)
                return rc;
            sb_use = ws + need_a;
            sb_mode = 0;
        }
    }
    const bool plain_scales = sa_mode == 0 && sb_mode == 0;
    PTOAMD_REQUIRE((reinterpret_cast<uintptr_t>(sa_use) & (sa_mode == 0 ? 3u : 1u)) == 0 &&
                       (reinterpret_cast<uintptr_t>(sb_use) & (sb_mode == 0 ? 3u : 1u)) == 0,
                   PTOAMD_E_ALIGNMENT, "%s: scale arrays must be 4-byte aligned (2-byte in the boxed and pair-major layouts)", who);
    const uint8_t* sa_nd = sa_use;
    const uint8_t* sb_dn = sb_use;
    TileGemmParams p{};
    p.a = reinterpret_cast<const uint8_t*>(a);
    p.b = reinterpret_cast<const uint8_t*>(b);
    p.c = c; p.c_in = c_in; p.sa = sa_nd; p.sb = sb_dn; p.bias = bias;
    p.m = m; p.n = n; p.k_bytes = (int)k_bytes; p.lda_bytes = lda_b; p.ldb_bytes = ldb_b; p.ldc = ldc;
    p.scale_ld = kg; p.out_kind = out_kind; p.group_m = 4;
    p.sa_mode = sa_mode; p.sb_mode = sb_mode;
    p.b_nd = b_in_kernel; p.b_esz = 1;
    int op;
    if (e1m2) {
        op = TOP_FP8_E4E4;
        p.k_bytes = k;  // one E4M3 byte per element once expanded; the row pitches stay those of the packed operands
        p.a_expand = a_type == PTOAMD_E2M1 ? 1 : 2;
        p.b_expand = b_type == PTOAMD_E2M1 ? 1 : 2;
    } else if (a4)
        op = TOP_FP4;
    else if (a_type == PTOAMD_E4M3)
        op = b_type == PTOAMD_E4M3 ? TOP_FP8_E4E4 : TOP_FP8_E4E5;
    else
        op = b_type == PTOAMD_E5M2 ? TOP_FP8_E5E5 : TOP_FP8_E5E4;
    // the DMA tiles fetch scales as 16-byte chunks per row: 4 slabs of fp8, 2 of fp4
    const long k_slabs = k_bytes / 128;
    const bool scale_dma_ok = plain_scales && !b_in_kernel && (kg % 16) == 0 && aligned16(sa_nd) && aligned16(sb_dn) &&
                              (k_slabs % (a4 ? 2 : 4)) == 0;
    const int tile = e1m2 ? pick_tile(m, n, k, true, false, false)
                          : pick_tile(m, n, k_bytes, true, a4, scale_dma_ok && dma_offsets_fit(m, n, lda_b, ldb_b, k_bytes));
    PTOAMD_HIP_CHECK(launch_tiles(tile, op, p, stream));
    set_last_kernel(tile_kernel_name(tile_as_launched(tile, op, m, n), op));
    return PTOAMD_OK;
}

int ptoamd_gemm_mx(void* c, int c_type, const void* a, const void* b, int a_type, int b_type, const uint8_t* sa,
                   const uint8_t* sb, int sa_layout, int sb_layout, const float* c_in, int m, int n, int k, int lda,
                   int ldb, int ldc, int b_layout, void* stream_)
{
    return gemm_mx_common("ptoamd_gemm_mx", c, c_type, a, b, a_type, b_type, sa, sb, sa_layout, sb_layout, c_in, m, n, k, lda, ldb,
                          ldc, b_layout, nullptr, 0, stream_);
}

int ptoamd_gemm_mx_bias(void* c, int c_type, const void* a, const void* b, int a_type, int b_type, const uint8_t* sa,
                        const uint8_t* sb, int sa_layout, int sb_layout, const float* c_in, const float* bias, int m, int n,
                        int k, int lda, int ldb, int ldc, int b_layout, void* stream_)
{
    return gemm_mx_common("ptoamd_gemm_mx_bias", c, c_type, a, b, a_type, b_type, sa, sb, sa_layout, sb_layout, c_in, m, n, k, lda,
                          ldb, ldc, b_layout, nullptr, 0, stream_, bias);
}

int ptoamd_gemm_mx_ws(void* c, int c_type, const void* a, const void* b, int a_type, int b_type, const uint8_t* sa,
                      const uint8_t* sb, int sa_layout, int sb_layout, const float* c_in, int m, int n, int k, int lda,
                      int ldb, int ldc, int b_layout, void* workspace, size_t workspace_bytes, void* stream_)
{
    PTOAMD_REQUIRE(workspace == nullptr || (reinterpret_cast<uintptr_t>(workspace) & 255u) == 0, PTOAMD_E_ALIGNMENT,
                   "ptoamd_gemm_mx_ws: the workspace must be 256-byte aligned");
    return gemm_mx_common("ptoamd_gemm_mx_ws", c, c_type, a, b, a_type, b_type, sa, sb, sa_layout, sb_layout, c_in, m, n, k, lda,
                          ldb, ldc, b_layout, reinterpret_cast<uint8_t*>(workspace), workspace ? workspace_bytes : 0, stream_);
}

int ptoamd_gemm_mx_static(void* c, int c_type, const void* a, const void* b, int a_type, int b_type, const uint8_t* sa,
                          const uint8_t* sb, int sa_layout, int sb_layout, const float* c_in, int m, int n, int k, int lda,
                          int ldb, int ldc, int b_layout, void* stream_)
{
    const size_t need = ptoamd_gemm_mx_workspace_bytes(m, n, k, sa_layout, sb_layout);
    PTOAMD_REQUIRE(need <= (size_t)PTOAMD_STATIC_SCRATCH_BYTES, PTOAMD_E_UNSUPPORTED,
                   "ptoamd_gemm_mx_static: re-laying these scales needs %zu bytes, the static scratch holds %d "
                   "(use ptoamd_gemm_mx_ws with a workspace of that size)", need, PTOAMD_STATIC_SCRATCH_BYTES);
    uint8_t* ws = nullptr;
    const int rc = static_scratch(&ws);
    if (rc != PTOAMD_OK)
        return rc;
    return gemm_mx_common("ptoamd_gemm_mx_static", c, c_type, a, b, a_type, b_type, sa, sb, sa_layout, sb_layout, c_in, m, n, k,
                          lda, ldb, ldc, b_layout, ws, PTOAMD_STATIC_SCRATCH_BYTES, stream_);
}

size_t ptoamd_gemm_mx_workspace_bytes_b_nd(int m, int n, int k, int sa_layout, int sb_layout, int b_type)
{
    if (m <= 0 || n <= 0 || k <= 0)
        return 0;
    const size_t scales = (ptoamd_gemm_mx_workspace_bytes(m, n, k, sa_layout, sb_layout) + 255) & ~(size_t)255;
    if (b_type != PTOAMD_E4M3 && b_type != PTOAMD_E5M2)
        return scales;  // packed fp4 codes are not transposed
    return scales + (size_t)n * (size_t)ws_row_bytes(k);
}

size_t ptoamd_gemm_mx_workspace_bytes(int m, int n, int k, int sa_layout, int sb_layout)
{
    if (m <= 0 || n <= 0 || k <= 0)
        return 0;
    const size_t kg = (size_t)k / 32;
    const size_t need_a = sa_layout != PTOAMD_MX_A_ND ? (((size_t)m * kg + 255) & ~(size_t)255) : 0;
    const size_t need_b = sb_layout != PTOAMD_MX_B_DN ? (size_t)n * kg : 0;
    return need_a + need_b;
}

}  // extern "C"
