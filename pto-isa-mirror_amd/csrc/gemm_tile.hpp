// Tiled MFMA GEMM for gfx950: the TLOAD -> TMATMUL_ACC -> TSTORE pipeline of one PTO kernel as one HIP kernel.
//
//   TLOAD (GM -> L1 Mat tile)        128-bit coalesced global loads of a [rows][128 B] K-slab, staged into LDS
//   TMOV/TEXTRACT (L1 -> L0A/L0B)    ds_read_b128 of MFMA operand fragments from the swizzled LDS slab
//   TMATMUL / TMATMUL_ACC (Cube)     v_mfma_* on 32x32 (or 16x16) blocks, accumulators (the L0C Acc tile) live in registers
//   TSTORE (L0C -> GM, fix-pipe)     register epilogue: relu / dequant scales / f32->bf16|f16 RNE, then global stores
//
// Both operands are read K-contiguous: A is [M][K] row-major and B is [N][K] (Layout::DN).  A K-slab is 128 bytes per
// row whatever the element type (64 bf16/f16, 128 fp8/int8, 256 fp4), so one loader and one LDS layout serve all types.
// The LDS slab is double buffered: slab kt+1 is fetched into registers while slab kt is multiplied, then written to
// the other buffer; one __syncthreads per slab replaces the MTE2/MTE1/M event chain of the reference kernels
// (kernels/manual/a5/matmul_mxfp8_performance/mxmatmul_performance_kernel.cpp:115-150).
#pragma once
#include <type_traits>
#include "device_types.hpp"
#include "lds_dma.hpp"

namespace ptoamd {

// tile id that asks a launcher to give all its kernels their launch attributes on the current device and launch nothing
constexpr int TILE_PREPARE_ALL = -1000;

struct TileGemmParams {
    const uint8_t* a;       // [m][lda_bytes]
    const uint8_t* b;       // [n][ldb_bytes]
    void* c;                // [m][ldc] of the output type
    const void* c_in;       // optional accumulator input, [m][ldc] f32 / i32
    const void* bias;       // optional TMATMUL_BIAS row, [n] f32 / i32, added to every row after the K loop
    int32_t* acc_out;       // optional raw int32 accumulators (W8A8), [m][ldc]
    const uint8_t* sa;      // MX: [m][k/32] E8M0
    const uint8_t* sb;      // MX: [n][k/32] E8M0
    const float* row_scale; // W8A8: [m]
    const float* col_scale; // W8A8: [n]
    int m, n;
    int k_bytes;            // bytes per operand row that take part in the contraction
    long lda_bytes, ldb_bytes;
    int ldc;
    int scale_ld;           // MX: bytes per scale row (k / 32)
    int relu;               // bit 0: relu; bit 1: the fix-pipe's saturate-inf control (half / bfloat16 quantising drains)
    int out_kind;           // OutKind
    int group_m;            // tile-order grouping for L2 reuse
    int b_nd;               // register-staged tiles only: b is [k][ldb_bytes] (rows of N), transposed on the way into LDS
    int b_esz;              // element bytes of B (1 or 2) when b_nd is set
    // register-staged tiles only: how the E8M0 bytes of a tile row are laid out.  Every MX layout keeps the two scales of
    // a K-group pair adjacent: byte (x, g) of row / column x sits at base(x) + (g / 2) * pair_stride + g % 2.
    //   0  [X][K/32] (MX_A_ND, MX_B_DN): base = x * scale_ld, pair_stride 2 (plain rows; the DMA tiles need this one)
    //   1  16-row x 2-group boxes (MX_A_ZZ, MX_B_NN): base = (x / 16) * scale_ld * 16 + (x % 16) * 2, pair_stride 32
    //   2  pair-major (MX_A_DN, MX_B_ND): base = x * 2, pair_stride = 2 * rows (m for A, n for B)
    int sa_mode, sb_mode;
    // OUT_Q8 / OUT_QF16: the fix-pipe quantisation words of the drain, one for the whole matrix or one per column
    const uint64_t* qwords;
    int q_per_column;
    int atomic_add;         // OUT_F32 / OUT_I32 only: C += result with atomic adds (TSTORE<AtomicAdd>)
    // register-staged E4M3 x E4M3 tiles only: the operand arrives as packed fp4 codes (two per byte, even k in the low
    // nibble; lda_bytes / ldb_bytes are the packed row pitches, k_bytes counts elements) and the loader expands every
    // code to the E4M3 byte of the same value: 0 = no, 1 = E2M1, 2 = E1M2.  Every value of either fp4 format is an E4M3
    // value, and the scaled MFMA has no E1M2 operand format.
    int a_expand, b_expand;
};

__device__ __forceinline__ long mx_scale_base(int mode, int x, int scale_ld)
{
    return mode == 0 ? (long)x * scale_ld : (mode == 1 ? (long)(x >> 4) * scale_ld * 16 + (x & 15) * 2 : (long)x * 2);
}
__device__ __forceinline__ long mx_pair_stride(int mode, int rows) { return mode == 0 ? 2 : (mode == 1 ? 32 : 2L * rows); }

// OUT_Q8: one byte per element, signed or unsigned as the quantisation word says; OUT_QF16 / OUT_QBF16: half / bfloat16
// through the same words; OUT_QS16: int32 accumulators shifted right into int16 (the word's shift field)
enum OutKind { OUT_F32 = 0, OUT_F16 = 1, OUT_BF16 = 2, OUT_I32 = 3, OUT_W8A8_BF16 = 4, OUT_Q8 = 5, OUT_QF16 = 6, OUT_QBF16 = 7,
               OUT_QS16 = 8 };

// ---- MFMA operand traits ------------------------------------------------------------------------------------
// Every mma() hands the matrix instruction B's fragment as its first operand and A's as its second, so a 32x32
// accumulator block comes out transposed: lane (l32, lhi) holds row l32 of the block and register r its column
// 8 (r / 4) + 4 lhi + r % 4 -- four consecutive columns per register quad, which the epilogue packs into one 8- or
// 16-byte piece of an output row.  The sums themselves are the same (products commute, k runs in the same order).
// FRAG_BYTES: operand bytes one lane feeds one MFMA; a k-step spans 2 * FRAG_BYTES of a slab row (lanes 0-31 take
// the first half, lanes 32-63 the second), so a 128-byte slab is 128 / (2 * FRAG_BYTES) k-steps.
struct OpBF16 {
    static constexpr int BLK = 32, ACC_REGS = 16;
    using Acc = f32x16;
    using Elem = float;
    static constexpr int FRAG_BYTES = 16;
    static constexpr bool SCALED = false;
    static constexpr int GROUPS_PER_SLAB = 0;
    __device__ static __forceinline__ void mma(Acc& c, const uint4* a, const uint4* b, uint32_t, uint32_t)
    {
        c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, b[0]), __builtin_bit_cast(bf16x8, a[0]),
                                                    c, 0, 0, 0);
    }
    template <int SEL>
    __device__ static __forceinline__ void mma_sel(Acc& c, const uint4* a, const uint4* b, uint32_t sa, uint32_t sb)
    {
        mma(c, a, b, sa, sb);
    }
};
struct OpF16 {
    static constexpr int BLK = 32, ACC_REGS = 16;
    using Acc = f32x16;
    using Elem = float;
    static constexpr int FRAG_BYTES = 16;
    static constexpr bool SCALED = false;
    static constexpr int GROUPS_PER_SLAB = 0;
    __device__ static __forceinline__ void mma(Acc& c, const uint4* a, const uint4* b, uint32_t, uint32_t)
    {
        c = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, b[0]), __builtin_bit_cast(f16x8, a[0]), c,
                                                   0, 0, 0);
    }
    template <int SEL>
    __device__ static __forceinline__ void mma_sel(Acc& c, const uint4* a, const uint4* b, uint32_t sa, uint32_t sb)
    {
        mma(c, a, b, sa, sb);
    }
};
struct OpI8 {
    static constexpr int BLK = 32, ACC_REGS = 16;
    using Acc = i32x16;
    using Elem = int32_t;
    static constexpr int FRAG_BYTES = 16;
    static constexpr bool SCALED = false;
    static constexpr int GROUPS_PER_SLAB = 0;
    __device__ static __forceinline__ void mma(Acc& c, const uint4* a, const uint4* b, uint32_t, uint32_t)
    {
        c = __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(i32x4, b[0]), __builtin_bit_cast(i32x4, a[0]), c,
                                                  0, 0, 0);
    }
    template <int SEL>
    __device__ static __forceinline__ void mma_sel(Acc& c, const uint4* a, const uint4* b, uint32_t sa, uint32_t sb)
    {
        mma(c, a, b, sa, sb);
    }
};
// The same three operand types on the 16x16 matrix instructions (k = 32 elements of 16 bits, 64 of 8 bits): a block is
// 16 x 16, the four lane groups of 16 take consecutive 16-byte chunks, so a k-step spans 64 bytes of a slab row.  Lane
// (l % 16, l / 16) holds row l % 16 of the (transposed) block and its columns 4 (l / 16) .. + 3.  Per FLOP these
// instructions draw less power than the 32x32 forms: a loop of nothing but MFMAs on random operands sustains 1.97 GHz
// (bf16) and 2.18 GHz (int8) against 1.74 and 1.85 GHz, which is what bounds the large tiles.
struct OpBF16x16 {
    static constexpr int BLK = 16, ACC_REGS = 4;
    using Acc = f32x4;
    using Elem = float;
    static constexpr int FRAG_BYTES = 16;
    static constexpr bool SCALED = false;
    static constexpr int GROUPS_PER_SLAB = 0;
    __device__ static __forceinline__ void mma(Acc& c, const uint4* a, const uint4* b, uint32_t, uint32_t)
    {
        c = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, b[0]), __builtin_bit_cast(bf16x8, a[0]),
                                                    c, 0, 0, 0);
    }
    template <int SEL>
    __device__ static __forceinline__ void mma_sel(Acc& c, const uint4* a, const uint4* b, uint32_t sa, uint32_t sb)
    {
        mma(c, a, b, sa, sb);
    }
};
struct OpF16x16 {
    static constexpr int BLK = 16, ACC_REGS = 4;
    using Acc = f32x4;
    using Elem = float;
    static constexpr int FRAG_BYTES = 16;
    static constexpr bool SCALED = false;
    static constexpr int GROUPS_PER_SLAB = 0;
    __device__ static __forceinline__ void mma(Acc& c, const uint4* a, const uint4* b, uint32_t, uint32_t)
    {
        c = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, b[0]), __builtin_bit_cast(f16x8, a[0]), c,
                                                   0, 0, 0);
    }
    template <int SEL>
    __device__ static __forceinline__ void mma_sel(Acc& c, const uint4* a, const uint4* b, uint32_t sa, uint32_t sb)
    {
        mma(c, a, b, sa, sb);
    }
};
struct OpI8x16 {
    static constexpr int BLK = 16, ACC_REGS = 4;
    using Acc = i32x4;
    using Elem = int32_t;
    static constexpr int FRAG_BYTES = 16;
    static constexpr bool SCALED = false;
    static constexpr int GROUPS_PER_SLAB = 0;
    __device__ static __forceinline__ void mma(Acc& c, const uint4* a, const uint4* b, uint32_t, uint32_t)
    {
        c = __builtin_amdgcn_mfma_i32_16x16x64_i8(__builtin_bit_cast(i32x4, b[0]), __builtin_bit_cast(i32x4, a[0]), c,
                                                  0, 0, 0);
    }
    template <int SEL>
    __device__ static __forceinline__ void mma_sel(Acc& c, const uint4* a, const uint4* b, uint32_t sa, uint32_t sb)
    {
        mma(c, a, b, sa, sb);
    }
};
// fp8 (E4M3 = format 0, E5M2 = format 1) through the block-scaled MFMA; each lane's 32 bytes are one MX group.
// Without scale pointers both scales are 2^0 (E8M0 127) and the instruction is a plain fp8 TMATMUL.
template <int AFMT, int BFMT>
struct OpFP8 {
    static constexpr int BLK = 32, ACC_REGS = 16;
    using Acc = f32x16;
    using Elem = float;
    static constexpr int FRAG_BYTES = 32;
    static constexpr bool SCALED = true;
    static constexpr int GROUPS_PER_SLAB = 4;
    __device__ static __forceinline__ void mma(Acc& c, const uint4* a, const uint4* b, uint32_t sa, uint32_t sb)
    {
        i32x8 av, bv;
        av.s0 = a[0].x; av.s1 = a[0].y; av.s2 = a[0].z; av.s3 = a[0].w;
        av.s4 = a[1].x; av.s5 = a[1].y; av.s6 = a[1].z; av.s7 = a[1].w;
        bv.s0 = b[0].x; bv.s1 = b[0].y; bv.s2 = b[0].z; bv.s3 = b[0].w;
        bv.s4 = b[1].x; bv.s5 = b[1].y; bv.s6 = b[1].z; bv.s7 = b[1].w;
        c = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(bv, av, c, BFMT, AFMT, 0, (int)sb, 0, (int)sa);
    }
    // the scales are byte SEL of the dwords sa / sb (the instruction's own byte select: no VALU extraction)
    template <int SEL>
    __device__ static __forceinline__ void mma_sel(Acc& c, const uint4* a, const uint4* b, uint32_t sa, uint32_t sb)
    {
        i32x8 av, bv;
        av.s0 = a[0].x; av.s1 = a[0].y; av.s2 = a[0].z; av.s3 = a[0].w;
        av.s4 = a[1].x; av.s5 = a[1].y; av.s6 = a[1].z; av.s7 = a[1].w;
        bv.s0 = b[0].x; bv.s1 = b[0].y; bv.s2 = b[0].z; bv.s3 = b[0].w;
        bv.s4 = b[1].x; bv.s5 = b[1].y; bv.s6 = b[1].z; bv.s7 = b[1].w;
        c = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(bv, av, c, BFMT, AFMT, SEL, (int)sb, SEL, (int)sa);
    }
};
// The same operands on the 16x16x128 scaled MFMA: a lane holds 32 bytes of one of 16 rows, the whole 128-element K
// extent of a slab goes in one instruction, and each lane supplies one scale byte (lane group b: MX block b of the row).
template <int AFMT, int BFMT>
struct OpFP8x16 {
    static constexpr int BLK = 16, ACC_REGS = 4;
    using Acc = f32x4;
    using Elem = float;
    static constexpr int FRAG_BYTES = 32;
    static constexpr bool SCALED = true;
    static constexpr int GROUPS_PER_SLAB = 4;
    __device__ static __forceinline__ void mma(Acc& c, const uint4* a, const uint4* b, uint32_t sa, uint32_t sb)
    {
        i32x8 av, bv;
        av.s0 = a[0].x; av.s1 = a[0].y; av.s2 = a[0].z; av.s3 = a[0].w;
        av.s4 = a[1].x; av.s5 = a[1].y; av.s6 = a[1].z; av.s7 = a[1].w;
        bv.s0 = b[0].x; bv.s1 = b[0].y; bv.s2 = b[0].z; bv.s3 = b[0].w;
        bv.s4 = b[1].x; bv.s5 = b[1].y; bv.s6 = b[1].z; bv.s7 = b[1].w;
        c = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(bv, av, c, BFMT, AFMT, 0, (int)sb, 0, (int)sa);
    }
};
// 16 packed fp4 codes (8 bytes, even k in the low nibble) -> the 16 E4M3 bytes of the same values.  mode 1: E2M1
// (0, 0.5, 1, 1.5, 2, 3, 4, 6), mode 2: E1M2 (0, 0.25, ... 1.75); bit 3 of a code is the sign.
__device__ __forceinline__ uint4 expand_fp4_to_e4m3(uint2 x, int mode)
{
    const uint32_t lut_lo = mode == 1 ? 0x3C383000u : 0x34302800u;  // codes 0..3
    const uint32_t lut_hi = mode == 1 ? 0x4C484440u : 0x3E3C3A38u;  // codes 4..7
    uint32_t out[4];
    const uint32_t w[2] = {x.x, x.y};
#pragma unroll
    for (int d = 0; d < 2; ++d) {
        const uint32_t lo_n = w[d] & 0x0F0F0F0Fu, hi_n = (w[d] >> 4) & 0x0F0F0F0Fu;  // elements 0, 2, 4, 6 / 1, 3, 5, 7
        const uint32_t lo_e = __builtin_amdgcn_perm(lut_hi, lut_lo, lo_n & 0x07070707u) | ((lo_n & 0x08080808u) << 4);
        const uint32_t hi_e = __builtin_amdgcn_perm(lut_hi, lut_lo, hi_n & 0x07070707u) | ((hi_n & 0x08080808u) << 4);
        out[2 * d] = __builtin_amdgcn_perm(hi_e, lo_e, 0x05010400u);
        out[2 * d + 1] = __builtin_amdgcn_perm(hi_e, lo_e, 0x07030602u);
    }
    return make_uint4(out[0], out[1], out[2], out[3]);
}
template <class Op>
constexpr bool expands_fp4 = std::is_same<Op, OpFP8<0, 0>>::value;

// fp4 E2M1 (format 4): 32 elements = 16 bytes per lane = one MX group
struct OpFP4 {
    static constexpr int BLK = 32, ACC_REGS = 16;
    using Acc = f32x16;
    using Elem = float;
    static constexpr int FRAG_BYTES = 16;
    static constexpr bool SCALED = true;
    static constexpr int GROUPS_PER_SLAB = 8;
    __device__ static __forceinline__ void mma(Acc& c, const uint4* a, const uint4* b, uint32_t sa, uint32_t sb)
    {
        i32x8 av = {0, 0, 0, 0, 0, 0, 0, 0}, bv = {0, 0, 0, 0, 0, 0, 0, 0};
        av.s0 = a[0].x; av.s1 = a[0].y; av.s2 = a[0].z; av.s3 = a[0].w;
        bv.s0 = b[0].x; bv.s1 = b[0].y; bv.s2 = b[0].z; bv.s3 = b[0].w;
        c = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(bv, av, c, 4, 4, 0, (int)sb, 0, (int)sa);
    }
    template <int SEL>
    __device__ static __forceinline__ void mma_sel(Acc& c, const uint4* a, const uint4* b, uint32_t sa, uint32_t sb)
    {
        i32x8 av = {0, 0, 0, 0, 0, 0, 0, 0}, bv = {0, 0, 0, 0, 0, 0, 0, 0};
        av.s0 = a[0].x; av.s1 = a[0].y; av.s2 = a[0].z; av.s3 = a[0].w;
        bv.s0 = b[0].x; bv.s1 = b[0].y; bv.s2 = b[0].z; bv.s3 = b[0].w;
        c = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(bv, av, c, 4, 4, SEL, (int)sb, SEL, (int)sa);
    }
};

// 16-byte chunk swizzle inside a 128-byte slab row: consecutive rows land in different banks for ds_read_b128
__device__ __forceinline__ int swizzle_chunk(int row, int chunk) { return chunk ^ ((row >> 1) & 7) ^ ((row & 1) << 2); }

// Which 16-byte chunk of a slab row holds piece f of lane-half lhi's fragment for k-step s.
// 16-byte fragments: the two lane halves take consecutive chunks.  32-byte fp8 fragments of the 32x32x64 scaled MFMA:
// registers 0-3 of a lane belong to the k-step's first MX block (32 elements) and registers 4-7 to its second, each
// block being split 16 + 16 bytes over the two lane halves, while lane half h supplies the E8M0 scale of block h.
// (LG lane groups per wave: 2 for the 32x32 instructions, 4 for the 16x16 ones, which have 16-byte fragments only.)
template <int FR, int LG = 2>
__device__ __forceinline__ int frag_chunk(int s, int lhi, int f)
{
    if (FR == 1)
        return LG * s + lhi;
    return 4 * s + 2 * f + lhi;
}

// RING_: slabs the operand ring of the direct-to-LDS kernel holds (2: the copy-in of slab kt + 2 starts when slab kt is
// done with its buffer; 3: that of slab kt + 3, one more slab of time for it to land, for tiles whose slab is short).
template <int BM_, int BN_, int WAVES_M_, int WAVES_N_, class Op_, int RING_ = 2>
struct TileCfg {
    static constexpr int BM = BM_, BN = BN_, WAVES_M = WAVES_M_, WAVES_N = WAVES_N_, RING = RING_;
    using Op = Op_;
    static constexpr int THREADS = WAVES_M * WAVES_N * 64;
    static constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N;  // per-wave output tile
    static constexpr int BLK = Op::BLK, LG = 64 / BLK;            // MFMA block edge; lane groups of BLK lanes per wave
    static constexpr int MB = WTM / BLK, NB = WTN / BLK;          // MFMA blocks per wave
    static constexpr int SLAB = 128;                              // bytes of K per slab row
    static constexpr int KSTEPS = SLAB / (LG * Op::FRAG_BYTES);
    static constexpr int A_BYTES = BM * SLAB, B_BYTES = BN * SLAB, STAGE_BYTES = A_BYTES + B_BYTES;
    // the direct-to-LDS kernel of a block-scaled operand type keeps two buffers of 16 scale bytes per tile row behind
    // the operand ring
    static constexpr int SCALE_BYTES = Op::SCALED ? 2 * (BM + BN) * 16 : 0;
    static constexpr int LDS_BYTES = RING * STAGE_BYTES + SCALE_BYTES;
    static_assert(LDS_BYTES <= 160 * 1024, "the ring and the scale buffers fit the CU's LDS");
    static constexpr int LA = BM * 8 / THREADS, LB = BN * 8 / THREADS;  // 16-byte chunks per thread per slab
    static_assert(BM % (32 * WAVES_M) == 0 && BN % (32 * WAVES_N) == 0, "wave tiles are made of 32x32 blocks");
    static_assert(BLK == 32 || Op::FRAG_BYTES == 16 || Op::SCALED, "the plain 16x16 instructions take 16-byte fragments");
    static_assert((BM * 8) % THREADS == 0 && (BN * 8) % THREADS == 0, "slab chunks must divide over the workgroup");
};

// ---- TSTORE: drains one wave's accumulator blocks through the fix-pipe epilogue ------------------------------------
// The output kind and FULL (no bounds checks: the wave's tile lies inside the matrix) are run-time properties, but the
// dispatch on them sits *inside* the compile-time loop over 32x32 blocks: each variant then touches the 16 registers
// of one block only.  A dispatch around the whole loop keeps every accumulator live across the branch, which with 128
// or 256 accumulator registers per lane pushes them through scratch memory.  The TMATMUL_ACC input is folded in here:
// C = Cin + A.B.
// column (inside its 32x32 block) of accumulator register r of a lane in half lhi
// (a 16x16 block has one quad per lane: column 4 (lane / 16) + r)
template <int BLK = 32>
__device__ __forceinline__ constexpr int acc_col(int r, int lhi) { return BLK == 32 ? 8 * (r >> 2) + 4 * lhi + (r & 3) : 4 * lhi + r; }

// The optional terms (accumulator input, bias row, relu) are applied in passes over the block's 16 registers, one
// wave-uniform branch per term and block; tested per element they turn the epilogue into thousands of basic blocks,
// hundreds of KiB of code, and the instruction fetch -- not the stores -- sets its duration.
// gi: the lane's row of C; col_b: first column of the block.
// RELU: apply p.relu here (the quantising kinds clamp at zero after the quantisation instead).
template <bool FULL, bool RELU, class Cfg, class Acc>
__device__ __forceinline__ Acc tstore_terms(const TileGemmParams& p, Acc v, int gi, int col_b, int lhi,
                                             const typename Cfg::Op::Elem* bias_blk = nullptr)
{
    using Elem = typename Cfg::Op::Elem;
    const Elem* cin = reinterpret_cast<const Elem*>(p.c_in);
    // one branch per block when no term applies (the common case): a 16x16 block has four registers, and three
    // separate tests per block cost more than the block's conversions
    if (cin == nullptr && p.bias == nullptr && !(RELU && (p.relu & 1)))
        return v;
    if (cin != nullptr) {
#pragma unroll
        for (int r = 0; r < Cfg::Op::ACC_REGS; ++r) {
            const int gj = col_b + acc_col<Cfg::BLK>(r, lhi);
            if (FULL || (gi < p.m && gj < p.n))
                v[r] += cin[(long)gi * p.ldc + gj];
        }
    }
    if (p.bias != nullptr) {
#pragma unroll
        for (int r = 0; r < Cfg::Op::ACC_REGS; ++r) {
            const int gj = col_b + acc_col<Cfg::BLK>(r, lhi);
            if (bias_blk != nullptr)  // (a literal at every call site) the block's bias values, fetched by the caller
                v[r] += bias_blk[r];
            else if (FULL || gj < p.n)
                v[r] += reinterpret_cast<const Elem*>(p.bias)[gj];
        }
    }
    if (RELU && (p.relu & 1)) {
#pragma unroll
        for (int r = 0; r < Cfg::Op::ACC_REGS; ++r)
            v[r] = v[r] > 0 ? v[r] : 0;
    }
    return v;
}

// bits of one output element (1- and 2-byte kinds in the low part); W8A8: ((float)acc * scale_a[i]) * scale_b[j] -> bf16,
// each step rounded to f32; the quantising kinds: fix-pipe word `qw`, then relu
template <int KIND, class V>
__device__ __forceinline__ uint32_t tstore_bits(V v, float rs, float cs, uint64_t qw = 0, bool q_vector = false, int relu_flags = 0,
                                                int q16_kind = OUT_QF16)
{
    const bool relu = (relu_flags & 1) != 0, sat_inf = (relu_flags & 2) != 0;
    if (KIND == OUT_F32)
        return __builtin_bit_cast(uint32_t, (float)v);
    if (KIND == OUT_I32)
        return (uint32_t)(int32_t)v;
    if (KIND == OUT_F16)
        return f32_to_f16_bits((float)v);
    if (KIND == OUT_BF16)
        return f32_to_bf16_bits((float)v);
    constexpr bool src_int = std::is_same<V, int32_t>::value || std::is_same<V, int>::value;
    if (KIND == OUT_Q8) {
        float r = q_vector ? fixpipe_quantize<true, true, src_int>((float)v, qw) : fixpipe_quantize<false, true, src_int>((float)v, qw);
        if (relu)
            r = r > 0 ? r : 0;
        return (uint32_t)(int32_t)r & 0xFFu;
    }
    if (KIND == OUT_QF16) {
        // the three 16-bit targets of the quantiser share one instance; which one is a (uniform) run-time choice
        if (src_int && q16_kind == OUT_QS16) {
            int32_t r = fixpipe_shift_s16((int32_t)v, qw);
            if (relu)
                r = r > 0 ? r : 0;
            return (uint32_t)r & 0xFFFFu;
        }
        if (q16_kind == OUT_QBF16) {
            float r = __fmul_rn((float)v, q_vector ? fixpipe_word_scale<true>(qw) : fixpipe_word_scale<false>(qw));
            if (!src_int && sat_inf)
                r = fixpipe_saturate_inf<false>(r);
            if (relu)
                r = r > 0 ? r : 0;
            return f32_to_bf16_bits(r);
        }
        float r = q_vector ? fixpipe_quantize<true, false, src_int>((float)v, qw) : fixpipe_quantize<false, false, src_int>((float)v, qw);
        if (!src_int && sat_inf)
            r = fixpipe_saturate_inf<true>(r);
        if (relu)
            r = r > 0 ? r : 0;
        return (uint32_t)f32_to_f16_bits(r);
    }
    return f32_to_bf16_bits(__fmul_rn(__fmul_rn((float)v, rs), cs));
}
// The byte targets' quantisation word, decoded once: scale, offset and the lower clamp bound (the upper one is 255 above it).
struct ByteQuant {
    float scale, offset, lo;
};
template <bool VECTOR>
__device__ __forceinline__ ByteQuant decode_byte_quant(uint64_t word)
{
    return ByteQuant{fixpipe_word_scale<VECTOR>(word), (float)(uint32_t)((word >> 37) & 0x1FFu), ((word >> 46) & 1u) ? -128.0f : 0.0f};
}
// the same arithmetic as fixpipe_quantize<., true, .> followed by the relu and the narrowing of tstore_bits<OUT_Q8>
__device__ __forceinline__ uint32_t byte_quant_bits(float acc, const ByteQuant& q, bool relu)
{
    const float rounded = rintf(__fadd_rn(__fmul_rn(acc, q.scale), q.offset));
    const float hi = q.lo + 255.0f;
    float r = rounded < q.lo ? q.lo : (rounded > hi ? hi : rounded);
    if (relu)
        r = r > 0 ? r : 0;
    return (uint32_t)(int32_t)r & 0xFFu;
}
template <int KIND>
constexpr int out_bytes = (KIND == OUT_F32 || KIND == OUT_I32) ? 4 : (KIND == OUT_Q8 ? 1 : 2);
template <int KIND>
constexpr bool out_quant = KIND == OUT_Q8 || KIND == OUT_QF16;  // (OUT_QF16 instances also serve OUT_QBF16 and OUT_QS16)

// Element-wise form: any alignment, any edge.  A lane's elements are 4-column runs of one row, so this form is slow
// (short scattered stores); whole, aligned wave tiles take the staged form below.
template <int KIND, bool FULL, class Cfg, class Acc>
__device__ __forceinline__ void tstore_block(const TileGemmParams& p, const Acc& acc, int row_b, int col_b, int l32, int lhi)
{
    const int gi = row_b + l32;
    const float rs = (KIND == OUT_W8A8_BF16 && (FULL || gi < p.m)) ? p.row_scale[gi] : 1.0f;
    const Acc v = tstore_terms<FULL, !out_quant<KIND>, Cfg>(p, acc, gi, col_b, lhi);
    const bool raw = KIND == OUT_W8A8_BF16 && p.acc_out != nullptr;
#pragma unroll
    for (int r = 0; r < Cfg::Op::ACC_REGS; ++r) {
        const int gj = col_b + acc_col<Cfg::BLK>(r, lhi);
        if (FULL || (gi < p.m && gj < p.n)) {
            const long o = (long)gi * p.ldc + gj;
            const float cs = KIND == OUT_W8A8_BF16 ? p.col_scale[gj] : 1.0f;
            const uint64_t qw = out_quant<KIND> ? p.qwords[p.q_per_column ? gj : 0] : 0;
            const uint32_t bits = tstore_bits<KIND>(v[r], rs, cs, qw, p.q_per_column != 0, p.relu, p.out_kind);
            if (KIND == OUT_F32 && p.atomic_add)
                atomicAdd(reinterpret_cast<float*>(p.c) + o, __builtin_bit_cast(float, bits));
            else if (KIND == OUT_I32 && p.atomic_add)
                atomicAdd(reinterpret_cast<int*>(p.c) + o, (int)bits);
            else if (out_bytes<KIND> == 4)
                reinterpret_cast<uint32_t*>(p.c)[o] = bits;
            else if (out_bytes<KIND> == 2)
                reinterpret_cast<uint16_t*>(p.c)[o] = (uint16_t)bits;
            else
                reinterpret_cast<uint8_t*>(p.c)[o] = (uint8_t)bits;
            if (raw)
                p.acc_out[o] = (int32_t)v[r];
        }
    }
}

// float accumulators drain to f32 / f16 / bf16, int32 accumulators to int32 or (W8A8) scaled bf16: only those forms are
// compiled for an operand type (the host rejects the other combinations)
template <bool FULL, class Cfg, class Acc>
__device__ __forceinline__ void tstore_block_kind(const TileGemmParams& p, const Acc& acc, int row_b, int col_b, int l32, int lhi)
{
    if (p.out_kind == OUT_Q8) {
        tstore_block<OUT_Q8, FULL, Cfg>(p, acc, row_b, col_b, l32, lhi);
    } else if (p.out_kind >= OUT_QF16) {
        tstore_block<OUT_QF16, FULL, Cfg>(p, acc, row_b, col_b, l32, lhi);
    } else if constexpr (std::is_same<typename Cfg::Op::Elem, int32_t>::value) {
        if (p.out_kind == OUT_I32)
            tstore_block<OUT_I32, FULL, Cfg>(p, acc, row_b, col_b, l32, lhi);
        else
            tstore_block<OUT_W8A8_BF16, FULL, Cfg>(p, acc, row_b, col_b, l32, lhi);
    } else {
        switch (p.out_kind) {
            case OUT_F32: tstore_block<OUT_F32, FULL, Cfg>(p, acc, row_b, col_b, l32, lhi); break;
            case OUT_F16: tstore_block<OUT_F16, FULL, Cfg>(p, acc, row_b, col_b, l32, lhi); break;
            default: tstore_block<OUT_BF16, FULL, Cfg>(p, acc, row_b, col_b, l32, lhi); break;
        }
    }
}

// ---- TSTORE through LDS ------------------------------------------------------------------------------------------------
// A wave converts one 32-row band (one or two block rows) of its tile into a private, padded LDS region -- a lane writes its four consecutive
// columns of a register quad as one 8-byte (16-bit outputs) or 16-byte (32-bit outputs) piece -- reads the band back as
// 16-byte row chunks and stores whole row pieces of the wave tile's width.  LDS operations of one wave execute in
// order, so the region is reused for the next band without a barrier.
template <class Cfg>
struct StagedStore {
    // sized for 4-byte outputs; the 16 pad bytes per row keep the 32 rows a band's lanes write off each other's banks
    static constexpr int WAVE_BYTES = 32 * (Cfg::WTN * 4 + 16);
    static_assert(Cfg::THREADS / 64 * WAVE_BYTES <= Cfg::LDS_BYTES, "staging regions fit in the operand ring");
    static_assert((32 * Cfg::WTN / 16) % 64 == 0, "a band is a whole number of 64-lane reads, down to one-byte outputs");
};

// `stage` is the calling wave's private LDS region of StagedStore<Cfg>::WAVE_BYTES bytes.  The wave tile's columns lie
// inside the matrix (checked by the caller); its last rows may lie past row m - 1: they are computed on clamped row
// indices and not stored.  Rows of C need no alignment: a row piece leaves as 16-byte stores at whatever address it
// starts (the part takes unaligned vector stores; on 16-byte aligned rows they are whole 128-byte lines).
template <int KIND, class Cfg, class Acc>
__device__ __forceinline__ void tstore_staged(const TileGemmParams& p, Acc (&acc)[Cfg::MB][Cfg::NB], int row0, int col0,
                                              int l32, int lhi, uint8_t* stage)
{
    constexpr int ESZ = out_bytes<KIND>, BLK = Cfg::BLK;
    constexpr int BPB = 32 / BLK;  // block rows per 32-row band (two for the 16x16 instructions)
    constexpr int ROW_BYTES = Cfg::WTN * ESZ + 16, CHUNKS = Cfg::WTN * ESZ / 16, ITERS = 32 * CHUNKS / 64;
    const int lane = lhi * BLK + l32;
    // W8A8: a lane's column scales are the same for every block row of the wave tile; fetched once here (fetched where
    // they are used they are 128 separate loads per lane, and the store phase takes twice as long)
    // (nothing below may be scheduled up into the K loop's last slab, where every register is taken)
    __builtin_amdgcn_sched_barrier(0);
    // What depends on the column only is the same for every block row of the wave tile and is fetched once, up front:
    // fetched per block (with the blocks kept apart for register pressure) every block pays a load latency of its own.
    // (Only where a lane has at most 16 columns -- the 16x16 blocks of the large tile -- and one kind of item at a time:
    // next to 128 accumulator registers more than that spills.)
    using Elem = typename Cfg::Op::Elem;
    constexpr bool PRE = Cfg::NB * Cfg::Op::ACC_REGS <= 16;
    constexpr bool PRE_BIAS = PRE && !out_quant<KIND>, PRE_QW = PRE && out_quant<KIND>;
    Elem bias_pre[Cfg::NB][Cfg::Op::ACC_REGS];
    const bool has_bias = PRE_BIAS && p.bias != nullptr;
    if (has_bias) {
        static_for<Cfg::NB>([&](auto jc) {
            constexpr int j = decltype(jc)::value;
#pragma unroll
            for (int r = 0; r < Cfg::Op::ACC_REGS; ++r)
                bias_pre[j][r] = reinterpret_cast<const Elem*>(p.bias)[col0 + j * BLK + acc_col<BLK>(r, lhi)];
        });
    }
    // (byte targets keep the words decoded -- three floats per column instead of a 64-bit word taken apart per element)
    constexpr bool Q8 = KIND == OUT_Q8;
    uint64_t qw_pre[Cfg::NB][Cfg::Op::ACC_REGS];
    ByteQuant bq_pre[Cfg::NB][Cfg::Op::ACC_REGS];
    uint64_t qw0 = 0;
    ByteQuant bq0{};
    if constexpr (out_quant<KIND>) {
        qw0 = p.qwords[0];
        if (Q8 && !p.q_per_column)
            bq0 = decode_byte_quant<false>(qw0);
        if (PRE_QW && p.q_per_column) {
            static_for<Cfg::NB>([&](auto jc) {
                constexpr int j = decltype(jc)::value;
#pragma unroll
                for (int r = 0; r < Cfg::Op::ACC_REGS; ++r) {
                    const uint64_t w = p.qwords[col0 + j * BLK + acc_col<BLK>(r, lhi)];
                    if (Q8)
                        bq_pre[j][r] = decode_byte_quant<true>(w);
                    else
                        qw_pre[j][r] = w;
                }
            });
        }
    }
    float cs_pre[Cfg::NB][Cfg::Op::ACC_REGS], rs_pre[Cfg::MB];
    if constexpr (KIND == OUT_W8A8_BF16) {
#pragma unroll
        for (int i = 0; i < Cfg::MB; ++i)  // the row scales likewise: one load latency instead of one per block row
            rs_pre[i] = p.row_scale[min(row0 + i * BLK + l32, p.m - 1)];
        static_for<Cfg::NB>([&](auto jc) {
            constexpr int j = decltype(jc)::value;
#pragma unroll
            for (int r = 0; r < Cfg::Op::ACC_REGS; ++r)
                cs_pre[j][r] = p.col_scale[col0 + j * BLK + acc_col<BLK>(r, lhi)];
        });
    }
    static_for<Cfg::MB / BPB>([&](auto bc) {
        constexpr int band = decltype(bc)::value;
        static_for<BPB>([&](auto hc) {
            constexpr int i = band * BPB + decltype(hc)::value;
            const int srow = decltype(hc)::value * BLK + l32;  // row inside the band
            const int gi = min(row0 + i * BLK + l32, p.m - 1);
            const float rs = KIND == OUT_W8A8_BF16 ? rs_pre[i] : 1.0f;
            static_for<Cfg::NB>([&](auto jc) {
                constexpr int j = decltype(jc)::value;
                __builtin_amdgcn_sched_barrier(0);
                const int col_b = col0 + j * BLK;
                const Acc v = tstore_terms<true, !out_quant<KIND>, Cfg>(p, acc[i][j], gi, col_b, lhi,
                                                                      PRE_BIAS ? bias_pre[j] : nullptr);  // (read only where p.bias is set)
#pragma unroll
                for (int g = 0; g < Cfg::Op::ACC_REGS / 4; ++g) {
                    const int qc = acc_col<BLK>(4 * g, lhi);  // first of the quad's four columns
                    uint8_t* dst = stage + srow * ROW_BYTES + (j * BLK + qc) * ESZ;
                    if constexpr (KIND == OUT_BF16 || KIND == OUT_W8A8_BF16) {  // packed conversion: one instruction per pair
                        float f[4];
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            f[e] = (float)v[4 * g + e];
                            if (KIND == OUT_W8A8_BF16)
                                f[e] = __fmul_rn(__fmul_rn(f[e], rs), cs_pre[j][4 * g + e]);
                        }
                        *reinterpret_cast<uint2*>(dst) = make_uint2(f32x2_to_bf16x2_bits(f[0], f[1]), f32x2_to_bf16x2_bits(f[2], f[3]));
                    } else {
                        uint32_t bits[4];
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            if (Q8 && (PRE_QW || !p.q_per_column)) {
                                bits[e] = byte_quant_bits((float)v[4 * g + e], p.q_per_column ? bq_pre[j][4 * g + e] : bq0, (p.relu & 1) != 0);
                                continue;
                            }
                            const uint64_t qw = !out_quant<KIND> ? 0 : !p.q_per_column ? qw0 : (PRE_QW && !Q8) ? qw_pre[j][4 * g + e] : p.qwords[col_b + qc + e];
                            bits[e] = tstore_bits<KIND>(v[4 * g + e], rs, 1.0f, qw, p.q_per_column != 0, p.relu, p.out_kind);
                        }
                        if (ESZ == 4)
                            *reinterpret_cast<uint4*>(dst) = make_uint4(bits[0], bits[1], bits[2], bits[3]);
                        else if (ESZ == 2)
                            *reinterpret_cast<uint2*>(dst) = make_uint2(bits[0] | (bits[1] << 16), bits[2] | (bits[3] << 16));
                        else
                            *reinterpret_cast<uint32_t*>(dst) = bits[0] | (bits[1] << 8) | (bits[2] << 16) | (bits[3] << 24);
                    }
                }
            });
        });
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int it = 0; it < ITERS; ++it) {
            const int q = it * 64 + lane, row = q / CHUNKS, ch = q % CHUNKS;
            const uint4 v = *reinterpret_cast<const uint4*>(stage + row * ROW_BYTES + ch * 16);
            typedef unsigned int nt_u32x4 __attribute__((ext_vector_type(4), aligned(1)));
            nt_u32x4* dst = reinterpret_cast<nt_u32x4*>(reinterpret_cast<uint8_t*>(p.c) +
                                                        ((long)(row0 + band * 32 + row) * p.ldc + col0) * ESZ + ch * 16);
            const nt_u32x4 vv = {v.x, v.y, v.z, v.w};
            if (row0 + band * 32 + row < p.m)
                __builtin_nontemporal_store(vv, dst);  // C is not read again by this kernel: keep it out of the L2's way (plain stores end TSTORE
                                                   // 0.3 us sooner, but their write-backs cost the next launch 1 us)
        }
    });
}

// `stage`: the wave's private LDS region for the staged form, free of other uses from here on; nullptr = element-wise
template <class Cfg, class Acc>
__device__ __forceinline__ void tstore(const TileGemmParams& p, Acc (&acc)[Cfg::MB][Cfg::NB], int row0, int col0, int l32,
                                       int lhi, uint8_t* stage = nullptr)
{
    // the staged form takes wave tiles whose columns are all inside the matrix (rows past m - 1 are skipped row by row)
    const bool cols_inside = row0 < p.m && col0 + Cfg::WTN <= p.n;
    const bool raw_acc = p.out_kind == OUT_W8A8_BF16 && p.acc_out != nullptr;
    if (stage != nullptr && cols_inside && !p.atomic_add && !raw_acc) {
        if (p.out_kind >= OUT_QF16) {
            tstore_staged<OUT_QF16, Cfg>(p, acc, row0, col0, l32, lhi, stage);
        } else if (p.out_kind == OUT_Q8) {
            tstore_staged<OUT_Q8, Cfg>(p, acc, row0, col0, l32, lhi, stage);
        } else if constexpr (std::is_same<typename Cfg::Op::Elem, int32_t>::value) {
            if (p.out_kind == OUT_I32)
                tstore_staged<OUT_I32, Cfg>(p, acc, row0, col0, l32, lhi, stage);
            else
                tstore_staged<OUT_W8A8_BF16, Cfg>(p, acc, row0, col0, l32, lhi, stage);
        } else {
            switch (p.out_kind) {
                case OUT_F32: tstore_staged<OUT_F32, Cfg>(p, acc, row0, col0, l32, lhi, stage); break;
                case OUT_F16: tstore_staged<OUT_F16, Cfg>(p, acc, row0, col0, l32, lhi, stage); break;
                default: tstore_staged<OUT_BF16, Cfg>(p, acc, row0, col0, l32, lhi, stage); break;
            }
        }
        return;
    }
    static_for<Cfg::MB * Cfg::NB>([&](auto bc) {
        constexpr int i = decltype(bc)::value / Cfg::NB, j = decltype(bc)::value % Cfg::NB;
        // keep the address arithmetic of one 32x32 block from being hoisted over the others (register pressure)
        __builtin_amdgcn_sched_barrier(0);
        const Acc block = acc[i][j];
        // (bounds-checked also where the wave's tile lies inside the matrix: this form is store-bound either way, and a
        // second, unchecked copy of every output kind costs more compile time than it saves run time)
        tstore_block_kind<false, Cfg>(p, block, row0 + i * Cfg::BLK, col0 + j * Cfg::BLK, l32, lhi);
    });
}

// 16 bytes of a row starting at `g`, of which only the first `rem` belong to the row (rem >= 16: a whole chunk, at any
// alignment; rem <= 0: nothing, zeros).  A partial chunk is read as the 16 bytes ending at the row's end -- the row is at
// least 16 bytes long -- and shifted down by the bytes that precede the chunk.
__device__ __forceinline__ uint4 load_unaligned16(const uint8_t* g)
{
    uint32_t w[4];
    __builtin_memcpy(w, g, 16);  // one global_load_dwordx4: the target takes vector memory accesses at any alignment
    return make_uint4(w[0], w[1], w[2], w[3]);
}
__device__ __forceinline__ uint4 load_chunk_tail(const uint8_t* g, int rem)
{
    if (rem >= 16)
        return load_unaligned16(g);
    if (rem <= 0)
        return make_uint4(0, 0, 0, 0);
    const uint4 w = load_unaligned16(g + rem - 16);
    const uint64_t lo = ((uint64_t)w.y << 32) | w.x, hi = ((uint64_t)w.w << 32) | w.z;
    const int sh = (16 - rem) * 8;  // 8 .. 120 bits
    uint64_t rlo, rhi;
    if (sh >= 64) {
        rlo = hi >> (sh - 64);
        rhi = 0;
    } else {
        rlo = (lo >> sh) | (hi << (64 - sh));
        rhi = hi >> sh;
    }
    return make_uint4((uint32_t)rlo, (uint32_t)(rlo >> 32), (uint32_t)rhi, (uint32_t)(rhi >> 32));
}

// RAGGED: some row of A or B does not end on a 16-byte chunk boundary (see the loader below).  A compile-time form, so
// that the kernel for whole chunks carries neither the tail-masking code nor a branch in its K loop.
template <class Cfg, bool RAGGED>
__global__ void __launch_bounds__(Cfg::THREADS) gemm_tile_kernel(const TileGemmParams p)
{
    using Op = typename Cfg::Op;
    using Acc = typename Op::Acc;
    constexpr int BM = Cfg::BM, BN = Cfg::BN, MB = Cfg::MB, NB = Cfg::NB, LA = Cfg::LA, LB = Cfg::LB;
    constexpr int NT = Cfg::THREADS, FR = Op::FRAG_BYTES / 16;
    static_assert(Op::BLK == 32, "the register-staged tiles use the 32x32 instructions");
    extern __shared__ __align__(16) uint8_t smem[];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave % Cfg::WAVES_M, wn = wave / Cfg::WAVES_M;
    const int l32 = lane & 31, lhi = lane >> 5;

    // ---- workgroup -> output tile.  Workgroups are dealt round-robin to the 8 XCDs, so ids congruent mod 8 share an
    // L2; give each XCD a contiguous run of tiles and walk tiles in groups of group_m rows so a run reuses few panels.
    const int tiles_m = (p.m + BM - 1) / BM, tiles_n = (p.n + BN - 1) / BN;
    const int grid = tiles_m * tiles_n;
    int lid = blockIdx.x;
    if ((grid & 7) == 0)
        lid = (lid & 7) * (grid >> 3) + (lid >> 3);
    const int per_group = p.group_m * tiles_n;
    const int first_m = (lid / per_group) * p.group_m;
    const int gsize = min(tiles_m - first_m, p.group_m);
    const int tm = first_m + (lid % per_group) % gsize;
    const int tn = (lid % per_group) / gsize;
    const int m0 = tm * BM, n0 = tn * BN;

    // ---- TLOAD addressing: thread t moves chunk (t % 8) of rows t / 8 + i * NT / 8
    const int ld_chunk = tid & 7, ld_row = tid >> 3;
    const uint8_t* ga[LA];
    const uint8_t* gb[LB];
    int sa_off[LA], sb_off[LB];
    const int a_exp = expands_fp4<Op> ? p.a_expand : 0, b_exp = expands_fp4<Op> ? p.b_expand : 0;
#pragma unroll
    for (int i = 0; i < LA; ++i) {
        const int r = ld_row + i * (NT / 8);
        ga[i] = p.a + (long)min(m0 + r, p.m - 1) * p.lda_bytes + (a_exp ? ld_chunk * 8 : ld_chunk * 16);
        sa_off[i] = r * 128 + swizzle_chunk(r, ld_chunk) * 16;
    }
    // B as [N][K] (Layout::DN): the same chunks as A.  B as [K][N] (Layout::ND, p.b_nd): a 16-byte chunk holds EPC
    // consecutive columns of one k; the thread scatters its elements into the K-contiguous LDS rows of those columns,
    // so the slab in LDS, the fragment reads and the MFMA loop are the same for both layouts and no transposed copy
    // of B is made in global memory.  Chunk c of a slab: k = 8 * EPC * (c / BN) ... , see below.
    int b_koff[LB];          // byte offset (along K) of the chunk's first element inside a slab; huge = never loaded
    int sb_k[LB], sb_n[LB];  // b_nd: the chunk's k-chunk (0..7) and first column inside the tile
    const long b_slab_stride = p.b_nd ? (long)(128 / p.b_esz) * p.ldb_bytes : 128;
#pragma unroll
    for (int i = 0; i < LB; ++i) {
        const int r = ld_row + i * (NT / 8);
        if (!p.b_nd) {
            gb[i] = p.b + (long)min(n0 + r, p.n - 1) * p.ldb_bytes + (b_exp ? ld_chunk * 8 : ld_chunk * 16);
            sb_off[i] = Cfg::A_BYTES + r * 128 + swizzle_chunk(r, ld_chunk) * 16;
            b_koff[i] = ld_chunk * 16;
            sb_k[i] = sb_n[i] = 0;
        } else {
            const int epc = 16 / p.b_esz;  // elements per chunk = k rows per LDS chunk
            const int c = tid + i * NT;
            const int k_lo = c % epc, nc = (c / epc) % (BN / epc), k_hi = c / BN;
            const int krow = k_hi * epc + k_lo;
            const int cols_left = p.n - (n0 + nc * epc);  // columns of B from this chunk's first one on
            const bool inside = cols_left > 0;
            gb[i] = p.b + (long)krow * p.ldb_bytes + (long)(inside ? n0 + nc * epc : 0) * p.b_esz;
            sb_off[i] = Cfg::A_BYTES + nc * epc * 128 + k_lo * p.b_esz;
            b_koff[i] = inside ? krow * p.b_esz : (1 << 30);
            sb_k[i] = k_hi;
            sb_n[i] = nc * epc;
        }
    }
    const int k_slabs = (p.k_bytes + 127) / 128;

    uint4 ra[LA], rb[LB];
    // Rows need no alignment: a chunk is read with a 16-byte load at whatever address it starts (the part supports
    // unaligned global accesses).  Two forms of the slab load; the ragged one exists in the RAGGED kernel only and is
    // chosen there per slab by a workgroup-uniform test:
    //   whole   every chunk of the slab lies inside its row, or outside it as a whole (rows of whole 16-byte chunks);
    //   ragged  the row's last chunk holds fewer than 16 of the row's bytes (K * esz % 16 != 0; B row-major: N * esz % 16
    //           != 0): that chunk is read as the 16 bytes that END at the row's end and shifted down, so nothing past the
    //           row is touched (the bytes after a matrix's last row may not be mapped) and the lanes beyond K are zero.
    const bool ragged_k = (p.k_bytes & 15) != 0;
    const bool ragged_n = p.b_nd && (((long)p.n * p.b_esz) & 15) != 0;
    auto tload_whole = [&](int kt) {
        const bool live = kt * 128 + ld_chunk * 16 < p.k_bytes;  // partial last slab: missing chunks are zero
#pragma unroll
        for (int i = 0; i < LA; ++i) {
            if (expands_fp4<Op> && a_exp)
                ra[i] = live ? expand_fp4_to_e4m3(*reinterpret_cast<const uint2*>(ga[i] + (long)kt * 64), a_exp) : make_uint4(0, 0, 0, 0);
            else
                ra[i] = live ? load_unaligned16(ga[i] + (long)kt * 128) : make_uint4(0, 0, 0, 0);
        }
#pragma unroll
        for (int i = 0; i < LB; ++i) {
            if (expands_fp4<Op> && b_exp)  // (B is [N][K] here: the host sends row-major packed B elsewhere)
                rb[i] = live ? expand_fp4_to_e4m3(*reinterpret_cast<const uint2*>(gb[i] + (long)kt * 64), b_exp) : make_uint4(0, 0, 0, 0);
            else
                rb[i] = kt * 128 + b_koff[i] < p.k_bytes ? load_unaligned16(gb[i] + kt * b_slab_stride) : make_uint4(0, 0, 0, 0);
        }
    };
    auto tload_ragged = [&](int kt) {
        const int rem = p.k_bytes - (kt * 128 + ld_chunk * 16);  // bytes of the row from this chunk on; <= 0: none
#pragma unroll
        for (int i = 0; i < LA; ++i)
            ra[i] = load_chunk_tail(ga[i] + (long)kt * 128, rem);
#pragma unroll
        for (int i = 0; i < LB; ++i) {
            if (!p.b_nd) {
                rb[i] = load_chunk_tail(gb[i] + (long)kt * 128, rem);
            } else {  // a chunk of B's row k runs along N and ends with the row's columns
                const int epc = 16 / p.b_esz;
                const int nc = ((tid + i * NT) / epc) % (BN / epc);
                const int cols_left = p.n - (n0 + nc * epc);
                rb[i] = kt * 128 + b_koff[i] < p.k_bytes ? load_chunk_tail(gb[i] + kt * b_slab_stride, min(cols_left, epc) * p.b_esz)
                                                         : make_uint4(0, 0, 0, 0);
            }
        }
    };
    // (the fp4-expanding loads read 8-byte half chunks of rows that are whole slabs: never ragged)
    auto tload = [&](int kt) {
        if constexpr (RAGGED) {
            if (ragged_n || (ragged_k && (kt + 1) * 128 > p.k_bytes)) {
                tload_ragged(kt);
                return;
            }
        }
        tload_whole(kt);
    };
    auto stage = [&](int buf) {
        uint8_t* base = smem + buf * Cfg::STAGE_BYTES;
#pragma unroll
        for (int i = 0; i < LA; ++i)
            *reinterpret_cast<uint4*>(base + sa_off[i]) = ra[i];
        if (!p.b_nd) {
#pragma unroll
            for (int i = 0; i < LB; ++i)
                *reinterpret_cast<uint4*>(base + sb_off[i]) = rb[i];
        } else if (p.b_esz == 2) {
#pragma unroll
            for (int i = 0; i < LB; ++i) {
                const uint32_t w[4] = {rb[i].x, rb[i].y, rb[i].z, rb[i].w};
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    *reinterpret_cast<uint16_t*>(base + sb_off[i] + e * 128 + swizzle_chunk(sb_n[i] + e, sb_k[i]) * 16) =
                        (uint16_t)(w[e >> 1] >> (16 * (e & 1)));
            }
        } else {
#pragma unroll
            for (int i = 0; i < LB; ++i) {
                const uint32_t w[4] = {rb[i].x, rb[i].y, rb[i].z, rb[i].w};
#pragma unroll
                for (int e = 0; e < 16; ++e)
                    *(base + sb_off[i] + e * 128 + swizzle_chunk(sb_n[i] + e, sb_k[i]) * 16) = (uint8_t)(w[e >> 2] >> (8 * (e & 3)));
            }
        }
    };

    // ---- MX block scales: one E8M0 byte per row per 32 elements, fetched per slab straight into registers
    constexpr int SW = Op::SCALED ? Op::GROUPS_PER_SLAB / 4 : 1;  // dwords of scales per row per slab
    uint32_t sca[MB][SW], scb[NB][SW], sca_n[MB][SW], scb_n[NB][SW];
    const uint8_t* gsa[MB];
    const uint8_t* gsb[NB];
    const bool has_scales = Op::SCALED && p.sa != nullptr;
    const long spa = mx_pair_stride(p.sa_mode, p.m), spb = mx_pair_stride(p.sb_mode, p.n);
    if (has_scales) {
#pragma unroll
        for (int i = 0; i < MB; ++i)
            gsa[i] = p.sa + mx_scale_base(p.sa_mode, min(m0 + wm * Cfg::WTM + i * 32 + l32, p.m - 1), p.scale_ld);
#pragma unroll
        for (int j = 0; j < NB; ++j)
            gsb[j] = p.sb + mx_scale_base(p.sb_mode, min(n0 + wn * Cfg::WTN + j * 32 + l32, p.n - 1), p.scale_ld);
    }
    // the SW dwords (4 SW scale bytes) of slab kt of one row: one dword load per dword in the plain layout, two 2-byte
    // loads (one K-group pair each) in the others
    auto load_row_scales = [&](const uint8_t* row, int mode, long pair_stride, int kt, int w) -> uint32_t {
        if (mode == 0)
            return *reinterpret_cast<const uint32_t*>(row + (long)kt * (SW * 4) + w * 4);
        const long pair = (long)kt * (SW * 2) + w * 2;
        const uint32_t lo = *reinterpret_cast<const uint16_t*>(row + pair * pair_stride);
        const uint32_t hi = *reinterpret_cast<const uint16_t*>(row + (pair + 1) * pair_stride);
        return lo | (hi << 16);
    };
    auto load_scales = [&](int kt) {
        if (has_scales) {
#pragma unroll
            for (int w = 0; w < SW; ++w) {
#pragma unroll
                for (int i = 0; i < MB; ++i)
                    sca_n[i][w] = load_row_scales(gsa[i], p.sa_mode, spa, kt, w);
#pragma unroll
                for (int j = 0; j < NB; ++j)
                    scb_n[j][w] = load_row_scales(gsb[j], p.sb_mode, spb, kt, w);
            }
        }
    };

    // ---- Acc tile (L0C) in registers
    Acc acc[MB][NB];
#pragma unroll
    for (int i = 0; i < MB; ++i)
#pragma unroll
        for (int j = 0; j < NB; ++j) {
#pragma unroll
            for (int r = 0; r < 16; ++r)
                acc[i][j][r] = 0;
        }
    // ---- fragment addressing (TMOV/TEXTRACT): lane reads row l32 of a 32-row block, half lhi of the k-step
    int fa_row[MB], fb_row[NB];
#pragma unroll
    for (int i = 0; i < MB; ++i)
        fa_row[i] = wm * Cfg::WTM + i * 32 + l32;
#pragma unroll
    for (int j = 0; j < NB; ++j)
        fb_row[j] = wn * Cfg::WTN + j * 32 + l32;

    tload(0);
    load_scales(0);
    stage(0);
    __syncthreads();

    for (int kt = 0; kt < k_slabs; ++kt) {
        const int cur = kt & 1;
        if (has_scales) {
#pragma unroll
            for (int w = 0; w < SW; ++w) {
#pragma unroll
                for (int i = 0; i < MB; ++i)
                    sca[i][w] = sca_n[i][w];
#pragma unroll
                for (int j = 0; j < NB; ++j)
                    scb[j][w] = scb_n[j][w];
            }
        }
        if (kt + 1 < k_slabs) {
            tload(kt + 1);
            load_scales(kt + 1);
        }
        const uint8_t* sA = smem + cur * Cfg::STAGE_BYTES;
        const uint8_t* sB = sA + Cfg::A_BYTES;
#pragma unroll
        for (int s = 0; s < Cfg::KSTEPS; ++s) {
            uint4 fa[MB][FR], fb[NB][FR];
#pragma unroll
            for (int i = 0; i < MB; ++i)
#pragma unroll
                for (int f = 0; f < FR; ++f) {
                    const int chunk = frag_chunk<FR>(s, lhi, f);
                    fa[i][f] = *reinterpret_cast<const uint4*>(sA + fa_row[i] * 128 + swizzle_chunk(fa_row[i], chunk) * 16);
                }
#pragma unroll
            for (int j = 0; j < NB; ++j)
#pragma unroll
                for (int f = 0; f < FR; ++f) {
                    const int chunk = frag_chunk<FR>(s, lhi, f);
                    fb[j][f] = *reinterpret_cast<const uint4*>(sB + fb_row[j] * 128 + swizzle_chunk(fb_row[j], chunk) * 16);
                }
#pragma unroll
            for (int i = 0; i < MB; ++i)
#pragma unroll
                for (int j = 0; j < NB; ++j) {
                    uint32_t xa = 127u, xb = 127u;
                    if (has_scales) {
                        const int g = 2 * s + lhi;  // MX group of this lane inside the slab
                        xa = (sca[i][s >> 1] >> ((g & 3) * 8)) & 0xFFu;  // (2 s + lhi) >> 2 == s >> 1
                        xb = (scb[j][s >> 1] >> ((g & 3) * 8)) & 0xFFu;
                    }
                    Op::mma(acc[i][j], fa[i], fb[j], xa, xb);
                }
        }
        if (kt + 1 < k_slabs)
            stage(cur ^ 1);
        __syncthreads();
    }

    // ---- TSTORE: drain the accumulators through the epilogue (the ring is free after the loop's last barrier)
    tstore<Cfg>(p, acc, m0 + wm * Cfg::WTM, n0 + wn * Cfg::WTN, l32, lhi, smem + wave * StagedStore<Cfg>::WAVE_BYTES);
}

// One launcher per (tile shape, operand type); defined in gemm_tile_<op>.hip, called from gemm.hip.
// tile: 0 = 256x256 (8 waves), 1 = 128x128 (4 waves), 2 = 64x64 (4 waves)
enum TileOp { TOP_BF16 = 0, TOP_F16, TOP_I8, TOP_FP8_E4E4, TOP_FP8_E5E5, TOP_FP8_E4E5, TOP_FP8_E5E4, TOP_FP4, TOP_COUNT };
hipError_t launch_gemm_tile(int tile, int op, const TileGemmParams& p, hipStream_t stream);
void tile_shape(int tile, int* bm, int* bn);

}  // namespace ptoamd
