// Block-scaled fp8 GEMM tile on the 16x16x128 scaled MFMA: the direct-to-LDS kernel of gemm_tile_dtl.hpp re-cut for an
// instruction that consumes a whole 128-byte slab row per issue.
//
//   operands   v_mfma_scale_f32_16x16x128_f8f6f4: a lane holds 32 bytes of one row, as two 16-byte pieces.  Piece f of
//              lane group g (lanes 16 g .. 16 g + 15) is chunk 4 f + g of the slab row, and belongs to MX block
//              2 f + g / 2 (two lane groups share a block's 32 elements); the E8M0 scale of block b comes from the
//              lanes of group b.  One scale byte per lane and row block, read from the LDS scale rows as bytes
//              (16 rows x 16 bytes per read: no two rows share a bank).
//   registers  one set of fragments for the whole wave tile (MB + NB row blocks of 32 bytes per lane), refilled in
//              place: the MFMAs walk the accumulator blocks row by row, so A's row block i is free after its NB
//              MFMAs and B's blocks are free one by one in the last row.  Every refill reads the NEXT slab, so the
//              first MFMA of a slab never waits for LDS.
//   sync       one workgroup barrier per slab, in front of row BAR_ROW: behind it slab kt + 1 has landed and every
//              wave holds slab kt in registers, so the refills (slab kt + 1) and the DMAs of slab kt + 2 (into the
//              buffer slab kt occupied) follow it.  Rows in front of the barrier get their refills right after it.
#pragma once
#include "gemm_tile_dtl.hpp"

namespace ptoamd {

#ifndef PTOAMD_MX16_BAR_ROW
#define PTOAMD_MX16_BAR_ROW 2
#endif

template <class Cfg>
__global__ void __launch_bounds__(Cfg::THREADS) gemm_tile_mx16_kernel(const TileGemmParams p)
{
    using Op = typename Cfg::Op;
    using Acc = typename Op::Acc;
    constexpr int BM = Cfg::BM, BN = Cfg::BN, MB = Cfg::MB, NB = Cfg::NB, LA = Cfg::LA, LB = Cfg::LB;
    constexpr int NT = Cfg::THREADS, NMMA = MB * NB, NDMA = LA + LB, BAR_ROW = PTOAMD_MX16_BAR_ROW;
    static_assert(Cfg::BLK == 16 && Op::FRAG_BYTES == 32 && Cfg::KSTEPS == 1 && Cfg::RING == 2 && Op::SCALED,
                  "one 16x16x128 k-step per slab, two ring buffers");
    static_assert(BAR_ROW >= 0 && BAR_ROW < MB - 1, "the barrier sits in front of a row that is not the last");
    static_assert((NT / 8) % 16 == 0, "the swizzle of a lane's row must not depend on the piece index");
    extern __shared__ __align__(16) uint8_t smem[];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave % Cfg::WAVES_M, wn = wave / Cfg::WAVES_M;
    const int l16 = lane & 15, lg = lane >> 4;

    // tile order: as in gemm_tile_dtl_kernel (ids regrouped per XCD, then group_m tile rows at a time)
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

    // ---- TLOAD: 1 KiB pieces per wave, swizzled on the global-address side (the DMA writes lanes linearly).  The tile
    // lies inside the matrix (the launcher sends other shapes to the 32x32x64 form), so a piece is a scalar base --
    // 64 rows further down per piece -- plus one lane offset per operand.
    const int ld_row = tid >> 3;
    const int ld_chunk = swizzle_chunk(ld_row, tid & 7);
    const uint32_t goff_a = (uint32_t)((long)(m0 + ld_row) * p.lda_bytes + ld_chunk * 16);
    const uint32_t goff_b = (uint32_t)((long)(n0 + ld_row) * p.ldb_bytes + ld_chunk * 16);
    const int k_slabs = p.k_bytes / 128;
    const uint32_t lds_wave_base = __builtin_amdgcn_readfirstlane(lds_address(smem) + wave * 1024);
    auto tload_piece = [&](int kt, int buf, int q) __attribute__((always_inline)) {
        const uint32_t dst = lds_wave_base + buf * Cfg::STAGE_BYTES;
        if (q < LA)
            lds_dma16_off(p.a + (long)kt * 128 + (long)q * (NT / 8) * p.lda_bytes, goff_a, dst + q * (NT * 16));
        else
            lds_dma16_off(p.b + (long)kt * 128 + (long)(q - LA) * (NT / 8) * p.ldb_bytes, goff_b, dst + Cfg::A_BYTES + (q - LA) * (NT * 16));
    };
    auto tload = [&](int kt, int buf) __attribute__((always_inline)) {
#pragma unroll
        for (int q = 0; q < NDMA; ++q)
            tload_piece(kt, buf, q);
    };

    // ---- E8M0 scales: 16 bytes (four slabs' worth) of every tile row per DMA, two LDS buffers behind the ring
    constexpr int SPG = 4, SROWS = BM + BN, NSI = SROWS / 64, NW = NT / 64;
    static_assert(SROWS % 64 == 0 && BM % 64 == 0, "one scale DMA covers 64 rows of one operand");
    constexpr int SC_BASE = 2 * Cfg::STAGE_BYTES;
    const bool has_scales = p.sa != nullptr;
    static_assert(NSI == NW && BM / 64 == NW / 2, "one scale DMA per wave and chunk: the first half of the waves takes A's rows");
    const uint32_t lds_scales = lds_address(smem) + SC_BASE;
    const uint8_t* sc_base = wave < NW / 2 ? p.sa + (long)(m0 + wave * 64) * p.scale_ld
                                           : p.sb + (long)(n0 + (wave - NW / 2) * 64) * p.scale_ld;
    const uint32_t sc_lane = lane * p.scale_ld;
    auto tload_scales = [&](int g) __attribute__((always_inline)) {
        if (has_scales)
            lds_dma16_off(sc_base + (long)g * 16, sc_lane, lds_scales + (g & 1) * (SROWS * 16) + wave * 1024);
    };

    Acc acc[MB][NB];
#pragma unroll
    for (int i = 0; i < MB; ++i)
#pragma unroll
        for (int j = 0; j < NB; ++j)
#pragma unroll
            for (int r = 0; r < Op::ACC_REGS; ++r)
                acc[i][j][r] = 0;

    // ---- fragments and scales of the wave tile.  Row blocks are 16 rows = 2 KiB of slab apart, which leaves the
    // swizzle term (a function of row % 16) alone; piece 1 is piece 0's chunk XOR 4.
    // The lane addresses are running values: they point into the buffer (and the part of the scale rows) the next
    // refill reads, and move on when a slab's refills are all issued.
    uint32_t fa0 = (wm * Cfg::WTM + l16) * 128 + ((lg ^ swizzle_chunk(l16, 0)) << 4), fa1 = fa0 ^ 64u;
    uint32_t fb0 = Cfg::A_BYTES + (wn * Cfg::WTN + l16) * 128 + ((lg ^ swizzle_chunk(l16, 0)) << 4), fb1 = fb0 ^ 64u;
    // slab kt's part of a scale row: buffer (kt / 4) & 1, bytes 4 (kt % 4) .. + 3, the lane's MX block being byte lg
    auto scale_off = [&](int kt) { return ((kt / SPG) & 1) * (SROWS * 16) + (kt % SPG) * 4; };
    uint32_t sa_at = SC_BASE + (wm * Cfg::WTM + l16) * 16 + lg, sb_at = SC_BASE + (BM + wn * Cfg::WTN + l16) * 16 + lg;
    uint4 fa[MB][2], fb[NB][2];
    uint32_t sa[MB], sb[NB];
    auto read_a = [&](int i) __attribute__((always_inline)) {
        fa[i][0] = *reinterpret_cast<const uint4*>(smem + fa0 + i * (16 * 128));
        fa[i][1] = *reinterpret_cast<const uint4*>(smem + fa1 + i * (16 * 128));
        sa[i] = smem[sa_at + i * 256];
    };
    auto read_b = [&](int j) __attribute__((always_inline)) {
        fb[j][0] = *reinterpret_cast<const uint4*>(smem + fb0 + j * (16 * 128));
        fb[j][1] = *reinterpret_cast<const uint4*>(smem + fb1 + j * (16 * 128));
        sb[j] = smem[sb_at + j * 256];
    };
    // the refills after slab kt's are those of slab kt + 1, which read slab kt + 2
    auto advance_reads = [&](int kt) __attribute__((always_inline)) {
        const int d = ((kt + 2) & 1) ? Cfg::STAGE_BYTES : -Cfg::STAGE_BYTES;
        const int ds = scale_off(kt + 2) - scale_off(kt + 1);
        fa0 += d; fa1 += d; fb0 += d; fb1 += d;
        sa_at += ds; sb_at += ds;
    };

    // ---- prologue: slab 0 and the first scale chunk landed, slab 1 in flight, slab 0 in registers
    tload(0, 0);
    tload_scales(0);
    if (!has_scales) {  // without scale arrays every block has the scale 1 (E8M0 127)
        for (int o = tid * 16; o < 2 * SROWS * 16; o += NT * 16)
            *reinterpret_cast<uint4*>(smem + SC_BASE + o) = make_uint4(0x7F7F7F7Fu, 0x7F7F7F7Fu, 0x7F7F7F7Fu, 0x7F7F7F7Fu);
    }
    if (k_slabs > 1) {
        tload(1, 1);
        __builtin_amdgcn_s_waitcnt(0x0F70 | (NDMA & 15) | ((NDMA >> 4) << 14));  // vmcnt(NDMA): all but slab 1
    } else {
        __builtin_amdgcn_s_waitcnt(0x0F70);
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < NB; ++j)
        read_b(j);
#pragma unroll
    for (int i = 0; i < MB; ++i)
        read_a(i);
    advance_reads(-1);

    // One slab: `more` = slab kt + 1 exists (refill from it), `dma` = slab kt + 2 exists (copy it into the buffer this
    // slab leaves); literal at the call sites.
    auto slab = [&](int kt, int cur, bool more, bool dma) __attribute__((always_inline)) {
        // the next scale chunk overwrites the buffer whose last readers finished before the previous slab's barrier
        if (kt % SPG == 0 && (kt / SPG + 1) * SPG < k_slabs)
            tload_scales(kt / SPG + 1);
        static_for<NMMA>([&](auto xc) {
            constexpr int x = decltype(xc)::value;
            constexpr int i = x / NB, j = x % NB;
            if constexpr (x == BAR_ROW * NB) {
                // slab kt + 1 has landed (this wave's share; the barrier adds everyone else's), and every wave has
                // slab kt in registers.  The last slab keeps the barrier: behind it no wave reads the ring any more
                // and the epilogue may stage through it.
                __builtin_amdgcn_s_waitcnt(0x0F70);
                __syncthreads();
                if (more)
                    static_for<BAR_ROW>([&](auto rc) { read_a(decltype(rc)::value); });
            }
            Op::mma(acc[i][j], fa[i], fb[j], sa[i], sb[j]);
            // refills stay behind the MFMA that frees their registers
            __builtin_amdgcn_sched_barrier(0);
            if (more) {
                if constexpr (i == MB - 1)
                    read_b(j);
                if constexpr (j == NB - 1 && i >= BAR_ROW)
                    read_a(i);
            }
            if (dma) {
                // the copy-in of slab kt + 2, spread over the MFMAs behind the barrier
                constexpr int SPAN = NMMA - BAR_ROW * NB;
                constexpr int y = x - BAR_ROW * NB;
                if constexpr (y >= 0) {
                    constexpr int q0 = y * NDMA / SPAN, q1 = (y + 1) * NDMA / SPAN;
                    static_for<q1 - q0>([&](auto qc) { tload_piece(kt + 2, cur, q0 + decltype(qc)::value); });
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        });
        if (more)
            advance_reads(kt);
    };
    int kt = 0;
    for (; kt + 2 < k_slabs; ++kt)
        slab(kt, kt & 1, true, true);
    if (kt + 1 < k_slabs) {
        slab(kt, kt & 1, true, false);
        ++kt;
    }
    slab(kt, kt & 1, false, false);

    tstore<Cfg>(p, acc, m0 + wm * Cfg::WTM, n0 + wn * Cfg::WTN, l16, lg, smem + wave * StagedStore<Cfg>::WAVE_BYTES);
}

}  // namespace ptoamd
