// Tiled MFMA GEMM, direct-to-LDS form: the steady-state kernel for shapes whose K extent is a whole number of
// 128-byte slabs.  Same tile instructions as gemm_tile.hpp, different engines:
//
//   TLOAD      global_load_lds_dwordx4: each wave DMAs 1 KiB pieces of the next K-slab straight into the LDS ring
//              (no register staging); the bank swizzle is applied on the global-address side, because the DMA
//              writes lanes linearly.
//   TEXTRACT   operand fragments of k-step s+1 are read (ds_read_b128) while the MFMAs of k-step s run; two register
//              sets alternate, so the matrix pipe never waits on LDS inside a slab.
//   sync       one workgroup barrier per slab, placed before the last k-step: by then every wave has drained its reads
//              of the current slab (so it can be overwritten by slab kt+2) and its DMA of slab kt+1 has landed, and the
//              last k-step's MFMAs cover the first fragment reads of slab kt+1.  This replaces the four-flag
//              MTE2/MTE1/M hand-shake of the reference kernels.
#pragma once
#include <type_traits>
#include <utility>

#include "gemm_tile.hpp"
#include "lds_dma.hpp"

namespace ptoamd {

// Scheduling recipe for one k-step: NM MFMAs interleaved evenly with ND LDS reads (next k-step's fragments) and NV
// LDS-DMA issues (a later slab).  Without it the compiler shortens the fragment live ranges, re-uses the registers and
// puts the reads right in front of the MFMAs that need them, which exposes the LDS latency on every k-step.
template <int I, int NM, int ND, int NV>
struct SchedKStep {
    __device__ static __forceinline__ void run()
    {
        constexpr int nd = (I + 1) * ND / NM - I * ND / NM;
        constexpr int nv = (I + 1) * NV / NM - I * NV / NM;
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // one MFMA
        if constexpr (nd > 0)
            __builtin_amdgcn_sched_group_barrier(0x100, nd, 0);  // LDS reads
        if constexpr (nv > 0)
            __builtin_amdgcn_sched_group_barrier(0x020, nv, 0);  // VMEM reads (LDS-DMA)
        SchedKStep<I + 1, NM, ND, NV>::run();
    }
};
template <int NM, int ND, int NV>
struct SchedKStep<NM, NM, ND, NV> {
    __device__ static __forceinline__ void run() {}
};
template <int NM, int ND, int NV>
__device__ __forceinline__ void sched_kstep()
{
    SchedKStep<0, NM, ND, NV>::run();
}

// DMA issue plan.  A slab's copy-in can start only when the barrier before the last k-step of slab kt has freed the
// buffer, and must have landed by the same barrier of slab kt + 1.  Issuing all of it in that one k-step makes a burst
// the CU's 64 B/clk global -> LDS path cannot absorb (64 one-KiB DMAs need ~1000 clocks, twice the k-step), and the
// MFMAs queued behind the stalled DMA instructions wait.  So a share of the pieces is held back for the first k-step
// of the following slab: measured on the bf16 4096^3 GEMM, (8) 112.7 us, (6, 2) and (4, 4) 110.7 us (int8 alike),
// anything issued later than that first k-step loses again (the data has less time to land), and so does any split
// for the 32-byte-fragment types whose slab has only two k-steps (fp8: 109 -> 112 us), which keep the single phase.  Shares are eighths of the slab's pieces
// per phase: phase 0 = the last k-step of the slab that frees the buffer, phase f > 0 = k-step f - 1 of the next slab.
#ifndef PTOAMD_DMA_PHASES
#define PTOAMD_DMA_PHASES 4, 4
#endif
// The 16x16 instructions' slab has two long k-steps (32 MFMAs of a 128 x 64 wave tile each); their phase 1 is the FIRST
// HALF of the next slab's first k-step, half a k-step ahead of the barrier that needs the data.
#ifndef PTOAMD_DMA_PHASES_16
#define PTOAMD_DMA_PHASES_16 8
#endif
// (ONE_PHASE: rings deeper than two slabs have a whole slab of slack and issue everything in phase 0)
template <int NDMA, int KS, int BLK = 32, bool ONE_PHASE = false>
__host__ __device__ constexpr int dma_phase_begin(int phase)
{
    if (ONE_PHASE)
        return phase >= 1 ? NDMA : 0;
    constexpr int share32[] = {PTOAMD_DMA_PHASES};
    constexpr int share16[] = {PTOAMD_DMA_PHASES_16};
    constexpr int n = BLK == 16 ? sizeof(share16) / sizeof(share16[0]) : sizeof(share32) / sizeof(share32[0]);
    int eighths = 0;
    for (int f = 0; f < phase && f < n; ++f)
        eighths += BLK == 16 ? share16[f] : share32[f];
    // two k-steps per slab of the 32x32 instructions (fp8): phase 1 would be the k-step before the barrier
    if (phase >= n || phase >= KS || (KS < 4 && BLK == 32 && phase >= 1))
        eighths = 8;
    return eighths * NDMA / 8;
}

// RAGGED: K is not a whole number of 128-byte slabs (and at least one).  The last slab's copy-in then goes lane by
// lane: a chunk that lies inside its row is DMAed as always, the chunk the row ends in is read through registers as the
// 16 bytes that END at the row's end (nothing past a row is touched) and written to the lane's LDS position with the
// bytes past K zero, and chunks past K are written as zeros -- so the MFMAs run over a whole slab and the products
// beyond K vanish.  A compile-time form: the kernel for whole slabs carries none of it.  Its slabs go out in one DMA
// phase, so that a slab is requested in exactly one place.
template <class Cfg, bool RAGGED = false>
__global__ void __launch_bounds__(Cfg::THREADS) gemm_tile_dtl_kernel(const TileGemmParams p)
{
    static_assert(!RAGGED || (Cfg::RING == 2 && !Cfg::Op::SCALED), "the ragged-K form exists for the two-slab ring of the plain types");
    using Op = typename Cfg::Op;
    using Acc = typename Op::Acc;
    constexpr int BM = Cfg::BM, BN = Cfg::BN, MB = Cfg::MB, NB = Cfg::NB, LA = Cfg::LA, LB = Cfg::LB;
    constexpr int NT = Cfg::THREADS, FR = Op::FRAG_BYTES / 16, KS = Cfg::KSTEPS, RING = Cfg::RING;
    static_assert(KS % 2 == 0, "fragment register sets alternate per k-step");
    static_assert((NT / 8) % 16 == 0, "the swizzle of a lane's row must not depend on the piece index");
    extern __shared__ __align__(16) uint8_t smem[];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: keeps the tile bookkeeping in scalar registers
    const int wm = wave % Cfg::WAVES_M, wn = wave / Cfg::WAVES_M;
    // l32: the lane's row inside an MFMA block (32 or 16 rows), lhi: its lane group (0-1 or 0-3)
    constexpr int BLK = Cfg::BLK, LG = Cfg::LG;
    const int l32 = lane % BLK, lhi = lane / BLK;

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

    // ---- TLOAD addressing.  Piece i of a slab is rows i * NT/8 .. + NT/8; lane `tid` lands at LDS position
    // (row = tid / 8, slot = tid % 8) of the piece and therefore fetches logical chunk slot ^ swizzle(row).
    const int ld_row = tid >> 3;
    const int ld_chunk = swizzle_chunk(ld_row, tid & 7);
    uint32_t goff_a[LA], goff_b[LB];
#pragma unroll
    for (int i = 0; i < LA; ++i)
        goff_a[i] = (uint32_t)((long)min(m0 + ld_row + i * (NT / 8), p.m - 1) * p.lda_bytes + ld_chunk * 16);
#pragma unroll
    for (int i = 0; i < LB; ++i)
        goff_b[i] = (uint32_t)((long)min(n0 + ld_row + i * (NT / 8), p.n - 1) * p.ldb_bytes + ld_chunk * 16);
    const int k_slabs = RAGGED ? (p.k_bytes + 127) / 128 : p.k_bytes / 128;

    const uint32_t lds_wave_base = __builtin_amdgcn_readfirstlane(lds_address(smem) + wave * 1024);
    // DMA number q (0 .. LA + LB - 1) of slab kt into ring buffer buf
    auto tload_piece = [&](int kt, int buf, int q) __attribute__((always_inline)) {
        const uint32_t dst = lds_wave_base + buf * Cfg::STAGE_BYTES;
        if (q < LA)
            lds_dma16_off(p.a + (long)kt * 128, goff_a[q], dst + q * (NT * 16));
        else
            lds_dma16_off(p.b + (long)kt * 128, goff_b[q - LA], dst + Cfg::A_BYTES + (q - LA) * (NT * 16));
    };
    // the same for the last slab of a ragged K (see RAGGED above)
    auto tload_piece_last = [&](int buf, int q) __attribute__((always_inline)) {
        const int kt = k_slabs - 1;
        const int rem = p.k_bytes - kt * 128 - ld_chunk * 16;  // bytes of the lane's row from its chunk on
        const bool is_a = q < LA;
        const int piece = is_a ? q : q - LA;
        const int lds_off = buf * Cfg::STAGE_BYTES + (is_a ? 0 : Cfg::A_BYTES) + piece * (NT * 16);
        const uint8_t* base = (is_a ? p.a : p.b) + (long)kt * 128;
        const uint32_t goff = is_a ? goff_a[piece] : goff_b[piece];
        if (rem >= 16)
            lds_dma16_off(base, goff, lds_wave_base + lds_off);
        else
            *reinterpret_cast<uint4*>(smem + lds_off + tid * 16) = load_chunk_tail(base + goff, rem);
    };
    auto tload = [&](int kt, int buf) __attribute__((always_inline)) {
        if (RAGGED && kt == k_slabs - 1) {
#pragma unroll
            for (int q = 0; q < LA + LB; ++q)
                tload_piece_last(buf, q);
            return;
        }
#pragma unroll
        for (int q = 0; q < LA + LB; ++q)
            tload_piece(kt, buf, q);
    };

    // ---- MX block scales.  A lane needs the E8M0 bytes of its own rows, 4 (fp8) or 8 (fp4) per row per slab; fetched
    // per lane from global memory they are 64 separate small requests per load instruction and keep the CU's address
    // unit busier than the operand DMAs do.  Instead the 16 scale bytes of every row of the tile -- SPG slabs' worth --
    // are DMAed into one of two LDS scale buffers, one instruction per 64 rows, and each wave reads the dwords of its
    // rows from there.  Chunk g + 1 is requested when slab g * SPG starts and read from the last k-step of
    // slab (g + 1) * SPG - 1 on, i.e. at least one slab barrier (with its vmcnt(0)) later.
    constexpr int GPS = Op::SCALED ? Op::GROUPS_PER_SLAB : 4;  // scale bytes per row per slab
    constexpr int SW = GPS / 4, SPG = 16 / GPS;
    constexpr int SROWS = BM + BN, NSI = SROWS / 64, NW = NT / 64, NSW = (NSI + NW - 1) / NW;
    static_assert(SROWS % 64 == 0 && BM % 64 == 0, "one scale DMA covers 64 rows of one operand");
    // The scale dwords of slab kt + 1 are read one k-step ahead (after slab kt's barrier), so that the slab's first
    // MFMA does not wait for an LDS round trip.  PTOAMD_SCALES_AT_SLAB_START reads them when the slab starts instead
    // (one register set fewer) for the 32-byte fragments of a large wave tile.
#ifdef PTOAMD_SCALES_AT_SLAB_START
    constexpr bool SC_AHEAD = !(Op::FRAG_BYTES == 32 && MB * NB >= 8);
#else
    constexpr bool SC_AHEAD = true;
#endif
    uint32_t sca[MB][SW], scb[NB][SW], sca_n[MB][SW], scb_n[NB][SW];
    const bool has_scales = Op::SCALED && p.sa != nullptr;
#pragma unroll
    for (int w = 0; w < SW; ++w) {
#pragma unroll
        for (int i = 0; i < MB; ++i)
            sca_n[i][w] = 0x7F7F7F7Fu;
#pragma unroll
        for (int j = 0; j < NB; ++j)
            scb_n[j][w] = 0x7F7F7F7Fu;
    }
    const uint8_t* sc_src[NSW];
    const uint32_t lds_scales = lds_address(smem) + RING * Cfg::STAGE_BYTES;
    if (has_scales) {
#pragma unroll
        for (int w = 0; w < NSW; ++w) {
            const int r = (wave + w * NW) * 64 + lane;  // row of [A rows | B rows]; past the end for idle waves (unused)
            sc_src[w] = r < BM ? p.sa + (long)min(m0 + r, p.m - 1) * p.scale_ld
                               : p.sb + (long)min(n0 + max(r - BM, 0), p.n - 1) * p.scale_ld;
        }
    }
    auto tload_scales = [&](int g) __attribute__((always_inline)) {
        if (has_scales) {
#pragma unroll
            for (int w = 0; w < NSW; ++w) {
                const int i = wave + w * NW;
                if (i < NSI)
                    lds_dma16(sc_src[w] + (long)g * 16, lds_scales + (g & 1) * (SROWS * 16) + i * 1024);
            }
        }
    };
    // slab kt's scales of this lane's rows, LDS -> sca_n / scb_n
    // (No test of has_scales here: a branch between two k-steps lets the compiler sink the earlier k-step's MFMAs
    // below it, away from the fragment reads they should overlap.  Without scale arrays the LDS scale area is filled
    // with E8M0 127 once, in the prologue.)
    auto read_scales = [&](int kt) __attribute__((always_inline)) {
        if (Op::SCALED) {
            const uint8_t* base = smem + RING * Cfg::STAGE_BYTES + ((kt / SPG) & 1) * (SROWS * 16) + (kt % SPG) * GPS;
#pragma unroll
            for (int w = 0; w < SW; ++w) {
#pragma unroll
                for (int i = 0; i < MB; ++i)
                    sca_n[i][w] = *reinterpret_cast<const uint32_t*>(base + (wm * Cfg::WTM + i * BLK + l32) * 16 + w * 4);
#pragma unroll
                for (int j = 0; j < NB; ++j)
                    scb_n[j][w] = *reinterpret_cast<const uint32_t*>(base + (BM + wn * Cfg::WTN + j * BLK + l32) * 16 + w * 4);
            }
        }
    };

    // ---- Acc tile
    Acc acc[MB][NB];
#pragma unroll
    for (int i = 0; i < MB; ++i)
#pragma unroll
        for (int j = 0; j < NB; ++j)
#pragma unroll
            for (int r = 0; r < Op::ACC_REGS; ++r)
                acc[i][j][r] = 0;
    // ---- fragment addressing.  A lane reads row l32 of every block of its wave tile; blocks are BLK * 128 bytes
    // apart and the swizzle depends on row % 16 only, so one lane-constant per operand serves all blocks: the byte
    // offset of (row, chunk lhi ^ swizzle).  Chunk c = c0 + lhi with c0 a multiple of the lane-group count, and
    // (c0 + lhi) ^ swz = c0 ^ (lhi ^ swz), so the address of chunk c is that constant XOR (c0 << 4): one VALU op per
    // k-step piece, shared by the blocks.
    static_assert(Cfg::WTM % 32 == 0 && Cfg::WTN % 32 == 0, "wave tiles start on 32-row boundaries");
    const uint32_t fa_lane = (wm * Cfg::WTM + l32) * 128 + ((lhi ^ swizzle_chunk(l32, 0)) << 4);
    const uint32_t fb_lane = Cfg::A_BYTES + (wn * Cfg::WTN + l32) * 128 + ((lhi ^ swizzle_chunk(l32, 0)) << 4);
    // Two fragment register sets (next k-step's reads overlap this k-step's MFMAs).  Where 32-byte fragments of a large
    // wave tile would not fit the register file twice next to the accumulators (HYBRID), only the fragments that stay
    // live until the end of a k-step get a second copy -- all of B and A's last row block; the other A row blocks are
    // refilled in place right after their last MFMA, several MFMAs before the next k-step reads them.  16 waves
    // (128 registers per lane) keep one set, refilled piecewise, and the SIMD's other waves cover the LDS latency.
    // (The hybrid read schedule needs one first-column MFMA per double-buffered fragment, NB + 1 <= MB; the square wave
    // tile of the 4-wave form has accumulators for 16 blocks and keeps the single set.)
    constexpr bool BIG_FRAGS = (MB + NB) * FR >= 12;  // 48 or more registers per fragment set
    constexpr bool HYBRID = BIG_FRAGS && NT <= 512 && NB + 1 <= MB;
    constexpr int SETS = (NT > 512 || (BIG_FRAGS && !HYBRID)) ? 1 : 2;
    uint4 fa[SETS][MB][FR], fb[SETS][NB][FR];
    constexpr int NREAD = (MB + NB) * FR, NMMA = MB * NB, NDMA = LA + LB;
    // fragment read number q of k-step s of ring buffer buf into register set `set`; B fragments come first because the
    // first MFMAs of a k-step need all of B's first block but only A's first
    auto textract_piece = [&](int set, int buf, int s, int q) __attribute__((always_inline)) {
        const uint8_t* base = smem + buf * Cfg::STAGE_BYTES;
        if (q < NB * FR) {
            const int j = q / FR, f = q % FR;
            fb[set][j][f] = *reinterpret_cast<const uint4*>(base + (fb_lane ^ (frag_chunk<FR, LG>(s, 0, f) << 4)) + j * (BLK * 128));
        } else {
            const int i = (q - NB * FR) / FR, f = (q - NB * FR) % FR;
            fa[set][i][f] = *reinterpret_cast<const uint4*>(base + (fa_lane ^ (frag_chunk<FR, LG>(s, 0, f) << 4)) + i * (BLK * 128));
        }
    };
    // One k-step: the MFMAs of step s (register set s & 1), with the fragment reads of the next step (register set
    // (s + 1) & 1, from buffer rbuf step rs) and, in a slab's last step, the DMAs of slab dkt spread between them.
    auto kstep = [&](auto phase, int s, bool reads, int rbuf, int rs, bool dmas, int dkt, int dbuf, auto lastdma) __attribute__((always_inline)) {
        constexpr int PH = decltype(phase)::value;
        constexpr bool LASTDMA = decltype(lastdma)::value;  // the DMAs of this k-step are those of a ragged K's last slab
        constexpr int DQ0 = dma_phase_begin<NDMA, KS, BLK, (Cfg::RING > 2 || RAGGED)>(PH), DN = dma_phase_begin<NDMA, KS, BLK, (Cfg::RING > 2 || RAGGED)>(PH + 1) - DQ0;
        constexpr int DSPAN = (BLK == 16 && PH > 0) ? NMMA / 2 : NMMA;  // MFMAs the phase's DMAs are spread over
        const int set = SETS == 2 ? (s & 1) : 0;
        const int nset = SETS == 2 ? (set ^ 1) : 0;
        static_for<NMMA>([&](auto xc) {
            constexpr int x = decltype(xc)::value;
            constexpr int i = x / NB, j = x % NB;
            const int aset = (HYBRID && i != MB - 1) ? 0 : set;  // register set of A's row block i
            // MX group 2 s + lhi of the slab lives in dword s >> 1 (either lane half) at byte 2 (s & 1) + lhi; the
            // dwords were shifted right by 8 lhi when the slab started, so both halves select byte 2 (s & 1) and the
            // instruction's own byte select does the extraction.  Without scale arrays every byte is E8M0 127.
            if (s & 1)
                Op::template mma_sel<2>(acc[i][j], fa[aset][i], fb[set][j], sca[i][s >> 1], scb[j][s >> 1]);
            else
                Op::template mma_sel<0>(acc[i][j], fa[aset][i], fb[set][j], sca[i][s >> 1], scb[j][s >> 1]);
            if (reads) {
                if constexpr (HYBRID) {
                    // pinned behind the MFMA that frees the registers (hoisted above it the refill would need a second
                    // copy after all).  First-column MFMAs 0 .. NB - 1 are followed by the next step's B blocks and
                    // MFMA NB by A's last row block, into the other set; a row's last MFMA by that row's refill.
                    __builtin_amdgcn_sched_barrier(0);
                    if constexpr (j == 0 && i < NB)
                        static_for<FR>([&](auto fc) { textract_piece(nset, rbuf, rs, i * FR + decltype(fc)::value); });
                    if constexpr (j == 0 && i == NB)
                        static_for<FR>([&](auto fc) { textract_piece(nset, rbuf, rs, NB * FR + (MB - 1) * FR + decltype(fc)::value); });
                    if constexpr (j == NB - 1 && i < MB - 1)
                        static_for<FR>([&](auto fc) { textract_piece(0, rbuf, rs, NB * FR + i * FR + decltype(fc)::value); });
                    __builtin_amdgcn_sched_barrier(0);
                } else if constexpr (SETS == 2) {
                    constexpr int q0 = x * NREAD / NMMA, q1 = (x + 1) * NREAD / NMMA;
                    static_for<q1 - q0>([&](auto qc) { textract_piece(nset, rbuf, rs, q0 + decltype(qc)::value); });
                } else {
                    // keep the refill behind the MFMA that frees the registers: hoisted above it, the reads would need a
                    // second set of fragment registers after all
                    __builtin_amdgcn_sched_barrier(0);
                    if constexpr (j == NB - 1)  // row i of A is free once its last MFMA has issued
                        static_for<FR>([&](auto fc) { textract_piece(0, rbuf, rs, NB * FR + i * FR + decltype(fc)::value); });
                    if constexpr (x == NMMA - 1)  // B is free after the last MFMA
                        static_for<NB * FR>([&](auto qc) { textract_piece(0, rbuf, rs, decltype(qc)::value); });
                }
            }
            if (dmas) {
                constexpr int xa = x < DSPAN ? x : DSPAN, xb = x + 1 < DSPAN ? x + 1 : DSPAN;
                constexpr int q0 = DQ0 + xa * DN / DSPAN, q1 = DQ0 + xb * DN / DSPAN;
                static_for<q1 - q0>([&](auto qc) {
                    if constexpr (LASTDMA)
                        tload_piece_last(dbuf, q0 + decltype(qc)::value);
                    else
                        tload_piece(dkt, dbuf, q0 + decltype(qc)::value);
                });
            }
        });
        if constexpr (SETS == 2 && !HYBRID)
            sched_kstep<NMMA, NREAD, 0>();
    };

    // ---- prologue: slabs 0 and 1 in flight, first fragments in registers
    tload(0, 0);
    tload_scales(0);
    if (Op::SCALED && !has_scales) {
        for (int o = tid * 16; o < 2 * SROWS * 16; o += NT * 16)
            *reinterpret_cast<uint4*>(smem + RING * Cfg::STAGE_BYTES + o) = make_uint4(0x7F7F7F7Fu, 0x7F7F7F7Fu, 0x7F7F7F7Fu, 0x7F7F7F7Fu);
    }
    // slab 1's first DMAs go out now but only slab 0 (and the scales) are waited for: the counter retires loads in
    // order, so "at most N1 outstanding" means everything issued before slab 1's pieces has landed; slab 1 is covered
    // by the first slab's barrier
    constexpr int N1 = dma_phase_begin<NDMA, KS, BLK, (Cfg::RING > 2 || RAGGED)>(1);
    // A deeper ring starts slabs 1 .. RING - 1 whole as well (it is built for the types whose slab goes out in one
    // phase), so that from the first slab on the copy-in runs RING - 1 slabs ahead.  At the barrier of slab kt the ring
    // may leave WAITN DMAs in flight: those of the slabs after kt + 1, but no more than were issued after the scale
    // chunk that is read at that barrier (requested SPG - 1 slabs earlier).
    static_assert(RING == 2 || N1 == NDMA, "rings deeper than two slabs issue a slab's DMAs in one phase");
    constexpr int WAITN = RING == 2 ? 0 : ((RING - 2 < SPG - 1 || !Op::SCALED) ? RING - 2 : SPG - 1) * NDMA;
    static_assert(WAITN < 64 && (RING - 1) * NDMA < 64, "vmcnt is a 6-bit count");
    if (RING > 2 && k_slabs >= RING) {
        static_for<RING - 1>([&](auto sc) { tload(decltype(sc)::value + 1, decltype(sc)::value + 1); });
        constexpr int W0 = (RING - 1) * NDMA;
        __builtin_amdgcn_s_waitcnt(0x0F70 | (W0 & 15) | ((W0 >> 4) << 14));  // slab 0 and the scales have landed
    } else if (RING > 2) {
        for (int s1 = 1; s1 < k_slabs; ++s1)
            tload(s1, s1);
        __builtin_amdgcn_s_waitcnt(0x0F70);
    } else if (RAGGED && k_slabs > 1) {
        tload(1, 1);  // (one phase: N1 = NDMA; slab 1 may be the ragged last one, whose register-loaded chunks are not DMAs)
        __builtin_amdgcn_s_waitcnt(0x0F70);
    } else if (k_slabs > 1) {
        static_for<N1>([&](auto qc) { tload_piece(1, 1, decltype(qc)::value); });
        __builtin_amdgcn_s_waitcnt(0x0F70 | (N1 & 15) | ((N1 >> 4) << 14));  // vmcnt(N1)
    } else {
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this wave's DMAs have landed
    }
    __syncthreads();
#pragma unroll
    for (int q = 0; q < NREAD; ++q)
        textract_piece(0, 0, 0, q);
    read_scales(0);

    // One slab.  `more` = slab kt+1 exists (read its first fragments in the last k-step), `dma` = slab kt+2 exists
    // (start its DMA into the buffer this slab frees); both are literal at the call sites so the branches fold.
    // (always_inline: out of line, a lambda takes the accumulators by reference and they live in scratch memory)
    // `cur` / `nxt`: ring buffers of slab kt and kt + 1; slab kt + RING - 1 ... goes into the buffer slab kt frees.
    // `steady`: slabs kt + 1 .. kt + RING - 1 are all in flight or landed (the barrier may then leave WAITN DMAs pending).
    auto slab = [&](int kt, int cur, bool more, bool dma, auto steady, auto lastdma) __attribute__((always_inline)) {
        const int nxt = RING == 2 ? (cur ^ 1) : (cur + 1 == RING ? 0 : cur + 1);
        if (Op::SCALED) {
            // The request for the next scale chunk sits here, at the top of the slab, and not between two k-steps: a
            // branch between them splits the slab into basic blocks, and the compiler then sinks the first k-step's
            // MFMAs (pure register operations) below the barrier into the block that uses their results, where they
            // no longer overlap the fragment reads.  The buffer it overwrites was last read a whole slab ago (every
            // wave has passed the previous slab's barrier, and consumed those scale dwords before it).
            if (kt % SPG == 0 && (kt / SPG + 1) * SPG < k_slabs)
                tload_scales(kt / SPG + 1);
            if constexpr (!SC_AHEAD)
                read_scales(kt);
#pragma unroll
            for (int w = 0; w < SW; ++w) {
#pragma unroll
                for (int i = 0; i < MB; ++i)
                    sca[i][w] = sca_n[i][w] >> (8 * lhi);
#pragma unroll
                for (int j = 0; j < NB; ++j)
                    scb[j][w] = scb_n[j][w] >> (8 * lhi);
            }
        }
        static_for<KS - 1>([&](auto sc) {
            constexpr int s = decltype(sc)::value;
            kstep(std::integral_constant<int, s + 1>{}, s, true, cur, s + 1, more, kt + 1, nxt, std::false_type{});
        });
        // every wave is done reading slab kt, and its DMAs of slab kt+1 (issued RING - 1 slabs ago) have landed
        constexpr int WN = decltype(steady)::value ? WAITN : 0;
        __builtin_amdgcn_s_waitcnt(0x0F70 | (WN & 15) | ((WN >> 4) << 14));  // vmcnt(WN)
        __syncthreads();
        if (SC_AHEAD && more)
            read_scales(kt + 1);
        kstep(std::integral_constant<int, 0>{}, KS - 1, more, nxt, 0, dma, kt + RING, cur, lastdma);
    };
    int kt = 0, cur = 0;
    if constexpr (RING == 2) {
        // (ragged K: the slab that requests the last one is peeled off the loop)
        for (; kt + (RAGGED ? 3 : 2) < k_slabs; ++kt)
            slab(kt, kt & 1, true, true, std::true_type{}, std::false_type{});
        if constexpr (RAGGED) {
            if (kt + 2 < k_slabs) {
                slab(kt, kt & 1, true, true, std::true_type{}, std::true_type{});
                ++kt;
            }
        }
        if (kt + 1 < k_slabs) {
            slab(kt, kt & 1, true, false, std::false_type{}, std::false_type{});
            ++kt;
        }
        slab(kt, kt & 1, false, false, std::false_type{}, std::false_type{});
    } else {
        const auto advance = [&]() {
            ++kt;
            cur = cur + 1 == RING ? 0 : cur + 1;
        };
        while (kt + RING < k_slabs) {
            slab(kt, cur, true, true, std::true_type{}, std::false_type{});
            advance();
        }
        // the last RING slabs (or fewer): nothing more to start; the barrier waits for everything in flight
        while (kt + 1 < k_slabs) {
            slab(kt, cur, true, false, std::false_type{}, std::false_type{});
            advance();
        }
        slab(kt, cur, false, false, std::false_type{}, std::false_type{});
    }

    // ---- TSTORE.  No wave reads the ring after the last slab's barrier (its fragment reads were issued before it) and
    // no DMA is in flight, so each wave may reuse a piece of it for the staged store without another barrier.
    tstore<Cfg>(p, acc, m0 + wm * Cfg::WTM, n0 + wn * Cfg::WTN, l32, lhi, smem + wave * StagedStore<Cfg>::WAVE_BYTES);
}

}  // namespace ptoamd
