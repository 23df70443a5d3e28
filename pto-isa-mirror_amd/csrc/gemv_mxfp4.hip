// Decode-shaped weight-only MXFP4 GEMV/GEMM (m <= 16): out[m][n] = sum_k A[m][k] * (e2m1 W[n][k] * 2^(sw[n][k/32]-127)).
//
// The shape is HBM-bound (every weight byte is read once, ~60 FLOP per byte).  What limits a streaming read on this
// memory system is the shape of each wave's load: 16 rows x 64 bytes per instruction (the natural MFMA operand
// pattern) tops out near 3.4 TB/s, 512 contiguous bytes per half wave reaches 5+ TB/s.  Two kernels:
//
//   * split-K (k % 1024 == 0, the decode shapes): a workgroup of 8 waves owns a run of 16-row strips; wave s owns
//     k-slice s (1024 k) of every strip and keeps its activation fragments for that slice in registers for the whole
//     kernel (128 VGPRs, loaded once).  Weights and scales stream global -> LDS by LDS-DMA into a per-wave
//     double-buffered region (512 contiguous bytes per row, two rows per instruction, no VGPRs, no barriers: a wave
//     reads back only what it wrote), are re-read as MFMA operand fragments (16 bytes = one MX group per lane, feeding
//     four MFMAs; row pairs padded and odd rows half-swapped on the global side, so the reads are conflict-free),
//     dequantised in registers and multiplied on
//     v_mfma_f32_16x16x32_bf16.  The 8 k-slice partials of a strip are summed through LDS in a fixed order.
//   * streaming (k % 512 == 0 otherwise): a wave owns 16 rows over the full K, register prefetch four chunks deep,
//     activations staged per chunk through LDS.
// Dequantisation: v_cvt_scalef32_pk_bf16_fp4 (fp4 pair * 2^e -> bf16 pair, exact).
#include "common_host.hpp"
#include "device_types.hpp"
#include "lds_dma.hpp"

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
    const uint8_t* wp;  // packed weights (gemv_mxfp4_pack_kernel), loader-wave kernel only: w and sw are then unused
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

// ---- split-K kernel -------------------------------------------------------------------------------------------
constexpr int SK_SLICE = 1024;                     // k per wave slice
constexpr int SK_WAVES = 8;
constexpr int SK_RMAX = 8;                         // strips whose accumulators a wave holds at once
constexpr int SK_PAIR = 2 * (SK_SLICE / 2) + 16;   // LDS bytes of a row pair: 2 x 512 plus one 16-byte pad
constexpr int SK_WBYTES = 8 * SK_PAIR;             // one strip's weight slice: 16 rows x 512 bytes (+ pads)
constexpr int SK_SBYTES = 16 * (SK_SLICE / 32);    // and its scales: 16 rows x 32 bytes
constexpr int SK_STAGE = SK_WBYTES + SK_SBYTES;
constexpr int SK_WAVE_LDS = 2 * SK_STAGE;          // double buffer, private to the wave
constexpr int SK_LDS = SK_WAVES * SK_WAVE_LDS;     // 138 KiB of the CU's 160 KiB
constexpr int SK_VM_PER_STRIP = 10;                // LDS-DMA instructions per strip: 8 weight + 2 scale
static_assert(SK_RMAX * 64 * 16 <= SK_WAVE_LDS, "a wave's partial sums reuse its own staging region");

// ksw = 1 << ksw_log2 waves share one strip's K (wave & (ksw - 1) = first k-slice, then every ksw-th);
// 8 / ksw row groups work on different strips.  Workgroup b owns strips [b * strips_per_wg, (b + 1) * strips_per_wg).
template <bool HW_CVT>
__global__ void __launch_bounds__(SK_WAVES * 64) gemv_mxfp4_splitk_kernel(const GemvParams p, int ksw_log2, int strips_per_wg)
{
    extern __shared__ __align__(16) uint8_t smem[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l16 = lane & 15, q = lane >> 4;
    const int ksw = 1 << ksw_log2, rgs = SK_WAVES >> ksw_log2;
    const int slice = wave & (ksw - 1), rg = wave >> ksw_log2;
    const int s_begin = blockIdx.x * strips_per_wg, s_end = min(s_begin + strips_per_wg, p.n_groups);
    const int ks = p.k / SK_SLICE, sb = p.k / 32;
    uint8_t* my = smem + wave * SK_WAVE_LDS;
    const uint32_t my_lds = lds_address(my);
    // k-assignment inside a 1024-k slice: MFMA step (j, t), j < 8, t < 4, multiplies k = 32 (4 j + q) + 8 t .. + 7 in lane
    // quarter q, so a lane's 16-byte weight read (one MX group = chunk 4 j + q of the row) feeds the four steps t.
    // Rows sit in LDS as pairs (2 x 512 bytes + 16 pad) with the 128-byte halves of odd rows swapped (chunk ^ 8):
    //   weights      chunk 4 j + q of row l16 is at (j & 2 ? wread1 : wread0) + 64 j
    //   activations  piece 16 jj + 4 q + t of a quarter (jj < 2) is at aread + 16 (16 jj + t)
    const int lrow = (l16 >> 1) * SK_PAIR + (l16 & 1) * 512;
    const int wread0 = lrow + 16 * q + 128 * (l16 & 1), wread1 = lrow + 16 * q - 128 * (l16 & 1);
    const int aread = lrow + (((4 * q) ^ (8 * (l16 & 1))) << 4);
    const int mine = s_end > s_begin + rg ? (s_end - s_begin - rg + rgs - 1) / rgs : 0;  // strips of this row group
    const int most = (s_end - s_begin + rgs - 1) / rgs;                                   // ... of row group 0

    for (int b0 = 0; b0 < most; b0 += SK_RMAX) {
        const int cnt = max(0, min(SK_RMAX, mine - b0));
        f32x4 acc[SK_RMAX];
#pragma unroll
        for (int i = 0; i < SK_RMAX; ++i)
            acc[i] = f32x4{0, 0, 0, 0};

        for (int kb = slice; kb < ks && cnt > 0; kb += ksw) {
            // 16 rows x 512 bytes -> one LDS stage.  One LDS-DMA moves a row pair (2 x 512 contiguous bytes); pairs are
            // 16 bytes apart in LDS and odd rows swap their 128-byte halves (chunk ^ 8), so that the fragment reads
            // below are conflict-free with lane-constant base addresses.  Addresses are a wave-uniform base plus a
            // 32-bit lane offset; rows past rlim re-read row rlim.
            auto issue_rows = [&](const uint8_t* base, uint32_t row_bytes, int rlim, uint32_t dst, int ln) {
                const int hi = ln >> 5;
                const uint32_t chunk_off = ((ln & 31) ^ (8 * hi)) * 16;
#pragma unroll
                for (int d = 0; d < 8; ++d)
                    lds_dma16_off(base, __umul24(min(2 * d + hi, rlim), row_bytes) + chunk_off, dst + d * SK_PAIR);
            };
            // weight strip i of the batch (and its scales) -> buffer i & 1
            auto issue = [&](int i) {
                const int strip = s_begin + rg + rgs * (b0 + i);
                const int rlim = min(15, p.n - 1 - strip * 16);
                const uint8_t* wbase = p.w + (long)strip * 16 * p.ldw_bytes + kb * (SK_SLICE / 2);
                const uint8_t* sbase = p.sw + (long)strip * 16 * sb + kb * (SK_SLICE / 32);
                const uint32_t dst = my_lds + (i & 1) * SK_STAGE;
                // (the lane id is made opaque here so that these few VALU ops are redone per strip rather than
                // precomputed for all strips of the batch and parked in scratch memory)
                int ln = lane;
                asm volatile("" : "+v"(ln));
                issue_rows(wbase, (uint32_t)p.ldw_bytes, rlim, dst, ln);
#pragma unroll
                for (int d = 0; d < 2; ++d)
                    lds_dma4_off(sbase, __umul24(min(8 * d + (ln >> 3), rlim), (uint32_t)sb) + (ln & 7) * 4,
                                 dst + SK_WBYTES + d * 256);
            };
            // activation quarter j (256 k of the slice, 16 rows x 512 bytes) -> buffer j & 1; rows past m - 1 re-read
            // row m - 1 (their output rows are never stored)
            auto issue_a = [&](int j) {
                int ln = lane;
                asm volatile("" : "+v"(ln));
                issue_rows(reinterpret_cast<const uint8_t*>(p.a) + (long)kb * (SK_SLICE * 2) + j * 512, (uint32_t)p.lda * 2,
                           p.m - 1, my_lds + (j & 1) * SK_STAGE, ln);
            };

            // Activation fragments of this k-slice: areg[4 j + t] holds A[m = l16][32 (4 j + q) + 8 t .. + 7].  Loading
            // them straight from global memory would make 64 separate 16-byte requests per instruction (the row index
            // is the fast lane index); instead the four quarters (256 k each) run through the same LDS-DMA pipeline as
            // the weight strips, ahead of them.
            uint4 areg[32];
            issue_a(0);
            issue_a(1);
            static_for<4>([&](auto jc) {
                constexpr int j = decltype(jc)::value;
                if (j < 3 || cnt > 0)
                    __builtin_amdgcn_s_waitcnt(0x0F70 | (j < 3 ? 8 : SK_VM_PER_STRIP));  // all but the next stage's DMAs
                else
                    __builtin_amdgcn_s_waitcnt(0x0F70);
                asm volatile("" ::: "memory");
                const uint8_t* buf = my + (j & 1) * SK_STAGE;
#pragma unroll
                for (int x = 0; x < 8; ++x)  // x = 4 jj + t: the fragment of step (2 j + jj, t)
                    areg[8 * j + x] = *reinterpret_cast<const uint4*>(buf + aread + 16 * (16 * (x >> 2) + (x & 3)));
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                if (j + 2 < 4)
                    issue_a(j + 2);
                else if (j - 2 < cnt)
                    issue(j - 2);
            });
            static_for<SK_RMAX>([&](auto ic) {
                constexpr int i = decltype(ic)::value;
                if (i < cnt) {
                    // LDS-DMAs retire in issue order: strip i is complete once only strip i + 1's are outstanding
                    if (i + 1 < cnt)
                        __builtin_amdgcn_s_waitcnt(0x0F70 | SK_VM_PER_STRIP);
                    else
                        __builtin_amdgcn_s_waitcnt(0x0F70);
                    asm volatile("" ::: "memory");
                    const uint8_t* buf = my + (i & 1) * SK_STAGE;
                    const uint4 sc0 = *reinterpret_cast<const uint4*>(buf + SK_WBYTES + l16 * 32);
                    const uint4 sc1 = *reinterpret_cast<const uint4*>(buf + SK_WBYTES + l16 * 32 + 16);
                    const uint32_t sc[8] = {sc0.x, sc0.y, sc0.z, sc0.w, sc1.x, sc1.y, sc1.z, sc1.w};
                    static_for<2>([&](auto hc) {
                        constexpr int h = decltype(hc)::value;
                        uint4 wv[4];
#pragma unroll
                        for (int jj = 0; jj < 4; ++jj) {  // MX group 4 j + q of the slice, j = 4 h + jj
                            const int j = 4 * h + jj;
                            wv[jj] = *reinterpret_cast<const uint4*>(buf + ((j & 2) ? wread1 : wread0) + 64 * j);
                        }
                        if (h == 1) {
                            // the buffer is refilled only after every read of it has returned
                            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                            if (i + 2 < cnt)
                                issue(i + 2);
                        }
#pragma unroll
                        for (int jj = 0; jj < 4; ++jj) {
                            const int j = 4 * h + jj;
                            const float scale = e8m0_to_f32((sc[j] >> (8 * q)) & 0xFFu);  // scale byte 4 j + q
                            const uint32_t xs[4] = {wv[jj].x, wv[jj].y, wv[jj].z, wv[jj].w};
#pragma unroll
                            for (int t = 0; t < 4; ++t) {
                                const uint4 w8 = dequant8<HW_CVT>(xs[t], scale);
                                acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, areg[4 * j + t]),
                                                                                __builtin_bit_cast(bf16x8, w8), acc[i], 0, 0, 0);
                            }
                        }
                    });
                }
            });
        }

        // sum the k-slice partials of each strip in slice order; every wave parks its accumulators in its own region
        f32x4* part = reinterpret_cast<f32x4*>(my);
#pragma unroll
        for (int i = 0; i < SK_RMAX; ++i)
            part[i * 64 + lane] = acc[i];
        __syncthreads();
        for (int idx = tid; idx < rgs * SK_RMAX * 64; idx += SK_WAVES * 64) {
            const int rg2 = idx / (SK_RMAX * 64), i = (idx >> 6) & (SK_RMAX - 1), ln = idx & 63;
            const int strip = s_begin + rg2 + rgs * (b0 + i);
            if (strip >= s_end)
                continue;
            f32x4 sum = {0, 0, 0, 0};
            for (int s = 0; s < ksw; ++s) {
                const f32x4 v = reinterpret_cast<const f32x4*>(smem + (rg2 * ksw + s) * SK_WAVE_LDS)[i * 64 + ln];
                sum[0] += v[0]; sum[1] += v[1]; sum[2] += v[2]; sum[3] += v[3];
            }
            const int gj = strip * 16 + (ln & 15);
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int gi = 4 * (ln >> 4) + r;
                if (gi < p.m && gj < p.n) {
                    if (p.out_bf16)
                        reinterpret_cast<uint16_t*>(p.out)[(long)gi * p.ldc + gj] = f32_to_bf16_bits(sum[r]);
                    else
                        reinterpret_cast<float*>(p.out)[(long)gi * p.ldc + gj] = sum[r];
                }
            }
        }
        __syncthreads();
    }
}

// ---- split-K kernel with loader waves (k % 2048 == 0) ----------------------------------------------------------
// Same products and the same partition of K into 512-wide slices as the split-K kernel above; the ORDER in which a
// workgroup adds its chunks is rotated (see K below), so the fp32 sums agree with that kernel's to rounding (1e-5
// relative in the tests), not bit for bit.  The order is a function of blockIdx.x and of the grid, which follows the
// device's compute-unit count: results are deterministic on one device and launch shape, and not reproducible bit for
// bit across devices with different CU counts.  A caller that needs one order everywhere sets PTOAMD_GEMV_NO_WIDE=1
// (the split-K kernel above: its order of additions depends on k alone).  Two things hold that kernel back: its 512-byte row
// pieces (an LDS-DMA that covers 1 KiB of one row streams about a fifth faster, non-temporal another 13 %: a weight byte
// is read once and stays out of the memory-side cache), and that a wave which both computes and issues its own DMAs
// sits in the issue whenever the CU's memory queue is full, its matrix pipe idle, while the queue runs dry during its
// MFMAs.  Here the roles are split: waves 4-7 only load, waves 0-3 only compute.
//   K       is walked in chunks of 2048 (workgroup b starts at chunk b % chunks: with every workgroup on the same
//           quarter of the rows at the same time, part of the memory channels sits idle).  Compute wave c owns k-slice c
//           (512 k) of the chunk and keeps its activation fragments in registers.  It loads them itself -- its own DMA
//           counter sees nothing else -- through three private 4 KiB buffers, one MFMA j-step (16 rows x 256 bytes,
//           chunk c of row r at c ^ r) at a time, and it loads the next chunk's while it works on this one.
//   stage   one strip of 16 weight rows x one chunk: row r is one piece of 1 KiB at r KiB (16-byte chunk c at position
//           c ^ r, applied on the global side, so that the 16 rows a 16-lane group reads at one chunk index fall into
//           16 different bank groups), then 16 x 64 scale bytes.  A ring of six stages: the loaders run up to six ahead.
//   sync    one workgroup barrier per stage t: every loader's pieces of stage t have landed, and every compute wave has
//           its fragments of stage t - 1 in registers, so after it the loaders refill that slot with stage t + 5 while
//           the compute waves read stage t.  (Two barriers per stage -- landed / consumed -- ran 0.2 us slower; with
//           no synchronisation at all, results wrong, the launch takes 23.8 instead of 24.6 us: what is left is the
//           memory system's, not the barriers'.)
constexpr int WD_CHUNK = 2048;                       // k per chunk
constexpr int WD_WBYTES = 16 * (WD_CHUNK / 2);       // 16 KiB
constexpr int WD_SBYTES = 16 * (WD_CHUNK / 32);      // 1 KiB
constexpr int WD_STAGE = WD_WBYTES + WD_SBYTES;
constexpr int WD_RING = 6;
constexpr int WD_ABYTES = 3 * 4096;                  // activation staging of one compute wave (also its partial sums)
constexpr int WD_LDS = WD_RING * WD_STAGE + 4 * WD_ABYTES;   // 150 KiB
constexpr int WD_VM_PER_STAGE = 5;                   // LDS-DMA instructions per loader wave per stage: 4 weight + 1 scale
static_assert(SK_RMAX * 64 * 16 <= WD_ABYTES, "a compute wave's partial sums fit its staging region");
static_assert(WD_LDS <= 160 * 1024, "LDS capacity");

// s_waitcnt vmcnt(n) alone, n < 64 (the count is split over bits 3:0 and 15:14 of the immediate)
#define PTOAMD_WAIT_VM(n) __builtin_amdgcn_s_waitcnt(0x0F70 | ((n) & 15) | (((n) >> 4) << 14))

__device__ __forceinline__ void wg_barrier() { asm volatile("s_barrier" ::: "memory"); }

// PACKED: the weights come as the stages this kernel consumes.  Block number strip * (k / 2048) + chunk of the packed
// buffer's first region holds the 16 row pieces of (strip of 16 rows, chunk of 2048 k), their 16-byte chunks already at
// the swizzled positions (16 KiB); the same block number of the second region holds the 16 x 64 scale bytes (1 KiB).  A
// stage is then two contiguous runs of memory instead of 16 pieces 1 KiB long and a row pitch apart plus 16 scale
// pieces, and streams 4 - 5 % faster (23.4 against 24.5 us on 16 x 28672 x 8192; with the scales inside one 17 KiB block
// per stage, which takes the code blocks off their 16 KiB alignment, 23.8 us).
template <bool HW_CVT, bool PACKED = false>
__global__ void __launch_bounds__(512) gemv_mxfp4_splitk_wide_kernel(const GemvParams p, int strips_per_wg)
{
    extern __shared__ __align__(16) uint8_t smem[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const bool loader = wave >= 4;
    const int wc = wave & 3;                          // compute: k-slice of the chunk; loader: which quarter of a stage
    const int l16 = lane & 15, q = lane >> 4;
    const int s_begin = blockIdx.x * strips_per_wg, s_end = min(s_begin + strips_per_wg, p.n_groups);
    const int nsteps = s_end - s_begin, kchunks = p.k / WD_CHUNK, sb = p.k / 32;
    const int kc_first = blockIdx.x % kchunks;        // chunk number x of this workgroup is chunk (kc_first + x) % kchunks of K
    const uint32_t lds0 = lds_address(smem);
    uint8_t* mine = smem + WD_RING * WD_STAGE + wc * WD_ABYTES;      // compute wave's private region
    const uint32_t mine_lds = lds0 + WD_RING * WD_STAGE + wc * WD_ABYTES;
    // fragment read addresses of a compute lane inside a stage: weight chunk 4 j + q of its slice is at wread ^ (64 j)
    const int wread = l16 * 1024 + 256 * wc + ((q ^ l16) << 4);
    const int sread = WD_WBYTES + l16 * 64 + wc * 16;
    const int aread = l16 * 256 + (((4 * q) ^ l16) << 4);   // activation fragment t of a j-step is at aread ^ (16 t)

    // ---- loader side: stage number x of this workgroup (batch b0, chunk kc, strip i of the batch) -> ring slot x % 6
    int nx_b0 = 0, nx_kc = 0, nx_i = 0, issued = 0;   // the next stage to issue
    auto issue_next = [&]() {
        if (nx_b0 >= nsteps)
            return;
        const int strip = s_begin + nx_b0 + nx_i;
        const int kc = (kc_first + nx_kc) % kchunks;
        const uint32_t dst = lds0 + (issued % WD_RING) * WD_STAGE;
        const int rlim = min(15, p.n - 1 - strip * 16);
        const int e = wc * 64 + lane;   // 64 dwords = the scales of four rows
        if constexpr (PACKED) {
            const long idx = (long)strip * kchunks + kc;
            const uint8_t* blk = p.wp + idx * WD_WBYTES;
#pragma unroll
            for (int d = 0; d < 4; ++d) {
                const int r = 4 * wc + d;
                lds_dma16_off_nt(blk, (uint32_t)(r * 1024 + (lane << 4)), dst + r * 1024);
            }
            lds_dma4_off_nt(p.wp + (long)p.n_groups * kchunks * WD_WBYTES + idx * WD_SBYTES, (uint32_t)(e * 4), dst + WD_WBYTES + wc * 256);
        } else {
            const uint8_t* wbase = p.w + (long)strip * 16 * p.ldw_bytes + (long)kc * (WD_CHUNK / 2);
#pragma unroll
            for (int d = 0; d < 4; ++d) {
                const int r = 4 * wc + d;   // a loader takes four neighbouring rows (slightly faster than every fourth)
                lds_dma16_off_nt(wbase, (uint32_t)(min(r, rlim) * (int)p.ldw_bytes) + (uint32_t)((lane ^ r) << 4), dst + r * 1024);
            }
            lds_dma4_off_nt(p.sw + (long)strip * 16 * sb + (long)kc * (WD_CHUNK / 32), (uint32_t)(min(e >> 4, rlim) * sb + (e & 15) * 4),
                            dst + WD_WBYTES + wc * 256);
        }
        ++issued;
        if (++nx_i == min(SK_RMAX, nsteps - nx_b0)) {
            nx_i = 0;
            if (++nx_kc == kchunks) {
                nx_kc = 0;
                nx_b0 += SK_RMAX;
            }
        }
    };
    if (loader) {
#pragma unroll 1
        for (int x = 0; x < WD_RING; ++x)
            issue_next();
    }

    // ---- compute side: activation fragments of this wave's k-slice of a chunk, areg[4 e + t] =
    // A[l16][2048 kc + 512 wc + 128 e + 32 q + 8 t .. + 7]; rows past m - 1 re-read row m - 1 (their outputs are never stored).
    // anext collects the next chunk's while the current chunk is being multiplied.
    uint4 areg[16], anext[16];
    const uint8_t* abase = nullptr;
    auto issue_a = [&](int e) {
        int ln = lane;
        asm volatile("" : "+v"(ln));
#pragma unroll
        for (int d = 0; d < 4; ++d) {
            const int row = 4 * d + (ln >> 4), pos = ln & 15;
            lds_dma16_off(abase + e * 256, (uint32_t)(min(row, p.m - 1) * (int)p.lda * 2 + ((pos ^ row) << 4)),
                          mine_lds + (e % 3) * 4096 + d * 1024);
        }
    };
    auto prefetch_begin = [&](int kc) {
        abase = reinterpret_cast<const uint8_t*>(p.a) + (long)(kc * 4 + wc) * 1024;
        issue_a(0);
        issue_a(1);
        issue_a(2);
    };
    auto prefetch_step = [&](auto ec) {
        constexpr int e = decltype(ec)::value;
        PTOAMD_WAIT_VM(4 * (e < 2 ? 2 : 3 - e));   // all but the j-steps issued after e
        asm volatile("" ::: "memory");
        const uint8_t* buf = mine + (e % 3) * 4096;
#pragma unroll
        for (int t = 0; t < 4; ++t)
            anext[4 * e + t] = *reinterpret_cast<const uint4*>(buf + (aread ^ (16 * t)));
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        if (e == 0)
            issue_a(3);
    };
    if (!loader) {
        prefetch_begin(kc_first);
        static_for<4>([&](auto ec) { prefetch_step(ec); });
    }

    int consumed = 0;   // stages taken so far
    for (int b0 = 0; b0 < nsteps; b0 += SK_RMAX) {
        const int cnt = min(SK_RMAX, nsteps - b0);
        f32x4 acc[SK_RMAX];
#pragma unroll
        for (int i = 0; i < SK_RMAX; ++i)
            acc[i] = f32x4{0, 0, 0, 0};

        for (int kcx = 0; kcx < kchunks; ++kcx) {
            // the chunk after this one, if the workgroup has one and its activations differ
            const bool more = kchunks > 1 && (kcx + 1 < kchunks || b0 + SK_RMAX < nsteps);
            if (!loader) {
                if (kchunks > 1 || (b0 == 0 && kcx == 0)) {
#pragma unroll
                    for (int x = 0; x < 16; ++x)
                        areg[x] = anext[x];
                }
                if (more)
                    prefetch_begin((kc_first + kcx + 1) % kchunks);
            }

            static_for<SK_RMAX>([&](auto ic) {
                constexpr int i = decltype(ic)::value;
                if (i < cnt) {
                    if (loader) {   // own pieces of this stage have landed once only the stages issued after it are outstanding
                        switch (issued - consumed - 1) {
                            case 0: PTOAMD_WAIT_VM(0); break;
                            case 1: PTOAMD_WAIT_VM(WD_VM_PER_STAGE); break;
                            case 2: PTOAMD_WAIT_VM(2 * WD_VM_PER_STAGE); break;
                            case 3: PTOAMD_WAIT_VM(3 * WD_VM_PER_STAGE); break;
                            case 4: PTOAMD_WAIT_VM(4 * WD_VM_PER_STAGE); break;
                            default: PTOAMD_WAIT_VM(5 * WD_VM_PER_STAGE); break;
                        }
                    }
                    // The one barrier of a stage: every loader's pieces of this stage have landed, and every compute
                    // wave has the previous stage's fragments in registers (it waited for those reads before its
                    // MFMAs), so the loaders refill the previous stage's slot right away while the compute waves read
                    // this one.
                    wg_barrier();
                    const uint8_t* buf = smem + (consumed % WD_RING) * WD_STAGE;
                    ++consumed;
                    if (loader) {
                        if (consumed > 1)
                            issue_next();
                    } else {
                        uint4 sc4, wv[4];
                        sc4 = *reinterpret_cast<const uint4*>(buf + sread);
#pragma unroll
                        for (int j = 0; j < 4; ++j)
                            wv[j] = *reinterpret_cast<const uint4*>(buf + (wread ^ (64 * j)));
                        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                        const uint32_t sc[4] = {sc4.x, sc4.y, sc4.z, sc4.w};
#pragma unroll
                        for (int j = 0; j < 4; ++j) {
                            const float scale = e8m0_to_f32((sc[j] >> (8 * q)) & 0xFFu);  // scale byte 4 j + q of the slice
                            const uint32_t xs[4] = {wv[j].x, wv[j].y, wv[j].z, wv[j].w};
#pragma unroll
                            for (int t = 0; t < 4; ++t) {
                                const uint4 w8 = dequant8<HW_CVT>(xs[t], scale);
                                acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, areg[4 * j + t]),
                                                                                __builtin_bit_cast(bf16x8, w8), acc[i], 0, 0, 0);
                            }
                        }
                        if (i < 4 && more)
                            prefetch_step(std::integral_constant<int, (i < 4 ? i : 0)>{});
                    }
                }
            });
            if (!loader && more)   // a batch of fewer than four strips: the rest of the next chunk's activations
                static_for<4>([&](auto ec) {
                    if (decltype(ec)::value >= cnt)
                        prefetch_step(ec);
                });
        }

        // sum the four k-slice partials of each strip in slice order; every compute wave parks its accumulators in its
        // own region, then all 512 threads take one output lane each
        if (!loader) {
            f32x4* part = reinterpret_cast<f32x4*>(mine);
#pragma unroll
            for (int i = 0; i < SK_RMAX; ++i)
                part[i * 64 + lane] = acc[i];
        }
        __syncthreads();
        {
            const int i = tid >> 6, strip = s_begin + b0 + i;
            if (i < cnt) {
                f32x4 sum = {0, 0, 0, 0};
                for (int s = 0; s < 4; ++s) {
                    const f32x4 v = reinterpret_cast<const f32x4*>(smem + WD_RING * WD_STAGE + s * WD_ABYTES)[i * 64 + lane];
                    sum[0] += v[0]; sum[1] += v[1]; sum[2] += v[2]; sum[3] += v[3];
                }
                const int gj = strip * 16 + l16;
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int gi = 4 * q + r;
                    if (gi < p.m && gj < p.n) {
                        if (p.out_bf16)
                            reinterpret_cast<uint16_t*>(p.out)[(long)gi * p.ldc + gj] = f32_to_bf16_bits(sum[r]);
                        else
                            reinterpret_cast<float*>(p.out)[(long)gi * p.ldc + gj] = sum[r];
                    }
                }
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

// Weights [n][ldw_bytes] + scales [n][k / 32] -> the stage blocks of the PACKED loader-wave kernel.  One workgroup per
// block (strip, chunk): thread t moves 16-byte position t % 64 of rows t / 64, t / 64 + 4, ...; a row past n - 1 repeats
// row n - 1, as the loader of the plain form does (its outputs are never stored).
__global__ void __launch_bounds__(256) gemv_mxfp4_pack_kernel(uint8_t* __restrict__ packed, const uint8_t* __restrict__ w,
                                                               const uint8_t* __restrict__ sw, int n, int k, long ldw_bytes, long ldsw)
{
    const int kchunks = k / WD_CHUNK, strip = blockIdx.x / kchunks, kc = blockIdx.x % kchunks;
    uint8_t* blk = packed + (long)blockIdx.x * WD_WBYTES;
    uint8_t* sblk = packed + (long)gridDim.x * WD_WBYTES + (long)blockIdx.x * WD_SBYTES;
    const int pos = threadIdx.x & 63;
    for (int r = threadIdx.x >> 6; r < 16; r += 4) {
        const long row = min(strip * 16 + r, n - 1);
        const uint4 v = *reinterpret_cast<const uint4*>(w + row * ldw_bytes + (long)kc * (WD_CHUNK / 2) + ((pos ^ r) << 4));
        *reinterpret_cast<uint4*>(blk + r * 1024 + (pos << 4)) = v;
    }
    {
        const int e = threadIdx.x;  // dword e of the 16 x 64 scale bytes
        const long row = min(strip * 16 + (e >> 4), n - 1);
        *reinterpret_cast<uint32_t*>(sblk + e * 4) =
            *reinterpret_cast<const uint32_t*>(sw + row * ldsw + (long)kc * (WD_CHUNK / 32) + (e & 15) * 4);
    }
}

int prepare_gemv_kernels()
{
    PTOAMD_HIP_CHECK(ensure_dynamic_lds(reinterpret_cast<const void*>(gemv_mxfp4_splitk_wide_kernel<true, true>), WD_LDS));
    PTOAMD_HIP_CHECK(ensure_dynamic_lds(reinterpret_cast<const void*>(gemv_mxfp4_splitk_wide_kernel<false>), WD_LDS));
    PTOAMD_HIP_CHECK(ensure_dynamic_lds(reinterpret_cast<const void*>(gemv_mxfp4_splitk_wide_kernel<true>), WD_LDS));
    PTOAMD_HIP_CHECK(ensure_dynamic_lds(reinterpret_cast<const void*>(gemv_mxfp4_splitk_kernel<false>), SK_LDS));
    PTOAMD_HIP_CHECK(ensure_dynamic_lds(reinterpret_cast<const void*>(gemv_mxfp4_splitk_kernel<true>), SK_LDS));
    return PTOAMD_OK;
}

}  // namespace ptoamd

using namespace ptoamd;

extern "C" int ptoamd_gemv_mxfp4(void* out, int c_type, const void* a_bf16, const uint8_t* w, const uint8_t* sw, int m,
                                 int n, int k, int lda, int ldw, int ldc, void* stream_)
{
    hipStream_t stream = as_stream(stream_);
    TraceScope trace("TGEMV_MX", "cube", m, n, k);
    trace.in(a_bf16, m, k, "ND", PTOAMD_BF16).in(w, k, n, "DN", PTOAMD_E2M1).in(sw, k / 32, n, "MX_B_DN", 100).out(out, m, n, "ND", c_type);
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
    const Options& opt = options();
    const bool stream_ok = !opt.force_generic && k % GEMV_CHUNK == 0 && (reinterpret_cast<uintptr_t>(a_bf16) & 15u) == 0 &&
                           (reinterpret_cast<uintptr_t>(w) & 15u) == 0 && (reinterpret_cast<uintptr_t>(sw) & 15u) == 0 &&
                           (lda % 8) == 0 && (p.ldw_bytes % 16) == 0;
    if (!stream_ok) {
        dim3 block(128), grid((n + 127) / 128, m);
        hipLaunchKernelGGL(gemv_mxfp4_generic_kernel, grid, block, 0, stream, p);
        PTOAMD_HIP_CHECK(hipGetLastError());
        set_last_kernel("gemv_mxfp4_generic");
        return PTOAMD_OK;
    }
    const int cus = device_compute_units();
    const bool swc = opt.gemv_sw_cvt;
    const bool sk_ok = k % SK_SLICE == 0 && (reinterpret_cast<uintptr_t>(sw) & 3u) == 0 && !opt.gemv_no_splitk;
    // loader-wave form: K in chunks of 2048; rows are addressed with 32-bit lane offsets
    if (sk_ok && k % WD_CHUNK == 0 && (long)lda * 2 * 16 < (1L << 31) && p.ldw_bytes * 16 < (1L << 31) && !opt.gemv_no_wide) {
        const int spw = (p.n_groups + cus - 1) / cus;    // strips per workgroup
        const int grid = (p.n_groups + spw - 1) / spw;
        const void* fn = swc ? reinterpret_cast<const void*>(gemv_mxfp4_splitk_wide_kernel<false>)
                             : reinterpret_cast<const void*>(gemv_mxfp4_splitk_wide_kernel<true>);
        PTOAMD_HIP_CHECK(ensure_dynamic_lds(fn, WD_LDS));
        if (swc)
            hipLaunchKernelGGL(gemv_mxfp4_splitk_wide_kernel<false>, dim3(grid), dim3(512), WD_LDS, stream, p, spw);
        else
            hipLaunchKernelGGL(gemv_mxfp4_splitk_wide_kernel<true>, dim3(grid), dim3(512), WD_LDS, stream, p, spw);
        PTOAMD_HIP_CHECK(hipGetLastError());
        set_last_kernel(swc ? "gemv_mxfp4_splitk_wide_swcvt" : "gemv_mxfp4_splitk_wide");
        return PTOAMD_OK;
    }
    // (row pitches are multiplied as 24-bit integers in the kernel's address arithmetic)
    if (sk_ok && (long)lda * 2 < (1L << 24) && p.ldw_bytes < (1L << 24)) {
        const int ks = k / SK_SLICE;
        int ksw_log2 = 0;
        while (ksw_log2 < 3 && (2 << ksw_log2) <= ks)
            ++ksw_log2;
        const int rgs = SK_WAVES >> ksw_log2;
        int spw = (p.n_groups + cus - 1) / cus;          // strips per workgroup, a multiple of the row-group count
        spw = (spw + rgs - 1) / rgs * rgs;
        const int grid = (p.n_groups + spw - 1) / spw;
        const void* fn = swc ? reinterpret_cast<const void*>(gemv_mxfp4_splitk_kernel<false>)
                             : reinterpret_cast<const void*>(gemv_mxfp4_splitk_kernel<true>);
        PTOAMD_HIP_CHECK(ensure_dynamic_lds(fn, SK_LDS));
        if (swc)
            hipLaunchKernelGGL(gemv_mxfp4_splitk_kernel<false>, dim3(grid), dim3(SK_WAVES * 64), SK_LDS, stream, p, ksw_log2, spw);
        else
            hipLaunchKernelGGL(gemv_mxfp4_splitk_kernel<true>, dim3(grid), dim3(SK_WAVES * 64), SK_LDS, stream, p, ksw_log2, spw);
        PTOAMD_HIP_CHECK(hipGetLastError());
        set_last_kernel(swc ? "gemv_mxfp4_splitk_swcvt" : "gemv_mxfp4_splitk");
        return PTOAMD_OK;
    }
    // streaming kernel: 16 rows per wave; 7 waves per workgroup when that tiles the row groups more evenly over the
    // CUs than 8, else 8
    const int g7 = (p.n_groups + 6) / 7, g8 = (p.n_groups + 7) / 8;
    const auto rounds = [&](int blocks) { return (blocks + cus - 1) / cus; };
    const bool use7 = rounds(g7) * 7 < rounds(g8) * 8;
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

// ---- the pre-packed form: weights stored once in the order the loader waves consume them ------------------------------
extern "C" size_t ptoamd_gemv_mxfp4_packed_bytes(int n, int k)
{
    if (n <= 0 || k <= 0 || k % WD_CHUNK != 0)
        return 0;
    return (size_t)((n + 15) / 16) * (size_t)(k / WD_CHUNK) * (size_t)WD_STAGE;
}

extern "C" int ptoamd_gemv_mxfp4_pack(void* packed, const uint8_t* w, const uint8_t* sw, int n, int k, int ldw, void* stream_)
{
    hipStream_t stream = as_stream(stream_);
    PTOAMD_REQUIRE(packed && w && sw, PTOAMD_E_INVALID, "ptoamd_gemv_mxfp4_pack: null operand");
    PTOAMD_REQUIRE(n > 0 && k > 0, PTOAMD_E_INVALID, "ptoamd_gemv_mxfp4_pack: n, k must be positive");
    PTOAMD_REQUIRE(k % WD_CHUNK == 0, PTOAMD_E_UNSUPPORTED, "ptoamd_gemv_mxfp4_pack: k = %d must be a multiple of %d", k, WD_CHUNK);
    PTOAMD_REQUIRE(ldw >= k && ldw % 32 == 0, PTOAMD_E_INVALID, "ptoamd_gemv_mxfp4_pack: ldw must be at least k and a multiple of 32");
    PTOAMD_REQUIRE((reinterpret_cast<uintptr_t>(packed) & 15u) == 0 && (reinterpret_cast<uintptr_t>(w) & 15u) == 0 &&
                       (reinterpret_cast<uintptr_t>(sw) & 3u) == 0,
                   PTOAMD_E_ALIGNMENT, "ptoamd_gemv_mxfp4_pack: packed and w must be 16-byte aligned, sw 4-byte aligned");
    const long blocks = (long)((n + 15) / 16) * (k / WD_CHUNK);
    PTOAMD_REQUIRE(blocks < (1L << 31), PTOAMD_E_UNSUPPORTED, "ptoamd_gemv_mxfp4_pack: too many blocks");
    hipLaunchKernelGGL(gemv_mxfp4_pack_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, reinterpret_cast<uint8_t*>(packed), w, sw,
                       n, k, (long)ldw / 2, (long)k / 32);
    PTOAMD_HIP_CHECK(hipGetLastError());
    set_last_kernel("gemv_mxfp4_pack");
    return PTOAMD_OK;
}

extern "C" int ptoamd_gemv_mxfp4_packed(void* out, int c_type, const void* a_bf16, const void* packed, int m, int n, int k,
                                        int lda, int ldc, void* stream_)
{
    hipStream_t stream = as_stream(stream_);
    TraceScope trace("TGEMV_MX", "cube", m, n, k);
    trace.in(a_bf16, m, k, "ND", PTOAMD_BF16).in(packed, k, n, "packed", PTOAMD_E2M1).out(out, m, n, "ND", c_type);
    PTOAMD_REQUIRE(out && a_bf16 && packed, PTOAMD_E_INVALID, "ptoamd_gemv_mxfp4_packed: null operand");
    PTOAMD_REQUIRE(m > 0 && n > 0 && k > 0, PTOAMD_E_INVALID, "ptoamd_gemv_mxfp4_packed: m, n, k must be positive");
    PTOAMD_REQUIRE(m <= 16, PTOAMD_E_UNSUPPORTED, "ptoamd_gemv_mxfp4_packed: m = %d exceeds the decode batch of 16", m);
    PTOAMD_REQUIRE(k % WD_CHUNK == 0, PTOAMD_E_UNSUPPORTED, "ptoamd_gemv_mxfp4_packed: k = %d must be a multiple of %d", k, WD_CHUNK);
    PTOAMD_REQUIRE(c_type == PTOAMD_F32 || c_type == PTOAMD_BF16, PTOAMD_E_UNSUPPORTED, "ptoamd_gemv_mxfp4_packed: output is f32 or bf16");
    PTOAMD_REQUIRE(lda >= k && ldc >= n && lda % 8 == 0 && (long)lda * 2 * 16 < (1L << 31), PTOAMD_E_INVALID,
                   "ptoamd_gemv_mxfp4_packed: lda must be at least k and a multiple of 8, ldc at least n");
    PTOAMD_REQUIRE((reinterpret_cast<uintptr_t>(a_bf16) & 15u) == 0 && (reinterpret_cast<uintptr_t>(packed) & 15u) == 0,
                   PTOAMD_E_ALIGNMENT, "ptoamd_gemv_mxfp4_packed: a and packed must be 16-byte aligned");
    GemvParams p{};
    p.a = reinterpret_cast<const uint16_t*>(a_bf16);
    p.wp = reinterpret_cast<const uint8_t*>(packed);
    p.out = out;
    p.m = m; p.n = n; p.k = k; p.lda = lda; p.ldc = ldc;
    p.out_bf16 = c_type == PTOAMD_BF16;
    p.n_groups = (n + 15) / 16;
    const int cus = device_compute_units();
    const int spw = (p.n_groups + cus - 1) / cus;
    const int grid = (p.n_groups + spw - 1) / spw;
    PTOAMD_HIP_CHECK(ensure_dynamic_lds(reinterpret_cast<const void*>(gemv_mxfp4_splitk_wide_kernel<true, true>), WD_LDS));
    hipLaunchKernelGGL((gemv_mxfp4_splitk_wide_kernel<true, true>), dim3(grid), dim3(512), WD_LDS, stream, p, spw);
    PTOAMD_HIP_CHECK(hipGetLastError());
    set_last_kernel("gemv_mxfp4_splitk_wide_packed");
    return PTOAMD_OK;
}

