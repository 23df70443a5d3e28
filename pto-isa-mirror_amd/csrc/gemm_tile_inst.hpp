// Instantiates gemm_tile_kernel for one operand type at the three tile shapes.  Included by gemm_tile_<op>.hip with
// PTOAMD_TILE_OP (the traits type) and PTOAMD_TILE_FN (the launcher's name) defined, so the operand types compile in
// parallel translation units.
#include "common_host.hpp"
#include "gemm_tile_dtl.hpp"
#include "gemm_tile_mx16.hpp"

namespace ptoamd {

template <class Cfg>
static hipError_t launch_cfg(const TileGemmParams& p, hipStream_t stream)
{
    hipError_t e = ensure_dynamic_lds(reinterpret_cast<const void*>(&gemm_tile_kernel<Cfg, false>), Cfg::LDS_BYTES);
    if (e == hipSuccess)
        e = ensure_dynamic_lds(reinterpret_cast<const void*>(&gemm_tile_kernel<Cfg, true>), Cfg::LDS_BYTES);
    if (e != hipSuccess || p.m <= 0)  // m = 0: only make the kernels ready to launch on the current device
        return e;
    const int tiles = ((p.m + Cfg::BM - 1) / Cfg::BM) * ((p.n + Cfg::BN - 1) / Cfg::BN);
    // rows that do not end on a 16-byte chunk boundary take the kernel with the tail-masking loader
    const bool ragged = (p.k_bytes & 15) != 0 || (p.b_nd && (((long)p.n * p.b_esz) & 15) != 0);
    if (ragged)
        hipLaunchKernelGGL((gemm_tile_kernel<Cfg, true>), dim3(tiles), dim3(Cfg::THREADS), Cfg::LDS_BYTES, stream, p);
    else
        hipLaunchKernelGGL((gemm_tile_kernel<Cfg, false>), dim3(tiles), dim3(Cfg::THREADS), Cfg::LDS_BYTES, stream, p);
    return hipGetLastError();
}

// RAGGED_K: this tile also exists in the form that takes a K extent of any length (the plain types' 256 x 256 and
// 128 x 128 tiles); the launcher picks it when K is not a whole number of 128-byte slabs.
template <class Cfg, bool RAGGED_K = false>
static hipError_t launch_dtl(const TileGemmParams& p, hipStream_t stream)
{
    hipError_t e = ensure_dynamic_lds(reinterpret_cast<const void*>(&gemm_tile_dtl_kernel<Cfg, false>), Cfg::LDS_BYTES);
    if constexpr (RAGGED_K) {
        if (e == hipSuccess)
            e = ensure_dynamic_lds(reinterpret_cast<const void*>(&gemm_tile_dtl_kernel<Cfg, true>), Cfg::LDS_BYTES);
    }
    if (e != hipSuccess || p.m <= 0)
        return e;
    const int tiles = ((p.m + Cfg::BM - 1) / Cfg::BM) * ((p.n + Cfg::BN - 1) / Cfg::BN);
    if (p.k_bytes % 128 != 0) {
        if constexpr (RAGGED_K) {
            hipLaunchKernelGGL((gemm_tile_dtl_kernel<Cfg, true>), dim3(tiles), dim3(Cfg::THREADS), Cfg::LDS_BYTES, stream, p);
            return hipGetLastError();
        }
        return hipErrorInvalidValue;  // the dispatcher sends such a K to this form only where it exists
    }
    hipLaunchKernelGGL((gemm_tile_dtl_kernel<Cfg, false>), dim3(tiles), dim3(Cfg::THREADS), Cfg::LDS_BYTES, stream, p);
    return hipGetLastError();
}

// the 256 x 256 tile of the block-scaled fp8 types on the 16x16x128 instruction (whole 128-byte slabs of K only)
template <class Cfg>
static hipError_t launch_mx16(const TileGemmParams& p, hipStream_t stream)
{
    const hipError_t e = ensure_dynamic_lds(reinterpret_cast<const void*>(&gemm_tile_mx16_kernel<Cfg>), Cfg::LDS_BYTES);
    if (e != hipSuccess || p.m <= 0)
        return e;
    if (p.k_bytes % 128 != 0)
        return hipErrorInvalidValue;
    const int tiles = ((p.m + Cfg::BM - 1) / Cfg::BM) * ((p.n + Cfg::BN - 1) / Cfg::BN);
    hipLaunchKernelGGL((gemm_tile_mx16_kernel<Cfg>), dim3(tiles), dim3(Cfg::THREADS), Cfg::LDS_BYTES, stream, p);
    return hipGetLastError();
}

#ifdef PTOAMD_TILE_RAGGED_K
#define PTOAMD_RK true
#else
#define PTOAMD_RK false
#endif

hipError_t PTOAMD_TILE_FN(int tile, const TileGemmParams& p, hipStream_t stream)
{
    if (tile == TILE_PREPARE_ALL) {  // every kernel of this unit gets its launch attributes on the current device
        TileGemmParams none{};
        for (int t : {4, 3, 5, 6, 7, 1, 2}) {
            const hipError_t e = PTOAMD_TILE_FN(t, none, stream);
            if (e != hipSuccess)
                return e;
        }
        return hipSuccess;
    }
    switch (tile) {
        // (tile id 3 was a four-wave form of the 256 x 256 tile, 128 x 128 per wave: never faster than the eight-wave form
        // and a third of this translation unit's compile time; the id now selects tile 4)
#ifdef PTOAMD_TILE_OP16  // the large eight-wave tile runs on the 16x16 instructions where the operand type has them
        case 3:
        case 4: return launch_dtl<TileCfg<256, 256, 2, 4, PTOAMD_TILE_OP16>, PTOAMD_RK>(p, stream);
#elif defined(PTOAMD_TILE_MX16)  // block-scaled fp8: id 3 is the large tile on the 16x16x128 instruction
        case 3:  // (tiles that lie inside the matrix; a ragged edge takes the 32x32x64 form, whose loader clamps its rows)
            if (p.m % 256 == 0 && p.n % 256 == 0)
                return launch_mx16<TileCfg<256, 256, 2, 4, PTOAMD_TILE_MX16>>(p, stream);
            return launch_dtl<TileCfg<256, 256, 2, 4, PTOAMD_TILE_OP>, PTOAMD_RK>(p, stream);
        case 4: return launch_dtl<TileCfg<256, 256, 2, 4, PTOAMD_TILE_OP>, PTOAMD_RK>(p, stream);
#else
        case 3:
        case 4: return launch_dtl<TileCfg<256, 256, 2, 4, PTOAMD_TILE_OP>, PTOAMD_RK>(p, stream);
#endif
        case 5: return launch_dtl<TileCfg<128, 128, 2, 2, PTOAMD_TILE_OP>, PTOAMD_RK>(p, stream);
        case 6: return launch_dtl<TileCfg<256, 128, 4, 2, PTOAMD_TILE_OP>>(p, stream);
#ifdef PTOAMD_TILE_RING3  // block-scaled types: the 256 x 128 tile with a ring of three slabs
        case 7: return launch_dtl<TileCfg<256, 128, 4, 2, PTOAMD_TILE_OP, 3>>(p, stream);
#else
        case 7: return launch_dtl<TileCfg<256, 128, 4, 2, PTOAMD_TILE_OP>>(p, stream);
#endif
        case 0:  // (once a register-staged 256 x 256 tile: it kept part of its working set in scratch memory)
        case 1: return launch_cfg<TileCfg<128, 128, 2, 2, PTOAMD_TILE_OP>>(p, stream);
        default: return launch_cfg<TileCfg<64, 64, 2, 2, PTOAMD_TILE_OP>>(p, stream);
    }
}

}  // namespace ptoamd
