// Asynchronous global -> LDS copies (LDS-DMA) for the tile instructions: one instruction moves 64 lanes x 16 bytes from
// per-lane global addresses to 1 KiB of LDS, lane-linear, without passing through registers.  The copies complete in
// issue order on the wave's vector-memory counter; dma_wait() is the wait for all of this wave's copies.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace pto {
namespace amd {

typedef __attribute__((address_space(3))) void* lds_void_ptr;

// (M0 holds the LDS address of an LDS-DMA and is named as clobbered; the compiler notes that it reserves the register)
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"

// LDS byte address of a pointer into the arena
__device__ __forceinline__ uint32_t lds_address_of(const void* generic_ptr)
{
    return (uint32_t)(uintptr_t)(lds_void_ptr)(generic_ptr);
}

// 64 lanes x 16 bytes: lane l copies *gptr to LDS bytes [lds_base + 16 l, + 16).  lds_base must be wave-uniform.
// Written as inline assembly so that the compiler does not make later LDS reads of other tiles wait for it; the tile
// instructions that read the destination wait themselves (dma_wait + workgroup barrier).
__device__ __forceinline__ void lds_dma16(const uint8_t* gptr, uint32_t lds_base)
{
    const uint32_t base = __builtin_amdgcn_readfirstlane(lds_base);
    asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(gptr), "s"(base) : "memory", "m0");
}
// the same addressed as a wave-uniform 64-bit base plus a 32-bit per-lane byte offset
__device__ __forceinline__ void lds_dma16_off(const uint8_t* base_ptr, uint32_t lane_off, uint32_t lds_base)
{
    const uint32_t base = __builtin_amdgcn_readfirstlane(lds_base);
    const uint64_t g = (uint64_t)(uintptr_t)base_ptr;
    const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)g);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(g >> 32));
    const uint64_t gs = ((uint64_t)hi << 32) | (uint64_t)lo;
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1" : : "v"(lane_off), "s"(gs), "s"(base) : "memory", "m0");
}
#pragma clang diagnostic pop
// all vector-memory loads of this wave, LDS-DMAs included, have landed
__device__ __forceinline__ void dma_wait()
{
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0); expcnt / lgkmcnt not waited for
}

}  // namespace amd
}  // namespace pto
