// Compile-time loops and direct global -> LDS copies (LDS-DMA) shared by the tile GEMM and the decode GEMV kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <utility>

namespace ptoamd {

typedef __attribute__((address_space(3))) void* lds_ptr_t;

// Compile-time loop: f(std::integral_constant<int, I>{}) for I = 0 .. N-1.  Keeps every register-array index a literal
// (a `#pragma unroll` the compiler declines leaves the accumulators indexed at run time, i.e. in scratch memory).
template <int... Is, class F>
__device__ __forceinline__ void static_for_impl(std::integer_sequence<int, Is...>, F&& f)
{
    (f(std::integral_constant<int, Is>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void static_for(F&& f)
{
    static_for_impl(std::make_integer_sequence<int, N>{}, static_cast<F&&>(f));
}

// One LDS-DMA: 64 lanes x 16 bytes from per-lane global addresses to LDS bytes [lds_base, lds_base + 1024), lane-linear.
// Issued as inline assembly on purpose: when the compiler sees an LDS-DMA it makes every later LDS read wait for it
// (vmcnt(0)), since it cannot prove that the reads touch the other half of the ring; that wait would serialise the
// slab prefetch with the MFMAs.  The kernel waits for its DMAs itself, right before the barrier that publishes a slab.
__device__ __forceinline__ void lds_dma16(const uint8_t* gptr, uint32_t lds_base)
{
    const uint32_t base = __builtin_amdgcn_readfirstlane(lds_base);  // wave-uniform by construction
    asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(gptr), "s"(base) : "memory", "m0");
}
__device__ __forceinline__ uint32_t lds_address(const void* generic_ptr)
{
    return (uint32_t)(uintptr_t)(lds_ptr_t)(generic_ptr);
}

// The 4-byte form: 64 lanes x 4 bytes to LDS bytes [lds_base, lds_base + 256), lane-linear.
__device__ __forceinline__ void lds_dma4(const uint8_t* gptr, uint32_t lds_base)
{
    const uint32_t base = __builtin_amdgcn_readfirstlane(lds_base);
    asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dword %0, off" : : "v"(gptr), "s"(base) : "memory", "m0");
}

// A 64-bit value known to be wave-uniform, moved to scalar registers (readfirstlane returns a signed int: each half
// goes through uint32_t so the low half is not sign-extended over the high half).
__device__ __forceinline__ uint64_t uniform_u64(uint64_t v)
{
    const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)v);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(v >> 32));
    return ((uint64_t)hi << 32) | (uint64_t)lo;
}

// The same copies addressed as a wave-uniform base plus a 32-bit per-lane byte offset (no 64-bit address VGPRs).
__device__ __forceinline__ void lds_dma16_off(const uint8_t* base_ptr, uint32_t lane_off, uint32_t lds_base)
{
    const uint32_t base = __builtin_amdgcn_readfirstlane(lds_base);
    const uint64_t g = (uint64_t)(uintptr_t)base_ptr;
    const uint64_t gs = uniform_u64(g);
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1" : : "v"(lane_off), "s"(gs), "s"(base) : "memory", "m0");
}
// Non-temporal forms for data that is read once (a weight stream): the lines are not kept in the memory-side cache, and
// a streaming read runs about 13 % faster on this part (6.5 against 5.75 TB/s for 1 KiB-per-instruction row reads).
__device__ __forceinline__ void lds_dma16_off_nt(const uint8_t* base_ptr, uint32_t lane_off, uint32_t lds_base)
{
    const uint32_t base = __builtin_amdgcn_readfirstlane(lds_base);
    const uint64_t g = (uint64_t)(uintptr_t)base_ptr;
    const uint64_t gs = uniform_u64(g);
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1 nt" : : "v"(lane_off), "s"(gs), "s"(base) : "memory", "m0");
}
__device__ __forceinline__ void lds_dma4_off_nt(const uint8_t* base_ptr, uint32_t lane_off, uint32_t lds_base)
{
    const uint32_t base = __builtin_amdgcn_readfirstlane(lds_base);
    const uint64_t g = (uint64_t)(uintptr_t)base_ptr;
    const uint64_t gs = uniform_u64(g);
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dword %0, %1 nt" : : "v"(lane_off), "s"(gs), "s"(base) : "memory", "m0");
}
__device__ __forceinline__ void lds_dma4_off(const uint8_t* base_ptr, uint32_t lane_off, uint32_t lds_base)
{
    const uint32_t base = __builtin_amdgcn_readfirstlane(lds_base);
    const uint64_t g = (uint64_t)(uintptr_t)base_ptr;
    const uint64_t gs = uniform_u64(g);
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dword %0, %1" : : "v"(lane_off), "s"(gs), "s"(base) : "memory", "m0");
}

}  // namespace ptoamd
