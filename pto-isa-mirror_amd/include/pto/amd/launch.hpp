// Running a core program: pto::amd::launch<&Kernel<...>>(blocks, stream, args...) starts `blocks` cores (workgroups of
// PTO_AMD_THREADS threads) with the core's LDS arena; get_block_idx() / get_block_num() name them, like the `<<<>>>`
// launch of the reference's NPU tests and LaunchKernelMultiCore of its CPU simulator (common/cpu_stub.hpp:367-427).
#pragma once
#include <atomic>

#include "tile.hpp"

namespace pto {
namespace amd {

template <auto Kernel, typename... Args>
__attribute__((global)) __launch_bounds__(PTO_AMD_THREADS) void core_entry(Args... args)
{
    Kernel(args...);
}

// returns hipSuccess (0) or the HIP error of the launch
template <auto Kernel, typename... Args>
inline int launch(int blocks, void* stream, Args... args)
{
    auto* entry = core_entry<Kernel, Args...>;
    // the attribute belongs to (kernel, device): remember per device which ones have it (devices past 63 set it every time)
    static std::atomic<uint64_t> configured{0};
    int dev = 0;
    if (const hipError_t e = hipGetDevice(&dev); e != hipSuccess)
        return (int)e;
    const uint64_t bit = dev < 64 ? (1ull << dev) : 0;
    if (!(configured.load(std::memory_order_acquire) & bit)) {
        const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(entry),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, (int)LDS_TOTAL);
        if (e != hipSuccess)
            return (int)e;
        configured.fetch_or(bit, std::memory_order_release);
    }
    hipLaunchKernelGGL(entry, dim3(blocks), dim3(PTO_AMD_THREADS), LDS_TOTAL, static_cast<hipStream_t>(stream), args...);
    return (int)hipGetLastError();
}

// the sticky status word of this translation unit's cores (0 = no constraint violated); synchronises the device
inline int device_status()
{
    int v = -1;
    if (hipMemcpyFromSymbol(&v, HIP_SYMBOL(g_status), sizeof(int)) != hipSuccess)
        return -1;
    return v;
}

// clears the status word (after a test that provoked a violation on purpose)
inline int reset_device_status()
{
    const int zero = 0;
    return (int)hipMemcpyToSymbol(HIP_SYMBOL(g_status), &zero, sizeof(int));
}

}  // namespace amd
}  // namespace pto
