// Running a core program: pto::amd::launch<&Kernel<...>>(blocks, stream, args...) starts `blocks` cores (workgroups of
// PTO_AMD_THREADS threads) with the core's LDS arena; get_block_idx() / get_block_num() name them, like the `<<<>>>`
// launch of the reference's NPU tests and LaunchKernelMultiCore of its CPU simulator (common/cpu_stub.hpp:367-427).
#pragma once
#include <atomic>
#ifdef PTO_AMD_TRACE
#include <stdio.h>
#include <stdlib.h>
#include <unistd.h>

#include <vector>
#endif

#include "tile.hpp"
#include "trace.hpp"

namespace pto {
namespace amd {

template <auto Kernel, typename... Args>
__attribute__((global)) __launch_bounds__(PTO_AMD_THREADS) void core_entry(Args... args)
{
    Kernel(args...);
}

#ifdef PTO_AMD_TRACE
// After a traced launch: wait for it, read the records of the traced core and append them as JSON lines (field names of
// the reference's InstructionTraceRecord, cpu/trace.hpp:80-88) to $PTOAMD_TRACE_DIR/ptoamd_instr_trace_<pid>.jsonl.
inline int write_instruction_trace(hipStream_t stream)
{
    hipError_t e = hipStreamSynchronize(stream);
    if (e != hipSuccess)
        return (int)e;
    unsigned int count = 0;
    if ((e = hipMemcpyFromSymbol(&count, HIP_SYMBOL(g_trace_count), sizeof count)) != hipSuccess)
        return (int)e;
    const unsigned int kept = count < PTO_AMD_TRACE_MAX ? count : PTO_AMD_TRACE_MAX;
    std::vector<TraceRecord> rec(kept);
    if (kept > 0 && (e = hipMemcpyFromSymbol(rec.data(), HIP_SYMBOL(g_trace), kept * sizeof(TraceRecord))) != hipSuccess)
        return (int)e;
    const char* dir = getenv("PTOAMD_TRACE_DIR");
    if (dir == nullptr || *dir == 0)
        return 0;
    char path[1024];
    snprintf(path, sizeof path, "%s/ptoamd_instr_trace_%ld.jsonl", dir, (long)getpid());
    FILE* f = fopen(path, "a");
    if (f == nullptr)
        return 0;
    for (unsigned int i = 0; i < kept; ++i) {
        const TraceRecord& r = rec[i];
        fprintf(f, "{\"block_idx\": %u, \"subblock_id\": 0, \"sequence_id\": %u, \"opcode\": \"%s\"", r.block_idx, i, trace_op_name(r.opcode));
        for (int side = 0; side < 2; ++side) {
            fprintf(f, ", \"%s\": [", side == 0 ? "output_tiles" : "input_tiles");
            bool first = true;
            for (int k = 0; k < 4; ++k) {
                const TraceOperand& o = r.operands[k];
                if (!o.used || (k < r.n_out) != (side == 0))
                    continue;
                fprintf(f, "%s{\"address\": %llu, \"shape\": [%d, %d], \"layout\": \"%s\", \"dtype\": \"%s\"}", first ? "" : ", ",
                        (unsigned long long)o.address, o.rows, o.cols, trace_place_name(o.place), trace_dtype_name(o.dtype));
                first = false;
            }
            fprintf(f, "]");
        }
        fprintf(f, "}\n");
    }
    if (count > kept)
        fprintf(f, "{\"dropped_records\": %u}\n", count - kept);
    fclose(f);
    return 0;
}
#endif

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
#ifdef PTO_AMD_TRACE
    const unsigned int zero = 0;
    if (const hipError_t e = hipMemcpyToSymbol(HIP_SYMBOL(g_trace_count), &zero, sizeof zero); e != hipSuccess)
        return (int)e;
#endif
    hipLaunchKernelGGL(entry, dim3(blocks), dim3(PTO_AMD_THREADS), LDS_TOTAL, static_cast<hipStream_t>(stream), args...);
    const int rc = (int)hipGetLastError();
#ifdef PTO_AMD_TRACE
    if (rc == 0)
        return write_instruction_trace(static_cast<hipStream_t>(stream));
#endif
    return rc;
}

// the sticky status word of this translation unit's cores (0 = no constraint violated); synchronises the device
inline int device_status()
{
    int v = -1;
    if (hipMemcpyFromSymbol(&v, HIP_SYMBOL(g_status), sizeof(int)) != hipSuccess)
        return -1;
    return v;
}

// sets the task cookie the cores of this translation unit read (reference: set_task_cookie, common/cpu_stub.hpp:498);
// a synchronous copy: launches that follow see it
inline int set_task_cookie(uint64_t cookie)
{
    const unsigned long long v = cookie;
    return (int)hipMemcpyToSymbol(HIP_SYMBOL(g_task_cookie), &v, sizeof v);
}

// clears the status word (after a test that provoked a violation on purpose)
inline int reset_device_status()
{
    const int zero = 0;
    return (int)hipMemcpyToSymbol(HIP_SYMBOL(g_status), &zero, sizeof(int));
}

}  // namespace amd
}  // namespace pto
