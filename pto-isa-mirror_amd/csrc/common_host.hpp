// Host-side plumbing shared by the C-ABI translation units: error text, HIP status checks, stream casts.
#pragma once
#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdio.h>

#include "../../include/ptoamd.h"

namespace ptoamd {

void set_error(const char* fmt, ...);
void set_last_kernel(const char* name);
// sets hipFuncAttributeMaxDynamicSharedMemorySize once per (kernel, current device); thread-safe
hipError_t ensure_dynamic_lds(const void* kernel, int bytes);

// Everything a first launch would otherwise set up lazily, done for the current device: the dynamic-LDS attribute of
// every tile and GEMV kernel and the device address of the library's static scratch array.  After it, no entry point
// calls anything but kernel launches (a requirement of callers that capture launches into a HIP graph).
int prepare_gemm_kernels();
int prepare_gemv_kernels();

inline hipStream_t as_stream(void* s) { return reinterpret_cast<hipStream_t>(s); }

// The environment switches of the dispatchers, read once per process (and again by ptoamd_reload_options): a launch
// tests plain fields instead of calling getenv.
struct Options {
    int tile = -1;               // PTOAMD_TILE=0..6: run this tile shape; -1 = choose by problem size
    bool mx_16x16 = false;       // PTOAMD_MX_16X16=1: the block-scaled fp8 256 x 256 tile runs on the 16x16x128 instruction
    bool no_tail_split = false;  // PTOAMD_NO_TAIL_SPLIT=1: never split a half-full last round off as smaller tiles
    int tail_tile = 0;           // PTOAMD_TAIL_TILE=5|6|7: the tail's tile; 0 = 256x128 ring-3 tiles (block-scaled) or 128x128
    bool force_generic = false;  // PTOAMD_FORCE_GENERIC=1: everything runs on the order-exact generic kernels
    bool b_nd_in_loader = false; // PTOAMD_B_ND_IN_LOADER=1: a row-major B is transposed by the loader even when a workspace is given
    bool gemv_sw_cvt = false;    // PTOAMD_GEMV_SW_CVT=1: decode fp4 weights with integer arithmetic
    bool gemv_no_splitk = false; // PTOAMD_GEMV_NO_SPLITK=1 / PTOAMD_GEMV_NO_WIDE=1: skip those GEMV kernels
    bool gemv_no_wide = false;
};
const Options& options();
// compute units of the current device (cached per device ordinal)
int device_compute_units();

// One record per C-ABI launch, written as a JSON line to $PTOAMD_TRACE_DIR/ptoamd_trace_<pid>.jsonl when that variable
// names a directory (no-op otherwise).  Field names follow the reference simulator's InstructionTraceRecord
// (include/pto/cpu/trace.hpp:67-87: sequence_id, opcode, input_tiles / output_tiles with address, shape, layout, dtype),
// plus what identifies the launch here: the pipeline (cube / vector), m / n / k and the kernel that ran.  An entry point
// declares a scope on entry; the record is written when the scope ends, if a kernel was launched inside it.
class TraceScope {
public:
    TraceScope(const char* opcode, const char* pipeline, long m, long n, long k);
    ~TraceScope();
    TraceScope& in(const void* address, long rows, long cols, const char* layout, int dtype);
    TraceScope& out(const void* address, long rows, long cols, const char* layout, int dtype);
    TraceScope(const TraceScope&) = delete;
    TraceScope& operator=(const TraceScope&) = delete;

private:
    struct Tile { const void* address; long rows, cols; const char* layout; int dtype; };
    bool on_;
    const char *opcode_, *pipeline_;
    long m_, n_, k_;
    unsigned long launches_before_;
    Tile in_[6], out_[4];
    int nin_ = 0, nout_ = 0;
};

#define PTOAMD_HIP_CHECK(expr)                                                                   \
    do {                                                                                         \
        hipError_t e_ = (expr);                                                                  \
        if (e_ != hipSuccess) {                                                                  \
            ::ptoamd::set_error("%s failed: %s (%s:%d)", #expr, hipGetErrorString(e_), __FILE__, __LINE__); \
            return PTOAMD_E_HIP;                                                                 \
        }                                                                                        \
    } while (0)

#define PTOAMD_REQUIRE(cond, code, ...)         \
    do {                                        \
        if (!(cond)) {                          \
            ::ptoamd::set_error(__VA_ARGS__);   \
            return (code);                      \
        }                                       \
    } while (0)

}  // namespace ptoamd
