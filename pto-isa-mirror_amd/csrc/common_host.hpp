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

inline hipStream_t as_stream(void* s) { return reinterpret_cast<hipStream_t>(s); }

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
