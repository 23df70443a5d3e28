// The one-byte MX element types (float8_e4m3_t, float8_e5m2_t, float8_e8m0_t, float4_e2m1x2_t, float4_e1m2x2_t) that
// kernel sources reach through "pto/cpu/MXTypes.hpp" (reference: include/pto/cpu/MXTypes.hpp:339-345); on this
// backend they are storage types declared in pto/amd/base.hpp, decoded in registers (pto/amd/device_types.hpp).
#pragma once
#include "../amd/base.hpp"
