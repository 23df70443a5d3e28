// PTO tile-instruction API for the gfx950 backend: the header a PTO kernel source includes
// (`#include <pto/pto-inst.hpp>`), reference: include/pto/pto-inst.hpp:11-33.
//
// Execution model.  One PTO "core" is one workgroup of PTO_AMD_THREADS threads.  Mat / Left / Right / Vec / Bias tiles
// live in LDS (the L1 / L0A / L0B / UB / bias-table address spaces are regions of one dynamic LDS arena, and
// TASSIGN's byte address is an offset inside the tile's region); Acc tiles live in registers, spread over the waves as
// MFMA accumulator blocks.  Every T* instruction is a workgroup-collective device function: all threads of the core
// call it with the same arguments.  Event flags (set_flag / wait_flag / pipe_barrier) keep their names; ordering is by
// workgroup barriers inside the instructions.
//
// A kernel source keeps the reference spelling (`__global__ AICORE void Kernel(__gm__ T* out, ...)`): inside this
// header `__global__` marks a core program, which compiles to a device function, and
// `pto::amd::launch<&Kernel<...>>(blocks, stream, args...)` runs it, one workgroup per block.
#pragma once
#include "amd/base.hpp"
#include "amd/tile.hpp"
#include "amd/instr.hpp"
#include "amd/convert.hpp"
#include "amd/quant.hpp"
#include "amd/launch.hpp"
