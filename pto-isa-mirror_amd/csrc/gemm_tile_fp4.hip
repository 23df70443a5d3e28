// gemm_tile_kernel instantiated for OpFP4
#define PTOAMD_TILE_OP OpFP4
#define PTOAMD_TILE_RING3
#define PTOAMD_TILE_FN launch_gemm_tile_fp4
#include "gemm_tile_inst.hpp"
