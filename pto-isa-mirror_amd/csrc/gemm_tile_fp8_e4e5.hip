// gemm_tile_kernel instantiated for OpFP8<0, 1>
#define PTOAMD_TILE_OP OpFP8<0, 1>
#define PTOAMD_TILE_RING3
#define PTOAMD_TILE_MX16 OpFP8x16<0, 1>
#define PTOAMD_TILE_FN launch_gemm_tile_fp8_e4e5
#include "gemm_tile_inst.hpp"
