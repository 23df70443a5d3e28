// gemm_tile_kernel instantiated for OpI8
#define PTOAMD_TILE_OP OpI8
#define PTOAMD_TILE_OP16 OpI8x16
#define PTOAMD_TILE_RAGGED_K
#define PTOAMD_TILE_FN launch_gemm_tile_i8
#include "gemm_tile_inst.hpp"
