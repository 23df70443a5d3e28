// gemm_tile_kernel instantiated for OpBF16
#define PTOAMD_TILE_OP OpBF16
#define PTOAMD_TILE_OP16 OpBF16x16
#define PTOAMD_TILE_RAGGED_K
#define PTOAMD_TILE_FN launch_gemm_tile_bf16
#include "gemm_tile_inst.hpp"
