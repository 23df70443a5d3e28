// gemm_tile_kernel instantiated for OpF16
#define PTOAMD_TILE_OP OpF16
#define PTOAMD_TILE_OP16 OpF16x16
#define PTOAMD_TILE_RAGGED_K
#define PTOAMD_TILE_FN launch_gemm_tile_f16
#include "gemm_tile_inst.hpp"
