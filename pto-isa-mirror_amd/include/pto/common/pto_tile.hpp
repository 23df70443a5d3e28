// Tile<>, GlobalTensor<>, Shape / Stride, TileShape2D / BaseShape2D and the tile aliases (reference:
// include/pto/common/pto_tile.hpp); on this backend they live in pto/amd/base.hpp and pto/amd/tile.hpp.
#pragma once
#include "../amd/base.hpp"
#include "../amd/tile.hpp"
