// Tile kernel instances of one shape (CfgN64); see qgemm_tile.hpp.
#include "qgemm_tile.hpp"

LQ_DEFINE_TILE_LAUNCHER(launch_tile_c6, CfgN64, true)
