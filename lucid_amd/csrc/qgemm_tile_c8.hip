// Tile kernel instances of one shape (CfgMid4); see qgemm_tile.hpp.
#include "qgemm_tile.hpp"

LQ_DEFINE_TILE_LAUNCHER(launch_tile_c8, CfgMid4, false)
