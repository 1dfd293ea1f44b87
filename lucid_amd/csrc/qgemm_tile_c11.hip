// Tile kernel instances of one shape (CfgBig8); see qgemm_tile.hpp.
#include "qgemm_tile.hpp"

LQ_DEFINE_TILE_LAUNCHER(launch_tile_c11, CfgBig8, false)
