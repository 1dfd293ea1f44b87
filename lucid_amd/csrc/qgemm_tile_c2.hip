// Tile kernel instances of one shape (CfgBig64); see qgemm_tile.hpp.
#include "qgemm_tile.hpp"

LQ_DEFINE_TILE_LAUNCHER(launch_tile_c2, CfgBig64, false)
