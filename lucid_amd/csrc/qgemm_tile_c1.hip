// Tile kernel instances of one shape (CfgBig); see qgemm_tile.hpp.
#include "qgemm_tile.hpp"

LQ_DEFINE_TILE_LAUNCHER(launch_tile_c1, CfgBig, false)
