// Tile kernel instances of one shape (CfgWide); see qgemm_tile.hpp.
#include "qgemm_tile.hpp"

LQ_DEFINE_TILE_LAUNCHER(launch_tile_c3, CfgWide, true)
