// Tile kernel instances of one shape (CfgTall3); see qgemm_tile.hpp.
#include "qgemm_tile.hpp"

LQ_DEFINE_TILE_LAUNCHER(launch_tile_c7, CfgTall3, false)
