// Tile kernel instances of one shape (CfgTall8); see qgemm_tile.hpp.
#include "qgemm_tile.hpp"

LQ_DEFINE_TILE_LAUNCHER(launch_tile_c12, CfgTall8, false)
