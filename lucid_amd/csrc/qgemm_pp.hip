// Instances of the eight-wavefront ping-pong GEMM kernel; see qgemm_pp.hpp.
#include "qgemm_pp.hpp"

namespace lq {

// which: 0 = 256 x 352 tiles (N = 11008 is 32 of them wide less a sliver: with M = 2048 exactly
// one tile per CU), 1 = 256 x 256 tiles, 2 = 256 x 192 tiles (N = 768 as four columns of tiles:
// 200 tiles for 12 608 rows where 256-wide ones give 150 for the 256 CUs), 3 = 224 x 192 and
// 4 = 160 x 256 tiles (more, smaller tiles for the same shapes)
int launch_pp_shape(const GemmArgs& g, int which, hipStream_t st) {
    switch (which) {
    case 0: return launch_pp<PPCfg352>(g, st);
    case 1: return launch_pp<PPCfg256>(g, st);
    case 2: return launch_pp<PPCfg192>(g, st);
    case 3: return launch_pp<PPCfg224x192>(g, st);
    default: return launch_pp<PPCfg160x256>(g, st);
    }
}

}  // namespace lq
