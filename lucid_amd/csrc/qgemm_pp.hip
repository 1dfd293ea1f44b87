// Instances of the eight-wavefront ping-pong GEMM kernel; see qgemm_pp.hpp.
#include "qgemm_pp.hpp"

namespace lq {

// which: 0 = 256 x 352 tiles (N = 11008 is 32 of them wide less a sliver: with M = 2048 exactly
// one tile per CU), 1 = 256 x 256 tiles
int launch_pp_shape(const GemmArgs& g, int which, hipStream_t st) {
    return which == 0 ? launch_pp<PPCfg352>(g, st) : launch_pp<PPCfg256>(g, st);
}

}  // namespace lq
