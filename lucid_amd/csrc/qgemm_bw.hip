// Instances of the one-wavefront-per-SIMD GEMM kernel; see qgemm_bw.hpp.
#include "qgemm_bw.hpp"

namespace lq {

int launch_bw_shape(const GemmArgs& g, int which, hipStream_t st) {
    (void)which;
    LQ_REQUIRE(g.K >= 256 && g.K % 128 == 0, LQ_ERR_SHAPE,
               "one-wavefront-per-SIMD kernel: K = %d is not a multiple of 128 (or below 256)", g.K);
    LQ_REQUIRE(size_t(g.M) * g.K < 0xffffffffull && size_t(g.N) * g.K < 0xffffffffull, LQ_ERR_SHAPE,
               "one-wavefront-per-SIMD kernel: an operand of 4 GiB or more");
    LQ_REQUIRE(!g.gelu && g.range == nullptr, LQ_ERR_NOT_IMPLEMENTED,
               "one-wavefront-per-SIMD kernel: GELU / kept range are not built for it");
    switch (g.out_mode) {
    case OUT_F16: return launch_bw_mode<BWCfg352, OUT_F16>(g, st);
    case OUT_ACC_I32: return launch_bw_mode<BWCfg352, OUT_ACC_I32>(g, st);
    default: return fail(LQ_ERR_NOT_IMPLEMENTED, "one-wavefront-per-SIMD kernel: output mode %d", g.out_mode);
    }
}

}  // namespace lq
