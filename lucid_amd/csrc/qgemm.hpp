// Internal interface between the GEMM / convolution translation units.
#pragma once
#include "common.hpp"

namespace lq {

enum { OUT_ACC_I32 = 0, OUT_F32 = 1, OUT_F16 = 2, OUT_REQUANT_I8 = 3, OUT_FAKEQUANT_F32 = 4 };
// Internal variant of OUT_F32 (never an ABI value): float32 output with a GELU and / or a
// kept range.  A template mode of its own, so that the plain float epilogue carries neither.
constexpr int OUT_F32X = 5;
// Likewise OUT_REQUANT_I8 followed by the fused join on codes.
constexpr int OUT_REQUANT_JOIN = 6;

struct GemmArgs {
    const int8_t* a;      // [M,K] activation codes as stored
    const int8_t* w;      // [N,K] weight codes
    int M, N, K;
    const int32_t* wsum;  // [N] sum_k w[n,k]; may be null when a_zp == 0
    int a_zp;             // zero point of the stored activation codes
    const float* a_zp_dev; // optional device scalar: effective zero point = int(*a_zp_dev) + a_zp
    const float* a_scale; // [M] or [1]
    int a_scale_per_row;
    const float* w_scale; // [N]
    const void* bias;     // [N] f32 / f16, or null
    int bias_dtype;
    int relu;
    int out_mode;
    const float* out_scale;  // device scalars, used by the two requantizing modes
    const float* out_zp;
    int out_qmin, out_qmax, out_offset;
    void* out;            // [M, ldo]
    long ldo;
    const float* residual;  // optional [M, ldr] float32 added to y after the activation (float outputs only)
    long ldr;
    int gelu;             // OUT_F32: exact-erf GELU after the bias / ReLU (before a residual)
    float* range;         // OUT_F32, one block per tile: min / max of the stored tile go to the block's slot
                          // (either one selects the OUT_F32X instance of the kernels)
    // Optional join on codes after the requantize (OUT_REQUANT_I8 only): the layer's code
    // and join_q[m, n] are dequantized with their own grids, added, optionally clamped at
    // zero, and requantized to (join_out_*): QFunctional.add / add_relu fused in.
    const int8_t* join_q;   // [M, join_ld] stored codes, or null
    long join_ld;
    int join_off;           // storage offset of join_q's codes
    const float* join_scale;
    const float* join_zp;
    int join_relu;
    const float* join_out_scale;
    const float* join_out_zp;
    int join_out_qmin, join_out_qmax, join_out_offset;
    const int8_t* zeros;  // >= 16 zero bytes, source for K-tail chunks
    // Implicit-GEMM convolution (tile kernel instantiated with CONV = 1): the
    // A operand is gathered from NHWC activation codes; row m is output pixel
    // (b, oh, ow), column k is ((kh*KW + kw)*Cg + ci).  N is then the output
    // channels of ONE group and blockIdx.y selects the group.
    const int8_t* cx;       // NHWC codes
    const int8_t* pad_src;  // 16 bytes holding the zero-point code (out-of-image taps)
    int cH, cW, cCin, cOH, cOW, cKW, cCg, csh, csw, cph, cpw, cdh, cdw;
    // CONV = 2, volumetric: NDHWC codes, row m is output voxel (b, od, oh, ow), column k is
    // (((kd*KH + kh)*KW + kw)*Cg + ci)
    int cD, cOD, cKH, csd, cpd, cdd;
    // stream-K scratch (set by the launcher)
    int* sk_counters;
    int32_t* sk_slabs;
    int sk_tiles;  // the last sk_tiles tile ids are shared between workers
};


// Validates a join description against the output mode and copies it into g
// (ld 0 = n_cols).
inline int set_join(GemmArgs& g, const lq_join_args& j, int out_mode, long n_cols, const char* who) {
    g.join_q = nullptr;
    if (j.q == nullptr) return LQ_OK;
    LQ_REQUIRE(out_mode == OUT_REQUANT_I8, LQ_ERR_VALUE, "%s: a join on codes needs out_mode REQUANT_I8", who);
    LQ_REQUIRE(j.scale && j.zp && j.out_scale && j.out_zp, LQ_ERR_VALUE, "%s: join qparams are NULL", who);
    LQ_REQUIRE(j.out_qmin <= j.out_qmax && j.out_qmin + j.out_offset >= -128 && j.out_qmax + j.out_offset <= 127,
               LQ_ERR_VALUE, "%s: join output grid [%d,%d] + offset %d does not fit int8", who, j.out_qmin,
               j.out_qmax, j.out_offset);
    const long ld = j.ld ? j.ld : n_cols;
    LQ_REQUIRE(ld >= n_cols, LQ_ERR_SHAPE, "%s: join row stride %ld < %ld columns", who, ld, n_cols);
    g.join_q = j.q; g.join_ld = ld; g.join_off = j.offset; g.join_scale = j.scale; g.join_zp = j.zp;
    g.join_relu = j.relu; g.join_out_scale = j.out_scale; g.join_out_zp = j.out_zp;
    g.join_out_qmin = j.out_qmin; g.join_out_qmax = j.out_qmax; g.join_out_offset = j.out_offset;
    return LQ_OK;
}

// 256 blocks of 16 bytes; block v is filled with byte value v.  Block 0 is the
// zero source for K-tail chunks, block (uint8)zp the source for out-of-image
// convolution taps.
int pad_table(const int8_t** table);

// Launches the MFMA tile kernel on a filled-in GemmArgs.  conv = 1 gathers the A operand
// from NHWC codes, conv = 2 from NDHWC codes (cx / c* fields); `groups` becomes gridDim.y.
// The volumetric gather is built for tile shapes 3, 5, 6 and 9, one block per tile.
int run_tile_kernel(const GemmArgs& g, int conv, int groups, int tile_config, hipStream_t st);


// Chooses between the tile, skinny and naive kernels (force_path: 0 = choose,
// 1 = tile, 2 = skinny, 3 = naive) and launches.
int run_gemm(const GemmArgs& g, int force_path, int tile_config, hipStream_t st);

// Second pass of a layer whose weight codes are affine (zero points w_zp[n]).  acc is the
// raw [M, N] sum_k a*w (contiguous), asum[m * asum_ld + n / n_per_group] the sum of the
// activation codes that met column n's weights (kdot of them).  Forms
//     acc - a_zp*wsum[n] - w_zp[n]*asum + kdot*a_zp*w_zp[n]
// and stores it through the epilogue that g describes (g.out / g.ldo / g.out_mode ...).
int launch_affine_fixup(const GemmArgs& g, const int32_t* acc, const int32_t* asum, int asum_ld,
                        int n_per_group, const int32_t* w_zp, int kdot, hipStream_t st);

}  // namespace lq
