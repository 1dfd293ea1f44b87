// Float32 2-d convolution for the calibration pass of a prepared model and the forward of
// the QAT layers: im2col + GEMM, as Lucid's CPU path does it
// (IBackend::conv_nd_forward, CpuBackend.h:8124-8257; Im2Col.cpp:59-100; zero padding in the
// float domain).  One-off work next to the int8 inference path, so it is built from the float
// GEMM already here rather than a kernel of its own.
#include "common.hpp"

using namespace lq;

namespace {

// patches[m, (c, kh, kw)] for the channels [c0, c0 + cg) of an NCHW image; m = (b, oh, ow).
// The column order is that of a filter [cg, KH, KW] flattened, so the GEMM's second operand
// is the OIHW weight as it lies.
__global__ __launch_bounds__(256) void im2col_nchw_f32_kernel(const float* __restrict__ x, float* __restrict__ out,
                                                              int B, int C, int H, int W, int KH, int KW, int sh,
                                                              int sw, int ph, int pw, int dh, int dw, int OH, int OW,
                                                              int c0, int cg) {
    const size_t K = size_t(cg) * KH * KW;
    const size_t total = size_t(B) * OH * OW * K;
    for (size_t i = size_t(blockIdx.x) * 256 + threadIdx.x; i < total; i += size_t(gridDim.x) * 256) {
        const size_t m = i / K;
        const int k = int(i - m * K);
        const int c = k / (KH * KW), r = k - c * (KH * KW), kh = r / KW, kw = r - kh * KW;
        const int ow = int(m % OW), oh = int((m / OW) % OH), b = int(m / (size_t(OW) * OH));
        const int ih = oh * sh - ph + kh * dh, iw = ow * sw - pw + kw * dw;
        float v = 0.0f;
        if (ih >= 0 && ih < H && iw >= 0 && iw < W) v = x[((size_t(b) * C + c0 + c) * H + ih) * W + iw];
        out[i] = v;
    }
}

// rows[m, n] (m = (b, pixel)) -> NCHW channels [c0, c0 + N) of out
__global__ __launch_bounds__(256) void rows_to_nchw_f32_kernel(const float* __restrict__ rows, float* __restrict__ out,
                                                               int B, int P, int N, int Ctot, int c0) {
    const size_t total = size_t(B) * P * N;
    for (size_t i = size_t(blockIdx.x) * 256 + threadIdx.x; i < total; i += size_t(gridDim.x) * 256) {
        // i runs over the output so that the writes are contiguous: (b, n, p)
        const int p = int(i % P), n = int((i / P) % N), b = int(i / (size_t(P) * N));
        out[(size_t(b) * Ctot + c0 + n) * P + p] = rows[(size_t(b) * P + p) * N + n];
    }
}

}  // namespace

extern "C" {

int lq_conv2d_f32(const float* x, const float* w, const float* bias, float* out, int B, int Cin, int H, int W, int Cout,
                  int KH, int KW, int stride_h, int stride_w, int pad_h, int pad_w, int dil_h, int dil_w, int groups,
                  lq_stream stream) {
    LQ_REQUIRE(x && w && out, LQ_ERR_VALUE, "conv2d_f32: NULL pointer");
    LQ_REQUIRE(B >= 0 && Cin > 0 && Cout > 0 && H > 0 && W > 0 && KH > 0 && KW > 0 && groups > 0 &&
                   Cin % groups == 0 && Cout % groups == 0,
               LQ_ERR_SHAPE, "conv2d_f32: bad shape");
    LQ_REQUIRE(stride_h > 0 && stride_w > 0 && dil_h > 0 && dil_w > 0 && pad_h >= 0 && pad_w >= 0, LQ_ERR_VALUE,
               "conv2d_f32: bad geometry");
    const int OH = (H + 2 * pad_h - dil_h * (KH - 1) - 1) / stride_h + 1;  // ConvNd.cpp:56-59
    const int OW = (W + 2 * pad_w - dil_w * (KW - 1) - 1) / stride_w + 1;
    LQ_REQUIRE(OH > 0 && OW > 0, LQ_ERR_SHAPE, "conv2d_f32: empty output (%d x %d)", OH, OW);
    if (B == 0) return LQ_OK;
    const int cg = Cin / groups, ng = Cout / groups;
    const size_t M = size_t(B) * OH * OW, K = size_t(cg) * KH * KW;
    LQ_REQUIRE(M <= 0x7fffffffull && K <= 0x7fffffffull, LQ_ERR_SHAPE, "conv2d_f32: problem too large");
    float* patches = nullptr;
    float* rows = nullptr;
    int rc = lq_alloc(reinterpret_cast<void**>(&patches), M * K * sizeof(float));
    if (rc) return rc;
    rc = lq_alloc(reinterpret_cast<void**>(&rows), M * size_t(ng) * sizeof(float));
    if (rc) {
        (void)lq_free(patches);
        return rc;
    }
    hipStream_t st = as_stream(stream);
    auto blocks = [](size_t n) { return unsigned(n / 256 + 1 > 65536 ? 65536 : n / 256 + 1); };
    for (int g = 0; g < groups && rc == LQ_OK; ++g) {
        hipLaunchKernelGGL(im2col_nchw_f32_kernel, dim3(blocks(M * K)), dim3(256), 0, st, x, patches, B, Cin, H, W, KH,
                           KW, stride_h, stride_w, pad_h, pad_w, dil_h, dil_w, OH, OW, g * cg, cg);
        rc = lq_sgemm_nt_f32(patches, w + size_t(g) * ng * K, bias ? bias + size_t(g) * ng : nullptr, rows, int(M), ng,
                             int(K), stream);
        if (rc) break;
        hipLaunchKernelGGL(rows_to_nchw_f32_kernel, dim3(blocks(M * ng)), dim3(256), 0, st, rows, out, B, OH * OW, ng,
                           Cout, g * ng);
    }
    // a calibration-time operator: wait for the launches before the scratch goes back to the pool
    const hipError_t e = hipStreamSynchronize(st);
    (void)lq_free(patches);
    (void)lq_free(rows);
    if (rc) return rc;
    LQ_HIP(e);
    return LQ_OK;
}

}  // extern "C"
