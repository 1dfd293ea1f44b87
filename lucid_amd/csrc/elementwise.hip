// Small elementwise members of the quantized path: float ReLU between
// dynamic-quantized layers, running min/max folding for observers, and the
// residual join on codes.
#include "common.hpp"

using namespace lq;

namespace {

// vrelu_f32 (lucid/_C/backend/cpu/Vdsp.cpp:130-133): (x < 0) ? 0 : x, NaN passes.
__global__ __launch_bounds__(256) void relu_f32_kernel(const float* __restrict__ x,
                                                       float* __restrict__ out, size_t n) {
    size_t i = (size_t(blockIdx.x) * 256 + threadIdx.x) * 4;
    const size_t stride = size_t(gridDim.x) * 256 * 4;
    const bool vec = aligned16(x) && aligned16(out);
    for (; i < n; i += stride) {
        if (vec && i + 4 <= n) {
            float4 v = *reinterpret_cast<const float4*>(x + i);
            v.x = v.x < 0.0f ? 0.0f : v.x;
            v.y = v.y < 0.0f ? 0.0f : v.y;
            v.z = v.z < 0.0f ? 0.0f : v.z;
            v.w = v.w < 0.0f ? 0.0f : v.w;
            *reinterpret_cast<float4*>(out + i) = v;
        } else {
            for (size_t e = i; e < n && e < i + 4; ++e) out[e] = x[e] < 0.0f ? 0.0f : x[e];
        }
    }
}

// running = minimum(running, current), running = maximum(running, current)
// with vDSP_vmin / vDSP_vmax semantics (NaN propagates, Vdsp.cpp:140-151);
// `current` may be a single value broadcast over C (scalar seed, observer.py:649-651).
__global__ void minmax_fold_kernel(float* run_min, float* run_max, const float* cur_min,
                                   const float* cur_max, size_t C, int run_is_scalar,
                                   float* out_min, float* out_max) {
    size_t c = size_t(blockIdx.x) * blockDim.x + threadIdx.x;
    if (c >= C) return;
    const float rmn = run_min[run_is_scalar ? 0 : c], rmx = run_max[run_is_scalar ? 0 : c];
    const float cmn = cur_min[c], cmx = cur_max[c];
    const float qnan = __builtin_nanf("");
    out_min[c] = (rmn != rmn || cmn != cmn) ? qnan : (rmn < cmn ? rmn : cmn);
    out_max[c] = (rmx != rmx || cmx != cmx) ? qnan : (rmx > cmx ? rmx : cmx);
}

// y[m, n] = act(y[m, n] + bias[n]) in place: the float bias and optional ReLU that
// follow the weight-only matmul (lucid/nn/quantized/mlx_linear.py forward).
__global__ __launch_bounds__(256) void bias_act_kernel(float* __restrict__ y, const float* __restrict__ bias,
                                                       size_t total, int N, int relu) {
    const size_t i = size_t(blockIdx.x) * 256 + threadIdx.x;
    if (i >= total) return;
    float v = y[i];
    if (bias) v = v + bias[i % N];
    if (relu) v = (v < 0.0f) ? 0.0f : v;
    y[i] = v;
}

// Moving-average observers (lucid/quantization/observer.py:490-506,1000-1018):
// new = seed ? cur : run + c * (cur - run), float32 steps in that order.
// Per-tensor (mode 0): seed where the running minimum is infinite, elementwise.
// Per-channel (mode 1): seed everything when EVERY running minimum is infinite
// (the scalar +-inf start), else average everything.  One block.
__global__ __launch_bounds__(1024) void minmax_ema_kernel(const float* run_min, const float* run_max,
                                                          const float* cur_min, const float* cur_max, size_t C,
                                                          int run_is_scalar, int mode, float c, float* out_min,
                                                          float* out_max) {
    __shared__ int s_not_inf;
    if (threadIdx.x == 0) s_not_inf = 0;
    __syncthreads();
    if (mode == 1) {
        const size_t nrun = run_is_scalar ? 1 : C;
        int any = 0;
        for (size_t i = threadIdx.x; i < nrun; i += 1024) any |= !isinf(run_min[i]);
        if (any) atomicOr(&s_not_inf, 1);
        __syncthreads();
    }
    const bool seed_all = mode == 1 && s_not_inf == 0;
    for (size_t i = threadIdx.x; i < C; i += 1024) {
        const float rmn = run_min[run_is_scalar ? 0 : i], rmx = run_max[run_is_scalar ? 0 : i];
        const float cmn = cur_min[i], cmx = cur_max[i];
        const bool seed = mode == 1 ? seed_all : isinf(rmn);
        const float dmn = cmn - rmn, dmx = cmx - rmx;
        const float emn = c * dmn, emx = c * dmx;
        out_min[i] = seed ? cmn : rmn + emn;
        out_max[i] = seed ? cmx : rmx + emx;
    }
}

// lucid.histc (CpuBackend.h:13276-13316): `bins` equal-width buckets over
// [lo, hi] in double arithmetic, bin = (int64)((v - lo) / step) with the right
// edge folded into the last bin, values outside the range skipped.  Counts are
// exact integers (LDS then global atomics) and leave as float32.
__global__ __launch_bounds__(256) void histc_kernel(const float* __restrict__ x, size_t n, double lo, double hi,
                                                    double step, int bins,
                                                    unsigned long long* __restrict__ counts) {
    extern __shared__ unsigned s_hist[];
    for (int b = threadIdx.x; b < bins; b += 256) s_hist[b] = 0;
    __syncthreads();
    const size_t stride = size_t(gridDim.x) * 256;
    for (size_t i = size_t(blockIdx.x) * 256 + threadIdx.x; i < n; i += stride) {
        const double v = double(x[i]);
        if (v < lo || v > hi) continue;  // NaN fails neither test in C++; see below
        long long bin = (long long)((v - lo) / step);
        if (bin >= bins) bin = bins - 1;
        if (bin >= 0) atomicAdd(&s_hist[bin], 1u);
    }
    __syncthreads();
    for (int b = threadIdx.x; b < bins; b += 256)
        if (s_hist[b]) atomicAdd(&counts[b], (unsigned long long)s_hist[b]);
}

__global__ void histc_finish_kernel(const unsigned long long* counts, int bins, float* out) {
    const int b = blockIdx.x * blockDim.x + threadIdx.x;
    if (b < bins) out[b] = float(double(counts[b]));  // the reference counts in double, then casts
}

__device__ __forceinline__ float q_core(float x, float s, float z, float lo, float hi) {
    float t = x / s;
    float r = __builtin_rintf(t);
    float u = r + z;
    u = (u < lo) ? lo : ((u > hi) ? hi : u);
    return u;
}

// fq(relu(x + y)) on codes (lucid/nn/quantized/functional_module.py:224-230):
// x = (qa - za)*sa, y = (qb - zb)*sb, each a float32 step, then the usual requantize.
__global__ __launch_bounds__(256) void add_requant_kernel(const int8_t* __restrict__ qa, int a_off,
                                                          const float* sa, const float* za,
                                                          const int8_t* __restrict__ qb, int b_off,
                                                          const float* sb, const float* zb,
                                                          size_t n, int relu, const float* S_,
                                                          const float* Z_, float lo, float hi,
                                                          int out_off, int8_t* __restrict__ out) {
    const float s_a = sa[0], z_a = za[0], s_b = sb[0], z_b = zb[0], S = S_[0], Z = Z_[0];
    size_t i = (size_t(blockIdx.x) * 256 + threadIdx.x) * 4;
    const size_t stride = size_t(gridDim.x) * 256 * 4;
    const bool vec = (reinterpret_cast<uintptr_t>(qa) | reinterpret_cast<uintptr_t>(qb) |
                      reinterpret_cast<uintptr_t>(out)) % 4 == 0;
    for (; i < n; i += stride) {
        int8_t a[4], b[4], o[4];
        const int cnt = n - i < 4 ? int(n - i) : 4;
        if (vec && cnt == 4) {
            *reinterpret_cast<uint32_t*>(a) = *reinterpret_cast<const uint32_t*>(qa + i);
            *reinterpret_cast<uint32_t*>(b) = *reinterpret_cast<const uint32_t*>(qb + i);
        } else {
            for (int e = 0; e < cnt; ++e) { a[e] = qa[i + e]; b[e] = qb[i + e]; }
        }
        for (int e = 0; e < cnt; ++e) {
            float xa = (float(int(a[e]) - a_off) - z_a) * s_a;
            float xb = (float(int(b[e]) - b_off) - z_b) * s_b;
            float y = xa + xb;
            if (relu) y = (y < 0.0f) ? 0.0f : y;
            float qv = q_core(y, S, Z, lo, hi);
            o[e] = int8_t(((qv != qv) ? 0 : int(qv)) + out_off);
        }
        if (vec && cnt == 4)
            *reinterpret_cast<uint32_t*>(out + i) = *reinterpret_cast<const uint32_t*>(o);
        else
            for (int e = 0; e < cnt; ++e) out[i + e] = o[e];
    }
}

// fq(act(x OP y)) on codes with OP in {add, mul} and y either a second code tensor
// or a float scalar (QFunctional.add / mul / add_relu / add_scalar / mul_scalar,
// lucid/nn/quantized/functional_module.py:224-246): dequantize each operand with
// its own float32 steps, apply OP in float32, requantize.
__global__ __launch_bounds__(256) void binary_requant_kernel(int op, const int8_t* __restrict__ qa, int a_off,
                                                             const float* sa, const float* za,
                                                             const int8_t* __restrict__ qb, int b_off,
                                                             const float* sb, const float* zb, float scalar,
                                                             size_t n, int relu, const float* S_, const float* Z_,
                                                             float lo, float hi, int out_off,
                                                             int8_t* __restrict__ out) {
    const float s_a = sa[0], z_a = za[0], S = S_[0], Z = Z_[0];
    const float s_b = qb ? sb[0] : 1.0f, z_b = qb ? zb[0] : 0.0f;
    const size_t stride = size_t(gridDim.x) * 256;
    for (size_t i = size_t(blockIdx.x) * 256 + threadIdx.x; i < n; i += stride) {
        const float xa = (float(int(qa[i]) - a_off) - z_a) * s_a;
        const float xb = qb ? (float(int(qb[i]) - b_off) - z_b) * s_b : scalar;
        float y = op == 0 ? xa + xb : xa * xb;
        if (relu) y = (y < 0.0f) ? 0.0f : y;
        const float qv = q_core(y, S, Z, lo, hi);
        out[i] = int8_t(((qv != qv) ? 0 : int(qv)) + out_off);
    }
}

// One operand of a quantized concatenation: codes [rows, cols] on their own grid
// re-expressed on the output grid, written at row stride out_ld (the operand's
// column slot inside the concatenated rows).
__global__ __launch_bounds__(256) void requant_rows_kernel(const int8_t* __restrict__ q, int off, const float* s_,
                                                           const float* z_, size_t rows, size_t cols,
                                                           int8_t* __restrict__ out, size_t out_ld, const float* S_,
                                                           const float* Z_, float lo, float hi, int out_off) {
    const float s = s_[0], z = z_[0], S = S_[0], Z = Z_[0];
    const size_t n = rows * cols, stride = size_t(gridDim.x) * 256;
    for (size_t i = size_t(blockIdx.x) * 256 + threadIdx.x; i < n; i += stride) {
        const size_t r = i / cols, c = i - r * cols;
        const float x = (float(int(q[i]) - off) - z) * s;
        const float qv = q_core(x, S, Z, lo, hi);
        out[r * out_ld + c] = int8_t(((qv != qv) ? 0 : int(qv)) + out_off);
    }
}

// Global average pool of NHWC codes to float32 [B, C]: the exact integer sum of
// the codes, then ((sum - HW*(Z + off)) * S) / HW in float32.
__global__ __launch_bounds__(256) void global_avgpool_nhwc_kernel(const int8_t* __restrict__ q, int off,
                                                                  int B, int HW, int C,
                                                                  const float* scale, const float* zp,
                                                                  float* __restrict__ out) {
    const int c = blockIdx.x * 64 + (threadIdx.x & 63), b = blockIdx.y;
    const int part = threadIdx.x >> 6;  // 4 slices of the pixels
    __shared__ int red[4][64];
    int s = 0;
    if (c < C) {
#pragma unroll 8
        for (int p = part; p < HW; p += 4) s += q[(size_t(b) * HW + p) * C + c];  // (unrolled: the loads go out together)
    }
    red[part][threadIdx.x & 63] = s;
    __syncthreads();
    if (part == 0 && c < C) {
        s = red[0][threadIdx.x] + red[1][threadIdx.x] + red[2][threadIdx.x] + red[3][threadIdx.x];
        const float total = float(s - off * HW) - float(HW) * zp[0];
        out[size_t(b) * C + c] = (total * scale[0]) / float(HW);
    }
}

// Quantized Linear on a float activation that is NOT on a grid (Lucid's own
// formulation, lucid/nn/quantized/linear.py:199-215): y = x @ dequant(W)^T + b.
// One wavefront per output; lanes stride over k and the partial sums are
// folded by a butterfly, so the float summation order differs from a
// sequential loop (Lucid's own order is Accelerate's and is not pinned either).
__global__ __launch_bounds__(256) void qlinear_w8a32_kernel(
    const float* __restrict__ x, const int8_t* __restrict__ w, const float* __restrict__ w_scale,
    const float* __restrict__ w_zp, const float* __restrict__ bias, int M, int N, int K, int relu,
    int do_fq, const float* S_, const float* Z_, float lo, float hi, float* __restrict__ out) {
    const int lane = threadIdx.x & 63;
    const size_t o = size_t(blockIdx.x) * 4 + (threadIdx.x >> 6);
    if (o >= size_t(M) * N) return;
    const int m = int(o / N), n = int(o % N);
    const float ws = w_scale[n], wz = w_zp[n];
    const float* xr = x + size_t(m) * K;
    const int8_t* wr = w + size_t(n) * K;
    float acc = 0.0f;
    for (int k = lane; k < K; k += 64) {
        const float wv = (float(int(wr[k])) - wz) * ws;  // dequantize, _functional.py:281
        acc = acc + xr[k] * wv;
    }
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) acc = acc + __shfl_xor(acc, d, 64);
    if (lane != 0) return;
    float y = acc;
    if (bias) y = y + bias[n];
    if (relu) y = (y < 0.0f) ? 0.0f : y;
    if (do_fq) {
        const float S = S_[0], Z = Z_[0];
        const float qv = q_core(y, S, Z, lo, hi);
        y = (qv - Z) * S;
    }
    out[o] = y;
}

// The same for a batch of rows: a wavefront owns a 4-column x 8-row patch of the output, so
// that a weight chunk is decoded once for eight rows and an activation chunk is used for four
// columns (K % 4 == 0, 16-byte aligned x, 4-byte aligned w).  A lane takes four consecutive k
// per step; partial sums are folded by the same butterfly.
__global__ __launch_bounds__(256) void qlinear_w8a32_patch_kernel(
    const float* __restrict__ x, const int8_t* __restrict__ w, const float* __restrict__ w_scale,
    const float* __restrict__ w_zp, const float* __restrict__ bias, int M, int N, int K, int relu,
    int do_fq, const float* S_, const float* Z_, float lo, float hi, float* __restrict__ out) {
    constexpr int NT = 4, MT = 8;
    const int lane = threadIdx.x & 63;
    const int n0 = (blockIdx.x * 4 + (threadIdx.x >> 6)) * NT, m0 = blockIdx.y * MT;
    if (n0 >= N) return;
    float ws[NT], wz[NT];
    const int8_t* wr[NT];
#pragma unroll
    for (int j = 0; j < NT; ++j) {
        const int n = n0 + j < N ? n0 + j : N - 1;  // clamped columns are computed and dropped
        ws[j] = w_scale[n], wz[j] = w_zp[n], wr[j] = w + size_t(n) * K;
    }
    const float* xr[MT];
#pragma unroll
    for (int i = 0; i < MT; ++i) xr[i] = x + size_t(m0 + i < M ? m0 + i : M - 1) * K;
    float acc[MT][NT];
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int j = 0; j < NT; ++j) acc[i][j] = 0.0f;
    for (int k = lane * 4; k < K; k += 256) {
        float wv[NT][4];
#pragma unroll
        for (int j = 0; j < NT; ++j) {
            const uint32_t c = *reinterpret_cast<const uint32_t*>(wr[j] + k);
#pragma unroll
            for (int e = 0; e < 4; ++e)
                wv[j][e] = (float(int(int8_t((c >> (8 * e)) & 0xff))) - wz[j]) * ws[j];  // dequantize, _functional.py:281
        }
#pragma unroll
        for (int i = 0; i < MT; ++i) {
            const float4 xv = *reinterpret_cast<const float4*>(xr[i] + k);
#pragma unroll
            for (int j = 0; j < NT; ++j) {
                float a = acc[i][j];
                a = a + xv.x * wv[j][0];
                a = a + xv.y * wv[j][1];
                a = a + xv.z * wv[j][2];
                a = a + xv.w * wv[j][3];
                acc[i][j] = a;
            }
        }
    }
    const float S = do_fq ? S_[0] : 1.0f, Z = do_fq ? Z_[0] : 0.0f;
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int j = 0; j < NT; ++j) {
            float y = acc[i][j];
#pragma unroll
            for (int d = 32; d >= 1; d >>= 1) y = y + __shfl_xor(y, d, 64);
            if (lane != 0 || m0 + i >= M || n0 + j >= N) continue;
            if (bias) y = y + bias[n0 + j];
            if (relu) y = (y < 0.0f) ? 0.0f : y;
            if (do_fq) y = (q_core(y, S, Z, lo, hi) - Z) * S;
            out[size_t(m0 + i) * N + n0 + j] = y;
        }
}

// Long K: the block's four wavefronts share one 4-column x 8-row patch and take every fourth
// 256-wide k step each (four times the loads in flight per output); partial sums meet in
// LDS, then each wavefront folds and stores eight of the 32 outputs.
__global__ __launch_bounds__(256) void qlinear_w8a32_patch_k4_kernel(
    const float* __restrict__ x, const int8_t* __restrict__ w, const float* __restrict__ w_scale,
    const float* __restrict__ w_zp, const float* __restrict__ bias, int M, int N, int K, int relu,
    int do_fq, const float* S_, const float* Z_, float lo, float hi, float* __restrict__ out) {
    constexpr int NT = 4, MT = 8;
    __shared__ float red[4][MT * NT][64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int n0 = blockIdx.x * NT, m0 = blockIdx.y * MT;
    float ws[NT], wz[NT];
    const int8_t* wr[NT];
#pragma unroll
    for (int j = 0; j < NT; ++j) {
        const int n = n0 + j < N ? n0 + j : N - 1;  // clamped columns are computed and dropped
        ws[j] = w_scale[n], wz[j] = w_zp[n], wr[j] = w + size_t(n) * K;
    }
    const float* xr[MT];
#pragma unroll
    for (int i = 0; i < MT; ++i) xr[i] = x + size_t(m0 + i < M ? m0 + i : M - 1) * K;
    float acc[MT][NT];
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int j = 0; j < NT; ++j) acc[i][j] = 0.0f;
    for (int k = wave * 256 + lane * 4; k < K; k += 1024) {
        float wv[NT][4];
#pragma unroll
        for (int j = 0; j < NT; ++j) {
            const uint32_t c = *reinterpret_cast<const uint32_t*>(wr[j] + k);
#pragma unroll
            for (int e = 0; e < 4; ++e)
                wv[j][e] = (float(int(int8_t((c >> (8 * e)) & 0xff))) - wz[j]) * ws[j];  // dequantize, _functional.py:281
        }
#pragma unroll
        for (int i = 0; i < MT; ++i) {
            const float4 xv = *reinterpret_cast<const float4*>(xr[i] + k);
#pragma unroll
            for (int j = 0; j < NT; ++j) {
                float a = acc[i][j];
                a = a + xv.x * wv[j][0];
                a = a + xv.y * wv[j][1];
                a = a + xv.z * wv[j][2];
                a = a + xv.w * wv[j][3];
                acc[i][j] = a;
            }
        }
    }
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int j = 0; j < NT; ++j) red[wave][i * NT + j][lane] = acc[i][j];
    __syncthreads();
    const float S = do_fq ? S_[0] : 1.0f, Z = do_fq ? Z_[0] : 0.0f;
#pragma unroll
    for (int o = 0; o < 8; ++o) {
        const int idx = wave * 8 + o, i = idx / NT, j = idx % NT;
        float y = ((red[0][idx][lane] + red[1][idx][lane]) + red[2][idx][lane]) + red[3][idx][lane];
#pragma unroll
        for (int d = 32; d >= 1; d >>= 1) y = y + __shfl_xor(y, d, 64);
        if (lane != 0 || m0 + i >= M || n0 + j >= N) continue;
        if (bias) y = y + bias[n0 + j];
        if (relu) y = (y < 0.0f) ? 0.0f : y;
        if (do_fq) y = (q_core(y, S, Z, lo, hi) - Z) * S;
        out[size_t(m0 + i) * N + n0 + j] = y;
    }
}

inline unsigned grid_for(size_t n, size_t per_block) {
    size_t b = (n + per_block - 1) / per_block;
    if (b < 1) b = 1;
    return unsigned(b > 65536 ? 65536 : b);
}

}  // namespace

extern "C" {

int lq_relu_f32(const float* x, float* out, size_t n, lq_stream stream) {
    if (n == 0) return LQ_OK;
    LQ_REQUIRE(x && out, LQ_ERR_VALUE, "relu_f32: NULL pointer");
    hipLaunchKernelGGL(relu_f32_kernel, dim3(grid_for(n, 1024)), dim3(256), 0, as_stream(stream), x, out,
                       n);
    LQ_CHECK_LAUNCH("relu_f32");
    return LQ_OK;
}

int lq_minmax_fold(const float* run_min, const float* run_max, const float* cur_min,
                   const float* cur_max, size_t C, int run_is_scalar, float* out_min,
                   float* out_max, lq_stream stream) {
    if (C == 0) return LQ_OK;
    LQ_REQUIRE(run_min && run_max && cur_min && cur_max && out_min && out_max, LQ_ERR_VALUE,
               "minmax_fold: NULL pointer");
    hipLaunchKernelGGL(minmax_fold_kernel, dim3(unsigned((C + 255) / 256)), dim3(256), 0,
                       as_stream(stream), const_cast<float*>(run_min), const_cast<float*>(run_max),
                       cur_min, cur_max, C, run_is_scalar, out_min, out_max);
    LQ_CHECK_LAUNCH("minmax_fold");
    return LQ_OK;
}

int lq_bias_act_f32(float* y, const float* bias, size_t M, int N, int relu, lq_stream stream) {
    if (M * size_t(N) == 0) return LQ_OK;
    LQ_REQUIRE(y && N > 0, LQ_ERR_VALUE, "bias_act: bad arguments");
    const size_t total = M * size_t(N);
    LQ_REQUIRE((total + 255) / 256 < 0x7fffffffull, LQ_ERR_SHAPE, "bias_act: tensor too large");
    hipLaunchKernelGGL(bias_act_kernel, dim3(unsigned((total + 255) / 256)), dim3(256), 0, as_stream(stream), y,
                       bias, total, N, relu);
    LQ_CHECK_LAUNCH("bias_act");
    return LQ_OK;
}

int lq_minmax_ema(const float* run_min, const float* run_max, const float* cur_min, const float* cur_max,
                  size_t C, int run_is_scalar, int per_channel, float averaging_constant, float* out_min,
                  float* out_max, lq_stream stream) {
    if (C == 0) return LQ_OK;
    LQ_REQUIRE(run_min && run_max && cur_min && cur_max && out_min && out_max, LQ_ERR_VALUE,
               "minmax_ema: NULL pointer");
    hipLaunchKernelGGL(minmax_ema_kernel, dim3(1), dim3(1024), 0, as_stream(stream), run_min, run_max, cur_min,
                       cur_max, C, run_is_scalar, per_channel ? 1 : 0, averaging_constant, out_min, out_max);
    LQ_CHECK_LAUNCH("minmax_ema");
    return LQ_OK;
}

int lq_histc_f32(const float* x, size_t n, double lo, double hi, int bins, float* out, lq_stream stream) {
    LQ_REQUIRE(out, LQ_ERR_VALUE, "histc: NULL output");
    LQ_REQUIRE(bins > 0 && bins <= 16384, LQ_ERR_VALUE, "histc: bins must be in 1..16384 (got %d)", bins);
    LQ_REQUIRE(hi > lo, LQ_ERR_VALUE, "histc: hi must be > lo");  // Histogram.cpp:105-106
    LQ_REQUIRE(n == 0 || x, LQ_ERR_VALUE, "histc: NULL input");
    hipStream_t st = as_stream(stream);
    void* ws = nullptr;
    int rc = workspace(size_t(bins) * sizeof(unsigned long long), as_stream(stream), &ws);
    if (rc) return rc;
    auto* counts = static_cast<unsigned long long*>(ws);
    rc = lq_fill_bytes(counts, 0, size_t(bins) * sizeof(unsigned long long), stream);
    if (rc) return rc;
    if (n) {
        size_t blocks = (n + 256 * 16 - 1) / (256 * 16);
        if (blocks > 4096) blocks = 4096;
        hipLaunchKernelGGL(histc_kernel, dim3(unsigned(blocks)), dim3(256), size_t(bins) * sizeof(unsigned), st, x,
                           n, lo, hi, (hi - lo) / double(bins), bins, counts);
        LQ_CHECK_LAUNCH("histc");
    }
    hipLaunchKernelGGL(histc_finish_kernel, dim3(unsigned((bins + 255) / 256)), dim3(256), 0, st, counts, bins, out);
    LQ_CHECK_LAUNCH("histc_finish");
    return LQ_OK;
}

int lq_add_requant_i8(const int8_t* qa, int a_offset, const float* a_scale, const float* a_zp,
                      const int8_t* qb, int b_offset, const float* b_scale, const float* b_zp,
                      size_t n, int relu, const float* out_scale, const float* out_zp, int out_qmin,
                      int out_qmax, int out_offset, int8_t* out, lq_stream stream) {
    if (n == 0) return LQ_OK;
    LQ_REQUIRE(qa && qb && out && a_scale && a_zp && b_scale && b_zp && out_scale && out_zp,
               LQ_ERR_VALUE, "add_requant_i8: NULL pointer");
    LQ_REQUIRE(out_qmin <= out_qmax && out_qmin + out_offset >= -128 && out_qmax + out_offset <= 127,
               LQ_ERR_VALUE, "add_requant_i8: output grid [%d,%d] + offset %d does not fit int8",
               out_qmin, out_qmax, out_offset);
    hipLaunchKernelGGL(add_requant_kernel, dim3(grid_for(n, 1024)), dim3(256), 0, as_stream(stream), qa,
                       a_offset, a_scale, a_zp, qb, b_offset, b_scale, b_zp, n, relu, out_scale, out_zp,
                       float(out_qmin), float(out_qmax), out_offset, out);
    LQ_CHECK_LAUNCH("add_requant_i8");
    return LQ_OK;
}

int lq_binary_requant_i8(int op, const int8_t* qa, int a_offset, const float* a_scale, const float* a_zp,
                         const int8_t* qb, int b_offset, const float* b_scale, const float* b_zp, float scalar,
                         size_t n, int relu, const float* out_scale, const float* out_zp, int out_qmin,
                         int out_qmax, int out_offset, int8_t* out, lq_stream stream) {
    if (n == 0) return LQ_OK;
    LQ_REQUIRE(op == 0 || op == 1, LQ_ERR_VALUE, "binary_requant_i8: op must be 0 (add) or 1 (mul)");
    LQ_REQUIRE(qa && out && a_scale && a_zp && out_scale && out_zp && (!qb || (b_scale && b_zp)), LQ_ERR_VALUE,
               "binary_requant_i8: NULL pointer");
    LQ_REQUIRE(out_qmin <= out_qmax && out_qmin + out_offset >= -128 && out_qmax + out_offset <= 127,
               LQ_ERR_VALUE, "binary_requant_i8: output grid [%d,%d] + offset %d does not fit int8", out_qmin,
               out_qmax, out_offset);
    hipLaunchKernelGGL(binary_requant_kernel, dim3(grid_for(n, 256)), dim3(256), 0, as_stream(stream), op, qa,
                       a_offset, a_scale, a_zp, qb, b_offset, b_scale, b_zp, scalar, n, relu, out_scale, out_zp,
                       float(out_qmin), float(out_qmax), out_offset, out);
    LQ_CHECK_LAUNCH("binary_requant_i8");
    return LQ_OK;
}

int lq_requant_rows_i8(const int8_t* q, int q_offset, const float* scale, const float* zp, size_t rows,
                       size_t cols, int8_t* out, size_t out_ld, const float* out_scale, const float* out_zp,
                       int out_qmin, int out_qmax, int out_offset, lq_stream stream) {
    if (rows * cols == 0) return LQ_OK;
    LQ_REQUIRE(q && out && scale && zp && out_scale && out_zp, LQ_ERR_VALUE, "requant_rows_i8: NULL pointer");
    LQ_REQUIRE(out_ld >= cols, LQ_ERR_SHAPE, "requant_rows_i8: output row stride smaller than the row");
    LQ_REQUIRE(out_qmin <= out_qmax && out_qmin + out_offset >= -128 && out_qmax + out_offset <= 127,
               LQ_ERR_VALUE, "requant_rows_i8: output grid [%d,%d] + offset %d does not fit int8", out_qmin,
               out_qmax, out_offset);
    hipLaunchKernelGGL(requant_rows_kernel, dim3(grid_for(rows * cols, 256)), dim3(256), 0, as_stream(stream), q,
                       q_offset, scale, zp, rows, cols, out, out_ld, out_scale, out_zp, float(out_qmin),
                       float(out_qmax), out_offset);
    LQ_CHECK_LAUNCH("requant_rows_i8");
    return LQ_OK;
}

int lq_global_avgpool_nhwc_i8(const int8_t* q, int code_offset, int B, int H, int W, int C,
                              const float* scale, const float* zp, float* out, lq_stream stream) {
    if (size_t(B) * C == 0) return LQ_OK;
    LQ_REQUIRE(q && scale && zp && out, LQ_ERR_VALUE, "global_avgpool_nhwc_i8: NULL pointer");
    LQ_REQUIRE(H > 0 && W > 0 && size_t(H) * W < (1u << 23), LQ_ERR_SHAPE,
               "global_avgpool_nhwc_i8: bad spatial extent %d x %d", H, W);
    LQ_REQUIRE(B <= 65535, LQ_ERR_SHAPE, "global_avgpool_nhwc_i8: batch too large");
    hipLaunchKernelGGL(global_avgpool_nhwc_kernel, dim3(unsigned((C + 63) / 64), unsigned(B)), dim3(256), 0,
                       as_stream(stream), q, code_offset, B, H * W, C, scale, zp, out);
    LQ_CHECK_LAUNCH("global_avgpool_nhwc_i8");
    return LQ_OK;
}

int lq_qlinear_w8a32(const float* x, const int8_t* w, const float* w_scale, const float* w_zp,
                     const float* bias, int M, int N, int K, int relu, int fake_quantize_out,
                     const float* out_scale, const float* out_zp, int out_qmin, int out_qmax,
                     float* out, lq_stream stream) {
    LQ_REQUIRE(M >= 0 && N >= 0 && K >= 0, LQ_ERR_SHAPE, "qlinear_w8a32: negative extent");
    if (size_t(M) * N == 0) return LQ_OK;
    LQ_REQUIRE(out && w_scale && w_zp && (K == 0 || (x && w)), LQ_ERR_VALUE,
               "qlinear_w8a32: NULL pointer");
    LQ_REQUIRE(!fake_quantize_out || (out_scale && out_zp && out_qmin <= out_qmax), LQ_ERR_VALUE,
               "qlinear_w8a32: output qparams missing");
    const size_t outputs = size_t(M) * N;
    LQ_REQUIRE((outputs + 3) / 4 <= 0x7fffffffull, LQ_ERR_SHAPE, "qlinear_w8a32: too many outputs");
    const bool patch_ok = M >= 4 && K % 4 == 0 && aligned16(x) && (reinterpret_cast<uintptr_t>(w) & 3u) == 0 &&
                          (M + 7) / 8 <= 65535;
    // few patches and a long K: one patch per block, K split between its wavefronts
    if (patch_ok && K >= 1024 && size_t((N + 3) / 4) * size_t((M + 7) / 8) <= 4096) {
        hipLaunchKernelGGL(qlinear_w8a32_patch_k4_kernel, dim3(unsigned((N + 3) / 4), unsigned((M + 7) / 8)), dim3(256),
                           0, as_stream(stream), x, w, w_scale, w_zp, bias, M, N, K, relu, fake_quantize_out,
                           out_scale, out_zp, float(out_qmin), float(out_qmax), out);
        LQ_CHECK_LAUNCH("qlinear_w8a32");
        return LQ_OK;
    }
    if (patch_ok) {
        hipLaunchKernelGGL(qlinear_w8a32_patch_kernel, dim3(unsigned((N + 15) / 16), unsigned((M + 7) / 8)), dim3(256),
                           0, as_stream(stream), x, w, w_scale, w_zp, bias, M, N, K, relu, fake_quantize_out,
                           out_scale, out_zp, float(out_qmin), float(out_qmax), out);
        LQ_CHECK_LAUNCH("qlinear_w8a32");
        return LQ_OK;
    }
    hipLaunchKernelGGL(qlinear_w8a32_kernel, dim3(unsigned((outputs + 3) / 4)), dim3(256), 0,
                       as_stream(stream), x, w, w_scale, w_zp, bias, M, N, K, relu, fake_quantize_out,
                       out_scale, out_zp, float(out_qmin), float(out_qmax), out);
    LQ_CHECK_LAUNCH("qlinear_w8a32");
    return LQ_OK;
}

}  // extern "C"
