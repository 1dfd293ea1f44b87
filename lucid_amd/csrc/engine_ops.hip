// The engine primitives that Lucid's quantization composites are written in, one kernel
// per IBackend call: elementwise binary arithmetic, round, clip, astype, the broadcast
// materialisation, axis min / max reductions, and the eval-mode BatchNorm forward.  The
// fused kernels of the quantize family replace chains of these; they exist so that the
// composite itself (lucid/quantization/_functional.py:180,281) can run on device memory
// call for call, and as the specification the fused kernels are tested against.
#include "common.hpp"

#include <type_traits>

using namespace lq;

namespace {

enum { OP_ADD = 0, OP_SUB = 1, OP_MUL = 2, OP_DIV = 3, OP_MAXIMUM = 4, OP_MINIMUM = 5 };

template <int OP>
__device__ __forceinline__ float binary_value(float a, float b) {
    if (OP == OP_ADD) return a + b;
    if (OP == OP_SUB) return a - b;
    if (OP == OP_MUL) return a * b;
    if (OP == OP_DIV) return a / b;  // IEEE division (vDSP_vdiv, Vdsp.cpp:47-48)
    // vDSP_vmax / vDSP_vmin on float: a NaN in either operand gives NaN (Vdsp.cpp:140-151)
    if (a != a || b != b) return __builtin_nanf("");
    if (OP == OP_MAXIMUM) return a > b ? a : b;
    return a < b ? a : b;
}

template <int OP>
__global__ __launch_bounds__(256) void binary_f32_kernel(const float* __restrict__ a, const float* __restrict__ b,
                                                         float* __restrict__ out, size_t n) {
    size_t i = (size_t(blockIdx.x) * 256 + threadIdx.x) * 4;
    const size_t stride = size_t(gridDim.x) * 256 * 4;
    const bool vec = aligned16(a) && aligned16(b) && aligned16(out);
    for (; i < n; i += stride) {
        if (vec && i + 4 <= n) {
            const float4 x = *reinterpret_cast<const float4*>(a + i);
            const float4 y = *reinterpret_cast<const float4*>(b + i);
            float4 r;
            r.x = binary_value<OP>(x.x, y.x);
            r.y = binary_value<OP>(x.y, y.y);
            r.z = binary_value<OP>(x.z, y.z);
            r.w = binary_value<OP>(x.w, y.w);
            *reinterpret_cast<float4*>(out + i) = r;
        } else {
            for (size_t e = i; e < n && e < i + 4; ++e) out[e] = binary_value<OP>(a[e], b[e]);
        }
    }
}

// mode 0: round half to even (vvnintf, Vforce.cpp:136); mode 1: clip with the float casts
// of the bounds, NaN falling through both comparisons (CpuBackend.h:6880-6891).
template <int MODE>
__global__ __launch_bounds__(256) void unary_f32_kernel(const float* __restrict__ x, float* __restrict__ out, size_t n,
                                                        float lo, float hi) {
    for (size_t i = size_t(blockIdx.x) * 256 + threadIdx.x; i < n; i += size_t(gridDim.x) * 256) {
        float v = x[i];
        if (MODE == 0) {
            v = rintf(v);
        } else {
            if (v < lo)
                v = lo;
            else if (v > hi)
                v = hi;
        }
        out[i] = v;
    }
}

// static_cast between element types (CpuBackend.h:6214-6236).  float -> integer goes
// through int32 with saturation and NaN -> 0 (C leaves both undefined; the quantize
// composite clips first, so neither occurs on its path), then truncates to the width.
__device__ __forceinline__ int32_t float_to_i32(float v) {
    if (v != v) return 0;
    if (v >= 2147483648.0f) return 2147483647;
    if (v <= -2147483648.0f) return int32_t(-2147483647 - 1);
    return int32_t(v);
}

template <typename From, typename To>
__global__ __launch_bounds__(256) void astype_kernel(const From* __restrict__ src, To* __restrict__ dst, size_t n) {
    for (size_t i = size_t(blockIdx.x) * 256 + threadIdx.x; i < n; i += size_t(gridDim.x) * 256) {
        if constexpr (std::is_same<From, float>::value && std::is_integral<To>::value)
            dst[i] = To(float_to_i32(src[i]));
        else if constexpr (std::is_same<From, _Float16>::value && std::is_integral<To>::value)
            dst[i] = To(float_to_i32(float(src[i])));
        else
            dst[i] = To(src[i]);
    }
}

// out[o, c, i] = src[c]: the materialised broadcast of a per-channel operand
// (kernel/BinaryKernel.h:591-606 after _reshape_for_channel, _functional.py:45-54).
__global__ __launch_bounds__(256) void broadcast_f32_kernel(const float* __restrict__ src, float* __restrict__ out,
                                                            size_t total, size_t C, size_t inner) {
    for (size_t i = size_t(blockIdx.x) * 256 + threadIdx.x; i < total; i += size_t(gridDim.x) * 256)
        out[i] = src[(i / inner) % C];
}

// x viewed as [A][R][B], reduced over R: one wavefront per output (a, b).  min and max
// propagate NaN as the reference's reduction does (Reduce.cpp:87-125).
__global__ __launch_bounds__(256) void reduce_mid_minmax_kernel(const float* __restrict__ x, size_t A, size_t R, size_t B,
                                                                float* __restrict__ mn, float* __restrict__ mx) {
    const int lane = threadIdx.x & 63;
    const size_t waves = size_t(gridDim.x) * 4;
    for (size_t o = size_t(blockIdx.x) * 4 + (threadIdx.x >> 6); o < A * B; o += waves) {
        const size_t a = o / B, b = o % B;
        const float* p = x + a * R * B + b;
        float lo = __builtin_inff(), hi = -__builtin_inff();
        bool nan = false;
        for (size_t r = lane; r < R; r += 64) {
            const float v = p[r * B];
            nan |= v != v;
            lo = fminf(lo, v);
            hi = fmaxf(hi, v);
        }
        for (int s = 32; s > 0; s >>= 1) {
            lo = fminf(lo, __shfl_xor(lo, s));
            hi = fmaxf(hi, __shfl_xor(hi, s));
            nan |= __shfl_xor(int(nan), s) != 0;
        }
        if (lane == 0) {
            mn[o] = nan ? __builtin_nanf("") : lo;
            mx[o] = nan ? __builtin_nanf("") : hi;
        }
    }
}

// rstd[c] = 1 / float(sqrt(double(var[c]) + eps)) (CpuBackend.h:9190-9191)
__global__ void batchnorm_rstd_kernel(const float* __restrict__ var, double eps, int C, float* __restrict__ rstd) {
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c < C) rstd[c] = 1.0f / float(sqrt(double(var[c]) + eps));
}

// y = g * (x - m) * r + b per channel, float32 steps in that order (CpuBackend.h:9192-9198).
// A block owns one chunk of one (batch, channel) row, so the four parameters are uniform.
__global__ __launch_bounds__(256) void batchnorm_eval_rows_kernel(const float* __restrict__ x, float* __restrict__ y,
                                                                  size_t rows, int C, size_t inner, size_t chunks,
                                                                  const float* __restrict__ mean,
                                                                  const float* __restrict__ rstd,
                                                                  const float* __restrict__ gamma,
                                                                  const float* __restrict__ beta) {
    constexpr size_t CHUNK = 4096;
    const bool vec = (inner % 4 == 0) && aligned16(x) && aligned16(y);
    for (size_t t = blockIdx.x; t < rows * chunks; t += gridDim.x) {
        const size_t row = t / chunks, chunk = t % chunks;
        const int c = int(row % size_t(C));
        const float m = mean[c], r = rstd[c], g = gamma ? gamma[c] : 1.0f, b = beta ? beta[c] : 0.0f;
        const size_t lo = chunk * CHUNK, hi = lo + CHUNK < inner ? lo + CHUNK : inner;
        const float* xr = x + row * inner;
        float* yr = y + row * inner;
        if (vec) {
            for (size_t i = lo + size_t(threadIdx.x) * 4; i < hi; i += 1024) {
                float4 v = *reinterpret_cast<const float4*>(xr + i);
                v.x = g * (v.x - m) * r + b;
                v.y = g * (v.y - m) * r + b;
                v.z = g * (v.z - m) * r + b;
                v.w = g * (v.w - m) * r + b;
                *reinterpret_cast<float4*>(yr + i) = v;
            }
        } else {
            for (size_t i = lo + threadIdx.x; i < hi; i += 256) yr[i] = g * (xr[i] - m) * r + b;
        }
    }
}

// The same for short rows (a (N, C) input, small feature maps): one element per lane.
__global__ __launch_bounds__(256) void batchnorm_eval_flat_kernel(const float* __restrict__ x, float* __restrict__ y,
                                                                  size_t total, int C, size_t inner,
                                                                  const float* __restrict__ mean,
                                                                  const float* __restrict__ rstd,
                                                                  const float* __restrict__ gamma,
                                                                  const float* __restrict__ beta) {
    for (size_t i = size_t(blockIdx.x) * 256 + threadIdx.x; i < total; i += size_t(gridDim.x) * 256) {
        const int c = int((i / inner) % size_t(C));
        const float g = gamma ? gamma[c] : 1.0f, b = beta ? beta[c] : 0.0f;
        y[i] = g * (x[i] - mean[c]) * rstd[c] + b;
    }
}

inline unsigned grid_for(size_t work_items, size_t per_block) {
    size_t b = (work_items + per_block - 1) / per_block;
    if (b < 1) b = 1;
    return unsigned(b > 65536 ? 65536 : b);
}

template <int OP>
int launch_binary(const float* a, const float* b, float* out, size_t n, lq_stream stream, const char* name) {
    if (n == 0) return LQ_OK;
    LQ_REQUIRE(a && b && out, LQ_ERR_VALUE, "%s: NULL pointer", name);
    hipLaunchKernelGGL(binary_f32_kernel<OP>, dim3(grid_for(n, 1024)), dim3(256), 0, as_stream(stream), a, b, out, n);
    LQ_CHECK_LAUNCH("binary_f32");
    return LQ_OK;
}

template <typename From>
int astype_from(const void* src, void* dst, int dst_dtype, size_t n, hipStream_t st) {
    const From* s = static_cast<const From*>(src);
    const dim3 grid(grid_for(n, 256)), block(256);
    switch (dst_dtype) {
    case LQ_I8: hipLaunchKernelGGL((astype_kernel<From, int8_t>), grid, block, 0, st, s, static_cast<int8_t*>(dst), n); break;
    case LQ_I16: hipLaunchKernelGGL((astype_kernel<From, int16_t>), grid, block, 0, st, s, static_cast<int16_t*>(dst), n); break;
    case LQ_I32: hipLaunchKernelGGL((astype_kernel<From, int32_t>), grid, block, 0, st, s, static_cast<int32_t*>(dst), n); break;
    case LQ_F16: hipLaunchKernelGGL((astype_kernel<From, _Float16>), grid, block, 0, st, s, static_cast<_Float16*>(dst), n); break;
    case LQ_F32: hipLaunchKernelGGL((astype_kernel<From, float>), grid, block, 0, st, s, static_cast<float*>(dst), n); break;
    default: return fail(LQ_ERR_DTYPE, "astype: destination dtype %d is not one of int8 / int16 / int32 / float16 / float32", dst_dtype);
    }
    LQ_CHECK_LAUNCH("astype");
    return LQ_OK;
}

}  // namespace

extern "C" {

int lq_sub_f32(const float* a, const float* b, float* out, size_t n, lq_stream stream) {
    return launch_binary<OP_SUB>(a, b, out, n, stream, "sub_f32");
}
int lq_mul_f32(const float* a, const float* b, float* out, size_t n, lq_stream stream) {
    return launch_binary<OP_MUL>(a, b, out, n, stream, "mul_f32");
}
int lq_div_f32(const float* a, const float* b, float* out, size_t n, lq_stream stream) {
    return launch_binary<OP_DIV>(a, b, out, n, stream, "div_f32");
}
int lq_maximum_f32(const float* a, const float* b, float* out, size_t n, lq_stream stream) {
    return launch_binary<OP_MAXIMUM>(a, b, out, n, stream, "maximum_f32");
}
int lq_minimum_f32(const float* a, const float* b, float* out, size_t n, lq_stream stream) {
    return launch_binary<OP_MINIMUM>(a, b, out, n, stream, "minimum_f32");
}

int lq_round_f32(const float* x, float* out, size_t n, lq_stream stream) {
    if (n == 0) return LQ_OK;
    LQ_REQUIRE(x && out, LQ_ERR_VALUE, "round_f32: NULL pointer");
    hipLaunchKernelGGL(unary_f32_kernel<0>, dim3(grid_for(n, 256)), dim3(256), 0, as_stream(stream), x, out, n, 0.0f, 0.0f);
    LQ_CHECK_LAUNCH("round_f32");
    return LQ_OK;
}

int lq_clip_f32(const float* x, float* out, size_t n, double min_v, double max_v, lq_stream stream) {
    if (n == 0) return LQ_OK;
    LQ_REQUIRE(x && out, LQ_ERR_VALUE, "clip_f32: NULL pointer");
    hipLaunchKernelGGL(unary_f32_kernel<1>, dim3(grid_for(n, 256)), dim3(256), 0, as_stream(stream), x, out, n,
                       float(min_v), float(max_v));
    LQ_CHECK_LAUNCH("clip_f32");
    return LQ_OK;
}

int lq_astype(const void* src, int src_dtype, void* dst, int dst_dtype, size_t n, lq_stream stream) {
    if (n == 0) return LQ_OK;
    LQ_REQUIRE(src && dst, LQ_ERR_VALUE, "astype: NULL pointer");
    hipStream_t st = as_stream(stream);
    switch (src_dtype) {
    case LQ_I8: return astype_from<int8_t>(src, dst, dst_dtype, n, st);
    case LQ_I16: return astype_from<int16_t>(src, dst, dst_dtype, n, st);
    case LQ_I32: return astype_from<int32_t>(src, dst, dst_dtype, n, st);
    case LQ_F16: return astype_from<_Float16>(src, dst, dst_dtype, n, st);
    case LQ_F32: return astype_from<float>(src, dst, dst_dtype, n, st);
    default: return fail(LQ_ERR_DTYPE, "astype: source dtype %d is not one of int8 / int16 / int32 / float16 / float32", src_dtype);
    }
}

int lq_broadcast_f32(const float* src, float* out, size_t outer, size_t C, size_t inner, lq_stream stream) {
    const size_t total = outer * C * inner;
    if (total == 0) return LQ_OK;
    LQ_REQUIRE(src && out, LQ_ERR_VALUE, "broadcast_f32: NULL pointer");
    hipLaunchKernelGGL(broadcast_f32_kernel, dim3(grid_for(total, 256)), dim3(256), 0, as_stream(stream), src, out, total,
                       C, inner);
    LQ_CHECK_LAUNCH("broadcast_f32");
    return LQ_OK;
}

int lq_reduce_minmax(const float* x, const int64_t* shape, int ndim, const int* axes, int n_axes, float* mn, float* mx,
                     lq_stream stream) {
    LQ_REQUIRE(ndim >= 0 && ndim <= 16 && (ndim == 0 || shape), LQ_ERR_VALUE, "reduce_minmax: bad shape");
    LQ_REQUIRE(n_axes >= 0 && (n_axes == 0 || axes), LQ_ERR_VALUE, "reduce_minmax: bad axes");
    bool reduced[16] = {};
    for (int i = 0; i < n_axes; ++i) {
        const int ax = axes[i] < 0 ? axes[i] + ndim : axes[i];
        LQ_REQUIRE(ax >= 0 && ax < ndim, LQ_ERR_VALUE, "reduce_minmax: axis %d out of range for %d dimensions", axes[i], ndim);
        LQ_REQUIRE(!reduced[ax], LQ_ERR_VALUE, "reduce_minmax: axis %d given twice", axes[i]);
        reduced[ax] = true;
    }
    if (n_axes == 0)  // no axes = all of them (ReduceOpts with an empty list)
        for (int d = 0; d < ndim; ++d) reduced[d] = true;
    // merge neighbouring dimensions of the same kind (extent-1 dimensions join either side)
    size_t ext[17];
    bool kind[17];
    int groups = 0;
    for (int d = 0; d < ndim; ++d) {
        LQ_REQUIRE(shape[d] >= 0, LQ_ERR_SHAPE, "reduce_minmax: negative extent");
        if (shape[d] == 1) continue;
        if (groups > 0 && kind[groups - 1] == reduced[d]) {
            ext[groups - 1] *= size_t(shape[d]);
        } else {
            ext[groups] = size_t(shape[d]);
            kind[groups++] = reduced[d];
        }
    }
    size_t total = 1, n_red = 1;
    for (int gi = 0; gi < groups; ++gi) {
        total *= ext[gi];
        if (kind[gi]) n_red *= ext[gi];
    }
    LQ_REQUIRE(total > 0 && n_red > 0, LQ_ERR_SHAPE, "reduce_minmax: min / max of an empty range");
    LQ_REQUIRE(x && mn && mx, LQ_ERR_VALUE, "reduce_minmax: NULL pointer");
    // views [outer][C][inner] with C kept (lq_minmax) or [A][R][B] with R reduced
    if (groups == 0) return lq_minmax(x, 1, 1, 1, mn, mx, stream);
    if (groups == 1) return kind[0] ? lq_minmax(x, 1, 1, ext[0], mn, mx, stream) : lq_minmax(x, 1, ext[0], 1, mn, mx, stream);
    if (groups == 2 && kind[0]) return lq_minmax(x, ext[0], ext[1], 1, mn, mx, stream);
    if (groups == 2 && !kind[0] && ext[1] >= 4096) return lq_minmax(x, 1, ext[0], ext[1], mn, mx, stream);
    if (groups == 3 && kind[0]) return lq_minmax(x, ext[0], ext[1], ext[2], mn, mx, stream);
    size_t A, R, B;
    if (groups == 2) {
        A = ext[0]; R = ext[1]; B = 1;
    } else if (groups == 3) {
        A = ext[0]; R = ext[1]; B = ext[2];
    } else {
        return fail(LQ_ERR_NOT_IMPLEMENTED,
                    "reduce_minmax: the reduced axes must merge into one run, or into the two ends of the shape");
    }
    hipLaunchKernelGGL(reduce_mid_minmax_kernel, dim3(grid_for(A * B, 4)), dim3(256), 0, as_stream(stream), x, A, R, B, mn, mx);
    LQ_CHECK_LAUNCH("reduce_minmax");
    return LQ_OK;
}

int lq_batchnorm_eval_f32(const float* x, float* out, size_t B, int C, size_t spatial, const float* mean,
                          const float* var, const float* gamma, const float* beta, double eps, lq_stream stream) {
    const size_t total = B * size_t(C > 0 ? C : 0) * spatial;
    if (total == 0) return LQ_OK;
    LQ_REQUIRE(x && out && mean && var, LQ_ERR_VALUE, "batchnorm_eval_f32: NULL pointer");
    hipStream_t st = as_stream(stream);
    void* ws = nullptr;
    int rc = workspace(size_t(C) * 4, st, &ws);
    if (rc) return rc;
    float* rstd = static_cast<float*>(ws);
    hipLaunchKernelGGL(batchnorm_rstd_kernel, dim3((C + 255) / 256), dim3(256), 0, st, var, eps, C, rstd);
    LQ_CHECK_LAUNCH("batchnorm_rstd");
    if (spatial >= 256) {
        const size_t chunks = (spatial + 4095) / 4096;
        hipLaunchKernelGGL(batchnorm_eval_rows_kernel, dim3(grid_for(B * C * chunks, 1)), dim3(256), 0, st, x, out,
                           B * size_t(C), C, spatial, chunks, mean, rstd, gamma, beta);
    } else {
        hipLaunchKernelGGL(batchnorm_eval_flat_kernel, dim3(grid_for(total, 256)), dim3(256), 0, st, x, out, total, C,
                           spatial, mean, rstd, gamma, beta);
    }
    LQ_CHECK_LAUNCH("batchnorm_eval");
    return LQ_OK;
}

}  // extern "C"
