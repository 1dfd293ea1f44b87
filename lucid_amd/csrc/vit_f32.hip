// float32 companions of the int8 Linear path: what a ViT block does between its
// quantized Linears.  Lucid's dynamic-quantized ViT keeps LayerNorm, attention,
// GELU, the residual adds and the patch embedding in float32
// (lucid/models/vision/vit/_model.py:132-161,202-204,275-278,449-458); these kernels
// are those steps on gfx950, in float32 end to end:
//
//   lq_layernorm_f32        lucid/_C/backend/cpu/Norm.cpp:35-65
//   lq_gelu_f32             lucid/nn/functional/activations.py:219 (approximate="none", erf)
//   lq_add_f32              residual add
//   lq_attention_f32        scaled dot-product attention, CpuBackend.h:7603-7730,
//                           read straight from the packed qkv activation
//   lq_patchify_f32 + lq_sgemm_nt_f32   the stride = kernel patch convolution as a GEMM
//   lq_assemble_tokens_f32  class token + position table
//   lq_patch_embed_f32      the three above in one launch: the GEMM gathers the patches itself
//
// Matrix products use the float32 MFMA instructions; results agree with a CPU
// float32 evaluation to rounding-order differences (tested to 1e-4 relative).
#include "common.hpp"
#include "qepilogue.hpp"
#include "range_slots.hpp"

using namespace lq;

namespace {

typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}

// ---------------------------------------------------------------- LayerNorm
// One wavefront per row; the row (a few KiB) is re-read from cache for the
// variance and the output pass.  mean, centred values, var = dot(c,c)/N,
// rstd = 1/sqrt(var+eps), y = (c*rstd)*gamma + beta: the reference's steps.
constexpr int LN_ROWS_PER_WAVE = 1;
constexpr int LN_KEEP = 8;  // float4 per lane held in registers: rows of up to 2048 floats

__global__ __launch_bounds__(256) void layernorm_kernel(const float* __restrict__ x,
                                                        const float* __restrict__ gamma,
                                                        const float* __restrict__ beta,
                                                        float* __restrict__ out, long rows, int cols,
                                                        float eps, float* range) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const bool vec = (cols % 4 == 0) && aligned16(x) && aligned16(out) && aligned16(gamma) && aligned16(beta);
    const float inv_n = 1.0f / float(cols);
    float lo = __builtin_inff(), hi = -__builtin_inff();
    int nan = 0;
    auto track = [&](float y) {
        nan |= (y != y);
        lo = fminf(lo, y);
        hi = fmaxf(hi, y);
    };
    for (int rr = 0; rr < LN_ROWS_PER_WAVE; ++rr) {
        const long row = (long(blockIdx.x) * 4 + wave) * LN_ROWS_PER_WAVE + rr;
        if (row >= rows) break;
        const float* xr = x + row * cols;
        float* yr = out + row * cols;
        if (vec && cols <= LN_KEEP * 256) {
            // the row stays in registers (one trip to memory instead of three); the sums run
            // over the same values in the same order as below
            float4 v[LN_KEEP];
#pragma unroll
            for (int u = 0; u < LN_KEEP; ++u) {
                const int c = lane * 4 + u * 256;
                if (c < cols) v[u] = *reinterpret_cast<const float4*>(xr + c);
            }
            float s = 0.0f;
#pragma unroll
            for (int u = 0; u < LN_KEEP; ++u)
                if (lane * 4 + u * 256 < cols) s += (v[u].x + v[u].y) + (v[u].z + v[u].w);
            const float mean = wave_sum(s) * inv_n;
            float q = 0.0f;
#pragma unroll
            for (int u = 0; u < LN_KEEP; ++u)
                if (lane * 4 + u * 256 < cols) {
                    const float a = v[u].x - mean, b = v[u].y - mean, cc = v[u].z - mean, d = v[u].w - mean;
                    q += (a * a + b * b) + (cc * cc + d * d);
                }
            const float var = wave_sum(q) * inv_n;
            const float rstd = 1.0f / sqrtf(var + eps);
#pragma unroll
            for (int u = 0; u < LN_KEEP; ++u) {
                const int c = lane * 4 + u * 256;
                if (c < cols) {
                    const float4 g = *reinterpret_cast<const float4*>(gamma + c);
                    const float4 b = *reinterpret_cast<const float4*>(beta + c);
                    float4 y;
                    y.x = ((v[u].x - mean) * rstd) * g.x + b.x;
                    y.y = ((v[u].y - mean) * rstd) * g.y + b.y;
                    y.z = ((v[u].z - mean) * rstd) * g.z + b.z;
                    y.w = ((v[u].w - mean) * rstd) * g.w + b.w;
                    *reinterpret_cast<float4*>(yr + c) = y;
                    track(y.x), track(y.y), track(y.z), track(y.w);
                }
            }
            continue;
        }
        float s = 0.0f;
        if (vec) {
            for (int c = lane * 4; c < cols; c += 256) {
                const float4 v = *reinterpret_cast<const float4*>(xr + c);
                s += (v.x + v.y) + (v.z + v.w);
            }
        } else {
            for (int c = lane; c < cols; c += 64) s += xr[c];
        }
        const float mean = wave_sum(s) * inv_n;
        float q = 0.0f;
        if (vec) {
            for (int c = lane * 4; c < cols; c += 256) {
                const float4 v = *reinterpret_cast<const float4*>(xr + c);
                const float a = v.x - mean, b = v.y - mean, cc = v.z - mean, d = v.w - mean;
                q += (a * a + b * b) + (cc * cc + d * d);
            }
        } else {
            for (int c = lane; c < cols; c += 64) {
                const float a = xr[c] - mean;
                q += a * a;
            }
        }
        const float var = wave_sum(q) * inv_n;
        const float rstd = 1.0f / sqrtf(var + eps);
        if (vec) {
            for (int c = lane * 4; c < cols; c += 256) {
                const float4 v = *reinterpret_cast<const float4*>(xr + c);
                const float4 g = *reinterpret_cast<const float4*>(gamma + c);
                const float4 b = *reinterpret_cast<const float4*>(beta + c);
                float4 y;
                y.x = ((v.x - mean) * rstd) * g.x + b.x;
                y.y = ((v.y - mean) * rstd) * g.y + b.y;
                y.z = ((v.z - mean) * rstd) * g.z + b.z;
                y.w = ((v.w - mean) * rstd) * g.w + b.w;
                *reinterpret_cast<float4*>(yr + c) = y;
                track(y.x), track(y.y), track(y.z), track(y.w);
            }
        } else {
            for (int c = lane; c < cols; c += 64) {
                const float y = ((xr[c] - mean) * rstd) * gamma[c] + beta[c];
                yr[c] = y;
                track(y);
            }
        }
    }
    if (range) range_block_store(range, lo, hi, nan);
}

// LayerNorm feeding a dynamic quantizer without ever storing its float32 output: the first
// kernel takes each row's mean and 1/sqrt(var + eps) and the range of the normalized values, the
// second (after the qparams have been derived from that range) normalizes again - the same
// expressions on the same inputs, so the same bits - and writes int8 codes.  x is read twice
// and 1 byte per element written, where LayerNorm + quantize read it twice, write it once as
// float32 and read that back.  Rows of up to 2048 floats, vector-aligned.
template <int KEEP>  // float4 per lane held in registers: 4 for rows of up to 1024 floats, else KEEP
__global__ __launch_bounds__(256) void layernorm_stats_kernel(const float* __restrict__ x,
                                                              const float* __restrict__ gamma,
                                                              const float* __restrict__ beta, long rows, int cols,
                                                              float eps, float* __restrict__ stats, float* range) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const float inv_n = 1.0f / float(cols);
    float lo = __builtin_inff(), hi = -__builtin_inff();
    int nan = 0;
    auto track = [&](float y) {
        nan |= (y != y);
        lo = fminf(lo, y);
        hi = fmaxf(hi, y);
    };
    const long row = long(blockIdx.x) * 4 + wave;
    if (row < rows) {
        const float* xr = x + row * cols;
        float4 v[KEEP], gv[KEEP], bv[KEEP];
#pragma unroll
        for (int u = 0; u < KEEP; ++u) {
            const int c = lane * 4 + u * 256;
            if (c < cols) v[u] = *reinterpret_cast<const float4*>(xr + c);
        }
        // gamma and beta are needed after the two reductions: requested now, they arrive under them
#pragma unroll
        for (int u = 0; u < KEEP; ++u) {
            const int c = lane * 4 + u * 256;
            if (c < cols) {
                gv[u] = *reinterpret_cast<const float4*>(gamma + c);
                bv[u] = *reinterpret_cast<const float4*>(beta + c);
            }
        }
        float s = 0.0f;
#pragma unroll
        for (int u = 0; u < KEEP; ++u)
            if (lane * 4 + u * 256 < cols) s += (v[u].x + v[u].y) + (v[u].z + v[u].w);
        const float mean = wave_sum(s) * inv_n;
        float q = 0.0f;
#pragma unroll
        for (int u = 0; u < KEEP; ++u)
            if (lane * 4 + u * 256 < cols) {
                const float a = v[u].x - mean, b = v[u].y - mean, cc = v[u].z - mean, d = v[u].w - mean;
                q += (a * a + b * b) + (cc * cc + d * d);
            }
        const float var = wave_sum(q) * inv_n;
        const float rstd = 1.0f / sqrtf(var + eps);
        if (lane == 0) stats[2 * row] = mean, stats[2 * row + 1] = rstd;
#pragma unroll
        for (int u = 0; u < KEEP; ++u) {
            const int c = lane * 4 + u * 256;
            if (c < cols) {
                const float4 g = gv[u], b = bv[u];
                track(((v[u].x - mean) * rstd) * g.x + b.x);
                track(((v[u].y - mean) * rstd) * g.y + b.y);
                track(((v[u].z - mean) * rstd) * g.z + b.z);
                track(((v[u].w - mean) * rstd) * g.w + b.w);
            }
        }
    }
    range_block_store(range, lo, hi, nan);
}

__global__ __launch_bounds__(256) void layernorm_quantize_kernel(const float* __restrict__ x,
                                                                 const float* __restrict__ gamma,
                                                                 const float* __restrict__ beta,
                                                                 const float* __restrict__ stats, long rows, int cols,
                                                                 const float* __restrict__ scale,
                                                                 const float* __restrict__ zp, float qlo, float qhi,
                                                                 int off, int8_t* __restrict__ q) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const long row = long(blockIdx.x) * 4 + wave;
    if (row >= rows) return;
    const QGrid G = make_qgrid(scale[0], zp[0], qlo, qhi, true);
    const float mean = stats[2 * row], rstd = stats[2 * row + 1];
    const float* xr = x + row * cols;
    int8_t* qr = q + row * cols;
#pragma unroll
    for (int u = 0; u < LN_KEEP; ++u) {
        const int c = lane * 4 + u * 256;
        if (c < cols) {
            const float4 v = *reinterpret_cast<const float4*>(xr + c);
            const float4 g = *reinterpret_cast<const float4*>(gamma + c);
            const float4 b = *reinterpret_cast<const float4*>(beta + c);
            const int c0 = int(quant_fast<false>(((v.x - mean) * rstd) * g.x + b.x, G)) + off;
            const int c1 = int(quant_fast<false>(((v.y - mean) * rstd) * g.y + b.y, G)) + off;
            const int c2 = int(quant_fast<false>(((v.z - mean) * rstd) * g.z + b.z, G)) + off;
            const int c3 = int(quant_fast<false>(((v.w - mean) * rstd) * g.w + b.w, G)) + off;
            *reinterpret_cast<uint32_t*>(qr + c) = uint32_t(c0 & 0xff) | (uint32_t(c1 & 0xff) << 8) |
                                                   (uint32_t(c2 & 0xff) << 16) | (uint32_t(c3) << 24);
        }
    }
}

// ---------------------------------------------------------------- elementwise
__device__ __forceinline__ float gelu_erf(float x) {
    return (0.5f * x) * (1.0f + lq::erf_as(x * 0.70710678118654752440f));
}

// Four float4 per thread (block-strided, so each access of a wavefront is
// contiguous); the optional range costs one partial slot per block.
constexpr int GELU_PER_THREAD = 4;

__global__ __launch_bounds__(256) void gelu_kernel(const float* __restrict__ x, float* __restrict__ out,
                                                   size_t n, int vec, float* range) {
    float lo = __builtin_inff(), hi = -__builtin_inff();
    int nan = 0;
    auto track = [&](float y) {
        nan |= (y != y);
        lo = fminf(lo, y);
        hi = fmaxf(hi, y);
    };
    const size_t base = size_t(blockIdx.x) * (256 * GELU_PER_THREAD) + threadIdx.x;
    if (vec) {
        float4 v[GELU_PER_THREAD];
#pragma unroll
        for (int u = 0; u < GELU_PER_THREAD; ++u) {
            const size_t i = base + size_t(u) * 256;
            if (i * 4 < n) v[u] = reinterpret_cast<const float4*>(x)[i];
        }
#pragma unroll
        for (int u = 0; u < GELU_PER_THREAD; ++u) {
            const size_t i = base + size_t(u) * 256;
            if (i * 4 < n) {
                float4 y = {gelu_erf(v[u].x), gelu_erf(v[u].y), gelu_erf(v[u].z), gelu_erf(v[u].w)};
                reinterpret_cast<float4*>(out)[i] = y;
                track(y.x), track(y.y), track(y.z), track(y.w);
            }
        }
    } else {
#pragma unroll
        for (int u = 0; u < GELU_PER_THREAD; ++u) {
            const size_t i = base + size_t(u) * 256;
            if (i < n) {
                const float y = gelu_erf(x[i]);
                out[i] = y;
                track(y);
            }
        }
    }
    if (range) range_block_store(range, lo, hi, nan);
}

// dst[r, :] = src[r * src_row_stride : r * src_row_stride + cols]
__global__ __launch_bounds__(256) void gather_rows_kernel(const float* __restrict__ src, size_t src_row_stride,
                                                          float* __restrict__ dst, size_t rows, size_t cols) {
    const size_t i = size_t(blockIdx.x) * 256 + threadIdx.x;
    if (i >= rows * cols) return;
    const size_t r = i / cols, c = i - r * cols;
    dst[i] = src[r * src_row_stride + c];
}

__global__ __launch_bounds__(256) void add_kernel(const float* __restrict__ a, const float* __restrict__ b,
                                                  float* __restrict__ out, size_t n, int vec) {
    const size_t i = size_t(blockIdx.x) * 256 + threadIdx.x;
    if (vec) {
        if (i * 4 >= n) return;
        const float4 u = reinterpret_cast<const float4*>(a)[i];
        const float4 v = reinterpret_cast<const float4*>(b)[i];
        float4 y = {u.x + v.x, u.y + v.y, u.z + v.z, u.w + v.w};
        reinterpret_cast<float4*>(out)[i] = y;
    } else if (i < n) {
        out[i] = a[i] + b[i];
    }
}

// image [B,C,H,W] -> patch rows [B*(H/p)*(W/p), C*p*p], column order (c, ph, pw):
// the im2col of a convolution whose stride equals its kernel
__global__ __launch_bounds__(256) void patchify_kernel(const float* __restrict__ img, float* __restrict__ out,
                                                       int B, int C, int H, int W, int p) {
    const int gh = H / p, gw = W / p, K = C * p * p;
    const size_t total = size_t(B) * gh * gw * K;
    const size_t i = size_t(blockIdx.x) * 256 + threadIdx.x;
    if (i >= total) return;
    const int k = int(i % K);
    const size_t row = i / K;
    const int pw = k % p, ph = (k / p) % p, c = k / (p * p);
    const int gx = int(row % gw), gy = int((row / gw) % gh), b = int(row / (size_t(gw) * gh));
    out[i] = img[((size_t(b) * C + c) * H + (gy * p + ph)) * W + (gx * p + pw)];
}

// tokens[b,0,:] = cls + pos[0]; tokens[b,1+i,:] = patches[b,i,:] + pos[1+i]
__global__ __launch_bounds__(256) void assemble_tokens_kernel(const float* __restrict__ patches,
                                                              const float* __restrict__ cls,
                                                              const float* __restrict__ pos,
                                                              float* __restrict__ out, int B, int T, int D) {
    const size_t total = size_t(B) * T * D;
    const size_t i = size_t(blockIdx.x) * 256 + threadIdx.x;
    if (i >= total) return;
    const int d = int(i % D);
    const int t = int((i / D) % T);
    const size_t b = i / (size_t(D) * T);
    const float v = t == 0 ? cls[d] : patches[(b * (T - 1) + (t - 1)) * D + d];
    out[i] = v + pos[size_t(t) * D + d];
}

// (e0, e1) = h + m + l part by part, each part a pair of bfloat16 (e0's in the low half): the
// packed conversion rounds to nearest, the remainders are exact (8 + 8 + 8 significant bits with
// signed remainders).  A NaN stays a NaN in every part; an infinity turns into a NaN in the
// lower parts, so a non-finite input gives a non-finite output.
typedef __bf16 at_bf2 __attribute__((ext_vector_type(2)));
typedef float at_f2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t at_pk(float a, float b) {
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(at_f2{a, b}, at_bf2));
}
__device__ __forceinline__ void at_split3x2(float e0, float e1, uint32_t& h, uint32_t& m, uint32_t& l) {
    h = at_pk(e0, e1);
    e0 -= __uint_as_float(h << 16), e1 -= __uint_as_float(h & 0xffff0000u);
    m = at_pk(e0, e1);
    e0 -= __uint_as_float(m << 16), e1 -= __uint_as_float(m & 0xffff0000u);
    l = at_pk(e0, e1);
}

typedef __bf16 sg_v8bf __attribute__((ext_vector_type(8)));

// ---------------------------------------------------------------- float32 GEMM, out = a . w^T + bias
// float32 operands on the bfloat16 matrix instruction: both operands are split into three
// bfloat16 parts when a tile is written to LDS (at_split3x2), and six part products per k step
// (hi.hi, hi.mid, mid.hi, hi.lo, lo.hi, mid.mid, smallest first, accumulated in float32) give
// every product 2^-24 relative accuracy - a float32 GEMM at six instructions of
// v_mfma_f32_32x32x16_bf16 per 16 k, against eight of v_mfma_f32_32x32x2_f32 at four times the
// cycles each.
//
// 128 x 128 x 32 block tile, 4 wavefronts of 64 x 64; the next tile's operands wait in registers
// while the current one is multiplied.  LDS: per part 256 rows (A's 128, then W's) of 32
// bfloat16 = 64 bytes; the 16-byte chunk k of row r sits at chunk k ^ ((r / 4) % 4), which puts
// the 16 rows of a fragment pass on 16 different bank groups.
constexpr int SG_BM = 128, SG_BN = 128, SG_BK = 32, SG_ROWS = SG_BM + SG_BN;

__device__ __forceinline__ int sg_index(int row, int k) {  // k a multiple of 4
    return row * SG_BK + ((((k >> 3) ^ ((row >> 2) & 3)) << 3) | (k & 7));
}

// PATCH: the A operand is an image [B,C,H,W] read as the rows of its p x p patches (row = (b, gy,
// gx), column = (c, ph, pw): four consecutive columns are four consecutive pixels of one image
// row when p is a multiple of 4), and the result row (b, i) lands on token row 1 + i of image b
// with the position table added; the blocks of the first row tile also write the class-token rows.
struct PatchForm {
    int C, H, W, p, gw, per_image;  // per_image = (H/p) * (W/p) patches
    int B, log2p;                   // log2p = -1 when p is not a power of two
    const float* cls;  // [N]
    const float* pos;  // [(1 + per_image), N]
};

// PATCH 0: a is a plain [M,K] matrix.  1: patch rows with p a power of two and every group of
// four columns one aligned 16-byte load (no branch and no division in the loop).  2: patch rows
// of any geometry, element by element.
template <int PATCH>
__global__ __launch_bounds__(256, 2) void sgemm_nt_kernel(const float* __restrict__ a, const float* __restrict__ w,
                                                          const float* __restrict__ bias, float* __restrict__ out,
                                                          int M, int N, int K, PatchForm pf) {
    __shared__ __attribute__((aligned(16))) uint16_t sp[3][SG_ROWS * SG_BK];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int m0 = blockIdx.y * SG_BM, n0 = blockIdx.x * SG_BN;
    // loader: piece tid + 256 u = row (tid + 256 u) / 8 of either operand, four consecutive k at 4 * (tid % 8)
    const int lrow = tid >> 3, lk = (tid & 7) * 4;
    const bool vec = (K % 4 == 0) && aligned16(w) && (PATCH != 0 || aligned16(a));
    size_t patch_at[4];  // PATCH: where the patch of loader row u starts in the image
    if constexpr (PATCH != 0) {
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int row = min(m0 + lrow + 32 * u, M - 1);
            const int b = row / pf.per_image, i = row - b * pf.per_image;
            const int gy = i / pf.gw, gx = i - gy * pf.gw;
            patch_at[u] = (size_t(b) * pf.C * pf.H + size_t(gy) * pf.p) * pf.W + size_t(gx) * pf.p;
        }
    }
    v16f acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    float4 ra[4], rb[4];
    auto fetch_row = [&](const float* base, int row, int rows, int k) {
        float4 v = {0.f, 0.f, 0.f, 0.f};
        if (row < rows) {
            const float* p = base + size_t(row) * K + k;
            if (vec && k + 3 < K) {
                v = *reinterpret_cast<const float4*>(p);
            } else {
                if (k < K) v.x = p[0];
                if (k + 1 < K) v.y = p[1];
                if (k + 2 < K) v.z = p[2];
                if (k + 3 < K) v.w = p[3];
            }
        }
        return v;
    };
    // PATCH: column k of a patch row is pixel (c, ph, pw) of the patch.  Loads go to clamped
    // (always valid) addresses and what lies past M or K is zeroed afterwards, so that the four
    // loads of a fetch are issued back to back.
    auto fetch_patches = [&](int k) {
        if constexpr (PATCH == 1) {
            const int kk = min(k, K - 4);
            const int pw = kk & (pf.p - 1), ph = (kk >> pf.log2p) & (pf.p - 1), c = kk >> (2 * pf.log2p);
            const size_t pixel = (size_t(c) * pf.H + ph) * pf.W + pw;
#pragma unroll
            for (int u = 0; u < 4; ++u) ra[u] = *reinterpret_cast<const float4*>(a + patch_at[u] + pixel);
            if (k >= K) {
#pragma unroll
                for (int u = 0; u < 4; ++u) ra[u] = float4{0.f, 0.f, 0.f, 0.f};
            }
        } else {
            const int pp = pf.p * pf.p;
            size_t pixel[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int kk = min(k + e, K - 1);
                const int c = kk / pp, r = kk - c * pp;
                const int ph = r / pf.p, pw = r - ph * pf.p;
                pixel[e] = (size_t(c) * pf.H + ph) * pf.W + pw;
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const float* p = a + patch_at[u];
                ra[u] = float4{p[pixel[0]], p[pixel[1]], p[pixel[2]], p[pixel[3]]};
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                if (k >= K) ra[u].x = 0.f;
                if (k + 1 >= K) ra[u].y = 0.f;
                if (k + 2 >= K) ra[u].z = 0.f;
                if (k + 3 >= K) ra[u].w = 0.f;
            }
        }
#pragma unroll
        for (int u = 0; u < 4; ++u)
            if (m0 + lrow + 32 * u >= M) ra[u] = float4{0.f, 0.f, 0.f, 0.f};
    };
    // plain rows in the aligned case: the row is clamped instead of tested (a row past the end
    // only feeds results that are never stored) and a k past the end is zeroed afterwards
    auto fetch_rows_vec = [&](const float* base, int row0, int rows, int k, float4 (&r)[4]) {
        const int kk = min(k, K - 4);
#pragma unroll
        for (int u = 0; u < 4; ++u)
            r[u] = *reinterpret_cast<const float4*>(base + size_t(min(row0 + 32 * u, rows - 1)) * K + kk);
        if (k >= K) {
#pragma unroll
            for (int u = 0; u < 4; ++u) r[u] = float4{0.f, 0.f, 0.f, 0.f};
        }
    };
    auto fetch = [&](int k0) {
        if constexpr (PATCH != 0) fetch_patches(k0 + lk);
        if (vec) {
            if constexpr (PATCH == 0) fetch_rows_vec(a, m0 + lrow, M, k0 + lk, ra);
            fetch_rows_vec(w, n0 + lrow, N, k0 + lk, rb);
        } else {
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                if constexpr (PATCH == 0) ra[u] = fetch_row(a, m0 + lrow + 32 * u, M, k0 + lk);
                rb[u] = fetch_row(w, n0 + lrow + 32 * u, N, k0 + lk);
            }
        }
    };
    auto stash_one = [&](int row, float4 v) {
        uint32_t lo[3], hi[3];
        at_split3x2(v.x, v.y, lo[0], lo[1], lo[2]);
        at_split3x2(v.z, v.w, hi[0], hi[1], hi[2]);
        const int at = sg_index(row, lk);
#pragma unroll
        for (int p = 0; p < 3; ++p) *reinterpret_cast<uint2*>(&sp[p][at]) = uint2{lo[p], hi[p]};
    };
    auto stash = [&] {
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            stash_one(lrow + 32 * u, ra[u]);
            stash_one(SG_BM + lrow + 32 * u, rb[u]);
        }
    };
    const int nk = (K + SG_BK - 1) / SG_BK;
    const int fr = lane & 31, kg = lane >> 5;
    fetch(0);
    for (int t = 0; t < nk; ++t) {
        stash();
        __syncthreads();
        if (t + 1 < nk) fetch((t + 1) * SG_BK);
#pragma unroll
        for (int ks = 0; ks < SG_BK / 16; ++ks) {
            uint4 fa[2][3], fb[2][3];
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                const int at = sg_index(wm * 64 + i * 32 + fr, 16 * ks + 8 * kg);
#pragma unroll
                for (int p = 0; p < 3; ++p) fa[i][p] = *reinterpret_cast<const uint4*>(&sp[p][at]);
            }
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const int at = sg_index(SG_BM + wn * 64 + j * 32 + fr, 16 * ks + 8 * kg);
#pragma unroll
                for (int p = 0; p < 3; ++p) fb[j][p] = *reinterpret_cast<const uint4*>(&sp[p][at]);
            }
            auto mm = [&](int pa, int pb) {
#pragma unroll
                for (int i = 0; i < 2; ++i)
#pragma unroll
                    for (int j = 0; j < 2; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(sg_v8bf, fa[i][pa]),
                                                                            __builtin_bit_cast(sg_v8bf, fb[j][pb]),
                                                                            acc[i][j], 0, 0, 0);
            };
            mm(1, 1), mm(0, 2), mm(2, 0), mm(0, 1), mm(1, 0), mm(0, 0);
        }
        __syncthreads();  // the tile has been read: the next one may be written
    }
    // result layout of the 32x32 MFMA: column = lane % 32, row = 8*(r/4) + 4*(lane/32) + r%4
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int n = n0 + wn * 64 + j * 32 + (lane & 31);
            if (n >= N) continue;
            const float bv = bias ? bias[n] : 0.0f;
            if constexpr (PATCH != 0) {
                // the sixteen position values are requested before the first store: a store
                // between two loads would make each load wait for the one before it
                float pv[16];
                size_t at[16];
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int mq = m0 + wm * 64 + i * 32 + 8 * q + 4 * (lane >> 5);
                    int b = mq / pf.per_image, t = mq - b * pf.per_image;
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        at[4 * q + r] = (size_t(b) * (pf.per_image + 1) + 1 + t) * N + n;
                        pv[4 * q + r] = mq + r < M ? pf.pos[size_t(1 + t) * N + n] : 0.0f;
                        if (++t == pf.per_image) t = 0, ++b;
                    }
                }
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int m = m0 + wm * 64 + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                    if (m < M) out[at[r]] = (acc[i][j][r] + bv) + pv[r];
                }
            } else {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int m = m0 + wm * 64 + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                    if (m < M) out[size_t(m) * N + n] = acc[i][j][r] + bv;
                }
            }
        }
    if constexpr (PATCH != 0) {
        // class-token rows: token 0 of every image, this block's 128 columns
        if (blockIdx.y == 0) {
            const int n = n0 + (tid & 127);
            if (n < N) {
                const float v = pf.cls[n] + pf.pos[n];
                for (int b = tid >> 7; b < pf.B; b += 2) out[size_t(b) * (pf.per_image + 1) * N + n] = v;
            }
        }
    }
}

// ---------------------------------------------------------------- attention
// One block per (batch, head); one wavefront per 16 queries; head dim 64, at
// most 208 tokens.  qkv is the packed activation [B, T, 3, H, 64] of the qkv
// Linear; out is [B, T, H*64].
//
// float32 operands on the bfloat16 matrix instruction.  A float32 is the exact sum of three
// bfloat16 values (8 + 8 + 8 significant bits: at_split3x2), and a product a * b keeps 2^-24
// relative accuracy with six of the nine part products (hi.hi, hi.mid, mid.hi, hi.lo, lo.hi,
// mid.mid; the three left out are below 2^-24 of |a b|).  Part products are exact in float32
// and accumulate in float32, so each dot product is as accurate as a float32 one, and
// v_mfma_f32_16x16x32_bf16 runs sixteen times the rate of v_mfma_f32_16x16x4_f32: six
// instructions of the one replace eight of the other at a sixth of the time each.
//
// The three parts of K (row-major) and of V^T ([column][key]) are both in LDS from the start -
// 79 872 + 81 408 bytes of the CU's 160 KiB - so after the one barrier that follows the splits
// a wavefront runs scores, softmax and P . V on its own, and the 13 wavefronts (four on one
// SIMD, three on the others) drift apart instead of waiting for each other between phases.
//
// Per wavefront: S^T = K . Q^T as 13 tiles of 16 keys x 16 queries (accumulators stay in
// registers), softmax over the keys of each query (a lane holds 52 of a query's keys, the other
// three lane groups the rest), then O = P . V where the S^T accumulators ARE the A operand:
// register r of tile t holds P[query = lane%16][key = 16t + 4*(lane/16) + r], so two tiles give
// a lane the eight k slots of an instruction, which is a valid k-slice assignment as long as V
// is read with the same one ([column][key] keeps a lane's four keys of a tile in 8 contiguous
// bytes); the thirteenth tile goes through the 16-key form of the instruction alone.
constexpr int AT_D = 64, AT_TMAX = 208;
// K: rows of 64 bfloat16 = 128 bytes = all 32 banks; the 16-byte chunk k of row r sits at chunk
// k ^ (r % 8), so the 16 rows of a fragment (same logical chunk) cover every bank exactly twice
constexpr int AT_PART_K = AT_TMAX * AT_D;
// V^T: 106 dwords per row = 10 mod 32: the 16 rows a fragment reads (8 bytes each) fall on 16
// different bank pairs
constexpr int AT_VLD = AT_TMAX + 4;
constexpr int AT_PART_V = AT_D * AT_VLD;  // elements of one part
constexpr size_t AT_K_BYTES = size_t(3) * AT_PART_K * 2;
constexpr size_t AT_SMEM = AT_K_BYTES + size_t(3) * AT_PART_V * 2;
static_assert(AT_SMEM + 1024 <= 160 * 1024, "LDS of a CU, with the range reduction's few words");

typedef __bf16 at_v8bf __attribute__((ext_vector_type(8)));
typedef short at_v4s __attribute__((ext_vector_type(4)));

__device__ __forceinline__ int at_k_index(int row, int col) {  // col a multiple of 4
    return row * AT_D + ((((col >> 3) ^ (row & 7)) << 3) | (col & 7));
}

// acc += a * b from the parts, smallest terms first
__device__ __forceinline__ v4f at_mma6(const uint4 (&a)[3], const uint4 (&b)[3], v4f acc) {
    auto mm = [&](const uint4& x, const uint4& y) {
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(at_v8bf, x), __builtin_bit_cast(at_v8bf, y), acc,
                                                      0, 0, 0);
    };
    mm(a[1], b[1]);
    mm(a[0], b[2]);
    mm(a[2], b[0]);
    mm(a[0], b[1]);
    mm(a[1], b[0]);
    mm(a[0], b[0]);
    return acc;
}
// the same over 16 k slots (four per lane)
__device__ __forceinline__ v4f at_mma6_k16(const uint2 (&a)[3], const uint2 (&b)[3], v4f acc) {
    auto mm = [&](const uint2& x, const uint2& y) {
        acc = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(at_v4s, x), __builtin_bit_cast(at_v4s, y), acc,
                                                        0, 0, 0);
    };
    mm(a[1], b[1]);
    mm(a[0], b[2]);
    mm(a[2], b[0]);
    mm(a[0], b[1]);
    mm(a[1], b[0]);
    mm(a[0], b[0]);
    return acc;
}

__global__ __launch_bounds__(1024) void attention_kernel(const float* __restrict__ qkv, float* __restrict__ out,
                                                        int B, int T, int H, float scale, float* range) {
    extern __shared__ __attribute__((aligned(16))) uint16_t at_smem[];
    uint16_t* const k_lds = at_smem;
    uint16_t* const v_lds = at_smem + 3 * AT_PART_K;
    const int b = blockIdx.x / H, h = blockIdx.x % H;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const size_t tok_stride = size_t(3) * H * AT_D;
    const float* base = qkv + size_t(b) * T * tok_stride + size_t(h) * AT_D;
    // K and V are requested before anything is used (a block of 13 wavefronts holds all of both: four
    // 16-byte pieces of each per thread).  A thread's V pieces are two pairs of consecutive keys at the
    // same four columns: V^T keeps a column's keys contiguous, so a pair of keys is one dword of each part
    constexpr int kPieces = AT_TMAX * (AT_D / 4), kHeld = 4;
    constexpr int kPairs = (AT_TMAX / 2) * (AT_D / 4);
    float4 kheld[kHeld], vheld[kHeld];
#pragma unroll
    for (int u = 0; u < kHeld; ++u) {
        const int i = tid + u * int(blockDim.x), row = i / (AT_D / 4), c4 = (i % (AT_D / 4)) * 4;
        kheld[u] = float4{0.f, 0.f, 0.f, 0.f};
        if (i < kPieces && row < T) kheld[u] = *reinterpret_cast<const float4*>(base + size_t(row) * tok_stride + size_t(H) * AT_D + c4);
    }
#pragma unroll
    for (int u = 0; u < kHeld; ++u) {
        const int i = tid + (u >> 1) * int(blockDim.x), row = 2 * (i / (AT_D / 4)) + (u & 1), c4 = (i % (AT_D / 4)) * 4;
        vheld[u] = float4{0.f, 0.f, 0.f, 0.f};
        if (i < kPairs && row < T) vheld[u] = *reinterpret_cast<const float4*>(base + size_t(row) * tok_stride + size_t(2) * H * AT_D + c4);
    }
    // One wavefront per tile of 16 queries.  With 4 n + 1 tiles one SIMD would hold a wavefront more
    // than the others and everybody would wait for it: the launch then has three more wavefronts,
    // and the last tile's four each compute its scores but only one 16-column tile of its output.
    const int tiles = (T + 15) / 16;
    const bool shared_last = int(blockDim.x) > tiles * 64;
    const int q0 = (wave < tiles ? wave : tiles - 1) * 16;
    const int only_j = (shared_last && wave >= tiles - 1) ? wave - (tiles - 1) : -1;  // wavefront-uniform
    const int g = lane >> 4, c = lane & 15;
    // the lane's slice of its query row: Q[q0 + c][32 u + 8 g + 0..7]
    float4 qheld[2 * (AT_D / 32)];
    {
        const int q = q0 + c;
        const float* qp = base + size_t(q < T ? q : T - 1) * tok_stride;
#pragma unroll
        for (int u = 0; u < AT_D / 32; ++u) {
            qheld[2 * u] = *reinterpret_cast<const float4*>(qp + 32 * u + 8 * g);
            qheld[2 * u + 1] = *reinterpret_cast<const float4*>(qp + 32 * u + 8 * g + 4);
        }
    }
    // K rows into LDS as three bfloat16 parts (rows past T are zero)
    auto place_k = [&](int i, float4 kv) {
        const int row = i / (AT_D / 4), c4 = (i % (AT_D / 4)) * 4;
        uint32_t lo[3], hi[3];
        at_split3x2(kv.x, kv.y, lo[0], lo[1], lo[2]);
        at_split3x2(kv.z, kv.w, hi[0], hi[1], hi[2]);
        const int at = at_k_index(row, c4);
#pragma unroll
        for (int p = 0; p < 3; ++p) *reinterpret_cast<uint2*>(k_lds + p * AT_PART_K + at) = uint2{lo[p], hi[p]};
    };
#pragma unroll
    for (int u = 0; u < kHeld; ++u) {
        const int i = tid + u * int(blockDim.x);
        if (i < kPieces) place_k(i, kheld[u]);
    }
    for (int i = tid + kHeld * int(blockDim.x); i < kPieces; i += blockDim.x) {  // fewer than 13 wavefronts
        const int row = i / (AT_D / 4), c4 = (i % (AT_D / 4)) * 4;
        float4 kv = {0.f, 0.f, 0.f, 0.f};
        if (row < T) kv = *reinterpret_cast<const float4*>(base + size_t(row) * tok_stride + size_t(H) * AT_D + c4);
        place_k(i, kv);
    }
    // V^T's parts: keys 2 pair and 2 pair + 1 at columns c4 .. c4 + 3 (keys past T are zero)
    auto place_v = [&](int i, float4 v0, float4 v1) {
        const int pair = i / (AT_D / 4), c4 = (i % (AT_D / 4)) * 4;
        const float a[4] = {v0.x, v0.y, v0.z, v0.w}, bb[4] = {v1.x, v1.y, v1.z, v1.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            uint32_t d[3];
            at_split3x2(a[e], bb[e], d[0], d[1], d[2]);
#pragma unroll
            for (int p = 0; p < 3; ++p)
                *reinterpret_cast<uint32_t*>(v_lds + p * AT_PART_V + (c4 + e) * AT_VLD + 2 * pair) = d[p];
        }
    };
#pragma unroll
    for (int u = 0; u < kHeld / 2; ++u) {
        const int i = tid + u * int(blockDim.x);
        if (i < kPairs) place_v(i, vheld[2 * u], vheld[2 * u + 1]);
    }
    for (int i = tid + (kHeld / 2) * int(blockDim.x); i < kPairs; i += blockDim.x) {  // fewer than 13 wavefronts
        const int pair = i / (AT_D / 4), c4 = (i % (AT_D / 4)) * 4;
        float4 v0 = {0.f, 0.f, 0.f, 0.f}, v1 = {0.f, 0.f, 0.f, 0.f};
        const float* vp = base + size_t(2) * H * AT_D + c4;
        if (2 * pair < T) v0 = *reinterpret_cast<const float4*>(vp + size_t(2 * pair) * tok_stride);
        if (2 * pair + 1 < T) v1 = *reinterpret_cast<const float4*>(vp + size_t(2 * pair + 1) * tok_stride);
        place_v(i, v0, v1);
    }
    // B operand of S^T, pre-scaled so that S = scale * log2(e) * Q.K^T (the scores are kept in the
    // base-2 domain, so that the softmax numerators are one v_exp_f32 each)
    uint4 qf[AT_D / 32][3];
    {
        const float qs = scale * 1.4426950408889634f;
#pragma unroll
        for (int u = 0; u < AT_D / 32; ++u) {
            const float4 a = qheld[2 * u], bq = qheld[2 * u + 1];
            const float v[8] = {a.x * qs, a.y * qs, a.z * qs, a.w * qs, bq.x * qs, bq.y * qs, bq.z * qs, bq.w * qs};
            uint32_t d[3][4];
#pragma unroll
            for (int e = 0; e < 4; ++e) at_split3x2(v[2 * e], v[2 * e + 1], d[0][e], d[1][e], d[2][e]);
#pragma unroll
            for (int p = 0; p < 3; ++p) qf[u][p] = uint4{d[p][0], d[p][1], d[p][2], d[p][3]};
        }
    }
    __syncthreads();  // the only one before the range reduction: from here on a wavefront is on its own
    constexpr int NT = AT_TMAX / 16;
    v4f st[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) st[t] = v4f{0.f, 0.f, 0.f, 0.f};
    // k slice outermost: the 13 tiles' accumulators are independent chains
#pragma unroll
    for (int u = 0; u < AT_D / 32; ++u)
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            uint4 kf[3];
            const int at = at_k_index(16 * t + c, 32 * u + 8 * g);
#pragma unroll
            for (int p = 0; p < 3; ++p) kf[p] = *reinterpret_cast<const uint4*>(k_lds + p * AT_PART_K + at);
            st[t] = at_mma6(kf, qf[u], st[t]);
        }
    // st[t][r] = S[query q0 + c][key 16t + 4g + r]
    float mx = -__builtin_inff();
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int key = 16 * t + 4 * g + r;
            if (key >= T) st[t][r] = -__builtin_inff();
            mx = fmaxf(mx, st[t][r]);
        }
    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    float sum = 0.0f;
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const float e = __builtin_amdgcn_exp2f(st[t][r] - mx);  // 2^(-inf) = 0 for the padded keys
            st[t][r] = e;
            sum += e;
        }
    sum += __shfl_xor(sum, 16, 64);
    sum += __shfl_xor(sum, 32, 64);
    const float inv = sum > 0.0f ? 1.0f / sum : 0.0f;

    // O[q][n] = sum_key P[q][key] V[key][n], four 16-wide column tiles; tile j of the output holds
    // head-dim columns 16 j + c: the 16 lanes of a fragment read consecutive V^T rows (rows 4 c + j,
    // which would let a lane store four consecutive floats, fall on four bank pairs only)
    static_assert(NT % 2 == 1, "tile pairs and one single tile");
    v4f o[AT_D / 16];
#pragma unroll
    for (int j = 0; j < AT_D / 16; ++j) o[j] = v4f{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int tp = 0; tp < NT / 2; ++tp) {
        // the eight k slots of this lane: keys 32 tp + 4 g + 0..3 and 32 tp + 16 + 4 g + 0..3
        float pv[8];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            pv[r] = st[2 * tp][r] * inv;
            pv[4 + r] = st[2 * tp + 1][r] * inv;
        }
        uint32_t d[3][4];
#pragma unroll
        for (int e = 0; e < 4; ++e) at_split3x2(pv[2 * e], pv[2 * e + 1], d[0][e], d[1][e], d[2][e]);
        uint4 pf[3];
#pragma unroll
        for (int p = 0; p < 3; ++p) pf[p] = uint4{d[p][0], d[p][1], d[p][2], d[p][3]};
#pragma unroll
        for (int j = 0; j < AT_D / 16; ++j) {
            if (only_j >= 0 && only_j != j) continue;
            uint4 vf[3];
#pragma unroll
            for (int p = 0; p < 3; ++p) {
                const uint16_t* vrow = v_lds + p * AT_PART_V + (16 * j + c) * AT_VLD + 32 * tp + 4 * g;
                const uint2 lo = *reinterpret_cast<const uint2*>(vrow), hi = *reinterpret_cast<const uint2*>(vrow + 16);
                vf[p] = uint4{lo.x, lo.y, hi.x, hi.y};
            }
            o[j] = at_mma6(pf, vf, o[j]);
        }
    }
    {
        // the last tile: keys 16 (NT - 1) + 4 g + 0..3, four k slots per lane
        float pv[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) pv[r] = st[NT - 1][r] * inv;
        uint32_t d[3][2];
#pragma unroll
        for (int e = 0; e < 2; ++e) at_split3x2(pv[2 * e], pv[2 * e + 1], d[0][e], d[1][e], d[2][e]);
        uint2 pf[3];
#pragma unroll
        for (int p = 0; p < 3; ++p) pf[p] = uint2{d[p][0], d[p][1]};
#pragma unroll
        for (int j = 0; j < AT_D / 16; ++j) {
            if (only_j >= 0 && only_j != j) continue;
            uint2 vf[3];
#pragma unroll
            for (int p = 0; p < 3; ++p)
                vf[p] = *reinterpret_cast<const uint2*>(v_lds + p * AT_PART_V + (16 * j + c) * AT_VLD + 16 * (NT - 1) + 4 * g);
            o[j] = at_mma6_k16(pf, vf, o[j]);
        }
    }
    // result layout of the 16x16 MFMA: column slot = lane % 16, row = 4*(lane/16) + r; the 16 lanes
    // of a row store 64 consecutive bytes
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int q = q0 + 4 * g + r;
        if (q < T) {
            float* orow = out + (size_t(b) * T + q) * (size_t(H) * AT_D) + size_t(h) * AT_D + c;
#pragma unroll
            for (int j = 0; j < AT_D / 16; ++j)
                if (only_j < 0 || only_j == j) orow[16 * j] = o[j][r];
        }
    }
    if (range) {
        float lo = __builtin_inff(), hi = -__builtin_inff();
        int nan = 0;
#pragma unroll
        for (int j = 0; j < AT_D / 16; ++j)
#pragma unroll
            for (int r = 0; r < 4; ++r)
                if (q0 + 4 * g + r < T && (only_j < 0 || only_j == j)) {
                    nan |= (o[j][r] != o[j][r]);
                    lo = fminf(lo, o[j][r]);
                    hi = fmaxf(hi, o[j][r]);
                }
        range_block_store(range, lo, hi, nan);
    }
}

unsigned blocks_for(size_t n) { return unsigned((n + 255) / 256); }

}  // namespace

extern "C" {

int lq_layernorm_f32(const float* x, const float* gamma, const float* beta, float* out, long rows, int cols,
                     float eps, float* range, void* stream) {
    LQ_REQUIRE(x && gamma && beta && out, LQ_ERR_VALUE, "layernorm: null pointer");
    LQ_REQUIRE(rows >= 0 && cols > 0, LQ_ERR_SHAPE, "layernorm: bad shape (%ld, %d)", rows, cols);
    if (rows == 0) return LQ_OK;
    const long per_block = 4L * LN_ROWS_PER_WAVE;
    LQ_REQUIRE((rows + per_block - 1) / per_block < 0x7fffffffL, LQ_ERR_SHAPE, "layernorm: too many rows");
    LQ_REQUIRE(range == nullptr || (rows + per_block - 1) / per_block <= kRangeSlots, LQ_ERR_SHAPE,
               "layernorm: %ld rows are too many for a kept range (at most %ld)", rows,
               long(kRangeSlots) * per_block);
    layernorm_kernel<<<unsigned((rows + per_block - 1) / per_block), 256, 0, as_stream(stream)>>>(
        x, gamma, beta, out, rows, cols, eps, range);
    LQ_CHECK_LAUNCH();
    return LQ_OK;
}

int lq_layernorm_stats_f32(const float* x, const float* gamma, const float* beta, long rows, int cols, float eps,
                           float* stats, float* range, void* stream) {
    LQ_REQUIRE(x && gamma && beta && stats && range, LQ_ERR_VALUE, "layernorm_stats: null pointer");
    LQ_REQUIRE(rows >= 0 && cols > 0, LQ_ERR_SHAPE, "layernorm_stats: bad shape (%ld, %d)", rows, cols);
    LQ_REQUIRE(cols % 4 == 0 && cols <= LN_KEEP * 256 && aligned16(x) && aligned16(gamma) && aligned16(beta),
               LQ_ERR_NOT_IMPLEMENTED,
               "layernorm_stats: rows of %d floats; the fused form takes vector-aligned rows of a multiple of 4, "
               "at most %d (use lq_layernorm_f32 + lq_quantize)", cols, LN_KEEP * 256);
    if (rows == 0) return LQ_OK;
    const long blocks = (rows + 3) / 4;
    LQ_REQUIRE(blocks <= kRangeSlots, LQ_ERR_SHAPE, "layernorm_stats: %ld rows are too many for a kept range", rows);
    if (cols <= 4 * 256)
        layernorm_stats_kernel<4><<<unsigned(blocks), 256, 0, as_stream(stream)>>>(x, gamma, beta, rows, cols, eps, stats, range);
    else
        layernorm_stats_kernel<LN_KEEP><<<unsigned(blocks), 256, 0, as_stream(stream)>>>(x, gamma, beta, rows, cols, eps, stats,
                                                                                          range);
    LQ_CHECK_LAUNCH();
    return LQ_OK;
}

int lq_layernorm_quantize_i8(const float* x, const float* gamma, const float* beta, const float* stats, long rows,
                             int cols, const float* scale, const float* zp, int qmin, int qmax, int code_offset,
                             int8_t* q, void* stream) {
    LQ_REQUIRE(x && gamma && beta && stats && scale && zp && q, LQ_ERR_VALUE, "layernorm_quantize: null pointer");
    LQ_REQUIRE(rows >= 0 && cols > 0, LQ_ERR_SHAPE, "layernorm_quantize: bad shape (%ld, %d)", rows, cols);
    LQ_REQUIRE(cols % 4 == 0 && cols <= LN_KEEP * 256 && aligned16(x) && aligned16(gamma) && aligned16(beta) &&
                   (reinterpret_cast<uintptr_t>(q) & 3u) == 0,
               LQ_ERR_NOT_IMPLEMENTED, "layernorm_quantize: rows of %d floats are not what the fused form takes", cols);
    LQ_REQUIRE(qmax > qmin && qmin + code_offset >= -128 && qmax + code_offset <= 127, LQ_ERR_VALUE,
               "layernorm_quantize: grid [%d,%d] + offset %d does not fit int8", qmin, qmax, code_offset);
    if (rows == 0) return LQ_OK;
    layernorm_quantize_kernel<<<unsigned((rows + 3) / 4), 256, 0, as_stream(stream)>>>(
        x, gamma, beta, stats, rows, cols, scale, zp, float(qmin), float(qmax), code_offset, q);
    LQ_CHECK_LAUNCH();
    return LQ_OK;
}

int lq_gelu_f32(const float* x, float* out, size_t n, float* range, void* stream) {
    LQ_REQUIRE(x && out, LQ_ERR_VALUE, "gelu: null pointer");
    if (n == 0) return LQ_OK;
    const int vec = (n % 4 == 0) && aligned16(x) && aligned16(out);
    const size_t units = vec ? n / 4 : n;
    const size_t blocks = (units + 256 * GELU_PER_THREAD - 1) / (256 * GELU_PER_THREAD);
    LQ_REQUIRE(blocks < 0x7fffffffull, LQ_ERR_SHAPE, "gelu: tensor too large");
    LQ_REQUIRE(range == nullptr || blocks <= size_t(kRangeSlots), LQ_ERR_SHAPE,
               "gelu: %zu elements are too many for a kept range (at most %zu)", n,
               size_t(kRangeSlots) * 256 * GELU_PER_THREAD * 4);
    gelu_kernel<<<unsigned(blocks), 256, 0, as_stream(stream)>>>(x, out, n, vec, range);
    LQ_CHECK_LAUNCH();
    return LQ_OK;
}

int lq_add_f32(const float* a, const float* b, float* out, size_t n, void* stream) {
    LQ_REQUIRE(a && b && out, LQ_ERR_VALUE, "add: null pointer");
    if (n == 0) return LQ_OK;
    const int vec = (n % 4 == 0) && aligned16(a) && aligned16(b) && aligned16(out);
    add_kernel<<<blocks_for(vec ? n / 4 : n), 256, 0, as_stream(stream)>>>(a, b, out, n, vec);
    LQ_CHECK_LAUNCH();
    return LQ_OK;
}

int lq_patchify_f32(const float* img, float* out, int B, int C, int H, int W, int patch, void* stream) {
    LQ_REQUIRE(img && out, LQ_ERR_VALUE, "patchify: null pointer");
    LQ_REQUIRE(B >= 0 && C > 0 && H > 0 && W > 0 && patch > 0 && H % patch == 0 && W % patch == 0, LQ_ERR_SHAPE,
               "patchify: image %dx%dx%dx%d is not a whole number of %d-pixel patches", B, C, H, W, patch);
    const size_t total = size_t(B) * C * H * W;
    if (total == 0) return LQ_OK;
    patchify_kernel<<<blocks_for(total), 256, 0, as_stream(stream)>>>(img, out, B, C, H, W, patch);
    LQ_CHECK_LAUNCH();
    return LQ_OK;
}

int lq_assemble_tokens_f32(const float* patches, const float* cls, const float* pos, float* out, int B, int T,
                           int D, void* stream) {
    LQ_REQUIRE(patches && cls && pos && out, LQ_ERR_VALUE, "assemble_tokens: null pointer");
    LQ_REQUIRE(B >= 0 && T >= 1 && D > 0, LQ_ERR_SHAPE, "assemble_tokens: bad shape");
    const size_t total = size_t(B) * T * D;
    if (total == 0) return LQ_OK;
    assemble_tokens_kernel<<<blocks_for(total), 256, 0, as_stream(stream)>>>(patches, cls, pos, out, B, T, D);
    LQ_CHECK_LAUNCH();
    return LQ_OK;
}

int lq_sgemm_nt_f32(const float* a, const float* w, const float* bias, float* out, int M, int N, int K,
                    void* stream) {
    LQ_REQUIRE(a && w && out, LQ_ERR_VALUE, "sgemm: null pointer");
    LQ_REQUIRE(M >= 0 && N >= 0 && K > 0, LQ_ERR_SHAPE, "sgemm: bad shape (%d, %d, %d)", M, N, K);
    if (M == 0 || N == 0) return LQ_OK;
    dim3 grid((N + SG_BN - 1) / SG_BN, (M + SG_BM - 1) / SG_BM);
    LQ_REQUIRE(grid.y < 65536, LQ_ERR_SHAPE, "sgemm: M too large");
    sgemm_nt_kernel<0><<<grid, 256, 0, as_stream(stream)>>>(a, w, bias, out, M, N, K, PatchForm{});
    LQ_CHECK_LAUNCH();
    return LQ_OK;
}

int lq_patch_embed_f32(const float* img, const float* w, const float* bias, const float* cls, const float* pos,
                       float* out, int B, int C, int H, int W, int patch, int D, void* stream) {
    LQ_REQUIRE(img && w && cls && pos && out, LQ_ERR_VALUE, "patch_embed: null pointer");
    LQ_REQUIRE(B >= 0 && C > 0 && H > 0 && W > 0 && D > 0 && patch > 0 && H % patch == 0 && W % patch == 0,
               LQ_ERR_SHAPE, "patch_embed: image %dx%dx%dx%d is not a whole number of %d-pixel patches", B, C, H, W,
               patch);
    const int per_image = (H / patch) * (W / patch);
    const size_t rows = size_t(B) * per_image, K = size_t(C) * patch * patch;
    LQ_REQUIRE(rows < (size_t(1) << 31) && K < (size_t(1) << 31), LQ_ERR_SHAPE, "patch_embed: too many patch rows");
    if (B == 0) return LQ_OK;
    dim3 grid((D + SG_BN - 1) / SG_BN, (unsigned(rows) + SG_BM - 1) / SG_BM);
    LQ_REQUIRE(grid.y < 65536, LQ_ERR_SHAPE, "patch_embed: too many patch rows");
    int log2p = -1;
    for (int e = 0; e < 15; ++e)
        if ((1 << e) == patch) log2p = e;
    const PatchForm pf{C, H, W, patch, W / patch, per_image, B, log2p, cls, pos};
    if (log2p >= 2 && W % 4 == 0 && aligned16(img))
        sgemm_nt_kernel<1><<<grid, 256, 0, as_stream(stream)>>>(img, w, bias, out, int(rows), D, int(K), pf);
    else
        sgemm_nt_kernel<2><<<grid, 256, 0, as_stream(stream)>>>(img, w, bias, out, int(rows), D, int(K), pf);
    LQ_CHECK_LAUNCH();
    return LQ_OK;
}

int lq_gather_rows_f32(const float* src, size_t src_row_stride, float* dst, size_t rows, size_t cols,
                       void* stream) {
    LQ_REQUIRE(src && dst, LQ_ERR_VALUE, "gather_rows: null pointer");
    LQ_REQUIRE(src_row_stride >= cols, LQ_ERR_SHAPE, "gather_rows: row stride smaller than the row");
    if (rows * cols == 0) return LQ_OK;
    gather_rows_kernel<<<blocks_for(rows * cols), 256, 0, as_stream(stream)>>>(src, src_row_stride, dst, rows, cols);
    LQ_CHECK_LAUNCH();
    return LQ_OK;
}

int lq_attention_f32(const float* qkv, float* out, int B, int T, int H, int D, float scale, float* range,
                     void* stream) {
    LQ_REQUIRE(qkv && out, LQ_ERR_VALUE, "attention: null pointer");
    LQ_REQUIRE(B >= 0 && T >= 1 && H >= 1, LQ_ERR_SHAPE, "attention: bad shape");
    LQ_REQUIRE(D == AT_D && T <= AT_TMAX, LQ_ERR_NOT_IMPLEMENTED,
               "attention: head dim %d / %d tokens; this kernel handles head dim 64 and up to 208 tokens", D, T);
    LQ_REQUIRE(aligned16(qkv), LQ_ERR_VALUE, "attention: qkv must be 16-byte aligned");
    if (B == 0) return LQ_OK;
    LQ_REQUIRE(range == nullptr || long(B) * H <= kRangeSlots, LQ_ERR_SHAPE,
               "attention: too many (batch, head) pairs for a kept range");
    const int tiles = (T + 15) / 16;
    const int waves = tiles + ((tiles > 1 && tiles % 4 == 1) ? 3 : 0);  // see the kernel: the last tile shared by four
    constexpr size_t kSmem = AT_SMEM;
    static DeviceOnce attr_once;
    if (int rc = allow_dynamic_lds(attr_once, reinterpret_cast<const void*>(attention_kernel), int(kSmem))) return rc;
    attention_kernel<<<unsigned(B) * H, waves * 64, kSmem, as_stream(stream)>>>(qkv, out, B, T, H, scale,
                                                                                 range);
    LQ_CHECK_LAUNCH();
    return LQ_OK;
}

}  // extern "C"
