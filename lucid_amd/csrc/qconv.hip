// Quantized Conv2d forward for gfx950: convolution lowered to the int8 MFMA
// GEMM, plus the layout helpers around it.
//
// Activations are int8 codes in NHWC, weights int8 [Cout][KH][KW][Cin/groups],
// the result is NHWC in the form the epilogue mode asks for.  The GEMM view is
// M = B*OH*OW, N = Cout/groups, K = KH*KW*Cin/groups.  Out-of-image taps read
// the activation zero-point code: Lucid pads the float image with 0.0
// (lucid/_C/backend/cpu/Im2Col.cpp:59-100), which on the activation grid is
// the code Z.  Three routes:
//   gemm     : 1x1, stride 1, no padding -> the NHWC tensor IS the A matrix
//   implicit : Cin/groups % 16 == 0 -> the tile kernel gathers A on the fly
//   packed   : at most four input channels (an RGB stem) -> image repacked once to
//              4 channels with the padding materialised; a filter row is then
//              contiguous bytes and the tile kernel gathers it without im2col
//   im2col   : anything else -> explicit int8 im2col into the workspace with K
//              padded to a multiple of 16, then the GEMM
//   naive    : one output per lane, any shape (checking aid)
#include "common.hpp"
#include "qepilogue.hpp"
#include "qgemm.hpp"

using namespace lq;

namespace {

struct ConvShape {
    int B, H, W, Cin, Cout, KH, KW, OH, OW;
    int sh, sw, ph, pw, dh, dw, groups;
};

// ---------------------------------------------------------------- naive
__global__ __launch_bounds__(256) void qconv_naive_kernel(GemmArgs g, ConvShape c, const int8_t* x,
                                                          const int8_t* w) {
    const int Cg = c.Cin / c.groups, Og = c.Cout / c.groups;
    const size_t total = size_t(c.B) * c.OH * c.OW * c.Cout;
    float S = 1.0f, Z = 0.0f;
    if (g.out_mode == OUT_REQUANT_I8 || g.out_mode == OUT_FAKEQUANT_F32) {
        S = g.out_scale[0];
        Z = g.out_zp[0];
    }
    const float as = g.a_scale ? g.a_scale[0] : 1.0f;
    for (size_t idx = size_t(blockIdx.x) * 256 + threadIdx.x; idx < total;
         idx += size_t(gridDim.x) * 256) {
        const int co = int(idx % c.Cout);
        size_t p = idx / c.Cout;
        const int ow = int(p % c.OW);
        p /= c.OW;
        const int oh = int(p % c.OH);
        const int b = int(p / c.OH);
        const int grp = co / Og;
        int32_t acc = 0;
        for (int kh = 0; kh < c.KH; ++kh)
            for (int kw = 0; kw < c.KW; ++kw) {
                const int ih = oh * c.sh - c.ph + kh * c.dh, iw = ow * c.sw - c.pw + kw * c.dw;
                const int8_t* wr = w + ((size_t(co) * c.KH + kh) * c.KW + kw) * Cg;
                if (ih < 0 || ih >= c.H || iw < 0 || iw >= c.W) {
                    int ws = 0;
                    for (int ci = 0; ci < Cg; ++ci) ws += wr[ci];
                    acc += g.a_zp * ws;
                } else {
                    const int8_t* xr = x + ((size_t(b) * c.H + ih) * c.W + iw) * c.Cin + grp * Cg;
                    for (int ci = 0; ci < Cg; ++ci) acc += int(xr[ci]) * int(wr[ci]);
                }
            }
        const int m = int(idx / c.Cout);
        epilogue_store(g, m, co, acc, as, load_col(g, co), S, Z);
    }
}

// ---------------------------------------------------------------- explicit im2col
// cols[m][k], k = (kh*KW + kw)*Cg + ci for k < K, zero for K <= k < Kp.
__global__ __launch_bounds__(256) void im2col_i8_kernel(const int8_t* __restrict__ x,
                                                        int8_t* __restrict__ cols, ConvShape c,
                                                        int grp, int K, int Kp, int8_t pad_code) {
    const int Cg = c.Cin / c.groups;
    const size_t total = size_t(c.B) * c.OH * c.OW * Kp;
    for (size_t idx = size_t(blockIdx.x) * 256 + threadIdx.x; idx < total;
         idx += size_t(gridDim.x) * 256) {
        const int k = int(idx % Kp);
        size_t m = idx / Kp;
        int8_t v = 0;
        if (k < K) {
            const int ci = k % Cg, tap = k / Cg;
            const int kw = tap % c.KW, kh = tap / c.KW;
            const int ow = int(m % c.OW);
            size_t q = m / c.OW;
            const int oh = int(q % c.OH), b = int(q / c.OH);
            const int ih = oh * c.sh - c.ph + kh * c.dh, iw = ow * c.sw - c.pw + kw * c.dw;
            v = (ih < 0 || ih >= c.H || iw < 0 || iw >= c.W)
                    ? pad_code
                    : x[((size_t(b) * c.H + ih) * c.W + iw) * c.Cin + grp * Cg + ci];
        }
        cols[idx] = v;
    }
}

// weight rows of one group, K bytes each, copied into rows of Kp bytes (zero tail)
__global__ void pad_rows_kernel(const int8_t* __restrict__ w, int8_t* __restrict__ out, int rows,
                                int K, int Kp) {
    const size_t total = size_t(rows) * Kp;
    for (size_t idx = size_t(blockIdx.x) * blockDim.x + threadIdx.x; idx < total;
         idx += size_t(gridDim.x) * blockDim.x) {
        const int k = int(idx % Kp);
        const size_t r = idx / Kp;
        out[idx] = k < K ? w[r * K + k] : int8_t(0);
    }
}

// ---------------------------------------------------------------- few input channels
// A convolution over at most four input channels (an RGB stem) as an implicit GEMM
// without im2col: the image is copied once into a 4-channel, spatially pre-padded
// buffer - padding and the spare channels hold the zero-point code -, so that four
// neighbouring pixels of a row are one 16-byte chunk and a filter row of KWp = KW
// rounded up to 4 taps is KWp * 4 contiguous bytes.  The tile kernel then gathers it as a
// convolution over 16-byte "super pixels": KWp / 4 taps per filter row, each four real
// pixels apart, no bounds to check.  The filter gets zeros in the added taps and channel.
__global__ __launch_bounds__(256) void pack4_padded_kernel(const int8_t* __restrict__ x, int B, int H, int W, int C,
                                                           int ph, int pw, int Hp, int Wp, int fill,
                                                           uint32_t* __restrict__ out) {
    const size_t n = size_t(B) * Hp * Wp, stride = size_t(gridDim.x) * 256;
    const uint32_t f = uint32_t(uint8_t(fill));
    for (size_t i = size_t(blockIdx.x) * 256 + threadIdx.x; i < n; i += stride) {
        const int wp = int(i % Wp);
        size_t r = i / Wp;
        const int hp = int(r % Hp), b = int(r / Hp);
        const int h = hp - ph, w = wp - pw;
        uint32_t v = f | (f << 8) | (f << 16) | (f << 24);
        if (h >= 0 && h < H && w >= 0 && w < W) {
            const int8_t* src = x + ((size_t(b) * H + h) * W + w) * C;
            v = 0;
            for (int c = 0; c < 4; ++c) v |= (c < C ? uint32_t(uint8_t(src[c])) : f) << (8 * c);
        }
        out[i] = v;
    }
}

// w [Cout, KH, KW, C] -> [Cout, KH, KWp, 4], zeros in the added taps and channels
__global__ void pack4_filter_kernel(const int8_t* __restrict__ w, int Cout, int KH, int KW, int C, int KWp,
                                    int8_t* __restrict__ out) {
    const size_t total = size_t(Cout) * KH * KWp * 4;
    for (size_t idx = size_t(blockIdx.x) * blockDim.x + threadIdx.x; idx < total;
         idx += size_t(gridDim.x) * blockDim.x) {
        const int c = int(idx % 4);
        size_t r = idx / 4;
        const int kw = int(r % KWp);
        r /= KWp;  // = co * KH + kh
        out[idx] = (c < C && kw < KW) ? w[(r * KW + kw) * C + c] : int8_t(0);
    }
}

// ---------------------------------------------------------------- layout helpers
__device__ __forceinline__ float q_core_local(float x, float s, float z, float lo, float hi) {
    float t = x / s;
    float r = __builtin_rintf(t);
    float u = r + z;
    u = (u < lo) ? lo : ((u > hi) ? hi : u);
    return u;
}

// float32 NCHW -> int8 NHWC codes (per-tensor qparams): the entry Quantize of a
// convolutional model.  A block transposes a [C-tile][W-tile] patch through LDS.
__global__ __launch_bounds__(256) void quantize_nchw_to_nhwc_kernel(
    const float* __restrict__ x, int8_t* __restrict__ q, int B, int C, int HW, const float* scale,
    const float* zp, float lo, float hi, int off) {
    __shared__ int8_t tile[32][33];
    const float s = scale[0], z = zp[0];
    const int b = blockIdx.z, c0 = blockIdx.y * 32, p0 = blockIdx.x * 32;
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;  // 32 x 8
    for (int j = ty; j < 32; j += 8) {
        const int c = c0 + j, p = p0 + tx;
        int8_t v = 0;
        if (c < C && p < HW) {
            float u = q_core_local(x[(size_t(b) * C + c) * HW + p], s, z, lo, hi);
            v = int8_t(((u != u) ? 0 : int(u)) + off);
        }
        tile[j][tx] = v;
    }
    __syncthreads();
    for (int j = ty; j < 32; j += 8) {
        const int p = p0 + j, c = c0 + tx;
        if (c < C && p < HW) q[(size_t(b) * HW + p) * C + c] = tile[tx][j];
    }
}

// int8 NHWC codes -> float32 NCHW: the float view of a convolutional activation
__global__ __launch_bounds__(256) void dequantize_nhwc_to_nchw_kernel(
    const int8_t* __restrict__ q, int off, float* __restrict__ out, int B, int C, int HW,
    const float* scale, const float* zp) {
    __shared__ float tile[32][33];
    const float s = scale[0], z = zp[0];
    const int b = blockIdx.z, c0 = blockIdx.y * 32, p0 = blockIdx.x * 32;
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
    for (int j = ty; j < 32; j += 8) {
        const int p = p0 + j, c = c0 + tx;
        float v = 0.0f;
        if (c < C && p < HW) v = (float(int(q[(size_t(b) * HW + p) * C + c]) - off) - z) * s;
        tile[j][tx] = v;
    }
    __syncthreads();
    for (int j = ty; j < 32; j += 8) {
        const int c = c0 + j, p = p0 + tx;
        if (c < C && p < HW) out[(size_t(b) * C + c) * HW + p] = tile[tx][j];
    }
}

// weight codes OIHW -> O,KH,KW,I (the K order of the implicit GEMM); one-time
__global__ void repack_oihw_to_ohwi_kernel(const int8_t* __restrict__ w, int8_t* __restrict__ out,
                                           int O, int I, int KH, int KW) {
    const size_t total = size_t(O) * I * KH * KW;
    for (size_t idx = size_t(blockIdx.x) * blockDim.x + threadIdx.x; idx < total;
         idx += size_t(gridDim.x) * blockDim.x) {
        const int i = int(idx % I);
        size_t r = idx / I;
        const int kw = int(r % KW);
        r /= KW;
        const int kh = int(r % KH);
        const int o = int(r / KH);
        out[idx] = w[((size_t(o) * I + i) * KH + kh) * KW + kw];
    }
}

// Volumetric convolution as an explicit GEMM.  x: codes in channels-last order
// (B, D, H, W, C); cols: [B*OD*OH*OW, KD*KH*KW*Cg] with k = ((kd*KH + kh)*KW + kw)*Cg + c over
// the channels [c0, c0 + Cg) of one group; taps in the padding read pad_code (the zero point's
// stored code).  `ins` > 1 spreads the input over a grid with ins - 1 zero-point codes between
// neighbours (the zero insertion of a transposed convolution) without materialising it.
// A lane moves VEC consecutive channels of one tap (16 where the channel counts and pointers
// allow, else 1), consecutive lanes consecutive chunks: reads and writes are contiguous runs.
struct Vol3 {
    int d, h, w;
};

template <int VEC>
__global__ void im2col_ndhwc_i8_kernel(const int8_t* __restrict__ x, int8_t* __restrict__ cols, int C, Vol3 in,
                                       int c0, int Cg, Vol3 kern, Vol3 stride, Vol3 pad, Vol3 dil, Vol3 ins,
                                       Vol3 out, int pad_code, size_t units) {
    const int chunks = Cg / VEC;
    const unsigned pad4 = unsigned(pad_code & 0xff) * 0x01010101u;
    for (size_t idx = size_t(blockIdx.x) * blockDim.x + threadIdx.x; idx < units;
         idx += size_t(gridDim.x) * blockDim.x) {
        const int chunk = int(idx % chunks);
        size_t r = idx / chunks;
        const int taps = kern.d * kern.h * kern.w;
        int tap = int(r % taps);
        size_t m = r / taps;
        const int kw = tap % kern.w;
        tap /= kern.w;
        const int kh = tap % kern.h, kd = tap / kern.h;
        const int ow = int(m % out.w);
        m /= out.w;
        const int oh = int(m % out.h);
        m /= out.h;
        const int od = int(m % out.d);
        const size_t b = m / out.d;
        // coordinates on the spread grid; a real sample sits at every ins-th of them
        const int vd = od * stride.d - pad.d + kd * dil.d;
        const int vh = oh * stride.h - pad.h + kh * dil.h;
        const int vw = ow * stride.w - pad.w + kw * dil.w;
        const int8_t* src = nullptr;
        if (vd >= 0 && vh >= 0 && vw >= 0 && vd % ins.d == 0 && vh % ins.h == 0 && vw % ins.w == 0) {
            const int id = vd / ins.d, ih = vh / ins.h, iw = vw / ins.w;
            if (id < in.d && ih < in.h && iw < in.w)
                src = x + (((b * in.d + id) * in.h + ih) * size_t(in.w) + iw) * C + c0 + chunk * VEC;
        }
        int8_t* dst = cols + idx * VEC;  // (m, tap, chunk) in this order IS the matrix order
        if (VEC == 16) {
            uint4 v = {pad4, pad4, pad4, pad4};
            if (src) v = *reinterpret_cast<const uint4*>(src);
            *reinterpret_cast<uint4*>(dst) = v;
        } else {
            *dst = src ? *src : int8_t(pad_code);
        }
    }
}

// Batched byte transpose through LDS: src[b] is R x Cn (rows contiguous), dst[b] is Cn x R;
// batches are src_stride / dst_stride bytes apart (so a destination may be a channel slice of
// a larger tensor).  64 x 64 tiles; a wavefront reads and writes 64 consecutive bytes.
__global__ __launch_bounds__(256) void transpose_i8_kernel(const int8_t* __restrict__ src, int8_t* __restrict__ dst,
                                                           size_t R, size_t Cn, size_t src_stride,
                                                           size_t dst_stride, unsigned tiles_c) {
    __shared__ int8_t tile[64][65];
    const size_t r0 = size_t(blockIdx.x / tiles_c) * 64, c0 = size_t(blockIdx.x % tiles_c) * 64;
    const int8_t* s = src + size_t(blockIdx.y) * src_stride;
    int8_t* d = dst + size_t(blockIdx.y) * dst_stride;
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
#pragma unroll
    for (int j = 0; j < 16; ++j) {
        const size_t r = r0 + j * 4 + w, c = c0 + lane;
        if (r < R && c < Cn) tile[j * 4 + w][lane] = s[r * Cn + c];
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < 16; ++j) {
        const size_t c = c0 + j * 4 + w, r = r0 + lane;
        if (r < R && c < Cn) d[c * R + r] = tile[lane][j * 4 + w];
    }
}

// Non-zero padding modes of F.pad on NHWC codes (reflect / replicate / circular):
// the padded float image is a gather of the original, so the padded code image is
// the same gather of the codes.  One lane per 16 channels when C % 16 == 0, else per byte.
__device__ __forceinline__ int pad_source(int i, int n, int mode) {
    if (i >= 0 && i < n) return i;
    if (mode == 1) {  // reflect: -1 -> 1, n -> n - 2 (no edge repeat)
        i = i < 0 ? -i : 2 * (n - 1) - i;
        return i;
    }
    if (mode == 2) return i < 0 ? 0 : n - 1;  // replicate
    i %= n;                                   // circular
    return i < 0 ? i + n : i;
}

__global__ __launch_bounds__(256) void pad_nhwc_i8_kernel(const int8_t* __restrict__ x, int8_t* __restrict__ out,
                                                          int B, int H, int W, int C, int pt, int pl, int OH,
                                                          int OW, int mode, int vec) {
    const int cunits = vec ? C / 16 : C;
    const size_t total = size_t(B) * OH * OW * cunits;
    const size_t i = size_t(blockIdx.x) * 256 + threadIdx.x;
    if (i >= total) return;
    const int cu = int(i % cunits);
    const size_t pix = i / cunits;
    const int ow = int(pix % OW), oh = int((pix / OW) % OH);
    const size_t b = pix / (size_t(OW) * OH);
    const int ih = pad_source(oh - pt, H, mode), iw = pad_source(ow - pl, W, mode);
    const size_t src = ((b * H + ih) * W + iw) * C, dst = pix * C;
    if (vec)
        reinterpret_cast<uint4*>(out + dst)[cu] = reinterpret_cast<const uint4*>(x + src)[cu];
    else
        out[dst + cu] = x[src + cu];
}


// F.pad on the last two axes of a float tensor viewed as `planes` images of H x W: mode 0 pads
// with zeros, 1 / 2 / 3 are reflect / replicate / circular.  One lane per output element.
__global__ __launch_bounds__(256) void pad_planes_f32_kernel(const float* __restrict__ x, float* __restrict__ out,
                                                             size_t planes, int H, int W, int pt, int pl, int OH,
                                                             int OW, int mode) {
    const size_t total = planes * OH * OW;
    const size_t i = size_t(blockIdx.x) * 256 + threadIdx.x;
    if (i >= total) return;
    const int ow = int(i % OW), oh = int((i / OW) % OH);
    const size_t p = i / (size_t(OW) * OH);
    const int ih0 = oh - pt, iw0 = ow - pl;
    float v = 0.0f;
    if (mode != 0 || (ih0 >= 0 && ih0 < H && iw0 >= 0 && iw0 < W)) {
        const int ih = pad_source(ih0, H, mode), iw = pad_source(iw0, W, mode);
        v = x[(p * H + ih) * W + iw];
    }
    out[i] = v;
}

// max-pool on codes, NHWC.  Quantisation is monotone, so the maximum of the
// codes is the code of the maximum; padded taps never win.
__global__ __launch_bounds__(256) void maxpool_nhwc_i8_kernel(const int8_t* __restrict__ x,
                                                              int8_t* __restrict__ out, int B, int H,
                                                              int W, int C, int KH, int KW, int sh,
                                                              int sw, int ph, int pw, int OH, int OW) {
    const size_t total = size_t(B) * OH * OW * C;
    for (size_t idx = size_t(blockIdx.x) * 256 + threadIdx.x; idx < total;
         idx += size_t(gridDim.x) * 256) {
        const int c = int(idx % C);
        size_t p = idx / C;
        const int ow = int(p % OW);
        p /= OW;
        const int oh = int(p % OH);
        const int b = int(p / OH);
        int best = -128;
        for (int kh = 0; kh < KH; ++kh)
            for (int kw = 0; kw < KW; ++kw) {
                const int ih = oh * sh - ph + kh, iw = ow * sw - pw + kw;
                if (ih < 0 || ih >= H || iw < 0 || iw >= W) continue;
                const int v = x[((size_t(b) * H + ih) * W + iw) * C + c];
                best = v > best ? v : best;
            }
        out[idx] = int8_t(best);
    }
}

// The same, sixteen channels per lane (C % 16 == 0, 16-byte aligned tensors): a lane
// keeps a running per-byte maximum of 16-byte loads.
__device__ __forceinline__ uint32_t max_i8x4(uint32_t a, uint32_t b) {
    uint32_t r = 0;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const int x = int(int8_t((a >> (8 * e)) & 0xff)), y = int(int8_t((b >> (8 * e)) & 0xff));
        r |= uint32_t(uint8_t(x > y ? x : y)) << (8 * e);
    }
    return r;
}

__global__ __launch_bounds__(256) void maxpool_nhwc_i8x16_kernel(const uint4* __restrict__ x, uint4* __restrict__ out,
                                                                 int B, int H, int W, int C16, int KH, int KW,
                                                                 int sh, int sw, int ph, int pw, int OH, int OW) {
    const size_t total = size_t(B) * OH * OW * C16;
    for (size_t idx = size_t(blockIdx.x) * 256 + threadIdx.x; idx < total; idx += size_t(gridDim.x) * 256) {
        const int c = int(idx % C16);
        size_t p = idx / C16;
        const int ow = int(p % OW);
        p /= OW;
        const int oh = int(p % OH), b = int(p / OH);
        uint4 best = {0x80808080u, 0x80808080u, 0x80808080u, 0x80808080u};  // -128 in every byte
        for (int kh = 0; kh < KH; ++kh) {
            const int ih = oh * sh - ph + kh;
            if (ih < 0 || ih >= H) continue;
            for (int kw = 0; kw < KW; ++kw) {
                const int iw = ow * sw - pw + kw;
                if (iw < 0 || iw >= W) continue;
                const uint4 v = x[((size_t(b) * H + ih) * W + iw) * C16 + c];
                best.x = max_i8x4(best.x, v.x);
                best.y = max_i8x4(best.y, v.y);
                best.z = max_i8x4(best.z, v.z);
                best.w = max_i8x4(best.w, v.w);
            }
        }
        out[idx] = best;
    }
}

// The same with the window size known at compile time: every tap's 16 bytes are requested before
// the first maximum is taken (taps outside the image read a clamped address and are replaced by
// -128).  With run-time loops and their bounds tests each tap's load was waited for before the next
// one was requested: nine memory round trips in a row for a 3 x 3 window.
template <int KH, int KW>
__global__ __launch_bounds__(256) void maxpool_nhwc_i8x16_fixed_kernel(const uint4* __restrict__ x, uint4* __restrict__ out,
                                                                       int B, int H, int W, int C16, int sh, int sw,
                                                                       int ph, int pw, int OH, int OW) {
    const size_t total = size_t(B) * OH * OW * C16;
    for (size_t idx = size_t(blockIdx.x) * 256 + threadIdx.x; idx < total; idx += size_t(gridDim.x) * 256) {
        const int c = int(idx % C16);
        size_t p = idx / C16;
        const int ow = int(p % OW);
        p /= OW;
        const int oh = int(p % OH), b = int(p / OH);
        uint4 v[KH][KW];
        bool ok[KH][KW];
#pragma unroll
        for (int kh = 0; kh < KH; ++kh) {
            const int ih = oh * sh - ph + kh;
            const int ihc = ih < 0 ? 0 : (ih >= H ? H - 1 : ih);
#pragma unroll
            for (int kw = 0; kw < KW; ++kw) {
                const int iw = ow * sw - pw + kw;
                const int iwc = iw < 0 ? 0 : (iw >= W ? W - 1 : iw);
                ok[kh][kw] = ih == ihc && iw == iwc;
                v[kh][kw] = x[((size_t(b) * H + ihc) * W + iwc) * C16 + c];
            }
        }
        uint4 best = {0x80808080u, 0x80808080u, 0x80808080u, 0x80808080u};  // -128 in every byte
#pragma unroll
        for (int kh = 0; kh < KH; ++kh)
#pragma unroll
            for (int kw = 0; kw < KW; ++kw) {
                const uint4 t = v[kh][kw];
                const bool k = ok[kh][kw];
                best.x = max_i8x4(best.x, k ? t.x : 0x80808080u);
                best.y = max_i8x4(best.y, k ? t.y : 0x80808080u);
                best.z = max_i8x4(best.z, k ? t.z : 0x80808080u);
                best.w = max_i8x4(best.w, k ? t.w : 0x80808080u);
            }
        out[idx] = best;
    }
}

// float32 NCHW -> int8 NHWC for at most four channels (an RGB image): one pixel per
// lane, plane reads and pixel writes both contiguous across a wavefront.
__global__ __launch_bounds__(256) void quantize_nchw_to_nhwc_small_c_kernel(
    const float* __restrict__ x, int8_t* __restrict__ q, int C, size_t HW, const float* scale, const float* zp,
    float lo, float hi, int off) {
    const float s = scale[0], z = zp[0];
    const size_t b = blockIdx.y;
    for (size_t p = size_t(blockIdx.x) * 256 + threadIdx.x; p < HW; p += size_t(gridDim.x) * 256) {
        int8_t v[4];
        for (int c = 0; c < C; ++c) {
            const float u = q_core_local(x[(b * C + c) * HW + p], s, z, lo, hi);
            v[c] = int8_t(((u != u) ? 0 : int(u)) + off);
        }
        int8_t* dst = q + (b * HW + p) * C;
        if (C == 4)
            *reinterpret_cast<uint32_t*>(dst) = *reinterpret_cast<const uint32_t*>(v);
        else
            for (int c = 0; c < C; ++c) dst[c] = v[c];
    }
}

// float32 NCHW (at most four channels) -> the packed four-channel, spatially pre-padded code
// image of the few-channel route, in one pass: what lq_quantize_nchw_to_nhwc followed by
// pack4_padded_kernel writes (the same quantization arithmetic; padding and spare channels hold
// `fill`, the zero-point code).  A lane writes four consecutive packed pixels of one row as one
// 16-byte store (rows of the packed image are a multiple of four pixels); its up to twelve
// inputs are loaded from clamped addresses, all before the first is used, and what lies in the
// padding is replaced afterwards.  Block = 64 quads x 4 rows, grid = (quads, rows, images).
__global__ __launch_bounds__(256) void quantize_nchw_to_packed4_kernel(
    const float* __restrict__ x, int B, int C, int H, int W, int ph, int pw, int Hp, int Wp, const float* scale,
    const float* zp, float lo, float hi, int off, int fill, uint4* __restrict__ out) {
    const int qx = blockIdx.x * 64 + (threadIdx.x & 63), hp = blockIdx.y * 4 + (threadIdx.x >> 6), b = blockIdx.z;
    if (qx * 4 >= Wp || hp >= Hp) return;
    const float s = scale[0], z = zp[0];
    const int h = hp - ph, w0 = qx * 4 - pw;
    const bool row_in = h >= 0 && h < H;
    const size_t HW = size_t(H) * W;
    const float* xr = x + size_t(b) * C * HW + size_t(row_in ? h : 0) * W;
    float v[4][4];
#pragma unroll
    for (int c = 0; c < 4; ++c)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int w = w0 + j;
            v[c][j] = c < C ? xr[size_t(c) * HW + (w < 0 ? 0 : (w >= W ? W - 1 : w))] : 0.0f;
        }
    const uint32_t f = uint32_t(uint8_t(fill));
    uint32_t px[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int w = w0 + j;
        uint32_t p = 0;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            uint32_t code = f;
            if (c < C) {
                const float u = q_core_local(v[c][j], s, z, lo, hi);
                code = uint32_t(uint8_t(int8_t(((u != u) ? 0 : int(u)) + off)));
            }
            p |= code << (8 * c);
        }
        px[j] = (row_in && w >= 0 && w < W) ? p : (f | (f << 8) | (f << 16) | (f << 24));
    }
    out[(size_t(b) * Hp + hp) * (Wp / 4) + qx] = uint4{px[0], px[1], px[2], px[3]};
}

// Extents of the packed image of a few-channel layer: rows start 16-byte aligned and the last
// output's window of KWp pixels lies inside the row.
void packed4_geometry(const lq_qconv2d_args* p, int OW, int* KWp, int* Hp, int* Wp) {
    *KWp = (p->KW + 3) / 4 * 4;
    *Hp = p->H + p->pad_h_lo + p->pad_h_hi;
    int wp = p->W + p->pad_w_lo + p->pad_w_hi;
    const int need = (OW - 1) * p->stride_w + *KWp;
    wp = wp > need ? wp : need;
    *Wp = (wp + 3) / 4 * 4;
}

inline unsigned grid_1d(size_t n, unsigned per_block = 256) {
    size_t b = (n + per_block - 1) / per_block;
    if (b < 1) b = 1;
    return unsigned(b > 262144 ? 262144 : b);
}

}  // namespace

extern "C" {

int lq_qconv2d_i8(const lq_qconv2d_args* p, lq_stream stream) {
    LQ_REQUIRE(p, LQ_ERR_VALUE, "qconv2d_i8: args is NULL");
    LQ_REQUIRE(p->B >= 0 && p->H > 0 && p->W > 0 && p->Cin > 0 && p->Cout > 0 && p->KH > 0 &&
                   p->KW > 0,
               LQ_ERR_SHAPE, "qconv2d_i8: non-positive extent");
    LQ_REQUIRE(p->groups >= 1 && p->Cin % p->groups == 0 && p->Cout % p->groups == 0, LQ_ERR_SHAPE,
               "qconv2d_i8: channels (%d -> %d) not divisible by groups %d", p->Cin, p->Cout,
               p->groups);
    LQ_REQUIRE(p->stride_h >= 1 && p->stride_w >= 1 && p->dil_h >= 1 && p->dil_w >= 1 &&
                   p->pad_h_lo >= 0 && p->pad_h_hi >= 0 && p->pad_w_lo >= 0 && p->pad_w_hi >= 0,
               LQ_ERR_VALUE, "qconv2d_i8: bad stride / dilation / padding");
    // output extent, lucid/_C/nn/ConvNd.cpp:56-59
    const int OH = (p->H + p->pad_h_lo + p->pad_h_hi - p->dil_h * (p->KH - 1) - 1) / p->stride_h + 1;
    const int OW = (p->W + p->pad_w_lo + p->pad_w_hi - p->dil_w * (p->KW - 1) - 1) / p->stride_w + 1;
    LQ_REQUIRE(OH > 0 && OW > 0, LQ_ERR_SHAPE, "qconv2d_i8: empty output (%d x %d)", OH, OW);
    if (p->B == 0) return LQ_OK;
    LQ_REQUIRE(p->x && p->w && p->out, LQ_ERR_VALUE, "qconv2d_i8: NULL tensor pointer");
    LQ_REQUIRE(p->out_mode >= OUT_ACC_I32 && p->out_mode <= OUT_FAKEQUANT_F32, LQ_ERR_VALUE,
               "qconv2d_i8: unknown out_mode %d", p->out_mode);
    LQ_REQUIRE(p->a_zp >= -128 && p->a_zp <= 127, LQ_ERR_VALUE,
               "qconv2d_i8: activation zero point %d is not an int8 code", p->a_zp);
    const int Cg = p->Cin / p->groups, Og = p->Cout / p->groups;
    const long K = long(p->KH) * p->KW * Cg;
    LQ_REQUIRE(K <= 131071, LQ_ERR_SHAPE, "qconv2d_i8: K = %ld overflows the int32 accumulator", K);
    const size_t M = size_t(p->B) * OH * OW;
    LQ_REQUIRE(M <= 0x7fffffffull && size_t(p->B) * p->H * p->W * p->Cin < 0xffffffffull,
               LQ_ERR_SHAPE, "qconv2d_i8: tensor too large for 32-bit indexing");
    if (p->out_mode != OUT_ACC_I32) {
        LQ_REQUIRE(p->w_scale && p->a_scale, LQ_ERR_VALUE, "qconv2d_i8: scale pointer is NULL");
        LQ_REQUIRE(p->a_zp == 0 || p->wsum, LQ_ERR_VALUE,
                   "qconv2d_i8: a non-zero activation zero point needs the filter sums");
        LQ_REQUIRE(p->bias == nullptr || p->bias_dtype == LQ_F32 || p->bias_dtype == LQ_F16,
                   LQ_ERR_DTYPE, "qconv2d_i8: bias must be float32 or float16");
    }
    if (p->out_mode == OUT_REQUANT_I8 || p->out_mode == OUT_FAKEQUANT_F32) {
        LQ_REQUIRE(p->out_scale && p->out_zp, LQ_ERR_VALUE, "qconv2d_i8: output qparams are NULL");
        if (p->out_mode == OUT_REQUANT_I8)
            LQ_REQUIRE(p->out_qmin + p->out_offset >= -128 && p->out_qmax + p->out_offset <= 127,
                       LQ_ERR_VALUE, "qconv2d_i8: output grid + offset does not fit int8");
    }

    hipStream_t st = as_stream(stream);
    GemmArgs g{};
    g.a = p->x; g.w = p->w; g.M = int(M); g.N = Og; g.K = int(K);
    g.wsum = p->wsum; g.a_zp = p->a_zp; g.a_zp_dev = nullptr;
    g.a_scale = p->a_scale; g.a_scale_per_row = 0; g.w_scale = p->w_scale;
    g.bias = p->bias; g.bias_dtype = p->bias_dtype; g.relu = p->relu; g.out_mode = p->out_mode;
    g.out_scale = p->out_scale; g.out_zp = p->out_zp;
    g.out_qmin = p->out_qmin; g.out_qmax = p->out_qmax; g.out_offset = p->out_offset;
    g.out = p->out; g.ldo = p->Cout;
    g.cx = p->x; g.cH = p->H; g.cW = p->W; g.cCin = p->Cin; g.cOH = OH; g.cOW = OW; g.cKW = p->KW;
    g.cCg = Cg; g.csh = p->stride_h; g.csw = p->stride_w; g.cph = p->pad_h_lo; g.cpw = p->pad_w_lo;
    g.cdh = p->dil_h; g.cdw = p->dil_w;
    const int jrc = set_join(g, p->join, p->out_mode, p->Cout, "qconv2d_i8");
    if (jrc) return jrc;

    LQ_REQUIRE(p->w_zp == nullptr || p->out_mode != OUT_ACC_I32, LQ_ERR_VALUE,
               "qconv2d_i8: mode ACC_I32 returns the raw sums a * w; weight zero points cannot be applied to it");
    LQ_REQUIRE(p->w_zp == nullptr || p->force_path != 6, LQ_ERR_VALUE,
               "qconv2d_i8: affine filters take the NHWC image (the window sums are gathered from it), not the packed one");
    if (p->w_zp) {
        // affine filters: the raw accumulators, then the window sums of the image as a
        // convolution with one all-ones filter per group (taps in the padding read the
        // code a_zp, as in the main pass), then the corrections and the epilogue proper
        LQ_REQUIRE(p->wsum, LQ_ERR_VALUE, "qconv2d_i8: affine filters need the filter sums");
        LQ_REQUIRE(K <= 33025, LQ_ERR_SHAPE,
                   "qconv2d_i8: K = %ld overflows the int32 accumulator with affine filters", K);
        const size_t acc_bytes = (M * p->Cout * 4 + 255) / 256 * 256;
        const size_t sum_bytes = (M * p->groups * 4 + 255) / 256 * 256;
        const size_t ones_bytes = size_t(p->groups) * K;
        void* tmp = nullptr;
        bool fresh = false;
        int rc = stream_buffer(3, acc_bytes + sum_bytes + ones_bytes, 0, st, &tmp, &fresh);
        if (rc) return rc;
        int32_t* acc = static_cast<int32_t*>(tmp);
        int32_t* asum = reinterpret_cast<int32_t*>(static_cast<char*>(tmp) + acc_bytes);
        int8_t* ones = static_cast<int8_t*>(tmp) + acc_bytes + sum_bytes;
        rc = lq_fill_bytes(ones, 1, ones_bytes, stream);
        if (rc) return rc;
        lq_qconv2d_args raw = *p;
        raw.w_zp = nullptr; raw.out_mode = OUT_ACC_I32; raw.out = acc; raw.join = lq_join_args{};
        raw.bias = nullptr; raw.relu = 0;
        rc = lq_qconv2d_i8(&raw, stream);
        if (rc) return rc;
        lq_qconv2d_args win = raw;
        win.w = ones; win.Cout = p->groups; win.out = asum; win.tile_config = 0;
        rc = lq_qconv2d_i8(&win, stream);
        if (rc) return rc;
        g.N = p->Cout;
        return launch_affine_fixup(g, acc, asum, p->groups, Og, p->w_zp, int(K), st);
    }

    const bool is_gemm = p->KH == 1 && p->KW == 1 && p->stride_h == 1 && p->stride_w == 1 &&
                         p->pad_h_lo == 0 && p->pad_h_hi == 0 && p->pad_w_lo == 0 &&
                         p->pad_w_hi == 0 && p->groups == 1;
    const bool aligned = aligned16(p->x) && aligned16(p->w);
    int path = p->force_path;  // 0 = choose, 1 = gemm, 2 = implicit, 3 = im2col, 4 = naive, 5 = packed 4-channel,
                               // 6 = packed 4-channel with x and w already packed
    const bool few_channels = p->Cin <= 4 && p->groups == 1 && p->dil_w == 1 && p->KH * ((p->KW + 3) / 4) * 16 <= 131071;
    if (path == 0) {
        if (is_gemm && p->Cin % 16 == 0 && aligned)
            path = 1;
        else if (Cg % 16 == 0 && aligned)
            path = 2;
        else if (few_channels)
            path = 5;
        else
            path = 3;
    }
    if (path == 5 || path == 6) {
        LQ_REQUIRE(few_channels, LQ_ERR_VALUE,
                   "qconv2d_i8: the packed route needs Cin <= 4, groups == 1 and dilation_w == 1");
        int KWp, Hp, Wp;
        packed4_geometry(p, OW, &KWp, &Hp, &Wp);
        LQ_REQUIRE(size_t(p->B) * Hp * Wp * 4 < 0xffffffffull, LQ_ERR_SHAPE, "qconv2d_i8: padded image too large");
        const int8_t* img = p->x;
        const int8_t* flt = p->w;
        if (path == 5) {
            const size_t img_bytes = (size_t(p->B) * Hp * Wp * 4 + 255) / 256 * 256;
            const size_t flt_bytes = (size_t(p->Cout) * p->KH * KWp * 4 + 255) / 256 * 256;
            void* ws = nullptr;
            int rc = workspace(img_bytes + flt_bytes, st, &ws);
            if (rc) return rc;
            int8_t* wimg = static_cast<int8_t*>(ws);
            int8_t* wflt = wimg + img_bytes;
            hipLaunchKernelGGL(pack4_padded_kernel, dim3(grid_1d(size_t(p->B) * Hp * Wp)), dim3(256), 0, st, p->x, p->B,
                               p->H, p->W, p->Cin, p->pad_h_lo, p->pad_w_lo, Hp, Wp, p->a_zp,
                               reinterpret_cast<uint32_t*>(wimg));
            LQ_CHECK_LAUNCH("pack4_padded");
            hipLaunchKernelGGL(pack4_filter_kernel, dim3(grid_1d(size_t(p->Cout) * p->KH * KWp * 4)), dim3(256), 0, st,
                               p->w, p->Cout, p->KH, p->KW, p->Cin, KWp, wflt);
            LQ_CHECK_LAUNCH("pack4_filter");
            img = wimg, flt = wflt;
        } else {
            // x: [B, Hp, Wp, 4] from lq_quantize_nchw_to_packed4, w: [Cout, KH, KWp, 4] from lq_pack4_filter_i8
            LQ_REQUIRE(aligned16(img) && aligned16(flt), LQ_ERR_VALUE, "qconv2d_i8: packed tensors must be 16-byte aligned");
        }
        GemmArgs gg = g;
        gg.w = flt; gg.K = p->KH * KWp * 4; gg.N = p->Cout;
        gg.cx = img; gg.cH = Hp; gg.cW = Wp; gg.cCin = 4; gg.cCg = 16; gg.cKW = KWp / 4;
        gg.cph = 0; gg.cpw = 0; gg.cdw = 4;  // a tap of the gather = four real pixels
        return run_tile_kernel(gg, 1, 1, p->tile_config, st);
    }
    if (path == 1) {
        LQ_REQUIRE(is_gemm, LQ_ERR_VALUE, "qconv2d_i8: the gemm route needs a 1x1 stride-1 unpadded conv");
        g.N = p->Cout;
        return run_gemm(g, 0, p->tile_config, st);
    }
    if (path == 2) {
        LQ_REQUIRE(Cg % 16 == 0 && aligned, LQ_ERR_VALUE,
                   "qconv2d_i8: the implicit route needs Cin/groups %% 16 == 0 and aligned tensors");
        return run_tile_kernel(g, 1, p->groups, p->tile_config, st);
    }
    if (path == 4) {
        ConvShape c{p->B, p->H, p->W, p->Cin, p->Cout, p->KH, p->KW, OH, OW, p->stride_h,
                    p->stride_w, p->pad_h_lo, p->pad_w_lo, p->dil_h, p->dil_w, p->groups};
        g.N = p->Cout;
        hipLaunchKernelGGL(qconv_naive_kernel, dim3(grid_1d(M * p->Cout)), dim3(256), 0, st, g, c, p->x,
                           p->w);
        LQ_CHECK_LAUNCH("qconv_naive");
        return LQ_OK;
    }
    LQ_REQUIRE(path == 3, LQ_ERR_VALUE, "qconv2d_i8: unknown force_path %d", path);
    // explicit im2col, one group at a time
    const int Kp = int((K + 15) / 16 * 16);
    const size_t cols_bytes = (M * Kp + 255) / 256 * 256;
    const size_t w_bytes = (size_t(Og) * Kp + 255) / 256 * 256;
    void* ws = nullptr;
    int rc = workspace(cols_bytes + w_bytes, st, &ws);
    if (rc) return rc;
    int8_t* cols = static_cast<int8_t*>(ws);
    int8_t* wpad = cols + cols_bytes;
    ConvShape c{p->B, p->H, p->W, p->Cin, p->Cout, p->KH, p->KW, OH, OW, p->stride_h, p->stride_w,
                p->pad_h_lo, p->pad_w_lo, p->dil_h, p->dil_w, p->groups};
    for (int grp = 0; grp < p->groups; ++grp) {
        hipLaunchKernelGGL(im2col_i8_kernel, dim3(grid_1d(M * Kp)), dim3(256), 0, st, p->x, cols, c, grp,
                           int(K), Kp, int8_t(p->a_zp));
        LQ_CHECK_LAUNCH("im2col_i8");
        hipLaunchKernelGGL(pad_rows_kernel, dim3(grid_1d(size_t(Og) * Kp)), dim3(256), 0, st,
                           p->w + size_t(grp) * Og * K, wpad, Og, int(K), Kp);
        LQ_CHECK_LAUNCH("pad_rows");
        GemmArgs gg = g;
        gg.a = cols; gg.w = wpad; gg.K = Kp; gg.N = Og;
        const size_t col0 = size_t(grp) * Og;
        gg.wsum = g.wsum ? g.wsum + col0 : nullptr;
        gg.w_scale = g.w_scale ? g.w_scale + col0 : nullptr;
        if (g.bias)
            gg.bias = static_cast<const char*>(g.bias) + col0 * (g.bias_dtype == LQ_F16 ? 2 : 4);
        const size_t esz = g.out_mode == OUT_F16 ? 2 : (g.out_mode == OUT_REQUANT_I8 ? 1 : 4);
        gg.out = static_cast<char*>(g.out) + col0 * esz;
        if (g.join_q) gg.join_q = g.join_q + col0;
        rc = run_gemm(gg, 0, p->tile_config, st);
        if (rc) return rc;
    }
    return LQ_OK;
}

int lq_qconv3d_i8(const lq_qconv3d_args* p, lq_stream stream) {
    LQ_REQUIRE(p, LQ_ERR_VALUE, "qconv3d_i8: args is NULL");
    LQ_REQUIRE(p->B >= 0 && p->D > 0 && p->H > 0 && p->W > 0 && p->Cin > 0 && p->Cout > 0 && p->KD > 0 &&
                   p->KH > 0 && p->KW > 0,
               LQ_ERR_SHAPE, "qconv3d_i8: non-positive extent");
    LQ_REQUIRE(p->groups >= 1 && p->Cin % p->groups == 0 && p->Cout % p->groups == 0, LQ_ERR_SHAPE,
               "qconv3d_i8: channels (%d -> %d) not divisible by groups %d", p->Cin, p->Cout, p->groups);
    int out3[3];
    const int in3[3] = {p->D, p->H, p->W}, k3[3] = {p->KD, p->KH, p->KW};
    for (int i = 0; i < 3; ++i) {
        LQ_REQUIRE(p->stride[i] >= 1 && p->dilation[i] >= 1 && p->pad_lo[i] >= 0 && p->pad_hi[i] >= 0, LQ_ERR_VALUE,
                   "qconv3d_i8: bad stride / dilation / padding");
        // output extent, lucid/_C/nn/ConvNd.cpp:56-59
        out3[i] = (in3[i] + p->pad_lo[i] + p->pad_hi[i] - p->dilation[i] * (k3[i] - 1) - 1) / p->stride[i] + 1;
        LQ_REQUIRE(out3[i] > 0, LQ_ERR_SHAPE, "qconv3d_i8: empty output");
    }
    if (p->B == 0) return LQ_OK;
    LQ_REQUIRE(p->x && p->w && p->out, LQ_ERR_VALUE, "qconv3d_i8: NULL tensor pointer");
    LQ_REQUIRE(p->out_mode >= OUT_ACC_I32 && p->out_mode <= OUT_FAKEQUANT_F32, LQ_ERR_VALUE,
               "qconv3d_i8: unknown out_mode %d", p->out_mode);
    LQ_REQUIRE(p->a_zp >= -128 && p->a_zp <= 127, LQ_ERR_VALUE,
               "qconv3d_i8: activation zero point %d is not an int8 code", p->a_zp);
    const int Cg = p->Cin / p->groups, Og = p->Cout / p->groups;
    const long K = long(p->KD) * p->KH * p->KW * Cg;
    LQ_REQUIRE(K <= 131071, LQ_ERR_SHAPE, "qconv3d_i8: K = %ld overflows the int32 accumulator", K);
    const size_t M = size_t(p->B) * out3[0] * out3[1] * out3[2];
    LQ_REQUIRE(M <= 0x7fffffffull && size_t(p->B) * p->D * p->H * p->W * p->Cin < 0x7fffffffull, LQ_ERR_SHAPE,
               "qconv3d_i8: tensor too large for 32-bit indexing");
    // the gather keeps a voxel's (h, w) origin in 16 bits each
    LQ_REQUIRE(p->H + p->pad_lo[1] + p->pad_hi[1] < 32768 && p->W + p->pad_lo[2] + p->pad_hi[2] < 32768, LQ_ERR_SHAPE,
               "qconv3d_i8: a padded plane of 32768 or more rows / columns");
    LQ_REQUIRE(Cg % 16 == 0 && aligned16(p->x) && aligned16(p->w), LQ_ERR_NOT_IMPLEMENTED,
               "qconv3d_i8: the gather needs Cin/groups %% 16 == 0 (got %d) and 16-byte aligned tensors; use "
               "lq_im2col_ndhwc_i8 + lq_qlinear_i8",
               Cg);
    if (p->out_mode != OUT_ACC_I32) {
        LQ_REQUIRE(p->w_scale && p->a_scale, LQ_ERR_VALUE, "qconv3d_i8: scale pointer is NULL");
        LQ_REQUIRE(p->a_zp == 0 || p->wsum, LQ_ERR_VALUE,
                   "qconv3d_i8: a non-zero activation zero point needs the filter sums");
        LQ_REQUIRE(p->bias == nullptr || p->bias_dtype == LQ_F32 || p->bias_dtype == LQ_F16, LQ_ERR_DTYPE,
                   "qconv3d_i8: bias must be float32 or float16");
    }
    if (p->out_mode == OUT_REQUANT_I8 || p->out_mode == OUT_FAKEQUANT_F32) {
        LQ_REQUIRE(p->out_scale && p->out_zp, LQ_ERR_VALUE, "qconv3d_i8: output qparams are NULL");
        if (p->out_mode == OUT_REQUANT_I8)
            LQ_REQUIRE(p->out_qmin + p->out_offset >= -128 && p->out_qmax + p->out_offset <= 127, LQ_ERR_VALUE,
                       "qconv3d_i8: output grid + offset does not fit int8");
    }
    hipStream_t st = as_stream(stream);
    GemmArgs g{};
    g.a = p->x; g.w = p->w; g.M = int(M); g.N = Og; g.K = int(K);
    g.wsum = p->wsum; g.a_zp = p->a_zp; g.a_zp_dev = nullptr;
    g.a_scale = p->a_scale; g.a_scale_per_row = 0; g.w_scale = p->w_scale;
    g.bias = p->bias; g.bias_dtype = p->bias_dtype; g.relu = p->relu; g.out_mode = p->out_mode;
    g.out_scale = p->out_scale; g.out_zp = p->out_zp;
    g.out_qmin = p->out_qmin; g.out_qmax = p->out_qmax; g.out_offset = p->out_offset;
    g.out = p->out; g.ldo = p->Cout;
    g.cx = p->x; g.cD = p->D; g.cH = p->H; g.cW = p->W; g.cCin = p->Cin; g.cCg = Cg;
    g.cOD = out3[0]; g.cOH = out3[1]; g.cOW = out3[2]; g.cKH = p->KH; g.cKW = p->KW;
    g.csd = p->stride[0]; g.csh = p->stride[1]; g.csw = p->stride[2];
    g.cpd = p->pad_lo[0]; g.cph = p->pad_lo[1]; g.cpw = p->pad_lo[2];
    g.cdd = p->dilation[0]; g.cdh = p->dilation[1]; g.cdw = p->dilation[2];

    LQ_REQUIRE(p->w_zp == nullptr || p->out_mode != OUT_ACC_I32, LQ_ERR_VALUE,
               "qconv3d_i8: mode ACC_I32 returns the raw sums a * w; weight zero points cannot be applied to it");
    if (p->w_zp) {
        // affine filters, as in lq_qconv2d_i8: raw accumulators, the window sums of the volume
        // from one all-ones filter per group, then the corrections and the epilogue proper
        LQ_REQUIRE(p->wsum, LQ_ERR_VALUE, "qconv3d_i8: affine filters need the filter sums");
        LQ_REQUIRE(K <= 33025, LQ_ERR_SHAPE, "qconv3d_i8: K = %ld overflows the int32 accumulator with affine filters",
                   K);
        const size_t acc_bytes = (M * p->Cout * 4 + 255) / 256 * 256;
        const size_t sum_bytes = (M * p->groups * 4 + 255) / 256 * 256;
        const size_t ones_bytes = size_t(p->groups) * K;
        void* tmp = nullptr;
        bool fresh = false;
        int rc = stream_buffer(3, acc_bytes + sum_bytes + ones_bytes, 0, st, &tmp, &fresh);
        if (rc) return rc;
        int32_t* acc = static_cast<int32_t*>(tmp);
        int32_t* asum = reinterpret_cast<int32_t*>(static_cast<char*>(tmp) + acc_bytes);
        int8_t* ones = static_cast<int8_t*>(tmp) + acc_bytes + sum_bytes;
        rc = lq_fill_bytes(ones, 1, ones_bytes, stream);
        if (rc) return rc;
        lq_qconv3d_args raw = *p;
        raw.w_zp = nullptr; raw.out_mode = OUT_ACC_I32; raw.out = acc; raw.bias = nullptr; raw.relu = 0;
        rc = lq_qconv3d_i8(&raw, stream);
        if (rc) return rc;
        lq_qconv3d_args win = raw;
        win.w = ones; win.Cout = p->groups; win.out = asum; win.tile_config = 0;
        rc = lq_qconv3d_i8(&win, stream);
        if (rc) return rc;
        g.N = p->Cout;
        return launch_affine_fixup(g, acc, asum, p->groups, Og, p->w_zp, int(K), st);
    }
    return run_tile_kernel(g, 2, p->groups, p->tile_config, st);
}

int lq_quantize_nchw_to_nhwc(const float* x, int8_t* q, int code_offset, int B, int C, int H, int W,
                             const float* scale, const float* zp, int qmin, int qmax,
                             lq_stream stream) {
    if (size_t(B) * C * H * W == 0) return LQ_OK;
    LQ_REQUIRE(x && q && scale && zp, LQ_ERR_VALUE, "quantize_nchw_to_nhwc: NULL pointer");
    LQ_REQUIRE(qmin <= qmax && qmin + code_offset >= -128 && qmax + code_offset <= 127, LQ_ERR_VALUE,
               "quantize_nchw_to_nhwc: grid [%d,%d] + offset %d does not fit int8", qmin, qmax,
               code_offset);
    LQ_REQUIRE(B <= 65535 && (C + 31) / 32 <= 65535, LQ_ERR_SHAPE, "quantize_nchw_to_nhwc: too large");
    const int HW = H * W;
    if (C <= 4) {
        const unsigned gx = unsigned((HW + 255) / 256 < 1024 ? (HW + 255) / 256 : 1024);
        hipLaunchKernelGGL(quantize_nchw_to_nhwc_small_c_kernel, dim3(gx, B), dim3(256), 0, as_stream(stream), x, q, C,
                           size_t(HW), scale, zp, float(qmin), float(qmax), code_offset);
        LQ_CHECK_LAUNCH("quantize_nchw_to_nhwc");
        return LQ_OK;
    }
    hipLaunchKernelGGL(quantize_nchw_to_nhwc_kernel, dim3((HW + 31) / 32, (C + 31) / 32, B), dim3(256), 0,
                       as_stream(stream), x, q, B, C, HW, scale, zp, float(qmin), float(qmax),
                       code_offset);
    LQ_CHECK_LAUNCH("quantize_nchw_to_nhwc");
    return LQ_OK;
}

int lq_qconv2d_packed4_geometry(const lq_qconv2d_args* p, int* Hp, int* Wp, int* KWp) {
    LQ_REQUIRE(p && Hp && Wp && KWp, LQ_ERR_VALUE, "qconv2d_packed4_geometry: NULL pointer");
    LQ_REQUIRE(p->H > 0 && p->W > 0 && p->KW > 0 && p->stride_w >= 1 && p->dil_w == 1 && p->Cin >= 1 && p->Cin <= 4 &&
                   p->groups == 1 && p->pad_h_lo >= 0 && p->pad_h_hi >= 0 && p->pad_w_lo >= 0 && p->pad_w_hi >= 0,
               LQ_ERR_VALUE, "qconv2d_packed4_geometry: the packed route needs Cin <= 4, groups == 1 and dilation_w == 1");
    const int OW = (p->W + p->pad_w_lo + p->pad_w_hi - (p->KW - 1) - 1) / p->stride_w + 1;
    LQ_REQUIRE(OW > 0, LQ_ERR_SHAPE, "qconv2d_packed4_geometry: empty output");
    packed4_geometry(p, OW, KWp, Hp, Wp);
    return LQ_OK;
}

int lq_quantize_nchw_to_packed4(const float* x, int8_t* out, int code_offset, int B, int C, int H, int W,
                                int pad_h_lo, int pad_w_lo, int Hp, int Wp, const float* scale, const float* zp,
                                int qmin, int qmax, int fill_code, lq_stream stream) {
    if (size_t(B) * Hp * Wp == 0) return LQ_OK;
    LQ_REQUIRE(x && out && scale && zp, LQ_ERR_VALUE, "quantize_nchw_to_packed4: NULL pointer");
    LQ_REQUIRE(C >= 1 && C <= 4 && H > 0 && W > 0 && pad_h_lo >= 0 && pad_w_lo >= 0 && Hp >= H + pad_h_lo &&
                   Wp >= W + pad_w_lo && Wp % 4 == 0,
               LQ_ERR_SHAPE, "quantize_nchw_to_packed4: the packed image [%d, %d] does not hold %d x %d at (%d, %d)", Hp,
               Wp, H, W, pad_h_lo, pad_w_lo);
    LQ_REQUIRE(qmin <= qmax && qmin + code_offset >= -128 && qmax + code_offset <= 127 && fill_code >= -128 &&
                   fill_code <= 127,
               LQ_ERR_VALUE, "quantize_nchw_to_packed4: grid [%d,%d] + offset %d does not fit int8", qmin, qmax,
               code_offset);
    LQ_REQUIRE(aligned16(out), LQ_ERR_VALUE, "quantize_nchw_to_packed4: out must be 16-byte aligned");
    LQ_REQUIRE(Wp % 4 == 0 && B <= 65535 && (Hp + 3) / 4 <= 65535, LQ_ERR_SHAPE,
               "quantize_nchw_to_packed4: packed rows must be a multiple of 4 pixels (Wp = %d); at most 65535 images", Wp);
    hipLaunchKernelGGL(quantize_nchw_to_packed4_kernel, dim3(unsigned((Wp / 4 + 63) / 64), unsigned((Hp + 3) / 4), unsigned(B)),
                       dim3(256), 0, as_stream(stream), x, B, C, H, W, pad_h_lo, pad_w_lo, Hp, Wp, scale, zp, float(qmin),
                       float(qmax), code_offset, fill_code, reinterpret_cast<uint4*>(out));
    LQ_CHECK_LAUNCH("quantize_nchw_to_packed4");
    return LQ_OK;
}

int lq_pack4_filter_i8(const int8_t* w, int8_t* out, int Cout, int KH, int KW, int Cin, lq_stream stream) {
    if (size_t(Cout) * KH * KW == 0) return LQ_OK;
    LQ_REQUIRE(w && out, LQ_ERR_VALUE, "pack4_filter_i8: NULL pointer");
    LQ_REQUIRE(Cin >= 1 && Cin <= 4 && Cout > 0 && KH > 0 && KW > 0, LQ_ERR_SHAPE, "pack4_filter_i8: bad shape");
    const int KWp = (KW + 3) / 4 * 4;
    hipLaunchKernelGGL(pack4_filter_kernel, dim3(grid_1d(size_t(Cout) * KH * KWp * 4)), dim3(256), 0,
                       as_stream(stream), w, Cout, KH, KW, Cin, KWp, out);
    LQ_CHECK_LAUNCH("pack4_filter");
    return LQ_OK;
}

int lq_dequantize_nhwc_to_nchw(const int8_t* q, int code_offset, float* out, int B, int C, int H,
                               int W, const float* scale, const float* zp, lq_stream stream) {
    if (size_t(B) * C * H * W == 0) return LQ_OK;
    LQ_REQUIRE(q && out && scale && zp, LQ_ERR_VALUE, "dequantize_nhwc_to_nchw: NULL pointer");
    LQ_REQUIRE(B <= 65535 && (C + 31) / 32 <= 65535, LQ_ERR_SHAPE, "dequantize_nhwc_to_nchw: too large");
    const int HW = H * W;
    hipLaunchKernelGGL(dequantize_nhwc_to_nchw_kernel, dim3((HW + 31) / 32, (C + 31) / 32, B), dim3(256),
                       0, as_stream(stream), q, code_offset, out, B, C, HW, scale, zp);
    LQ_CHECK_LAUNCH("dequantize_nhwc_to_nchw");
    return LQ_OK;
}

int lq_repack_oihw_to_ohwi_i8(const int8_t* w, int8_t* out, int O, int I, int KH, int KW,
                              lq_stream stream) {
    const size_t total = size_t(O) * I * KH * KW;
    if (total == 0) return LQ_OK;
    LQ_REQUIRE(w && out, LQ_ERR_VALUE, "repack_oihw_to_ohwi_i8: NULL pointer");
    hipLaunchKernelGGL(repack_oihw_to_ohwi_kernel, dim3(grid_1d(total)), dim3(256), 0, as_stream(stream),
                       w, out, O, I, KH, KW);
    LQ_CHECK_LAUNCH("repack_oihw_to_ohwi");
    return LQ_OK;
}

int lq_im2col_ndhwc_i8(const int8_t* x, int8_t* cols, int B, int D, int H, int W, int C, int c0, int Cg,
                       const int* kernel, const int* stride, const int* pad_lo, const int* dilation,
                       const int* insert, const int* out_size, int pad_code, lq_stream stream) {
    LQ_REQUIRE(kernel && stride && pad_lo && dilation && insert && out_size, LQ_ERR_VALUE,
               "im2col_ndhwc: NULL geometry");
    LQ_REQUIRE(B >= 0 && C > 0 && D > 0 && H > 0 && W > 0, LQ_ERR_SHAPE, "im2col_ndhwc: bad input shape");
    LQ_REQUIRE(c0 >= 0 && Cg > 0 && c0 + Cg <= C, LQ_ERR_SHAPE, "im2col_ndhwc: channels [%d, %d) of %d", c0,
               c0 + Cg, C);
    LQ_REQUIRE(pad_code >= -128 && pad_code <= 127, LQ_ERR_VALUE, "im2col_ndhwc: padding code %d is no int8", pad_code);
    // any tap outside the spread input reads the padding code, so out_size needs no upper bound:
    // high-side padding, e.g. a transposed convolution's output_padding, is simply more outputs
    for (int i = 0; i < 3; ++i)
        LQ_REQUIRE(kernel[i] > 0 && stride[i] > 0 && dilation[i] > 0 && insert[i] > 0 && pad_lo[i] >= 0 &&
                       out_size[i] >= 0,
                   LQ_ERR_VALUE, "im2col_ndhwc: bad geometry in dimension %d", i);
    const size_t M = size_t(B) * out_size[0] * out_size[1] * out_size[2];
    const size_t total = M * kernel[0] * kernel[1] * kernel[2] * Cg;
    if (total == 0) return LQ_OK;
    LQ_REQUIRE(x && cols, LQ_ERR_VALUE, "im2col_ndhwc: NULL pointer");
    const bool vec = C % 16 == 0 && Cg % 16 == 0 && c0 % 16 == 0 && aligned16(x) && aligned16(cols);
    const Vol3 in{D, H, W}, kn{kernel[0], kernel[1], kernel[2]}, st{stride[0], stride[1], stride[2]},
        pd{pad_lo[0], pad_lo[1], pad_lo[2]}, dl{dilation[0], dilation[1], dilation[2]},
        is{insert[0], insert[1], insert[2]}, ot{out_size[0], out_size[1], out_size[2]};
    if (vec)
        hipLaunchKernelGGL(im2col_ndhwc_i8_kernel<16>, dim3(grid_1d(total / 16)), dim3(256), 0, as_stream(stream), x,
                           cols, C, in, c0, Cg, kn, st, pd, dl, is, ot, pad_code, total / 16);
    else
        hipLaunchKernelGGL(im2col_ndhwc_i8_kernel<1>, dim3(grid_1d(total)), dim3(256), 0, as_stream(stream), x, cols,
                           C, in, c0, Cg, kn, st, pd, dl, is, ot, pad_code, total);
    LQ_CHECK_LAUNCH("im2col_ndhwc");
    return LQ_OK;
}

int lq_transpose_i8(const int8_t* src, int8_t* dst, int batches, size_t R, size_t Cn, size_t src_stride,
                    size_t dst_stride, lq_stream stream) {
    LQ_REQUIRE(batches >= 0 && batches < 65536, LQ_ERR_SHAPE, "transpose_i8: %d batches (at most 65535)", batches);
    if (batches == 0 || R == 0 || Cn == 0) return LQ_OK;
    LQ_REQUIRE(src && dst, LQ_ERR_VALUE, "transpose_i8: NULL pointer");
    LQ_REQUIRE(src_stride >= R * Cn && dst_stride >= R * Cn, LQ_ERR_SHAPE,
               "transpose_i8: batch stride smaller than a %zu x %zu matrix", R, Cn);
    const size_t tiles_r = (R + 63) / 64, tiles_c = (Cn + 63) / 64;
    LQ_REQUIRE(tiles_r * tiles_c < 0x7fffffffull && tiles_c < 0x7fffffffull, LQ_ERR_SHAPE,
               "transpose_i8: matrix too large");
    hipLaunchKernelGGL(transpose_i8_kernel, dim3(unsigned(tiles_r * tiles_c), unsigned(batches)), dim3(256), 0,
                       as_stream(stream), src, dst, R, Cn, src_stride, dst_stride, unsigned(tiles_c));
    LQ_CHECK_LAUNCH("transpose_i8");
    return LQ_OK;
}

int lq_pad_nhwc_i8(const int8_t* x, int8_t* out, int B, int H, int W, int C, int pad_top, int pad_bottom,
                   int pad_left, int pad_right, int mode, lq_stream stream) {
    LQ_REQUIRE(x && out, LQ_ERR_VALUE, "pad: NULL pointer");
    LQ_REQUIRE(B >= 0 && H > 0 && W > 0 && C > 0, LQ_ERR_SHAPE, "pad: bad shape");
    LQ_REQUIRE(pad_top >= 0 && pad_bottom >= 0 && pad_left >= 0 && pad_right >= 0, LQ_ERR_VALUE,
               "pad: negative padding");
    LQ_REQUIRE(mode >= 1 && mode <= 3, LQ_ERR_VALUE, "pad: mode must be 1 (reflect), 2 (replicate) or 3 (circular)");
    if (mode == 1)  // F.pad's rule for reflect: the pad must be smaller than the dimension
        LQ_REQUIRE(pad_top < H && pad_bottom < H && pad_left < W && pad_right < W, LQ_ERR_VALUE,
                   "pad: reflect padding must be smaller than the image");
    if (mode == 3)
        LQ_REQUIRE(pad_top <= H && pad_bottom <= H && pad_left <= W && pad_right <= W, LQ_ERR_VALUE,
                   "pad: circular padding must not exceed the image");
    const int OH = H + pad_top + pad_bottom, OW = W + pad_left + pad_right;
    const int vec = (C % 16 == 0) && aligned16(x) && aligned16(out);
    const size_t total = size_t(B) * OH * OW * (vec ? C / 16 : C);
    if (total == 0) return LQ_OK;
    LQ_REQUIRE((total + 255) / 256 < 0x7fffffffull, LQ_ERR_SHAPE, "pad: tensor too large");
    hipLaunchKernelGGL(pad_nhwc_i8_kernel, dim3(unsigned((total + 255) / 256)), dim3(256), 0, as_stream(stream), x,
                       out, B, H, W, C, pad_top, pad_left, OH, OW, mode, vec);
    LQ_CHECK_LAUNCH("pad_nhwc_i8");
    return LQ_OK;
}

int lq_pad_planes_f32(const float* x, float* out, size_t planes, int H, int W, int pad_top, int pad_bottom,
                      int pad_left, int pad_right, int mode, lq_stream stream) {
    LQ_REQUIRE(mode >= 0 && mode <= 3, LQ_ERR_VALUE, "pad_planes_f32: mode %d (0 zeros, 1 reflect, 2 replicate, 3 circular)", mode);
    LQ_REQUIRE(H > 0 && W > 0 && pad_top >= 0 && pad_bottom >= 0 && pad_left >= 0 && pad_right >= 0, LQ_ERR_VALUE,
               "pad_planes_f32: bad extents");
    if (mode == 1)
        LQ_REQUIRE(pad_top < H && pad_bottom < H && pad_left < W && pad_right < W, LQ_ERR_VALUE,
                   "pad_planes_f32: reflect padding must be smaller than the image");
    if (mode == 3)
        LQ_REQUIRE(pad_top <= H && pad_bottom <= H && pad_left <= W && pad_right <= W, LQ_ERR_VALUE,
                   "pad_planes_f32: circular padding must not exceed the image");
    const int OH = H + pad_top + pad_bottom, OW = W + pad_left + pad_right;
    const size_t total = planes * OH * OW;
    if (total == 0) return LQ_OK;
    LQ_REQUIRE(x && out, LQ_ERR_VALUE, "pad_planes_f32: NULL pointer");
    LQ_REQUIRE((total + 255) / 256 < 0x7fffffffull, LQ_ERR_SHAPE, "pad_planes_f32: tensor too large");
    hipLaunchKernelGGL(pad_planes_f32_kernel, dim3(unsigned((total + 255) / 256)), dim3(256), 0, as_stream(stream), x, out,
                       planes, H, W, pad_top, pad_left, OH, OW, mode);
    LQ_CHECK_LAUNCH("pad_planes_f32");
    return LQ_OK;
}

int lq_maxpool2d_nhwc_i8(const int8_t* x, int8_t* out, int B, int H, int W, int C, int KH, int KW,
                         int stride_h, int stride_w, int pad_h, int pad_w, lq_stream stream) {
    LQ_REQUIRE(KH > 0 && KW > 0 && stride_h > 0 && stride_w > 0 && pad_h >= 0 && pad_w >= 0,
               LQ_ERR_VALUE, "maxpool2d_nhwc_i8: bad window");
    LQ_REQUIRE(2 * pad_h <= KH && 2 * pad_w <= KW, LQ_ERR_VALUE,
               "maxpool2d_nhwc_i8: padding larger than half the window");
    const int OH = (H + 2 * pad_h - KH) / stride_h + 1, OW = (W + 2 * pad_w - KW) / stride_w + 1;
    LQ_REQUIRE(OH > 0 && OW > 0, LQ_ERR_SHAPE, "maxpool2d_nhwc_i8: empty output");
    const size_t total = size_t(B) * OH * OW * C;
    if (total == 0) return LQ_OK;
    LQ_REQUIRE(x && out, LQ_ERR_VALUE, "maxpool2d_nhwc_i8: NULL pointer");
    if (C % 16 == 0 && aligned16(x) && aligned16(out)) {
        if ((KH == 3 && KW == 3) || (KH == 2 && KW == 2)) {
            const dim3 grid{grid_1d(total / 16)};
            const uint4* xi = reinterpret_cast<const uint4*>(x);
            uint4* oi = reinterpret_cast<uint4*>(out);
            if (KH == 3)
                hipLaunchKernelGGL((maxpool_nhwc_i8x16_fixed_kernel<3, 3>), grid, dim3(256), 0, as_stream(stream), xi, oi,
                                   B, H, W, C / 16, stride_h, stride_w, pad_h, pad_w, OH, OW);
            else
                hipLaunchKernelGGL((maxpool_nhwc_i8x16_fixed_kernel<2, 2>), grid, dim3(256), 0, as_stream(stream), xi, oi,
                                   B, H, W, C / 16, stride_h, stride_w, pad_h, pad_w, OH, OW);
            LQ_CHECK_LAUNCH("maxpool2d_nhwc_i8");
            return LQ_OK;
        }
        hipLaunchKernelGGL(maxpool_nhwc_i8x16_kernel, dim3(grid_1d(total / 16)), dim3(256), 0, as_stream(stream),
                           reinterpret_cast<const uint4*>(x), reinterpret_cast<uint4*>(out), B, H, W, C / 16, KH, KW,
                           stride_h, stride_w, pad_h, pad_w, OH, OW);
        LQ_CHECK_LAUNCH("maxpool2d_nhwc_i8");
        return LQ_OK;
    }
    hipLaunchKernelGGL(maxpool_nhwc_i8_kernel, dim3(grid_1d(total)), dim3(256), 0, as_stream(stream), x,
                       out, B, H, W, C, KH, KW, stride_h, stride_w, pad_h, pad_w, OH, OW);
    LQ_CHECK_LAUNCH("maxpool2d_nhwc_i8");
    return LQ_OK;
}

}  // extern "C"
