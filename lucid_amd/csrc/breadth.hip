// Quantized module breadth beyond Linear / Conv2d: int8 embedding tables
// (lucid/nn/quantized/sparse.py:22-336), activations that requantize their result
// (lucid/nn/quantized/activation.py:22-486), zero insertion for transposed
// convolutions (lucid/nn/quantized/conv_transpose.py) and the gate arithmetic of the
// weight-only LSTM (lucid/nn/quantized/dynamic/rnn.py).
//
// Lucid dequantizes the whole table and then gathers float rows; here only the rows
// that are asked for are read, and decoded on the way out - the values are the same
// (float(code) - z) * s per element.
#include "common.hpp"
#include "qepilogue.hpp"

using namespace lq;

namespace {

__device__ __forceinline__ long long read_index(const void* p, int is64, size_t i) {
    return is64 ? static_cast<const long long*>(p)[i] : (long long)static_cast<const int*>(p)[i];
}

// min and max of an index tensor, one block (index tensors are small next to the
// tables they address): out[0] = min, out[1] = max.
__global__ __launch_bounds__(1024) void index_minmax_kernel(const void* idx, int is64, size_t n, long long* out) {
    __shared__ long long smin[16], smax[16];
    long long lo = 0x7fffffffffffffffll, hi = -0x7fffffffffffffffll - 1;
    for (size_t i = threadIdx.x; i < n; i += 1024) {
        const long long v = read_index(idx, is64, i);
        lo = v < lo ? v : lo;
        hi = v > hi ? v : hi;
    }
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) {
        const long long ol = __shfl_xor(lo, d, 64), oh = __shfl_xor(hi, d, 64);
        lo = ol < lo ? ol : lo;
        hi = oh > hi ? oh : hi;
    }
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    if (lane == 0) smin[wave] = lo, smax[wave] = hi;
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < 16; ++w) {
            lo = smin[w] < lo ? smin[w] : lo;
            hi = smax[w] > hi ? smax[w] : hi;
        }
        out[0] = lo;
        out[1] = hi;
    }
}

// F.embedding on the dequantized table (CpuBackend.h:8970-9010): row i of the output
// is zeros when idx[i] == padding_idx >= 0, else the decoded table row.  One block row
// of 64 lanes per output row chunk; ids outside the table give zeros (the host has
// already refused them).
__global__ __launch_bounds__(256) void embedding_i8_kernel(const int8_t* __restrict__ table,
                                                           const float* __restrict__ scale,
                                                           const float* __restrict__ zp, int num, int D,
                                                           const void* __restrict__ idx, int is64, size_t n_idx,
                                                           int padding_idx, float* __restrict__ out) {
    const size_t row = size_t(blockIdx.x) * 4 + (threadIdx.x >> 6);
    if (row >= n_idx) return;
    const int lane = threadIdx.x & 63;
    const long long id = read_index(idx, is64, row);
    float* dst = out + row * size_t(D);
    const bool zero = (padding_idx >= 0 && id == padding_idx) || id < 0 || id >= num;
    if (zero) {
        for (int d = lane; d < D; d += 64) dst[d] = 0.0f;
        return;
    }
    const int8_t* src = table + size_t(id) * D;
    const float s = scale[id], z = zp[id];
    if ((D & 3) == 0) {
        for (int d = lane * 4; d < D; d += 256) {
            const uint32_t w = *reinterpret_cast<const uint32_t*>(src + d);
            float4 o;
            o.x = (float(int(int8_t(w & 0xff))) - z) * s;
            o.y = (float(int(int8_t((w >> 8) & 0xff))) - z) * s;
            o.z = (float(int(int8_t((w >> 16) & 0xff))) - z) * s;
            o.w = (float(int(int8_t(w >> 24))) - z) * s;
            *reinterpret_cast<float4*>(dst + d) = o;
        }
    } else {
        for (int d = lane; d < D; d += 64) dst[d] = (float(int(src[d])) - z) * s;
    }
}

// F.embedding_bag on the dequantized table (CpuBackend.h:5989-6088): bag b covers the
// flat indices [offsets[b], offsets[b+1]) (the last one runs to n_idx); padding and
// out-of-table ids are skipped; sum adds rows in index order; mean divides by the
// number of rows added (if any); max starts from the lowest float and an empty bag
// gives zeros.  One wavefront per bag, lanes over the embedding dimension, so every
// output element sees its addends in the reference's order.
__global__ __launch_bounds__(256) void embedding_bag_i8_kernel(const int8_t* __restrict__ table,
                                                               const float* __restrict__ scale,
                                                               const float* __restrict__ zp, int num, int D,
                                                               const void* __restrict__ idx, int is64,
                                                               long long n_idx, const void* __restrict__ offsets,
                                                               int off64, int fixed_len, int B, int mode,
                                                               int padding_idx, float* __restrict__ out) {
    const int b = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (b >= B) return;
    const int lane = threadIdx.x & 63;
    long long start, end;
    if (offsets) {
        start = read_index(offsets, off64, b);
        end = b + 1 < B ? read_index(offsets, off64, b + 1) : n_idx;
    } else {  // 2-d indices: every row is a bag of fixed_len entries
        start = (long long)b * fixed_len;
        end = start + fixed_len;
    }
    start = start < 0 ? 0 : start;
    end = end > n_idx ? n_idx : end;
    for (int d0 = lane; d0 < D; d0 += 64) {
        float acc = mode == 2 ? -3.402823466e+38f : 0.0f;
        int count = 0;
        for (long long k = start; k < end; ++k) {
            const long long id = read_index(idx, is64, size_t(k));
            if (id == padding_idx || id < 0 || id >= num) continue;
            const float v = (float(int(table[size_t(id) * D + d0])) - zp[id]) * scale[id];
            if (mode == 2)
                acc = v > acc ? v : acc;
            else
                acc = acc + v;
            ++count;
        }
        if (mode == 2 && count == 0) acc = 0.0f;
        if (mode == 1 && count > 0) acc = acc / float(count);
        out[size_t(b) * D + d0] = acc;
    }
}

// ---------------------------------------------------------------- activations
// The float32 formulas of the CPU engine: leaky_relu CpuBackend.h:1722-1723,
// elu :1783-1785, hard_sigmoid :2001-2002, hard_swish :2064-2065 (min / max written
// as the comparisons std::min / std::max make, so a NaN passes), sigmoid :1049-1060
// (1 / (1 + exp(-x))), tanh.
__device__ __forceinline__ float act_apply(int kind, float x, float alpha) {
    switch (kind) {
    case 0: return 1.0f / (1.0f + expf(-x));
    case 1:
    case 2: {
        float t = (x + 3.0f) / 6.0f;
        t = (t < 0.0f) ? 0.0f : t;
        t = (1.0f < t) ? 1.0f : t;
        return kind == 1 ? x * t : t;
    }
    case 3: return tanhf(x);
    case 4: return x >= 0.0f ? x : alpha * (expf(x) - 1.0f);
    default: return x >= 0.0f ? x : alpha * x;
    }
}

// Activation on a float tensor, optionally fake-quantized to (S, Z) as
// _QuantizedActivation.forward does (activation.py:44-53).
__global__ __launch_bounds__(256) void act_f32_kernel(int kind, float alpha, const float* __restrict__ x,
                                                      float* __restrict__ out, size_t n, int fq, const float* S_,
                                                      const float* Z_, float lo, float hi) {
    const float S = fq ? S_[0] : 1.0f, Z = fq ? Z_[0] : 0.0f;
    const size_t stride = size_t(gridDim.x) * 256;
    for (size_t i = size_t(blockIdx.x) * 256 + threadIdx.x; i < n; i += stride) {
        float y = act_apply(kind, x[i], alpha);
        if (fq) y = (q_core(y, S, Z, lo, hi) - Z) * S;
        out[i] = y;
    }
}

// The same on codes: an input on a per-tensor grid takes at most 256 values, so every
// block first tabulates requantize(act(dequantize(code))) for the 256 stored codes in
// LDS and then maps 16 codes per lane through the table.  The result is what the float
// formulation gives element by element.
__global__ __launch_bounds__(256) void act_requant_i8_kernel(int kind, float alpha, const int8_t* __restrict__ q,
                                                             int in_off, const float* s_, const float* z_,
                                                             size_t n, const float* S_, const float* Z_, float lo,
                                                             float hi, int out_off, int8_t* __restrict__ out) {
    __shared__ int8_t lut[256];
    {
        const int stored = int(threadIdx.x) - 128;
        const float x = (float(stored - in_off) - z_[0]) * s_[0];
        const float qv = q_core(act_apply(kind, x, alpha), S_[0], Z_[0], lo, hi);
        lut[threadIdx.x] = int8_t(((qv != qv) ? 0 : int(qv)) + out_off);
    }
    __syncthreads();
    const size_t stride = size_t(gridDim.x) * 256 * 16;
    const bool vec = aligned16(q) && aligned16(out);
    for (size_t i = (size_t(blockIdx.x) * 256 + threadIdx.x) * 16; i < n; i += stride) {
        if (vec && i + 16 <= n) {
            const uint4 v = *reinterpret_cast<const uint4*>(q + i);
            const uint32_t in[4] = {v.x, v.y, v.z, v.w};
            uint32_t o[4];
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                o[w] = 0;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int c = int(int8_t((in[w] >> (8 * e)) & 0xff)) + 128;
                    o[w] |= uint32_t(uint8_t(lut[c])) << (8 * e);
                }
            }
            *reinterpret_cast<uint4*>(out + i) = uint4{o[0], o[1], o[2], o[3]};
        } else {
            for (size_t e = i; e < n && e < i + 16; ++e) out[e] = lut[int(q[e]) + 128];
        }
    }
}

// ---------------------------------------------------------------- transposed convolution
// Zero insertion: NHWC codes [B, H, W, C] -> [B, (H-1)*sh+1+eh, (W-1)*sw+1+ew, C] with the
// input's pixels at multiples of the stride and every other byte the code of real
// zero (`fill`, the stored zero point).  A stride-1 convolution of the result with the
// flipped kernel is the transposed convolution.
__global__ __launch_bounds__(256) void dilate_nhwc_i8_kernel(const int8_t* __restrict__ x, int B, int H, int W, int C,
                                                             int sh, int sw, int OH, int OW, int fill,
                                                             int8_t* __restrict__ out) {
    const size_t n = size_t(B) * OH * OW * C, stride = size_t(gridDim.x) * 256;
    for (size_t i = size_t(blockIdx.x) * 256 + threadIdx.x; i < n; i += stride) {
        const int c = int(i % C);
        size_t p = i / C;
        const int ow = int(p % OW);
        p /= OW;
        const int oh = int(p % OH), b = int(p / OH);
        int8_t v = int8_t(fill);
        if (oh % sh == 0 && ow % sw == 0) {
            const int h = oh / sh, w = ow / sw;
            if (h < H && w < W) v = x[((size_t(b) * H + h) * W + w) * C + c];
        }
        out[i] = v;
    }
}

// ---------------------------------------------------------------- LSTM cell
// One time step of the gates (CpuBackend.h:13456-13506; i, f, g, o in this order
// along the 4H axis): raw = x W_ih^T + h W_hh^T + (b_ih + b_hh),
// c' = sigmoid(f) * c + sigmoid(i) * tanh(g), h' = sigmoid(o) * tanh(c').
__device__ __forceinline__ float sigmoidf_(float x) { return 1.0f / (1.0f + expf(-x)); }

__global__ __launch_bounds__(256) void lstm_cell_kernel(const float* __restrict__ gx, const float* __restrict__ gh,
                                                        const float* __restrict__ bias,
                                                        const float* __restrict__ c_in, int B, int H, size_t gx_ld,
                                                        float* __restrict__ h_out, float* __restrict__ c_out,
                                                        float* __restrict__ y, size_t y_ld) {
    const size_t n = size_t(B) * H, stride = size_t(gridDim.x) * 256;
    for (size_t e = size_t(blockIdx.x) * 256 + threadIdx.x; e < n; e += stride) {
        const size_t b = e / H, j = e - b * H;
        const float* px = gx + b * gx_ld;
        const float* ph = gh + b * 4 * size_t(H);
        const size_t H2 = 2 * size_t(H), H3 = 3 * size_t(H);
        const float bi = bias ? bias[j] : 0.0f, bf = bias ? bias[H + j] : 0.0f;
        const float bg = bias ? bias[H2 + j] : 0.0f, bo = bias ? bias[H3 + j] : 0.0f;
        const float ig = sigmoidf_((px[j] + ph[j]) + bi);
        const float fg = sigmoidf_((px[H + j] + ph[H + j]) + bf);
        const float gg = tanhf((px[H2 + j] + ph[H2 + j]) + bg);
        const float og = sigmoidf_((px[H3 + j] + ph[H3 + j]) + bo);
        const float c = fg * c_in[e] + ig * gg;
        const float h = og * tanhf(c);
        c_out[e] = c;
        h_out[e] = h;
        if (y) y[b * y_ld + j] = h;
    }
}

inline unsigned grid_for(size_t n, size_t per_block) {
    size_t b = (n + per_block - 1) / per_block;
    return unsigned(b < 1 ? 1 : (b > 65536 ? 65536 : b));
}

int check_out_grid(const char* who, int qmin, int qmax, int off) {
    LQ_REQUIRE(qmin <= qmax && qmin + off >= -128 && qmax + off <= 127, LQ_ERR_VALUE,
               "%s: output grid [%d,%d] + offset %d does not fit int8", who, qmin, qmax, off);
    return LQ_OK;
}

}  // namespace

extern "C" {

int lq_index_minmax(const void* idx, int idx_is_64, size_t n, long long* out2, lq_stream stream) {
    LQ_REQUIRE(n > 0, LQ_ERR_SHAPE, "index_minmax: empty index tensor");
    LQ_REQUIRE(idx && out2, LQ_ERR_VALUE, "index_minmax: NULL pointer");
    hipLaunchKernelGGL(index_minmax_kernel, dim3(1), dim3(1024), 0, as_stream(stream), idx, idx_is_64, n, out2);
    LQ_CHECK_LAUNCH("index_minmax");
    return LQ_OK;
}

int lq_embedding_i8(const int8_t* table, const float* scale, const float* zp, int num_embeddings, int dim,
                    const void* idx, int idx_is_64, size_t n_idx, int padding_idx, float* out, lq_stream stream) {
    LQ_REQUIRE(num_embeddings >= 0 && dim >= 0, LQ_ERR_SHAPE, "embedding_i8: negative extent");
    if (n_idx == 0 || dim == 0) return LQ_OK;
    LQ_REQUIRE(table && scale && zp && idx && out, LQ_ERR_VALUE, "embedding_i8: NULL pointer");
    LQ_REQUIRE((n_idx + 3) / 4 <= 0x7fffffffull, LQ_ERR_SHAPE, "embedding_i8: too many indices");
    LQ_REQUIRE(dim % 4 != 0 || (aligned16(out) && (reinterpret_cast<uintptr_t>(table) & 3u) == 0), LQ_ERR_VALUE,
               "embedding_i8: table must be 4-byte and output 16-byte aligned");
    hipLaunchKernelGGL(embedding_i8_kernel, dim3(unsigned((n_idx + 3) / 4)), dim3(256), 0, as_stream(stream), table,
                       scale, zp, num_embeddings, dim, idx, idx_is_64, n_idx, padding_idx, out);
    LQ_CHECK_LAUNCH("embedding_i8");
    return LQ_OK;
}

int lq_embedding_bag_i8(const int8_t* table, const float* scale, const float* zp, int num_embeddings, int dim,
                        const void* idx, int idx_is_64, size_t n_idx, const void* offsets, int offsets_is_64,
                        int fixed_len, int bags, int mode, int padding_idx, float* out, lq_stream stream) {
    LQ_REQUIRE(num_embeddings >= 0 && dim >= 0 && bags >= 0, LQ_ERR_SHAPE, "embedding_bag_i8: negative extent");
    LQ_REQUIRE(mode >= 0 && mode <= 2, LQ_ERR_VALUE, "embedding_bag_i8: mode must be 0 (sum), 1 (mean) or 2 (max)");
    if (bags == 0 || dim == 0) return LQ_OK;
    LQ_REQUIRE(table && scale && zp && out && (n_idx == 0 || idx), LQ_ERR_VALUE, "embedding_bag_i8: NULL pointer");
    LQ_REQUIRE(offsets || (fixed_len >= 0 && size_t(bags) * size_t(fixed_len) == n_idx), LQ_ERR_SHAPE,
               "embedding_bag_i8: without offsets the indices must be bags x fixed_len");
    hipLaunchKernelGGL(embedding_bag_i8_kernel, dim3(unsigned((bags + 3) / 4)), dim3(256), 0, as_stream(stream),
                       table, scale, zp, num_embeddings, dim, idx, idx_is_64, (long long)n_idx, offsets,
                       offsets_is_64, fixed_len, bags, mode, padding_idx, out);
    LQ_CHECK_LAUNCH("embedding_bag_i8");
    return LQ_OK;
}

int lq_act_f32(int kind, float alpha, const float* x, float* out, size_t n, int fake_quantize_out,
               const float* out_scale, const float* out_zp, int out_qmin, int out_qmax, lq_stream stream) {
    LQ_REQUIRE(kind >= 0 && kind <= 5, LQ_ERR_VALUE, "act_f32: unknown activation %d", kind);
    if (n == 0) return LQ_OK;
    LQ_REQUIRE(x && out, LQ_ERR_VALUE, "act_f32: NULL pointer");
    LQ_REQUIRE(!fake_quantize_out || (out_scale && out_zp && out_qmin <= out_qmax), LQ_ERR_VALUE,
               "act_f32: output qparams missing");
    hipLaunchKernelGGL(act_f32_kernel, dim3(grid_for(n, 256)), dim3(256), 0, as_stream(stream), kind, alpha, x, out,
                       n, fake_quantize_out, out_scale, out_zp, float(out_qmin), float(out_qmax));
    LQ_CHECK_LAUNCH("act_f32");
    return LQ_OK;
}

int lq_act_requant_i8(int kind, float alpha, const int8_t* q, int q_offset, const float* scale, const float* zp,
                      size_t n, const float* out_scale, const float* out_zp, int out_qmin, int out_qmax,
                      int out_offset, int8_t* out, lq_stream stream) {
    LQ_REQUIRE(kind >= 0 && kind <= 5, LQ_ERR_VALUE, "act_requant_i8: unknown activation %d", kind);
    if (n == 0) return LQ_OK;
    LQ_REQUIRE(q && out && scale && zp && out_scale && out_zp, LQ_ERR_VALUE, "act_requant_i8: NULL pointer");
    int rc = check_out_grid("act_requant_i8", out_qmin, out_qmax, out_offset);
    if (rc) return rc;
    hipLaunchKernelGGL(act_requant_i8_kernel, dim3(grid_for(n, 4096)), dim3(256), 0, as_stream(stream), kind, alpha,
                       q, q_offset, scale, zp, n, out_scale, out_zp, float(out_qmin), float(out_qmax), out_offset,
                       out);
    LQ_CHECK_LAUNCH("act_requant_i8");
    return LQ_OK;
}

int lq_dilate_nhwc_i8(const int8_t* x, int B, int H, int W, int C, int stride_h, int stride_w, int extra_h,
                      int extra_w, int fill, int8_t* out, lq_stream stream) {
    LQ_REQUIRE(B >= 0 && H > 0 && W > 0 && C > 0, LQ_ERR_SHAPE, "dilate_nhwc_i8: bad extent");
    LQ_REQUIRE(stride_h >= 1 && stride_w >= 1 && extra_h >= 0 && extra_w >= 0, LQ_ERR_VALUE,
               "dilate_nhwc_i8: bad stride / extra rows");
    LQ_REQUIRE(fill >= -128 && fill <= 127, LQ_ERR_VALUE, "dilate_nhwc_i8: fill %d is not an int8 code", fill);
    if (B == 0) return LQ_OK;
    LQ_REQUIRE(x && out, LQ_ERR_VALUE, "dilate_nhwc_i8: NULL pointer");
    const int OH = (H - 1) * stride_h + 1 + extra_h, OW = (W - 1) * stride_w + 1 + extra_w;
    const size_t n = size_t(B) * OH * OW * C;
    hipLaunchKernelGGL(dilate_nhwc_i8_kernel, dim3(grid_for(n, 1024)), dim3(256), 0, as_stream(stream), x, B, H, W, C,
                       stride_h, stride_w, OH, OW, fill, out);
    LQ_CHECK_LAUNCH("dilate_nhwc_i8");
    return LQ_OK;
}

int lq_lstm_cell_f32(const float* gates_x, size_t gates_x_ld, const float* gates_h, const float* bias,
                     const float* c_in, int batch, int hidden,
                     float* h_out, float* c_out, float* y, size_t y_ld, lq_stream stream) {
    LQ_REQUIRE(batch >= 0 && hidden >= 0, LQ_ERR_SHAPE, "lstm_cell_f32: negative extent");
    if (size_t(batch) * hidden == 0) return LQ_OK;
    LQ_REQUIRE(gates_x && gates_h && c_in && h_out && c_out, LQ_ERR_VALUE, "lstm_cell_f32: NULL pointer");
    LQ_REQUIRE(!y || y_ld >= size_t(hidden), LQ_ERR_SHAPE, "lstm_cell_f32: output row stride smaller than hidden");
    LQ_REQUIRE(gates_x_ld >= size_t(4) * hidden, LQ_ERR_SHAPE, "lstm_cell_f32: gate row stride smaller than 4 * hidden");
    hipLaunchKernelGGL(lstm_cell_kernel, dim3(grid_for(size_t(batch) * hidden, 256)), dim3(256), 0,
                       as_stream(stream), gates_x, gates_h, bias, c_in, batch, hidden, gates_x_ld, h_out, c_out, y, y_ld);
    LQ_CHECK_LAUNCH("lstm_cell_f32");
    return LQ_OK;
}

}  // extern "C"
