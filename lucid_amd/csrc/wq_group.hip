// Group-wise affine weight-only quantization (int4 / int8 codes packed in 32-bit
// words) and the matmul that decodes it on the fly - the operator set Lucid binds
// as engine.quantized.{quantize, dequantize, quantized_matmul}
// (lucid/_C/ops/quantized/QuantizedMatmul.cpp:47-115, lucid/quantization/_qgemm.py:69-320)
// on top of MLX.  MLX is not part of the Lucid checkout; this follows the published
// contract (mlx.core.quantize documentation, restated in _qgemm.py:84-97,167-171):
//
//   per row, per group of `group_size` consecutive elements:
//     s = (max - min) / (2^bits - 1),  beta = min
//     c_i = clip(round((w_i - beta) / s), 0, 2^bits - 1)      w_i ~ c_i * s + beta
//   codes little-endian inside a word: code j of a word sits at bits [j*bits, (j+1)*bits)
//   y = x . w_hat^T, float32
//
// A constant group (max == min) gets s = 1e-7-floored, so its codes are 0 and it
// decodes to beta exactly.  The decode side takes scales and biases as given (any
// sign), so weights packed elsewhere under the same contract load unchanged.
#include "common.hpp"

using namespace lq;

namespace {

__device__ __forceinline__ float wave_min(float v) {
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) v = fminf(v, __shfl_xor(v, d, 64));
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) v = fmaxf(v, __shfl_xor(v, d, 64));
    return v;
}

// One wavefront per group.  Lane l owns elements l, l + 64 (group_size 128) of the group.
__global__ __launch_bounds__(256) void wq_quantize_kernel(const float* __restrict__ w, size_t groups, int gs,
                                                          int bits, uint32_t* __restrict__ packed,
                                                          float* __restrict__ scales, float* __restrict__ biases) {
    const size_t g = size_t(blockIdx.x) * 4 + (threadIdx.x >> 6);
    if (g >= groups) return;
    const int lane = threadIdx.x & 63;
    const float* src = w + g * gs;
    const int per_word = 32 / bits;
    const float nmax = float((1 << bits) - 1);
    float lo = __builtin_inff(), hi = -__builtin_inff();
    for (int i = lane; i < gs; i += 64) {
        const float v = src[i];
        lo = fminf(lo, v);
        hi = fmaxf(hi, v);
    }
    lo = wave_min(lo);
    hi = wave_max(hi);
    float s = (hi - lo) / nmax;
    s = s < 1e-7f ? 1e-7f : s;
    if (lane == 0) scales[g] = s, biases[g] = lo;
    // one lane per output word
    uint32_t* dst = packed + g * (gs / per_word);
    for (int wd = lane; wd < gs / per_word; wd += 64) {
        uint32_t word = 0;
        for (int j = 0; j < per_word; ++j) {
            float q = __builtin_rintf((src[wd * per_word + j] - lo) / s);
            q = q < 0.0f ? 0.0f : (q > nmax ? nmax : q);
            word |= uint32_t(q) << (j * bits);
        }
        dst[wd] = word;
    }
}

__global__ __launch_bounds__(256) void wq_dequantize_kernel(const uint32_t* __restrict__ packed,
                                                            const float* __restrict__ scales,
                                                            const float* __restrict__ biases, size_t words, int gs,
                                                            int bits, float* __restrict__ out) {
    const size_t wd = size_t(blockIdx.x) * 256 + threadIdx.x;
    if (wd >= words) return;
    const int per_word = 32 / bits;
    const uint32_t mask = (1u << bits) - 1u;
    const size_t first = wd * per_word, g = first / gs;
    const float s = scales[g], b = biases[g];
    const uint32_t word = packed[wd];
    for (int j = 0; j < per_word; ++j) out[first + j] = float((word >> (j * bits)) & mask) * s + b;
}

// Decode-shaped matmul: y[m, n] = sum_k x[m, k] * (c[n, k] * s[n, g(k)] + b[n, g(k)]), m < MT.
// A block stages the MT activation rows in LDS once and computes WQ_ROWS output
// columns with them, four per wavefront; a lane takes 16 bytes of codes (32 int4
// or 16 int8 codes, never straddling a group) per step, so a wavefront streams
// 1 KiB of contiguous weight per load.  Per group: acc += s * sum(c*x) + b * sum(x).
constexpr int WQ_ROWS = 16;

template <int BITS, int MT>
__global__ __launch_bounds__(256) void wq_gemv_kernel(const float* __restrict__ x, const uint32_t* __restrict__ packed,
                                                      const float* __restrict__ scales,
                                                      const float* __restrict__ biases, int M, int N, int K, int gs,
                                                      int m0, float* __restrict__ out) {
    // Activation rows in LDS, permuted so that the lanes of a wavefront read
    // consecutive 16-byte slots: k = CODES*L + 4*j + e is stored at [m][j][L][e]
    // (lane L of a step reads quad j of its CODES-long chunk).
    extern __shared__ __attribute__((aligned(16))) float sx[];
    constexpr int CODES = 128 / BITS;  // codes per 16-byte load
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int rows = M - m0 < MT ? M - m0 : MT;
    const int chunks = K / CODES;
    for (int i = tid * 4; i < MT * K; i += 256 * 4) {
        const int m = i / K, k = i - m * K;
        float4 v = {0.f, 0.f, 0.f, 0.f};
        if (m < rows) v = *reinterpret_cast<const float4*>(x + size_t(m0 + m) * K + k);
        const int L = k / CODES, j = (k % CODES) / 4;
        *reinterpret_cast<float4*>(sx + m * K + (j * chunks + L) * 4) = v;
    }
    __syncthreads();
    const int words_per_row = K * BITS / 32, groups_per_row = K / gs;
    for (int r = 0; r < WQ_ROWS / 4; ++r) {
        const int n = blockIdx.x * WQ_ROWS + wave * (WQ_ROWS / 4) + r;
        if (n >= N) break;
        const uint32_t* wrow = packed + size_t(n) * words_per_row;
        const float* srow = scales + size_t(n) * groups_per_row;
        const float* brow = biases + size_t(n) * groups_per_row;
        float acc[MT];
#pragma unroll
        for (int m = 0; m < MT; ++m) acc[m] = 0.0f;
        for (int k = lane * CODES; k < K; k += 64 * CODES) {
            const uint4 wv = *reinterpret_cast<const uint4*>(wrow + k * BITS / 32);
            const int g = k / gs;
            const float s = srow[g], b = brow[g];
            const uint32_t words[4] = {wv.x, wv.y, wv.z, wv.w};
            float dot[MT], sum[MT];
#pragma unroll
            for (int m = 0; m < MT; ++m) dot[m] = 0.0f, sum[m] = 0.0f;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
#pragma unroll
                for (int j = 0; j < 32 / BITS; j += 4) {
                    const int quad = (q * (32 / BITS) + j) / 4;  // quad of this lane's chunk
                    float c[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        c[e] = float((words[q] >> ((j + e) * BITS)) & ((1u << BITS) - 1u));
#pragma unroll
                    for (int m = 0; m < MT; ++m) {
                        const float4 xv =
                            *reinterpret_cast<const float4*>(sx + m * K + (quad * chunks + k / CODES) * 4);
                        dot[m] += c[0] * xv.x + c[1] * xv.y + c[2] * xv.z + c[3] * xv.w;
                        sum[m] += (xv.x + xv.y) + (xv.z + xv.w);
                    }
                }
            }
#pragma unroll
            for (int m = 0; m < MT; ++m) acc[m] += s * dot[m] + b * sum[m];
        }
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            float v = acc[m];
#pragma unroll
            for (int d = 32; d >= 1; d >>= 1) v += __shfl_xor(v, d, 64);
            if (lane == 0 && m < rows) out[size_t(m0 + m) * N + n] = v;
        }
    }
}

template <int BITS, int MT>
int launch_gemv(const float* x, const uint32_t* packed, const float* scales, const float* biases, int M, int N,
                int K, int gs, int m0, float* out, hipStream_t st) {
    const size_t smem = size_t(MT) * K * sizeof(float);
    const void* fn = reinterpret_cast<const void*>(wq_gemv_kernel<BITS, MT>);
    static size_t attr = 0;
    if (smem > attr) {
        LQ_HIP(hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, int(smem)));
        attr = smem;
    }
    hipLaunchKernelGGL((wq_gemv_kernel<BITS, MT>), dim3(unsigned((N + WQ_ROWS - 1) / WQ_ROWS)), dim3(256), smem, st, x,
                       packed, scales, biases, M, N, K, gs, m0, out);
    LQ_CHECK_LAUNCH("wq_gemv");
    return LQ_OK;
}

int check_group(const char* who, int K, int gs, int bits) {
    LQ_REQUIRE(bits == 4 || bits == 8, LQ_ERR_VALUE, "%s: bits must be 4 or 8 (got %d)", who, bits);
    LQ_REQUIRE(gs == 32 || gs == 64 || gs == 128, LQ_ERR_VALUE, "%s: group_size must be 32, 64 or 128 (got %d)", who,
               gs);
    LQ_REQUIRE(K > 0 && K % gs == 0, LQ_ERR_SHAPE, "%s: the quantized axis (%d) must be a multiple of group_size %d",
               who, K, gs);
    return LQ_OK;
}

}  // namespace

extern "C" {

int lq_sgemm_nt_f32(const float* a, const float* w, const float* bias, float* out, int M, int N, int K, void* stream);

int lq_wq_quantize(const float* w, int N, int K, int group_size, int bits, uint32_t* packed, float* scales,
                   float* biases, lq_stream stream) {
    int rc = check_group("wq_quantize", K, group_size, bits);
    if (rc) return rc;
    LQ_REQUIRE(N >= 0, LQ_ERR_SHAPE, "wq_quantize: negative row count");
    if (N == 0) return LQ_OK;
    LQ_REQUIRE(w && packed && scales && biases, LQ_ERR_VALUE, "wq_quantize: NULL pointer");
    const size_t groups = size_t(N) * (K / group_size);
    LQ_REQUIRE((groups + 3) / 4 < 0x7fffffffull, LQ_ERR_SHAPE, "wq_quantize: tensor too large");
    hipLaunchKernelGGL(wq_quantize_kernel, dim3(unsigned((groups + 3) / 4)), dim3(256), 0, as_stream(stream), w,
                       groups, group_size, bits, packed, scales, biases);
    LQ_CHECK_LAUNCH("wq_quantize");
    return LQ_OK;
}

int lq_wq_dequantize(const uint32_t* packed, const float* scales, const float* biases, int N, int K, int group_size,
                     int bits, float* out, lq_stream stream) {
    int rc = check_group("wq_dequantize", K, group_size, bits);
    if (rc) return rc;
    LQ_REQUIRE(N >= 0, LQ_ERR_SHAPE, "wq_dequantize: negative row count");
    if (N == 0) return LQ_OK;
    LQ_REQUIRE(packed && scales && biases && out, LQ_ERR_VALUE, "wq_dequantize: NULL pointer");
    const size_t words = size_t(N) * K * bits / 32;
    LQ_REQUIRE((words + 255) / 256 < 0x7fffffffull, LQ_ERR_SHAPE, "wq_dequantize: tensor too large");
    hipLaunchKernelGGL(wq_dequantize_kernel, dim3(unsigned((words + 255) / 256)), dim3(256), 0, as_stream(stream),
                       packed, scales, biases, words, group_size, bits, out);
    LQ_CHECK_LAUNCH("wq_dequantize");
    return LQ_OK;
}

int lq_wq_matmul(const float* x, const uint32_t* packed, const float* scales, const float* biases, int M, int N, int K,
                 int group_size, int bits, float* out, lq_stream stream) {
    int rc = check_group("wq_matmul", K, group_size, bits);
    if (rc) return rc;
    LQ_REQUIRE(M >= 0 && N >= 0, LQ_ERR_SHAPE, "wq_matmul: negative extent");
    if (M == 0 || N == 0) return LQ_OK;
    LQ_REQUIRE(x && packed && scales && biases && out, LQ_ERR_VALUE, "wq_matmul: NULL pointer");
    hipStream_t st = as_stream(stream);
    const bool fused_ok = aligned16(x) && aligned16(packed) && K % 4 == 0 && (K * bits / 8) % 16 == 0 &&
                          size_t(4) * K * sizeof(float) <= 64 * 1024;
    if (M <= 16 && fused_ok) {
        // decode shapes: weights are read once per pass of up to four activation rows
        for (int m0 = 0; m0 < M; m0 += 4) {
            const int rows = M - m0;
            if (bits == 4)
                rc = rows == 1 ? launch_gemv<4, 1>(x, packed, scales, biases, M, N, K, group_size, m0, out, st)
                     : rows == 2 ? launch_gemv<4, 2>(x, packed, scales, biases, M, N, K, group_size, m0, out, st)
                                 : launch_gemv<4, 4>(x, packed, scales, biases, M, N, K, group_size, m0, out, st);
            else
                rc = rows == 1 ? launch_gemv<8, 1>(x, packed, scales, biases, M, N, K, group_size, m0, out, st)
                     : rows == 2 ? launch_gemv<8, 2>(x, packed, scales, biases, M, N, K, group_size, m0, out, st)
                                 : launch_gemv<8, 4>(x, packed, scales, biases, M, N, K, group_size, m0, out, st);
            if (rc) return rc;
        }
        return LQ_OK;
    }
    // compute-bound shapes: decode once into the workspace, then the float32 MFMA GEMM
    void* ws = nullptr;
    rc = workspace(size_t(N) * K * sizeof(float), &ws);
    if (rc) return rc;
    rc = lq_wq_dequantize(packed, scales, biases, N, K, group_size, bits, static_cast<float*>(ws), stream);
    if (rc) return rc;
    return lq_sgemm_nt_f32(x, static_cast<const float*>(ws), nullptr, out, M, N, K, stream);
}

}  // extern "C"
