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

// One activation row (decode): the same scheme with the weight stream software-pipelined.
// A wavefront owns four weight rows and walks K in steps of 64 * CODES; the 16-byte code
// loads (and scale / bias) of all four rows for the next step are in flight while the current
// step is multiplied, and the first step's loads are issued before x is staged, so the only
// exposed memory latency is the first one.  K % (64 * CODES) == 0.
template <int BITS>
__global__ __launch_bounds__(256) void wq_gemv1_kernel(const float* x, const uint32_t* packed, const float* scales,
                                                       const float* biases, int N, int K, int gs, float* out) {
    extern __shared__ __attribute__((aligned(16))) float sx[];
    constexpr int CODES = 128 / BITS, QUADS = CODES / 4, RW = WQ_ROWS / 4;
    constexpr uint32_t MASK = (1u << BITS) - 1u;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int chunks = K / CODES, steps = chunks / 64;
    const int gs_shift = 31 - __builtin_clz(gs);
    const int words_per_row = K * BITS / 32, groups_per_row = K >> gs_shift;
    const uint4* wrow[RW];
    const float* srow[RW];
    const float* brow[RW];
#pragma unroll
    for (int r = 0; r < RW; ++r) {
        int n = blockIdx.x * WQ_ROWS + wave * RW + r;
        n = n < N ? n : N - 1;  // clamped rows are computed and dropped at the store
        wrow[r] = reinterpret_cast<const uint4*>(packed + size_t(n) * words_per_row);
        srow[r] = scales + size_t(n) * groups_per_row;
        brow[r] = biases + size_t(n) * groups_per_row;
    }
    struct Operands {
        uint4 w[RW];
        float s[RW], b[RW];
    };
    // Scales and biases of the wavefront's rows.  With at most 64 groups per row (and RW = 4) they
    // come in two wavefront-wide direct loads into LDS - 16 lanes x 16 bytes per row and array -
    // instead of two 4-byte loads per row and step: a load instruction costs the memory pipeline
    // about the same whatever it carries.  Layout: sb[wave][array][row][64].
    const bool sb_lds = RW == 4 && groups_per_row <= 64 && groups_per_row % 4 == 0 &&
                        ((reinterpret_cast<uintptr_t>(scales) | reinterpret_cast<uintptr_t>(biases)) & 15u) == 0;
    float* const sb = sx + K + wave * 512;
    auto fetch = [&](int step, Operands& o) {
        const int L = step * 64 + lane, g = (L * CODES) >> gs_shift;  // group sizes are powers of two
#pragma unroll
        for (int r = 0; r < RW; ++r) o.w[r] = wrow[r][L];
        if (!sb_lds) {
#pragma unroll
            for (int r = 0; r < RW; ++r) o.s[r] = srow[r][g], o.b[r] = brow[r][g];
        }
    };
    auto pin = [] {
        asm volatile("" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
    };
    Operands o0, o1;
    fetch(0, o0);
    if (sb_lds) {
        const int r = lane >> 4;
        int part = (lane & 15) * 4;
        part = part < groups_per_row ? part : groups_per_row - 4;  // lanes past the row's groups repeat its last four
        typedef __attribute__((address_space(1))) void* gptr;
        typedef __attribute__((address_space(3))) void* lptr;
        __builtin_amdgcn_global_load_lds((gptr)(srow[r % RW] + part), (lptr)(sb), 16, 0, 0);
        __builtin_amdgcn_global_load_lds((gptr)(brow[r % RW] + part), (lptr)(sb + 256), 16, 0, 0);
    }
    pin();
    for (int i = tid * 4; i < K; i += 256 * 4) {
        const float4 v = *reinterpret_cast<const float4*>(x + i);
        const int L = i / CODES, j = (i % CODES) / 4;
        *reinterpret_cast<float4*>(sx + (j * chunks + L) * 4) = v;
    }
    // the activation loads above are younger than the direct loads: once they have been consumed (they
    // were, by the LDS stores), the scales and biases have landed as well
    __builtin_amdgcn_s_waitcnt(0x0070 | (0xF << 8));  // vmcnt(0)
    __syncthreads();
    float acc[RW];
#pragma unroll
    for (int r = 0; r < RW; ++r) acc[r] = 0.0f;
    auto compute = [&](int step, Operands& o) {
        const int L = step * 64 + lane;
        if (sb_lds) {
            const int g = (L * CODES) >> gs_shift;
#pragma unroll
            for (int r = 0; r < RW; ++r) o.s[r] = sb[r * 64 + g], o.b[r] = sb[256 + r * 64 + g];
        }
        float dot[RW], sum = 0.0f;
#pragma unroll
        for (int r = 0; r < RW; ++r) dot[r] = 0.0f;
#pragma unroll
        for (int quad = 0; quad < QUADS; ++quad) {
            const float4 xv = *reinterpret_cast<const float4*>(sx + (quad * chunks + L) * 4);
            sum += (xv.x + xv.y) + (xv.z + xv.w);
#pragma unroll
            for (int r = 0; r < RW; ++r) {
                const uint32_t words[4] = {o.w[r].x, o.w[r].y, o.w[r].z, o.w[r].w};
                float c[4];
                if (BITS == 4) {
                    // the even nibbles of a word as the bytes of `lo`, the odd ones as the bytes of `hi`
                    // (three instructions per eight codes), then one byte-to-float conversion per code:
                    // five instructions less per word than a bit-field extract and a conversion per code
                    const uint32_t word = words[quad >> 1];
                    const uint32_t lo = word & 0x0f0f0f0fu, hi = (word >> 4) & 0x0f0f0f0fu;
                    const int sh = (quad & 1) * 16;  // a constant once the quad loop is unrolled
                    c[0] = float((lo >> sh) & 0xffu), c[1] = float((hi >> sh) & 0xffu);
                    c[2] = float((lo >> (sh + 8)) & 0xffu), c[3] = float((hi >> (sh + 8)) & 0xffu);
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int j = quad * 4 + e;  // code index inside the 16-byte load
                        c[e] = float((words[j * BITS / 32] >> ((j * BITS) % 32)) & MASK);
                    }
                }
                // fused multiply-adds by name (contraction is off for this library): the decode
                // loop is bound by vector instructions, not by memory
                dot[r] = __builtin_fmaf(c[0], xv.x, dot[r]);
                dot[r] = __builtin_fmaf(c[1], xv.y, dot[r]);
                dot[r] = __builtin_fmaf(c[2], xv.z, dot[r]);
                dot[r] = __builtin_fmaf(c[3], xv.w, dot[r]);
            }
        }
#pragma unroll
        for (int r = 0; r < RW; ++r) acc[r] += o.s[r] * dot[r] + o.b[r] * sum;
    };
    const int last = steps - 1;
    int step = 0;
    for (;;) {
        fetch(step + 1 < steps ? step + 1 : last, o1);
        pin();
        compute(step, o0);
        pin();
        if (++step >= steps) break;
        fetch(step + 1 < steps ? step + 1 : last, o0);
        pin();
        compute(step, o1);
        pin();
        if (++step >= steps) break;
    }
#pragma unroll
    for (int r = 0; r < RW; ++r) {
        float v = acc[r];
#pragma unroll
        for (int d = 32; d >= 1; d >>= 1) v += __shfl_xor(v, d, 64);
        const int n = blockIdx.x * WQ_ROWS + wave * RW + r;
        if (lane == 0 && n < N) out[n] = v;
    }
}

template <int BITS>
int launch_gemv1(const float* x, const uint32_t* packed, const float* scales, const float* biases, int N, int K,
                 int gs, float* out, hipStream_t st) {
    const size_t smem = size_t(K) * sizeof(float) + 4 * 512 * sizeof(float);  // x, then scales / biases per wavefront
    const void* fn = reinterpret_cast<const void*>(wq_gemv1_kernel<BITS>);
    static size_t attr = 0;
    if (smem > attr) {
        LQ_HIP(hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, int(smem)));
        attr = smem;
    }
    hipLaunchKernelGGL((wq_gemv1_kernel<BITS>), dim3(unsigned((N + WQ_ROWS - 1) / WQ_ROWS)), dim3(256), smem, st, x,
                       packed, scales, biases, N, K, gs, out);
    LQ_CHECK_LAUNCH("wq_gemv1");
    return LQ_OK;
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

// Small-batch matmul on the matrix cores: up to 16 activation rows against 32 weight
// rows per block.  The weight is the A operand of v_mfma_f32_16x16x4_f32 and x^T the B
// operand, so a lane holds one weight row r = lane % 16 (two row blocks) and one
// activation row of the same index, and the four k slots of an instruction belong to
// the four lane quarters q = lane / 16.  A quarter owns CODES consecutive k of a step -
// exactly the codes of one 16-byte load, all in one group - so nothing is shuffled
// between lanes: code j of the load meets x[k0 + j] in instruction j.  Weights are
// decoded as c * s + b (the dequantize kernel's expression) right before use.  The four
// eight wavefronts of a block take the k steps round-robin (two per SIMD, each with
// four independent accumulator chains, so dependent MFMAs do not wait on each other)
// and add their partial tiles through LDS in a fixed order.
//
// Read straight from x, a lane's 16-byte loads would touch 64 different cache lines per
// instruction (16 rows x 4 quarters).  A pre-pass therefore lays x out in the order the
// lanes consume it - float4 number (step * XV + j) * 64 + lane of a 16-row block - so
// that every load of the main kernel is one contiguous KiB per wavefront; rows past M
// are written as zeros there.
typedef float v4f __attribute__((ext_vector_type(4)));

template <int BITS>
__global__ __launch_bounds__(256) void wq_arrange_x_kernel(const float* __restrict__ x, int M, int K,
                                                           float4* __restrict__ xt) {
    constexpr int CODES = 128 / BITS, STEP = 4 * CODES, XV = CODES / 4;
    const int per_block = K / STEP * XV * 64;  // float4 per 16-row block
    const int idx = blockIdx.x * 256 + threadIdx.x;
    if (idx >= per_block) return;
    const int lane = idx & 63, sj = idx >> 6, j = sj % XV, step = sj / XV;
    const int m = blockIdx.y * 16 + (lane & 15), k = step * STEP + (lane >> 4) * CODES + 4 * j;
    float4 v = {0.f, 0.f, 0.f, 0.f};
    if (m < M) v = *reinterpret_cast<const float4*>(x + size_t(m) * K + k);
    xt[size_t(blockIdx.y) * per_block + idx] = v;
}

template <int BITS>
__global__ __launch_bounds__(512) void wq_mfma_kernel(const float4* xt, const uint32_t* packed, const float* scales,
                                                      const float* biases, int M, int N, int K, int gs, float* out) {
    constexpr int CODES = 128 / BITS;  // codes per 16-byte load: 32 or 16
    constexpr int STEP = 4 * CODES;    // k covered by one wavefront step
    constexpr int XV = CODES / 4;      // float4 loads of x per step
    constexpr uint32_t MASK = (1u << BITS) - 1u;
    constexpr int WAVES = 8;
    __shared__ __attribute__((aligned(16))) float red[WAVES][2][64][4];
    // the wavefront index as a scalar, so that the step loop branches uniformly
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int r = lane & 15, q = lane >> 4;
    const int n_base = blockIdx.x * 32;
    const int words_per_row = K * BITS / 32, groups_per_row = K / gs;
    const int gs_shift = 31 - __builtin_clz(gs);  // group sizes are powers of two
    const int m0 = blockIdx.y * 16;
    const float4* xblk = xt + size_t(blockIdx.y) * (K / STEP * XV * 64) + lane;
    const uint32_t* wrow[2];
    const float* srow[2];
    const float* brow[2];
#pragma unroll
    for (int rb = 0; rb < 2; ++rb) {
        int n = n_base + rb * 16 + r;
        n = n < N ? n : N - 1;  // clamped rows are computed and dropped at the store
        wrow[rb] = packed + size_t(n) * words_per_row;
        srow[rb] = scales + size_t(n) * groups_per_row;
        brow[rb] = biases + size_t(n) * groups_per_row;
    }
    v4f acc[2][2] = {{{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}}, {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}}};
    const int steps = K / STEP;

    // Two register sets, named at compile time (a run-time buffer index would put the
    // arrays in scratch memory): the loads of the next step are issued before this one
    // is used.
    struct Operands {
        uint4 wv[2];
        float sc[2], bi[2];
        float4 xv[XV];
    };
    auto fetch = [&](int step, Operands& o) {
        const int k0 = step * STEP + q * CODES;
#pragma unroll
        for (int rb = 0; rb < 2; ++rb) {
            o.wv[rb] = *reinterpret_cast<const uint4*>(wrow[rb] + k0 * BITS / 32);
            o.sc[rb] = srow[rb][k0 >> gs_shift];
            o.bi[rb] = brow[rb][k0 >> gs_shift];
        }
#pragma unroll
        for (int j = 0; j < XV; ++j) o.xv[j] = xblk[(step * XV + j) * 64];
    };
    auto compute = [&](const Operands& o) {
#pragma unroll
        for (int rb = 0; rb < 2; ++rb) {
            const uint32_t words[4] = {o.wv[rb].x, o.wv[rb].y, o.wv[rb].z, o.wv[rb].w};
            const float s = o.sc[rb], b = o.bi[rb];
#pragma unroll
            for (int j = 0; j < CODES; ++j) {
                const uint32_t code = (words[j * BITS / 32] >> ((j * BITS) % 32)) & MASK;
                const float wval = float(code) * s + b;
                const float4 xq = o.xv[j / 4];
                const float xval = (j % 4) == 0 ? xq.x : ((j % 4) == 1 ? xq.y : ((j % 4) == 2 ? xq.z : xq.w));
                acc[rb][j & 1] = __builtin_amdgcn_mfma_f32_16x16x4f32(wval, xval, acc[rb][j & 1], 0, 0, 0);
            }
        }
    };
    // The look-ahead fetch is unconditional (past the end it re-reads the last step and
    // the result is dropped): a branch around it would make the compiler wait, at the
    // join, as if the new loads had not been issued - that is, for them.
    // keeps the look-ahead loads ahead of the MFMAs: neither the optimizer (memory clobber;
    // the pointers are not __restrict__ for that reason) nor the instruction scheduler may
    // move a load across this point
    auto pin = [] {
        asm volatile("" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
    };
    Operands o0, o1;
    int step = wave;
    const int last = steps - 1;
    if (step < steps) {
        fetch(step, o0);
        for (;;) {
            fetch(step + WAVES < steps ? step + WAVES : last, o1);
            pin();
            compute(o0);
            pin();
            step += WAVES;
            if (step >= steps) break;
            fetch(step + WAVES < steps ? step + WAVES : last, o0);
            pin();
            compute(o1);
            pin();
            step += WAVES;
            if (step >= steps) break;
        }
    }
#pragma unroll
    for (int rb = 0; rb < 2; ++rb) *reinterpret_cast<v4f*>(red[wave][rb][lane]) = acc[rb][0] + acc[rb][1];
    __syncthreads();
    // D[i][j]: lane holds i = 4 * (lane / 16) + t, j = lane % 16  ->  out[m0 + j][n_base + rb*16 + i]
    {
        const int e = threadIdx.x;  // 2 * 64 * 4 = 512 values, one per thread
        const int rb = e >> 8, l = (e >> 2) & 63, t = e & 3;
        float v = red[0][rb][l][t];
#pragma unroll
        for (int w = 1; w < WAVES; ++w) v += red[w][rb][l][t];
        const int n = n_base + rb * 16 + 4 * (l >> 4) + t, mm = m0 + (l & 15);
        if (n < N && mm < M) out[size_t(mm) * N + n] = v;
    }
}

template <int BITS>
int launch_wq_mfma(const float* x, const uint32_t* packed, const float* scales, const float* biases, int M, int N,
                   int K, int gs, float* out, hipStream_t st) {
    constexpr int STEP = 512 / BITS;
    const int mblocks = (M + 15) / 16;
    void* ws = nullptr;
    const int rc = workspace(size_t(mblocks) * 16 * K * sizeof(float), st, &ws);
    if (rc) return rc;
    const int per_block = K / STEP * (32 / BITS) * 64;
    hipLaunchKernelGGL((wq_arrange_x_kernel<BITS>), dim3(unsigned((per_block + 255) / 256), unsigned(mblocks)),
                       dim3(256), 0, st, x, M, K, static_cast<float4*>(ws));
    LQ_CHECK_LAUNCH("wq_arrange_x");
    hipLaunchKernelGGL((wq_mfma_kernel<BITS>), dim3(unsigned((N + 31) / 32), unsigned(mblocks)), dim3(512), 0, st,
                       static_cast<const float4*>(ws), packed, scales, biases, M, N, K, gs, out);
    LQ_CHECK_LAUNCH("wq_mfma");
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
    // 16 activation rows per launch on the matrix cores; a step covers 512 / bits weights per row
    const bool mfma_ok = aligned16(x) && aligned16(packed) && K % (512 / bits) == 0;
    if (M > 1 && M <= 64 && mfma_ok)
        return bits == 4 ? launch_wq_mfma<4>(x, packed, scales, biases, M, N, K, group_size, out, st)
                         : launch_wq_mfma<8>(x, packed, scales, biases, M, N, K, group_size, out, st);
    if (M == 1 && fused_ok && K % (8192 / bits) == 0)
        return bits == 4 ? launch_gemv1<4>(x, packed, scales, biases, N, K, group_size, out, st)
                         : launch_gemv1<8>(x, packed, scales, biases, N, K, group_size, out, st);
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
    rc = workspace(size_t(N) * K * sizeof(float), st, &ws);
    if (rc) return rc;
    rc = lq_wq_dequantize(packed, scales, biases, N, K, group_size, bits, static_cast<float*>(ws), stream);
    if (rc) return rc;
    return lq_sgemm_nt_f32(x, static_cast<const float*>(ws), nullptr, out, M, N, K, stream);
}

}  // extern "C"
