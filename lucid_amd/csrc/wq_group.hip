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

// Small-batch matmul on the matrix cores (2 .. 64 activation rows, 16 per block row).
//
// y[m, n] = sum over groups g of  s[n, g] * (sum_{k in g} c[n, k] x[m, k])  +  b[n, g] * (sum_{k in g} x[m, k]):
// the inner sums run on v_mfma_f32_16x16x32_bf16 with the codes themselves as one operand -
// an 8-bit code is exact in bfloat16, a 4-bit code c is formed as the bit pattern 0x4300 | c
// = 128 + c (one AND-OR per two codes) and the 128 goes into the bias term - and x as the
// other, split into three bfloat16 parts x = hi + mid + lo (exact: 8 + 8 + 8 significant
// bits, wq_split3x2), one MFMA each.  Products are exact and accumulate in float32, so nothing of x or
// of the weight is rounded before the sums.
//
// Operand layout of the instruction: lane = (row % 16) + 16 * quarter holds eight k of its
// row, quarter q the k slots 8q .. 8q+7 of the instruction's 32.  x is the A operand (rows
// m) and the codes the B operand (rows n), so an accumulator lane holds column n = lane % 16
// and rows m = 4 * quarter + 0..3, and s, b are one value per lane.
//
// A lane streams its weight row with 16-byte loads (32 int4 / 16 int8 codes; the four
// quarters of a row take consecutive loads: a "window" of 128 / 64 k, 1 KiB per wavefront
// load over 16 rows).  An instruction must stay inside one group, because the scale is
// applied to its sum.  With group_size >= the window that holds as loaded (register j of
// every quarter feeds instruction j).  With two groups per window the registers are
// exchanged between lane halves (v_permlane32_swap: instructions 0, 1 then hold the first
// two quarters' k, instructions 2, 3 the last two), with four groups the 4 x 4 (register,
// quarter) matrix is transposed (v_permlane32_swap + v_permlane16_swap), so instruction i
// holds the k of quarter i.  Which k a slot of an instruction ends up with does not matter
// as long as x follows: the block writes the three parts of its x range into LDS in exactly
// that order.  The sum of x over a group segment comes from the same fragments against a
// row of ones (one more accumulator tile per wavefront), already in the layout the lanes
// need it in.
//
// Every block needs the x of its k range next to its weights (64 bytes of x per k against
// rows / 2 or rows bytes of codes), and every block converts it again.  So a block takes
// many rows (256: eight wavefronts with two 16-row tiles each) and a short k range (512),
// keeps that range's fragments in LDS for all its wavefronts, and requests all its weights
// at once when it starts.  The k ranges of a row tile are blocks of their own (grid.y); each
// writes its partial sums to a slab, and the last one to arrive (an arrival counter per row
// tile, reset by that block) adds the slabs in index order - the result does not depend on
// the order of arrival - and stores.  One launch, no workspace besides the slabs.
typedef float v4f __attribute__((ext_vector_type(4)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));

// LDS a block may ask for: 48 KiB of x fragments and the tables of 256 rows x 16 groups
constexpr int kWqMaxLds = 512 / 32 * 3 * 64 * 16 + 2 * 256 * 17 * 4;

template <int BITS>
struct WqGeom {
    static constexpr int CODES = 128 / BITS;  // codes per 16-byte load: 32 or 16
    static constexpr int WK = 4 * CODES;      // k per window: 128 or 64
    static constexpr int NI = WK / 32;        // instructions (k steps of 32) per window: 4 or 2
};

// How the registers are exchanged for a group size: 0 = not at all, 1 = between lane halves,
// 2 = transposed; the window then holds 1, 2 or 4 group segments.
__host__ __device__ inline int wq_swap_mode(int bits, int gs) {
    const int window = 512 / bits;
    return gs >= window ? 0 : (gs * 2 == window ? 1 : 2);
}

// After the exchange, register rho of quarter q holds what quarter q_src loaded as register j_src.
__host__ __device__ inline void wq_source(int sw, int rho, int q, int& q_src, int& j_src) {
    q_src = q, j_src = rho;
    if (sw == 1 && (rho < 2) != (q < 2)) {
        q_src = rho < 2 ? q - 2 : q + 2;
        j_src = rho < 2 ? rho + 2 : rho - 2;
    } else if (sw == 2) {
        q_src = rho, j_src = q;
    }
}

// upper lane half of a <-> lower lane half of b
__device__ __forceinline__ void wq_swap32(uint32_t& a, uint32_t& b) {
    const auto r = __builtin_amdgcn_permlane32_swap(a, b, false, false);
    a = r[0], b = r[1];
}
// odd 16-lane rows of a <-> even 16-lane rows of b
__device__ __forceinline__ void wq_swap16(uint32_t& a, uint32_t& b) {
    const auto r = __builtin_amdgcn_permlane16_swap(a, b, false, false);
    a = r[0], b = r[1];
}

// (e0, e1) = h + m + l part by part, each part a pair of bfloat16 (e0's in the low half): the
// packed conversion rounds to nearest, the remainders are exact (8 + 8 + 8 significant bits with
// signed remainders).  A NaN stays a NaN in every part; an infinity turns into a NaN in the
// lower parts, so a non-finite x gives a non-finite y.
typedef __bf16 wq_bf2 __attribute__((ext_vector_type(2)));
typedef float wq_f2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t wq_pk(float a, float b) {
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(wq_f2{a, b}, wq_bf2));
}
__device__ __forceinline__ void wq_split3x2(float e0, float e1, uint32_t& h, uint32_t& m, uint32_t& l) {
    h = wq_pk(e0, e1);
    e0 -= __uint_as_float(h << 16), e1 -= __uint_as_float(h & 0xffff0000u);
    m = wq_pk(e0, e1);
    e0 -= __uint_as_float(m << 16), e1 -= __uint_as_float(m & 0xffff0000u);
    l = wq_pk(e0, e1);
}

constexpr int kWqRows = 256;    // weight rows per block
constexpr int kWqSliceK = 512;  // k per block

// Where the A fragment of row m, lane quarter qd of instruction block `blk` sits among the block's
// 64 16-byte slots.  The threads of a wavefront that write the fragments share one m and differ in
// (block, quarter): with the plain slot m + 16 qd they would all hit the same four banks (a
// 64-way conflict: the writes took a tenth of the kernel); rotating m by 4 qd + blk spreads them
// evenly over the 16 bank groups.  A bijection within the block, so the reads of a whole block
// stay conflict-free.
__device__ __forceinline__ int wq_x_slot(int m, int qd, int blk) { return ((m + 4 * qd + blk) & 15) + 16 * qd; }

template <int BITS, int SW>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(4, 4))) void wq_mfma_kernel(
    const float* x, const uint32_t* packed, const float* scales, const float* biases, int M, int N, int K,
    int gs_shift, float* out, float* slabs, int* counters) {
    using G = WqGeom<BITS>;
    constexpr int CODES = G::CODES, WK = G::WK, NI = G::NI;
    constexpr int GW = 1 << SW, SEG = WK / GW;  // group segments per window and their length
    constexpr int IPS = NI / GW;                // instructions per segment
    constexpr int RB = 2, WAVES = 8, WPS = kWqSliceK / WK;  // windows per block: 4 or 8
    constexpr int UNITS = WPS * NI * 64;                    // (window, instruction, lane) triples of the block's x
    static_assert(IPS >= 1, "a segment is at least one instruction");
    static_assert(WAVES * RB * 16 == kWqRows && UNITS % 512 == 0, "");
    // Dynamic LDS: the x fragments of the block's windows ([window][instruction][part][lane],
    // 16 bytes each), then the block's rows of scales and of biases for the groups of those
    // windows - each row padded by one float: lanes of a quarter read 16 different rows at the
    // same group, and the odd stride spreads them over the banks.
    extern __shared__ __attribute__((aligned(16))) uint4 wq_lds[];
    __shared__ int s_arrived;
    // the wavefront index as a scalar, so that branches on it are uniform
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int r = lane & 15, q = lane >> 4;
    // the k ranges of a row tile are neighbours in the grid: they are dispatched together, so the pieces of a
    // weight row (one per k range) are requested at about the same time
    const int tile = blockIdx.y, ks = blockIdx.x, mb = blockIdx.z, slices = gridDim.x;
    const int n_base = tile * kWqRows + wave * (RB * 16), m0 = mb * 16;
    const int words_per_row = K * BITS / 32, groups_per_row = K >> gs_shift;
    const int windows = K / WK;
    const int w0 = ks * WPS;
    const int nw = windows - w0 < WPS ? windows - w0 : WPS;  // at least 1: the host sizes grid.y so
    // groups of this block's windows, and the row stride of the tables
    const int g0 = (w0 * WK) >> gs_shift;
    const int ng = (((w0 + nw) * WK - 1) >> gs_shift) - g0 + 1;
    const int gmax = kWqSliceK >> gs_shift, gp = (gmax < 1 ? 1 : gmax) + 1;

    // Every global load of the block is requested before anything is consumed, in the order of
    // consumption (the wait counter retires loads in order): the scale / bias tables (short, from
    // the L2), x, the weights.
    // Tables: 256 rows x gcap slots (gcap = the groups of a full k range, 4, 8 or 16), four slots per
    // 16-byte load where the rows allow it (a dword per lane costs the vector cache as many cycles
    // as 16 bytes per lane do).
    constexpr int kTabVec = kWqRows * 16 / 4 / 512;  // 16-byte loads per thread and table, at 16 groups per k range
    const int gcap = gp - 1, gsh = 31 - __builtin_clz(unsigned(gcap));  // a power of two: shifts, no division
    const bool tab_vec = ng == gcap && (groups_per_row & 3) == 0 && aligned16(scales) && aligned16(biases);
    float4 tab_s[kTabVec], tab_b[kTabVec];
    {
        const int row_first = tile * kWqRows;
#pragma unroll
        for (int u = 0; u < kTabVec; ++u) {
            const int i = (threadIdx.x + u * 512) * 4, row = i >> gsh, g = i & (gcap - 1);
            tab_s[u] = tab_b[u] = float4{0.f, 0.f, 0.f, 0.f};
            if (i < kWqRows * gcap) {
                const int n = row_first + row < N ? row_first + row : N - 1;
                const size_t at = size_t(n) * groups_per_row + g0 + g;
                if (tab_vec) {
                    tab_s[u] = *reinterpret_cast<const float4*>(scales + at);
                    tab_b[u] = *reinterpret_cast<const float4*>(biases + at);
                } else {
                    // ragged: the last k range of a K that is not a multiple of 512, or unaligned rows
                    if (g < ng) tab_s[u].x = scales[at], tab_b[u].x = biases[at];
                    if (g + 1 < ng) tab_s[u].y = scales[at + 1], tab_b[u].y = biases[at + 1];
                    if (g + 2 < ng) tab_s[u].z = scales[at + 2], tab_b[u].z = biases[at + 2];
                    if (g + 3 < ng) tab_s[u].w = scales[at + 3], tab_b[u].w = biases[at + 3];
                }
            }
        }
    }
    // x of the block's windows: a thread takes eight consecutive k of one row (a wavefront reads
    // 2 KiB of a row)
    constexpr int OCTS = kWqSliceK / 8;  // per row
    static_assert(16 * OCTS == UNITS, "");
    float4 raw[UNITS / 512][2];
#pragma unroll
    for (int u = 0; u < UNITS / 512; ++u) {
        const int unit = u * 512 + threadIdx.x, m = m0 + unit / OCTS, kl = (unit % OCTS) * 8;
        raw[u][0] = raw[u][1] = float4{0.f, 0.f, 0.f, 0.f};
        if (m < M && kl < nw * WK) {
            const float* src = x + size_t(m) * K + w0 * WK + kl;
            raw[u][0] = *reinterpret_cast<const float4*>(src);
            raw[u][1] = *reinterpret_cast<const float4*>(src + 4);
        }
    }
    // All the weights of this wavefront are requested now and used window by window.  For the
    // request a lane takes quarter lane % 4 of row lane / 4 - four neighbouring lanes read 64
    // contiguous bytes, where the operand layout (row lane % 16, quarter lane / 16) would make
    // every lane a cache access of its own -; a lane permutation below puts each 16 bytes
    // where the instruction wants them.
    uint4 wv[WPS][RB];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
        int n = n_base + rb * 16 + (lane >> 2);
        n = n < N ? n : N - 1;  // clamped rows are computed and dropped at the store
        const uint32_t* row = packed + size_t(n) * words_per_row + (lane & 3) * (CODES * BITS / 32);
#pragma unroll
        for (int wi = 0; wi < WPS; ++wi)
            // past the last window every lane reads the same 16 bytes: one cache line, dropped later
            wv[wi][rb] = *reinterpret_cast<const uint4*>(wi < nw ? row + (w0 + wi) * (WK * BITS / 32) : packed);
    }
    // The tables go to LDS, then x, split and laid out as fragments by the block itself: a thread
    // finds the (instruction, quarter) that holds its eight k - the exchange of registers is its
    // own inverse.
    uint4* x_lds = wq_lds;
    float* s_lds = reinterpret_cast<float*>(wq_lds + WPS * NI * 3 * 64);
    float* b_lds = s_lds + kWqRows * gp;
#pragma unroll
    for (int u = 0; u < kTabVec; ++u) {
        const int i = (threadIdx.x + u * 512) * 4, row = i >> gsh, g = i & (gcap - 1);
        if (i < kWqRows * gcap) {  // (slots past ng hold zeros and are never read)
            float* sd = s_lds + row * gp + g;
            float* bd = b_lds + row * gp + g;
            sd[0] = tab_s[u].x, sd[1] = tab_s[u].y, sd[2] = tab_s[u].z, sd[3] = tab_s[u].w;
            bd[0] = tab_b[u].x, bd[1] = tab_b[u].y, bd[2] = tab_b[u].z, bd[3] = tab_b[u].w;
        }
    }
    {
#pragma unroll
        for (int u = 0; u < UNITS / 512; ++u) {
            const int unit = u * 512 + threadIdx.x, ml = unit / OCTS, kl = (unit % OCTS) * 8;
            const int wi = kl / WK, off = kl % WK, qs = off / CODES, js = (off % CODES) / (32 / BITS);
            int qd, rho;
            wq_source(SW, js, qs, qd, rho);
            const int i = BITS == 4 ? rho : rho / 2;
            const float v[8] = {raw[u][0].x, raw[u][0].y, raw[u][0].z, raw[u][0].w,
                                raw[u][1].x, raw[u][1].y, raw[u][1].z, raw[u][1].w};
            uint32_t d3[3][4];
#pragma unroll
            for (int d = 0; d < 4; ++d) {
                // slots 2d, 2d+1: the 4-bit decode pairs nibble d with nibble d + 4
                const float e0 = BITS == 4 ? v[d] : v[2 * d], e1 = BITS == 4 ? v[d + 4] : v[2 * d + 1];
                wq_split3x2(e0, e1, d3[0][d], d3[1][d], d3[2][d]);
            }
            if (wi < nw) {
#pragma unroll
                for (int p = 0; p < 3; ++p)
                    x_lds[((wi * NI + i) * 3 + p) * 64 + wq_x_slot(ml, qd, wi * NI + i)] = uint4{d3[p][0], d3[p][1], d3[p][2], d3[p][3]};
            }
        }
    }
    __syncthreads();

    v4f y[RB];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) y[rb] = v4f{0.f, 0.f, 0.f, 0.f};
    const int row_in_tile = wave * (RB * 16) + r;
    const uint4 ones = {0x3f803f80u, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u};  // eight times 1.0
#pragma unroll
    for (int wi = 0; wi < WPS; ++wi) {
        if (wi < nw) {
            uint32_t wd[RB][4];
#pragma unroll
            for (int rb = 0; rb < RB; ++rb) {
                // lane (row r, quarter q) takes what lane 4 r + q loaded
                const int from = (4 * r + q) * 4;
                wd[rb][0] = uint32_t(__builtin_amdgcn_ds_bpermute(from, int(wv[wi][rb].x)));
                wd[rb][1] = uint32_t(__builtin_amdgcn_ds_bpermute(from, int(wv[wi][rb].y)));
                wd[rb][2] = uint32_t(__builtin_amdgcn_ds_bpermute(from, int(wv[wi][rb].z)));
                wd[rb][3] = uint32_t(__builtin_amdgcn_ds_bpermute(from, int(wv[wi][rb].w)));
                if (SW >= 1) wq_swap32(wd[rb][0], wd[rb][2]), wq_swap32(wd[rb][1], wd[rb][3]);
                if (SW == 2) wq_swap16(wd[rb][0], wd[rb][1]), wq_swap16(wd[rb][2], wd[rb][3]);
            }
#pragma unroll
            for (int e = 0; e < GW; ++e) {
                const int g = (((w0 + wi) * WK + e * SEG) >> gs_shift) - g0;
                // acc[RB]: the segment's sum of x, from the same fragments against a row of ones (every
                // column of that tile holds it: exactly the value each lane needs for its rows m)
                v4f acc[RB + 1];
#pragma unroll
                for (int rb = 0; rb <= RB; ++rb) acc[rb] = v4f{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ii = 0; ii < IPS; ++ii) {
                    const int i = e * IPS + ii;
                    uint4 cf[RB];
#pragma unroll
                    for (int rb = 0; rb < RB; ++rb) {
                        if (BITS == 4) {
                            const uint32_t c = wd[rb][i];
                            cf[rb].x = (c & 0x000f000fu) | 0x43004300u;
                            cf[rb].y = ((c >> 4) & 0x000f000fu) | 0x43004300u;
                            cf[rb].z = ((c >> 8) & 0x000f000fu) | 0x43004300u;
                            cf[rb].w = ((c >> 12) & 0x000f000fu) | 0x43004300u;
                        } else {
                            // a byte as a float has zeros below bit 16: its upper half is the bfloat16
                            const uint32_t a = wd[rb][2 * i], b = wd[rb][2 * i + 1];
                            const uint32_t a0 = __float_as_uint(float(a & 0xffu)), a1 = __float_as_uint(float((a >> 8) & 0xffu));
                            const uint32_t a2 = __float_as_uint(float((a >> 16) & 0xffu)), a3 = __float_as_uint(float(a >> 24));
                            const uint32_t b0 = __float_as_uint(float(b & 0xffu)), b1 = __float_as_uint(float((b >> 8) & 0xffu));
                            const uint32_t b2 = __float_as_uint(float((b >> 16) & 0xffu)), b3 = __float_as_uint(float(b >> 24));
                            cf[rb].x = __builtin_amdgcn_perm(a1, a0, 0x07060302u);
                            cf[rb].y = __builtin_amdgcn_perm(a3, a2, 0x07060302u);
                            cf[rb].z = __builtin_amdgcn_perm(b1, b0, 0x07060302u);
                            cf[rb].w = __builtin_amdgcn_perm(b3, b2, 0x07060302u);
                        }
                    }
#pragma unroll
                    for (int p = 0; p < 3; ++p) {
                        const v8bf xf = __builtin_bit_cast(v8bf, x_lds[((wi * NI + i) * 3 + p) * 64 + wq_x_slot(lane & 15, lane >> 4, wi * NI + i)]);
#pragma unroll
                        for (int rb = 0; rb < RB; ++rb)
                            acc[rb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xf, __builtin_bit_cast(v8bf, cf[rb]),
                                                                              acc[rb], 0, 0, 0);
                        acc[RB] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xf, __builtin_bit_cast(v8bf, ones), acc[RB], 0, 0, 0);
                    }
                }
#pragma unroll
                for (int rb = 0; rb < RB; ++rb) {
                    const float sc = s_lds[(row_in_tile + rb * 16) * gp + g];
                    const float bi = b_lds[(row_in_tile + rb * 16) * gp + g];
                    // the 4-bit codes entered as 128 + c
                    const float bz = BITS == 4 ? bi - 128.0f * sc : bi;
                    y[rb] = y[rb] + (acc[rb] * sc + acc[RB] * bz);
                }
            }
        }
    }

    // accumulator element t of a lane: row m = 4 * quarter + t, column n = lane % 16
    auto store_out = [&](const v4f (&v)[RB]) {
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
            const int n = n_base + rb * 16 + r;
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const int mm = m0 + 4 * q + t;
                if (n < N && mm < M) out[size_t(mm) * N + n] = v[rb][t];
            }
        }
    };
    if (slices == 1) {
        store_out(y);
        return;
    }
    // slab of (row tile, k range): [wavefront][tile of 16 rows][lane] x 16 bytes, written through to
    // device scope; then the arrival counter of the row tile
    constexpr unsigned kScopeDevice = 16;  // "sc1" cache-policy bit of buffer accesses
    constexpr unsigned kSlabBytes = WAVES * RB * 64 * 16;
    typedef unsigned v4u __attribute__((ext_vector_type(4)));
    const size_t tile_index = size_t(mb) * gridDim.y + tile;
    float* first_slab = slabs + tile_index * slices * (kSlabBytes / 4);
    const unsigned my_off = unsigned((wave * RB) * 64 + lane) * 16;
    {
        const __amdgpu_buffer_rsrc_t mine =
            __builtin_amdgcn_make_buffer_rsrc(first_slab + size_t(ks) * (kSlabBytes / 4), 0, kSlabBytes, 0x00020000);
#pragma unroll
        for (int rb = 0; rb < RB; ++rb)
            __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4u, y[rb]), mine, my_off + unsigned(rb * 64 * 16), 0,
                                                   kScopeDevice);
    }
    __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): this wavefront's partial sums have been written through
    __syncthreads();                      // ... and so have the other wavefronts'
    if (threadIdx.x == 0)
        s_arrived = __hip_atomic_fetch_add(&counters[tile_index], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    if (__builtin_amdgcn_readfirstlane(s_arrived) != slices - 1) return;
    v4f total[RB];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) total[rb] = v4f{0.f, 0.f, 0.f, 0.f};
    // eight slabs are requested together (one memory round trip, not eight); a slot past the
    // last slab re-reads the last one and is not added, so that the loads stay unconditional
    constexpr int kBatch = 8;
    for (int k0 = 0; k0 < slices; k0 += kBatch) {
        v4u part[kBatch][RB];
#pragma unroll
        for (int j = 0; j < kBatch; ++j) {
            const int k = k0 + j < slices ? k0 + j : slices - 1;
            const __amdgpu_buffer_rsrc_t other =
                __builtin_amdgcn_make_buffer_rsrc(first_slab + size_t(k) * (kSlabBytes / 4), 0, kSlabBytes, 0x00020000);
#pragma unroll
            for (int rb = 0; rb < RB; ++rb)
                part[j][rb] = __builtin_amdgcn_raw_buffer_load_b128(other, my_off + unsigned(rb * 64 * 16), 0, kScopeDevice);
        }
#pragma unroll
        for (int j = 0; j < kBatch; ++j)
            if (k0 + j < slices) {
#pragma unroll
                for (int rb = 0; rb < RB; ++rb) total[rb] = total[rb] + __builtin_bit_cast(v4f, part[j][rb]);
            }
    }
    store_out(total);
    if (threadIdx.x == 0) counters[tile_index] = 0;  // ready for the next launch
}


template <int BITS>
int launch_wq_mfma(const float* x, const uint32_t* packed, const float* scales, const float* biases, int M, int N,
                   int K, int gs, float* out, hipStream_t st) {
    using G = WqGeom<BITS>;
    constexpr int WPS = kWqSliceK / G::WK;
    const int sw = wq_swap_mode(BITS, gs);
    const int mblocks = (M + 15) / 16, windows = K / G::WK;
    const int tiles = (N + kWqRows - 1) / kWqRows, slices = (windows + WPS - 1) / WPS;
    SkScratch sk;
    if (slices > 1) {
        const int rc = sk_scratch(size_t(mblocks) * tiles, size_t(mblocks) * tiles * slices * (8 * 2 * 64 * 16), st, &sk);
        if (rc) return rc;
    }
    const dim3 grid{unsigned(slices), unsigned(tiles), unsigned(mblocks)};
    const int gs_shift = 31 - __builtin_clz(unsigned(gs));
    const int gmax = kWqSliceK / gs;
    const size_t lds = size_t(WPS) * G::NI * 3 * 64 * 16 + size_t(2) * kWqRows * ((gmax < 1 ? 1 : gmax) + 1) * 4;
#define LQ_WQ_LAUNCH(SWM)                                                                                         \
    do {                                                                                                          \
        static DeviceOnce attr_once;                                                                              \
        const int arc = allow_dynamic_lds(attr_once, reinterpret_cast<const void*>(wq_mfma_kernel<BITS, SWM>),    \
                                          kWqMaxLds);                                                             \
        if (arc) return arc;                                                                                      \
        hipLaunchKernelGGL((wq_mfma_kernel<BITS, SWM>), grid, dim3(512), lds, st, x, packed, scales, biases, M,   \
                           N, K, gs_shift, out, reinterpret_cast<float*>(sk.slabs), sk.counters);                 \
    } while (0)
    if (sw == 0)
        LQ_WQ_LAUNCH(0);
    else if (sw == 1)
        LQ_WQ_LAUNCH(1);
    else if constexpr (BITS == 4)
        LQ_WQ_LAUNCH(2);
#undef LQ_WQ_LAUNCH
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
