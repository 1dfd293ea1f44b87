// int8 x int8 -> int32 GEMM with a register-resident epilogue, for gfx950.
//
//   acc[m,n] = sum_k a[m,k] * w[n,k]                       (exact int32)
//   y        = f32(acc - a_zp * wsum[n]) * (a_scale[m|0] * w_scale[n]) + bias[n]
//   y        = relu(y)                                     (optional)
//   out      = acc | y (f32) | y (f16) | requantized int8 code | fake-quantized f32
//
// This is the kernel Lucid's quantized Linear promises "underneath"
// (lucid/nn/quantized/linear.py:3-9,199-215): the float formulation
// dequantize -> F.linear -> fake_quantize rewritten as its exact integer
// identity.  Three kernels:
//   tile   : 256x256x128 block tile, 4 wavefronts of 128x128, v_mfma_i32_32x32x32_i8,
//            K tiles double-buffered in LDS through direct global->LDS loads.
//   skinny : M <= 64 (decode shapes): weight rows streamed once from HBM
//            straight into v_mfma_i32_16x16x64_i8 operands, K split over the
//            block's wavefronts and reduced in LDS.
//   naive  : any shape / alignment, one output per lane.
#include "common.hpp"

using namespace lq;

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

#define LQ_GPTR(p) ((__attribute__((address_space(1))) void*)(p))
#define LQ_LPTR(p) ((__attribute__((address_space(3))) void*)(p))

enum { OUT_ACC_I32 = 0, OUT_F32 = 1, OUT_F16 = 2, OUT_REQUANT_I8 = 3, OUT_FAKEQUANT_F32 = 4 };

struct GemmArgs {
    const int8_t* a;      // [M,K] activation codes as stored
    const int8_t* w;      // [N,K] weight codes
    int M, N, K;
    const int32_t* wsum;  // [N] sum_k w[n,k]; may be null when a_zp == 0
    int a_zp;             // zero point of the stored activation codes
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
    const int8_t* zeros;  // >= 16 zero bytes, source for K-tail chunks
};

// ---------------------------------------------------------------- epilogue
struct ColParams {
    float ws, bias;
    int32_t corr;  // a_zp * wsum[n]
};

__device__ __forceinline__ ColParams load_col(const GemmArgs& g, int n) {
    ColParams c;
    c.ws = g.w_scale ? g.w_scale[n] : 1.0f;
    c.corr = (g.wsum && g.a_zp != 0) ? g.a_zp * g.wsum[n] : 0;
    if (g.bias == nullptr)
        c.bias = 0.0f;
    else if (g.bias_dtype == LQ_F16)
        c.bias = float(static_cast<const _Float16*>(g.bias)[n]);
    else
        c.bias = static_cast<const float*>(g.bias)[n];
    return c;
}

__device__ __forceinline__ float q_core(float x, float s, float z, float lo, float hi) {
    float t = x / s;
    float r = __builtin_rintf(t);
    float u = r + z;
    u = (u < lo) ? lo : ((u > hi) ? hi : u);
    return u;
}

// One output element.  Float steps are separate (no FMA) and in the order the
// CPU restatement uses, so results are bit-identical to it.
__device__ __forceinline__ void epilogue_store(const GemmArgs& g, int m, int n, int32_t acc,
                                               float as, const ColParams& c, float S, float Z) {
    const size_t idx = size_t(m) * size_t(g.ldo) + size_t(n);
    if (g.out_mode == OUT_ACC_I32) {
        static_cast<int32_t*>(g.out)[idx] = acc;
        return;
    }
    float f = float(acc - c.corr);
    float sc = as * c.ws;
    float y = f * sc;
    if (g.bias) y = y + c.bias;
    if (g.relu) y = (y < 0.0f) ? 0.0f : y;
    switch (g.out_mode) {
    case OUT_F32:
        static_cast<float*>(g.out)[idx] = y;
        break;
    case OUT_F16:
        static_cast<_Float16*>(g.out)[idx] = _Float16(y);
        break;
    case OUT_REQUANT_I8: {
        float qv = q_core(y, S, Z, float(g.out_qmin), float(g.out_qmax));
        int code = (qv != qv) ? 0 : int(qv);
        static_cast<int8_t*>(g.out)[idx] = int8_t(code + g.out_offset);
        break;
    }
    default: {  // OUT_FAKEQUANT_F32
        float qv = q_core(y, S, Z, float(g.out_qmin), float(g.out_qmax));
        static_cast<float*>(g.out)[idx] = (qv - Z) * S;
        break;
    }
    }
}

// ---------------------------------------------------------------- tile kernel
constexpr int BM = 256, BN = 256, BK = 128;
constexpr int kTileThreads = 256;
constexpr int kChunksPerRow = BK / 16;                 // 8 sixteen-byte chunks per tile row
constexpr int kStageBytes = (BM + BN) * BK;            // 64 KiB
constexpr int kTileSmem = 2 * kStageBytes;             // double buffered: 128 KiB of 160 KiB

// Blocks are handed to the 8 XCDs round-robin.  Give every XCD one contiguous
// range of logical tile ids so that the tiles sharing an L2 also share
// operand rows, then walk tiles m-fastest inside groups of 8 m-tiles.
__device__ __forceinline__ void tile_coords(int bid, int nblk, int tiles_m, int tiles_n, int* tm,
                                            int* tn) {
    const int q = nblk / 8, r = nblk % 8;
    const int xcd = bid % 8, local = bid / 8;
    const int lid = xcd * q + (xcd < r ? xcd : r) + local;
    constexpr int GM = 8;
    const int group_size = GM * tiles_n;
    const int group = lid / group_size;
    const int first_m = group * GM;
    const int gsz = tiles_m - first_m < GM ? tiles_m - first_m : GM;
    const int in_group = lid - group * group_size;
    *tm = first_m + in_group % gsz;
    *tn = in_group / gsz;
}

// LDS tile layout: row-major rows of BK bytes; the 16-byte chunk kc of row r
// sits at physical chunk kc ^ (r & 7), which makes both the 1 KiB
// wavefront-wide direct loads and the ds_read_b128 fragment reads free of
// bank conflicts.
__global__ __launch_bounds__(kTileThreads, 1) void qgemm_tile_kernel(GemmArgs g) {
    extern __shared__ __attribute__((aligned(1024))) int8_t smem[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int tiles_m = (g.M + BM - 1) / BM, tiles_n = (g.N + BN - 1) / BN;
    int tm, tn;
    tile_coords(blockIdx.x, gridDim.x, tiles_m, tiles_n, &tm, &tn);
    const int m0 = tm * BM, n0 = tn * BN;
    const int wm = wave >> 1, wn = wave & 1;  // 2 x 2 wavefronts, 128 x 128 each

    // ---- global -> LDS addressing.  Slot s = it*256 + tid holds row s/8,
    // physical chunk s%8.  (s/8) & 7 == (tid/8) & 7 for every it, so the
    // logical chunk a lane fetches is the same in all iterations.
    const int row_in_pass = tid >> 3;                      // 0..31
    const int kc = (tid & 7) ^ (row_in_pass & 7);          // logical chunk this lane fetches
    constexpr int kPasses = BM * kChunksPerRow / kTileThreads;  // 8 (BM == BN)
    unsigned a_off[kPasses], b_off[kPasses];
    const int a_rows = g.M - m0, b_rows = g.N - n0;        // valid rows in this tile (>= 1)
#pragma unroll
    for (int it = 0; it < kPasses; ++it) {
        int r = it * 32 + row_in_pass;
        int ra = r < a_rows ? r : a_rows - 1;              // clamp: reads stay in bounds,
        int rb = r < b_rows ? r : b_rows - 1;              // the rows are masked at the store
        a_off[it] = unsigned(ra) * unsigned(g.K) + unsigned(kc * 16);
        b_off[it] = unsigned(rb) * unsigned(g.K) + unsigned(kc * 16);
    }
    const int8_t* a_tile = g.a + size_t(m0) * g.K;
    const int8_t* b_tile = g.w + size_t(n0) * g.K;

    auto load_stage = [&](int k0, int8_t* stage) {
        const bool in_k = (k0 + kc * 16) < g.K;
        int8_t* sa = stage + wave * 1024;
        int8_t* sb = stage + BM * BK + wave * 1024;
#pragma unroll
        for (int it = 0; it < kPasses; ++it) {
            const int8_t* src = in_k ? a_tile + k0 + a_off[it] : g.zeros;
            __builtin_amdgcn_global_load_lds(LQ_GPTR(src), LQ_LPTR(sa + it * 4096), 16, 0, 0);
        }
#pragma unroll
        for (int it = 0; it < kPasses; ++it) {
            const int8_t* src = in_k ? b_tile + k0 + b_off[it] : g.zeros;
            __builtin_amdgcn_global_load_lds(LQ_GPTR(src), LQ_LPTR(sb + it * 4096), 16, 0, 0);
        }
    };

    v16i acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;

    // fragment addressing: lane holds row (lane & 31), 16 bytes of k at chunk
    // 2*kk + (lane >> 5) of the current 32-wide k step
    const int frag_row = lane & 31;
    const int frag_half = lane >> 5;
    const int a_row_base = (wm * 128 + frag_row) * BK;
    const int b_row_base = BM * BK + (wn * 128 + frag_row) * BK;
    const int sw = frag_row & 7;

    const int nk = (g.K + BK - 1) / BK;
    load_stage(0, smem);
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();

    for (int t = 0; t < nk; ++t) {
        int8_t* cur = smem + (t & 1) * kStageBytes;
        if (t + 1 < nk) load_stage((t + 1) * BK, smem + ((t + 1) & 1) * kStageBytes);
#pragma unroll
        for (int kk = 0; kk < BK / 32; ++kk) {
            const int pc = ((kk * 2 + frag_half) ^ sw) * 16;
            v4i af[4], bf[4];
#pragma unroll
            for (int i = 0; i < 4; ++i)
                af[i] = *reinterpret_cast<const v4i*>(cur + a_row_base + i * 32 * BK + pc);
#pragma unroll
            for (int j = 0; j < 4; ++j)
                bf[j] = *reinterpret_cast<const v4i*>(cur + b_row_base + j * 32 * BK + pc);
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[i], bf[j], acc[i][j], 0, 0, 0);
        }
        __builtin_amdgcn_s_waitcnt(0);
        __syncthreads();
    }

    // ---- epilogue.  acc[i][j][r] is row 8*(r/4) + 4*(lane>>5) + r%4, column lane&31
    float S = 1.0f, Z = 0.0f;
    if (g.out_mode == OUT_REQUANT_I8 || g.out_mode == OUT_FAKEQUANT_F32) {
        S = g.out_scale[0];
        Z = g.out_zp[0];
    }
    const float as_uniform = g.a_scale ? g.a_scale[0] : 1.0f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int n = n0 + wn * 128 + j * 32 + (lane & 31);
        if (n >= g.N) continue;
        const ColParams c = load_col(g, n);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int mb = m0 + wm * 128 + i * 32 + 4 * (lane >> 5);
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int m = mb + 8 * (r >> 2) + (r & 3);
                if (m < g.M) {
                    const float as = g.a_scale_per_row ? g.a_scale[m] : as_uniform;
                    epilogue_store(g, m, n, acc[i][j][r], as, c, S, Z);
                }
            }
        }
    }
}

// ---------------------------------------------------------------- skinny kernel
// M <= 16*MT.  A block owns 16 weight rows; its 4 wavefronts each take a
// quarter of K.  Lane (n = lane&15, g = lane>>4) reads 64 contiguous bytes of
// weight row n per 256-byte K block; the activation operand uses the same
// byte -> k mapping, so the dot products are unchanged.
template <int MT>
__global__ __launch_bounds__(256) void qgemm_skinny_kernel(GemmArgs g) {
    __shared__ int red[3][MT][4][64];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n_base = blockIdx.x * 16;
    const int ln = lane & 15, lg = lane >> 4;
    const int n = n_base + ln;
    const int nr = n < g.N ? n : g.N - 1;

    // K range of this wavefront, in 256-byte blocks; the tail block may be partial
    const int kblocks = (g.K + 255) / 256;
    const int per = (kblocks + 3) / 4;
    const int kb0 = wave * per;
    const int kb1 = kb0 + per < kblocks ? kb0 + per : kblocks;

    v4i acc[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[t] = v4i{0, 0, 0, 0};

    const int8_t* wrow = g.w + size_t(nr) * g.K;
    for (int kb = kb0; kb < kb1; ++kb) {
        const int kbase = kb * 256 + lg * 64;
        v4i wf[4];
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const int k = kbase + c * 16;
            wf[c] = k < g.K ? *reinterpret_cast<const v4i*>(wrow + k) : v4i{0, 0, 0, 0};
        }
#pragma unroll
        for (int t = 0; t < MT; ++t) {
            const int m = t * 16 + ln;
            const int8_t* arow = g.a + size_t(m < g.M ? m : g.M - 1) * g.K;
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const int k = kbase + c * 16;
                v4i af = (k < g.K && m < g.M) ? *reinterpret_cast<const v4i*>(arow + k)
                                              : v4i{0, 0, 0, 0};
                acc[t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(af, wf[c], acc[t], 0, 0, 0);
            }
        }
    }

    // reduce the four K slices (exact integer adds)
    if (wave > 0) {
#pragma unroll
        for (int t = 0; t < MT; ++t)
#pragma unroll
            for (int r = 0; r < 4; ++r) red[wave - 1][t][r][lane] = acc[t][r];
    }
    __syncthreads();
    if (wave != 0) return;
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
        for (int r = 0; r < 4; ++r)
            acc[t][r] += red[0][t][r][lane] + red[1][t][r][lane] + red[2][t][r][lane];

    if (n >= g.N) return;
    float S = 1.0f, Z = 0.0f;
    if (g.out_mode == OUT_REQUANT_I8 || g.out_mode == OUT_FAKEQUANT_F32) {
        S = g.out_scale[0];
        Z = g.out_zp[0];
    }
    const ColParams c = load_col(g, n);
    const float as_uniform = g.a_scale ? g.a_scale[0] : 1.0f;
    // acc[t][r] is row t*16 + 4*(lane>>4) + r, column lane&15
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int m = t * 16 + 4 * lg + r;
            if (m < g.M) {
                const float as = g.a_scale_per_row ? g.a_scale[m] : as_uniform;
                epilogue_store(g, m, n, acc[t][r], as, c, S, Z);
            }
        }
}

// ---------------------------------------------------------------- naive kernel
__global__ __launch_bounds__(256) void qgemm_naive_kernel(GemmArgs g) {
    const size_t total = size_t(g.M) * g.N;
    float S = 1.0f, Z = 0.0f;
    if (g.out_mode == OUT_REQUANT_I8 || g.out_mode == OUT_FAKEQUANT_F32) {
        S = g.out_scale[0];
        Z = g.out_zp[0];
    }
    for (size_t idx = size_t(blockIdx.x) * 256 + threadIdx.x; idx < total;
         idx += size_t(gridDim.x) * 256) {
        const int m = int(idx / g.N), n = int(idx % g.N);
        const int8_t* ar = g.a + size_t(m) * g.K;
        const int8_t* wr = g.w + size_t(n) * g.K;
        int32_t acc = 0;
        for (int k = 0; k < g.K; ++k) acc += int(ar[k]) * int(wr[k]);
        const float as = g.a_scale ? g.a_scale[g.a_scale_per_row ? m : 0] : 1.0f;
        epilogue_store(g, m, n, acc, as, load_col(g, n), S, Z);
    }
}

__global__ void rowsum_i8_kernel(const int8_t* __restrict__ w, int32_t* __restrict__ out, int N,
                                 int K) {
    // one wavefront per row
    const int row = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    if (row >= N) return;
    const int8_t* p = w + size_t(row) * K;
    int s = 0;
    for (int k = lane; k < K; k += 64) s += p[k];
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) s += __shfl_xor(s, d, 64);
    if (lane == 0) out[row] = s;
}

}  // namespace

// ---------------------------------------------------------------- host side
namespace lq {

// 16 zero bytes per device for K-tail chunks of the tile kernel.
int zero_block(const int8_t** ptr) {
    static void* zeros[16] = {nullptr};
    int dev = 0;
    LQ_HIP(hipGetDevice(&dev));
    LQ_REQUIRE(dev >= 0 && dev < 16, LQ_ERR_DEVICE, "device index %d out of range", dev);
    if (!zeros[dev]) {
        void* p = nullptr;
        LQ_HIP(hipMalloc(&p, 256));
        LQ_HIP(hipMemset(p, 0, 256));
        zeros[dev] = p;
    }
    *ptr = static_cast<const int8_t*>(zeros[dev]);
    return LQ_OK;
}

}  // namespace lq

extern "C" {

int lq_rowsum_i8(const int8_t* w, int32_t* out, int N, int K, lq_stream stream) {
    if (N == 0) return LQ_OK;
    LQ_REQUIRE(w && out, LQ_ERR_VALUE, "rowsum_i8: NULL pointer");
    LQ_REQUIRE(N > 0 && K >= 0, LQ_ERR_SHAPE, "rowsum_i8: bad shape (%d,%d)", N, K);
    hipLaunchKernelGGL(rowsum_i8_kernel, dim3(unsigned((N + 3) / 4)), dim3(256), 0, as_stream(stream), w,
                       out, N, K);
    LQ_CHECK_LAUNCH("rowsum_i8");
    return LQ_OK;
}

int lq_qlinear_i8(const lq_qlinear_args* p, lq_stream stream) {
    LQ_REQUIRE(p, LQ_ERR_VALUE, "qlinear_i8: args is NULL");
    LQ_REQUIRE(p->M >= 0 && p->N >= 0 && p->K >= 0, LQ_ERR_SHAPE, "qlinear_i8: negative extent");
    if (p->M == 0 || p->N == 0) return LQ_OK;
    LQ_REQUIRE(p->out, LQ_ERR_VALUE, "qlinear_i8: out is NULL");
    LQ_REQUIRE(p->K == 0 || (p->a && p->w), LQ_ERR_VALUE, "qlinear_i8: operand pointer is NULL");
    LQ_REQUIRE(p->out_mode >= OUT_ACC_I32 && p->out_mode <= OUT_FAKEQUANT_F32, LQ_ERR_VALUE,
               "qlinear_i8: unknown out_mode %d", p->out_mode);
    // |acc| <= K * 128 * 128 must stay inside int32
    LQ_REQUIRE(p->K <= 131071, LQ_ERR_SHAPE, "qlinear_i8: K = %d overflows the int32 accumulator",
               p->K);
    const long ldo = p->ldo ? p->ldo : p->N;
    LQ_REQUIRE(ldo >= p->N, LQ_ERR_SHAPE, "qlinear_i8: ldo %ld < N %d", ldo, p->N);
    if (p->out_mode != OUT_ACC_I32) {
        LQ_REQUIRE(p->w_scale && p->a_scale, LQ_ERR_VALUE, "qlinear_i8: scale pointer is NULL");
        LQ_REQUIRE(p->a_zp == 0 || p->wsum, LQ_ERR_VALUE,
                   "qlinear_i8: a_zp = %d needs the weight row sums", p->a_zp);
        LQ_REQUIRE(p->bias == nullptr || p->bias_dtype == LQ_F32 || p->bias_dtype == LQ_F16,
                   LQ_ERR_DTYPE, "qlinear_i8: bias must be float32 or float16 (dtype %d)",
                   p->bias_dtype);
    }
    if (p->out_mode == OUT_REQUANT_I8 || p->out_mode == OUT_FAKEQUANT_F32) {
        LQ_REQUIRE(p->out_scale && p->out_zp, LQ_ERR_VALUE, "qlinear_i8: output qparams are NULL");
        LQ_REQUIRE(p->out_qmin <= p->out_qmax, LQ_ERR_VALUE, "qlinear_i8: empty output grid");
        if (p->out_mode == OUT_REQUANT_I8)
            LQ_REQUIRE(p->out_qmin + p->out_offset >= -128 && p->out_qmax + p->out_offset <= 127,
                       LQ_ERR_VALUE, "qlinear_i8: output grid [%d,%d] + offset %d does not fit int8",
                       p->out_qmin, p->out_qmax, p->out_offset);
    }

    GemmArgs g;
    g.a = p->a; g.w = p->w; g.M = p->M; g.N = p->N; g.K = p->K;
    g.wsum = p->wsum; g.a_zp = p->a_zp;
    g.a_scale = p->a_scale; g.a_scale_per_row = p->a_scale_per_row; g.w_scale = p->w_scale;
    g.bias = p->bias; g.bias_dtype = p->bias_dtype; g.relu = p->relu; g.out_mode = p->out_mode;
    g.out_scale = p->out_scale; g.out_zp = p->out_zp;
    g.out_qmin = p->out_qmin; g.out_qmax = p->out_qmax; g.out_offset = p->out_offset;
    g.out = p->out; g.ldo = ldo; g.zeros = nullptr;

    hipStream_t st = as_stream(stream);
    const bool vec_ok = p->K % 16 == 0 && p->K > 0 && aligned16(p->a) && aligned16(p->w);
    int path = p->force_path;  // 0 = choose, 1 = tile, 2 = skinny, 3 = naive
    if (path == 0) path = !vec_ok ? 3 : (p->M <= 64 ? 2 : 1);
    LQ_REQUIRE(path == 3 || vec_ok, LQ_ERR_VALUE,
               "qlinear_i8: MFMA paths need K %% 16 == 0 and 16-byte aligned operands");
    if (path == 1) {
        LQ_REQUIRE(size_t(BM) * p->K < 0xffffffffull, LQ_ERR_SHAPE, "qlinear_i8: K too large");
        int rc = zero_block(&g.zeros);
        if (rc) return rc;
        static bool attr_set = false;
        if (!attr_set) {
            LQ_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(qgemm_tile_kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, kTileSmem));
            attr_set = true;
        }
        const int tiles = ((p->M + BM - 1) / BM) * ((p->N + BN - 1) / BN);
        hipLaunchKernelGGL(qgemm_tile_kernel, dim3(tiles), dim3(kTileThreads), kTileSmem, st, g);
        LQ_CHECK_LAUNCH("qgemm_tile");
    } else if (path == 2) {
        LQ_REQUIRE(p->M <= 64, LQ_ERR_SHAPE, "qlinear_i8: skinny path needs M <= 64 (M = %d)", p->M);
        dim3 grid{unsigned((p->N + 15) / 16)}, block{256};
        if (p->M <= 16)
            hipLaunchKernelGGL((qgemm_skinny_kernel<1>), grid, block, 0, st, g);
        else if (p->M <= 32)
            hipLaunchKernelGGL((qgemm_skinny_kernel<2>), grid, block, 0, st, g);
        else
            hipLaunchKernelGGL((qgemm_skinny_kernel<4>), grid, block, 0, st, g);
        LQ_CHECK_LAUNCH("qgemm_skinny");
    } else {
        size_t blocks = (size_t(p->M) * p->N + 255) / 256;
        if (blocks > 65536) blocks = 65536;
        hipLaunchKernelGGL(qgemm_naive_kernel, dim3(unsigned(blocks)), dim3(256), 0, st, g);
        LQ_CHECK_LAUNCH("qgemm_naive");
    }
    return LQ_OK;
}

}  // extern "C"
