// quantize / dequantize / fake_quantize / min-max / calculate_qparams for
// gfx950.  All of them are HBM-bound: the kernels issue 128-bit loads that a
// wavefront covers contiguously, keep several loads in flight per lane, and
// do the arithmetic in the order Lucid's CPU path does it
// (lucid/quantization/_functional.py:180, 281, 311-313): IEEE division,
// round-half-even, add zero point, clamp, cast.  No reciprocal, no FMA.
#include <mutex>
#include "common.hpp"
#include "range_slots.hpp"

using namespace lq;

namespace {

constexpr int kThreads = 256;

// Streaming access: every byte is touched once, so loads and stores carry the
// non-temporal hint and do not displace each other in L2 / Infinity Cache.
// (Measured on MI355X: 5 B/element quantize 239 us -> 207 us on 268 M elements.)
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float4 nt_load(const float4* p) {
    f32x4 v = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(p));
    return make_float4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ void nt_store(float4* p, float4 v) {
    f32x4 t = {v.x, v.y, v.z, v.w};
    __builtin_nontemporal_store(t, reinterpret_cast<f32x4*>(p));
}
__device__ __forceinline__ void nt_store(uint4* p, uint4 v) {
    u32x4 t = {v.x, v.y, v.z, v.w};
    __builtin_nontemporal_store(t, reinterpret_cast<u32x4*>(p));
}

// ---------------------------------------------------------------- element math
// clip keeps NaN (CpuBackend.h:6880-6891); the float->int cast maps NaN to 0.
__device__ __forceinline__ float q_core(float x, float s, float z, float lo, float hi) {
    float t = x / s;
    float r = __builtin_rintf(t);
    float u = r + z;
    u = (u < lo) ? lo : ((u > hi) ? hi : u);
    return u;
}

__device__ __forceinline__ int to_code(float c) { return (c != c) ? 0 : int(c); }

// rint(x / s) without dividing, bit-identical to the division.
// t0 = x * r with r = fl(1/s) is within 3 * 2^-24 * |x/s| of the correctly
// rounded quotient.  If t0 is further than that (with margin) from the nearest
// half-integer, both round to the same integer.  Otherwise - ties, near-ties,
// huge, infinite or NaN quotients - the lane redoes the IEEE division.
__device__ __forceinline__ bool rint_quotient_safe(float t0, float n) {
    const float frac = __builtin_fabsf(t0 - n);  // <= 0.5
    // false for NaN / inf t0 as well
    return (0.5f - frac) > 4.0e-7f * __builtin_fabsf(t0) && __builtin_fabsf(t0) < 4.0e6f;
}

__device__ __forceinline__ float clamp_code(float r, float z, float lo, float hi) {
    float u = r + z;
    return (u < lo) ? lo : ((u > hi) ? hi : u);
}

// four quotients at once; `r` is fl(1/s), uniform over the block
__device__ __forceinline__ float4 rint_div4(float4 v, float s, float r) {
    float4 t = {v.x * r, v.y * r, v.z * r, v.w * r};
    float4 n = {__builtin_rintf(t.x), __builtin_rintf(t.y), __builtin_rintf(t.z), __builtin_rintf(t.w)};
    // branch-free conjunction: the four tests are evaluated unconditionally
    const bool ok = (int(rint_quotient_safe(t.x, n.x)) & int(rint_quotient_safe(t.y, n.y)) &
                     int(rint_quotient_safe(t.z, n.z)) & int(rint_quotient_safe(t.w, n.w))) != 0;
    if (__builtin_expect(!ok, 0)) {
        n.x = __builtin_rintf(v.x / s);
        n.y = __builtin_rintf(v.y / s);
        n.z = __builtin_rintf(v.z / s);
        n.w = __builtin_rintf(v.w / s);
    }
    return n;
}

struct alignas(4) Code8x4 {
    int8_t v[4];
};
struct alignas(8) Code16x4 {
    int16_t v[4];
};

__device__ __forceinline__ Code8x4 nt_load(const Code8x4* p) {
    unsigned w = __builtin_nontemporal_load(reinterpret_cast<const unsigned*>(p));
    Code8x4 c;
    __builtin_memcpy(&c, &w, 4);
    return c;
}
__device__ __forceinline__ Code16x4 nt_load(const Code16x4* p) {
    u32x2 w = __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(p));
    Code16x4 c;
    __builtin_memcpy(&c, &w, 8);
    return c;
}
__device__ __forceinline__ void nt_store(Code8x4* p, Code8x4 c) {
    unsigned w;
    __builtin_memcpy(&w, &c, 4);
    __builtin_nontemporal_store(w, reinterpret_cast<unsigned*>(p));
}
__device__ __forceinline__ void nt_store(Code16x4* p, Code16x4 c) {
    u32x2 w;
    __builtin_memcpy(&w, &c, 8);
    __builtin_nontemporal_store(w, reinterpret_cast<u32x2*>(p));
}

template <typename CodeT>
struct CodeVec;
template <>
struct CodeVec<int8_t> {
    using type = Code8x4;
};
template <>
struct CodeVec<int16_t> {
    using type = Code16x4;
};

// ---------------------------------------------------------------- segment ops
// Each op works on groups of four consecutive elements ("quads") that share
// one (scale, zero_point).
template <typename CodeT>
struct QuantizeOp {
    using In = float4;
    using Vec = typename CodeVec<CodeT>::type;
    const float4* __restrict__ x;
    Vec* __restrict__ q;
    float lo, hi;
    int off;
    __device__ __forceinline__ In load(size_t i) const { return nt_load(&x[i]); }
    static constexpr int kMaxU = 2;  // loads in flight per lane; measured best for 4 B in / 1 B out
    __device__ __forceinline__ Vec pack(In v, float s, float z, float r) const {
        const float4 n = rint_div4(v, s, r);
        Vec o;
        o.v[0] = CodeT(to_code(clamp_code(n.x, z, lo, hi)) + off);
        o.v[1] = CodeT(to_code(clamp_code(n.y, z, lo, hi)) + off);
        o.v[2] = CodeT(to_code(clamp_code(n.z, z, lo, hi)) + off);
        o.v[3] = CodeT(to_code(clamp_code(n.w, z, lo, hi)) + off);
        return o;
    }
    __device__ __forceinline__ void store(size_t i, In v, float s, float z, float r) const {
        nt_store(&q[i], pack(v, s, z, r));
    }
    // scalar tail / generic path
    __device__ __forceinline__ void scalar(size_t e, float s, float z) const {
        const float* xs = reinterpret_cast<const float*>(x);
        CodeT* qs = reinterpret_cast<CodeT*>(q);
        qs[e] = CodeT(to_code(q_core(xs[e], s, z, lo, hi)) + off);
    }
};

template <typename CodeT>
struct DequantizeOp {
    using Vec = typename CodeVec<CodeT>::type;
    using In = Vec;
    static constexpr int kMaxU = 8;
    const Vec* __restrict__ q;
    float4* __restrict__ out;
    int off;
    __device__ __forceinline__ In load(size_t i) const { return nt_load(&q[i]); }
    __device__ __forceinline__ void store(size_t i, In v, float s, float z, float) const {
        float4 o;
        o.x = (float(int(v.v[0]) - off) - z) * s;
        o.y = (float(int(v.v[1]) - off) - z) * s;
        o.z = (float(int(v.v[2]) - off) - z) * s;
        o.w = (float(int(v.v[3]) - off) - z) * s;
        nt_store(&out[i], o);
    }
    __device__ __forceinline__ void scalar(size_t e, float s, float z) const {
        const CodeT* qs = reinterpret_cast<const CodeT*>(q);
        float* os = reinterpret_cast<float*>(out);
        os[e] = (float(int(qs[e]) - off) - z) * s;
    }
};

struct FakeQuantizeOp {
    using In = float4;
    static constexpr int kMaxU = 4;
    const float4* __restrict__ x;
    float4* __restrict__ out;
    float lo, hi;
    __device__ __forceinline__ In load(size_t i) const { return nt_load(&x[i]); }
    __device__ __forceinline__ void store(size_t i, In v, float s, float z, float r) const {
        const float4 n = rint_div4(v, s, r);
        float4 o;
        o.x = (clamp_code(n.x, z, lo, hi) - z) * s;
        o.y = (clamp_code(n.y, z, lo, hi) - z) * s;
        o.z = (clamp_code(n.z, z, lo, hi) - z) * s;
        o.w = (clamp_code(n.w, z, lo, hi) - z) * s;
        nt_store(&out[i], o);
    }
    __device__ __forceinline__ void scalar(size_t e, float s, float z) const {
        const float* xs = reinterpret_cast<const float*>(x);
        float* os = reinterpret_cast<float*>(out);
        os[e] = (q_core(xs[e], s, z, lo, hi) - z) * s;
    }
};

struct QParams {
    const float* scale;  // device, length C, or nullptr -> use the by-value pair
    const float* zp;
    float s_host, z_host;
};

// One block = one chunk of U*256 quads inside one [outer][C] segment, so the
// (scale, zero_point) pair is uniform across the block.  All U loads are
// issued before the first store.
template <typename Op, int U>
__global__ __launch_bounds__(kThreads) void seg_kernel(Op op, size_t inner4,
                                                       unsigned chunks_per_seg, size_t C,
                                                       QParams qp) {
    const size_t seg = blockIdx.x / chunks_per_seg;
    const unsigned chunk = blockIdx.x - unsigned(seg * chunks_per_seg);
    float s, z;
    if (qp.scale) {
        const size_t c = seg % C;
        s = qp.scale[c];
        z = qp.zp[c];
    } else {
        s = qp.s_host;
        z = qp.z_host;
    }
    const float r = 1.0f / s;  // once per lane; the per-element quotients use it under a guard
    const size_t base = seg * inner4;
    const size_t i0 = size_t(chunk) * (U * kThreads) + threadIdx.x;
    typename Op::In v[U];
    if (size_t(chunk + 1) * (U * kThreads) <= inner4) {  // whole chunk in range: no predicates
#pragma unroll
        for (int j = 0; j < U; ++j) v[j] = op.load(base + i0 + size_t(j) * kThreads);
#pragma unroll
        for (int j = 0; j < U; ++j) op.store(base + i0 + size_t(j) * kThreads, v[j], s, z, r);
        return;
    }
#pragma unroll
    for (int j = 0; j < U; ++j) {
        size_t i = i0 + size_t(j) * kThreads;
        if (i < inner4) v[j] = op.load(base + i);
    }
#pragma unroll
    for (int j = 0; j < U; ++j) {
        size_t i = i0 + size_t(j) * kThreads;
        if (i < inner4) op.store(base + i, v[j], s, z, r);
    }
}

// Any shape, any alignment: one element per thread, channel looked up per
// element.  Used for small or oddly shaped tensors (e.g. a 7x7x3 kernel).
template <typename Op>
__global__ __launch_bounds__(kThreads) void generic_kernel(Op op, size_t n, size_t C, size_t inner,
                                                           QParams qp) {
    size_t e = size_t(blockIdx.x) * kThreads + threadIdx.x;
    const size_t stride = size_t(gridDim.x) * kThreads;
    for (; e < n; e += stride) {
        float s, z;
        if (qp.scale) {
            const size_t c = (e / inner) % C;
            s = qp.scale[c];
            z = qp.zp[c];
        } else {
            s = qp.s_host;
            z = qp.z_host;
        }
        op.scalar(e, s, z);
    }
}

template <typename Op>
int launch_elementwise(Op op, size_t outer, size_t C, size_t inner, QParams qp, bool vec_ok,
                       hipStream_t st, const char* name) {
    const size_t n = outer * C * inner;
    if (n == 0) return LQ_OK;
    const size_t segs = outer * C;
    if (vec_ok && inner % 4 == 0 && inner >= 256) {
        const size_t inner4 = inner / 4;
        int U = inner4 >= 8 * kThreads ? 8 : (inner4 >= 4 * kThreads ? 4 : (inner4 >= 2 * kThreads ? 2 : 1));
        if (U > Op::kMaxU) U = Op::kMaxU;
        const size_t per_block = size_t(U) * kThreads;
        const size_t chunks = (inner4 + per_block - 1) / per_block;
        const size_t blocks = chunks * segs;
        LQ_REQUIRE(blocks <= 0x7fffffffull && chunks <= 0xffffffffull, LQ_ERR_SHAPE,
                   "%s: tensor too large for one launch (%zu blocks)", name, blocks);
        dim3 grid{unsigned(blocks)}, block{kThreads};
        switch (U) {
        case 8: hipLaunchKernelGGL((seg_kernel<Op, 8>), grid, block, 0, st, op, inner4, unsigned(chunks), C, qp); break;
        case 4: hipLaunchKernelGGL((seg_kernel<Op, 4>), grid, block, 0, st, op, inner4, unsigned(chunks), C, qp); break;
        case 2: hipLaunchKernelGGL((seg_kernel<Op, 2>), grid, block, 0, st, op, inner4, unsigned(chunks), C, qp); break;
        default: hipLaunchKernelGGL((seg_kernel<Op, 1>), grid, block, 0, st, op, inner4, unsigned(chunks), C, qp); break;
        }
    } else {
        size_t blocks = (n + kThreads - 1) / kThreads;
        if (blocks > 262144) blocks = 262144;
        hipLaunchKernelGGL((generic_kernel<Op>), dim3(unsigned(blocks)), dim3(kThreads), 0, st, op, n, C,
                           inner, qp);
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return hip_fail(e, name);
    return LQ_OK;
}

int make_qparams(const float* scale, const float* zp, int on_host, size_t C, QParams* qp,
                 const char* name) {
    LQ_REQUIRE(scale && zp, LQ_ERR_VALUE, "%s: scale / zero_point is NULL", name);
    if (on_host) {
        LQ_REQUIRE(C == 1, LQ_ERR_VALUE, "%s: host qparams are per-tensor only (C = %zu)", name, C);
        *qp = QParams{nullptr, nullptr, scale[0], zp[0]};
    } else {
        *qp = QParams{scale, zp, 0.f, 0.f};
    }
    return LQ_OK;
}

// ---------------------------------------------------------------- min / max
struct MinMax {
    float lo, hi;
    int nan;
};

__device__ __forceinline__ void mm_update(MinMax& m, float v) {
    m.nan |= (v != v);
    m.lo = fminf(m.lo, v);  // fminf/fmaxf drop NaN; the flag carries it
    m.hi = fmaxf(m.hi, v);
}

__device__ __forceinline__ MinMax mm_block_reduce(MinMax m) {
    // wavefront (64 lanes) butterfly, then across the block's waves via LDS
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) {
        m.lo = fminf(m.lo, __shfl_xor(m.lo, d, 64));
        m.hi = fmaxf(m.hi, __shfl_xor(m.hi, d, 64));
        m.nan |= __shfl_xor(m.nan, d, 64);
    }
    __shared__ float s_lo[16], s_hi[16];  // up to 1024 threads
    __shared__ int s_nan[16];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int nwaves = (blockDim.x + 63) >> 6;
    if (lane == 0) {
        s_lo[wave] = m.lo;
        s_hi[wave] = m.hi;
        s_nan[wave] = m.nan;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < nwaves; ++w) {
            m.lo = fminf(m.lo, s_lo[w]);
            m.hi = fmaxf(m.hi, s_hi[w]);
            m.nan |= s_nan[w];
        }
    }
    return m;
}

__device__ __forceinline__ void mm_write(MinMax m, float* mn, float* mx, size_t idx) {
    const float qnan = __builtin_nanf("");
    mn[idx] = m.nan ? qnan : m.lo;
    mx[idx] = m.nan ? qnan : m.hi;
}

// Channel elements lie in `outer` contiguous runs of `inner`.  Block
// (c, split) scans its slice of every run.  Partials are laid out
// [split][c]; with splits == 1 they are the final answer.
template <bool VEC>
__global__ __launch_bounds__(kThreads) void minmax_seg_kernel(const float* __restrict__ x,
                                                              size_t outer, size_t C, size_t inner,
                                                              unsigned splits, float* pmin,
                                                              float* pmax) {
    const size_t c = blockIdx.x / splits;
    const unsigned sp = blockIdx.x - unsigned(c * splits);
    MinMax m{__builtin_inff(), -__builtin_inff(), 0};
    if (VEC) {
        const size_t inner4 = inner / 4;
        const size_t per = (inner4 + splits - 1) / splits;
        const size_t lo4 = size_t(sp) * per;
        const size_t hi4 = lo4 + per < inner4 ? lo4 + per : inner4;
        for (size_t o = 0; o < outer; ++o) {
            const float4* p = reinterpret_cast<const float4*>(x + (o * C + c) * inner);
            size_t i = lo4 + threadIdx.x;
            // four independent loads in flight per lane
            for (; i + 3 * kThreads < hi4; i += 4 * kThreads) {
                float4 a = nt_load(&p[i]), b = nt_load(&p[i + kThreads]), d = nt_load(&p[i + 2 * kThreads]),
                       e = nt_load(&p[i + 3 * kThreads]);
                mm_update(m, a.x); mm_update(m, a.y); mm_update(m, a.z); mm_update(m, a.w);
                mm_update(m, b.x); mm_update(m, b.y); mm_update(m, b.z); mm_update(m, b.w);
                mm_update(m, d.x); mm_update(m, d.y); mm_update(m, d.z); mm_update(m, d.w);
                mm_update(m, e.x); mm_update(m, e.y); mm_update(m, e.z); mm_update(m, e.w);
            }
            for (; i < hi4; i += kThreads) {
                float4 a = nt_load(&p[i]);
                mm_update(m, a.x); mm_update(m, a.y); mm_update(m, a.z); mm_update(m, a.w);
            }
        }
    } else {
        const size_t per = (inner + splits - 1) / splits;
        const size_t lo = size_t(sp) * per;
        const size_t hi = lo + per < inner ? lo + per : inner;
        for (size_t o = 0; o < outer; ++o) {
            const float* p = x + (o * C + c) * inner;
            for (size_t i = lo + threadIdx.x; i < hi; i += kThreads) mm_update(m, p[i]);
        }
    }
    m = mm_block_reduce(m);
    if (threadIdx.x == 0) mm_write(m, pmin, pmax, size_t(sp) * C + c);
}

// Short runs (inner < 64, e.g. a channel-last tensor): view x as
// [outer][C*inner]; a thread owns one column and walks down a slice of rows,
// so a wavefront reads contiguous memory.  Partials [split][C*inner].
__global__ __launch_bounds__(kThreads) void minmax_col_kernel(const float* __restrict__ x,
                                                              size_t outer, size_t cols,
                                                              unsigned splits, float* pmin,
                                                              float* pmax) {
    const size_t col = size_t(blockIdx.x) * kThreads + threadIdx.x;
    const unsigned sp = blockIdx.y;
    if (col >= cols) return;
    const size_t per = (outer + splits - 1) / splits;
    const size_t lo = size_t(sp) * per;
    const size_t hi = lo + per < outer ? lo + per : outer;
    MinMax m{__builtin_inff(), -__builtin_inff(), 0};
    for (size_t r = lo; r < hi; ++r) mm_update(m, x[r * cols + col]);
    mm_write(m, pmin, pmax, size_t(sp) * cols + col);
}

// Folds partials [groups][C][inner_cols] into mn[C], mx[C]; one block per
// channel, four independent loads per thread in flight.
__global__ __launch_bounds__(256) void minmax_finalize_kernel(const float* __restrict__ pmin,
                                                              const float* __restrict__ pmax,
                                                              size_t C, unsigned groups,
                                                              unsigned inner_cols, float* mn,
                                                              float* mx) {
    const size_t c = blockIdx.x;
    MinMax m{__builtin_inff(), -__builtin_inff(), 0};
    const size_t per_c = size_t(groups) * inner_cols;
    for (size_t t0 = threadIdx.x; t0 < per_c; t0 += 4 * 256) {
        float a[4], b[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const size_t t = t0 + size_t(u) * 256;
            a[u] = __builtin_inff(), b[u] = -__builtin_inff();
            if (t < per_c) {
                const size_t g = t / inner_cols, i = t - g * inner_cols;
                const size_t idx = (g * C + c) * inner_cols + i;
                a[u] = pmin[idx], b[u] = pmax[idx];
            }
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            m.nan |= (a[u] != a[u]) | (b[u] != b[u]);
            m.lo = fminf(m.lo, a[u]);
            m.hi = fmaxf(m.hi, b[u]);
        }
    }
    m = mm_block_reduce(m);
    if (threadIdx.x == 0) mm_write(m, mn, mx, c);
}

__global__ void minmax_identity_kernel(float* mn, float* mx, size_t C) {
    size_t c = size_t(blockIdx.x) * blockDim.x + threadIdx.x;
    if (c < C) {
        mn[c] = __builtin_inff();
        mx[c] = -__builtin_inff();
    }
}

// ---------------------------------------------------------------- qparams
// vDSP_vmax / vDSP_vmin single precision propagate NaN (Vdsp.cpp:140-151).
__device__ __forceinline__ float vmaxf(float a, float b) {
    if (a != a || b != b) return __builtin_nanf("");
    return a > b ? a : b;
}
__device__ __forceinline__ float vminf(float a, float b) {
    if (a != a || b != b) return __builtin_nanf("");
    return a < b ? a : b;
}

// lucid/quantization/_qparams.py:198-215, float32 throughout.
__device__ __forceinline__ void qparams_of(float mn, float mx, int symmetric, int qmin, int qmax,
                                           int is_signed, float eps, float half_range, float* scale,
                                           float* zp) {
    float lo = vminf(mn, 0.0f);
    float hi = vmaxf(mx, 0.0f);
    if (symmetric) {
        float max_abs = vmaxf(fabsf(lo), fabsf(hi));
        *scale = vmaxf(max_abs / half_range, eps);
        *zp = is_signed ? 0.0f : float((qmax + qmin + 1) >> 1);
    } else {
        float s = vmaxf((hi - lo) / float(qmax - qmin), eps);
        float z = float(qmin) - __builtin_rintf(lo / s);
        float qlo = float(qmin), qhi = float(qmax);
        z = (z < qlo) ? qlo : ((z > qhi) ? qhi : z);
        *scale = s;
        *zp = z;
    }
}

__global__ void calc_qparams_kernel(const float* __restrict__ mn, const float* __restrict__ mx,
                                    size_t C, int symmetric, int qmin, int qmax, int is_signed,
                                    float eps, float half_range, float* scale, float* zp) {
    size_t c = size_t(blockIdx.x) * blockDim.x + threadIdx.x;
    if (c >= C) return;
    qparams_of(mn[c], mx[c], symmetric, qmin, qmax, is_signed, eps, half_range, &scale[c], &zp[c]);
}

// Per-tensor qparams from a range kept by the producing kernel (one block):
// reduce the partial slots, then calculate_qparams; also writes the range
// itself when asked.
__global__ __launch_bounds__(1024) void calc_qparams_from_range_kernel(const float* __restrict__ range,
                                                                        int symmetric, int qmin, int qmax,
                                                                        int is_signed, float eps,
                                                                        float half_range, float* scale,
                                                                        float* zp, float* mn_out,
                                                                        float* mx_out) {
    const unsigned n = reinterpret_cast<const unsigned*>(range)[0];
    MinMax m{__builtin_inff(), -__builtin_inff(), 0};
    for (unsigned i = threadIdx.x; i < n; i += 1024) {
        const float a = range[4 + i], b = range[4 + kRangeSlots + i];
        m.nan |= (a != a) | (b != b);
        m.lo = fminf(m.lo, a);
        m.hi = fmaxf(m.hi, b);
    }
    m = mm_block_reduce(m);
    if (threadIdx.x == 0) {
        float mn = m.lo, mx = m.hi;
        if (m.nan) mn = mx = __builtin_nanf("");
        if (mn_out) *mn_out = mn;
        if (mx_out) *mx_out = mx;
        qparams_of(mn, mx, symmetric, qmin, qmax, is_signed, eps, half_range, scale, zp);
    }
}

// Dynamic per-row quantization in one pass over x: a block holds one row in registers, takes
// its min / max (observer.py:634-653 with ch_axis = 0), turns them into the row's qparams
// (qparams_of) and writes the row's codes with QuantizeOp's arithmetic - the three separate
// launches' results, bit for bit, with x read once instead of twice.
template <int R>  // float4 per lane: rows of up to 1024 * R floats
__global__ __launch_bounds__(256) void quantize_rows_dynamic_kernel(
    const float4* __restrict__ x, int quads, int symmetric, int qmin, int qmax, int is_signed, float eps,
    float half_range, int off, float* __restrict__ scale, float* __restrict__ zp, float* __restrict__ mn_out,
    float* __restrict__ mx_out, Code8x4* __restrict__ q) {
    __shared__ float s_sz[2];
    const size_t row = blockIdx.x;
    const float4* xr = x + row * size_t(quads);
    float4 v[R];
    MinMax m{__builtin_inff(), -__builtin_inff(), 0};
#pragma unroll
    for (int u = 0; u < R; ++u) {
        const int i = u * 256 + int(threadIdx.x);
        if (i < quads) {
            v[u] = nt_load(&xr[i]);
            mm_update(m, v[u].x), mm_update(m, v[u].y), mm_update(m, v[u].z), mm_update(m, v[u].w);
        }
    }
    m = mm_block_reduce(m);
    if (threadIdx.x == 0) {
        const float qnan = __builtin_nanf("");
        const float mn = m.nan ? qnan : m.lo, mx = m.nan ? qnan : m.hi;
        float s, z;
        qparams_of(mn, mx, symmetric, qmin, qmax, is_signed, eps, half_range, &s, &z);
        scale[row] = s, zp[row] = z;
        if (mn_out) mn_out[row] = mn;
        if (mx_out) mx_out[row] = mx;
        s_sz[0] = s, s_sz[1] = z;
    }
    __syncthreads();
    const float s = s_sz[0], z = s_sz[1], r = 1.0f / s;
    const QuantizeOp<int8_t> op{nullptr, nullptr, float(double(qmin)), float(double(qmax)), off};
    Code8x4* qr = q + row * size_t(quads);
#pragma unroll
    for (int u = 0; u < R; ++u) {
        const int i = u * 256 + int(threadIdx.x);
        if (i < quads) nt_store(&qr[i], op.pack(v[u], s, z, r));
    }
}

// Dynamic per-tensor quantization of a small tensor in one launch (one block): global
// min / max (observer.py:363-375), qparams, codes.  Up to 16 float4 per lane (65536
// elements) stay in registers between the two phases, all their loads in flight at once;
// beyond that the block works in batches of 8 and re-reads x (from the L2) for the codes.
__global__ __launch_bounds__(1024) void quantize_tensor_dynamic_kernel(
    const float* __restrict__ x, size_t n, int symmetric, int qmin, int qmax, int is_signed, float eps,
    float half_range, int off, float* __restrict__ scale, float* __restrict__ zp, float* __restrict__ mn_out,
    float* __restrict__ mx_out, int8_t* __restrict__ q) {
    __shared__ float s_sz[2];
    constexpr int kKeep = 16, kBatch = 8;
    const bool vec = aligned16(x) && (reinterpret_cast<uintptr_t>(q) & 3u) == 0;
    const size_t quads = vec ? n / 4 : 0;
    const bool keep = quads <= size_t(kKeep) * 1024;
    const float4* x4 = reinterpret_cast<const float4*>(x);
    MinMax m{__builtin_inff(), -__builtin_inff(), 0};
    float4 v[kKeep];
    if (keep) {
#pragma unroll
        for (int u = 0; u < kKeep; ++u) {
            const size_t i = size_t(u) * 1024 + threadIdx.x;
            if (i < quads) v[u] = x4[i];
        }
#pragma unroll
        for (int u = 0; u < kKeep; ++u)
            if (size_t(u) * 1024 + threadIdx.x < quads)
                mm_update(m, v[u].x), mm_update(m, v[u].y), mm_update(m, v[u].z), mm_update(m, v[u].w);
    } else {
        for (size_t i0 = 0; i0 < quads; i0 += size_t(kBatch) * 1024) {
            float4 w[kBatch];
#pragma unroll
            for (int u = 0; u < kBatch; ++u) {
                const size_t i = i0 + size_t(u) * 1024 + threadIdx.x;
                if (i < quads) w[u] = x4[i];
            }
#pragma unroll
            for (int u = 0; u < kBatch; ++u)
                if (i0 + size_t(u) * 1024 + threadIdx.x < quads)
                    mm_update(m, w[u].x), mm_update(m, w[u].y), mm_update(m, w[u].z), mm_update(m, w[u].w);
        }
    }
    for (size_t e = quads * 4 + threadIdx.x; e < n; e += 1024) mm_update(m, x[e]);
    m = mm_block_reduce(m);
    if (threadIdx.x == 0) {
        const float qnan = __builtin_nanf("");
        const float mn = m.nan ? qnan : m.lo, mx = m.nan ? qnan : m.hi;
        float s, z;
        qparams_of(mn, mx, symmetric, qmin, qmax, is_signed, eps, half_range, &s, &z);
        *scale = s, *zp = z;
        if (mn_out) *mn_out = mn;
        if (mx_out) *mx_out = mx;
        s_sz[0] = s, s_sz[1] = z;
    }
    __syncthreads();
    const float s = s_sz[0], z = s_sz[1], r = 1.0f / s;
    const QuantizeOp<int8_t> op{x4, reinterpret_cast<Code8x4*>(q), float(double(qmin)), float(double(qmax)), off};
    if (keep) {
#pragma unroll
        for (int u = 0; u < kKeep; ++u) {
            const size_t i = size_t(u) * 1024 + threadIdx.x;
            if (i < quads) op.q[i] = op.pack(v[u], s, z, r);
        }
    } else {
        for (size_t i0 = 0; i0 < quads; i0 += size_t(kBatch) * 1024) {
            float4 w[kBatch];
#pragma unroll
            for (int u = 0; u < kBatch; ++u) {
                const size_t i = i0 + size_t(u) * 1024 + threadIdx.x;
                if (i < quads) w[u] = x4[i];
            }
#pragma unroll
            for (int u = 0; u < kBatch; ++u) {
                const size_t i = i0 + size_t(u) * 1024 + threadIdx.x;
                if (i < quads) op.q[i] = op.pack(w[u], s, z, r);
            }
        }
    }
    for (size_t e = quads * 4 + threadIdx.x; e < n; e += 1024) op.scalar(e, s, z);
}


// ---------------------------------------------------------------- static scratch (no-allocation entry point)
// lq_minmax_noalloc keeps the partial results of its two-stage reduction here instead of in
// the library's growable workspace, so that the call allocates nothing.  Each GPU holds its
// own copy of the array at its own address; the name below is only the host-side handle of
// the symbol, the device address comes from hipGetSymbolAddress, once per device.
constexpr size_t kNoAllocScratchBytes = size_t(1) << 20;
__device__ __align__(256) unsigned char scratch[kNoAllocScratchBytes];
void* g_scratch_ptr[16] = {nullptr};
std::mutex g_scratch_mutex;

int noalloc_scratch_ptr(void** out) {
    int dev = 0;
    LQ_HIP(hipGetDevice(&dev));
    LQ_REQUIRE(dev >= 0 && dev < 16, LQ_ERR_DEVICE, "device index %d out of range", dev);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        LQ_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        LQ_REQUIRE(p != nullptr, LQ_ERR_INTERNAL, "hipGetSymbolAddress returned a null address for the static scratch");
        g_scratch_ptr[dev] = p;
    }
    *out = g_scratch_ptr[dev];
    return LQ_OK;
}

// min / max launch sequence shared by lq_minmax and lq_minmax_noalloc.  `get_ws(nbytes, &ptr)`
// supplies the memory for the partial results of a two-stage reduction; `ws_limit` is the
// most it can supply: the number of slices per channel is cut down to fit (the result does
// not depend on it: min and max are exact in any order).
template <class GetWs>
int minmax_launch(const float* x, size_t outer, size_t C, size_t inner, float* mn, float* mx, hipStream_t st,
                  size_t ws_limit, GetWs get_ws) {
    LQ_REQUIRE(mn && mx, LQ_ERR_VALUE, "minmax: output pointer is NULL");
    LQ_REQUIRE(C >= 1, LQ_ERR_SHAPE, "minmax: C must be >= 1");
    const size_t per_channel = outer * inner;
    if (per_channel == 0) {  // empty reduction: identities (Reduce.cpp:95,107)
        hipLaunchKernelGGL(minmax_identity_kernel, dim3(unsigned((C + 255) / 256)), dim3(256), 0, st, mn,
                           mx, C);
        LQ_CHECK_LAUNCH("minmax_identity");
        return LQ_OK;
    }
    LQ_REQUIRE(x, LQ_ERR_VALUE, "minmax: x is NULL");
    LQ_REQUIRE(C <= 0x3fffffffull, LQ_ERR_SHAPE, "minmax: too many channels (%zu)", C);

    if (inner < 64 && C > 1) {
        const size_t cols = C * inner;
        // enough row slices to occupy the chip, at least 32 rows each
        size_t col_blocks = (cols + kThreads - 1) / kThreads;
        size_t splits = 2048 / col_blocks;
        if (splits > outer / 32) splits = outer / 32;
        if (splits < 1) splits = 1;
        if (splits > 65535) splits = 65535;
        LQ_REQUIRE(2 * cols * sizeof(float) <= ws_limit, LQ_ERR_SHAPE,
                   "minmax: %zu channel-inner columns need %zu bytes of partial results, more than the %zu available",
                   cols, 2 * cols * sizeof(float), ws_limit);
        if (splits > ws_limit / (2 * cols * sizeof(float))) splits = ws_limit / (2 * cols * sizeof(float));
        void* ws = nullptr;
        int rc = get_ws(2 * splits * cols * sizeof(float), &ws);
        if (rc) return rc;
        float* pmin = static_cast<float*>(ws);
        float* pmax = pmin + splits * cols;
        hipLaunchKernelGGL(minmax_col_kernel, dim3(unsigned(col_blocks), unsigned(splits)),
                           dim3(kThreads), 0, st, x, outer, cols, unsigned(splits), pmin, pmax);
        LQ_CHECK_LAUNCH("minmax_col");
        hipLaunchKernelGGL(minmax_finalize_kernel, dim3(unsigned(C)), dim3(256), 0, st, pmin, pmax, C,
                           unsigned(splits), unsigned(inner), mn, mx);
        LQ_CHECK_LAUNCH("minmax_finalize");
        return LQ_OK;
    }

    // contiguous runs: aim for ~2048 blocks, each slice at least 4096 elements
    size_t splits = 1;
    if (C < 2048) {
        splits = 2048 / C;
        size_t max_splits = inner / 4096;
        if (splits > max_splits) splits = max_splits;
        if (splits < 1) splits = 1;
    }
    const bool vec = (inner % 4 == 0) && aligned16(x);
    float *pmin = mn, *pmax = mx;
    if (splits > ws_limit / (2 * C * sizeof(float))) splits = ws_limit / (2 * C * sizeof(float));
    if (splits < 1) splits = 1;  // one block per channel writes mn / mx directly: no partials at all
    if (splits > 1) {
        void* ws = nullptr;
        int rc = get_ws(2 * splits * C * sizeof(float), &ws);
        if (rc) return rc;
        pmin = static_cast<float*>(ws);
        pmax = pmin + splits * C;
    }
    dim3 grid{unsigned(C * splits)}, block{kThreads};
    if (vec)
        hipLaunchKernelGGL((minmax_seg_kernel<true>), grid, block, 0, st, x, outer, C, inner,
                           unsigned(splits), pmin, pmax);
    else
        hipLaunchKernelGGL((minmax_seg_kernel<false>), grid, block, 0, st, x, outer, C, inner,
                           unsigned(splits), pmin, pmax);
    LQ_CHECK_LAUNCH("minmax_seg");
    if (splits > 1) {
        hipLaunchKernelGGL(minmax_finalize_kernel, dim3(unsigned(C)), dim3(256), 0, st, pmin, pmax, C,
                           unsigned(splits), 1u, mn, mx);
        LQ_CHECK_LAUNCH("minmax_finalize");
    }
    return LQ_OK;
}

// A whole dynamic-quantized Linear on a small activation in one launch
// (lucid/nn/quantized/dynamic/linear.py:87-99: x.min() / x.max(), calculate_qparams, quantize,
// dequantize-free integer GEMM, bias): every block takes the tensor's min / max and qparams and
// quantizes x into LDS itself - x is at most 65536 floats, so repeating that per block costs less
// than a separate launch and its round trip - but only its own 16 rows, and then computes a
// 16 x 16 block of the output: its 16 wavefronts split the k steps of v_mfma_i32_16x16x64_i8 (activation fragments from the LDS codes,
// weight rows from global memory), meet through LDS atomics, and one lane per output applies
// float(acc - zp * wsum[n]) * (s * w_scale[n]) + bias[n] (and the optional ReLU) in the order of
// the GEMM's epilogue.  Same bits as lq_quantize_tensor_dynamic_i8 followed by lq_qlinear_i8.
__global__ __launch_bounds__(1024) void dynamic_linear_small_kernel(
    const float* __restrict__ x, int M, int K, const int8_t* __restrict__ w, int N, const float* __restrict__ w_scale,
    const int32_t* __restrict__ wsum, const float* __restrict__ bias, int relu, int symmetric, int qmin, int qmax,
    int is_signed, float eps, float half_range, int off, float* __restrict__ out) {
    extern __shared__ __attribute__((aligned(16))) int8_t dl_smem[];
    __shared__ float s_sz[2];
    typedef int dl_v4i __attribute__((ext_vector_type(4)));
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    int8_t* const codes = dl_smem;                                     // [16][K]: the block's rows
    int* const red = reinterpret_cast<int*>(dl_smem + size_t(16) * K);  // [4][64]
    constexpr int kKeep = 16;
    const int quads = (M * K) >> 2;
    const float4* x4 = reinterpret_cast<const float4*>(x);
    // What does not depend on x is requested first, so that it arrives under the quantization: the
    // wavefront's first weight fragment and the output lane's column parameters.
    const int n0 = blockIdx.x * 16, m0 = blockIdx.y * 16;
    const int ln = lane & 15, lg = lane >> 4;
    // (requested with lane = 4 * row + chunk, so that four neighbouring lanes read 64 contiguous bytes,
    // and handed to the lane that multiplies it - row lane % 16, chunk lane / 16 - by dl_place)
    const int rq = lane >> 2, cq = lane & 3;
    const int8_t* wrow = w + size_t(n0 + rq < N ? n0 + rq : N - 1) * size_t(K);
    auto dl_place = [&](dl_v4i f) {
        const int from = (4 * ln + lg) * 4;
        return dl_v4i{__builtin_amdgcn_ds_bpermute(from, f[0]), __builtin_amdgcn_ds_bpermute(from, f[1]),
                      __builtin_amdgcn_ds_bpermute(from, f[2]), __builtin_amdgcn_ds_bpermute(from, f[3])};
    };
    const int ksteps = (K + 63) >> 6;
    const bool first_in_k = wave < ksteps && wave * 64 + cq * 16 < K;
    const dl_v4i wf_first = first_in_k ? *reinterpret_cast<const dl_v4i*>(wrow + wave * 64 + cq * 16) : dl_v4i{0, 0, 0, 0};
    const int out_n = n0 + (tid & 15);
    const bool out_lane = tid < 256 && out_n < N;
    const float c_ws = (out_lane && w_scale) ? w_scale[out_n] : 1.0f;
    const int c_wsum = (out_lane && wsum) ? wsum[out_n] : 0;
    const float c_bias = (out_lane && bias) ? bias[out_n] : -0.0f;
    MinMax m{__builtin_inff(), -__builtin_inff(), 0};
    float4 v[kKeep];
#pragma unroll
    for (int u = 0; u < kKeep; ++u) {
        const int i = u * 1024 + tid;
        if (i < quads) v[u] = x4[i];
    }
    if (tid < 256) red[tid] = 0;
    // the block's rows m0 .. m0+15 are a contiguous range of quads; rows past M (the last block's padding)
    // feed accumulator rows that are never stored
    const int q_lo = (m0 * K) >> 2;
    const int q_hi = ((m0 + 16 < M ? m0 + 16 : M) * K) >> 2;
    for (int i = q_hi - q_lo + tid; i < 4 * K; i += 1024) reinterpret_cast<unsigned*>(codes)[i] = 0u;
#pragma unroll
    for (int u = 0; u < kKeep; ++u)
        if (u * 1024 + tid < quads) mm_update(m, v[u].x), mm_update(m, v[u].y), mm_update(m, v[u].z), mm_update(m, v[u].w);
    m = mm_block_reduce(m);
    if (tid == 0) {
        const float qnan = __builtin_nanf("");
        float s, z;
        qparams_of(m.nan ? qnan : m.lo, m.nan ? qnan : m.hi, symmetric, qmin, qmax, is_signed, eps, half_range, &s, &z);
        s_sz[0] = s, s_sz[1] = z;
    }
    __syncthreads();
    const float s = s_sz[0], z = s_sz[1], r = 1.0f / s;
    const QuantizeOp<int8_t> op{x4, reinterpret_cast<Code8x4*>(codes), float(double(qmin)), float(double(qmax)), off};
#pragma unroll
    for (int u = 0; u < kKeep; ++u) {
        const int i = u * 1024 + tid;
        if (i >= q_lo && i < q_hi) op.q[i - q_lo] = op.pack(v[u], s, z, r);
    }
    __syncthreads();

    dl_v4i acc = dl_v4i{0, 0, 0, 0};
    for (int ks = wave; ks < ksteps; ks += 16) {
        const int k = ks * 64 + lg * 16;
        const bool in_k = k < K;  // K % 16 == 0: a 16-byte chunk is inside or outside as a whole
        const int kq = ks * 64 + cq * 16;
        const dl_v4i wf = dl_place(ks == wave ? wf_first
                                              : (kq < K ? *reinterpret_cast<const dl_v4i*>(wrow + kq) : dl_v4i{0, 0, 0, 0}));
        const dl_v4i af = in_k ? *reinterpret_cast<const dl_v4i*>(codes + size_t(ln) * K + k) : dl_v4i{0, 0, 0, 0};
        acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(af, wf, acc, 0, 0, 0);
    }
    if (wave < ksteps) {
#pragma unroll
        for (int q = 0; q < 4; ++q)
            __hip_atomic_fetch_add(&red[q * 64 + lane], acc[q], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
    __syncthreads();
    // red[q * 64 + lane]: activation row m0 + 4 (lane / 16) + q, weight row n0 + lane % 16
    if (tid < 256) {
        const int q = tid >> 6, l = tid & 63;
        const int mm = m0 + 4 * (l >> 4) + q, nn = n0 + (l & 15);
        if (mm < M && nn < N) {
            // GEMM epilogue, float32 output form: the zero point enters as an integer, the steps stay separate
            const int zp = int(z) + off;
            const int corr = (wsum != nullptr && zp != 0) ? zp * c_wsum : 0;
            const float f = float(red[tid] - corr);
            const float sc = s * c_ws;
            float y = f * sc;
            y = y + c_bias;
            const float floor = relu ? 0.0f : -__builtin_inff();
            y = (y < floor) ? floor : y;
            out[size_t(mm) * N + nn] = y;
        }
    }
}

// Two dynamic-quantized Linears with an optional ReLU after each, on a small activation, in ONE
// launch (the MLP Linear(784,256) -> ReLU -> Linear(256,10) at batch 64 is 0.43 MOP: three
// launches cost three round trips).  Layer 1 runs exactly as dynamic_linear_small_kernel runs it -
// a block per 16 x 16 tile of the hidden activation, so the 50 k inputs are quantized by 64 CUs
// at once - with each block's tile (ReLU applied) and its min / max written through to device
// scope; the block that arrives last (one counter, at most 64 arrivals) then owns the whole
// hidden activation - 64 KB, one round trip - and does for layer 2 what the separate operators
// do: the tensor's min / max (from the tiles'), calculate_qparams, the codes, the integer GEMM
// (one wavefront per 16 x 16 output tile), float(acc - zp * wsum[n]) * (s * w_scale[n]) + bias[n],
// ReLU.  Same bits as two lq_dynamic_linear_small_f32 calls (the ReLU between them folded into
// the first).  15.7 us for that MLP; with ONE block doing both layers it was 21 us (one CU's
// vector units quantized all 50 k inputs).  `hid`: [M][N1] float32, then 64 minima and 64 maxima;
// `counter`: zero between launches (the last block resets it).
__global__ __launch_bounds__(1024) void dynamic_mlp2_blocks_kernel(
    const float* __restrict__ x, int M, int K1, const int8_t* __restrict__ w1, int N1, const float* __restrict__ ws1,
    const int32_t* __restrict__ wsum1, const float* __restrict__ b1, int relu1, const int8_t* __restrict__ w2, int N2,
    const float* __restrict__ ws2, const int32_t* __restrict__ wsum2, const float* __restrict__ b2, int relu2,
    int symmetric, int qmin, int qmax, int is_signed, float eps, float half_range, int off, float* __restrict__ out,
    float* hid, int* counter) {
    extern __shared__ __attribute__((aligned(16))) int8_t mb_smem[];
    __shared__ float s_sz[4];
    __shared__ int s_arrived;
    typedef int mb_v4i __attribute__((ext_vector_type(4)));
    typedef unsigned mb_v4u __attribute__((ext_vector_type(4)));
    constexpr unsigned kScopeDevice = 16;  // "sc1" cache-policy bit of buffer accesses
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    int8_t* const codes = mb_smem;                                      // [16][K1]: the block's rows
    int* const red = reinterpret_cast<int*>(mb_smem + size_t(16) * K1);  // [4][64]
    int8_t* const codes2 = mb_smem + size_t(16) * K1 + 1024;             // [64][N1]: the last block's
    constexpr int kKeep = 16;
    const float qnan = __builtin_nanf("");
    const int quads = (M * K1) >> 2;
    const float4* x4 = reinterpret_cast<const float4*>(x);
    const int n0 = blockIdx.x * 16, m0 = blockIdx.y * 16;
    const int nblocks = gridDim.x * gridDim.y, bid = blockIdx.y * gridDim.x + blockIdx.x;
    const int ln = lane & 15, lg = lane >> 4;
    const int rq = lane >> 2, cq = lane & 3;
    const int8_t* wrow = w1 + size_t(n0 + rq < N1 ? n0 + rq : N1 - 1) * size_t(K1);
    auto place = [&](mb_v4i f) {
        const int from = (4 * ln + lg) * 4;
        return mb_v4i{__builtin_amdgcn_ds_bpermute(from, f[0]), __builtin_amdgcn_ds_bpermute(from, f[1]),
                      __builtin_amdgcn_ds_bpermute(from, f[2]), __builtin_amdgcn_ds_bpermute(from, f[3])};
    };
    const size_t hid_bytes = size_t(M) * N1 * 4;
    const __amdgpu_buffer_rsrc_t hbuf = __builtin_amdgcn_make_buffer_rsrc(hid, 0, int(hid_bytes) + 512, 0x00020000);
    const int ksteps = (K1 + 63) >> 6;
    const bool first_in_k = wave < ksteps && wave * 64 + cq * 16 < K1;
    const mb_v4i wf_first = first_in_k ? *reinterpret_cast<const mb_v4i*>(wrow + wave * 64 + cq * 16) : mb_v4i{0, 0, 0, 0};
    const int out_n = n0 + (tid & 15);
    const bool out_lane = tid < 256 && out_n < N1;
    const float c_ws = (out_lane && ws1) ? ws1[out_n] : 1.0f;
    const int c_wsum = (out_lane && wsum1) ? wsum1[out_n] : 0;
    const float c_bias = (out_lane && b1) ? b1[out_n] : -0.0f;
    MinMax m{__builtin_inff(), -__builtin_inff(), 0};
    float4 v[kKeep];
#pragma unroll
    for (int u = 0; u < kKeep; ++u) {
        const int i = u * 1024 + tid;
        if (i < quads) v[u] = x4[i];
    }
    if (tid < 256) red[tid] = 0;
    const int q_lo = (m0 * K1) >> 2;
    const int q_hi = ((m0 + 16 < M ? m0 + 16 : M) * K1) >> 2;
    for (int i = q_hi - q_lo + tid; i < 4 * K1; i += 1024) reinterpret_cast<unsigned*>(codes)[i] = 0u;
#pragma unroll
    for (int u = 0; u < kKeep; ++u)
        if (u * 1024 + tid < quads) mm_update(m, v[u].x), mm_update(m, v[u].y), mm_update(m, v[u].z), mm_update(m, v[u].w);
    m = mm_block_reduce(m);
    if (tid == 0) {
        float s, z;
        qparams_of(m.nan ? qnan : m.lo, m.nan ? qnan : m.hi, symmetric, qmin, qmax, is_signed, eps, half_range, &s, &z);
        s_sz[0] = s, s_sz[1] = z;
    }
    __syncthreads();
    const float s = s_sz[0], z = s_sz[1], r = 1.0f / s;
    {
        const QuantizeOp<int8_t> op{x4, reinterpret_cast<Code8x4*>(codes), float(double(qmin)), float(double(qmax)), off};
#pragma unroll
        for (int u = 0; u < kKeep; ++u) {
            const int i = u * 1024 + tid;
            if (i >= q_lo && i < q_hi) op.q[i - q_lo] = op.pack(v[u], s, z, r);
        }
    }
    __syncthreads();
    mb_v4i acc = mb_v4i{0, 0, 0, 0};
    for (int ks = wave; ks < ksteps; ks += 16) {
        const int k = ks * 64 + lg * 16;
        const bool in_k = k < K1;
        const int kq = ks * 64 + cq * 16;
        const mb_v4i wf = place(ks == wave ? wf_first
                                           : (kq < K1 ? *reinterpret_cast<const mb_v4i*>(wrow + kq) : mb_v4i{0, 0, 0, 0}));
        const mb_v4i af = in_k ? *reinterpret_cast<const mb_v4i*>(codes + size_t(ln) * K1 + k) : mb_v4i{0, 0, 0, 0};
        acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(af, wf, acc, 0, 0, 0);
    }
    if (wave < ksteps) {
#pragma unroll
        for (int q = 0; q < 4; ++q)
            __hip_atomic_fetch_add(&red[q * 64 + lane], acc[q], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
    __syncthreads();
    MinMax hm{__builtin_inff(), -__builtin_inff(), 0};
    if (tid < 256) {
        const int q = tid >> 6, l = tid & 63;
        const int mm = m0 + 4 * (l >> 4) + q, nn = n0 + (l & 15);
        if (mm < M && nn < N1) {
            const int zp = int(z) + off;
            const int corr = (wsum1 != nullptr && zp != 0) ? zp * c_wsum : 0;
            const float f = float(red[tid] - corr);
            const float sc = s * c_ws;
            float y = f * sc;
            y = y + c_bias;
            const float floor = relu1 ? 0.0f : -__builtin_inff();
            y = (y < floor) ? floor : y;
            __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(y), hbuf, unsigned(mm * N1 + nn) * 4, 0, kScopeDevice);
            mm_update(hm, y);
        }
    }
    hm = mm_block_reduce(hm);
    if (tid == 0) {
        const float lo = hm.nan ? qnan : hm.lo, hi = hm.nan ? qnan : hm.hi;
        __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(lo), hbuf, unsigned(hid_bytes) + bid * 4, 0, kScopeDevice);
        __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(hi), hbuf, unsigned(hid_bytes) + 256 + bid * 4, 0, kScopeDevice);
    }
    __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): this thread's part of the tile has been written through
    __syncthreads();
    if (tid == 0) s_arrived = __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    if (s_arrived != nblocks - 1) return;

    // ---- the last block: layer 2 on the whole hidden activation.  Everything it needs from
    // memory is requested together: the tiles' ranges, the activation, its weight fragments.
    float slot_lo = __builtin_inff(), slot_hi = -__builtin_inff();
    if (tid < nblocks) {
        slot_lo = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(hbuf, unsigned(hid_bytes) + tid * 4, 0, kScopeDevice));
        slot_hi = __uint_as_float(
            __builtin_amdgcn_raw_buffer_load_b32(hbuf, unsigned(hid_bytes) + 256 + tid * 4, 0, kScopeDevice));
    }
    const int quads2 = (M * N1) >> 2;  // at most 4096: four per thread
    mb_v4u h[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const int i = u * 1024 + tid;
        h[u] = __builtin_amdgcn_raw_buffer_load_b128(hbuf, unsigned(i < quads2 ? i : 0) * 16, 0, kScopeDevice);
    }
    constexpr int kSteps2 = 4;
    const int rb2 = wave & 3, cb2 = wave >> 2;
    const int n2 = cb2 * 16 + ln, nc2 = n2 < N2 ? n2 : N2 - 1;
    mb_v4i w2f[kSteps2];
    {
        const int r2 = cb2 * 16 + rq;
        const int8_t* wrow2 = w2 + size_t(r2 < N2 ? r2 : N2 - 1) * size_t(N1) + cq * 16;
#pragma unroll
        for (int ks = 0; ks < kSteps2; ++ks)
            w2f[ks] = ks * 64 + cq * 16 < N1 ? *reinterpret_cast<const mb_v4i*>(wrow2 + ks * 64) : mb_v4i{0, 0, 0, 0};
    }
    const float c_ws2 = ws2 ? ws2[nc2] : 1.0f;
    const int c_wsum2 = wsum2 ? wsum2[nc2] : 0;
    const float c_bias2 = b2 ? b2[nc2] : -0.0f;
    for (int i = quads2 + tid; i < 16 * N1; i += 1024) reinterpret_cast<unsigned*>(codes2)[i] = 0u;
    MinMax tm{slot_lo, slot_hi, int((slot_lo != slot_lo) | (slot_hi != slot_hi))};
    if (tm.nan) tm.lo = __builtin_inff(), tm.hi = -__builtin_inff();
    tm = mm_block_reduce(tm);
    if (tid == 0) {
        float s2, z2;
        qparams_of(tm.nan ? qnan : tm.lo, tm.nan ? qnan : tm.hi, symmetric, qmin, qmax, is_signed, eps, half_range, &s2, &z2);
        s_sz[2] = s2, s_sz[3] = z2;
        *counter = 0;  // ready for the next launch
    }
    __syncthreads();
    const float s2 = s_sz[2], z2 = s_sz[3];
    {
        const float r2 = 1.0f / s2;
        const QuantizeOp<int8_t> op{nullptr, reinterpret_cast<Code8x4*>(codes2), float(double(qmin)), float(double(qmax)), off};
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int i = u * 1024 + tid;
            if (i < quads2) op.q[i] = op.pack(__builtin_bit_cast(float4, h[u]), s2, z2, r2);
        }
    }
    __syncthreads();
    if (cb2 * 16 < N2 && rb2 * 16 < M) {
        const int zp = int(z2) + off;
        mb_v4i acc2 = mb_v4i{0, 0, 0, 0};
#pragma unroll
        for (int ks = 0; ks < kSteps2; ++ks) {
            const int k = ks * 64 + lg * 16;
            if (ks * 64 < N1) {  // uniform
                const mb_v4i af = k < N1 ? *reinterpret_cast<const mb_v4i*>(codes2 + size_t(16 * rb2 + ln) * N1 + k)
                                         : mb_v4i{0, 0, 0, 0};
                acc2 = __builtin_amdgcn_mfma_i32_16x16x64_i8(af, place(w2f[ks]), acc2, 0, 0, 0);
            }
        }
        const int corr = (wsum2 != nullptr && zp != 0) ? zp * c_wsum2 : 0;
        const float sc = s2 * c_ws2;
        const float floor = relu2 ? 0.0f : -__builtin_inff();
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int mm = 16 * rb2 + 4 * lg + q;
            if (mm < M && n2 < N2) {
                const float f = float(acc2[q] - corr);
                float y = f * sc;
                y = y + c_bias2;
                y = (y < floor) ? floor : y;
                out[size_t(mm) * N2 + n2] = y;
            }
        }
    }
}

}  // namespace

namespace lq {
int minmax_noalloc_init() {
    void* p = nullptr;
    return noalloc_scratch_ptr(&p);
}
}  // namespace lq

extern "C" {

int lq_quantize_tensor_dynamic_i8(const float* x, size_t n, int symmetric, int qmin, int qmax, int is_signed,
                                  float eps, int code_offset, float* scale, float* zp, float* mn_out,
                                  float* mx_out, int8_t* q, lq_stream stream) {
    LQ_REQUIRE(scale && zp && (n == 0 || (x && q)), LQ_ERR_VALUE, "quantize_tensor_dynamic: NULL pointer");
    LQ_REQUIRE(qmax > qmin && qmin + code_offset >= -128 && qmax + code_offset <= 127, LQ_ERR_VALUE,
               "quantize_tensor_dynamic: grid [%d,%d] + offset %d does not fit int8", qmin, qmax, code_offset);
    LQ_REQUIRE(n <= (size_t(1) << 18), LQ_ERR_NOT_IMPLEMENTED,
               "quantize_tensor_dynamic: the one-launch form is for tensors of up to 262144 elements (got %zu); "
               "use lq_minmax + lq_calc_qparams + lq_quantize", n);
    const float half_range = float((double(qmax) - double(qmin)) / 2.0);
    hipLaunchKernelGGL(quantize_tensor_dynamic_kernel, dim3(1), dim3(1024), 0, as_stream(stream), x, n, symmetric,
                       qmin, qmax, is_signed, eps, half_range, code_offset, scale, zp, mn_out, mx_out, q);
    LQ_CHECK_LAUNCH("quantize_tensor_dynamic");
    return LQ_OK;
}

int lq_dynamic_mlp2_small_f32(const float* x, int M, int K1, const int8_t* w1, int N1, const float* w1_scale,
                              const int32_t* w1sum, const float* bias1, int relu1, const int8_t* w2, int N2,
                              const float* w2_scale, const int32_t* w2sum, const float* bias2, int relu2, int symmetric,
                              int qmin, int qmax, int is_signed, float eps, int code_offset, float* out,
                              lq_stream stream) {
    if (M == 0 || N2 == 0) return LQ_OK;
    LQ_REQUIRE(x && w1 && w2 && out, LQ_ERR_VALUE, "dynamic_mlp2_small: NULL pointer");
    LQ_REQUIRE(qmax > qmin && qmin + code_offset >= -128 && qmax + code_offset <= 127, LQ_ERR_VALUE,
               "dynamic_mlp2_small: grid [%d,%d] + offset %d does not fit int8", qmin, qmax, code_offset);
    // a block holds 16 rows of x's codes; the last one also the hidden activation's codes (64 N1 bytes)
    LQ_REQUIRE(M > 0 && M <= 64 && K1 >= 16 && K1 % 16 == 0 && K1 <= 1024 && long(M) * K1 <= 65536 && N1 >= 16 &&
                   N1 % 16 == 0 && N1 <= 256 && N2 > 0 && N2 <= 64 && aligned16(x) && aligned16(w1) && aligned16(w2),
               LQ_ERR_NOT_IMPLEMENTED,
               "dynamic_mlp2_small: takes up to 64 rows, K1 %% 16 == 0 up to 1024, a hidden width that is a multiple of "
               "16 up to 256 and up to 64 outputs (got M = %d, K1 = %d, N1 = %d, N2 = %d); use two "
               "lq_dynamic_linear_small_f32 calls", M, K1, N1, N2);
    const float half_range = float((double(qmax) - double(qmin)) / 2.0);
    // the hidden activation and the tiles' ranges pass through the stream's split-K scratch
    SkScratch sk;
    const size_t hid_bytes = size_t(M) * N1 * 4;
    if (int rc = sk_scratch(1, hid_bytes + 512, as_stream(stream), &sk)) return rc;
    const size_t lds = size_t(16) * K1 + 1024 + size_t(64) * N1;
    static DeviceOnce attr_once;
    if (int rc = allow_dynamic_lds(attr_once, reinterpret_cast<const void*>(dynamic_mlp2_blocks_kernel), 64 * 1024))
        return rc;
    hipLaunchKernelGGL(dynamic_mlp2_blocks_kernel, dim3(unsigned(N1 / 16), unsigned((M + 15) / 16)), dim3(1024), lds,
                       as_stream(stream), x, M, K1, w1, N1, w1_scale, w1sum, bias1, relu1, w2, N2, w2_scale, w2sum, bias2,
                       relu2, symmetric, qmin, qmax, is_signed, eps, half_range, code_offset, out,
                       reinterpret_cast<float*>(sk.slabs), sk.counters);
    LQ_CHECK_LAUNCH("dynamic_mlp2_small");
    return LQ_OK;
}

int lq_dynamic_linear_small_f32(const float* x, int M, int K, const int8_t* w, int N, const float* w_scale,
                                const int32_t* wsum, const float* bias, int relu, int symmetric, int qmin, int qmax,
                                int is_signed, float eps, int code_offset, float* out, lq_stream stream) {
    if (M == 0 || N == 0) return LQ_OK;
    LQ_REQUIRE(x && w && out, LQ_ERR_VALUE, "dynamic_linear_small: NULL pointer");
    LQ_REQUIRE(qmax > qmin && qmin + code_offset >= -128 && qmax + code_offset <= 127, LQ_ERR_VALUE,
               "dynamic_linear_small: grid [%d,%d] + offset %d does not fit int8", qmin, qmax, code_offset);
    // 16 rows of codes (16 K bytes) + 1 KiB of reduction scratch have to fit the 96 KiB of dynamic
    // LDS the kernel is allowed: K <= 6080
    LQ_REQUIRE(M > 0 && M <= 64 && K >= 16 && K % 16 == 0 && long(M) * K <= 65536 && K <= 6080 && N > 0 &&
                   aligned16(x) && aligned16(w),
               LQ_ERR_NOT_IMPLEMENTED,
               "dynamic_linear_small: takes up to 64 rows, K %% 16 == 0 and K <= 6080, at most 65536 activations and "
               "16-byte aligned operands (got M = %d, K = %d); use lq_quantize_tensor_dynamic_i8 + lq_qlinear_i8", M, K);
    const float half_range = float((double(qmax) - double(qmin)) / 2.0);
    const int tiles = (M + 15) / 16;
    const size_t lds = size_t(16) * K + 256 * sizeof(int);
    static DeviceOnce attr_once;
    if (int rc = allow_dynamic_lds(attr_once, reinterpret_cast<const void*>(dynamic_linear_small_kernel), 96 * 1024))
        return rc;
    hipLaunchKernelGGL(dynamic_linear_small_kernel, dim3(unsigned((N + 15) / 16), unsigned(tiles)), dim3(1024), lds,
                       as_stream(stream), x,
                       M, K, w, N, w_scale, wsum, bias, relu, symmetric, qmin, qmax, is_signed, eps, half_range,
                       code_offset, out);
    LQ_CHECK_LAUNCH("dynamic_linear_small");
    return LQ_OK;
}

int lq_quantize_rows_dynamic_i8(const float* x, size_t rows, size_t cols, int symmetric, int qmin, int qmax,
                                int is_signed, float eps, int code_offset, float* scale, float* zp,
                                float* mn_out, float* mx_out, int8_t* q, lq_stream stream) {
    if (rows == 0) return LQ_OK;
    LQ_REQUIRE(x && q && scale && zp, LQ_ERR_VALUE, "quantize_rows_dynamic: NULL pointer");
    LQ_REQUIRE(qmax > qmin && qmin + code_offset >= -128 && qmax + code_offset <= 127, LQ_ERR_VALUE,
               "quantize_rows_dynamic: grid [%d,%d] + offset %d does not fit int8", qmin, qmax, code_offset);
    LQ_REQUIRE(cols >= 4 && cols % 4 == 0 && cols <= 16384 && aligned16(x) &&
                   (reinterpret_cast<uintptr_t>(q) & 3u) == 0 && rows <= 0x7fffffffull,
               LQ_ERR_NOT_IMPLEMENTED,
               "quantize_rows_dynamic: rows of %zu floats (a multiple of 4, at most 16384, 16-byte aligned) "
               "are what the one-pass kernel takes; use lq_minmax + lq_calc_qparams + lq_quantize", cols);
    const float half_range = float((double(qmax) - double(qmin)) / 2.0);
    const int quads = int(cols / 4);
    hipStream_t st = as_stream(stream);
    const float4* x4 = reinterpret_cast<const float4*>(x);
    Code8x4* q4 = reinterpret_cast<Code8x4*>(q);
#define LQ_ROWS_DYN(R)                                                                                      \
    hipLaunchKernelGGL(quantize_rows_dynamic_kernel<R>, dim3(unsigned(rows)), dim3(256), 0, st, x4, quads,  \
                       symmetric, qmin, qmax, is_signed, eps, half_range, code_offset, scale, zp, mn_out,   \
                       mx_out, q4)
    if (quads <= 256) LQ_ROWS_DYN(1);
    else if (quads <= 1024) LQ_ROWS_DYN(4);
    else if (quads <= 2048) LQ_ROWS_DYN(8);
    else LQ_ROWS_DYN(16);
#undef LQ_ROWS_DYN
    LQ_CHECK_LAUNCH("quantize_rows_dynamic");
    return LQ_OK;
}

int lq_minmax(const float* x, size_t outer, size_t C, size_t inner, float* mn, float* mx,
              lq_stream stream) {
    hipStream_t st = as_stream(stream);
    return minmax_launch(x, outer, C, inner, mn, mx, st, ~size_t(0),
                         [st](size_t nbytes, void** ws) { return workspace(nbytes, st, ws); });
}

int lq_minmax_noalloc(const float* x, size_t outer, size_t C, size_t inner, float* mn, float* mx,
                      lq_stream stream) {
    void* scratch = nullptr;
    int rc = noalloc_scratch_ptr(&scratch);
    if (rc) return rc;
    return minmax_launch(x, outer, C, inner, mn, mx, as_stream(stream), kNoAllocScratchBytes,
                         [scratch](size_t nbytes, void** ws) {
                             // minmax_launch sizes its partials to the limit it was given
                             LQ_REQUIRE(nbytes <= kNoAllocScratchBytes, LQ_ERR_SHAPE,
                                        "minmax_noalloc: %zu bytes of partials exceed the %zu-byte static scratch",
                                        nbytes, kNoAllocScratchBytes);
                             *ws = scratch;
                             return int(LQ_OK);
                         });
}

int lq_calc_qparams(const float* mn, const float* mx, size_t C, int symmetric, int qmin, int qmax,
                    int is_signed, float eps, float* scale, float* zp, lq_stream stream) {
    if (C == 0) return LQ_OK;
    LQ_REQUIRE(mn && mx && scale && zp, LQ_ERR_VALUE, "calc_qparams: NULL pointer");
    LQ_REQUIRE(qmax > qmin, LQ_ERR_VALUE, "calc_qparams: empty grid [%d,%d]", qmin, qmax);
    // (quant_max - quant_min) / 2.0 is a Python float promoted to float32
    const float half_range = float((double(qmax) - double(qmin)) / 2.0);
    hipLaunchKernelGGL(calc_qparams_kernel, dim3(unsigned((C + 255) / 256)), dim3(256), 0,
                       as_stream(stream), mn, mx, C, symmetric, qmin, qmax, is_signed, eps, half_range,
                       scale, zp);
    LQ_CHECK_LAUNCH("calc_qparams");
    return LQ_OK;
}

size_t lq_range_buffer_bytes(void) { return size_t(kRangeWords) * 4; }

int lq_calc_qparams_from_range(const float* range, int symmetric, int qmin, int qmax, int is_signed,
                               float eps, float* scale, float* zp, float* mn_out, float* mx_out,
                               lq_stream stream) {
    LQ_REQUIRE(range && scale && zp, LQ_ERR_VALUE, "calc_qparams_from_range: NULL pointer");
    LQ_REQUIRE(qmax > qmin, LQ_ERR_VALUE, "calc_qparams_from_range: empty grid [%d,%d]", qmin, qmax);
    const float half_range = float((double(qmax) - double(qmin)) / 2.0);
    hipLaunchKernelGGL(calc_qparams_from_range_kernel, dim3(1), dim3(1024), 0, as_stream(stream), range,
                       symmetric, qmin, qmax, is_signed, eps, half_range, scale, zp, mn_out, mx_out);
    LQ_CHECK_LAUNCH("calc_qparams_from_range");
    return LQ_OK;
}

int lq_quantize(const float* x, void* q, int q_dtype, int code_offset, size_t outer, size_t C,
                size_t inner, const float* scale, const float* zp, int qparams_on_host, int qmin,
                int qmax, lq_stream stream) {
    if (outer * C * inner == 0) return LQ_OK;
    LQ_REQUIRE(x && q, LQ_ERR_VALUE, "quantize: NULL tensor pointer");
    LQ_REQUIRE(q_dtype == LQ_I8 || q_dtype == LQ_I16, LQ_ERR_DTYPE,
               "quantize: code storage must be int8 or int16 (got dtype %d)", q_dtype);
    const int lim_lo = q_dtype == LQ_I8 ? -128 : -32768, lim_hi = q_dtype == LQ_I8 ? 127 : 32767;
    LQ_REQUIRE(qmin <= qmax && qmin + code_offset >= lim_lo && qmax + code_offset <= lim_hi,
               LQ_ERR_VALUE, "quantize: grid [%d,%d] + offset %d does not fit the code storage", qmin,
               qmax, code_offset);
    QParams qp;
    int rc = make_qparams(scale, zp, qparams_on_host, C, &qp, "quantize");
    if (rc) return rc;
    const float lo = float(double(qmin)), hi = float(double(qmax));
    if (q_dtype == LQ_I8) {
        QuantizeOp<int8_t> op{reinterpret_cast<const float4*>(x), reinterpret_cast<Code8x4*>(q), lo, hi,
                              code_offset};
        return launch_elementwise(op, outer, C, inner, qp, aligned16(x) && aligned16(q),
                                  as_stream(stream), "quantize");
    }
    QuantizeOp<int16_t> op{reinterpret_cast<const float4*>(x), reinterpret_cast<Code16x4*>(q), lo, hi,
                           code_offset};
    return launch_elementwise(op, outer, C, inner, qp, aligned16(x) && aligned16(q), as_stream(stream),
                              "quantize");
}

int lq_dequantize(const void* q, int q_dtype, int code_offset, float* out, size_t outer, size_t C,
                  size_t inner, const float* scale, const float* zp, int qparams_on_host,
                  lq_stream stream) {
    if (outer * C * inner == 0) return LQ_OK;
    LQ_REQUIRE(q && out, LQ_ERR_VALUE, "dequantize: NULL tensor pointer");
    LQ_REQUIRE(q_dtype == LQ_I8 || q_dtype == LQ_I16, LQ_ERR_DTYPE,
               "dequantize: code storage must be int8 or int16 (got dtype %d)", q_dtype);
    QParams qp;
    int rc = make_qparams(scale, zp, qparams_on_host, C, &qp, "dequantize");
    if (rc) return rc;
    if (q_dtype == LQ_I8) {
        DequantizeOp<int8_t> op{reinterpret_cast<const Code8x4*>(q), reinterpret_cast<float4*>(out),
                                code_offset};
        return launch_elementwise(op, outer, C, inner, qp, aligned16(q) && aligned16(out),
                                  as_stream(stream), "dequantize");
    }
    DequantizeOp<int16_t> op{reinterpret_cast<const Code16x4*>(q), reinterpret_cast<float4*>(out),
                             code_offset};
    return launch_elementwise(op, outer, C, inner, qp, aligned16(q) && aligned16(out),
                              as_stream(stream), "dequantize");
}

int lq_fake_quantize(const float* x, float* out, size_t outer, size_t C, size_t inner,
                     const float* scale, const float* zp, int qparams_on_host, int qmin, int qmax,
                     lq_stream stream) {
    if (outer * C * inner == 0) return LQ_OK;
    LQ_REQUIRE(x && out, LQ_ERR_VALUE, "fake_quantize: NULL tensor pointer");
    LQ_REQUIRE(qmin <= qmax, LQ_ERR_VALUE, "fake_quantize: empty grid [%d,%d]", qmin, qmax);
    QParams qp;
    int rc = make_qparams(scale, zp, qparams_on_host, C, &qp, "fake_quantize");
    if (rc) return rc;
    FakeQuantizeOp op{reinterpret_cast<const float4*>(x), reinterpret_cast<float4*>(out),
                      float(double(qmin)), float(double(qmax))};
    return launch_elementwise(op, outer, C, inner, qp, aligned16(x) && aligned16(out),
                              as_stream(stream), "fake_quantize");
}

}  // extern "C"
