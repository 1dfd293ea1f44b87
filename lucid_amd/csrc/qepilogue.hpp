// Device-side epilogue shared by the GEMM and convolution kernels.
#pragma once
#include "qgemm.hpp"

namespace lq {

// ---------------------------------------------------------------- epilogue
struct ColParams {
    float ws, bias;
    int32_t corr;  // a_zp * wsum[n]
};

// A missing bias is the additive identity -0.0f (y + -0.0f == y bit for bit,
// signed zeros and NaNs included), so the add needs no per-element test.
__device__ __forceinline__ ColParams load_col(const GemmArgs& g, int n) {
    ColParams c;
    c.ws = g.w_scale ? g.w_scale[n] : 1.0f;
    const int zp = g.a_zp_dev ? int(g.a_zp_dev[0]) + g.a_zp : g.a_zp;
    c.corr = (g.wsum && zp != 0) ? zp * g.wsum[n] : 0;
    if (g.bias == nullptr)
        c.bias = -0.0f;
    else if (g.bias_dtype == LQ_F16)
        c.bias = float(static_cast<const _Float16*>(g.bias)[n]);
    else
        c.bias = static_cast<const float*>(g.bias)[n];
    return c;
}

// The same for T columns at once, with every load issued before the first
// value is used (one memory round trip instead of one per load).
template <int T>
__device__ __forceinline__ void load_cols(const GemmArgs& g, const int (&n)[T], ColParams (&c)[T]) {
    const int zp = g.a_zp_dev ? int(g.a_zp_dev[0]) + g.a_zp : g.a_zp;
    int32_t wsum[T];
    uint32_t braw[T];
    if (g.w_scale) {
#pragma unroll
        for (int j = 0; j < T; ++j) c[j].ws = g.w_scale[n[j]];
    } else {
#pragma unroll
        for (int j = 0; j < T; ++j) c[j].ws = 1.0f;
    }
    if (g.wsum) {
#pragma unroll
        for (int j = 0; j < T; ++j) wsum[j] = g.wsum[n[j]];
    } else {
#pragma unroll
        for (int j = 0; j < T; ++j) wsum[j] = 0;
    }
    const bool f16 = g.bias != nullptr && g.bias_dtype == LQ_F16;
    if (f16) {
#pragma unroll
        for (int j = 0; j < T; ++j) braw[j] = static_cast<const uint16_t*>(g.bias)[n[j]];
    } else if (g.bias != nullptr) {
#pragma unroll
        for (int j = 0; j < T; ++j) braw[j] = static_cast<const uint32_t*>(g.bias)[n[j]];
    } else {
#pragma unroll
        for (int j = 0; j < T; ++j) braw[j] = 0x80000000u;  // -0.0f
    }
#pragma unroll
    for (int j = 0; j < T; ++j) {
        c[j].corr = zp * wsum[j];
        if (f16) {
            const uint16_t h = uint16_t(braw[j]);
            c[j].bias = float(__builtin_bit_cast(_Float16, h));
        } else {
            c[j].bias = __uint_as_float(braw[j]);
        }
    }
}

__device__ __forceinline__ float q_core(float x, float s, float z, float lo, float hi) {
    float t = x / s;
    float r = __builtin_rintf(t);
    float u = r + z;
    u = (u < lo) ? lo : ((u > hi) ? hi : u);
    return u;
}

// One output element.  Float steps are separate (no FMA) and in the order the
// CPU restatement uses, so results are bit-identical to it.  MODE is a
// compile-time constant so that each output form gets a tight loop.
// epilogue_value returns the element as 32 bits (float bits, or the integer
// for the accumulator / requantized-code forms); store_* narrows and writes.
template <int MODE>
__device__ __forceinline__ uint32_t epilogue_value(const GemmArgs& g, int32_t acc, float as,
                                                   const ColParams& c, float S, float Z) {
    if (MODE == OUT_ACC_I32) return uint32_t(acc);
    float f = float(acc - c.corr);
    float sc = as * c.ws;
    float y = f * sc;
    y = y + c.bias;
    // ReLU as a floor of 0, no ReLU as a floor of -inf: one compare and select either
    // way (a NaN fails the compare and passes through, as in the CPU formulation)
    const float floor = g.relu ? 0.0f : -__builtin_inff();
    y = (y < floor) ? floor : y;
    if (MODE == OUT_F32 || MODE == OUT_F16) return __float_as_uint(y);
    if (MODE == OUT_F32X) {
        // GELU, erf form (lucid/nn/functional/activations.py:219): the expression of the
        // stand-alone kernel, so fusing it changes no bit
        if (g.gelu) y = (0.5f * y) * (1.0f + erff(y * 0.70710678118654752440f));
        return __float_as_uint(y);
    }
    float qv = q_core(y, S, Z, float(g.out_qmin), float(g.out_qmax));
    if (MODE == OUT_REQUANT_I8 || MODE == OUT_REQUANT_JOIN) {
        int code = (qv != qv) ? 0 : int(qv);
        return uint32_t(code + g.out_offset);
    }
    return __float_as_uint((qv - Z) * S);  // OUT_FAKEQUANT_F32
}

// y + residual[m, n] for the float output forms (x + linear(...), the residual
// joins of a transformer block); the other forms ignore the operand.
template <int MODE>
__device__ __forceinline__ uint32_t add_residual(const GemmArgs& g, uint32_t bits, int m, int n) {
    if ((MODE == OUT_F32 || MODE == OUT_F16 || MODE == OUT_F32X) && g.residual)
        return __float_as_uint(__uint_as_float(bits) + g.residual[size_t(m) * size_t(g.ldr) + size_t(n)]);
    return bits;
}

// The fused residual join on codes (lucid/nn/quantized/functional_module.py:224-230 applied
// to this layer's output): both operands are dequantized in float32 with their own
// grids, added, optionally clamped at zero, and requantized.
struct JoinParams {
    float S1, Z1;          // this layer's output grid
    float s2, z2;          // the other operand's grid
    float S, Z, lo, hi;    // the join's output grid
};

__device__ __forceinline__ JoinParams load_join(const GemmArgs& g, float S1, float Z1) {
    JoinParams jp;
    jp.S1 = S1, jp.Z1 = Z1;
    jp.s2 = g.join_scale[0], jp.z2 = g.join_zp[0];
    jp.S = g.join_out_scale[0], jp.Z = g.join_out_zp[0];
    jp.lo = float(g.join_out_qmin), jp.hi = float(g.join_out_qmax);
    return jp;
}

// bits: this layer's stored code (code + out_offset); other: the partner's stored code
__device__ __forceinline__ uint32_t join_code(const GemmArgs& g, const JoinParams& jp, uint32_t bits, int other) {
    const float x1 = (float(int(bits) - g.out_offset) - jp.Z1) * jp.S1;
    const float x2 = (float(other - g.join_off) - jp.z2) * jp.s2;
    float y = x1 + x2;
    if (g.join_relu) y = (y < 0.0f) ? 0.0f : y;
    const float qv = q_core(y, jp.S, jp.Z, jp.lo, jp.hi);
    return uint32_t(((qv != qv) ? 0 : int(qv)) + g.join_out_offset);
}

// one element's residual step, whichever form the output mode has
template <int MODE>
__device__ __forceinline__ uint32_t finish_value(const GemmArgs& g, uint32_t bits, int m, int n, float S, float Z) {
    if (MODE == OUT_REQUANT_JOIN) {
        const JoinParams jp = load_join(g, S, Z);
        return join_code(g, jp, bits, int(g.join_q[size_t(m) * size_t(g.join_ld) + size_t(n)]));
    }
    return add_residual<MODE>(g, bits, m, n);
}

template <int MODE>
__device__ __forceinline__ void store_scalar(const GemmArgs& g, size_t idx, uint32_t v) {
    if (MODE == OUT_F16)
        static_cast<_Float16*>(g.out)[idx] = _Float16(__uint_as_float(v));
    else if (MODE == OUT_REQUANT_I8 || MODE == OUT_REQUANT_JOIN)
        static_cast<int8_t*>(g.out)[idx] = int8_t(int(v));
    else
        static_cast<uint32_t*>(g.out)[idx] = v;  // f32 / i32 bit patterns
}

// four consecutive elements; idx is a multiple of 4 and the row is 4-aligned
template <int MODE>
__device__ __forceinline__ void store_vec4(const GemmArgs& g, size_t idx, uint4 v) {
    if (MODE == OUT_F16) {
        typedef _Float16 h4 __attribute__((ext_vector_type(4)));
        h4 h = {_Float16(__uint_as_float(v.x)), _Float16(__uint_as_float(v.y)),
                _Float16(__uint_as_float(v.z)), _Float16(__uint_as_float(v.w))};
        *reinterpret_cast<h4*>(static_cast<_Float16*>(g.out) + idx) = h;
    } else if (MODE == OUT_REQUANT_I8 || MODE == OUT_REQUANT_JOIN) {
        uint32_t packed = (v.x & 0xffu) | ((v.y & 0xffu) << 8) | ((v.z & 0xffu) << 16) | (v.w << 24);
        *reinterpret_cast<uint32_t*>(static_cast<int8_t*>(g.out) + idx) = packed;
    } else {
        *reinterpret_cast<uint4*>(static_cast<uint32_t*>(g.out) + idx) = v;
    }
}

template <int MODE>
__device__ __forceinline__ void epilogue_store_t(const GemmArgs& g, int m, int n, int32_t acc,
                                                 float as, const ColParams& c, float S, float Z) {
    store_scalar<MODE>(g, size_t(m) * size_t(g.ldo) + size_t(n),
                       finish_value<MODE>(g, epilogue_value<MODE>(g, acc, as, c, S, Z), m, n, S, Z));
}

__device__ __forceinline__ void epilogue_store(const GemmArgs& g, int m, int n, int32_t acc,
                                               float as, const ColParams& c, float S, float Z) {
    switch (g.out_mode) {
    case OUT_ACC_I32: epilogue_store_t<OUT_ACC_I32>(g, m, n, acc, as, c, S, Z); break;
    case OUT_F32:
        if (g.gelu)
            epilogue_store_t<OUT_F32X>(g, m, n, acc, as, c, S, Z);
        else
            epilogue_store_t<OUT_F32>(g, m, n, acc, as, c, S, Z);
        break;
    case OUT_F16: epilogue_store_t<OUT_F16>(g, m, n, acc, as, c, S, Z); break;
    case OUT_REQUANT_I8:
        if (g.join_q)
            epilogue_store_t<OUT_REQUANT_JOIN>(g, m, n, acc, as, c, S, Z);
        else
            epilogue_store_t<OUT_REQUANT_I8>(g, m, n, acc, as, c, S, Z);
        break;
    default: epilogue_store_t<OUT_FAKEQUANT_F32>(g, m, n, acc, as, c, S, Z); break;
    }
}

}  // namespace lq
