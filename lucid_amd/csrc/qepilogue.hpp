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

// The plain form: one division per element (kernels that are bound by memory, not by it).
__device__ __forceinline__ float q_core(float x, float s, float z, float lo, float hi) {
    float t = x / s;
    float r = __builtin_rintf(t);
    float u = r + z;
    u = (u < lo) ? lo : ((u > hi) ? hi : u);
    return u;
}

// One quantization grid, with the reciprocal of its scale (see quant_fast) and, when a ReLU
// comes directly before the quantization, that floor folded into the bounds.
struct QGrid {
    float s, inv, z, lo, hi;  // z, lo, hi include `bias`
    float lof;       // lower bound of the multiplying route: max(lo, z) under a ReLU, else lo
    float loc, hic;  // lof - z and hi - z: the bounds of a code taken relative to z
    float bias;      // 0, or 128 for a signed range: codes come out as code + bias, in 0..255
    bool in_byte;    // ... so that four of them pack with v_cvt_pk_u8_f32 (see CodePack)
    bool relu;
};

// `fast`: the kernel quantizes many elements per lane, so one division to get the
// reciprocal pays.  A grid outside what quant_fast's argument covers (a scale outside a sane
// range, a zero point that is not an integer, a zero point or bounds beyond +-255) gets a NaN
// reciprocal, which sends every element down the dividing branch.
// `relu`: the value is max(x, 0) (a NaN kept), quantized.  For s > 0 dividing and rounding are
// monotone and take 0 to 0, so rint(max(x, 0) / s) = max(rint(x / s), 0): the floor becomes
// the lower bound max(lo, z) of the clamp, which is right when lo <= z <= hi; any other grid
// divides, and the dividing branch applies the floor as written.
// `biased`: the codes are wanted as code + 128 (signed range) or code + 0, within 0..255, so
// that they can be packed as unsigned bytes; the shift goes into z, lo and hi (small
// integers: nothing rounds).  A range that does not fit a byte, or a zero point that is not a
// small integer, stays unshifted with in_byte false.
__device__ __forceinline__ QGrid make_qgrid(float s, float z, float lo, float hi, bool fast, bool relu = false,
                                            bool biased = false) {
    QGrid G;
    const bool z_int = z == __builtin_rintf(z) && __builtin_fabsf(z) <= 255.0f;
    const float b = lo < 0.0f ? 128.0f : 0.0f;
    G.in_byte = biased && z_int && lo <= hi && lo + b >= 0.0f && hi + b <= 255.0f;
    G.bias = G.in_byte ? b : 0.0f;
    z += G.bias, lo += G.bias, hi += G.bias;
    G.s = s, G.z = z, G.lo = lo, G.hi = hi, G.relu = relu;
    const float a = __builtin_fabsf(s);
    bool ok = fast && a > 0x1p-60f && a < 0x1p60f && __builtin_fabsf(z) <= 255.0f && z == __builtin_rintf(z) &&
              __builtin_fabsf(lo) <= 255.0f && __builtin_fabsf(hi) <= 255.0f;
    if (relu) ok = ok && s > 0.0f && lo <= z && z <= hi;
    G.inv = ok ? 1.0f / s : __builtin_nanf("");
    G.lof = (relu && z > lo) ? z : lo;
    G.loc = G.lof - z, G.hic = hi - z;
    return G;
}

// clamp(rint(x / s) + z, lo, hi) with the correctly rounded IEEE quotient, bit for bit,
// mostly without dividing; a NaN becomes KEEP_NAN ? NaN : 0 (all plus G.bias).  CENTERED: the same code
// minus z (what dequantizing it starts with), from clamp(rint(x / s), lo - z, hi - z):
// all of these are integers far below 2^24, or the clamp decides.  (Its zero may be -0 where
// the difference is +0: equal as a number, and the join that consumes it adds before it rounds.)
// tp = x * fl(1/s) is within 2^-22.9 relative of the exact quotient e, and fl(x / s) within
// 2^-24.  rint only changes value at the half-integers.
//  * |tp| < 512: tp is within 6.2e-5 of e and fl(x / s) within 3.1e-5; when tp is farther
//    than 2^-12 = 2.4e-4 from every half-integer, both lie strictly between the same two of
//    them and round to the same integer.
//  * 512 <= |tp| < inf, with d passing the test: both rint(tp) and rint(fl(x / s)) are
//    beyond +-511 with the same sign, and with |z|, |lo|, |hi| <= 255 both clamp to the
//    same bound.
// Otherwise (a few elements in ten thousand, and whatever is infinite or NaN: d = NaN
// fails the test) the lane divides.
template <bool KEEP_NAN, bool CENTERED = false>
__device__ __forceinline__ float quant_fast(float x, const QGrid& G) {
    const float tp = x * G.inv;
    const float r = __builtin_rintf(tp);
    const float d = tp - r;  // exact where it matters
    float c = CENTERED ? __builtin_amdgcn_fmed3f(r, G.loc, G.hic) : __builtin_amdgcn_fmed3f(r + G.z, G.lof, G.hi);
    if (__builtin_expect(!(__builtin_fabsf(d) < 0.5f - 0x1p-12f), 0)) {
        const float xr = (G.relu && x < 0.0f) ? 0.0f : x;
        const float u = __builtin_rintf(xr / G.s) + G.z;
        c = (u != u) ? (KEEP_NAN ? u : G.bias) : __builtin_amdgcn_fmed3f(u, G.lo, G.hi);
        if (CENTERED) c = c - G.z;
    }
    return c;
}

// One output element.  Float steps are separate (no FMA) and in the order the
// CPU restatement uses, so results are bit-identical to it.  MODE is a
// compile-time constant so that each output form gets a tight loop.
// epilogue_value returns the element as 32 bits: float bits, the integer accumulator,
// the requantized code as a float (plus G.bias) or - ahead of a fused join - that code
// minus its zero point (finish_value / join_code take it from there); store_* narrows
// and writes.  G was made with relu = g.relu: the requantizing forms
// leave the floor to it.
// PRESCALED: c.ws already holds as * ws (one activation scale for all rows).
template <int MODE, bool PRESCALED = false>
__device__ __forceinline__ uint32_t epilogue_value(const GemmArgs& g, int32_t acc, float as,
                                                   const ColParams& c, const QGrid& G) {
    if (MODE == OUT_ACC_I32) return uint32_t(acc);
    float f = float(acc - c.corr);
    float sc = PRESCALED ? c.ws : as * c.ws;
    float y = f * sc;
    y = y + c.bias;
    if (MODE == OUT_REQUANT_JOIN) return __float_as_uint(quant_fast<false, true>(y, G));
    // still a float (plus G.bias): store_* narrows it and adds out_offset
    if (MODE == OUT_REQUANT_I8) return __float_as_uint(quant_fast<false>(y, G));
    // not the centered form: its -0 (from rint(x / s) = -0) would survive the multiplication
    if (MODE == OUT_FAKEQUANT_F32) return __float_as_uint((quant_fast<true>(y, G) - G.z) * G.s);
    // ReLU as a floor of 0, no ReLU as a floor of -inf: one compare and select either
    // way (a NaN fails the compare and passes through, as in the CPU formulation)
    const float floor = g.relu ? 0.0f : -__builtin_inff();
    y = (y < floor) ? floor : y;
    if (MODE == OUT_F32X) {
        // GELU, erf form (lucid/nn/functional/activations.py:219): the expression of the
        // stand-alone kernel, so fusing it changes no bit
        if (g.gelu) y = (0.5f * y) * (1.0f + erf_as(y * 0.70710678118654752440f));
    }
    return __float_as_uint(y);
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
    float S1;       // this layer's output scale (its code arrives minus the zero point)
    float s2, z2;   // the other operand's grid
    float k2;       // 128 + join_off + z2: what takes a stored byte + 128 to code - z2
    bool k2_exact;  // ... in one exact subtraction (an integer zero point of sane size)
    QGrid out;      // the join's output grid, with the join's ReLU
};

__device__ __forceinline__ JoinParams load_join(const GemmArgs& g, const QGrid& G, bool fast) {
    JoinParams jp;
    jp.S1 = G.s;
    jp.s2 = g.join_scale[0], jp.z2 = g.join_zp[0];
    jp.k2 = float(128 + g.join_off) + jp.z2;
    jp.k2_exact = jp.z2 == __builtin_rintf(jp.z2) && __builtin_fabsf(jp.z2) <= 0x1p20f && g.join_off >= -(1 << 20) &&
                  g.join_off <= (1 << 20);
    jp.out = make_qgrid(g.join_out_scale[0], g.join_out_zp[0], float(g.join_out_qmin), float(g.join_out_qmax), fast,
                        g.join_relu != 0, fast);
    return jp;
}

// bits: this layer's requantized code minus its zero point, as a float (what
// epilogue_value<OUT_REQUANT_JOIN> returned); other: the partner's stored code
__device__ __forceinline__ uint32_t join_code(const GemmArgs& g, const JoinParams& jp, uint32_t bits, int other) {
    const float x1 = __uint_as_float(bits) * jp.S1;
    const float x2 = (float(other - g.join_off) - jp.z2) * jp.s2;
    return __float_as_uint(quant_fast<false>(x1 + x2, jp.out));  // store_* narrows, adds join_out_offset
}

// The same with the partner's stored byte + 128 (0..255) already a float; needs jp.k2_exact.
__device__ __forceinline__ uint32_t join_code_biased(const JoinParams& jp, uint32_t bits, float other_biased) {
    const float x1 = __uint_as_float(bits) * jp.S1;
    const float x2 = (other_biased - jp.k2) * jp.s2;
    return __float_as_uint(quant_fast<false>(x1 + x2, jp.out));
}

// one element's residual step, whichever form the output mode has (jp: read by the join only)
template <int MODE>
__device__ __forceinline__ uint32_t finish_value(const GemmArgs& g, uint32_t bits, int m, int n, const JoinParams& jp) {
    if (MODE == OUT_REQUANT_JOIN)
        return join_code(g, jp, bits, int(g.join_q[size_t(m) * size_t(g.join_ld) + size_t(n)]));
    return add_residual<MODE>(g, bits, m, n);
}

// Codes leave epilogue_value / join_code as floats, plus the grid's bias and without their
// storage offset (-128 for the quint8 form, else 0).  stored byte = (value - bias + offset)
// mod 256: when the values lie in 0..255 and offset - bias is 0 or +-128 modulo 256, four of
// them are converted and packed by v_cvt_pk_u8_f32 and the offset is an XOR on the dword.
struct CodePack {
    int add;        // offset - bias
    uint32_t flip;  // 0x80808080 when add is 128 modulo 256
    bool pk;        // the packed route applies
};

template <int MODE>
__device__ __forceinline__ CodePack make_code_pack(const GemmArgs& g, const QGrid& G) {
    CodePack c;
    c.add = (MODE == OUT_REQUANT_JOIN ? g.join_out_offset : g.out_offset) - int(G.bias);
    c.pk = G.in_byte && (c.add & 0x7f) == 0;
    c.flip = (c.add & 0x80) ? 0x80808080u : 0u;
    return c;
}

template <int MODE>
__device__ __forceinline__ void store_scalar(const GemmArgs& g, size_t idx, uint32_t v, const CodePack& cpk) {
    if (MODE == OUT_F16)
        static_cast<_Float16*>(g.out)[idx] = _Float16(__uint_as_float(v));
    else if (MODE == OUT_REQUANT_I8 || MODE == OUT_REQUANT_JOIN)
        static_cast<int8_t*>(g.out)[idx] = int8_t(int(__uint_as_float(v)) + cpk.add);
    else
        static_cast<uint32_t*>(g.out)[idx] = v;  // f32 / i32 bit patterns
}

// four consecutive elements; idx is a multiple of 4 and the row is 4-aligned
template <int MODE>
__device__ __forceinline__ void store_vec4(const GemmArgs& g, size_t idx, uint4 v, const CodePack& cpk) {
    if (MODE == OUT_F16) {
        typedef _Float16 h4 __attribute__((ext_vector_type(4)));
        h4 h = {_Float16(__uint_as_float(v.x)), _Float16(__uint_as_float(v.y)),
                _Float16(__uint_as_float(v.z)), _Float16(__uint_as_float(v.w))};
        *reinterpret_cast<h4*>(static_cast<_Float16*>(g.out) + idx) = h;
    } else if (MODE == OUT_REQUANT_I8 || MODE == OUT_REQUANT_JOIN) {
        uint32_t packed;
        if (cpk.pk) {
            packed = __builtin_amdgcn_cvt_pk_u8_f32(__uint_as_float(v.x), 0, 0u);
            packed = __builtin_amdgcn_cvt_pk_u8_f32(__uint_as_float(v.y), 1, packed);
            packed = __builtin_amdgcn_cvt_pk_u8_f32(__uint_as_float(v.z), 2, packed);
            packed = __builtin_amdgcn_cvt_pk_u8_f32(__uint_as_float(v.w), 3, packed);
            packed ^= cpk.flip;
        } else {
            const uint32_t o = uint32_t(cpk.add);
            const uint32_t x = uint32_t(int(__uint_as_float(v.x))), y = uint32_t(int(__uint_as_float(v.y)));
            const uint32_t z = uint32_t(int(__uint_as_float(v.z))), w = uint32_t(int(__uint_as_float(v.w)));
            packed = ((x + o) & 0xffu) | (((y + o) & 0xffu) << 8) | (((z + o) & 0xffu) << 16) | ((w + o) << 24);
        }
        *reinterpret_cast<uint32_t*>(static_cast<int8_t*>(g.out) + idx) = packed;
    } else {
        *reinterpret_cast<uint4*>(static_cast<uint32_t*>(g.out) + idx) = v;
    }
}

template <int MODE>
__device__ __forceinline__ void epilogue_store_t(const GemmArgs& g, int m, int n, int32_t acc,
                                                 float as, const ColParams& c, float S, float Z) {
    // one element per call: no reciprocal, the grid divides
    const QGrid G = make_qgrid(S, Z, float(g.out_qmin), float(g.out_qmax), false, g.relu != 0);
    JoinParams jp;
    if (MODE == OUT_REQUANT_JOIN) jp = load_join(g, G, false);
    store_scalar<MODE>(g, size_t(m) * size_t(g.ldo) + size_t(n),
                       finish_value<MODE>(g, epilogue_value<MODE>(g, acc, as, c, G), m, n, jp),
                       make_code_pack<MODE>(g, MODE == OUT_REQUANT_JOIN ? jp.out : G));
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
