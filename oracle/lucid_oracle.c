/*
 * CPU restatement of Lucid's int8 quantized-inference path.
 *
 * TEST INFRASTRUCTURE ONLY.  This file is the checker the HIP kernels are
 * compared against and the timed CPU baseline; no product code may call it.
 *
 * Every function cites the reference source (paths relative to the Lucid
 * checkout) whose arithmetic it follows.  All float math is IEEE binary32,
 * round-to-nearest-even, no FTZ, no FMA contraction, no reciprocal
 * substitution (build with -ffp-contract=off -fno-fast-math).
 *
 * Two flavours exist for each op:
 *   *_faithful : the reference's pass structure (one full-tensor loop per
 *                engine call, broadcast operands materialised first).  This is
 *                what is timed as "Lucid's CPU path".
 *   (no suffix): one fused loop with the same per-element arithmetic.  It must
 *                be bit-identical to the faithful flavour (tested) and is the
 *                specification the GPU kernels implement.
 *
 * Parity pins (see tests/test_oracle_*.py):
 *   quantize / dequantize / fake_quantize : reference-held known answers,
 *       brute-force tie enumeration, numpy float32 closed forms.
 *   calc_qparams  : reference-held known answers + closed forms.
 *   minmax        : reference-held observer answers + numpy.
 *   f32_to_f16    : numpy float16 conversion on adversarial bit patterns.
 *   igemm (int32) : exact integer arithmetic; brute force int64 + numpy.
 *   qlinear/qconv epilogue : composition of the pinned pieces above.
 *   linear_faithful / conv2d_faithful float outputs : PARITY UNPINNED at the
 *       bit level - the reference sums through Apple Accelerate's cblas_sgemm
 *       whose accumulation order is not published; only the reference's own
 *       tolerance-level bounds apply.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define ORC_I8 1
#define ORC_I16 2

/* Thread count of the loops below (for timing the baseline on one core and on
 * all of them); returns the count now in force. */
int orc_set_threads(int n) {
#ifdef _OPENMP
    if (n > 0) omp_set_num_threads(n);
    return omp_get_max_threads();
#else
    (void)n;
    return 1;
#endif
}

/* ------------------------------------------------------------------ */
/* element arithmetic                                                  */
/* ------------------------------------------------------------------ */

/* lucid/quantization/_functional.py:180  clip(round(x / s) + z, qmin, qmax)
 * div   -> lucid/_C/backend/cpu/Vdsp.cpp:47-48 (vDSP_vdiv, IEEE division)
 * round -> lucid/_C/backend/cpu/Vforce.cpp:136 (vvnintf, ties to even)
 * clip  -> lucid/_C/backend/cpu/CpuBackend.h:6880-6891 (NaN falls through) */
static inline float q_core(float x, float s, float z, float lo, float hi) {
    float t = x / s;
    float r = nearbyintf(t);
    float u = r + z;
    if (u < lo)
        u = lo;
    else if (u > hi)
        u = hi;
    return u;
}

/* astype f32 -> intN is static_cast (CpuBackend.h:6214-6236).  NaN has no
 * defined integer value in C; the oracle maps it to 0 and the tests treat NaN
 * inputs as a documented divergence. */
static inline int32_t cast_code(float c) {
    if (c != c)
        return 0;
    return (int32_t)c;
}

static inline void store_code(void* q, int q_dtype, size_t i, int32_t v) {
    if (q_dtype == ORC_I8)
        ((int8_t*)q)[i] = (int8_t)v;
    else
        ((int16_t*)q)[i] = (int16_t)v;
}

static inline int32_t load_code(const void* q, int q_dtype, size_t i) {
    return q_dtype == ORC_I8 ? (int32_t)((const int8_t*)q)[i] : (int32_t)((const int16_t*)q)[i];
}

/* ------------------------------------------------------------------ */
/* quantize                                                            */
/* ------------------------------------------------------------------ */

/* Fused single pass.  Layout: x is contiguous row-major viewed as
 * [outer][C][inner]; scale/zp have length C (C == 1 for per-tensor), the
 * broadcast of _reshape_for_channel (_functional.py:45-54).
 * code_offset is added to the stored code (0 reproduces Lucid's storage;
 * -128 stores a quint8 code in an int8 for the signed MFMA operand). */
void orc_quantize(const float* x, void* q, int q_dtype, int code_offset, size_t outer, size_t C,
                  size_t inner, const float* scale, const float* zp, int qmin, int qmax) {
    const float lo = (float)(double)qmin, hi = (float)(double)qmax; /* CpuBackend.h:6882-6883 */
    for (size_t o = 0; o < outer; ++o)
        for (size_t c = 0; c < C; ++c) {
            const float s = scale[c], z = zp[c];
            size_t base = (o * C + c) * inner;
            for (size_t i = 0; i < inner; ++i)
                store_code(q, q_dtype, base + i,
                           cast_code(q_core(x[base + i], s, z, lo, hi)) + code_offset);
        }
}

/* Reference pass structure (_functional.py:164-182): materialise broadcast
 * s and z (kernel/BinaryKernel.h:591-606), then div, round, add, clip, astype
 * as five separate full-tensor loops with fresh temporaries. */
void orc_quantize_faithful(const float* x, void* q, int q_dtype, size_t outer, size_t C,
                           size_t inner, const float* scale, const float* zp, int qmin,
                           int qmax) {
    size_t n = outer * C * inner;
    float* sb = (float*)malloc(n * sizeof(float));
    float* zb = (float*)malloc(n * sizeof(float));
    float* t0 = (float*)malloc(n * sizeof(float));
    float* t1 = (float*)malloc(n * sizeof(float));
    for (size_t o = 0; o < outer; ++o)
        for (size_t c = 0; c < C; ++c)
            for (size_t i = 0; i < inner; ++i) {
                sb[(o * C + c) * inner + i] = scale[c];
                zb[(o * C + c) * inner + i] = zp[c];
            }
    for (size_t i = 0; i < n; ++i) t0[i] = x[i] / sb[i];          /* div   */
    for (size_t i = 0; i < n; ++i) t1[i] = nearbyintf(t0[i]);     /* round */
    for (size_t i = 0; i < n; ++i) t0[i] = t1[i] + zb[i];         /* add   */
    const float lo = (float)(double)qmin, hi = (float)(double)qmax;
    for (size_t i = 0; i < n; ++i) {                              /* clip  */
        float v = t0[i];
        if (v < lo)
            v = lo;
        else if (v > hi)
            v = hi;
        t1[i] = v;
    }
    for (size_t i = 0; i < n; ++i) store_code(q, q_dtype, i, cast_code(t1[i])); /* astype */
    free(sb);
    free(zb);
    free(t0);
    free(t1);
}

/* ------------------------------------------------------------------ */
/* dequantize   _functional.py:281   (q.to(f32) - z) * s               */
/* ------------------------------------------------------------------ */
void orc_dequantize(const void* q, int q_dtype, int code_offset, float* out, size_t outer,
                    size_t C, size_t inner, const float* scale, const float* zp) {
    for (size_t o = 0; o < outer; ++o)
        for (size_t c = 0; c < C; ++c) {
            const float s = scale[c], z = zp[c];
            size_t base = (o * C + c) * inner;
            for (size_t i = 0; i < inner; ++i) {
                float v = (float)(load_code(q, q_dtype, base + i) - code_offset);
                out[base + i] = (v - z) * s;
            }
        }
}

void orc_dequantize_faithful(const void* q, int q_dtype, float* out, size_t outer, size_t C,
                             size_t inner, const float* scale, const float* zp) {
    size_t n = outer * C * inner;
    float* sb = (float*)malloc(n * sizeof(float));
    float* zb = (float*)malloc(n * sizeof(float));
    float* t0 = (float*)malloc(n * sizeof(float));
    float* t1 = (float*)malloc(n * sizeof(float));
    for (size_t o = 0; o < outer; ++o)
        for (size_t c = 0; c < C; ++c)
            for (size_t i = 0; i < inner; ++i) {
                sb[(o * C + c) * inner + i] = scale[c];
                zb[(o * C + c) * inner + i] = zp[c];
            }
    for (size_t i = 0; i < n; ++i) t0[i] = (float)load_code(q, q_dtype, i); /* astype */
    for (size_t i = 0; i < n; ++i) t1[i] = t0[i] - zb[i];                   /* sub    */
    for (size_t i = 0; i < n; ++i) out[i] = t1[i] * sb[i];                  /* mul    */
    free(sb);
    free(zb);
    free(t0);
    free(t1);
}

/* ------------------------------------------------------------------ */
/* fake_quantize   _functional.py:311-313                              */
/*   q_pre = round(x/s)+z ; q = clip(q_pre) ; dq = (q - z) * s         */
/* ------------------------------------------------------------------ */
void orc_fake_quantize(const float* x, float* out, size_t outer, size_t C, size_t inner,
                       const float* scale, const float* zp, int qmin, int qmax) {
    const float lo = (float)(double)qmin, hi = (float)(double)qmax;
    for (size_t o = 0; o < outer; ++o)
        for (size_t c = 0; c < C; ++c) {
            const float s = scale[c], z = zp[c];
            size_t base = (o * C + c) * inner;
            for (size_t i = 0; i < inner; ++i) {
                float qv = q_core(x[base + i], s, z, lo, hi);
                out[base + i] = (qv - z) * s;
            }
        }
}

void orc_fake_quantize_faithful(const float* x, float* out, size_t outer, size_t C, size_t inner,
                                const float* scale, const float* zp, int qmin, int qmax) {
    size_t n = outer * C * inner;
    float* sb = (float*)malloc(n * sizeof(float));
    float* zb = (float*)malloc(n * sizeof(float));
    float* t0 = (float*)malloc(n * sizeof(float));
    float* t1 = (float*)malloc(n * sizeof(float));
    for (size_t o = 0; o < outer; ++o)
        for (size_t c = 0; c < C; ++c)
            for (size_t i = 0; i < inner; ++i) {
                sb[(o * C + c) * inner + i] = scale[c];
                zb[(o * C + c) * inner + i] = zp[c];
            }
    const float lo = (float)(double)qmin, hi = (float)(double)qmax;
    for (size_t i = 0; i < n; ++i) t0[i] = x[i] / sb[i];
    for (size_t i = 0; i < n; ++i) t1[i] = nearbyintf(t0[i]);
    for (size_t i = 0; i < n; ++i) t0[i] = t1[i] + zb[i];
    for (size_t i = 0; i < n; ++i) {
        float v = t0[i];
        if (v < lo)
            v = lo;
        else if (v > hi)
            v = hi;
        t1[i] = v;
    }
    for (size_t i = 0; i < n; ++i) t0[i] = t1[i] - zb[i];
    for (size_t i = 0; i < n; ++i) out[i] = t0[i] * sb[i];
    free(sb);
    free(zb);
    free(t0);
    free(t1);
}

/* ------------------------------------------------------------------ */
/* min / max reductions                                                */
/*   lucid/_C/backend/cpu/Reduce.cpp:87-125 : NaN-propagating, identity */
/*   -inf / +inf; observers (observer.py:363-375, 634-653) and           */
/*   nnqd.Linear (nn/quantized/dynamic/linear.py:87-89).                 */
/* ------------------------------------------------------------------ */
void orc_minmax(const float* x, size_t outer, size_t C, size_t inner, float* mn, float* mx) {
    for (size_t c = 0; c < C; ++c) {
        float lo = INFINITY, hi = -INFINITY;
        int nan = 0;
        for (size_t o = 0; o < outer; ++o) {
            const float* p = x + (o * C + c) * inner;
            for (size_t i = 0; i < inner; ++i) {
                float v = p[i];
                if (v != v) nan = 1;
                lo = v < lo ? v : lo;
                hi = v > hi ? v : hi;
            }
        }
        mn[c] = nan ? NAN : lo;
        mx[c] = nan ? NAN : hi;
    }
}

/* ------------------------------------------------------------------ */
/* calculate_qparams   lucid/quantization/_qparams.py:190-215          */
/* ------------------------------------------------------------------ */
/* elementwise maximum/minimum are vDSP_vmax/vmin (Vdsp.cpp:140-146): the
 * single-precision forms propagate NaN. */
static inline float vmaxf(float a, float b) {
    if (a != a || b != b) return NAN;
    return a > b ? a : b;
}
static inline float vminf(float a, float b) {
    if (a != a || b != b) return NAN;
    return a < b ? a : b;
}

void orc_calc_qparams(const float* mn, const float* mx, size_t C, int symmetric, int qmin,
                      int qmax, int is_signed, float eps, float* scale, float* zp) {
    for (size_t c = 0; c < C; ++c) {
        float lo = vminf(mn[c], 0.0f); /* _qparams.py:199 */
        float hi = vmaxf(mx[c], 0.0f); /* _qparams.py:200 */
        if (symmetric) {
            float max_abs = vmaxf(fabsf(lo), fabsf(hi));
            /* (quant_max - quant_min) / 2.0 is a Python float, promoted to f32 */
            float half_range = (float)(((double)qmax - (double)qmin) / 2.0);
            scale[c] = vmaxf(max_abs / half_range, eps);
            zp[c] = is_signed ? 0.0f : (float)((qmax + qmin + 1) >> 1);
        } else {
            float range = (float)(qmax - qmin);
            float s = vmaxf((hi - lo) / range, eps);
            float z = (float)qmin - nearbyintf(lo / s); /* __rsub__ in f32 */
            float qlo = (float)qmin, qhi = (float)qmax;
            if (z < qlo)
                z = qlo;
            else if (z > qhi)
                z = qhi;
            scale[c] = s;
            zp[c] = z;
        }
    }
}

/* ------------------------------------------------------------------ */
/* f32 -> f16 bits   lucid/_C/core/Half.h:80-110 (RNE, subnormals,     */
/* overflow -> inf)                                                    */
/* ------------------------------------------------------------------ */
uint16_t orc_f32_to_f16(float value) {
    uint32_t f;
    memcpy(&f, &value, 4);
    uint32_t sign = (f >> 16) & 0x8000u;
    uint32_t e8 = (f >> 23) & 0xffu;
    uint32_t mant = f & 0x7fffffu;
    if (e8 == 0xffu) return (uint16_t)(sign | 0x7c00u | (mant ? 0x200u : 0u));
    int32_t e = (int32_t)e8 - 127 + 15;
    if (e >= 0x1f) return (uint16_t)(sign | 0x7c00u);
    if (e <= 0) {
        if (e < -10) return (uint16_t)sign;
        mant |= 0x800000u;
        uint32_t shift = (uint32_t)(14 - e);
        uint32_t half = 1u << (shift - 1);
        uint32_t r = (mant + half - 1u + ((mant >> shift) & 1u)) >> shift;
        return (uint16_t)(sign | r);
    }
    uint32_t r = mant + 0x1000u - 1u + ((mant >> 13) & 1u);
    if (r & 0x800000u) {
        ++e;
        if (e >= 0x1f) return (uint16_t)(sign | 0x7c00u);
        return (uint16_t)(sign | ((uint32_t)e << 10));
    }
    return (uint16_t)(sign | ((uint32_t)e << 10) | (r >> 13));
}

float orc_f16_to_f32(uint16_t h) {
    uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    uint32_t e = (h >> 10) & 0x1fu, m = h & 0x3ffu, f;
    if (e == 0) {
        if (m == 0)
            f = sign;
        else {
            int sh = 0;
            while (!(m & 0x400u)) {
                m <<= 1;
                ++sh;
            }
            m &= 0x3ffu;
            f = sign | ((uint32_t)(127 - 15 - sh + 1) << 23) | (m << 13);
        }
    } else if (e == 0x1f)
        f = sign | 0x7f800000u | (m << 13);
    else
        f = sign | ((e - 15 + 127) << 23) | (m << 13);
    float out;
    memcpy(&out, &f, 4);
    return out;
}

void orc_f32_to_f16_array(const float* x, uint16_t* out, size_t n) {
    for (size_t i = 0; i < n; ++i) out[i] = orc_f32_to_f16(x[i]);
}

/* ------------------------------------------------------------------ */
/* integer GEMM  acc[m,n] = sum_k a[m,k] * w[n,k]   (int32, exact)      */
/* The definition is Lucid's own integer matmul: "exact as long as each */
/* dot product stays inside 2^53" (CpuBackend.h:4454-4465, 337-375).   */
/* ------------------------------------------------------------------ */
void orc_igemm(const int8_t* a, const int8_t* w, int32_t* acc, int M, int N, int K) {
#pragma omp parallel for schedule(static)
    for (int n = 0; n < N; ++n) {
        const int8_t* wr = w + (size_t)n * K;
        for (int m = 0; m < M; ++m) {
            const int8_t* ar = a + (size_t)m * K;
            int32_t s = 0;
            for (int k = 0; k < K; ++k) s += (int32_t)ar[k] * (int32_t)wr[k];
            acc[(size_t)m * N + n] = s;
        }
    }
}

/* Same product with activation codes held as Lucid stores quint8 (int16,
 * _qscheme.py:242-245); used to check the re-centring identity
 *   sum (xq - Z) w  ==  sum (xq - 128) w - (Z - 128) sum w. */
void orc_igemm_a16(const int16_t* a, const int8_t* w, int64_t* acc, int M, int N, int K) {
#pragma omp parallel for schedule(static)
    for (int n = 0; n < N; ++n) {
        const int8_t* wr = w + (size_t)n * K;
        for (int m = 0; m < M; ++m) {
            const int16_t* ar = a + (size_t)m * K;
            int64_t s = 0;
            for (int k = 0; k < K; ++k) s += (int64_t)ar[k] * (int64_t)wr[k];
            acc[(size_t)m * N + n] = s;
        }
    }
}

void orc_rowsum_i8(const int8_t* w, int32_t* out, int N, int K) {
    for (int n = 0; n < N; ++n) {
        int32_t s = 0;
        for (int k = 0; k < K; ++k) s += w[(size_t)n * K + k];
        out[n] = s;
    }
}

/* ------------------------------------------------------------------ */
/* quantized Linear, integer formulation                               */
/*   reference surface: nn/quantized/linear.py:199-215 (static),        */
/*   nn/quantized/dynamic/linear.py:84-99 (dynamic),                    */
/*   intrinsic.py:131-133 (ReLU before the output fake-quantize).       */
/*   y = f32(acc - a_zp * wsum[n]) * (a_scale[m] * w_scale[n]) + b[n]   */
/* ------------------------------------------------------------------ */
#define ORC_OUT_ACC_I32 0
#define ORC_OUT_F32 1
#define ORC_OUT_F16 2
#define ORC_OUT_REQUANT_I8 3
#define ORC_OUT_FAKEQUANT_F32 4

#define ORC_BIAS_NONE 0
#define ORC_BIAS_F32 6
#define ORC_BIAS_F16 5

static inline float epi_value(int32_t acc, int32_t a_zp, int32_t wsum, float as, float ws,
                              int bias_kind, const void* bias, size_t n, int relu) {
    int32_t t = acc - a_zp * wsum;
    float f = (float)t;
    float sc = as * ws;
    float y = f * sc;
    if (bias_kind == ORC_BIAS_F32)
        y = y + ((const float*)bias)[n];
    else if (bias_kind == ORC_BIAS_F16)
        y = y + orc_f16_to_f32(((const uint16_t*)bias)[n]);
    if (relu) y = (y < 0.0f) ? 0.0f : y; /* Vdsp.cpp:130-133 vrelu_f32 */
    return y;
}

/* rows index m (M of them), columns index n (N).  out_stride_* let the conv
 * wrapper write NCHW or NHWC. */
static void epilogue_store(float y, int out_mode, void* out, size_t idx, float S, float Z,
                           int qmin, int qmax, int out_offset) {
    switch (out_mode) {
    case ORC_OUT_F32:
        ((float*)out)[idx] = y;
        break;
    case ORC_OUT_F16:
        ((uint16_t*)out)[idx] = orc_f32_to_f16(y);
        break;
    case ORC_OUT_REQUANT_I8: {
        float qv = q_core(y, S, Z, (float)qmin, (float)qmax);
        ((int8_t*)out)[idx] = (int8_t)(cast_code(qv) + out_offset);
        break;
    }
    case ORC_OUT_FAKEQUANT_F32: {
        float qv = q_core(y, S, Z, (float)qmin, (float)qmax);
        ((float*)out)[idx] = (qv - Z) * S;
        break;
    }
    default:
        break;
    }
}

void orc_qlinear_epilogue(const int32_t* acc, int M, int N, int a_zp, const int32_t* wsum,
                          const float* a_scale, int a_scale_per_row, const float* w_scale,
                          int bias_kind, const void* bias, int relu, int out_mode,
                          float out_scale, float out_zp, int out_qmin, int out_qmax,
                          int out_offset, void* out) {
    for (int m = 0; m < M; ++m)
        for (int n = 0; n < N; ++n) {
            size_t idx = (size_t)m * N + n;
            if (out_mode == ORC_OUT_ACC_I32) {
                ((int32_t*)out)[idx] = acc[idx];
                continue;
            }
            float as = a_scale[a_scale_per_row ? m : 0];
            float y = epi_value(acc[idx], a_zp, wsum ? wsum[n] : 0, as, w_scale[n], bias_kind,
                                bias, (size_t)n, relu);
            epilogue_store(y, out_mode, out, idx, out_scale, out_zp, out_qmin, out_qmax,
                           out_offset);
        }
}

void orc_qlinear(const int8_t* a, const int8_t* w, int M, int N, int K, int a_zp,
                 const float* a_scale, int a_scale_per_row, const float* w_scale, int bias_kind,
                 const void* bias, int relu, int out_mode, float out_scale, float out_zp,
                 int out_qmin, int out_qmax, int out_offset, void* out) {
    int32_t* acc = (int32_t*)malloc((size_t)M * N * sizeof(int32_t));
    int32_t* wsum = (int32_t*)malloc((size_t)N * sizeof(int32_t));
    orc_igemm(a, w, acc, M, N, K);
    orc_rowsum_i8(w, wsum, N, K);
    orc_qlinear_epilogue(acc, M, N, a_zp, wsum, a_scale, a_scale_per_row, w_scale, bias_kind,
                         bias, relu, out_mode, out_scale, out_zp, out_qmin, out_qmax, out_offset,
                         out);
    free(acc);
    free(wsum);
}

/* The same Linear with affine weight codes: row n of w carries the zero point w_zp[n]
 * (per-channel affine weights, lucid/quantization/_qscheme.py per_channel_affine, as
 * from_float stores them in nn/quantized/linear.py:217-236).  The float composite
 * dequantizes both operands before the product (linear.py:199-215), so the exact
 * integer value under the two scales is
 *     eff[m,n] = sum_k (a[m,k] - a_zp) * (w[n,k] - w_zp[n]),
 * taken here term by term in 64 bits; the epilogue is orc_qlinear's with the
 * corrections already applied.  Mode ACC_I32 returns the raw sum_k a*w as before. */
void orc_qlinear_affine(const int8_t* a, const int8_t* w, const int32_t* w_zp, int M, int N,
                        int K, int a_zp, const float* a_scale, int a_scale_per_row,
                        const float* w_scale, int bias_kind, const void* bias, int relu,
                        int out_mode, float out_scale, float out_zp, int out_qmin,
                        int out_qmax, int out_offset, void* out) {
    int32_t* eff = (int32_t*)malloc((size_t)M * N * sizeof(int32_t));
#pragma omp parallel for schedule(static)
    for (int m = 0; m < M; ++m)
        for (int n = 0; n < N; ++n) {
            int64_t s = 0;
            const int64_t zw = (out_mode == ORC_OUT_ACC_I32 || !w_zp) ? 0 : w_zp[n];
            const int64_t za = out_mode == ORC_OUT_ACC_I32 ? 0 : a_zp;
            for (int k = 0; k < K; ++k)
                s += ((int64_t)a[(size_t)m * K + k] - za) * ((int64_t)w[(size_t)n * K + k] - zw);
            eff[(size_t)m * N + n] = (int32_t)s;
        }
    orc_qlinear_epilogue(eff, M, N, 0, NULL, a_scale, a_scale_per_row, w_scale, bias_kind, bias,
                         relu, out_mode, out_scale, out_zp, out_qmin, out_qmax, out_offset, out);
    free(eff);
}

/* ------------------------------------------------------------------ */
/* float GEMM used by the faithful path:  c[m,n] = sum_k a[m,k]*b[n,k]  */
/* (the reference calls cblas_sgemm with transB, CpuBackend.h:4493;    */
/* its summation order is Accelerate-internal, so this one is simply    */
/* ascending k).                                                       */
/* ------------------------------------------------------------------ */
void orc_sgemm_nt(const float* a, const float* b, float* c, int M, int N, int K) {
    /* pack b^T once so the inner loop vectorises over n with a fixed k order */
    float* bt = (float*)malloc((size_t)K * N * sizeof(float));
#pragma omp parallel for schedule(static)
    for (int n = 0; n < N; ++n)
        for (int k = 0; k < K; ++k) bt[(size_t)k * N + n] = b[(size_t)n * K + k];
#pragma omp parallel for schedule(static)
    for (int m0 = 0; m0 < M; m0 += 4) {
        int mb = M - m0 < 4 ? M - m0 : 4;
        for (int n0 = 0; n0 < N; n0 += 256) {
            int nb = N - n0 < 256 ? N - n0 : 256;
            float accb[4][256];
            for (int i = 0; i < mb; ++i)
                for (int j = 0; j < nb; ++j) accb[i][j] = 0.0f;
            for (int k = 0; k < K; ++k) {
                const float* br = bt + (size_t)k * N + n0;
                for (int i = 0; i < mb; ++i) {
                    float av = a[(size_t)(m0 + i) * K + k];
                    for (int j = 0; j < nb; ++j) accb[i][j] = accb[i][j] + av * br[j];
                }
            }
            for (int i = 0; i < mb; ++i)
                for (int j = 0; j < nb; ++j) c[(size_t)(m0 + i) * N + n0 + j] = accb[i][j];
        }
    }
    free(bt);
}

/* ------------------------------------------------------------------ */
/* quantized Linear, the reference's own float pass structure           */
/*   nn/quantized/linear.py:199-215 :                                   */
/*     W^ = dequantize(weight_int8)            (every call)             */
/*     y  = x @ W^T (+ bias)    CpuBackend.h:4525-4569, 11260-11268     */
/*     y  = relu(y)             (LinearReLU only)                       */
/*     out = fake_quantize(y, S, Z)   (skipped when do_fq == 0: the     */
/*           dynamic module returns the float result, dynamic/linear.py:99) */
/* ------------------------------------------------------------------ */
void orc_linear_faithful(const float* x, const int8_t* wq, const float* w_scale,
                         const float* w_zp, const float* bias, int M, int N, int K, int relu,
                         int do_fq, float S, float Z, int qmin, int qmax, float* out) {
    float* wf = (float*)malloc((size_t)N * K * sizeof(float));
    orc_dequantize_faithful(wq, ORC_I8, wf, 1, (size_t)N, (size_t)K, w_scale, w_zp);
    float* y = (float*)malloc((size_t)M * N * sizeof(float));
    orc_sgemm_nt(x, wf, y, M, N, K);
    if (bias)
        for (int m = 0; m < M; ++m)
            for (int n = 0; n < N; ++n) y[(size_t)m * N + n] = y[(size_t)m * N + n] + bias[n];
    if (relu)
        for (size_t i = 0; i < (size_t)M * N; ++i) y[i] = (y[i] < 0.0f) ? 0.0f : y[i];
    if (do_fq)
        orc_fake_quantize_faithful(y, out, 1, 1, (size_t)M * N, &S, &Z, qmin, qmax);
    else
        memcpy(out, y, (size_t)M * N * sizeof(float));
    free(wf);
    free(y);
}

/* ------------------------------------------------------------------ */
/* convolution                                                         */
/* ------------------------------------------------------------------ */
/* output extent, lucid/_C/nn/ConvNd.cpp:56-59 */
int orc_conv_out_size(int S, int K, int stride, int pad_lo, int pad_hi, int dil) {
    return (S + pad_lo + pad_hi - dil * (K - 1) - 1) / stride + 1;
}

/* Integer im2col for one image in NHWC code layout; out-of-bounds taps take
 * pad_code (the activation zero-point code: the reference pads the float
 * image with 0.0, lucid/_C/backend/cpu/Im2Col.cpp:59-100, and real 0.0 is the
 * code Z on the activation grid).
 * cols[(oh*OW+ow)][(kh*KW+kw)*Cg + ci] for group g. */
static void im2col_nhwc_i8(const int8_t* x, int H, int W, int Cin, int g, int Cg, int KH, int KW,
                           int OH, int OW, int sh, int sw, int ph, int pw, int dh, int dw,
                           int8_t pad_code, int8_t* cols) {
    int Kf = KH * KW * Cg;
    for (int oh = 0; oh < OH; ++oh)
        for (int ow = 0; ow < OW; ++ow) {
            int8_t* row = cols + (size_t)(oh * OW + ow) * Kf;
            for (int kh = 0; kh < KH; ++kh)
                for (int kw = 0; kw < KW; ++kw) {
                    int ih = oh * sh - ph + kh * dh, iw = ow * sw - pw + kw * dw;
                    int8_t* dst = row + (size_t)(kh * KW + kw) * Cg;
                    if (ih < 0 || ih >= H || iw < 0 || iw >= W) {
                        for (int ci = 0; ci < Cg; ++ci) dst[ci] = pad_code;
                    } else {
                        const int8_t* src = x + ((size_t)ih * W + iw) * Cin + (size_t)g * Cg;
                        for (int ci = 0; ci < Cg; ++ci) dst[ci] = src[ci];
                    }
                }
        }
}

/* Quantized Conv2d, integer formulation (surface: nn/quantized/conv.py:168-184,
 * intrinsic.py:334-336).  Activation codes NHWC int8 [B,H,W,Cin]; weight codes
 * [Cout][KH][KW][Cin/groups]; output NHWC [B,OH,OW,Cout] in out_mode's type.
 * pad is (lo_h, hi_h, lo_w, hi_w): "same" padding can be asymmetric
 * (nn/modules/conv.py:44-55). */
void orc_qconv2d(const int8_t* x, const int8_t* w, int B, int H, int W, int Cin, int Cout, int KH,
                 int KW, int sh, int sw, int ph_lo, int ph_hi, int pw_lo, int pw_hi, int dh,
                 int dw, int groups, int a_zp, float a_scale, const float* w_scale,
                 int bias_kind, const void* bias, int relu, int out_mode, float out_scale,
                 float out_zp, int out_qmin, int out_qmax, int out_offset, void* out) {
    int OH = orc_conv_out_size(H, KH, sh, ph_lo, ph_hi, dh);
    int OW = orc_conv_out_size(W, KW, sw, pw_lo, pw_hi, dw);
    int Cg = Cin / groups, Og = Cout / groups, Kf = KH * KW * Cg;
    size_t esz = out_mode == ORC_OUT_F16 ? 2 : (out_mode == ORC_OUT_REQUANT_I8 ? 1 : 4);
#pragma omp parallel for schedule(static)
    for (int b = 0; b < B; ++b) {
        int8_t* cols = (int8_t*)malloc((size_t)OH * OW * Kf);
        int32_t* acc = (int32_t*)malloc((size_t)OH * OW * Og * sizeof(int32_t));
        for (int g = 0; g < groups; ++g) {
            im2col_nhwc_i8(x + (size_t)b * H * W * Cin, H, W, Cin, g, Cg, KH, KW, OH, OW, sh, sw,
                           ph_lo, pw_lo, dh, dw, (int8_t)a_zp, cols);
            const int8_t* wg = w + (size_t)g * Og * Kf;
            for (int p = 0; p < OH * OW; ++p)
                for (int o = 0; o < Og; ++o) {
                    int32_t s = 0, ws = 0;
                    const int8_t* ar = cols + (size_t)p * Kf;
                    const int8_t* wr = wg + (size_t)o * Kf;
                    for (int k = 0; k < Kf; ++k) {
                        s += (int32_t)ar[k] * (int32_t)wr[k];
                        ws += wr[k];
                    }
                    int co = g * Og + o;
                    size_t idx = ((size_t)b * OH * OW + p) * Cout + co;
                    if (out_mode == ORC_OUT_ACC_I32) {
                        ((int32_t*)out)[idx] = s;
                        continue;
                    }
                    float y = epi_value(s, a_zp, ws, a_scale, w_scale[co], bias_kind, bias,
                                        (size_t)co, relu);
                    epilogue_store(y, out_mode, out, idx, out_scale, out_zp, out_qmin, out_qmax,
                                   out_offset);
                }
        }
        free(cols);
        free(acc);
    }
    (void)esz;
}

/* orc_qconv2d with affine filter codes: filter co carries the zero point w_zp[co]
 * (nn/quantized/conv.py from_float with a per-channel affine weight observer).  Taps in
 * the padding hold the code a_zp, i.e. the float value 0 that zero padding of the
 * dequantized image gives (Im2Col.cpp:59-100), so they contribute (a_zp - a_zp) * (...) = 0
 * exactly as in the float composite. */
void orc_qconv2d_affine(const int8_t* x, const int8_t* w, const int32_t* w_zp, int B, int H,
                        int W, int Cin, int Cout, int KH, int KW, int sh, int sw, int ph_lo,
                        int ph_hi, int pw_lo, int pw_hi, int dh, int dw, int groups, int a_zp,
                        float a_scale, const float* w_scale, int bias_kind, const void* bias,
                        int relu, int out_mode, float out_scale, float out_zp, int out_qmin,
                        int out_qmax, int out_offset, void* out) {
    int OH = orc_conv_out_size(H, KH, sh, ph_lo, ph_hi, dh);
    int OW = orc_conv_out_size(W, KW, sw, pw_lo, pw_hi, dw);
    int Cg = Cin / groups, Og = Cout / groups;
#pragma omp parallel for schedule(static)
    for (int b = 0; b < B; ++b)
        for (int oh = 0; oh < OH; ++oh)
            for (int ow = 0; ow < OW; ++ow)
                for (int co = 0; co < Cout; ++co) {
                    const int g = co / Og;
                    const int64_t zw = (out_mode == ORC_OUT_ACC_I32 || !w_zp) ? 0 : w_zp[co];
                    const int64_t za = out_mode == ORC_OUT_ACC_I32 ? 0 : a_zp;
                    int64_t s = 0;
                    for (int kh = 0; kh < KH; ++kh)
                        for (int kw = 0; kw < KW; ++kw) {
                            const int ih = oh * sh - ph_lo + kh * dh, iw = ow * sw - pw_lo + kw * dw;
                            const int inside = ih >= 0 && ih < H && iw >= 0 && iw < W;
                            for (int ci = 0; ci < Cg; ++ci) {
                                const int64_t av =
                                    inside ? x[(((size_t)b * H + ih) * W + iw) * Cin + g * Cg + ci]
                                           : a_zp;
                                const int64_t wv = w[(((size_t)co * KH + kh) * KW + kw) * Cg + ci];
                                s += (av - za) * (wv - zw);
                            }
                        }
                    size_t idx = (((size_t)b * OH + oh) * OW + ow) * Cout + co;
                    if (out_mode == ORC_OUT_ACC_I32) {
                        ((int32_t*)out)[idx] = (int32_t)s;
                        continue;
                    }
                    float y = epi_value((int32_t)s, 0, 0, a_scale, w_scale[co], bias_kind, bias,
                                        (size_t)co, relu);
                    epilogue_store(y, out_mode, out, idx, out_scale, out_zp, out_qmin, out_qmax,
                                   out_offset);
                }
}

/* Float im2col for one image, one group, NCHW (Im2Col.cpp:59-100): rows are
 * (ci, kh, kw), columns output positions; zero padding. */
static void im2col_nchw_f32(const float* x, int Cg, int H, int W, int KH, int KW, int OH, int OW,
                            int sh, int sw, int ph, int pw, int dh, int dw, float* cols) {
    for (int ci = 0; ci < Cg; ++ci)
        for (int kh = 0; kh < KH; ++kh)
            for (int kw = 0; kw < KW; ++kw) {
                float* row = cols + (size_t)((ci * KH + kh) * KW + kw) * OH * OW;
                for (int oh = 0; oh < OH; ++oh)
                    for (int ow = 0; ow < OW; ++ow) {
                        int ih = oh * sh - ph + kh * dh, iw = ow * sw - pw + kw * dw;
                        row[oh * OW + ow] = (ih < 0 || ih >= H || iw < 0 || iw >= W)
                                                ? 0.0f
                                                : x[((size_t)ci * H + ih) * W + iw];
                    }
            }
}

/* Quantized Conv2d, the reference's float pass structure
 * (nn/quantized/conv.py:168-184 -> CpuBackend.h:8124-8257): dequantize the
 * kernel, per image and per group im2col + GEMM (Cout_g x K_flat)(K_flat x O),
 * per-channel bias add, optional ReLU, fake_quantize.  NCHW / OIHW, symmetric
 * zero padding (asymmetric pads are pre-padded by the module, conv.py:104-123;
 * the caller does the same). */
void orc_conv2d_faithful(const float* x, const int8_t* wq, const float* w_scale,
                         const float* w_zp, const float* bias, int B, int Cin, int H, int W,
                         int Cout, int KH, int KW, int sh, int sw, int ph, int pw, int dh, int dw,
                         int groups, int relu, int do_fq, float S, float Z, int qmin, int qmax,
                         float* out) {
    int OH = orc_conv_out_size(H, KH, sh, ph, ph, dh);
    int OW = orc_conv_out_size(W, KW, sw, pw, pw, dw);
    int Cg = Cin / groups, Og = Cout / groups, Kf = Cg * KH * KW, O = OH * OW;
    size_t wn = (size_t)Cout * Kf;
    float* wf = (float*)malloc(wn * sizeof(float));
    orc_dequantize_faithful(wq, ORC_I8, wf, 1, (size_t)Cout, (size_t)Kf, w_scale, w_zp);
    size_t on = (size_t)B * Cout * O;
    float* y = (float*)malloc(on * sizeof(float));
#pragma omp parallel for schedule(static)
    for (int b = 0; b < B; ++b) {
        float* cols = (float*)malloc((size_t)Kf * O * sizeof(float));
        for (int g = 0; g < groups; ++g) {
            im2col_nchw_f32(x + ((size_t)b * Cin + (size_t)g * Cg) * H * W, Cg, H, W, KH, KW, OH,
                            OW, sh, sw, ph, pw, dh, dw, cols);
            for (int o = 0; o < Og; ++o) {
                float* yr = y + ((size_t)b * Cout + (size_t)g * Og + o) * O;
                for (int p = 0; p < O; ++p) yr[p] = 0.0f;
                const float* wr = wf + ((size_t)g * Og + o) * Kf;
                for (int k = 0; k < Kf; ++k) {
                    float wv = wr[k];
                    const float* cr = cols + (size_t)k * O;
                    for (int p = 0; p < O; ++p) yr[p] = yr[p] + wv * cr[p];
                }
            }
        }
        free(cols);
    }
    if (bias)
        for (int b = 0; b < B; ++b)
            for (int c = 0; c < Cout; ++c) {
                float* yr = y + ((size_t)b * Cout + c) * O;
                for (int p = 0; p < O; ++p) yr[p] = yr[p] + bias[c];
            }
    if (relu)
        for (size_t i = 0; i < on; ++i) y[i] = (y[i] < 0.0f) ? 0.0f : y[i];
    if (do_fq)
        orc_fake_quantize_faithful(y, out, 1, 1, on, &S, &Z, qmin, qmax);
    else
        memcpy(out, y, on * sizeof(float));
    free(wf);
    free(y);
}

/* ------------------------------------------------------------------ */
/* residual join   nn/quantized/functional_module.py:216-232            */
/*   add_relu: fq(relu(x + y)),  add: fq(x + y); x, y float-carried on  */
/*   their own grids.  Code-domain form: x = (qx - zx)*sx etc.          */
/* ------------------------------------------------------------------ */
void orc_add_requant(const int8_t* qa, int a_offset, float sa, float za, const int8_t* qb,
                     int b_offset, float sb, float zb, size_t n, int relu, float S, float Z,
                     int qmin, int qmax, int out_offset, int8_t* out) {
    for (size_t i = 0; i < n; ++i) {
        float xa = ((float)((int32_t)qa[i] - a_offset) - za) * sa;
        float xb = ((float)((int32_t)qb[i] - b_offset) - zb) * sb;
        float y = xa + xb;
        if (relu) y = (y < 0.0f) ? 0.0f : y;
        float qv = q_core(y, S, Z, (float)qmin, (float)qmax);
        out[i] = (int8_t)(cast_code(qv) + out_offset);
    }
}

/* max-pool on codes, NHWC.  Quantisation is monotone non-decreasing, so the
 * max of codes equals the code of the max; padding never wins (-inf in the
 * float domain = code minimum). */
void orc_maxpool2d_nhwc_i8(const int8_t* x, int B, int H, int W, int C, int KH, int KW, int sh,
                           int sw, int ph, int pw, int8_t* out) {
    int OH = (H + 2 * ph - KH) / sh + 1, OW = (W + 2 * pw - KW) / sw + 1;
    for (int b = 0; b < B; ++b)
        for (int oh = 0; oh < OH; ++oh)
            for (int ow = 0; ow < OW; ++ow)
                for (int c = 0; c < C; ++c) {
                    int best = -128;
                    for (int kh = 0; kh < KH; ++kh)
                        for (int kw = 0; kw < KW; ++kw) {
                            int ih = oh * sh - ph + kh, iw = ow * sw - pw + kw;
                            if (ih < 0 || ih >= H || iw < 0 || iw >= W) continue;
                            int v = x[(((size_t)b * H + ih) * W + iw) * C + c];
                            best = v > best ? v : best;
                        }
                    out[(((size_t)b * OH + oh) * OW + ow) * C + c] = (int8_t)best;
                }
}

/* ------------------------------------------------------------------ */
/* Eval-mode BatchNorm forward, IBackend::batch_norm_eval_forward      */
/* (lucid/_C/backend/cpu/CpuBackend.h:9163-9208): x is (B, C, spatial); */
/*   rstd[c] = 1 / (float)sqrt((double)var[c] + eps)                   */
/*   y       = g * (x - m) * r + b       float32, left to right        */
/* gamma / beta NULL = ones / zeros (nn/functional/normalization.py:91-101). */
void orc_batchnorm_eval(const float* x, float* y, size_t B, size_t C, size_t spatial,
                        const float* mean, const float* var, const float* gamma,
                        const float* beta, double eps) {
    for (size_t b = 0; b < B; ++b)
        for (size_t c = 0; c < C; ++c) {
            const float r = 1.0f / (float)sqrt((double)var[c] + eps);
            const float m = mean[c], g = gamma ? gamma[c] : 1.0f, bb = beta ? beta[c] : 0.0f;
            const float* xr = x + (b * C + c) * spatial;
            float* yr = y + (b * C + c) * spatial;
            for (size_t s = 0; s < spatial; ++s) yr[s] = g * (xr[s] - m) * r + bb;
        }
}
