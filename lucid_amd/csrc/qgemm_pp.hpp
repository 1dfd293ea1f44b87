// Eight-wavefront "ping-pong" tile kernel of the int8 GEMM for large problems.
//
// A CU has four SIMDs; the block puts two wavefronts on each.  The two never do
// the same thing at the same time: while one issues the MFMAs of a 64-byte k
// step on operand fragments it already holds in registers, the other reads its
// fragments of the next step from LDS and issues its share of the global -> LDS
// loads; at the workgroup barrier that ends each phase they swap roles.  The
// matrix cores of a SIMD therefore always have one wavefront whose only work is
// MFMAs, and LDS / global latency is paid by the other one.
//
//   block tile   BM x BN x 64 bytes of k per LDS stage, STAGES stages in flight
//   wavefronts   WM x WN = 8, each owning (BM/WM) x (BN/WN) outputs as TM x TN
//                tiles of v_mfma_i32_16x16x64_i8 (BN/WN need only be a multiple
//                of 16, so a 352-column tile covers N = 11008 in 32 tiles wide)
//   result       the MFMA takes the weight fragment as its first operand, so a lane's four
//                accumulator registers of a tile are four consecutive output columns of one
//                row: the epilogue packs and stores them directly, with no trip through LDS
//   phases       wavefronts 0..3 (group 0) and 4..7 (group 1) share SIMDs pairwise;
//                group 0: phase 2u = read + load for k step u, phase 2u+1 = MFMAs
//                group 1: one phase later
#pragma once
#include "common.hpp"
#include "qgemm.hpp"
#include "qepilogue.hpp"
#include "range_slots.hpp"

#include <utility>

namespace lq {
namespace {

typedef int pp_v4i __attribute__((ext_vector_type(4)));

#define LQ_PP_GPTR(p) ((__attribute__((address_space(1))) void*)(p))
#define LQ_PP_LPTR(p) ((__attribute__((address_space(3))) void*)(p))

template <int BM_, int BN_, int WM_, int WN_, int STAGES_>
struct PPCfg {
    static constexpr int BM = BM_, BN = BN_, BK = 64, WM = WM_, WN = WN_, STAGES = STAGES_;
    static constexpr int WAVES = WM * WN;
    static constexpr int THREADS = WAVES * 64;
    static constexpr int TM = BM / WM / 16, TN = BN / WN / 16;
    // one wavefront-wide 16-byte direct load fills 1 KiB = 16 rows of 64 bytes
    static constexpr int A_CHUNKS = BM / 16, B_CHUNKS = BN / 16;
    static constexpr int LA = (A_CHUNKS + WAVES - 1) / WAVES, LB = (B_CHUNKS + WAVES - 1) / WAVES;
    static constexpr int STAGE_BYTES = (BM + BN) * BK;
    // after the stage buffers: the block's column parameters (scale, bias, correction) as three
    // arrays of BN words, written once in the prologue and read by the epilogue
    static constexpr int PARAM_OFF = STAGES * STAGE_BYTES;
    static constexpr int SMEM = PARAM_OFF + 3 * BN * 4;
    static_assert(WAVES == 8, "two wavefronts per SIMD");
    static_assert(BM % (WM * 16) == 0 && BN % (WN * 16) == 0, "");
    static_assert(STAGES == 4, "operand pairs cycle through four 64-byte stages");
    static_assert(TM * TN > 2 * LB + 1 && 1 + 2 * LB <= 63, "");
    static_assert(SMEM <= 160 * 1024, "LDS of a CU");
    static_assert(BN <= THREADS, "one column parameter set per thread");
};

template <class F, int... X>
__device__ __forceinline__ void pp_static_for_impl(F& f, std::integer_sequence<int, X...>) {
    (f(std::integral_constant<int, X>{}), ...);
}
// f(integral_constant<int, 0>), ..., f(integral_constant<int, N-1>): a loop whose index is a constant expression
template <int N, class F>
__device__ __forceinline__ void pp_static_for(F&& f) {
    pp_static_for_impl(f, std::make_integer_sequence<int, N>{});
}

constexpr int pp_vmcnt_imm(int n) { return (n & 0xF) | ((n >> 4) << 14) | (0x7 << 4) | (0xF << 8); }

// Same tile walk as the four-wavefront kernel: every XCD (blocks are dealt to the
// eight XCDs round-robin) gets a contiguous range of tile ids, walked m-fastest in
// groups of 8 m-tiles, so tiles that share an L2 share operand rows.
__device__ __forceinline__ void pp_tile_coords(int bid, int nblk, int tiles_m, int tiles_n, int* tm, int* tn) {
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

typedef pp_v4i v4i_t;

// The four values of store_vec4 as the dwords it would write (1 for codes, 2 for float16, 4 for
// 32-bit outputs), for stores that first regroup them between lanes.
template <int MODE>
__device__ __forceinline__ void pp_pack(uint4 v, const CodePack& cpk, uint32_t* dw) {
    if (MODE == OUT_F16) {
        typedef _Float16 h2 __attribute__((ext_vector_type(2)));
        const h2 a = {_Float16(__uint_as_float(v.x)), _Float16(__uint_as_float(v.y))};
        const h2 b = {_Float16(__uint_as_float(v.z)), _Float16(__uint_as_float(v.w))};
        dw[0] = __builtin_bit_cast(uint32_t, a);
        dw[1] = __builtin_bit_cast(uint32_t, b);
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
        dw[0] = packed;
    } else {
        dw[0] = v.x, dw[1] = v.y, dw[2] = v.z, dw[3] = v.w;
    }
}

// Which column tile a wavefront keeps in accumulator column j.  Normally tile j.  When the
// wavefront has an odd number of column tiles and its first output column sits half a store
// run off an aligned position in memory (the second half of a 352-column tile starts at column
// 176; the epilogue stores pairs of tiles as runs of 32 columns, which for float16 are 64
// bytes), the tiles are rotated by one: column j holds tile (j + 1) % TN.  The pairs
// (0,1), (2,3), ... of accumulator columns are then the tiles (1,2), (3,4), ..., whose runs
// start on a multiple of their size, and the lone last column is tile 0.  A run that
// straddles two such segments reaches memory as two partial writes.  Only the LDS address
// of a B fragment and the column an accumulator is stored to depend on it.
template <int TN, int MODE>
__device__ __forceinline__ int pp_rotation(const GemmArgs& g, int wn0) {
    constexpr int esize = MODE == OUT_F16 ? 2 : ((MODE == OUT_REQUANT_I8 || MODE == OUT_REQUANT_JOIN) ? 1 : 4);
    if (TN % 2 == 0 || g.ldo % 32 != 0 || reinterpret_cast<uintptr_t>(g.out) % (16 * esize) != 0) return 0;
    return (reinterpret_cast<uintptr_t>(g.out) / esize + size_t(wn0)) % 32 == 16 ? 1 : 0;
}

// The register epilogue.  acc[i][j][r] is row wm0 + 16 i + lane % 16, column
// wn0 + 16 t + 4 (lane / 16) + r with t = the column tile of j (pp_rotation): four consecutive
// columns per lane and tile, so scale, bias, ReLU / requantize / join run on registers and the
// packed values are stored directly.  s_ws / s_bias / s_corr: the block's column parameters in
// LDS (column n0 first); as_row: this lane's row scales.
template <int TM, int TN, int MODE>
__device__ __forceinline__ void pp_epilogue(const GemmArgs& g, pp_v4i (&acc)[TM][TN], const float (&as_row)[TM],
                                            const float* s_ws, const float* s_bias, const int32_t* s_corr, int n0,
                                            int wm0, int wn0, int lane, int rot, float& r_lo, float& r_hi, int& r_nan) {
    if (wm0 >= g.M || wn0 >= g.N) return;
    // running range of what this lane stores (float32 output with a kept range only)
    const bool keep = MODE == OUT_F32X && g.range != nullptr;
    auto track = [&](uint32_t bits) {
        const float y = __uint_as_float(bits);
        r_nan |= (y != y);
        r_lo = fminf(r_lo, y);
        r_hi = fmaxf(r_hi, y);
    };
    float S = 1.0f, Z = 0.0f;
    constexpr bool kRequant = MODE == OUT_REQUANT_I8 || MODE == OUT_REQUANT_JOIN || MODE == OUT_FAKEQUANT_F32;
    if (kRequant) {
        S = g.out_scale[0];
        Z = g.out_zp[0];
    }
    const QGrid G = make_qgrid(S, Z, float(g.out_qmin), float(g.out_qmax), kRequant, g.relu != 0, MODE == OUT_REQUANT_I8);
    JoinParams jp;
    if (MODE == OUT_REQUANT_JOIN) jp = load_join(g, G, true);
    const CodePack cpk = make_code_pack<MODE>(g, MODE == OUT_REQUANT_JOIN ? jp.out : G);
    constexpr int esize = MODE == OUT_F16 ? 2 : ((MODE == OUT_REQUANT_I8 || MODE == OUT_REQUANT_JOIN) ? 1 : 4);
    constexpr bool kFloatOut = MODE == OUT_F32 || MODE == OUT_F16 || MODE == OUT_F32X;
    const bool prescaled = (MODE == OUT_REQUANT_I8 || MODE == OUT_REQUANT_JOIN) && !g.a_scale_per_row;
    const bool cols_in = wn0 + TN * 16 <= g.N, rows_in = wm0 + TM * 16 <= g.M;
    // uniform: every access of this wavefront may be a whole aligned vector
    const bool vec_out = cols_in && g.ldo % 4 == 0 && reinterpret_cast<uintptr_t>(g.out) % (4 * esize) == 0 &&
                         (!kFloatOut || g.residual == nullptr || (g.ldr % 4 == 0 && aligned16(g.residual))) &&
                         (MODE != OUT_REQUANT_JOIN ||
                          (g.join_ld % 4 == 0 && reinterpret_cast<uintptr_t>(g.join_q) % 4 == 0 && jp.k2_exact));
    // first column of the lane's four in the tile of accumulator column j: pairs are the
    // columns j = 2x, 2x + 1 (tiles j + rot), the lone last column of an odd TN is tile
    // rot ? 0 : TN - 1
    const int pair0 = wn0 + 16 * rot;
    const int last_tile = rot ? 0 : TN - 1;
    const int lane_col = 4 * (lane >> 4);
    // Wider stores for pairs of column tiles: the lanes of an even and the following odd row
    // group (16 lanes each) exchange one tile's packed values (v_permlane16_swap), after which an
    // even-group lane holds eight consecutive columns of the first tile and an odd-group lane
    // eight of the second.  A row then receives 64 contiguous bytes of float16 (32 of int8
    // codes, 128 of 32-bit values) from four lanes instead of half that.
    constexpr int kDw = MODE == OUT_F16 ? 2 : ((MODE == OUT_REQUANT_I8 || MODE == OUT_REQUANT_JOIN) ? 1 : 4);
    constexpr int kPairs = TN / 2;
    constexpr bool kLone = TN % 2 == 1;
    const bool wide = vec_out && g.ldo % 8 == 0 && reinterpret_cast<uintptr_t>(g.out) % 16 == 0;
    const int g_odd = (lane >> 4) & 1;
    const int swapped_col = 16 * g_odd + 4 * ((lane >> 4) & ~1);  // within a pair: first of the lane's 8 columns
    typedef unsigned v4u_t __attribute__((ext_vector_type(4)));
    typedef unsigned v2u_t __attribute__((ext_vector_type(2)));

    // ---- the plain float forms (aligned output, no residual, no ReLU, no zero-point correction)
    // when the matrix ends on a 16 x 16 tile boundary inside this sub-tile or beyond it: the same
    // float steps - convert, as * ws, multiply, add the bias - and nothing else.  Row pointers are
    // formed once and every store takes a constant offset from one of them; row blocks and column
    // tiles past the end of the matrix are skipped whole (the last tile column of N = 11008 holds
    // 96 real columns: without this its blocks, taking the element-wise route, finish many
    // microseconds after everybody else).
    if constexpr (MODE == OUT_F16 || MODE == OUT_F32) {
        const int zp = g.a_zp_dev ? int(g.a_zp_dev[0]) + g.a_zp : g.a_zp;
        const int ncols = g.N - wn0, nrows = g.M - wm0;
        const bool lean = g.ldo % 8 == 0 && reinterpret_cast<uintptr_t>(g.out) % 16 == 0 && g.residual == nullptr &&
                          !g.relu && (g.wsum == nullptr || zp == 0) && (ncols >= TN * 16 || ncols % 16 == 0) &&
                          (nrows >= TM * 16 || nrows % 16 == 0);
        if (lean) {
            const int vt = ncols >= TN * 16 ? TN : ncols / 16;  // column tiles and row blocks inside the matrix
            const int vr = nrows >= TM * 16 ? TM : nrows / 16;
            char* rows[TM];  // the lane's position in a pair's run, row block by row block
            rows[0] = static_cast<char*>(g.out) +
                      (size_t(wm0 + (lane & 15)) * size_t(g.ldo) + size_t(pair0 + swapped_col)) * esize;
            const size_t row_step = size_t(16) * size_t(g.ldo) * esize;
#pragma unroll
            for (int i = 1; i < TM; ++i) rows[i] = rows[i - 1] + row_step;
            auto value4 = [&](const pp_v4i& a, const float4& ws, const float4& b, float as, uint4& v) {
                v.x = __float_as_uint(float(a[0]) * (as * ws.x) + b.x);
                v.y = __float_as_uint(float(a[1]) * (as * ws.y) + b.y);
                v.z = __float_as_uint(float(a[2]) * (as * ws.z) + b.z);
                v.w = __float_as_uint(float(a[3]) * (as * ws.w) + b.w);
            };
            // accumulator column j, which is column tile t, from the lane's own layout (four columns)
            auto single = [&](auto j_tag, int t) {
                constexpr int j = decltype(j_tag)::value;
                const int cl = wn0 - n0 + 16 * t + lane_col;
                const float4 ws = *reinterpret_cast<const float4*>(s_ws + cl), b = *reinterpret_cast<const float4*>(s_bias + cl);
                const ptrdiff_t delta = ptrdiff_t(16 * t + lane_col - 16 * rot - swapped_col) * esize;
#pragma unroll
                for (int i = 0; i < TM; ++i) {
                    if (i >= vr) break;
                    uint4 v;
                    value4(acc[i][j], ws, b, as_row[i], v);
                    uint32_t p[kDw];
                    pp_pack<MODE>(v, cpk, p);
                    char* dst = rows[i] + delta;
                    if constexpr (kDw == 2)
                        *reinterpret_cast<v2u_t*>(dst) = v2u_t{p[0], p[1]};
                    else
                        *reinterpret_cast<v4u_t*>(dst) = v4u_t{p[0], p[1], p[2], p[3]};
                }
            };
            pp_static_for<kPairs>([&](auto x_tag) {
                constexpr int j = 2 * decltype(x_tag)::value;
                const int ta = j + rot;  // the pair's column tiles: ta, ta + 1
                if (ta + 1 >= vt) {
                    if (ta < vt) single(std::integral_constant<int, j>{}, ta);
                    return;
                }
                const int cl = pair0 - n0 + 16 * j + lane_col;  // the lane's own columns of the pair's first tile
                const float4 ws0 = *reinterpret_cast<const float4*>(s_ws + cl), b0 = *reinterpret_cast<const float4*>(s_bias + cl);
                const float4 ws1 = *reinterpret_cast<const float4*>(s_ws + cl + 16),
                             b1 = *reinterpret_cast<const float4*>(s_bias + cl + 16);
#pragma unroll
                for (int i = 0; i < TM; ++i) {
                    if (i >= vr) break;
                    uint4 v, w;
                    value4(acc[i][j], ws0, b0, as_row[i], v);
                    value4(acc[i][j + 1], ws1, b1, as_row[i], w);
                    uint32_t p[kDw], q[kDw], lo[kDw], hi[kDw];
                    pp_pack<MODE>(v, cpk, p);
                    pp_pack<MODE>(w, cpk, q);
#pragma unroll
                    for (int d = 0; d < kDw; ++d) {
                        const auto sw = __builtin_amdgcn_permlane16_swap(p[d], q[d], false, false);
                        lo[d] = sw[0], hi[d] = sw[1];
                    }
                    char* dst = rows[i] + 16 * j * esize;
                    if constexpr (kDw == 2) {
                        *reinterpret_cast<v4u_t*>(dst) = v4u_t{lo[0], lo[1], hi[0], hi[1]};
                    } else {
                        *reinterpret_cast<v4u_t*>(dst) = v4u_t{lo[0], lo[1], lo[2], lo[3]};
                        *reinterpret_cast<v4u_t*>(dst + 16) = v4u_t{hi[0], hi[1], hi[2], hi[3]};
                    }
                }
            });
            if constexpr (kLone) {
                if (last_tile < vt) single(std::integral_constant<int, TN - 1>{}, last_tile);
            }
            return;
        }
    }

    // ---- every other form.  The residual operand of a float output is requested first, every
    // tile of the wavefront at once: requested tile by tile, each of the TM * TN loads would be
    // waited for on its own (the operand was last touched several kernels ago and comes from
    // memory), which costs the ViT's proj and fc2 a third of their time.  In-place use
    // (out == residual) is unaffected: an element is still read before it is written, by its own lane.
    // (tiles of up to 24 sub-tiles per wavefront: the larger shapes have no registers to spare)
    constexpr bool kResidualForm = (MODE == OUT_F32 || MODE == OUT_F16 || MODE == OUT_F32X) && TM * TN <= 24;
    const bool res_ahead = kResidualForm && vec_out && g.residual != nullptr;
    float4 rres[kResidualForm ? TM : 1][kResidualForm ? TN : 1];
    if constexpr (kResidualForm) {
        if (res_ahead) {
#pragma unroll
            for (int i = 0; i < TM; ++i) {
                const int m = wm0 + 16 * i + (lane & 15);
                const float* rp = g.residual + size_t(rows_in || m < g.M ? m : 0) * size_t(g.ldr) + size_t(lane_col);
#pragma unroll
                for (int j = 0; j < TN; ++j) {
                    // accumulator column j is column tile j + rot (the lone last one: last_tile)
                    const int t = (kLone && j == TN - 1) ? last_tile : j + rot;
                    rres[i][j] = *reinterpret_cast<const float4*>(rp + wn0 + 16 * t);
                }
            }
        }
    }
    // values of one tile in the lane's own layout, residual / join applied; (ri, rj): the tile's
    // place among the wavefront's accumulators
    auto tile_values = [&](int m, const pp_v4i& a, const ColParams (&c4)[4], float as, int nq, uint4& v, int ri, int rj) {
        if (prescaled) {
            v.x = epilogue_value<MODE, true>(g, a[0], 1.0f, c4[0], G);
            v.y = epilogue_value<MODE, true>(g, a[1], 1.0f, c4[1], G);
            v.z = epilogue_value<MODE, true>(g, a[2], 1.0f, c4[2], G);
            v.w = epilogue_value<MODE, true>(g, a[3], 1.0f, c4[3], G);
        } else {
            v.x = epilogue_value<MODE, false>(g, a[0], as, c4[0], G);
            v.y = epilogue_value<MODE, false>(g, a[1], as, c4[1], G);
            v.z = epilogue_value<MODE, false>(g, a[2], as, c4[2], G);
            v.w = epilogue_value<MODE, false>(g, a[3], as, c4[3], G);
        }
        if (vec_out && (rows_in || m < g.M)) {
            if (kFloatOut && g.residual != nullptr) {
                const float4 rv = kResidualForm
                                      ? rres[kResidualForm ? ri : 0][kResidualForm ? rj : 0]
                                      : *reinterpret_cast<const float4*>(g.residual + size_t(m) * size_t(g.ldr) + size_t(nq));
                v.x = __float_as_uint(__uint_as_float(v.x) + rv.x);
                v.y = __float_as_uint(__uint_as_float(v.y) + rv.y);
                v.z = __float_as_uint(__uint_as_float(v.z) + rv.z);
                v.w = __float_as_uint(__uint_as_float(v.w) + rv.w);
            }
            if (MODE == OUT_REQUANT_JOIN) {
                const uint32_t jb = *reinterpret_cast<const uint32_t*>(g.join_q + size_t(m) * size_t(g.join_ld) + size_t(nq)) ^
                                    0x80808080u;  // stored bytes + 128, all four
                v.x = join_code_biased(jp, v.x, float(jb & 0xffu));
                v.y = join_code_biased(jp, v.y, float((jb >> 8) & 0xffu));
                v.z = join_code_biased(jp, v.z, float((jb >> 16) & 0xffu));
                v.w = join_code_biased(jp, v.w, float(jb >> 24));
            }
        }
    };
    auto load_c4 = [&](int nq, ColParams (&c4)[4]) {
        const int cl = nq - n0;  // column within the block tile, a multiple of 4
        const float4 ws = *reinterpret_cast<const float4*>(s_ws + cl);
        const float4 b = *reinterpret_cast<const float4*>(s_bias + cl);
        const int4 cr = *reinterpret_cast<const int4*>(s_corr + cl);
        c4[0] = ColParams{ws.x, b.x, cr.x}, c4[1] = ColParams{ws.y, b.y, cr.y};
        c4[2] = ColParams{ws.z, b.z, cr.z}, c4[3] = ColParams{ws.w, b.w, cr.w};
        if (prescaled) {
#pragma unroll
            for (int r = 0; r < 4; ++r) c4[r].ws = as_row[0] * c4[r].ws;
        }
    };
    // one tile stored from the lane's own layout (four consecutive columns)
    auto store_own = [&](int m, int nq, uint4 v) {
        if (!rows_in && m >= g.M) return;
        const size_t idx = size_t(m) * size_t(g.ldo) + size_t(nq);
        if (vec_out) {
            store_vec4<MODE>(g, idx, v, cpk);
        } else {
            const uint32_t e[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
            for (int k = 0; k < 4; ++k)
                if (nq + k < g.N) {
                    const uint32_t f = finish_value<MODE>(g, e[k], m, nq + k, jp);
                    if (MODE == OUT_F32X && keep) track(f);
                    store_scalar<MODE>(g, idx + k, f, cpk);
                }
        }
    };
    pp_static_for<kPairs>([&](auto x_tag) {
        constexpr int j = 2 * decltype(x_tag)::value;
        const int nq = pair0 + 16 * j + lane_col;
        ColParams c4[4], d4[4];
        load_c4(nq, c4);
        load_c4(nq + 16, d4);
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            const int m = wm0 + 16 * i + (lane & 15);
            uint4 v, w;
            tile_values(m, acc[i][j], c4, as_row[i], nq, v, i, j);
            tile_values(m, acc[i][j + 1], d4, as_row[i], nq + 16, w, i, j + 1);
            if (MODE == OUT_F32X && keep && vec_out && (rows_in || m < g.M)) {
                track(v.x), track(v.y), track(v.z), track(v.w);
                track(w.x), track(w.y), track(w.z), track(w.w);
            }
            if (!wide) {
                store_own(m, nq, v);
                store_own(m, nq + 16, w);
                continue;
            }
            uint32_t p[kDw], q[kDw], lo[kDw], hi[kDw];
            pp_pack<MODE>(v, cpk, p);
            pp_pack<MODE>(w, cpk, q);
#pragma unroll
            for (int d = 0; d < kDw; ++d) {
                const auto sw = __builtin_amdgcn_permlane16_swap(p[d], q[d], false, false);
                lo[d] = sw[0], hi[d] = sw[1];
            }
            if (!rows_in && m >= g.M) continue;
            char* dst = static_cast<char*>(g.out) +
                        (size_t(m) * size_t(g.ldo) + size_t(pair0 + 16 * j + swapped_col)) * esize;
            if constexpr (kDw == 1) {
                *reinterpret_cast<v2u_t*>(dst) = v2u_t{lo[0], hi[0]};
            } else if constexpr (kDw == 2) {
                *reinterpret_cast<v4u_t*>(dst) = v4u_t{lo[0], lo[1], hi[0], hi[1]};
            } else {
                *reinterpret_cast<v4u_t*>(dst) = v4u_t{lo[0], lo[1], lo[2], lo[3]};
                *reinterpret_cast<v4u_t*>(dst + 16) = v4u_t{hi[0], hi[1], hi[2], hi[3]};
            }
        }
    });
    if constexpr (kLone) {
        const int nq = wn0 + 16 * last_tile + lane_col;
        ColParams c4[4];
        load_c4(nq, c4);
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            const int m = wm0 + 16 * i + (lane & 15);
            uint4 v;
            tile_values(m, acc[i][TN - 1], c4, as_row[i], nq, v, i, TN - 1);
            if (MODE == OUT_F32X && keep && vec_out && (rows_in || m < g.M)) track(v.x), track(v.y), track(v.z), track(v.w);
            store_own(m, nq, v);
        }
    }
}

// K must be a multiple of 64 (the launcher checks); M and N are arbitrary: rows past
// the end of an operand read as zeros and are masked at the store.
template <class Cfg, int MODE>
__global__ __launch_bounds__(Cfg::THREADS) __attribute__((amdgpu_waves_per_eu(2, 2))) void qgemm_pp_kernel(GemmArgs g) {
    constexpr int BM = Cfg::BM, BN = Cfg::BN, BK = Cfg::BK, TM = Cfg::TM, TN = Cfg::TN;
    constexpr int STAGES = Cfg::STAGES, LA = Cfg::LA, LB = Cfg::LB;
    extern __shared__ __attribute__((aligned(1024))) int8_t smem[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int group = wave >> 2;  // wavefronts w and w + 4 share a SIMD
    const int wm = wave / Cfg::WN, wn = wave % Cfg::WN;
    const int tiles_m = (g.M + BM - 1) / BM, tiles_n = (g.N + BN - 1) / BN;
    int tm, tn;
    pp_tile_coords(blockIdx.x, gridDim.x, tiles_m, tiles_n, &tm, &tn);
    const int m0 = tm * BM, n0 = tn * BN;
    const int nk = g.K / BK;
    const int wm0 = m0 + wm * (TM * 16), wn0 = n0 + wn * (TN * 16);  // this wavefront's sub-tile
    const int rot = pp_rotation<TN, MODE>(g, wn0);

    // ---- global -> LDS: chunk c of an operand is its rows 16c .. 16c+15; lane l fills the slot
    // of row 16c + l/4, physical 16-byte chunk l%4, with the logical chunk (l%4) ^ ((row/2)%4).
    // (Measured: with this swizzle the fragment reads below - 16 rows x 4 chunks per instruction -
    // run at the rate of a contiguous ds_read_b128; with (row/4)%4, which suits fragments of 32
    // rows x 2 chunks, they take 40 % longer.)
    const int ld_row = lane >> 2;
    const int ld_kc = (lane & 3) ^ ((lane >> 3) & 3);
    // The operands are read through buffer descriptors: one 32-bit offset register per lane, the
    // k position in a scalar offset, and rows past the end of a matrix (the last tile in m or n)
    // read as zeros instead of needing a clamp.
    unsigned a_off[LA], b_off[LB];
    int a_chunk[LA], b_chunk[LB];
#pragma unroll
    for (int i = 0; i < LA; ++i) {
        a_chunk[i] = (wave + Cfg::WAVES * i) % Cfg::A_CHUNKS;
        a_off[i] = unsigned(m0 + a_chunk[i] * 16 + ld_row) * unsigned(g.K) + unsigned(ld_kc * 16);
    }
#pragma unroll
    for (int i = 0; i < LB; ++i) {
        b_chunk[i] = (wave + Cfg::WAVES * i) % Cfg::B_CHUNKS;
        b_off[i] = unsigned(n0 + b_chunk[i] * 16 + ld_row) * unsigned(g.K) + unsigned(ld_kc * 16);
    }
    const __amdgpu_buffer_rsrc_t a_rsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t*>(g.a), 0, unsigned(g.M) * unsigned(g.K), 0x00020000);
    const __amdgpu_buffer_rsrc_t b_rsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t*>(g.w), 0, unsigned(g.N) * unsigned(g.K), 0x00020000);

    // Direct load x (0 .. LA + LB - 1) of this wavefront for stage s of the k loop.  Stages past the
    // end reload the last one into a buffer nobody reads, which keeps the number of outstanding
    // loads - the vmcnt to wait for - the same throughout.
    auto stage_load = [&](int s, auto x_tag) {
        constexpr int x = decltype(x_tag)::value;
        const int sk = s < nk ? s : nk - 1;
        int8_t* buf = smem + (s % STAGES) * Cfg::STAGE_BYTES;
        if constexpr (x < LA) {
            __builtin_amdgcn_raw_ptr_buffer_load_lds(a_rsrc, LQ_PP_LPTR(buf + a_chunk[x] * 1024), 16, int(a_off[x]), sk * BK, 0,
                                                     0);
        } else {
            __builtin_amdgcn_raw_ptr_buffer_load_lds(b_rsrc, LQ_PP_LPTR(buf + BM * BK + b_chunk[x - LA] * 1024), 16,
                                                     int(b_off[x - LA]), sk * BK, 0, 0);
        }
    };
    // One operand's loads of this wavefront for the two consecutive stages s and s+1, issued
    // alternately so that the two 64-byte halves of each 128-byte line of a matrix row are
    // requested back to back: the second request finds the line the first one brought into the
    // CU's cache (loaded a whole stage apart, every line would be fetched from the L2 twice).
    auto pair_load_all = [&](int s, auto op_tag) {
        constexpr int first = decltype(op_tag)::value ? LA : 0;
        constexpr int n = 2 * (decltype(op_tag)::value ? LB : LA);
        pp_static_for<n>([&](auto c_tag) {
            constexpr int c = decltype(c_tag)::value;
            stage_load(s + (c & 1), std::integral_constant<int, first + c / 2>{});
        });
    };

    // ---- LDS -> registers: lane l of a 16 x 64 fragment holds row l%16, logical chunk l/16,
    // which sits at physical chunk (l/16) ^ ((row/2)%4).  B fragment j is the wavefront's column
    // tile (j + rot) % TN.
    const int fr_off = (lane & 15) * BK + (((lane >> 4) ^ ((lane >> 1) & 3)) * 16);
    const int a_frag0 = wm * (TM * 16) * BK + fr_off;
    const int b_frag0 = BM * BK + wn * (TN * 16) * BK + fr_off + rot * 16 * BK;
    const int b_frag_last = BM * BK + wn * (TN * 16) * BK + fr_off + (rot ? 0 : (TN - 1) * 16 * BK);
    pp_v4i af[TM], bf[TN];
    auto read_frags = [&](int s) {
        const int8_t* buf = smem + (s % STAGES) * Cfg::STAGE_BYTES;
#pragma unroll
        for (int i = 0; i < TM; ++i) af[i] = *reinterpret_cast<const pp_v4i*>(buf + a_frag0 + i * 16 * BK);
#pragma unroll
        for (int j = 0; j < TN - 1; ++j) bf[j] = *reinterpret_cast<const pp_v4i*>(buf + b_frag0 + j * 16 * BK);
        bf[TN - 1] = *reinterpret_cast<const pp_v4i*>(buf + b_frag_last);
    };

    pp_v4i acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = pp_v4i{0, 0, 0, 0};

    // The MFMAs of one k step, column by column; within a column the row order alternates, so
    // that only one operand changes from one instruction to the next (fewer operand bits
    // toggle: the MFMA-only rate on the same codes is 2 % higher in this order, and the launch 1 us shorter).
    constexpr int kMfmas = TM * TN;
    auto compute = [&]() {
        __builtin_amdgcn_s_setprio(2);
        pp_static_for<kMfmas>([&](auto x_tag) {
            constexpr int X = decltype(x_tag)::value;
            constexpr int j = X / TM;
            constexpr int i = (j & 1) ? TM - 1 - X % TM : X % TM;
            acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(bf[j], af[i], acc[i][j], 0, 0, 0);
        });
        __builtin_amdgcn_s_setprio(0);
    };
    // ---- prologue: the tile's column parameters are requested first (they go to LDS, where the
    // barriers of the main loop publish them), then the first stages.  Issue order per
    // wavefront: A(0,1), B(0), B(1,2); then step u adds A(u+2,u+3) when u is even and B(u+2,u+3)
    // when u is odd.
    float* s_ws = reinterpret_cast<float*>(smem + Cfg::PARAM_OFF);
    float* s_bias = s_ws + BN;
    int32_t* s_corr = reinterpret_cast<int32_t*>(s_bias + BN);
    ColParams c_mine{1.0f, -0.0f, 0};
    if (tid < BN) c_mine = load_col(g, n0 + tid < g.N ? n0 + tid : g.N - 1);
    __builtin_amdgcn_sched_barrier(0);
    pair_load_all(0, std::false_type{});
    pp_static_for<LB>([&](auto c) { stage_load(0, std::integral_constant<int, LA + decltype(c)::value>{}); });
    pair_load_all(1, std::true_type{});
    __builtin_amdgcn_sched_barrier(0);
    if (tid < BN) s_ws[tid] = c_mine.ws, s_bias[tid] = c_mine.bias, s_corr[tid] = c_mine.corr;
    __builtin_amdgcn_s_waitcnt(pp_vmcnt_imm(2 * LB));  // stage 0 has landed: only B(1,2) may be outstanding
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);

    // Row scales of this lane's TM rows, fetched during the wavefront's last read phase.
    float as_row[TM];
    auto fetch_params = [&]() {
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            const int m = wm0 + 16 * i + (lane & 15);
            as_row[i] = g.a_scale ? g.a_scale[(g.a_scale_per_row && m < g.M) ? m : 0] : 1.0f;
        }
    };
    // One k step of a wavefront: a read phase (the step's fragments, then the refill of operand
    // OP = u % 2 for the stages u+2, u+3, whose buffers held the stages u-2 and u-1: their last
    // readers finished in phase 2u-1), the barrier, and an MFMA phase of nothing but the 44
    // matrix instructions.  The direct loads are issued in the read phase by both groups: a
    // load instruction between two MFMAs of the same wavefront holds up the second one by
    // about 20 cycles (measured: 113 k cycles for the 64 steps with group 0's loads between its MFMAs,
    // 98 k with them here; 92 k is the MFMAs alone).  When the wavefront waits for its loads of stage u+1, what
    // it issued later is one load of the pair's second stage plus this step's pair.
    auto step = [&](int u, auto op_tag, bool trailing_barrier) {
        constexpr int kAllowed = 1 + 2 * (decltype(op_tag)::value ? LB : LA);
        read_frags(u);
        pair_load_all(u + 2, op_tag);
        if (u == nk - 1) fetch_params();
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_waitcnt(pp_vmcnt_imm(kAllowed));
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        compute();
        __builtin_amdgcn_sched_barrier(0);
        if (trailing_barrier) __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
    };
    // Group 0 reads in the even phases and computes in the odd ones, group 1 one phase later;
    // both pass the same number of barriers (group 1 skips the one after its last MFMAs).
    if (group == 1) {
        __builtin_amdgcn_s_barrier();  // phase 0 belongs to group 0
        __builtin_amdgcn_sched_barrier(0);
    }
    {
        int u = 0;
        for (; u + 1 < nk; u += 2) {
            step(u, std::false_type{}, true);
            step(u + 1, std::true_type{}, group == 0 || u + 2 < nk);
        }
        if (u < nk) step(u, std::false_type{}, group == 0);
    }
    // ---- epilogue: no staging through LDS and no barrier; group 0 runs it while group 1 still
    // issues its last MFMAs.
    __builtin_amdgcn_s_waitcnt(pp_vmcnt_imm(0));  // no direct load may land in LDS after this wavefront has ended
    float r_lo = __builtin_inff(), r_hi = -__builtin_inff();
    int r_nan = 0;
    pp_epilogue<TM, TN, MODE>(g, acc, as_row, s_ws, s_bias, s_corr, n0, wm0, wn0, lane, rot, r_lo, r_hi, r_nan);
    // one block per tile: the block's slot is the tile's (every wavefront has passed the same
    // number of barriers by now)
    if (MODE == OUT_F32X && g.range != nullptr) range_block_store(g.range, r_lo, r_hi, r_nan);
}

template <class Cfg, int MODE>
int launch_pp_mode(const GemmArgs& g, hipStream_t st) {
    const void* fn = reinterpret_cast<const void*>(qgemm_pp_kernel<Cfg, MODE>);
    static DeviceOnce attr_once;
    if (int rc = allow_dynamic_lds(attr_once, fn, Cfg::SMEM)) return rc;
    const int tiles = ((g.M + Cfg::BM - 1) / Cfg::BM) * ((g.N + Cfg::BN - 1) / Cfg::BN);
    GemmArgs copy = g;
    void* kargs[] = {&copy};
    LQ_HIP(hipLaunchKernel(fn, dim3(tiles), dim3(Cfg::THREADS), kargs, Cfg::SMEM, st));
    return LQ_OK;
}

template <class Cfg>
int launch_pp(const GemmArgs& g, hipStream_t st) {
    LQ_REQUIRE(g.K > 0 && g.K % 64 == 0, LQ_ERR_SHAPE, "ping-pong kernel: K = %d is not a multiple of 64", g.K);
    LQ_REQUIRE(size_t(g.M) * g.K < 0xffffffffull && size_t(g.N) * g.K < 0xffffffffull, LQ_ERR_SHAPE,
               "ping-pong kernel: an operand of 4 GiB or more");
    if (g.gelu || g.range != nullptr) {
        LQ_REQUIRE(g.out_mode == OUT_F32, LQ_ERR_VALUE, "ping-pong kernel: GELU / a kept range go with float32 output");
        const long tiles = long((g.M + Cfg::BM - 1) / Cfg::BM) * ((g.N + Cfg::BN - 1) / Cfg::BN);
        LQ_REQUIRE(g.range == nullptr || tiles <= kRangeSlots, LQ_ERR_SHAPE,
                   "ping-pong kernel: %ld tiles are too many for a kept range", tiles);
        return launch_pp_mode<Cfg, OUT_F32X>(g, st);
    }
    switch (g.out_mode) {
    case OUT_ACC_I32: return launch_pp_mode<Cfg, OUT_ACC_I32>(g, st);
    case OUT_F32: return launch_pp_mode<Cfg, OUT_F32>(g, st);
    case OUT_F16: return launch_pp_mode<Cfg, OUT_F16>(g, st);
    case OUT_REQUANT_I8:
        if (g.join_q != nullptr) return launch_pp_mode<Cfg, OUT_REQUANT_JOIN>(g, st);
        return launch_pp_mode<Cfg, OUT_REQUANT_I8>(g, st);
    default: return launch_pp_mode<Cfg, OUT_FAKEQUANT_F32>(g, st);
    }
}

using PPCfg352 = PPCfg<256, 352, 4, 2, 4>;
using PPCfg256 = PPCfg<256, 256, 4, 2, 4>;
using PPCfg192 = PPCfg<256, 192, 4, 2, 4>;
// shorter tiles for row counts that 256-row tiles split badly over the 256 CUs (12 608 rows x 768
// columns: 200 tiles of 256 x 192, but 228 of 224 x 192 and 237 of 160 x 256, each with less work)
using PPCfg224x192 = PPCfg<224, 192, 2, 4, 4>;
using PPCfg160x256 = PPCfg<160, 256, 2, 4, 4>;

}  // namespace
}  // namespace lq
