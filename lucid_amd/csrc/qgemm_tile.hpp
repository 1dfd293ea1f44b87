// MFMA tile kernel of the int8 GEMM / implicit-GEMM convolution: template and
// launcher.  Included by one small translation unit per tile shape, so the
// shapes compile in parallel.
#pragma once
#include "common.hpp"
#include "qgemm.hpp"
#include "qepilogue.hpp"
#include "range_slots.hpp"

#include <type_traits>

namespace lq {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef unsigned v4u __attribute__((ext_vector_type(4)));

#define LQ_GPTR(p) ((__attribute__((address_space(1))) void*)(p))
#define LQ_LPTR(p) ((__attribute__((address_space(3))) void*)(p))

// ---------------------------------------------------------------- tile kernel
// Compile-time shape of one tile kernel.
//   BM x BN x BK : block tile (BK bytes of k per LDS stage)
//   WM x WN      : wavefront grid; each wavefront owns (BM/WM) x (BN/WN) outputs
//                  as TM x TN MFMA tiles of 32 x 32
//   STAGES       : LDS stages; STAGES-1 of them are in flight from global memory
//   MINWAVES     : wavefronts per SIMD the register budget must allow
template <int BM_, int BN_, int BK_, int WM_, int WN_, int STAGES_, int MINWAVES_>
struct TileCfg {
    static constexpr int BM = BM_, BN = BN_, BK = BK_, WM = WM_, WN = WN_, STAGES = STAGES_;
    static constexpr int MINWAVES = MINWAVES_;
    static constexpr int THREADS = WM * WN * 64;
    static constexpr int TM = BM / WM / 32, TN = BN / WN / 32;
    static constexpr int C = BK / 16;              // 16-byte chunks per LDS row
    static constexpr int R = 16 / C;               // LDS rows per 256 bytes (one pass over 64 banks)
    static constexpr int ROWS_PER_PASS = THREADS / C;
    static constexpr int PA = BM / ROWS_PER_PASS, PB = BN / ROWS_PER_PASS;
    static constexpr int KSTEPS = BK / 32;
    static constexpr int STAGE_BYTES = (BM + BN) * BK;
    // Three blocks per CU leave 168 registers per lane and 53 KB of LDS per block:
    // fragments are then read just before use (the other wavefronts cover the
    // latency) and the epilogue stages 16 rows at a time.
    static constexpr bool PIPE = MINWAVES_ < 3;
    static constexpr int EPI_ROWS = MINWAVES_ < 3 ? 32 : 16;
    // words per staged output row: a multiple of 4 (16-byte reads) that puts row
    // r + 4 - the upper half-wavefront's row - 32 banks away from row r
    static constexpr int STAGE_STRIDE = TN * 32 + 8;
    static constexpr int STAGE_WORDS = EPI_ROWS * STAGE_STRIDE;
    static constexpr int EPI_BYTES = 4 * BM + THREADS / 64 * STAGE_WORDS * 4;
    static constexpr int SMEM = STAGES * STAGE_BYTES > EPI_BYTES ? STAGES * STAGE_BYTES : EPI_BYTES;
    static_assert(BK == 64 || BK == 128, "BK is 64 or 128 bytes");
    static_assert(ROWS_PER_PASS % 16 == 0 && BM % ROWS_PER_PASS == 0 && BN % ROWS_PER_PASS == 0, "");
    static_assert((STAGES - 2) * (PA + PB) <= 63, "vmcnt is a 6-bit counter");
};

// s_waitcnt immediate that waits for vmcnt <= n only (gfx9 encoding:
// vmcnt in bits [3:0] and [15:14], expcnt [6:4], lgkmcnt [11:8]).
constexpr int vmcnt_imm(int n) { return (n & 0xF) | ((n >> 4) << 14) | (0x7 << 4) | (0xF << 8); }

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

// Wavefront-private LDS traffic needs no workgroup barrier: one wavefront's LDS
// instructions execute in order.  This only keeps the compiler from moving
// accesses across the point.
__device__ __forceinline__ void wave_lds_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// Epilogue of one wavefront's sub-tile, in 32-row bands (or half bands).  The
// MFMA result layout gives a lane one column and sixteen scattered rows; the
// band is turned through a wavefront-private LDS area so that a lane ends up
// with four consecutive columns of one row and the wavefront writes contiguous
// row segments.  `interior` (uniform): the whole tile lies inside the output
// and rows are vector-aligned, so the stores need no per-lane tests.  `prescaled`
// (uniform): cp[].ws already carries the (single) activation scale, s_as is not read.
template <class Cfg, int MODE>
__device__ __forceinline__ void tile_epilogue(const GemmArgs& g, v16i (&acc)[Cfg::TM][Cfg::TN],
                                              const ColParams (&cp)[Cfg::TN], const float* s_as,
                                              uint32_t* stage, int m0, int n0, int n_limit, int wm,
                                              int wn, int lane, float S, float Z, bool interior,
                                              bool prescaled, float& r_lo, float& r_hi, int& r_nan) {
    constexpr int TM = Cfg::TM, TN = Cfg::TN, STRIDE = Cfg::STAGE_STRIDE;
    constexpr int QUADS_PER_ROW = TN * 8;            // four-column groups per staged row
    constexpr int EPI_ROWS = Cfg::EPI_ROWS;          // rows staged at a time (32 or 16)
    constexpr int PARTS = 32 / EPI_ROWS, RPP = 16 / PARTS;
    constexpr int PASSES = EPI_ROWS * QUADS_PER_ROW / 64;
    constexpr int ROWS_PER_PASS = 64 / QUADS_PER_ROW;
    static_assert(64 % QUADS_PER_ROW == 0 && RPP % 4 == 0, "");
    const int esize = MODE == OUT_F16 ? 2 : ((MODE == OUT_REQUANT_I8 || MODE == OUT_REQUANT_JOIN) ? 1 : 4);
    const bool vec_ok = (g.ldo % 4 == 0) && (reinterpret_cast<uintptr_t>(g.out) % (4 * esize) == 0);
    const int row0 = lane / QUADS_PER_ROW, cq = (lane % QUADS_PER_ROW) * 4;
    constexpr bool kRequant = MODE == OUT_REQUANT_I8 || MODE == OUT_REQUANT_JOIN || MODE == OUT_FAKEQUANT_F32;
    const QGrid G = make_qgrid(S, Z, float(g.out_qmin), float(g.out_qmax), kRequant, g.relu != 0,
                               MODE == OUT_REQUANT_I8);
    JoinParams jp;
    if (MODE == OUT_REQUANT_JOIN) {
        jp = load_join(g, G, true);
        interior = interior && jp.k2_exact;  // the vector path subtracts the partner's offsets in one step
    }
    const CodePack cpk = make_code_pack<MODE>(g, MODE == OUT_REQUANT_JOIN ? jp.out : G);
    // running range of what this lane stores (float32 output with a kept range only)
    const bool keep = MODE == OUT_F32X && g.range != nullptr;
    auto track = [&](uint32_t bits) {
        const float y = __uint_as_float(bits);
        r_nan |= (y != y);
        r_lo = fminf(r_lo, y);
        r_hi = fmaxf(r_hi, y);
    };
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int part = 0; part < PARTS; ++part) {
            const int band = wm * (TM * 32) + i * 32 + part * EPI_ROWS;
            const int m_first = m0 + band + row0, n = n0 + wn * (TN * 32) + cq;
            // residual rows of this part, requested before the arithmetic so that
            // their latency is paid under it (`interior` vouches for alignment)
            constexpr bool kFloatOut = MODE == OUT_F32 || MODE == OUT_F16 || MODE == OUT_F32X;
            const bool res_fast = kFloatOut && interior && g.residual != nullptr;
            float4 rv[kFloatOut ? PASSES : 1];
            if (kFloatOut && res_fast) {
                const float* rp = g.residual + size_t(m_first) * size_t(g.ldr) + size_t(n);
#pragma unroll
                for (int p = 0; p < PASSES; ++p)
                    rv[p] = *reinterpret_cast<const float4*>(rp + size_t(p) * ROWS_PER_PASS * size_t(g.ldr));
            }
            // the other operand of a fused join on codes: four codes per row, requested early too
            const bool join_fast = MODE == OUT_REQUANT_JOIN && interior;
            uint32_t jv[MODE == OUT_REQUANT_JOIN ? PASSES : 1];
            if (MODE == OUT_REQUANT_JOIN && join_fast) {
                const int8_t* jq = g.join_q + size_t(m_first) * size_t(g.join_ld) + size_t(n);
#pragma unroll
                for (int p = 0; p < PASSES; ++p)
                    jv[p] = *reinterpret_cast<const uint32_t*>(jq + size_t(p) * ROWS_PER_PASS * size_t(g.join_ld));
            }
            // this lane's rows of the part: groups of four consecutive rows
            if (prescaled) {
#pragma unroll
                for (int rr = 0; rr < RPP; ++rr) {
                    const int r = part * RPP + rr;
                    const int row = 8 * (rr >> 2) + 4 * (lane >> 5) + (rr & 3);  // row within the staged part
#pragma unroll
                    for (int j = 0; j < TN; ++j)
                        stage[row * STRIDE + j * 32 + (lane & 31)] =
                            epilogue_value<MODE, true>(g, acc[i][j][r], 1.0f, cp[j], G);
                }
            } else {
                float as[RPP];
#pragma unroll
                for (int q = 0; q < RPP / 4; ++q) {
                    const float4 v = *reinterpret_cast<const float4*>(s_as + band + 8 * q + 4 * (lane >> 5));
                    as[4 * q] = v.x, as[4 * q + 1] = v.y, as[4 * q + 2] = v.z, as[4 * q + 3] = v.w;
                }
#pragma unroll
                for (int rr = 0; rr < RPP; ++rr) {
                    const int r = part * RPP + rr;
                    const int row = 8 * (rr >> 2) + 4 * (lane >> 5) + (rr & 3);
#pragma unroll
                    for (int j = 0; j < TN; ++j)
                        stage[row * STRIDE + j * 32 + (lane & 31)] =
                            epilogue_value<MODE, false>(g, acc[i][j][r], as[rr], cp[j], G);
                }
            }
            wave_lds_sync();
            const uint32_t* src = stage + row0 * STRIDE + cq;
            if (interior) {
                uint4 v[PASSES];
#pragma unroll
                for (int p = 0; p < PASSES; ++p)
                    v[p] = *reinterpret_cast<const uint4*>(src + p * ROWS_PER_PASS * STRIDE);
                size_t idx = size_t(m_first) * size_t(g.ldo) + size_t(n);
                const size_t step = size_t(ROWS_PER_PASS) * size_t(g.ldo);
                if (kFloatOut && res_fast) {
#pragma unroll
                    for (int p = 0; p < PASSES; ++p) {
                        v[p].x = __float_as_uint(__uint_as_float(v[p].x) + rv[p].x);
                        v[p].y = __float_as_uint(__uint_as_float(v[p].y) + rv[p].y);
                        v[p].z = __float_as_uint(__uint_as_float(v[p].z) + rv[p].z);
                        v[p].w = __float_as_uint(__uint_as_float(v[p].w) + rv[p].w);
                    }
                }
                if (MODE == OUT_REQUANT_JOIN && join_fast) {
#pragma unroll
                    for (int p = 0; p < PASSES; ++p) {
                        const uint32_t b = jv[p] ^ 0x80808080u;  // stored bytes + 128, all four
                        v[p].x = join_code_biased(jp, v[p].x, float(b & 0xffu));
                        v[p].y = join_code_biased(jp, v[p].y, float((b >> 8) & 0xffu));
                        v[p].z = join_code_biased(jp, v[p].z, float((b >> 16) & 0xffu));
                        v[p].w = join_code_biased(jp, v[p].w, float(b >> 24));
                    }
                }
                if (MODE == OUT_F32X && keep) {
#pragma unroll
                    for (int p = 0; p < PASSES; ++p) track(v[p].x), track(v[p].y), track(v[p].z), track(v[p].w);
                }
#pragma unroll
                for (int p = 0; p < PASSES; ++p) {
                    store_vec4<MODE>(g, idx, v[p], cpk);
                    idx += step;
                }
            } else {
#pragma unroll 4
                for (int p = 0; p < PASSES; ++p) {
                    uint4 v = *reinterpret_cast<const uint4*>(src + p * ROWS_PER_PASS * STRIDE);
                    const int m = m_first + p * ROWS_PER_PASS;
                    if (m < g.M && n < n_limit) {
                        v.x = finish_value<MODE>(g, v.x, m, n, jp);
                        if (n + 1 < n_limit) v.y = finish_value<MODE>(g, v.y, m, n + 1, jp);
                        if (n + 2 < n_limit) v.z = finish_value<MODE>(g, v.z, m, n + 2, jp);
                        if (n + 3 < n_limit) v.w = finish_value<MODE>(g, v.w, m, n + 3, jp);
                        if (MODE == OUT_F32X && keep) {
                            track(v.x);
                            if (n + 1 < n_limit) track(v.y);
                            if (n + 2 < n_limit) track(v.z);
                            if (n + 3 < n_limit) track(v.w);
                        }
                        const size_t idx = size_t(m) * size_t(g.ldo) + size_t(n);
                        if (vec_ok && n + 4 <= n_limit) {
                            store_vec4<MODE>(g, idx, v, cpk);
                        } else {
                            store_scalar<MODE>(g, idx, v.x, cpk);
                            if (n + 1 < n_limit) store_scalar<MODE>(g, idx + 1, v.y, cpk);
                            if (n + 2 < n_limit) store_scalar<MODE>(g, idx + 2, v.z, cpk);
                            if (n + 3 < n_limit) store_scalar<MODE>(g, idx + 3, v.w, cpk);
                        }
                    }
                }
            }
            wave_lds_sync();
        }
    }
}

// LDS stage layout: BM rows of A then BN rows of B, each row BK bytes; the
// 16-byte chunk kc of row r sits at physical chunk kc ^ ((r / R) % C).  With
// 64 LDS banks a ds_read_b128 serves 16 lanes per pass; under this swizzle the
// 16 fragment rows of a pass fall on 16 different bank groups.  A wavefront's
// direct global->LDS load writes 1 KiB of consecutive slots, so the swizzle is
// applied on the global side: a lane fetches the chunk that belongs in its slot.
// Balanced split of `total` k-iterations over `workers`: the first `rem` workers
// take one iteration more.
struct IterSplit {
    int per, rem;
    __host__ __device__ IterSplit(long total, int workers)
        : per(int(total / workers)), rem(int(total % workers)) {}
    __host__ __device__ long begin(int w) const { return long(w) * per + (w < rem ? w : rem); }
    __host__ __device__ int owner(long it) const {
        const long cut = long(rem) * (per + 1);
        return it < cut ? int(it / (per + 1)) : rem + int((it - cut) / per);
    }
};

// SK = false: one block per tile (blockIdx.x -> tile, blockIdx.y -> group).
// SK = true ("stream-K"): gridDim.x workers split the tiles' k-iterations evenly;
// a worker's range may start and end in the middle of a tile.  A tile touched by
// several workers is finished without anybody waiting: every contributor stores
// its int32 partial accumulators into its own slab, then bumps the tile's
// arrival counter; whoever arrives last adds the other slabs to its registers
// and runs the epilogue.  Integer partial sums add exactly, so the result does
// not depend on who arrives when.
template <class Cfg, int MODE, int CONV, bool SK>
__global__ __launch_bounds__(Cfg::THREADS, Cfg::MINWAVES) void qgemm_tile_kernel(GemmArgs g) {
    constexpr int BM = Cfg::BM, BN = Cfg::BN, BK = Cfg::BK, TM = Cfg::TM, TN = Cfg::TN;
    constexpr int C = Cfg::C, R = Cfg::R, PA = Cfg::PA, PB = Cfg::PB, STAGES = Cfg::STAGES;
    constexpr int THREADS = Cfg::THREADS, KSTEPS = Cfg::KSTEPS;
    extern __shared__ __attribute__((aligned(1024))) int8_t smem[];
    __shared__ int s_flag;
    const int tid = threadIdx.x, lane = tid & 63;
    // wavefront index as a scalar: LDS stage addresses (the M0 operand of the direct
    // loads) then need no per-load readfirstlane
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int tiles_m = (g.M + BM - 1) / BM, tiles_n = (g.N + BN - 1) / BN;
    const int n_base = int(blockIdx.y) * g.N;  // first column of this group (0 for a plain GEMM)
    const int n_limit = n_base + g.N;
    const int wm = wave / Cfg::WN, wn = wave % Cfg::WN;
    const int nk = (g.K + BK - 1) / BK;

    // global -> LDS addressing: in pass `it` this lane fills the slot of row
    // it*ROWS_PER_PASS + tid/C, physical chunk tid%C.  ROWS_PER_PASS is a multiple
    // of 16, so the swizzle term - and the logical chunk fetched - is the same in
    // every pass.
    const int row_in_pass = tid / C;
    const int kc = (tid % C) ^ ((row_in_pass / R) % C);
    // fragment addressing: lane holds row (lane & 31), 16 bytes of k at chunk
    // 2*kk + (lane >> 5) of the current 32-wide k step
    const int frag_row = lane & 31;
    const int frag_half = lane >> 5;
    const int a_row_base = (wm * (TM * 32) + frag_row) * BK;
    const int b_row_base = BM * BK + (wn * (TN * 32) + frag_row) * BK;
    const int sw = (frag_row / R) % C;

    v16i acc[TM][TN];

    // Epilogue operands of the current tile.  They are fetched while the last
    // k-iteration of the tile runs, so their latency is paid under its MFMAs.
    static_assert(BM <= THREADS, "one row scale per thread");
    ColParams cp[TN];
    float as_mine = 1.0f;  // a_scale of row m0 + tid
    bool fetched = false;
    auto fetch_params = [&](int tm, int tn) {
        const int m0 = tm * BM, n0 = n_base + tn * BN;
        int n[TN];
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            n[j] = n0 + wn * (TN * 32) + j * 32 + (lane & 31);
            n[j] = n[j] < n_limit ? n[j] : n_limit - 1;
        }
        load_cols(g, n, cp);
        const int m = m0 + tid;
        as_mine = g.a_scale ? g.a_scale[(g.a_scale_per_row && m < g.M) ? m : 0] : 1.0f;
        fetched = true;
    };

    // k-iterations [kb, ke) of tile (tm, tn) into acc (zeroed first); ke == nk
    // also fetches the tile's epilogue operands
    auto run_segment = [&](int tm, int tn, int kb, int ke) {
        fetched = false;
        const int m0 = tm * BM, n0 = n_base + tn * BN;
        unsigned a_off[PA], b_off[PB];
        int a_hw[PA];  // CONV: top-left input coordinate of the pixel, (ih0 << 16) | (iw0 & 0xffff)
        int a_d[CONV == 2 ? PA : 1];  // volumetric: its first depth slice
        const int a_rows = g.M - m0, b_rows = n_limit - n0;  // valid rows in this tile (>= 1)
#pragma unroll
        for (int it = 0; it < PA; ++it) {
            int r = it * Cfg::ROWS_PER_PASS + row_in_pass;
            r = r < a_rows ? r : a_rows - 1;  // clamp: reads stay in bounds, rows are masked at the store
            if constexpr (CONV == 2) {
                const int m = m0 + r;
                const int plane = g.cOH * g.cOW, vol = g.cOD * plane;
                const int b = m / vol, rem = m - b * vol;
                const int od = rem / plane, rem2 = rem - od * plane;
                const int oh = rem2 / g.cOW, ow = rem2 - oh * g.cOW;
                const int id0 = od * g.csd - g.cpd, ih0 = oh * g.csh - g.cph, iw0 = ow * g.csw - g.cpw;
                a_hw[it] = (ih0 << 16) | (iw0 & 0xffff);
                a_d[it] = id0;
                a_off[it] = unsigned(((b * g.cD + id0) * g.cH + ih0) * g.cW + iw0) * unsigned(g.cCin) +
                            unsigned(int(blockIdx.y) * g.cCg);
            } else if (CONV) {
                const int m = m0 + r;
                const int pix = g.cOH * g.cOW;
                const int b = m / pix, rem = m - b * pix;
                const int oh = rem / g.cOW, ow = rem - oh * g.cOW;
                const int ih0 = oh * g.csh - g.cph, iw0 = ow * g.csw - g.cpw;
                a_hw[it] = (ih0 << 16) | (iw0 & 0xffff);
                // may wrap for ih0 / iw0 < 0; it is only used after the bounds check,
                // together with a tap offset that brings it back in range
                a_off[it] = unsigned((b * g.cH + ih0) * g.cW + iw0) * unsigned(g.cCin) +
                            unsigned(int(blockIdx.y) * g.cCg);
            } else {
                a_hw[it] = 0;
                a_off[it] = unsigned(r) * unsigned(g.K) + unsigned(kc * 16);
            }
        }
#pragma unroll
        for (int it = 0; it < PB; ++it) {
            int r = it * Cfg::ROWS_PER_PASS + row_in_pass;
            r = r < b_rows ? r : b_rows - 1;
            b_off[it] = unsigned(r) * unsigned(g.K) + unsigned(kc * 16);
        }
        const int8_t* a_tile = CONV ? g.cx : g.a + size_t(m0) * g.K;
        const int8_t* b_tile = g.w + size_t(n0) * g.K;
        const int k_end = ke * BK < g.K ? ke * BK : g.K;  // nothing is fetched past the segment
        // CONV: filter tap (kh, kw) and channel offset of this lane's 16 bytes in the next stage
        // to be loaded.  Stages are loaded in k order, BK bytes apart, so the position is found
        // by division once per segment and then stepped (the divisions by run-time values cost
        // more than the MFMAs of a small tile's k-iteration).
        int c_ci0 = 0, c_kh = 0, c_kw = 0, c_kd = 0;
        if (CONV) {
            const int k = kb * BK + kc * 16;
            int tap = k / g.cCg;
            c_ci0 = k - tap * g.cCg;
            if (CONV == 2) {
                const int taps_hw = g.cKH * g.cKW;
                c_kd = tap / taps_hw;
                tap -= c_kd * taps_hw;
            }
            c_kh = tap / g.cKW;
            c_kw = tap - c_kh * g.cKW;
        }

        // `full` (compile time): the whole stage lies inside K, so no lane needs the
        // zero source and the address is a uniform base plus a per-lane offset
        auto load_stage = [&](int k0, int8_t* stage, auto full) {
            const int k = k0 + kc * 16;
            const bool in_k = k < k_end;  // K-tail chunks and look-ahead stages: zeros
            int8_t* sa = stage + wave * 1024;
            int8_t* sb = stage + BM * BK + wave * 1024;
            if (!CONV && decltype(full)::value) {
                const int8_t* ab = a_tile + k0;
                const int8_t* bb = b_tile + k0;
#pragma unroll
                for (int it = 0; it < PA; ++it)
                    __builtin_amdgcn_global_load_lds(LQ_GPTR(ab + a_off[it]), LQ_LPTR(sa + it * (THREADS * 16)), 16, 0, 0);
#pragma unroll
                for (int it = 0; it < PB; ++it)
                    __builtin_amdgcn_global_load_lds(LQ_GPTR(bb + b_off[it]), LQ_LPTR(sb + it * (THREADS * 16)), 16, 0, 0);
                return;
            }
            if (CONV) {
                // this lane's 16 bytes lie inside one filter tap (Cg % 16 == 0)
                const int ci0 = c_ci0, kh = c_kh, kw = c_kw, kd = c_kd;
                c_ci0 += BK;  // on to the next stage
                while (c_ci0 >= g.cCg) {
                    c_ci0 -= g.cCg;
                    if (++c_kw == g.cKW) {
                        c_kw = 0, ++c_kh;
                        if (CONV == 2 && c_kh == g.cKH) c_kh = 0, ++c_kd;
                    }
                }
                const int dh = kh * g.cdh, dw = kw * g.cdw, dd = CONV == 2 ? kd * g.cdd : 0;
                const unsigned delta = unsigned((dd * g.cH + dh) * g.cW + dw) * unsigned(g.cCin) + unsigned(ci0);
#pragma unroll
                for (int it = 0; it < PA; ++it) {
                    const int ih = (a_hw[it] >> 16) + dh;
                    const int iw = int(short(a_hw[it] & 0xffff)) + dw;
                    bool ok = in_k && unsigned(ih) < unsigned(g.cH) && unsigned(iw) < unsigned(g.cW);
                    if constexpr (CONV == 2) ok = ok && unsigned(a_d[it] + dd) < unsigned(g.cD);
                    const int8_t* src = ok ? a_tile + (a_off[it] + delta) : g.pad_src;
                    __builtin_amdgcn_global_load_lds(LQ_GPTR(src), LQ_LPTR(sa + it * (THREADS * 16)), 16, 0, 0);
                }
            } else {
#pragma unroll
                for (int it = 0; it < PA; ++it) {
                    const int8_t* src = in_k ? a_tile + k0 + a_off[it] : g.zeros;
                    __builtin_amdgcn_global_load_lds(LQ_GPTR(src), LQ_LPTR(sa + it * (THREADS * 16)), 16, 0, 0);
                }
            }
#pragma unroll
            for (int it = 0; it < PB; ++it) {
                const int8_t* src = in_k ? b_tile + k0 + b_off[it] : g.zeros;
                __builtin_amdgcn_global_load_lds(LQ_GPTR(src), LQ_LPTR(sb + it * (THREADS * 16)), 16, 0, 0);
            }
        };

        auto read_frags = [&](const int8_t* stage, int kk, v4i (&af)[TM], v4i (&bf)[TN]) {
            const int pc = ((kk * 2 + frag_half) ^ sw) * 16;
#pragma unroll
            for (int i = 0; i < TM; ++i)
                af[i] = *reinterpret_cast<const v4i*>(stage + a_row_base + i * 32 * BK + pc);
#pragma unroll
            for (int j = 0; j < TN; ++j)
                bf[j] = *reinterpret_cast<const v4i*>(stage + b_row_base + j * 32 * BK + pc);
        };

#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;

        // All STAGES buffers are kept in flight.  The fragments of k step kk+1
        // are fetched from LDS while the MFMAs of step kk run; the hand-over to
        // the next stage (wait for its data, barrier, fetch its first fragments,
        // refill the buffer just drained) sits inside the last k step of the
        // current stage, so its latency is covered by that step's MFMAs.  Stages
        // past the end are loaded from the block of zeros, which keeps the number
        // of outstanding loads - and so the vmcnt to wait for - constant.
#pragma unroll
        for (int s = 0; s < STAGES; ++s)
            load_stage((kb + s) * BK, smem + s * Cfg::STAGE_BYTES, std::false_type{});
        __builtin_amdgcn_s_waitcnt(vmcnt_imm((STAGES - 1) * (PA + PB)));
        __syncthreads();

        if constexpr (TM * TN == 1) {
            // One MFMA per k step cannot cover the LDS latency of the next step's fragments, so
            // a wavefront holds the fragments of a whole stage: the registers of step kk are
            // refilled from the next stage right after the MFMA that consumed them, KSTEPS
            // MFMAs ahead of their use.  Two accumulators (even / odd steps) keep consecutive
            // MFMAs independent.  The hand-over (wait for the next stage's data, barrier) comes
            // first in the iteration, the refill of the stage just drained last, its address
            // arithmetic running beside the MFMAs.
            v4i fa[KSTEPS], fb[KSTEPS];
            v16i acc_odd;
#pragma unroll
            for (int r = 0; r < 16; ++r) acc_odd[r] = 0;
            auto read_step = [&](const int8_t* stage, int kk) {
                const int pc = ((kk * 2 + frag_half) ^ sw) * 16;
                fa[kk] = *reinterpret_cast<const v4i*>(stage + a_row_base + pc);
                fb[kk] = *reinterpret_cast<const v4i*>(stage + b_row_base + pc);
            };
#pragma unroll
            for (int kk = 0; kk < KSTEPS; ++kk) read_step(smem, kk);
            auto stage_steps = [&](int t, bool last_stage, auto full) {
                const int slot = t % STAGES;
                int8_t* cur = smem + slot * Cfg::STAGE_BYTES;
                const int8_t* nxt = smem + (slot + 1 == STAGES ? 0 : slot + 1) * Cfg::STAGE_BYTES;
                if (!last_stage) {
                    // lgkmcnt(0): this wavefront's reads of `cur` have landed in registers, so after
                    // the barrier nobody still reads the buffer that is refilled below
                    __builtin_amdgcn_s_waitcnt(vmcnt_imm((STAGES - 2) * (PA + PB)) & ~(0xF << 8));
                    __syncthreads();
                }
#pragma unroll
                for (int kk = 0; kk < KSTEPS; ++kk) {
                    if (kk & 1)
                        acc_odd = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[kk], fb[kk], acc_odd, 0, 0, 0);
                    else
                        acc[0][0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[kk], fb[kk], acc[0][0], 0, 0, 0);
                    if (!last_stage) read_step(nxt, kk);
                }
                if (!last_stage) load_stage((kb + t + STAGES) * BK, cur, full);
            };
            const int n_it = ke - kb;
            int n_full = (k_end / BK) - kb - STAGES;
            n_full = n_full < 0 ? 0 : (n_full > n_it - 1 ? n_it - 1 : n_full);
            int t = 0;
            for (; t < n_full; ++t) stage_steps(t, false, std::true_type{});
            for (; t + 1 < n_it; ++t) stage_steps(t, false, std::false_type{});
            if (ke == nk) fetch_params(tm, tn);
            stage_steps(n_it - 1, true, std::false_type{});
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[0][0][r] += acc_odd[r];
            __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));  // drain the zero-filled look-ahead stages
            __syncthreads();                            // all fragment reads done before LDS is reused
            return;
        }

        v4i af[2][TM], bf[2][TN];
        if (Cfg::PIPE) read_frags(smem, 0, af[0], bf[0]);

        auto k_steps = [&](int t, bool last_stage, auto full) {  // t counts from 0 within the segment
            const int slot = t % STAGES;
            int8_t* cur = smem + slot * Cfg::STAGE_BYTES;
            const int8_t* nxt = smem + (slot + 1 == STAGES ? 0 : slot + 1) * Cfg::STAGE_BYTES;
            if (!Cfg::PIPE) {
                // fragments are read right before their MFMAs; the CU's other
                // wavefronts fill the wait
#pragma unroll
                for (int kk = 0; kk < KSTEPS; ++kk) {
                    read_frags(cur, kk, af[0], bf[0]);
#pragma unroll
                    for (int i = 0; i < TM; ++i)
#pragma unroll
                        for (int j = 0; j < TN; ++j)
                            acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[0][i], bf[0][j], acc[i][j], 0, 0, 0);
                }
                if (!last_stage) {
                    __builtin_amdgcn_s_waitcnt(vmcnt_imm((STAGES - 2) * (PA + PB)));
                    __syncthreads();  // stage t+1 is complete in LDS; nobody reads stage t any more
                    load_stage((kb + t + STAGES) * BK, cur, full);
                }
                return;
            }
#pragma unroll
            for (int kk = 0; kk < KSTEPS; ++kk) {
                if (kk + 1 < KSTEPS) {
                    read_frags(cur, kk + 1, af[(kk + 1) & 1], bf[(kk + 1) & 1]);
                } else if (!last_stage) {
                    __builtin_amdgcn_s_waitcnt(vmcnt_imm((STAGES - 2) * (PA + PB)));
                    __syncthreads();  // stage t+1 is complete in LDS; nobody reads stage t any more
                    read_frags(nxt, 0, af[0], bf[0]);
                    load_stage((kb + t + STAGES) * BK, cur, full);
                }
#pragma unroll
                for (int i = 0; i < TM; ++i)
#pragma unroll
                    for (int j = 0; j < TN; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[kk & 1][i], bf[kk & 1][j],
                                                                          acc[i][j], 0, 0, 0);

                // issue order inside the step: one MFMA, then all LDS reads of the next
                // step's fragments, then the other MFMAs.  The compiler waits for every
                // outstanding LDS read before the first MFMA of a step, so the reads go
                // out as early as possible; the MFMA goes first so that this wait is not
                // held up by a read issued just before it.
                if (kk + 1 < KSTEPS) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                    __builtin_amdgcn_sched_group_barrier(0x100, TM + TN, 0);
                    __builtin_amdgcn_sched_group_barrier(0x008, TM * TN - 1, 0);
                } else if (!last_stage) {
                    // hand-over step: the refill loads go out one per MFMA after the reads
                    constexpr int NL = PA + PB < TM * TN - 1 ? PA + PB : TM * TN - 1;
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                    __builtin_amdgcn_sched_group_barrier(0x100, TM + TN, 0);
#pragma unroll
                    for (int x = 0; x < NL; ++x) {
                        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                        __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
                    }
                    __builtin_amdgcn_sched_group_barrier(0x020, PA + PB - NL, 0);
                    __builtin_amdgcn_sched_group_barrier(0x008, TM * TN - 1 - NL, 0);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        };
        const int n_it = ke - kb;
        // iterations whose refill stage (t + STAGES) lies wholly inside K come first
        int n_full = (k_end / BK) - kb - STAGES;
        n_full = n_full < 0 ? 0 : (n_full > n_it - 1 ? n_it - 1 : n_full);
        int t = 0;
        for (; t < n_full; ++t) k_steps(t, false, std::true_type{});
        for (; t + 1 < n_it; ++t) k_steps(t, false, std::false_type{});
        if (ke == nk) fetch_params(tm, tn);
        k_steps(n_it - 1, true, std::false_type{});
        __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));  // drain the zero-filled look-ahead stages
        __syncthreads();                            // all fragment reads done before LDS is reused
    };

    // Row scales are staged in LDS and column parameters are loaded before the
    // first store, so no global load sits between the stores.
    auto run_epilogue = [&](int tm, int tn) {
        const int m0 = tm * BM, n0 = n_base + tn * BN;
        float* s_as = reinterpret_cast<float*>(smem);
        uint32_t* stage = reinterpret_cast<uint32_t*>(smem + 4 * BM) + wave * Cfg::STAGE_WORDS;
        if (!fetched) fetch_params(tm, tn);  // a shared tile finished by a worker that did not end it
        if (tid < BM) s_as[tid] = as_mine;
        float S = 1.0f, Z = 0.0f;
        if (MODE == OUT_REQUANT_I8 || MODE == OUT_REQUANT_JOIN || MODE == OUT_FAKEQUANT_F32) {
            S = g.out_scale[0];
            Z = g.out_zp[0];
        }
        const int esize = MODE == OUT_F16 ? 2 : ((MODE == OUT_REQUANT_I8 || MODE == OUT_REQUANT_JOIN) ? 1 : 4);
        const bool interior = m0 + BM <= g.M && n0 + BN <= n_limit && g.ldo % 4 == 0 &&
                              reinterpret_cast<uintptr_t>(g.out) % (4 * esize) == 0 &&
                              (g.residual == nullptr ||
                               (g.ldr % 4 == 0 && reinterpret_cast<uintptr_t>(g.residual) % 16 == 0)) &&
                              (g.join_q == nullptr ||
                               (g.join_ld % 4 == 0 && reinterpret_cast<uintptr_t>(g.join_q) % 4 == 0));
        __syncthreads();
        float r_lo = __builtin_inff(), r_hi = -__builtin_inff();
        int r_nan = 0;
        // one activation scale for all rows (always so for a convolution): the kernels that
        // write codes fold it into the column scales (as * ws, the product every element would
        // form) and save each element that multiplication
        const bool prescaled = (MODE == OUT_REQUANT_I8 || MODE == OUT_REQUANT_JOIN) && (CONV || !g.a_scale_per_row);
        if (prescaled) {
#pragma unroll
            for (int j = 0; j < TN; ++j) cp[j].ws = as_mine * cp[j].ws;
        }
        tile_epilogue<Cfg, MODE>(g, acc, cp, s_as, stage, m0, n0, n_limit, wm, wn, lane, S, Z, interior, prescaled,
                                 r_lo, r_hi, r_nan);
        __syncthreads();  // the staging area is the next tile's first LDS stage
        // one block per tile here (the launcher sees to it), so the block's slot is the tile's
        if (MODE == OUT_F32X && !SK && g.range != nullptr) range_block_store(g.range, r_lo, r_hi, r_nan);
    };

    if (!SK) {
        int tm, tn;
        tile_coords(blockIdx.x, gridDim.x, tiles_m, tiles_n, &tm, &tn);
        run_segment(tm, tn, 0, nk);
        run_epilogue(tm, tn);
        return;
    }

    // ---- stream-K over the last g.sk_tiles tile ids, then the other tiles one
    // block per tile (worker w takes tiles w, w + workers, ...).  The shared tiles
    // come first: their partial sums are exchanged while every worker still has a
    // whole tile of its own to compute, and nobody ever waits for anybody.
    constexpr int kAccWords = TM * TN * 16;  // accumulator registers per lane
    const int workers = gridDim.x;
    const int tiles = tiles_m * tiles_n;
    const int dp_tiles = tiles - g.sk_tiles;
    const long total = long(g.sk_tiles) * nk;
    const IterSplit split(total, workers);
    // give every XCD a contiguous range of workers (blocks are dealt round-robin)
    const int wq = workers / 8, wr = workers % 8;
    const int xcd = blockIdx.x % 8;
    const int me = xcd * wq + (xcd < wr ? xcd : wr) + blockIdx.x / 8;
    // same m-fastest walk in groups of 8 m-tiles as tile_coords
    auto coords = [&](int tile, int* tm, int* tn) {
        constexpr int GM = 8;
        const int group_size = GM * tiles_n;
        const int group = tile / group_size;
        const int first_m = group * GM;
        const int gsz = tiles_m - first_m < GM ? tiles_m - first_m : GM;
        const int in_group = tile - group * group_size;
        *tm = first_m + in_group % gsz;
        *tn = in_group / gsz;
    };
    long it = split.begin(me);
    const long it_end = split.begin(me + 1);
    int dp_tile = me;
    int* counters = g.sk_counters + size_t(blockIdx.y) * g.sk_tiles;
    int32_t* slabs = g.sk_slabs + size_t(blockIdx.y) * workers * 2 * size_t(kAccWords) * THREADS;
    // one loop over both kinds of work, so that the segment and the epilogue are
    // instantiated once
    for (;;) {
        int tile, kb, ke, local = 0;
        if (it < it_end) {
            local = int(it / nk);  // index among the shared tiles
            kb = int(it - long(local) * nk);
            ke = (it_end - it) < (nk - kb) ? kb + int(it_end - it) : nk;
            tile = dp_tiles + local;
            it += ke - kb;
        } else if (dp_tile < dp_tiles) {
            tile = dp_tile;
            kb = 0;
            ke = nk;
            dp_tile += workers;
        } else {
            break;
        }
        int tm, tn;
        coords(tile, &tm, &tn);
        run_segment(tm, tn, kb, ke);
        bool finish = true;
        if (!(kb == 0 && ke == nk)) {
            const int w_first = split.owner(long(local) * nk);
            const int w_last = split.owner(long(local) * nk + nk - 1);
            // slab 0 holds a worker's leading partial tile, slab 1 its trailing one
            // (the address is the same in every lane; saying so keeps the buffer
            // descriptor in scalar registers)
            auto slab_of = [&](int w) -> int32_t* {
                const int first_local = int(split.begin(w) / nk);
                const uint64_t p = reinterpret_cast<uint64_t>(
                    slabs + (size_t(w) * 2 + (local == first_local ? 0 : 1)) * kAccWords * THREADS);
                const uint64_t lo = uint32_t(__builtin_amdgcn_readfirstlane(int(uint32_t(p))));
                const uint64_t hi = uint32_t(__builtin_amdgcn_readfirstlane(int(uint32_t(p >> 32))));
                return reinterpret_cast<int32_t*>((hi << 32) | lo);
            };
            // The XCDs' L2 caches are not coherent with each other.  Instead of
            // device-scope fences (which write back and invalidate a whole L2, under
            // the feet of the 63 other blocks that share it), every access to a slab
            // carries device scope itself: write-through stores, cache-bypassing loads.
            // They are plain (non-atomic) buffer accesses with the device-scope bit, so
            // the compiler keeps many of them in flight.
            // 16 bytes per lane and access: chunk q of a lane's accumulators sits at
            // (q * THREADS + tid) * 16 of the slab.
            constexpr unsigned kScopeDevice = 16;  // "sc1" cache-policy bit of buffer accesses
            constexpr unsigned kSlabBytes = kAccWords * THREADS * 4;
            const unsigned lane_off = unsigned(tid) * 16;
            {
                const __amdgpu_buffer_rsrc_t mine =
                    __builtin_amdgcn_make_buffer_rsrc(slab_of(me), 0, kSlabBytes, 0x00020000);
#pragma unroll
                for (int i = 0; i < TM; ++i)
#pragma unroll
                    for (int j = 0; j < TN; ++j)
#pragma unroll
                        for (int q = 0; q < 4; ++q) {
                            const v4u v = {unsigned(acc[i][j][4 * q]), unsigned(acc[i][j][4 * q + 1]),
                                           unsigned(acc[i][j][4 * q + 2]), unsigned(acc[i][j][4 * q + 3])};
                            __builtin_amdgcn_raw_buffer_store_b128(
                                v, mine, lane_off + unsigned(((i * TN + j) * 4 + q) * THREADS * 16), 0, kScopeDevice);
                        }
            }
            __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));  // this wavefront's partials have been written through
            __syncthreads();                            // ... and so have the other wavefronts'
            if (tid == 0)
                s_flag = __hip_atomic_fetch_add(&counters[local], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __syncthreads();
            // the other contributors have all arrived
            finish = __builtin_amdgcn_readfirstlane(s_flag) == (w_last - w_first);
            if (finish && TM * TN * 4 <= 8) {
                // small accumulators (64 x 64 tiles): the slabs of up to kGroup contributors
                // are requested together, one memory round trip for all of them instead of
                // one each.  A slot with no contributor re-reads this worker's own slab and
                // is not added, so that the loads stay unconditional.
                constexpr int kChunks = TM * TN * 4, kGroup = kChunks <= 8 ? 16 / kChunks : 1;
                for (int w0 = w_first; w0 <= w_last; w0 += kGroup) {
                    v4u v[kGroup][kChunks];
#pragma unroll
                    for (int x = 0; x < kGroup; ++x) {
                        const int w = w0 + x;
                        const bool use = w <= w_last && w != me;
                        const __amdgpu_buffer_rsrc_t other =
                            __builtin_amdgcn_make_buffer_rsrc(slab_of(use ? w : me), 0, kSlabBytes, 0x00020000);
#pragma unroll
                        for (int c = 0; c < kChunks; ++c)
                            v[x][c] = __builtin_amdgcn_raw_buffer_load_b128(other, lane_off + unsigned(c * THREADS * 16),
                                                                            0, kScopeDevice);
                    }
#pragma unroll
                    for (int x = 0; x < kGroup; ++x) {
                        const int w = w0 + x;
                        if (w <= w_last && w != me) {
#pragma unroll
                            for (int c = 0; c < kChunks; ++c) {
                                v16i& a = acc[(c / 4) / TN][(c / 4) % TN];
                                a[4 * (c % 4)] += int(v[x][c].x);
                                a[4 * (c % 4) + 1] += int(v[x][c].y);
                                a[4 * (c % 4) + 2] += int(v[x][c].z);
                                a[4 * (c % 4) + 3] += int(v[x][c].w);
                            }
                        }
                    }
                }
                if (tid == 0) counters[local] = 0;  // ready for the next launch
            } else if (finish) {
                for (int w = w_first; w <= w_last; ++w) {
                    if (w == me) continue;
                    const __amdgpu_buffer_rsrc_t other =
                        __builtin_amdgcn_make_buffer_rsrc(slab_of(w), 0, kSlabBytes, 0x00020000);
                    // eight 16-byte loads in flight per lane (the fragment registers of
                    // the main loop are free here), then their 32 additions
                    constexpr int kBatch = (TM * TN * 4) % 8 == 0 ? 8 : 4;
                    static_assert((TM * TN * 4) % kBatch == 0, "");
#pragma unroll
                    for (int c0 = 0; c0 < TM * TN * 4; c0 += kBatch) {
                        v4u v[kBatch];
#pragma unroll
                        for (int c = 0; c < kBatch; ++c)
                            v[c] = __builtin_amdgcn_raw_buffer_load_b128(
                                other, lane_off + unsigned((c0 + c) * THREADS * 16), 0, kScopeDevice);
#pragma unroll
                        for (int c = 0; c < kBatch; ++c) {
                            const int ij = (c0 + c) / 4, q = (c0 + c) % 4;
                            v16i& a = acc[ij / TN][ij % TN];
                            a[4 * q] += int(v[c].x);
                            a[4 * q + 1] += int(v[c].y);
                            a[4 * q + 2] += int(v[c].z);
                            a[4 * q + 3] += int(v[c].w);
                        }
                        __builtin_amdgcn_sched_group_barrier(0x020, kBatch, 0);
                        __builtin_amdgcn_sched_group_barrier(0x002, kBatch * 4, 0);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
                if (tid == 0) counters[local] = 0;  // ready for the next launch
            }
            __syncthreads();
        }
        if (finish) run_epilogue(tm, tn);
    }
}

// Tile shapes.  "big" keeps LDS traffic per MFMA lowest (one block per CU);
// "wide" and "mid" let two or more blocks share a CU so one block's barrier
// and epilogue overlap another's MFMAs, and waste less on ragged M / N.
using CfgBig = TileCfg<256, 256, 128, 2, 2, 2, 1>;
using CfgBig64 = TileCfg<256, 256, 64, 2, 2, 4, 1>;
using CfgWide = TileCfg<256, 128, 64, 2, 2, 3, 2>;
using CfgTall = TileCfg<128, 256, 64, 2, 2, 3, 2>;
using CfgMid = TileCfg<128, 128, 64, 2, 2, 4, 2>;
using CfgN64 = TileCfg<256, 64, 64, 4, 1, 3, 2>;  // 64 output columns (early ResNet stages)
using CfgTall3 = TileCfg<128, 256, 64, 2, 2, 2, 3>;  // three blocks per CU
using CfgMid4 = TileCfg<128, 128, 64, 2, 2, 2, 4>;   // four blocks per CU: short K, latency-bound tiles
using CfgSmall = TileCfg<64, 64, 64, 2, 2, 4, 4>;    // few rows (late convolution stages): more tiles than CUs
// the same tiles over a long K: half the k-iterations (and barriers) at twice the bytes each;
// measured 27 -> 21 us on a 1568 x 512 x 4608 convolution, where a tile's time is the chain
// wait - barrier - LDS read - MFMA of each k-iteration with nothing else on the CU to cover it
using CfgSmallK = TileCfg<64, 64, 128, 2, 2, 4, 2>;
// Eight wavefronts (two per SIMD, wavefront tiles of 128 x 64 and 64 x 64): one wavefront's
// barrier waits and LDS reads are covered by the other's MFMAs.  Measured against the
// four-wavefront shapes of the same block tile: 256 x 256 x 128 +4 % (2.34 against 2.26 POP/s
// at 8192 x 8192 x 4096), 128 x 256 x 64 +4 % on a 2816-column problem but -7 % on large ones.
// (A 4 x 2 wavefront grid gained half as much; raising the wavefront priority around the MFMAs
// lost 8 %; BK = 64 with four stages lost 7 %.)
using CfgBig8 = TileCfg<256, 256, 128, 2, 4, 2, 1>;
using CfgTall8 = TileCfg<128, 256, 64, 2, 4, 3, 2>;

}  // namespace

namespace {

template <class Cfg, int MODE, int CONV>
int launch_tile_mode(const GemmArgs& g, int groups, int schedule, hipStream_t st) {
    const void* fn_dp = reinterpret_cast<const void*>(qgemm_tile_kernel<Cfg, MODE, CONV, false>);
    // the volumetric gather is built for one block per tile only
    const void* fn_sk = reinterpret_cast<const void*>(qgemm_tile_kernel<Cfg, MODE, CONV, CONV != 2>);
    if (CONV == 2) {
        LQ_REQUIRE(schedule <= 1, LQ_ERR_NOT_IMPLEMENTED, "tile kernel: a volumetric convolution runs one block per tile");
        schedule = 1;
    }
    static DeviceOnce attr_once;
    if (int rc = device_once(attr_once, [&]() -> int {
            LQ_HIP(hipFuncSetAttribute(fn_dp, hipFuncAttributeMaxDynamicSharedMemorySize, Cfg::SMEM));
            LQ_HIP(hipFuncSetAttribute(fn_sk, hipFuncAttributeMaxDynamicSharedMemorySize, Cfg::SMEM));
            return LQ_OK;
        }))
        return rc;
    const int tiles = ((g.M + Cfg::BM - 1) / Cfg::BM) * ((g.N + Cfg::BN - 1) / Cfg::BN);
    const int nk = (g.K + Cfg::BK - 1) / Cfg::BK;
    // blocks that fit on the chip at once: 256 CUs x blocks per CU (LDS-bound)
    const int per_cu = (160 * 1024) / Cfg::SMEM < Cfg::MINWAVES ? (160 * 1024) / Cfg::SMEM : Cfg::MINWAVES;
    const int slots = 256 * (per_cu < 1 ? 1 : per_cu);
    // schedule: 0 = choose, 1 = one block per tile, 2 = stream-K over all tiles,
    // 3 = hybrid: stream-K over the tiles that would form a badly filled last round
    // of blocks (done first, so the partial sums are exchanged early), one block per
    // tile for the rest.
    // Both shared schedules are exact and tested, and both measured slower than one
    // block per tile at M=2048, N=11008, K=4096 (111 us): 136 us for the hybrid,
    // more for stream-K over everything.  The worker that finishes a shared tile
    // pays a reduction and a second epilogue on top of its own whole tile, which
    // costs more than the idle slots of the last round.  The automatic choice is
    // therefore always one block per tile.
    int sk_tiles = 0;
    const int slots_g = slots / groups;
    if (g.range != nullptr) {
        LQ_REQUIRE(long(tiles) * groups <= kRangeSlots, LQ_ERR_SHAPE,
                   "tile kernel: %ld tiles are too many for a kept range", long(tiles) * groups);
        schedule = 1;
    }
    if (schedule == 2) {
        sk_tiles = tiles;
    } else if (schedule == 3) {
        const int rem = slots_g > 0 ? tiles % slots_g : 0;
        if (slots_g > 0 && rem > 0 && tiles > slots_g) sk_tiles = rem;
    }
    const bool sk = sk_tiles > 0;
    GemmArgs copy = g;
    void* kargs[] = {&copy};
    if (!sk) {
        LQ_HIP(hipLaunchKernel(fn_dp, dim3(tiles, groups), dim3(Cfg::THREADS), kargs, Cfg::SMEM, st));
        return LQ_OK;
    }
    long workers = slots_g;
    if (workers < 1) workers = 1;
    if (workers > long(sk_tiles) * nk) workers = long(sk_tiles) * nk;
    if (schedule == 2 && long(tiles) * 2 <= workers) {
        // fewer tiles than block slots: a whole number of workers per tile, so that no
        // worker's range straddles two tiles (plain split-K, each piece >= 4 iterations)
        long split = workers / tiles;
        if (split > nk / 4) split = nk / 4;
        workers = long(tiles) * (split < 1 ? 1 : split);
    }
    SkScratch s;
    const size_t slab_words = size_t(Cfg::TM) * Cfg::TN * 16 * Cfg::THREADS;
    int rc = sk_scratch(size_t(sk_tiles) * groups, size_t(groups) * workers * 2 * slab_words * 4, st, &s);
    if (rc) return rc;
    copy.sk_counters = s.counters;
    copy.sk_slabs = s.slabs;
    copy.sk_tiles = sk_tiles;
    LQ_HIP(hipLaunchKernel(fn_sk, dim3(unsigned(workers), groups), dim3(Cfg::THREADS), kargs, Cfg::SMEM, st));
    return LQ_OK;
}

template <class Cfg, int CONV>
int launch_tile(const GemmArgs& g, int groups, int schedule, hipStream_t st) {
    LQ_REQUIRE(size_t(Cfg::BM > Cfg::BN ? Cfg::BM : Cfg::BN) * g.K < 0xffffffffull, LQ_ERR_SHAPE,
               "tile kernel: K too large");
    switch (g.out_mode) {
    case OUT_ACC_I32: return launch_tile_mode<Cfg, OUT_ACC_I32, CONV>(g, groups, schedule, st);
    case OUT_F32:
        if (g.gelu || g.range != nullptr) {
            if (CONV) return fail(LQ_ERR_NOT_IMPLEMENTED, "tile kernel: GELU / kept range are not built for convolutions");
            return launch_tile_mode<Cfg, OUT_F32X, 0>(g, groups, schedule, st);
        }
        return launch_tile_mode<Cfg, OUT_F32, CONV>(g, groups, schedule, st);
    case OUT_F16: return launch_tile_mode<Cfg, OUT_F16, CONV>(g, groups, schedule, st);
    case OUT_REQUANT_I8:
        if (g.join_q != nullptr) return launch_tile_mode<Cfg, OUT_REQUANT_JOIN, CONV>(g, groups, schedule, st);
        return launch_tile_mode<Cfg, OUT_REQUANT_I8, CONV>(g, groups, schedule, st);
    default: return launch_tile_mode<Cfg, OUT_FAKEQUANT_F32, CONV>(g, groups, schedule, st);
    }
}

}  // namespace
}  // namespace lq

// One per translation unit: the launcher of one tile shape.  conv: 0 = plain GEMM, 1 = gather
// from NHWC codes, 2 = from NDHWC codes (only in the units that pass WITH_3D = true).
#define LQ_DEFINE_TILE_LAUNCHER(NAME, CFG, WITH_3D)                                             \
    namespace lq {                                                                              \
    int NAME(const GemmArgs& g, int conv, int groups, int schedule, hipStream_t st) {           \
        if (conv == 2) {                                                                        \
            if constexpr (WITH_3D) return launch_tile<CFG, 2>(g, groups, schedule, st);         \
            return fail(LQ_ERR_NOT_IMPLEMENTED, "this tile shape has no volumetric gather");    \
        }                                                                                       \
        return conv ? launch_tile<CFG, 1>(g, groups, schedule, st)                              \
                    : launch_tile<CFG, 0>(g, groups, schedule, st);                             \
    }                                                                                           \
    }
