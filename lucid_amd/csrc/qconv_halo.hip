// Stride-1 int8 convolution (2-d or volumetric) on channels-last codes with the input held in
// LDS: a block owns a box of 256 (or 128, or 64) output positions and 64 output channels, loads the box's
// input halo - (TD + (KD-1) dd) x (TH + (KH-1) dh) x (TW + (KW-1) dw) positions x 64 channels -
// into LDS ONCE per 64-channel slice, and takes the A fragments of every filter tap from it
// at a shifted row.  The gather of the tile GEMM's loader fetches every input position once
// per tap through the L2 (27 times for a 3x3x3 filter); this one fetches it once per block.
// Filter rows are streamed per tap through a small ring of LDS stages.
//
//   LDS: halo rows of 64 bytes (one position's 64 channels), 16-byte chunk kc of row r at
//        physical chunk kc ^ ((r/2) % 4); then NB stages of 64 filter rows x 64 bytes, same
//        placement; then the block's 64 column parameter sets.
//   wavefront w: positions 16 TI w .. 16 TI (w+1) - 1 of the box (w fastest, then h, then d) x 64
//        channels (TI = 4, 2 or 1 tiles of 16 positions: boxes of 256, 128 or 64 positions - the
//        smaller boxes are for layers with too few positions to give 256 CUs a 256-position box
//        each), TI x 4 accumulator tiles of v_mfma_i32_16x16x64_i8 with the filter fragment as the first
//        operand, so a lane holds four consecutive output channels of one position and the
//        epilogue runs on registers (the helpers of qepilogue.hpp: same bits as the tile kernel).
#include "common.hpp"
#include "qgemm.hpp"
#include "qepilogue.hpp"

using namespace lq;

namespace {

typedef int hv4i __attribute__((ext_vector_type(4)));

#define LQ_HALO_GPTR(p) ((__attribute__((address_space(1))) void*)(p))
#define LQ_HALO_LPTR(p) ((__attribute__((address_space(3))) void*)(p))

constexpr int halo_vmcnt_imm(int n) { return (n & 0xF) | ((n >> 4) << 14) | (0x7 << 4) | (0xF << 8); }

constexpr int kRing = 6;  // filter stages in the ring

struct HaloGeom {
    int D, H, W, OD, OH, OW;     // input and output extents (D = OD = 1 for a 2-d layer)
    int KD, KH, KW, pd, ph, pw, dd, dh, dw;
    int ltd, lth, ltw;           // log2 of the box extents; their product is the box (256, 128 or 64)
    int HD, HH, HW;              // halo extents
    int halo_rows;               // HD * HH * HW rounded up to a multiple of 64
    int tiles_d, tiles_h, tiles_w;
    int n_tiles;                 // 64-column tiles per group
    int cblocks;                 // 64-channel slices per group
    int inv_hw, inv_hh;          // 2^20 / HW + 1, 2^20 / HH + 1
};

template <int MODE, int TI>
__global__ __launch_bounds__(256, 2) void qconv_halo_kernel(GemmArgs g, HaloGeom q) {
    extern __shared__ __attribute__((aligned(1024))) int8_t smem[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    int t = blockIdx.x;
    const int twi = t % q.tiles_w;
    t /= q.tiles_w;
    const int thi = t % q.tiles_h;
    t /= q.tiles_h;
    const int tdi = t % q.tiles_d;
    const int b = t / q.tiles_d;
    const int od0 = tdi << q.ltd, oh0 = thi << q.lth, ow0 = twi << q.ltw;
    const int grp = int(blockIdx.y) / q.n_tiles;
    const int n0 = (int(blockIdx.y) - grp * q.n_tiles) * 64;  // first column of the block within its group
    const int Og = g.N, Cg = g.cCg;
    const int taps = q.KD * q.KH * q.KW;

    int8_t* const halo = smem;
    int8_t* const ring = smem + size_t(q.halo_rows) * 64;
    float* const s_ws = reinterpret_cast<float*>(ring + kRing * 4096);
    float* const s_bias = s_ws + 64;
    int32_t* const s_corr = reinterpret_cast<int32_t*>(s_bias + 64);

    // ---- global -> LDS.  A wavefront-wide 16-byte direct load fills 16 rows x 64 bytes: lane l
    // writes the slot of row l/4, physical chunk l%4, and therefore fetches logical chunk
    // (l%4) ^ ((row/2)%4).
    const int ld_row = tid >> 2, ld_pc = tid & 3;
    auto load_halo = [&](int cb) {
        const int passes = q.halo_rows >> 6;
        const int hv = q.HD * q.HH * q.HW;
        const size_t chan = size_t(grp) * Cg + size_t(cb) * 64;
        for (int it = 0; it < passes; ++it) {
            const int r = it * 64 + ld_row;
            // r < 1024 and the divisors are below 2^10: the 20-bit reciprocals give exact quotients
            const int r2 = int((unsigned(r) * unsigned(q.inv_hw)) >> 20), hw = r - r2 * q.HW;
            const int hd = int((unsigned(r2) * unsigned(q.inv_hh)) >> 20), hh = r2 - hd * q.HH;
            const int id = od0 - q.pd + hd, ih = oh0 - q.ph + hh, iw = ow0 - q.pw + hw;
            const bool ok = r < hv && unsigned(id) < unsigned(q.D) && unsigned(ih) < unsigned(q.H) &&
                            unsigned(iw) < unsigned(q.W);
            const int lc = ld_pc ^ ((r >> 1) & 3);
            const int8_t* src =
                ok ? g.cx + ((size_t((b * q.D + id) * q.H + ih) * q.W + iw) * size_t(g.cCin) + chan + size_t(lc * 16))
                   : g.pad_src;
            __builtin_amdgcn_global_load_lds(LQ_HALO_GPTR(src), LQ_HALO_LPTR(halo + (it * 64 + wave * 16) * 64), 16, 0, 0);
        }
    };
    // filter rows of the block for tap t of slice cb: row n0 + tid/4 (clamped), 64 bytes at
    // k = t * Cg + cb * 64, into ring stage t % kRing
    const int b_row = n0 + ld_row < Og ? n0 + ld_row : Og - 1;
    const int8_t* const b_src = g.w + (size_t(grp) * Og + size_t(b_row)) * size_t(g.K) + size_t((ld_pc ^ ((ld_row >> 1) & 3)) * 16);
    auto load_filter = [&](int cb, int tap) {
        __builtin_amdgcn_global_load_lds(LQ_HALO_GPTR(b_src + size_t(tap) * Cg + size_t(cb) * 64),
                                         LQ_HALO_LPTR(ring + (tap % kRing) * 4096 + wave * 1024), 16, 0, 0);
    };

    // ---- LDS -> registers: lane l of a 16 x 64 fragment holds row l%16, logical chunk l/16
    const int fr = lane & 15, fc = lane >> 4;
    int a_row[TI];  // halo row of the lane's position in each of the wavefront's 16-row tiles, tap (0, 0, 0)
#pragma unroll
    for (int i = 0; i < TI; ++i) {
        const int v = wave * (16 * TI) + i * 16 + fr;
        const int vw = v & ((1 << q.ltw) - 1), vh = (v >> q.ltw) & ((1 << q.lth) - 1), vd = v >> (q.ltw + q.lth);
        a_row[i] = (vd * q.HH + vh) * q.HW + vw;
    }
    int b_off[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int r = j * 16 + fr;
        b_off[j] = r * 64 + ((fc ^ ((r >> 1) & 3)) << 4);
    }
    hv4i acc[TI][4];
#pragma unroll
    for (int i = 0; i < TI; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = hv4i{0, 0, 0, 0};

    // the block's column parameters go to LDS while the first loads are in flight
    ColParams c_mine{1.0f, -0.0f, 0};
    if (tid < 64) c_mine = load_col(g, grp * Og + (n0 + tid < Og ? n0 + tid : Og - 1));

    // fragments of tap (kd, kh, kw), whose filter rows sit in ring stage `stage`
    auto read_frags = [&](int kd, int kh, int kw, int stage, hv4i (&af)[TI], hv4i (&bf)[4]) {
        const int toff = ((kd * q.dd) * q.HH + kh * q.dh) * q.HW + kw * q.dw;
        const int8_t* st = ring + stage * 4096;
#pragma unroll
        for (int i = 0; i < TI; ++i) {
            const int hr = a_row[i] + toff;
            af[i] = *reinterpret_cast<const hv4i*>(halo + hr * 64 + ((fc ^ ((hr >> 1) & 3)) << 4));
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) bf[j] = *reinterpret_cast<const hv4i*>(st + b_off[j]);
    };
    auto next_tap = [&](int& kd, int& kh, int& kw) {
        if (++kw == q.KW) {
            kw = 0;
            if (++kh == q.KH) kh = 0, ++kd;
        }
    };
    // One tap: wait for the NEXT tap's filter stage, meet the other wavefronts (they have all
    // consumed the stage that is refilled now), request the stage kRing-1 taps ahead, read the
    // next tap's fragments into the other register set, and issue this tap's MFMAs on top of them.
    auto tap_step = [&](int cb, int tp, int& kd, int& kh, int& kw, hv4i (&af)[TI], hv4i (&bf)[4], hv4i (&an)[TI],
                        hv4i (&bn)[4]) {
        if (tp + 1 < taps) {
            if (tp + kRing - 1 <= taps)
                __builtin_amdgcn_s_waitcnt(halo_vmcnt_imm(kRing - 3));  // stages tp+2 .. tp+kRing-2 may be in flight
            else
                __builtin_amdgcn_s_waitcnt(halo_vmcnt_imm(0));
        }
        __syncthreads();
        if (tp + kRing - 1 < taps) load_filter(cb, tp + kRing - 1);
        if (tp + 1 < taps) {
            next_tap(kd, kh, kw);
            read_frags(kd, kh, kw, (tp + 1) % kRing, an, bn);
        }
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int i = 0; i < TI; ++i)
                acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(bf[j], af[i], acc[i][j], 0, 0, 0);
    };

    for (int cb = 0; cb < q.cblocks; ++cb) {
        // a new 64-channel slice: everyone has finished with the old halo and ring; the new halo and
        // the first filter stages are requested and awaited in full
        __syncthreads();
        load_halo(cb);
        for (int p = 0; p < kRing - 1 && p < taps; ++p) load_filter(cb, p);
        if (cb == 0 && tid < 64) s_ws[tid] = c_mine.ws, s_bias[tid] = c_mine.bias, s_corr[tid] = c_mine.corr;
        __builtin_amdgcn_s_waitcnt(halo_vmcnt_imm(0));
        __syncthreads();
        int kd = 0, kh = 0, kw = 0;
        hv4i a0[TI], b0[4], a1[TI], b1[4];
        read_frags(0, 0, 0, 0, a0, b0);
        int tp = 0;
        for (; tp + 1 < taps; tp += 2) {
            tap_step(cb, tp, kd, kh, kw, a0, b0, a1, b1);
            tap_step(cb, tp + 1, kd, kh, kw, a1, b1, a0, b0);
        }
        if (tp < taps) tap_step(cb, tp, kd, kh, kw, a0, b0, a1, b1);
    }

    // ---- epilogue on registers.  acc[i][j][r]: position 16 TI wave + 16 i + lane%16 of the box,
    // column n0 + 16 j + 4 (lane/16) + r of the group.
    float S = 1.0f, Z = 0.0f;
    constexpr bool kRequant = MODE == OUT_REQUANT_I8 || MODE == OUT_FAKEQUANT_F32;
    if (kRequant) {
        S = g.out_scale[0];
        Z = g.out_zp[0];
    }
    const QGrid G = make_qgrid(S, Z, float(g.out_qmin), float(g.out_qmax), kRequant, g.relu != 0, MODE == OUT_REQUANT_I8);
    const JoinParams jp{};
    const CodePack cpk = make_code_pack<MODE>(g, G);
    constexpr int esize = MODE == OUT_F16 ? 2 : (MODE == OUT_REQUANT_I8 ? 1 : 4);
    const float as = g.a_scale ? g.a_scale[0] : 1.0f;
    const bool prescaled = MODE == OUT_REQUANT_I8;
    const bool cols_in = n0 + 64 <= Og;
    const bool vec_out = cols_in && g.ldo % 4 == 0 && Og % 4 == 0 && reinterpret_cast<uintptr_t>(g.out) % (4 * esize) == 0;
    long m_row[TI];  // output row (position index over the whole batch) of each tile's lane row, -1 outside
#pragma unroll
    for (int i = 0; i < TI; ++i) {
        const int v = wave * (16 * TI) + i * 16 + fr;
        const int vw = v & ((1 << q.ltw) - 1), vh = (v >> q.ltw) & ((1 << q.lth) - 1), vd = v >> (q.ltw + q.lth);
        const int od = od0 + vd, oh = oh0 + vh, ow = ow0 + vw;
        m_row[i] = (od < q.OD && oh < q.OH && ow < q.OW) ? (long((b * q.OD + od) * q.OH + oh) * q.OW + ow) : -1;
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int cl = 16 * j + 4 * fc;  // column within the block, a multiple of 4
        const float4 ws = *reinterpret_cast<const float4*>(s_ws + cl);
        const float4 bs = *reinterpret_cast<const float4*>(s_bias + cl);
        const int4 cr = *reinterpret_cast<const int4*>(s_corr + cl);
        ColParams c4[4] = {ColParams{ws.x, bs.x, cr.x}, ColParams{ws.y, bs.y, cr.y}, ColParams{ws.z, bs.z, cr.z},
                           ColParams{ws.w, bs.w, cr.w}};
        if (prescaled) {
#pragma unroll
            for (int r = 0; r < 4; ++r) c4[r].ws = as * c4[r].ws;
        }
        const int nq = grp * Og + n0 + cl;  // global column of the lane's first value
#pragma unroll
        for (int i = 0; i < TI; ++i) {
            if (m_row[i] < 0) continue;
            const hv4i a = acc[i][j];
            uint4 v;
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
            const size_t idx = size_t(m_row[i]) * size_t(g.ldo) + size_t(nq);
            if (vec_out) {
                store_vec4<MODE>(g, idx, v, cpk);
            } else {
                const int left = Og - (n0 + cl);  // columns of the group from the lane's first one on
                const int m = int(m_row[i]);
                if (left > 0) store_scalar<MODE>(g, idx, finish_value<MODE>(g, v.x, m, nq, jp), cpk);
                if (left > 1) store_scalar<MODE>(g, idx + 1, finish_value<MODE>(g, v.y, m, nq + 1, jp), cpk);
                if (left > 2) store_scalar<MODE>(g, idx + 2, finish_value<MODE>(g, v.z, m, nq + 2, jp), cpk);
                if (left > 3) store_scalar<MODE>(g, idx + 3, finish_value<MODE>(g, v.w, m, nq + 3, jp), cpk);
            }
        }
    }
}

template <int MODE, int TI>
int launch_mode(const GemmArgs& g, const HaloGeom& q, dim3 grid, size_t lds, hipStream_t st) {
    const void* fn = reinterpret_cast<const void*>(qconv_halo_kernel<MODE, TI>);
    static DeviceOnce attr_once;
    if (int rc = allow_dynamic_lds(attr_once, fn, 96 * 1024)) return rc;
    GemmArgs gc = g;
    HaloGeom qc = q;
    void* kargs[] = {&gc, &qc};
    LQ_HIP(hipLaunchKernel(fn, grid, dim3(256), kargs, lds, st));
    return LQ_OK;
}

int ilog2(int v) {
    int l = 0;
    while ((1 << (l + 1)) <= v) ++l;
    return l;
}

}  // namespace

namespace lq {

// Whether the halo kernel can run the convolution described by g (conv = 1: NHWC, 2: NDHWC
// geometry in the c* fields; N = output channels of one group) with boxes of 2^lbox positions,
// and with which box.
static bool plan_halo(const GemmArgs& g, int conv, int lbox, HaloGeom* out) {
    if (conv != 1 && conv != 2) return false;
    HaloGeom q{};
    const bool vol = conv == 2;
    q.D = vol ? g.cD : 1, q.H = g.cH, q.W = g.cW;
    q.OD = vol ? g.cOD : 1, q.OH = g.cOH, q.OW = g.cOW;
    const int Cg = g.cCg;
    if (Cg <= 0 || Cg % 64 != 0 || g.K % Cg != 0) return false;
    const int taps = g.K / Cg;
    q.KW = g.cKW;
    if (q.KW <= 0 || taps % q.KW != 0) return false;
    if (vol) {
        q.KH = g.cKH;
        if (q.KH <= 0 || (taps / q.KW) % q.KH != 0) return false;
        q.KD = taps / q.KW / q.KH;
    } else {
        q.KH = taps / q.KW, q.KD = 1;
    }
    if ((vol && g.csd != 1) || g.csh != 1 || g.csw != 1) return false;
    q.pd = vol ? g.cpd : 0, q.ph = g.cph, q.pw = g.cpw;
    q.dd = vol ? g.cdd : 1, q.dh = g.cdh, q.dw = g.cdw;
    if (g.join_q != nullptr || g.residual != nullptr || g.gelu || g.range != nullptr || g.a_scale_per_row) return false;
    if (!aligned16(g.cx) || !aligned16(g.w)) return false;
    q.cblocks = Cg / 64;
    q.n_tiles = (g.N + 63) / 64;
    // the box: powers of two with product 2^lbox; fewest boxes first, then the smallest halo, then the widest rows
    long best_cost = -1;
    for (int ltw = 0; ltw <= lbox; ++ltw)
        for (int lth = 0; ltw + lth <= lbox; ++lth) {
            const int ltd = lbox - ltw - lth;
            const int tw = 1 << ltw, th = 1 << lth, td = 1 << ltd;
            if (td > 1 && !vol) continue;
            if (tw < 8 && q.OW >= 8) continue;  // fragment rows should be runs of consecutive halo rows
            const int HD = td + (q.KD - 1) * q.dd, HH = th + (q.KH - 1) * q.dh, HW = tw + (q.KW - 1) * q.dw;
            const long hv = long(HD) * HH * HW;
            if (hv > 1024) continue;
            const long boxes = long((q.OD + td - 1) / td) * ((q.OH + th - 1) / th) * ((q.OW + tw - 1) / tw);
            const long cost = boxes * 4096 + hv * 2 - ltw;
            if (best_cost < 0 || cost < best_cost) {
                best_cost = cost;
                q.ltd = ltd, q.lth = lth, q.ltw = ltw;
                q.HD = HD, q.HH = HH, q.HW = HW;
                q.halo_rows = int((hv + 63) / 64 * 64);
                q.tiles_d = (q.OD + td - 1) / td, q.tiles_h = (q.OH + th - 1) / th, q.tiles_w = (q.OW + tw - 1) / tw;
            }
        }
    if (best_cost < 0) return false;
    q.inv_hw = (1 << 20) / q.HW + 1, q.inv_hh = (1 << 20) / q.HH + 1;
    *out = q;
    return true;
}

bool conv_halo_applies(const GemmArgs& g, int conv, int lbox) {
    HaloGeom q;
    return (lbox == 8 || lbox == 7 || lbox == 6) && plan_halo(g, conv, lbox, &q);
}

int launch_conv_halo(const GemmArgs& g, int conv, int groups, int lbox, hipStream_t st) {
    HaloGeom q;
    LQ_REQUIRE(conv_halo_applies(g, conv, lbox) && plan_halo(g, conv, lbox, &q), LQ_ERR_NOT_IMPLEMENTED,
               "halo convolution: needs stride 1, Cin/groups %% 64 == 0, no join and a halo of at most 1024 positions");
    const long batch = long(g.M) / (long(q.OD) * q.OH * q.OW);
    const long boxes = batch * q.tiles_d * q.tiles_h * q.tiles_w;
    LQ_REQUIRE(boxes > 0 && boxes <= 0x7fffffffl && long(q.n_tiles) * groups <= 65535, LQ_ERR_SHAPE,
               "halo convolution: grid too large");
    const dim3 grid{unsigned(boxes), unsigned(q.n_tiles * groups)};
    const size_t lds = size_t(q.halo_rows) * 64 + kRing * 4096 + 3 * 64 * 4;
#define LQ_HALO_MODES(TI)                                                                   \
    switch (g.out_mode) {                                                                   \
    case OUT_ACC_I32: return launch_mode<OUT_ACC_I32, TI>(g, q, grid, lds, st);             \
    case OUT_F32: return launch_mode<OUT_F32, TI>(g, q, grid, lds, st);                     \
    case OUT_F16: return launch_mode<OUT_F16, TI>(g, q, grid, lds, st);                     \
    case OUT_REQUANT_I8: return launch_mode<OUT_REQUANT_I8, TI>(g, q, grid, lds, st);       \
    default: return launch_mode<OUT_FAKEQUANT_F32, TI>(g, q, grid, lds, st);                \
    }
    if (lbox == 8) {
        LQ_HALO_MODES(4)
    } else if (lbox == 7) {
        LQ_HALO_MODES(2)
    }
    LQ_HALO_MODES(1)
#undef LQ_HALO_MODES
}

}  // namespace lq
