// Four-wavefront tile kernel of the int8 GEMM with one wavefront per SIMD and the whole
// register file behind it: a wavefront owns 128 x 176 outputs (8 x 11 tiles of
// v_mfma_i32_16x16x64_i8 = 352 accumulator registers, 256 of them in the accumulation
// registers), so a 64-byte k step moves (128 + 176) x 64 bytes from LDS for 88 matrix
// instructions - 37 % fewer LDS bytes per instruction than eight wavefronts of 64 x 176.
//
//   block tile   BM x BN, wavefronts WM x WN = 4, four 64-byte k stages in LDS
//   main loop    software-pipelined inside the one wavefront: while the 88 MFMAs of step u
//                issue, the fragments of step u + 1 are read from LDS - a B fragment into its
//                own registers right after the eight MFMAs that were its last readers, the A
//                fragments into a second set - and on odd steps the direct global -> LDS loads
//                of stages u + 3, u + 4 go out between the column groups
//   sync         one workgroup barrier per TWO k steps: stages are loaded in pairs (the two
//                64-byte halves of each 128-byte line back to back), a pair is requested once
//                both stages of the pair before last have been read by everybody, and has to
//                have landed two steps later
//   MFMAs        written as inline assembly so that each accumulator's register class is
//                explicit (the compiler would move all of them through the 256 accumulation
//                registers).  The compiler therefore does not know that these instructions
//                complete late: it must never touch an accumulator between the first and the
//                last of them.  That is why the k loop is ONE loop with no peeled copies of
//                its body (with copies, the register assignment differs between them and the
//                compiler moves accumulators across - reading registers an MFMA is still
//                writing); stages past the end are loaded and read like the others and never
//                used.  The wait states before the epilogue's first read are inserted by hand,
//                and tests/test_abi.py checks the compiled loop for stray register moves.
#pragma once
#include "qgemm_pp.hpp"

namespace lq {
namespace {

template <int BM_, int BN_, int WM_, int WN_>
struct BWCfg {
    static constexpr int BM = BM_, BN = BN_, BK = 64, WM = WM_, WN = WN_, STAGES = 4;
    static constexpr int WAVES = WM * WN;
    static constexpr int THREADS = WAVES * 64;
    static constexpr int TM = BM / WM / 16, TN = BN / WN / 16;
    static constexpr int A_CHUNKS = BM / 16, B_CHUNKS = BN / 16;
    static constexpr int LA = (A_CHUNKS + WAVES - 1) / WAVES, LB = (B_CHUNKS + WAVES - 1) / WAVES;
    static constexpr int STAGE_BYTES = (BM + BN) * BK;
    static constexpr int PARAM_OFF = STAGES * STAGE_BYTES;
    static constexpr int SMEM = PARAM_OFF + 3 * BN * 4;
    // accumulator tiles of columns j < AJ live in accumulation registers (at most 256 of them)
    static constexpr int AJ = (64 / TM) < TN ? (64 / TM) : TN;
    static_assert(WAVES == 4, "one wavefront per SIMD");
    static_assert(BM % (WM * 16) == 0 && BN % (WN * 16) == 0, "");
    static_assert(TM <= TN, "A fragments of the next step are read behind the first TM column groups");
    static_assert(2 * (LA + LB) <= 2 * TN, "at most two direct loads behind a column group");
    static_assert(SMEM <= 160 * 1024, "LDS of a CU");
    static_assert(BN <= THREADS * 2, "at most two column parameter sets per thread");
};

template <bool AG>
__device__ __forceinline__ void bw_mfma(pp_v4i& c, const pp_v4i& b, const pp_v4i& a) {
    if constexpr (AG)
        asm volatile("v_mfma_i32_16x16x64_i8 %0, %1, %2, %0" : "+a"(c) : "v"(b), "v"(a));
    else
        asm volatile("v_mfma_i32_16x16x64_i8 %0, %1, %2, %0" : "+v"(c) : "v"(b), "v"(a));
}

// K must be a multiple of 128 and at least 256 (the launcher checks); M and N are arbitrary.
template <class Cfg, int MODE>
__global__ __launch_bounds__(Cfg::THREADS) __attribute__((amdgpu_waves_per_eu(1, 1))) void qgemm_bw_kernel(GemmArgs g) {
    constexpr int BM = Cfg::BM, BN = Cfg::BN, BK = Cfg::BK, TM = Cfg::TM, TN = Cfg::TN;
    constexpr int STAGES = Cfg::STAGES, LA = Cfg::LA, LB = Cfg::LB;
    extern __shared__ __attribute__((aligned(1024))) int8_t smem[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / Cfg::WN, wn = wave % Cfg::WN;
    const int tiles_m = (g.M + BM - 1) / BM, tiles_n = (g.N + BN - 1) / BN;
    int tm, tn;
    pp_tile_coords(blockIdx.x, gridDim.x, tiles_m, tiles_n, &tm, &tn);
    const int m0 = tm * BM, n0 = tn * BN;
    const int nk = g.K / BK;
    const int wm0 = m0 + wm * (TM * 16), wn0 = n0 + wn * (TN * 16);
    const int rot = pp_rotation<TN, MODE>(g, wn0);

    // global -> LDS: the placement of the eight-wavefront kernel (chunk c = rows 16c .. 16c+15,
    // lane l fills row 16c + l/4, physical 16-byte chunk l%4 with logical chunk (l%4) ^ ((row/2)%4))
    const int ld_row = lane >> 2;
    const int ld_kc = (lane & 3) ^ ((lane >> 3) & 3);
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

    // Direct load c (0 .. 2 (LA + LB) - 1) of this wavefront for the stage pair (s, s + 1): the
    // operand's chunk c / 2 for stage s + c % 2, so that the two 64-byte halves of every 128-byte
    // line are requested back to back.  A stage past the end reloads the last one into a buffer
    // nobody reads any more.
    auto pair_load = [&](int s, auto c_tag) {
        constexpr int c = decltype(c_tag)::value;
        constexpr int x = c / 2;
        const int st = s + (c & 1);
        const int sk = st < nk ? st : nk - 1;
        int8_t* buf = smem + (st % STAGES) * Cfg::STAGE_BYTES;
        if constexpr (x < LA) {
            __builtin_amdgcn_raw_ptr_buffer_load_lds(a_rsrc, LQ_PP_LPTR(buf + a_chunk[x] * 1024), 16, int(a_off[x]), sk * BK, 0,
                                                     0);
        } else {
            constexpr int xb = x - LA < LB ? x - LA : 0;
            __builtin_amdgcn_raw_ptr_buffer_load_lds(b_rsrc, LQ_PP_LPTR(buf + BM * BK + b_chunk[xb] * 1024), 16,
                                                     int(b_off[xb]), sk * BK, 0, 0);
        }
    };
    constexpr int kPairLoads = 2 * (LA + LB);

    // LDS -> registers: lane l of a 16 x 64 fragment holds row l%16, logical chunk l/16; B
    // fragment j is the wavefront's column tile (j + rot) % TN
    const int fr_off = (lane & 15) * BK + (((lane >> 4) ^ ((lane >> 1) & 3)) * 16);
    const int a_frag0 = wm * (TM * 16) * BK + fr_off;
    const int b_frag0 = BM * BK + wn * (TN * 16) * BK + fr_off + rot * 16 * BK;
    const int b_frag_last = BM * BK + wn * (TN * 16) * BK + fr_off + (rot ? 0 : (TN - 1) * 16 * BK);
    pp_v4i af[2][TM], bf[TN];
    pp_v4i acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = pp_v4i{0, 0, 0, 0};

    // ---- prologue: row scales and column parameters first (the column parameters are published
    // by the first barrier), then the stage pairs (0, 1) and (2, 3)
    float* s_ws = reinterpret_cast<float*>(smem + Cfg::PARAM_OFF);
    float* s_bias = s_ws + BN;
    int32_t* s_corr = reinterpret_cast<int32_t*>(s_bias + BN);
    float as_row[TM];
#pragma unroll
    for (int i = 0; i < TM; ++i) {
        const int m = wm0 + 16 * i + (lane & 15);
        as_row[i] = g.a_scale ? g.a_scale[(g.a_scale_per_row && m < g.M) ? m : 0] : 1.0f;
    }
    ColParams c_mine[2] = {ColParams{1.0f, -0.0f, 0}, ColParams{1.0f, -0.0f, 0}};
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const int col = tid + h * Cfg::THREADS;
        if (col < BN) c_mine[h] = load_col(g, n0 + col < g.N ? n0 + col : g.N - 1);
    }
    __builtin_amdgcn_sched_barrier(0);
    pp_static_for<kPairLoads>([&](auto c) { pair_load(0, c); });
    pp_static_for<kPairLoads>([&](auto c) { pair_load(2, c); });
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const int col = tid + h * Cfg::THREADS;
        if (col < BN) s_ws[col] = c_mine[h].ws, s_bias[col] = c_mine[h].bias, s_corr[col] = c_mine[h].corr;
    }
    __builtin_amdgcn_s_waitcnt(pp_vmcnt_imm(kPairLoads));  // stages 0 and 1 have landed
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < TM; ++i) af[0][i] = *reinterpret_cast<const pp_v4i*>(smem + a_frag0 + i * 16 * BK);
#pragma unroll
    for (int j = 0; j < TN - 1; ++j) bf[j] = *reinterpret_cast<const pp_v4i*>(smem + b_frag0 + j * 16 * BK);
    bf[TN - 1] = *reinterpret_cast<const pp_v4i*>(smem + b_frag_last);

    // One k step: the MFMAs of stage u from af[P] / bf, column group by column group, the row
    // order alternating so that one operand changes between neighbours.  Between them, one at a
    // time so that each issues in the shadow of a matrix instruction: behind the second MFMA of
    // group j the next stage's A fragment j (into the other set), behind the fourth and sixth the
    // direct loads, behind the last the next stage's B fragment j, into the registers its last
    // reader has just left.  SYNC (odd) steps begin with the wait for the wavefront's own loads
    // of the pair (u + 1, u + 2) and the barrier that publishes everybody's, and issue the loads
    // of the pair (u + 3, u + 4), whose buffers held the stages u - 1 and u: stage u was read
    // during step u - 1, which all wavefronts have finished once they are past this barrier.
    auto step = [&](int u, auto p_tag, auto sync_tag) {
        constexpr int P = decltype(p_tag)::value;
        constexpr bool SYNC = decltype(sync_tag)::value;
        const int8_t* nbuf = smem + ((u + 1) % STAGES) * Cfg::STAGE_BYTES;
        if constexpr (SYNC) {
            __builtin_amdgcn_s_waitcnt(pp_vmcnt_imm(0));
            __builtin_amdgcn_s_barrier();
            __builtin_amdgcn_sched_barrier(0);
        }
        pp_static_for<TN>([&](auto j_tag) {
            constexpr int j = decltype(j_tag)::value;
            pp_static_for<TM>([&](auto i_tag) {
                constexpr int ii = decltype(i_tag)::value;
                constexpr int i = (j & 1) ? TM - 1 - ii : ii;
                bw_mfma<(j < Cfg::AJ)>(acc[i][j], bf[j], af[P][i]);
                if constexpr (ii == 1 && j < TM)
                    af[P ^ 1][j] = *reinterpret_cast<const pp_v4i*>(nbuf + a_frag0 + j * 16 * BK);
                if constexpr (SYNC && ii == 3 && 2 * j < kPairLoads) pair_load(u + 3, std::integral_constant<int, 2 * j>{});
                if constexpr (SYNC && ii == 5 && 2 * j + 1 < kPairLoads)
                    pair_load(u + 3, std::integral_constant<int, 2 * j + 1>{});
                __builtin_amdgcn_sched_barrier(0);
            });
            bf[j] = *reinterpret_cast<const pp_v4i*>(nbuf + (j < TN - 1 ? b_frag0 + j * 16 * BK : b_frag_last));
            __builtin_amdgcn_sched_barrier(0);
        });
    };
    for (int u = 0; u < nk; u += 2) {
        step(u, std::integral_constant<int, 0>{}, std::false_type{});
        step(u + 1, std::integral_constant<int, 1>{}, std::true_type{});
    }
    __builtin_amdgcn_sched_barrier(0);
    // The last MFMAs' results are read by vector instructions next: an MFMA of four passes needs
    // its result left alone for a dozen cycles, which inline assembly hides from the compiler.
    asm volatile("s_nop 15\n\ts_nop 7" ::: "memory");
    __builtin_amdgcn_s_waitcnt(pp_vmcnt_imm(0));  // no direct load may land in LDS after this wavefront has ended
    __builtin_amdgcn_sched_barrier(0);
    float r_lo = 0.0f, r_hi = 0.0f;  // (no kept range in this kernel's output forms)
    int r_nan = 0;
    pp_epilogue<TM, TN, MODE>(g, acc, as_row, s_ws, s_bias, s_corr, n0, wm0, wn0, lane, rot, r_lo, r_hi, r_nan);
}

template <class Cfg, int MODE>
int launch_bw_mode(const GemmArgs& g, hipStream_t st) {
    const void* fn = reinterpret_cast<const void*>(qgemm_bw_kernel<Cfg, MODE>);
    static DeviceOnce attr_once;
    if (int rc = allow_dynamic_lds(attr_once, fn, Cfg::SMEM)) return rc;
    const int tiles = ((g.M + Cfg::BM - 1) / Cfg::BM) * ((g.N + Cfg::BN - 1) / Cfg::BN);
    GemmArgs copy = g;
    void* kargs[] = {&copy};
    LQ_HIP(hipLaunchKernel(fn, dim3(tiles), dim3(Cfg::THREADS), kargs, Cfg::SMEM, st));
    return LQ_OK;
}

using BWCfg352 = BWCfg<256, 352, 2, 2>;

}  // namespace
}  // namespace lq
