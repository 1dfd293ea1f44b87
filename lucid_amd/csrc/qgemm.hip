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
#include "qgemm.hpp"
#include "qepilogue.hpp"

#include "qgemm_tile.hpp"

#include <cstdlib>
#include <cstring>
#include <mutex>
#include <string>
#include <unordered_map>

using namespace lq;

namespace lq {
// The stream's stream-K scratch, grown to the requested sizes: arrival counters (zero
// between launches: freshly allocated ones are cleared by a kernel on the stream, which a
// graph capture records like any other launch) and the accumulator slabs.
int sk_scratch(size_t counters, size_t slab_bytes, hipStream_t st, SkScratch* out) {
    void* c = nullptr;
    bool fresh = false;
    int rc = stream_buffer(1, counters * sizeof(int), size_t(65536) * sizeof(int), st, &c, &fresh);
    if (rc) return rc;
    if (fresh) {
        const size_t bytes = counters * sizeof(int) < size_t(65536) * sizeof(int) ? size_t(65536) * sizeof(int)
                                                                                : counters * sizeof(int);
        rc = lq_fill_bytes(c, 0, bytes, reinterpret_cast<lq_stream>(st));
        if (rc) return rc;
    }
    void* s = nullptr;
    rc = stream_buffer(2, slab_bytes, 0, st, &s, nullptr);
    if (rc) return rc;
    out->counters = static_cast<int*>(c);
    out->slabs = static_cast<int32_t*>(s);
    return LQ_OK;
}

int launch_tile_c1(const GemmArgs&, int, int, int, hipStream_t);
int launch_tile_c2(const GemmArgs&, int, int, int, hipStream_t);
int launch_tile_c3(const GemmArgs&, int, int, int, hipStream_t);
int launch_tile_c4(const GemmArgs&, int, int, int, hipStream_t);
int launch_tile_c5(const GemmArgs&, int, int, int, hipStream_t);
int launch_tile_c6(const GemmArgs&, int, int, int, hipStream_t);
int launch_tile_c7(const GemmArgs&, int, int, int, hipStream_t);
int launch_tile_c8(const GemmArgs&, int, int, int, hipStream_t);
int launch_tile_c9(const GemmArgs&, int, int, int, hipStream_t);
int launch_tile_c10(const GemmArgs&, int, int, int, hipStream_t);
int launch_tile_c11(const GemmArgs&, int, int, int, hipStream_t);
int launch_tile_c12(const GemmArgs&, int, int, int, hipStream_t);
int launch_pp_shape(const GemmArgs&, int, hipStream_t);
int launch_bw_shape(const GemmArgs&, int, hipStream_t);
bool conv_halo_applies(const GemmArgs&, int conv, int lbox = 8);
int launch_conv_halo(const GemmArgs&, int conv, int groups, int lbox, hipStream_t);
bool conv_few_applies(const GemmArgs&, int conv, int groups);
int launch_conv_few(const GemmArgs&, int conv, int groups, hipStream_t);
}  // namespace lq

namespace {

int launch_tile_shape(const GemmArgs& g, int conv, int groups, int cfg, int schedule, hipStream_t st) {
    switch (cfg) {
    case 1: return launch_tile_c1(g, conv, groups, schedule, st);
    case 2: return launch_tile_c2(g, conv, groups, schedule, st);
    case 3: return launch_tile_c3(g, conv, groups, schedule, st);
    case 4: return launch_tile_c4(g, conv, groups, schedule, st);
    case 5: return launch_tile_c5(g, conv, groups, schedule, st);
    case 6: return launch_tile_c6(g, conv, groups, schedule, st);
    case 7: return launch_tile_c7(g, conv, groups, schedule, st);
    case 8: return launch_tile_c8(g, conv, groups, schedule, st);
    case 9: return launch_tile_c9(g, conv, groups, schedule, st);
    case 10: return launch_tile_c10(g, conv, groups, schedule, st);
    case 11: return launch_tile_c11(g, conv, groups, schedule, st);
    case 12: return launch_tile_c12(g, conv, groups, schedule, st);
    case 13:
    case 14:
    case 16:
    case 21:
    case 22:
        // the eight-wavefront ping-pong kernel (256 x 352 / 256 x 256 / 256 x 192 / 224 x 192 / 160 x 256
        // tiles): plain GEMMs, one block per tile
        LQ_REQUIRE(!conv && groups == 1, LQ_ERR_VALUE, "tile_config %d is for plain GEMMs", cfg);
        LQ_REQUIRE(schedule <= 1, LQ_ERR_VALUE, "tile_config %d runs one block per tile", cfg);
        return launch_pp_shape(g, cfg == 16 ? 2 : (cfg >= 21 ? cfg - 18 : cfg - 13), st);
    case 17:
        // one wavefront per SIMD, 256 x 352 tiles (plain GEMMs, K % 128 == 0)
        LQ_REQUIRE(!conv && groups == 1, LQ_ERR_VALUE, "tile_config %d is for plain GEMMs", cfg);
        LQ_REQUIRE(schedule <= 1, LQ_ERR_VALUE, "tile_config %d runs one block per tile", cfg);
        return launch_bw_shape(g, 0, st);
    case 15:
    case 18:
    case 19:
        // stride-1 convolution with the input halo held in LDS, one block per box of 256 / 128 / 64 outputs
        LQ_REQUIRE(conv, LQ_ERR_VALUE, "tile_config %d is for convolutions", cfg);
        LQ_REQUIRE(schedule <= 1, LQ_ERR_VALUE, "tile_config %d runs one block per tile", cfg);
        return launch_conv_halo(g, conv, groups, cfg == 15 ? 8 : (cfg == 18 ? 7 : 6), st);
    case 20:
        // at most four input channels on the packed image: filter in registers, input halo of 16 x 16 boxes in LDS
        LQ_REQUIRE(conv, LQ_ERR_VALUE, "tile_config %d is for convolutions", cfg);
        LQ_REQUIRE(schedule <= 1, LQ_ERR_VALUE, "tile_config %d runs one block per tile", cfg);
        return launch_conv_few(g, conv, groups, st);
    default: return fail(LQ_ERR_VALUE, "unknown tile_config %d", cfg);
    }
}

// Whether the eight-wavefront ping-pong kernel (shapes 13 and 14) can run the problem.
bool pp_applies(const GemmArgs& g, int conv, int groups) {
    // (a kept range needs a slot per tile: the shapes' tiles are at least 256 x 192)
    return !conv && groups == 1 && g.K > 0 && g.K % 64 == 0 && g.M >= 256 && g.N >= 256 &&
           ((!g.gelu && g.range == nullptr) || g.out_mode == OUT_F32) &&
           (g.range == nullptr || long((g.M + 255) / 256) * ((g.N + 191) / 192) <= 16384) &&
           size_t(g.M) * g.K < 0xffffffffull && size_t(g.N) * g.K < 0xffffffffull;
}

// Shape chosen from the problem size alone (what a launch gets when the tuner may not run: a
// stream under capture, LQ_TILE_AUTOTUNE=0, an in-place residual).  Large plain GEMMs go to
// the ping-pong kernel, with the tile width that wastes less of the 256 CUs: the cost of a
// shape is its rounds of 256 tiles times the tile's area.  Otherwise 128 x 256 tiles keep two
// blocks per CU busy; narrower tiles when N is small or when the wide ones would leave most
// of the CUs without work.
int heuristic_tile_shape(const GemmArgs& g, int conv, int groups) {
    const long mt128 = (g.M + 127) / 128;
    // an image of at most four channels with a block's worth of 16 x 16 boxes for every CU
    if (g.M >= 65536 && conv_few_applies(g, conv, groups)) return 20;
    // far fewer 128 x 128 tiles than CUs (a small batch in the late stages of a network): 64 x 64
    // tiles, four blocks per CU, with 128-byte k steps when K is long (plain and 2-d only)
    if (mt128 * ((g.N + 127) / 128) * groups < 128) return (g.K >= 1024 && conv != 2) ? 10 : 9;
    // (not with a GELU: its vector arithmetic needs a second block on the CU to overlap with)
    if (pp_applies(g, conv, groups) && g.K >= 512 && !g.gelu) {
        const long tm = (g.M + 255) / 256;
        const long t352 = tm * ((g.N + 351) / 352), t256 = tm * ((g.N + 255) / 256);
        // at least half a round of tiles, or the four-wavefront shapes below cover the chip better
        if (t256 >= 128) {
            const long t192 = tm * ((g.N + 191) / 192);
            const long c352 = ((t352 + 255) / 256) * 352, c256 = ((t256 + 255) / 256) * 256,
                       c192 = ((t192 + 255) / 256) * 192;
            if (c192 < c256 && c192 < c352) return 16;
            return c352 < c256 ? 13 : 14;
        }
    }
    if (g.N <= 64) return 6;
    if (g.N <= 128 || mt128 * ((g.N + 255) / 256) * groups < 256) return 5;
    return 4;
}

int launch_tile_cfg(const GemmArgs& g, int conv, int groups, int tile_config, hipStream_t st);
thread_local int t_last_tile_config = 0;  // what the last tile-kernel launch of this thread resolved to

constexpr int kSplitShape = 11;  // 256 x 256 x 128 tiles, eight wavefronts

// Two regions of one GEMM: the first a_tiles * 256 output columns go to the 256 x 256 shape
// (chosen so that its tiles fill whole rounds of the 256 CUs, one block each), the remaining
// columns are a problem of their own with whatever shape suits it.  The 256 x 256 shape has
// the best main loop (least LDS traffic per MFMA) but wastes most of a round when its tile
// count is not a multiple of the CU count; this keeps the one and avoids the other.
int launch_split(const GemmArgs& g, int a_tiles, hipStream_t st) {
    const long NA = long(a_tiles) * 256;
    if (NA <= 0 || NA >= g.N) return fail(LQ_ERR_VALUE, "tile split: %ld columns of %d", NA, g.N);
    GemmArgs ga = g;
    ga.N = int(NA);
    int rc = launch_tile_shape(ga, 0, 1, kSplitShape, 1, st);
    if (rc) return rc;
    GemmArgs gb = g;
    gb.N = g.N - int(NA);
    gb.w = g.w + size_t(NA) * g.K;
    if (g.wsum) gb.wsum = g.wsum + NA;
    if (g.w_scale) gb.w_scale = g.w_scale + NA;
    if (g.bias) gb.bias = static_cast<const char*>(g.bias) + NA * (g.bias_dtype == LQ_F16 ? 2 : 4);
    const size_t esz = g.out_mode == OUT_F16 ? 2 : (g.out_mode == OUT_REQUANT_I8 ? 1 : 4);
    gb.out = static_cast<char*>(g.out) + NA * esz;
    if (g.residual) gb.residual = g.residual + NA;
    if (g.join_q) gb.join_q = g.join_q + NA;
    return launch_tile_cfg(gb, 0, 1, 0, st);
}

// The best tile shape depends on how the tile count falls on the 256 CUs and on
// the epilogue's share, which no simple rule predicted well (at M = 12608 the
// winner changes between K = 768 and K = 3072).  So the first launch of a problem
// shape times each candidate on the caller's own operands (every shape gives
// bit-identical results) and the choice is kept for the life of the process.
// Not while the stream is being captured, and not when LQ_TILE_AUTOTUNE=0.
struct TuneKey {
    int M, N, K, mode, conv, groups, geom[14], flags;
    bool operator==(const TuneKey& o) const { return std::memcmp(this, &o, sizeof(TuneKey)) == 0; }
};
struct TuneKeyHash {
    size_t operator()(const TuneKey& k) const {
        const unsigned char* p = reinterpret_cast<const unsigned char*>(&k);
        size_t h = 1469598103934665603ull;
        for (size_t i = 0; i < sizeof(TuneKey); ++i) h = (h ^ p[i]) * 1099511628211ull;
        return h;
    }
};
std::mutex g_tune_mu;
std::unordered_map<TuneKey, int, TuneKeyHash> g_tune;

// One tuned choice as a line of text: "lq-tune-1" followed by the key's integers and the
// chosen tile_config.  What lq_tune_export writes and lq_tune_import reads.
constexpr int kTuneKeyInts = sizeof(TuneKey) / sizeof(int);
static_assert(sizeof(TuneKey) == kTuneKeyInts * sizeof(int), "the key is all ints");

int tune_import_text(const char* text, int* accepted) {
    int n_ok = 0;
    const char* p = text;
    while (p && *p) {
        const char* eol = std::strchr(p, '\n');
        std::string line(p, eol ? size_t(eol - p) : std::strlen(p));
        p = eol ? eol + 1 : nullptr;
        if (line.compare(0, 10, "lq-tune-1 ") != 0) continue;  // blank lines, comments, other versions
        int v[kTuneKeyInts + 1];
        const char* q = line.c_str() + 10;
        int got = 0;
        while (got < kTuneKeyInts + 1) {
            char* end = nullptr;
            const long x = std::strtol(q, &end, 10);
            if (end == q) break;
            v[got++] = int(x);
            q = end;
        }
        if (got != kTuneKeyInts + 1) return fail(LQ_ERR_VALUE, "tune_import: malformed line '%s'", line.c_str());
        const int shape = v[kTuneKeyInts] & 0xff;
        if (shape < 1 || shape > 22) return fail(LQ_ERR_VALUE, "tune_import: tile shape %d in '%s'", shape, line.c_str());
        TuneKey key;
        std::memcpy(&key, v, sizeof(key));
        std::lock_guard<std::mutex> lock(g_tune_mu);
        g_tune[key] = v[kTuneKeyInts];
        ++n_ok;
    }
    if (accepted) *accepted = n_ok;
    return LQ_OK;
}

// LQ_TUNE_FILE names a file of such lines that is read before the first lookup, so that a
// deployment pays for tuning once and not in every process (a missing file is not an error).
void tune_import_env_file() {
    static std::once_flag once;
    std::call_once(once, [] {
        const char* path = std::getenv("LQ_TUNE_FILE");
        if (!path || !*path) return;
        std::FILE* f = std::fopen(path, "r");
        if (!f) return;
        std::string text;
        char buf[4096];
        size_t n;
        while ((n = std::fread(buf, 1, sizeof buf, f)) > 0) text.append(buf, n);
        std::fclose(f);
        (void)tune_import_text(text.c_str(), nullptr);
    });
}

bool autotune_enabled() {
    static const bool on = [] {
        const char* e = std::getenv("LQ_TILE_AUTOTUNE");
        return !(e && e[0] == '0');
    }();
    return on;
}

int tuned_tile_shape(const GemmArgs& g, int conv, int groups, hipStream_t st, int* cfg_out) {
    TuneKey key;
    std::memset(&key, 0, sizeof(key));
    key.M = g.M, key.N = g.N, key.K = g.K, key.mode = g.out_mode, key.conv = conv, key.groups = groups;
    if (conv) {
        const int geom[8] = {g.cH, g.cW, g.cCin, g.cKW, g.csh * 16 + g.csw, g.cph * 256 + g.cpw,
                             g.cdh * 16 + g.cdw, g.cOW};
        std::memcpy(key.geom, geom, sizeof(geom));
    }
    if (conv == 2) {
        const int geom3[6] = {g.cD, g.cOD, g.cKH, g.csd, g.cpd, g.cdd};
        std::memcpy(key.geom + 8, geom3, sizeof(geom3));
    }
    key.flags = (g.residual ? 1 : 0) | (g.a_scale_per_row ? 2 : 0) | (g.bias ? 4 : 0) | (g.join_q ? 8 : 0) |
                (g.gelu ? 16 : 0) | (g.range ? 32 : 0);
    tune_import_env_file();
    {
        std::lock_guard<std::mutex> lock(g_tune_mu);
        auto it = g_tune.find(key);
        if (it != g_tune.end()) {
            *cfg_out = it->second;
            return LQ_OK;
        }
    }
    int fallback = heuristic_tile_shape(g, conv, groups);
    *cfg_out = fallback;
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    LQ_HIP(hipStreamIsCapturing(st, &capturing));
    // too little work to be worth timing: a handful of tiles whatever the shape
    const double ops = 2.0 * g.M * double(g.N) * g.K * groups;
    // timing launches the candidates many times into the caller's output: not when that output
    // is also an operand the epilogue reads (an in-place residual or join would be applied
    // once per timing launch)
    const bool in_place = (g.residual && static_cast<const void*>(g.residual) == g.out) ||
                          (g.join_q && static_cast<const void*>(g.join_q) == g.out);
    if (!autotune_enabled() || capturing != hipStreamCaptureStatusNone || ops < 5e8 || in_place) return LQ_OK;

    // candidates are whole tile_config values (shape | schedule << 8)
    int cands[24], n = 0;
    if (conv == 2) {
        // the shapes the volumetric gather is built for
        if (g.N <= 64) cands[n++] = 6;
        cands[n++] = 5;
        if (g.N > 64) cands[n++] = 3, cands[n++] = 4;
        if (long((g.M + 127) / 128) * ((g.N + 127) / 128) * groups < 256) cands[n++] = 9;
        if (conv_halo_applies(g, conv)) cands[n++] = 15;
    } else {
        if (g.N <= 64) cands[n++] = 6;
        cands[n++] = 5;
        if (g.K <= 256) cands[n++] = 8;  // one to four k-iterations: latency-bound tiles, four blocks per CU
        if (g.N > 64) cands[n++] = 3, cands[n++] = 4;
        if (g.N > 128 && g.M > 128) cands[n++] = 1, cands[n++] = 11;
        if (g.N > 128 && !conv) cands[n++] = 12;
        // large plain GEMMs: the ping-pong kernel's 256 x 352 and 256 x 256 tiles
        // (with a GELU in the epilogue they lose in the network - ViT-B/16 fc1: 5.22 against 5.08 ms per
        // batch - even where they tie in isolation: one block per CU, nothing overlaps its epilogue)
        if (pp_applies(g, conv, groups) && !g.gelu) {
            cands[n++] = 13, cands[n++] = 14, cands[n++] = 16;
            // shorter tiles where they put a block on more of the CUs in one round
            const long t192 = long((g.M + 255) / 256) * ((g.N + 191) / 192);
            const long t224 = long((g.M + 223) / 224) * ((g.N + 191) / 192);
            const long t160 = long((g.M + 159) / 160) * ((g.N + 255) / 256);
            if (t192 < 256 && t224 > t192 && t224 <= 256) cands[n++] = 21;
            if (t192 < 256 && t160 > t192 && t160 <= 256) cands[n++] = 22;
        }
        // a long K over few tiles (late convolution stages): split K between the idle CUs
        const long tiles128 = long((g.M + 127) / 128) * ((g.N + 127) / 128) * groups;
        if (tiles128 * 2 <= 512 && g.K >= 2048) cands[n++] = 5 | (2 << 8);
        if (tiles128 < 256) cands[n++] = 9;  // ... or cover the chip with 64 x 64 tiles
        if (tiles128 < 256 && g.K >= 1024) cands[n++] = 10;  // ... with 128-byte k-iterations
        // filters with several taps at stride 1: the input halo of a box of outputs held in LDS
        if (conv && g.K > g.cCg && conv_halo_applies(g, conv)) {
            cands[n++] = 15;
            // smaller boxes where 256-position boxes leave CUs without one
            const long boxes256 = (long(g.M) + 255) / 256 * ((g.N + 63) / 64) * groups;
            if (boxes256 < 1024 && conv_halo_applies(g, conv, 7)) cands[n++] = 18;
            if (boxes256 < 512 && conv_halo_applies(g, conv, 6)) cands[n++] = 19;
        }
        if (conv_few_applies(g, conv, groups)) cands[n++] = 20;
        // whole rounds of 256 x 256 tiles plus a remainder (see launch_split)
        if (!conv && groups == 1 && g.range == nullptr && g.M >= 256) {
            const long tiles_m = (g.M + 255) / 256, tiles_n = g.N / 256;
            const long rounds = tiles_m * tiles_n / 256;
            const long a_tiles = rounds > 0 ? rounds * 256 / tiles_m : 0;
            if (a_tiles > 0 && a_tiles * 256 < g.N && a_tiles < 32768)
                cands[n++] = kSplitShape | (1 << 8) | int(a_tiles << 16);
        }
    }
    hipEvent_t e0, e1;
    LQ_HIP(hipEventCreate(&e0));
    LQ_HIP(hipEventCreate(&e1));
    float best = 1e30f;
    int rc = LQ_OK;
    bool timed = true;
    for (int i = 0; i < n && rc == LQ_OK && timed; ++i) {
        const int shape = cands[i] & 0xff, sched = ((cands[i] >> 8) & 0xff) ? ((cands[i] >> 8) & 0xff) : 1;
        const int a_tiles = cands[i] >> 16;
        auto launch = [&] {
            return a_tiles ? launch_split(g, a_tiles, st) : launch_tile_shape(g, conv, groups, shape, sched, st);
        };
        rc = launch();  // warm: code load, attributes (and the remainder's own tuning)
        if (rc) break;
        // Candidates can be within a few percent of each other and the clock takes a while
        // to settle under load: every candidate runs for about a millisecond per timing (its
        // own launches warm the chip up for it), and the better of two timings counts.
        timed = hipEventRecord(e0, st) == hipSuccess;
        rc = launch();
        float one = 0.0f;
        timed = timed && rc == LQ_OK && hipEventRecord(e1, st) == hipSuccess &&
                hipEventSynchronize(e1) == hipSuccess && hipEventElapsedTime(&one, e0, e1) == hipSuccess;
        if (!timed || rc) break;
        int reps = one > 0.0f ? int(1.0f / one) : 4;
        reps = reps < 4 ? 4 : (reps > 40 ? 40 : reps);
        for (int pass = 0; pass < 2 && timed && rc == LQ_OK; ++pass) {
            timed = hipEventRecord(e0, st) == hipSuccess;
            for (int r = 0; r < reps && rc == LQ_OK; ++r) rc = launch();
            float ms = 0.0f;
            timed = timed && rc == LQ_OK && hipEventRecord(e1, st) == hipSuccess &&
                    hipEventSynchronize(e1) == hipSuccess && hipEventElapsedTime(&ms, e0, e1) == hipSuccess;
            if (timed && ms / reps < best) best = ms / reps, *cfg_out = cands[i];
        }
    }
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    if (!timed && rc == LQ_OK) {  // timing unavailable: keep the rule-based choice, do not cache
        *cfg_out = fallback;
        return LQ_OK;
    }
    if (rc) return rc;
    std::lock_guard<std::mutex> lock(g_tune_mu);
    g_tune[key] = *cfg_out;
    return LQ_OK;
}

// tile_config: low byte = tile shape (0 = choose, 1..9 = a specific one), next
// byte = schedule (0 = choose, 1 = block per tile, 2 = stream-K, 3 = stream-K over
// the leftover tiles only), bits 16..30 = number of leading 256-column tiles given to
// shape 1 with the remaining columns tuned separately (0 = no split).
int launch_tile_cfg(const GemmArgs& g, int conv, int groups, int tile_config, hipStream_t st) {
    int cfg = tile_config & 0xff;
    int schedule = (tile_config >> 8) & 0xff;
    int a_tiles = (tile_config >> 16) & 0x7fff;
    if (cfg == 0) {
        int tuned = 0;
        int rc = tuned_tile_shape(g, conv, groups, st, &tuned);
        if (rc) return rc;
        cfg = tuned & 0xff;
        if (schedule == 0) schedule = (tuned >> 8) & 0xff;
        a_tiles = tuned >> 16;
    }
    if (a_tiles > 0) {
        LQ_REQUIRE(!conv && groups == 1 && g.range == nullptr, LQ_ERR_VALUE,
                   "tile_config: a column split needs a plain GEMM without a kept range");
        const int rc = launch_split(g, a_tiles, st);
        t_last_tile_config = kSplitShape | (1 << 8) | (a_tiles << 16);
        return rc;
    }
    t_last_tile_config = cfg | ((schedule ? schedule : 1) << 8);
    return launch_tile_shape(g, conv, groups, cfg, schedule, st);
}

// ---------------------------------------------------------------- skinny kernel
// M <= 16*MT.  A block owns 16 weight rows; its 4 wavefronts each take a
// quarter of K.  In load c of a 256-byte K block, lane (n = lane&15, g = lane>>4) reads
// bytes [64c + 16g, 64c + 16g + 16) of weight row n, so the four lanes of a row fetch one
// whole 64-byte segment per instruction; the activation operand uses the same
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

    // Weight bytes are streamed once, so memory-level parallelism is what counts:
    // PF K blocks (4 KiB per wavefront each) are requested before the first MFMA.
    constexpr int PF = 4;
    const int8_t* wrow = g.w + size_t(nr) * g.K;
    for (int kbc = kb0; kbc < kb1; kbc += PF) {
        v4i wf[PF][4];
#pragma unroll
        for (int u = 0; u < PF; ++u) {
            const int kbase = (kbc + u) * 256 + lg * 16;
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const int k = kbase + c * 64;
                wf[u][c] = (kbc + u < kb1 && k < g.K) ? *reinterpret_cast<const v4i*>(wrow + k)
                                                     : v4i{0, 0, 0, 0};
            }
        }
#pragma unroll
        for (int u = 0; u < PF; ++u) {
            if (kbc + u >= kb1) break;
            const int kbase = (kbc + u) * 256 + lg * 16;
#pragma unroll
            for (int t = 0; t < MT; ++t) {
                const int m = t * 16 + ln;
                const int8_t* arow = g.a + size_t(m < g.M ? m : g.M - 1) * g.K;
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    const int k = kbase + c * 64;
                    v4i af = (k < g.K && m < g.M) ? *reinterpret_cast<const v4i*>(arow + k)
                                                  : v4i{0, 0, 0, 0};
                    acc[t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(af, wf[u][c], acc[t], 0, 0, 0);
                }
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

// ---------------------------------------------------------------- one activation row
// M == 1: the weight matrix is read exactly once and nothing else of size moves, so the
// kernel is a stream of 16-byte loads.  What the memory pipeline charges for is load
// instructions, whatever their active lanes or bytes (measured: the same 45 MB through
// 8-byte loads takes twice as long; an activation load with four active lanes costs as much
// as a full one), so every weight instruction moves a full KiB of one row and the activation
// row costs K / 1024 instructions per block: it is copied to LDS once and read from there.
// A wavefront owns four consecutive rows and requests all of their bytes (16 loads for
// K = 4096) before the first dot product; v_dot4_i32_i8 needs no operand layout, so there
// is no transposition.  Sums over the 64 lanes are exact integer adds.
__global__ __launch_bounds__(512) void qgemv1_kernel(GemmArgs g) {
    extern __shared__ int8_t a_lds[];  // K bytes rounded up to a multiple of 4 KiB
    constexpr int RW = 4;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, waves = blockDim.x >> 6;
    const int kchunks = (g.K + 4095) / 4096;
    // the activation row is requested first: loads return in order
    for (int k = tid * 16; k < kchunks * 4096; k += blockDim.x * 16) {
        const v4i v = k < g.K ? *reinterpret_cast<const v4i*>(g.a + k) : v4i{0, 0, 0, 0};
        *reinterpret_cast<v4i*>(a_lds + k) = v;
    }
    float S = 1.0f, Z = 0.0f;
    if (g.out_mode == OUT_REQUANT_I8 || g.out_mode == OUT_FAKEQUANT_F32) {
        S = g.out_scale[0];
        Z = g.out_zp[0];
    }
    const float as = g.a_scale ? g.a_scale[0] : 1.0f;
    const int nb = (blockIdx.x * waves + wave) * RW;
    // lane r finishes row nb + r: its column operands are requested before the weights
    const int n_mine = nb + (lane < RW ? lane : 0);
    ColParams cp{1.0f, -0.0f, 0};
    if (lane < RW && n_mine < g.N) cp = load_col(g, n_mine);

    int acc[RW];
#pragma unroll
    for (int r = 0; r < RW; ++r) acc[r] = 0;
    for (int kc = 0; kc < kchunks; ++kc) {
        v4i wv[RW][4];
#pragma unroll
        for (int r = 0; r < RW; ++r) {
            const int n = nb + r;
            const int8_t* row = g.w + size_t(n < g.N ? n : 0) * g.K;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int k = kc * 4096 + i * 1024 + lane * 16;
                wv[r][i] = (n < g.N && k < g.K) ? *reinterpret_cast<const v4i*>(row + k) : v4i{0, 0, 0, 0};
            }
        }
        if (kc == 0) __syncthreads();  // the activation row is in LDS (uniform: every wave runs chunk 0)
        v4i av[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) av[i] = *reinterpret_cast<const v4i*>(a_lds + kc * 4096 + i * 1024 + lane * 16);
#pragma unroll
        for (int r = 0; r < RW; ++r)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                acc[r] = __builtin_amdgcn_sdot4(wv[r][i].x, av[i].x, acc[r], false);
                acc[r] = __builtin_amdgcn_sdot4(wv[r][i].y, av[i].y, acc[r], false);
                acc[r] = __builtin_amdgcn_sdot4(wv[r][i].z, av[i].z, acc[r], false);
                acc[r] = __builtin_amdgcn_sdot4(wv[r][i].w, av[i].w, acc[r], false);
            }
    }
    // rotations inside each row of 16 lanes, then the four row totals through scalar registers
    int mine = 0;
#pragma unroll
    for (int r = 0; r < RW; ++r) {
        int v = acc[r];
        v += __builtin_amdgcn_update_dpp(0, v, 0x128, 0xf, 0xf, false);
        v += __builtin_amdgcn_update_dpp(0, v, 0x124, 0xf, 0xf, false);
        v += __builtin_amdgcn_update_dpp(0, v, 0x122, 0xf, 0xf, false);
        v += __builtin_amdgcn_update_dpp(0, v, 0x121, 0xf, 0xf, false);
        v = __builtin_amdgcn_readlane(v, 0) + __builtin_amdgcn_readlane(v, 16) + __builtin_amdgcn_readlane(v, 32) +
            __builtin_amdgcn_readlane(v, 48);
        if (lane == r) mine = v;
    }
    if (lane < RW && n_mine < g.N) epilogue_store(g, 0, n_mine, mine, as, cp, S, Z);
}

// ---------------------------------------------------------------- up to 16 activation rows
// 2 <= M <= 16, K >= 1024: one block of 16 wavefronts per compute unit's share of the rows
// (rows_per_block <= 16 G), the wavefronts split the 256-byte K blocks.  A wavefront loads
// the activation fragment of its K block once and uses it for all G row groups, so the
// activation costs 4 load instructions per 4 G weight instructions instead of one per MFMA,
// and all of a wavefront's weight bytes are requested before its first MFMA.  Partial sums
// meet in LDS through integer atomic adds (order-independent, hence deterministic); the
// wavefronts that finish early add theirs off the critical path.
template <int G>
__global__ __launch_bounds__(1024) void qgemm_skinny16_kernel(GemmArgs g, int rows_per_block) {
    __shared__ int red[G * 4 * 64];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, waves = blockDim.x >> 6;
    const int ln = lane & 15, lg = lane >> 4;
    for (int i = tid; i < G * 4 * 64; i += blockDim.x) red[i] = 0;
    const int n0 = blockIdx.x * rows_per_block;
    const int n_end = n0 + rows_per_block < g.N ? n0 + rows_per_block : g.N;

    // the epilogue's operands are requested first (wavefront j finishes row group j)
    float S = 1.0f, Z = 0.0f, as_uniform = 1.0f;
    ColParams cp{1.0f, -0.0f, 0};
    const int n_mine = n0 + wave * 16 + ln;
    if (wave < G && n_mine < n_end) {
        if (g.out_mode == OUT_REQUANT_I8 || g.out_mode == OUT_FAKEQUANT_F32) {
            S = g.out_scale[0];
            Z = g.out_zp[0];
        }
        cp = load_col(g, n_mine);
        as_uniform = g.a_scale ? g.a_scale[0] : 1.0f;
    }
    __syncthreads();  // the accumulators are zero before anyone adds to them

    const int kblocks = (g.K + 255) / 256;
    const bool m_ok = ln < g.M;
    const int8_t* arow = g.a + size_t(m_ok ? ln : 0) * g.K;
    v4i acc[G];
#pragma unroll
    for (int j = 0; j < G; ++j) acc[j] = v4i{0, 0, 0, 0};
    for (int kb = wave; kb < kblocks; kb += waves) {
        const int kbase = kb * 256 + lg * 16;
        v4i af[4], wf[G][4];
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const int k = kbase + c * 64;
            af[c] = (m_ok && k < g.K) ? *reinterpret_cast<const v4i*>(arow + k) : v4i{0, 0, 0, 0};
        }
#pragma unroll
        for (int j = 0; j < G; ++j) {
            const int n = n0 + j * 16 + ln;
            const int8_t* wrow = g.w + size_t(n < n_end ? n : n0) * g.K;
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const int k = kbase + c * 64;
                wf[j][c] = (n < n_end && k < g.K) ? *reinterpret_cast<const v4i*>(wrow + k) : v4i{0, 0, 0, 0};
            }
        }
#pragma unroll
        for (int c = 0; c < 4; ++c)
#pragma unroll
            for (int j = 0; j < G; ++j)
                acc[j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(af[c], wf[j][c], acc[j], 0, 0, 0);
    }
#pragma unroll
    for (int j = 0; j < G; ++j)
#pragma unroll
        for (int r = 0; r < 4; ++r)
            __hip_atomic_fetch_add(&red[(j * 4 + r) * 64 + lane], acc[j][r], __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_WORKGROUP);
    __syncthreads();
    if (wave >= G || n_mine >= n_end) return;
    // red[(j*4 + r)*64 + lane] is row 4*(lane>>4) + r of the activations, weight row n0 + 16 j + (lane&15)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int mm = 4 * lg + r;
        if (mm < g.M) {
            const float as = g.a_scale_per_row ? g.a_scale[mm] : as_uniform;
            epilogue_store(g, mm, n_mine, red[(wave * 4 + r) * 64 + lane], as, cp, S, Z);
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

// One thread per output element: the affine-weight corrections on the stored raw
// accumulator, in wrapping 32-bit arithmetic (the true value fits int32, so every partial
// wrap cancels), then the ordinary scalar epilogue.
__global__ __launch_bounds__(256) void affine_fixup_kernel(GemmArgs g, const int32_t* __restrict__ acc,
                                                           const int32_t* __restrict__ asum, int asum_ld,
                                                           int n_per_group, const int32_t* __restrict__ w_zp,
                                                           int kdot) {
    const size_t total = size_t(g.M) * g.N;
    float S = 1.0f, Z = 0.0f;
    if (g.out_mode == OUT_REQUANT_I8 || g.out_mode == OUT_FAKEQUANT_F32) {
        S = g.out_scale[0];
        Z = g.out_zp[0];
    }
    const int za = g.a_zp_dev ? int(g.a_zp_dev[0]) + g.a_zp : g.a_zp;
    for (size_t idx = size_t(blockIdx.x) * 256 + threadIdx.x; idx < total;
         idx += size_t(gridDim.x) * 256) {
        const int m = int(idx / g.N), n = int(idx % g.N);
        ColParams c = load_col(g, n);
        const uint32_t zw = uint32_t(w_zp[n]);
        const uint32_t rs = uint32_t(asum[size_t(m) * asum_ld + n / n_per_group]);
        const uint32_t eff = uint32_t(acc[idx]) - uint32_t(c.corr) - zw * rs + uint32_t(kdot) * uint32_t(za) * zw;
        c.corr = 0;
        const float as = g.a_scale ? g.a_scale[g.a_scale_per_row ? m : 0] : 1.0f;
        epilogue_store(g, m, n, int32_t(eff), as, c, S, Z);
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

int pad_table(const int8_t** table) {
    static void* tables[16] = {nullptr};
    static std::mutex mu;
    int dev = 0;
    LQ_HIP(hipGetDevice(&dev));
    LQ_REQUIRE(dev >= 0 && dev < 16, LQ_ERR_DEVICE, "device index %d out of range", dev);
    std::lock_guard<std::mutex> lock(mu);  // two threads' first calls must not both build it
    if (!tables[dev]) {
        uint8_t host[256 * 16];
        for (int v = 0; v < 256; ++v)
            for (int i = 0; i < 16; ++i) host[v * 16 + i] = uint8_t(v);
        void* p = nullptr;
        LQ_HIP(hipMalloc(&p, sizeof host));
        LQ_HIP(hipMemcpy(p, host, sizeof host, hipMemcpyHostToDevice));
        tables[dev] = p;
    }
    *table = static_cast<const int8_t*>(tables[dev]);
    return LQ_OK;
}

int run_tile_kernel(const GemmArgs& g_in, int conv, int groups, int tile_config, hipStream_t st) {
    GemmArgs g = g_in;
    const int8_t* table = nullptr;
    int rc = pad_table(&table);
    if (rc) return rc;
    g.zeros = table;
    if (conv) {
        const int zp = g.a_zp;  // the stored code of real 0.0
        g.pad_src = table + size_t(uint8_t(int8_t(zp))) * 16;
        return launch_tile_cfg(g, conv, groups, tile_config, st);
    }
    return launch_tile_cfg(g, 0, 1, tile_config, st);
}

int run_gemm(const GemmArgs& g_in, int force_path, int tile_config, hipStream_t st) {
    GemmArgs g = g_in;
    const bool vec_ok = g.K % 16 == 0 && g.K > 0 && aligned16(g.a) && aligned16(g.w);
    int path = force_path;  // 0 = choose, 1 = tile, 2 = skinny, 3 = naive
    if (path == 0) path = !vec_ok ? 3 : (g.M <= 64 && g.range == nullptr ? 2 : 1);
    // only the tile kernel keeps the range of what it writes
    LQ_REQUIRE(g.range == nullptr || path == 1, LQ_ERR_NOT_IMPLEMENTED,
               "qlinear_i8: a kept range needs the tile kernel (K %% 16 == 0, aligned operands)");
    LQ_REQUIRE(path == 3 || vec_ok, LQ_ERR_VALUE,
               "qlinear_i8: MFMA paths need K %% 16 == 0 and 16-byte aligned operands");
    if (path == 1) {
        int rc = run_tile_kernel(g, 0, 1, tile_config, st);
        if (rc) return rc;
    } else if (path == 2) {
        LQ_REQUIRE(g.M <= 64, LQ_ERR_SHAPE, "qlinear_i8: skinny path needs M <= 64 (M = %d)", g.M);
        if (g.M == 1 && g.K <= 65536) {
            // four rows per wavefront; as many wavefronts per block (up to 8) as still leave 256 blocks
            int waves = 8;
            while (waves > 1 && (g.N + 4 * waves - 1) / (4 * waves) < 256) waves >>= 1;
            const unsigned blocks = unsigned((g.N + 4 * waves - 1) / (4 * waves));
            const size_t lds = size_t((g.K + 4095) / 4096) * 4096;
            hipLaunchKernelGGL(qgemv1_kernel, dim3(blocks), dim3(waves * 64), lds, st, g);
            LQ_CHECK_LAUNCH("qgemv1");
            return LQ_OK;
        }
        if (g.M <= 16 && g.K >= 1024) {
            int R = (g.N + 255) / 256;  // one block per compute unit when the rows allow it
            R = R < 16 ? 16 : (R > 64 ? 64 : R);
            const int G = (R + 15) / 16;
            const dim3 grid16{unsigned((g.N + R - 1) / R)}, block16{1024};
            switch (G) {
            case 1: hipLaunchKernelGGL((qgemm_skinny16_kernel<1>), grid16, block16, 0, st, g, R); break;
            case 2: hipLaunchKernelGGL((qgemm_skinny16_kernel<2>), grid16, block16, 0, st, g, R); break;
            case 3: hipLaunchKernelGGL((qgemm_skinny16_kernel<3>), grid16, block16, 0, st, g, R); break;
            default: hipLaunchKernelGGL((qgemm_skinny16_kernel<4>), grid16, block16, 0, st, g, R); break;
            }
            LQ_CHECK_LAUNCH("qgemm_skinny16");
            return LQ_OK;
        }
        dim3 grid{unsigned((g.N + 15) / 16)}, block{256};
        if (g.M <= 16)
            hipLaunchKernelGGL((qgemm_skinny_kernel<1>), grid, block, 0, st, g);
        else if (g.M <= 32)
            hipLaunchKernelGGL((qgemm_skinny_kernel<2>), grid, block, 0, st, g);
        else
            hipLaunchKernelGGL((qgemm_skinny_kernel<4>), grid, block, 0, st, g);
        LQ_CHECK_LAUNCH("qgemm_skinny");
    } else {
        size_t blocks = (size_t(g.M) * g.N + 255) / 256;
        if (blocks > 65536) blocks = 65536;
        hipLaunchKernelGGL(qgemm_naive_kernel, dim3(unsigned(blocks)), dim3(256), 0, st, g);
        LQ_CHECK_LAUNCH("qgemm_naive");
    }
    return LQ_OK;
}

}  // namespace lq

namespace {

// x = every float32 bit pattern of [first, first + count): the tile epilogue's requantize
// (quant_fast: reciprocal multiply with a guard band, division for the rest), in its three
// forms (the code, the code minus the zero point, the code shifted into 0..255), against the
// plain [floor at zero,] divide-round-add-clamp, compared as the codes the two would store.
__global__ __launch_bounds__(256) void quant_route_check_kernel(float s, float z, float lo, float hi, int relu,
                                                                unsigned long long first,
                                                                unsigned long long count,
                                                                unsigned long long* mismatches,
                                                                unsigned long long* divided) {
    const lq::QGrid G = lq::make_qgrid(s, z, lo, hi, true, relu != 0);
    const lq::QGrid Gb = lq::make_qgrid(s, z, lo, hi, true, relu != 0, true);  // codes as unsigned bytes
    unsigned long long bad = 0, slow = 0;
    for (unsigned long long i = blockIdx.x * 256ull + threadIdx.x; i < count; i += gridDim.x * 256ull) {
        const float x = __uint_as_float(unsigned(first + i));
        const float fast = lq::quant_fast<false>(x, G);
        const float centered = lq::quant_fast<false, true>(x, G);
        const float xr = (relu && x < 0.0f) ? 0.0f : x;
        const float u = lq::q_core(xr, s, z, lo, hi);
        const float plain = (u != u) ? 0.0f : u;
        const float plain_c = plain - z;
        const float biased = lq::quant_fast<false>(x, Gb);
        bad += (__float_as_uint(fast) != __float_as_uint(plain) && !(fast == 0.0f && plain == 0.0f)) ||
               (__float_as_uint(centered) != __float_as_uint(plain_c) && !(centered == 0.0f && plain_c == 0.0f)) ||
               !(biased == plain + Gb.bias) || (Gb.in_byte && !(biased >= 0.0f && biased <= 255.0f));
        const float tp = x * G.inv;
        slow += !(__builtin_fabsf(tp - __builtin_rintf(tp)) < 0.5f - 0x1p-12f);
    }
    if (bad) atomicAdd(mismatches, bad);
    if (slow) atomicAdd(divided, slow);
}

}  // namespace

extern "C" {

int lq_selftest_requant_route(float scale, float zp, int qmin, int qmax, int relu, unsigned long long first_bits,
                              unsigned long long count, unsigned long long* mismatches,
                              unsigned long long* divided, lq_stream stream) {
    LQ_REQUIRE(mismatches && divided, LQ_ERR_VALUE, "selftest_requant_route: NULL counter");
    LQ_REQUIRE(first_bits + count <= (1ull << 32), LQ_ERR_VALUE, "selftest_requant_route: range beyond 2^32");
    hipStream_t st = as_stream(stream);
    int rc = lq_fill_bytes(mismatches, 0, sizeof(unsigned long long), stream);
    if (rc == LQ_OK) rc = lq_fill_bytes(divided, 0, sizeof(unsigned long long), stream);
    if (rc) return rc;
    if (count == 0) return LQ_OK;
    hipLaunchKernelGGL(quant_route_check_kernel, dim3(4096), dim3(256), 0, st, scale, zp, float(qmin), float(qmax),
                       relu, first_bits, count, mismatches, divided);
    LQ_CHECK_LAUNCH("selftest_requant_route");
    return LQ_OK;
}

int lq_last_tile_config(void) { return t_last_tile_config; }

int lq_tune_export(char* buf, size_t capacity, size_t* needed) {
    LQ_REQUIRE(needed, LQ_ERR_VALUE, "tune_export: needed is NULL");
    std::string text;
    {
        std::lock_guard<std::mutex> lock(g_tune_mu);
        for (const auto& kv : g_tune) {
            text += "lq-tune-1";
            int v[kTuneKeyInts];
            std::memcpy(v, &kv.first, sizeof(kv.first));
            for (int i = 0; i < kTuneKeyInts; ++i) text += " " + std::to_string(v[i]);
            text += " " + std::to_string(kv.second) + "\n";
        }
    }
    *needed = text.size() + 1;
    if (buf == nullptr) return LQ_OK;
    LQ_REQUIRE(capacity >= text.size() + 1, LQ_ERR_VALUE, "tune_export: %zu bytes needed, %zu given", text.size() + 1,
               capacity);
    std::memcpy(buf, text.c_str(), text.size() + 1);
    return LQ_OK;
}

int lq_tune_import(const char* text, int* accepted) {
    LQ_REQUIRE(text, LQ_ERR_VALUE, "tune_import: text is NULL");
    return tune_import_text(text, accepted);
}

}  // extern "C"

namespace lq {
int launch_affine_fixup(const GemmArgs& g, const int32_t* acc, const int32_t* asum, int asum_ld,
                        int n_per_group, const int32_t* w_zp, int kdot, hipStream_t st) {
    const size_t total = size_t(g.M) * g.N;
    size_t blocks = (total + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    hipLaunchKernelGGL(affine_fixup_kernel, dim3(unsigned(blocks)), dim3(256), 0, st, g, acc, asum, asum_ld,
                       n_per_group, w_zp, kdot);
    LQ_CHECK_LAUNCH("affine_fixup");
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

int lq_qlinear_i8_n(const lq_qlinear_args* p, int n, lq_stream stream) {
    LQ_REQUIRE(n >= 0, LQ_ERR_VALUE, "qlinear_i8_n: negative repeat count");
    for (int i = 0; i < n; ++i) {
        int rc = lq_qlinear_i8(p, stream);
        if (rc) return rc;
    }
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
        LQ_REQUIRE((p->a_zp == 0 && p->a_zp_dev == nullptr) || p->wsum, LQ_ERR_VALUE,
                   "qlinear_i8: a non-zero activation zero point needs the weight row sums");
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

    if (p->residual) {
        LQ_REQUIRE(p->out_mode == OUT_F32 || p->out_mode == OUT_F16, LQ_ERR_VALUE,
                   "qlinear_i8: a residual operand needs a float output mode");
        LQ_REQUIRE((p->ldr ? p->ldr : p->N) >= p->N, LQ_ERR_SHAPE, "qlinear_i8: ldr %ld < N %d", p->ldr,
                   p->N);
    }

    GemmArgs g{};
    g.residual = p->residual; g.ldr = p->ldr ? p->ldr : p->N;
    g.a = p->a; g.w = p->w; g.M = p->M; g.N = p->N; g.K = p->K;
    g.wsum = p->wsum; g.a_zp = p->a_zp; g.a_zp_dev = p->a_zp_dev;
    g.a_scale = p->a_scale; g.a_scale_per_row = p->a_scale_per_row; g.w_scale = p->w_scale;
    g.bias = p->bias; g.bias_dtype = p->bias_dtype; g.relu = p->relu; g.out_mode = p->out_mode;
    g.out_scale = p->out_scale; g.out_zp = p->out_zp;
    g.out_qmin = p->out_qmin; g.out_qmax = p->out_qmax; g.out_offset = p->out_offset;
    g.out = p->out; g.ldo = ldo; g.zeros = nullptr;
    g.cx = nullptr; g.pad_src = nullptr;
    const int jrc = set_join(g, p->join, p->out_mode, p->N, "qlinear_i8");
    if (jrc) return jrc;
    LQ_REQUIRE(p->gelu == 0 || p->out_mode == OUT_F32, LQ_ERR_VALUE, "qlinear_i8: GELU needs out_mode F32");
    LQ_REQUIRE(p->range == nullptr || p->out_mode == OUT_F32, LQ_ERR_VALUE,
               "qlinear_i8: a kept range needs out_mode F32");
    g.gelu = p->gelu != 0;
    g.range = p->range;

    LQ_REQUIRE(p->w_zp == nullptr || p->out_mode != OUT_ACC_I32, LQ_ERR_VALUE,
               "qlinear_i8: mode ACC_I32 returns the raw sums a * w; weight zero points cannot be applied to it");
    if (p->w_zp) {
        // affine weights: raw accumulators and the activation row sums into temporaries,
        // then one elementwise pass with the corrections and the epilogue proper
        LQ_REQUIRE(p->wsum, LQ_ERR_VALUE, "qlinear_i8: affine weights need the weight row sums");
        LQ_REQUIRE(p->range == nullptr, LQ_ERR_VALUE, "qlinear_i8: a kept range is not available with affine weights");
        LQ_REQUIRE(p->K <= 33025, LQ_ERR_SHAPE,
                   "qlinear_i8: K = %d overflows the int32 accumulator with affine weights", p->K);
        hipStream_t st = as_stream(stream);
        void* tmp = nullptr;
        bool fresh = false;
        const size_t acc_bytes = (size_t(p->M) * p->N * 4 + 255) / 256 * 256;
        int rc = stream_buffer(3, acc_bytes + size_t(p->M) * 4, 0, st, &tmp, &fresh);
        if (rc) return rc;
        int32_t* acc = static_cast<int32_t*>(tmp);
        int32_t* asum = reinterpret_cast<int32_t*>(static_cast<char*>(tmp) + acc_bytes);
        GemmArgs raw{};
        raw.a = p->a; raw.w = p->w; raw.M = p->M; raw.N = p->N; raw.K = p->K;
        raw.out_mode = OUT_ACC_I32; raw.out = acc; raw.ldo = p->N;
        rc = run_gemm(raw, p->force_path, p->tile_config, st);
        if (!rc) rc = lq_rowsum_i8(p->a, asum, p->M, p->K, stream);
        if (!rc) rc = launch_affine_fixup(g, acc, asum, 1, p->N, p->w_zp, p->K, st);
        return rc;
    }
    return run_gemm(g, p->force_path, p->tile_config, as_stream(stream));
}

}  // extern "C"
