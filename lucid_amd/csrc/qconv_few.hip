// int8 convolution of an image with at most four channels (an RGB stem), on the packed
// four-channel, spatially pre-padded code image: a block owns boxes of 16 x 16 output positions
// and 64 output channels.
//
// The whole filter row of such a layer is short (K = KH * roundup4(KW) * 4 bytes, at most 256:
// 224 for a 7 x 7 filter), so every wavefront keeps the filter fragments of its 64 channels in
// registers for the life of the block, and the only operand traffic per box is the box's
// input halo - ((16-1) sh + (KH-1) dh + 1) rows of (16-1) sw + roundup4(KW) pixels, 6 KB for
// the ResNet stem - loaded into LDS once.  The tile kernel's gather fetches each 16-byte
// group of pixels once per filter row and output position through the L2 instead.
//
//   k order  : (kh, pixel quad, pixel in quad, channel) - 16-byte chunk c = kh * KQ + quad is the
//              four pixels 4 quad .. 4 quad + 3 of filter row kh; chunks past K hold zero filter
//              codes
//   A operand: the filter.  Row i of column tile j stands for output channel
//              16 (i / 4) + 4 j + i % 4 of the block, so a lane's accumulators of the four
//              tiles are 16 consecutive channels of one position and a wavefront stores 16
//              positions x 64 channels as one contiguous kilobyte
//   B operand: the positions.  Lane l of a fragment holds output column ow0 + l % 16 and chunk
//              4 ks + l / 16, read from the halo at byte ((oh sh + kh dh) HWp + ow sw + 4 quad) 4
//              as four dwords (the address is only pixel-aligned)
//   wavefront w: output rows 4 w .. 4 w + 3 of the box, one 16-position tile at a time
#include "common.hpp"
#include "qgemm.hpp"
#include "qepilogue.hpp"

using namespace lq;

namespace {

typedef int fv4i __attribute__((ext_vector_type(4)));

struct FewGeom {
    int Hp, Wp, OH, OW;   // packed image extents (pixels) and output extents
    int KH, KQ, KC;       // filter rows, 16-byte chunks per filter row, chunks in all (K / 16)
    int sh, sw, dh;
    int HH, HWq;          // halo rows and 16-byte chunks per halo row
    int tiles_h, tiles_w;
    int boxes;            // batch * tiles_h * tiles_w
};

// four values of the requantizing epilogue (floats in 0..255 plus G.bias) as one dword of codes
__device__ __forceinline__ uint32_t few_pack_codes(uint4 v, const CodePack& cpk) {
    if (cpk.pk) {
        uint32_t packed = __builtin_amdgcn_cvt_pk_u8_f32(__uint_as_float(v.x), 0, 0u);
        packed = __builtin_amdgcn_cvt_pk_u8_f32(__uint_as_float(v.y), 1, packed);
        packed = __builtin_amdgcn_cvt_pk_u8_f32(__uint_as_float(v.z), 2, packed);
        packed = __builtin_amdgcn_cvt_pk_u8_f32(__uint_as_float(v.w), 3, packed);
        return packed ^ cpk.flip;
    }
    const uint32_t o = uint32_t(cpk.add);
    const uint32_t x = uint32_t(int(__uint_as_float(v.x))), y = uint32_t(int(__uint_as_float(v.y)));
    const uint32_t z = uint32_t(int(__uint_as_float(v.z))), w = uint32_t(int(__uint_as_float(v.w)));
    return ((x + o) & 0xffu) | (((y + o) & 0xffu) << 8) | (((z + o) & 0xffu) << 16) | ((w + o) << 24);
}

template <int MODE, int KS>
__global__ __launch_bounds__(256) void qconv_few_kernel(GemmArgs g, FewGeom q) {
    extern __shared__ __attribute__((aligned(16))) int8_t smem[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int fr = lane & 15, fc = lane >> 4;
    const int N = g.N, K = g.K;
    const int n0 = int(blockIdx.y) * 64;

    int8_t* const halo = smem;
    float* const s_ws = reinterpret_cast<float*>(smem + size_t(q.HH) * q.HWq * 16);
    float* const s_bias = s_ws + 64;
    int32_t* const s_corr = reinterpret_cast<int32_t*>(s_bias + 64);

    // ---- the filter fragments of the wavefront's 64 channels, for the life of the block
    fv4i bf[KS][4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        int ch = n0 + 16 * (fr >> 2) + 4 * j + (fr & 3);
        ch = ch < N ? ch : N - 1;
        const int8_t* row = g.w + size_t(ch) * size_t(K);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            const int c = ks * 4 + fc;
            bf[ks][j] = c < q.KC ? *reinterpret_cast<const fv4i*>(row + c * 16) : fv4i{0, 0, 0, 0};
        }
    }
    // ---- where the lane's chunk of each k step starts in the halo, for output row 0 of the box
    int a_off[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        int c = ks * 4 + fc;
        c = c < q.KC ? c : 0;  // met by zero filter codes: any readable address
        const int kh = c / q.KQ, quad = c - kh * q.KQ;
        a_off[ks] = ((kh * q.dh) * (q.HWq * 4) + fr * q.sw + 4 * quad) * 4;
    }
    if (tid < 64) {
        const ColParams c = load_col(g, n0 + tid < N ? n0 + tid : N - 1);
        s_ws[tid] = c.ws, s_bias[tid] = c.bias, s_corr[tid] = c.corr;
    }

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
    constexpr bool prescaled = MODE == OUT_REQUANT_I8;
    // a lane's 16 channels as whole 16-byte stores
    const bool vec_out = n0 + 64 <= N && g.ldo % 16 == 0 && reinterpret_cast<uintptr_t>(g.out) % (16 * esize) == 0;

    const int chunks = q.HH * q.HWq;
    for (int box = blockIdx.x; box < q.boxes; box += gridDim.x) {
        int t = box;
        const int twi = t % q.tiles_w;
        t /= q.tiles_w;
        const int thi = t % q.tiles_h;
        const int b = t / q.tiles_h;
        const int oh0 = thi * 16, ow0 = twi * 16;
        const int ih0 = oh0 * q.sh, iw0 = ow0 * q.sw;  // iw0 * 4 bytes is a multiple of 16

        __syncthreads();  // the previous box's fragments have been read (first pass: nothing to wait for)
        for (int i = tid; i < chunks; i += 256) {
            const int r = i / q.HWq, cq = i - r * q.HWq;
            const int ih = ih0 + r, pix = iw0 + cq * 4;
            // rows and pixel quads past the image belong to positions past the output: never stored
            fv4i v{0, 0, 0, 0};
            if (ih < q.Hp && pix < q.Wp)
                v = *reinterpret_cast<const fv4i*>(g.cx + ((size_t(b) * q.Hp + ih) * size_t(q.Wp) + pix) * 4);
            *reinterpret_cast<fv4i*>(halo + size_t(i) * 16) = v;
        }
        __syncthreads();

#pragma unroll 1
        for (int tt = 0; tt < 4; ++tt) {
            const int ohl = wave * 4 + tt;
            const int oh = oh0 + ohl, ow = ow0 + fr;
            if (oh >= q.OH) break;  // the same for every lane of the wavefront
            const int8_t* base = halo + size_t(ohl * q.sh) * size_t(q.HWq * 16);
            fv4i acc[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[j] = fv4i{0, 0, 0, 0};
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                const uint32_t* p = reinterpret_cast<const uint32_t*>(base + a_off[ks]);
                const fv4i af{int(p[0]), int(p[1]), int(p[2]), int(p[3])};
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(bf[ks][j], af, acc[j], 0, 0, 0);
            }
            if (ow >= q.OW) continue;
            // ---- epilogue on registers.  acc[j][r]: position (oh, ow), channel n0 + 16 fc + 4 j + r
            const long m = long(b * q.OH + oh) * q.OW + ow;
            const size_t idx0 = size_t(m) * size_t(g.ldo) + size_t(n0 + 16 * fc);
            uint32_t codes[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int cl = 16 * fc + 4 * j;
                const float4 ws = *reinterpret_cast<const float4*>(s_ws + cl);
                const float4 bs = *reinterpret_cast<const float4*>(s_bias + cl);
                const int4 cr = *reinterpret_cast<const int4*>(s_corr + cl);
                ColParams c4[4] = {ColParams{ws.x, bs.x, cr.x}, ColParams{ws.y, bs.y, cr.y}, ColParams{ws.z, bs.z, cr.z},
                                   ColParams{ws.w, bs.w, cr.w}};
                if (prescaled) {
#pragma unroll
                    for (int r = 0; r < 4; ++r) c4[r].ws = as * c4[r].ws;
                }
                const fv4i a = acc[j];
                uint4 v;
                v.x = epilogue_value<MODE, prescaled>(g, a[0], prescaled ? 1.0f : as, c4[0], G);
                v.y = epilogue_value<MODE, prescaled>(g, a[1], prescaled ? 1.0f : as, c4[1], G);
                v.z = epilogue_value<MODE, prescaled>(g, a[2], prescaled ? 1.0f : as, c4[2], G);
                v.w = epilogue_value<MODE, prescaled>(g, a[3], prescaled ? 1.0f : as, c4[3], G);
                if (vec_out) {
                    if (MODE == OUT_REQUANT_I8)
                        codes[j] = few_pack_codes(v, cpk);
                    else
                        store_vec4<MODE>(g, idx0 + 4 * j, v, cpk);
                } else {
                    const int nq = n0 + cl;
                    const int left = N - nq;
                    const size_t idx = idx0 + 4 * j;
                    if (left > 0) store_scalar<MODE>(g, idx, finish_value<MODE>(g, v.x, int(m), nq, jp), cpk);
                    if (left > 1) store_scalar<MODE>(g, idx + 1, finish_value<MODE>(g, v.y, int(m), nq + 1, jp), cpk);
                    if (left > 2) store_scalar<MODE>(g, idx + 2, finish_value<MODE>(g, v.z, int(m), nq + 2, jp), cpk);
                    if (left > 3) store_scalar<MODE>(g, idx + 3, finish_value<MODE>(g, v.w, int(m), nq + 3, jp), cpk);
                }
            }
            if (MODE == OUT_REQUANT_I8 && vec_out)
                *reinterpret_cast<uint4*>(static_cast<int8_t*>(g.out) + idx0) = uint4{codes[0], codes[1], codes[2], codes[3]};
        }
    }
}

template <int MODE, int KS>
int launch_few_mode(const GemmArgs& g, const FewGeom& q, dim3 grid, size_t lds, hipStream_t st) {
    const void* fn = reinterpret_cast<const void*>(qconv_few_kernel<MODE, KS>);
    GemmArgs gc = g;
    FewGeom qc = q;
    void* kargs[] = {&gc, &qc};
    LQ_HIP(hipLaunchKernel(fn, grid, dim3(256), kargs, lds, st));
    return LQ_OK;
}

template <int KS>
int launch_few_ks(const GemmArgs& g, const FewGeom& q, dim3 grid, size_t lds, hipStream_t st) {
    switch (g.out_mode) {
    case OUT_ACC_I32: return launch_few_mode<OUT_ACC_I32, KS>(g, q, grid, lds, st);
    case OUT_F32: return launch_few_mode<OUT_F32, KS>(g, q, grid, lds, st);
    case OUT_F16: return launch_few_mode<OUT_F16, KS>(g, q, grid, lds, st);
    case OUT_REQUANT_I8: return launch_few_mode<OUT_REQUANT_I8, KS>(g, q, grid, lds, st);
    default: return launch_few_mode<OUT_FAKEQUANT_F32, KS>(g, q, grid, lds, st);
    }
}

constexpr size_t kFewMaxHalo = 40 * 1024;  // with the column parameters: inside the 64 KiB a kernel gets unasked

// Whether g describes a convolution on the packed four-channel image (16-byte "channels" groups
// of four pixels, a tap four pixels wide) that the kernel takes, and its geometry.
bool plan_few(const GemmArgs& g, int conv, int groups, FewGeom* out) {
    if (conv != 1 || groups != 1) return false;
    if (g.cCin != 4 || g.cCg != 16 || g.cdw != 4 || g.cph != 0 || g.cpw != 0) return false;
    if (g.K <= 0 || g.K % 16 != 0 || g.K > 256 || g.cKW <= 0 || (g.K / 16) % g.cKW != 0) return false;
    if (g.join_q != nullptr || g.residual != nullptr || g.gelu || g.range != nullptr || g.a_scale_per_row) return false;
    if (g.csh < 1 || g.csw < 1 || g.cdh < 1 || g.cW % 4 != 0 || !aligned16(g.cx) || !aligned16(g.w)) return false;
    if (g.cOH <= 0 || g.cOW <= 0 || g.M % (g.cOH * g.cOW) != 0) return false;
    FewGeom q{};
    q.Hp = g.cH, q.Wp = g.cW, q.OH = g.cOH, q.OW = g.cOW;
    q.KQ = g.cKW, q.KC = g.K / 16, q.KH = q.KC / q.KQ;
    q.sh = g.csh, q.sw = g.csw, q.dh = g.cdh;
    q.HH = 15 * q.sh + (q.KH - 1) * q.dh + 1;
    q.HWq = (15 * q.sw + 4 * q.KQ + 3) / 4;
    if (size_t(q.HH) * q.HWq * 16 > kFewMaxHalo) return false;
    // every window of a stored position lies inside the image (the packed route's geometry)
    if ((q.OH - 1) * q.sh + (q.KH - 1) * q.dh + 1 > q.Hp || (q.OW - 1) * q.sw + 4 * q.KQ > q.Wp) return false;
    q.tiles_h = (q.OH + 15) / 16, q.tiles_w = (q.OW + 15) / 16;
    const long boxes = long(g.M / (g.cOH * g.cOW)) * q.tiles_h * q.tiles_w;
    if (boxes <= 0 || boxes > 0x7fffffffl || size_t(g.M) * size_t(g.ldo) > 0x7fffffffffffull) return false;
    q.boxes = int(boxes);
    *out = q;
    return true;
}

}  // namespace

namespace lq {

bool conv_few_applies(const GemmArgs& g, int conv, int groups) {
    FewGeom q;
    return plan_few(g, conv, groups, &q);
}

int launch_conv_few(const GemmArgs& g, int conv, int groups, hipStream_t st) {
    FewGeom q;
    LQ_REQUIRE(plan_few(g, conv, groups, &q), LQ_ERR_NOT_IMPLEMENTED,
               "few-channel convolution kernel: needs the packed four-channel image, K <= 256, no join and a halo "
               "of at most %zu bytes", kFewMaxHalo);
    const int n_tiles = (g.N + 63) / 64;
    LQ_REQUIRE(n_tiles <= 65535, LQ_ERR_SHAPE, "few-channel convolution kernel: grid too large");
    // a block keeps its filter fragments and walks boxes: about four blocks per CU, every block
    // with the same number of boxes (or one fewer)
    const int per_block = (q.boxes + 1023) / 1024;
    const dim3 grid{unsigned((q.boxes + per_block - 1) / per_block), unsigned(n_tiles)};
    const size_t lds = size_t(q.HH) * q.HWq * 16 + 3 * 64 * 4;
    switch ((g.K + 63) / 64) {
    case 1: return launch_few_ks<1>(g, q, grid, lds, st);
    case 2: return launch_few_ks<2>(g, q, grid, lds, st);
    case 3: return launch_few_ks<3>(g, q, grid, lds, st);
    default: return launch_few_ks<4>(g, q, grid, lds, st);
    }
}

}  // namespace lq
