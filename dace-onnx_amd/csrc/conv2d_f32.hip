// ONNX Conv, 2-D, NCHW, group 1, fp32: implicit GEMM on the gfx950 matrix cores.
//
// Replaces PureConv2D (daceml/onnx/op_implementations/img_op_implementations.py:
// 164-326: zero/bias init map + 7-deep accumulate map, zero pads only, stride
// term missing) and the cudnnConvolutionForward call of
// cudnn_implementations.py:303-322.
//
// GEMM view:  Y[oc, p] = sum_k W[oc, k] * Xcol[k, p]
//     k = (c, r, s) flattened -> W is a plain row-major [M, K] matrix;
//     p = (n, oy, ox) flattened -> for a fixed oc, consecutive p inside one image
//     are consecutive floats of Y, so the swapped-operand MFMA layout (four
//     consecutive p per lane) stores 16 bytes per lane straight into NCHW.
// Xcol is never materialised: the k x p tile is gathered from X into LDS with
// padding resolved by predication. Per thread the four p of its column group
// are decomposed once (registers); per k-tile only the two k rows it loads are
// decomposed, with multiply-shift division, so the gather's integer work hides
// in the shadow of the MFMAs. Each X element is re-read KH*KW times from L2 /
// L1, never from HBM: the activation tensor of a layer fits the 256 MB cache.
#include "common.h"
#include "gemm_tile.h"

#include <stdlib.h>

namespace mi355x {

// n / d for 0 <= n < 2^31 as umulhi(n, mul) >> shr (d == 1 special-cased).
struct FastDiv {
    uint32_t d, mul, shr;
};
static FastDiv make_fastdiv(int64_t d) {
    FastDiv f;
    f.d = (uint32_t)d;
    if (d == 1) { f.mul = 0; f.shr = 0; return f; }
    uint32_t l = 0;
    while ((1ull << l) < (uint64_t)d) ++l;  // ceil(log2 d)
    const uint32_t p = 31 + l;
    f.mul = (uint32_t)(((1ull << p) + (uint64_t)d - 1) / (uint64_t)d);
    f.shr = p - 32;
    return f;
}
__device__ __forceinline__ uint32_t fdiv(uint32_t n, const FastDiv& f) {
    return f.d == 1 ? n : (__umulhi(n, f.mul) >> f.shr);
}

struct ConvArgs {
    const float* X; const float* W; const float* bias; float* Y;
    int N, C, H, Wd, M, KH, KW, OH, OW;
    int pad_t, pad_l, stride_h, stride_w, dil_h, dil_w;
    int K;          // C*KH*KW
    int64_t P;      // N*OH*OW
    int OHW;
    FastDiv div_khw, div_kw, div_ohw, div_ow;
    int64_t tiles_m, tiles_p, nwg;
    int epi;
    int vec_w;      // W tile may use 16-byte loads
    int vec_y;      // Y may use 16-byte stores (OH*OW % 4 == 0, aligned)
};

template <int BM, int BN, int BK, int WAVES_M, int WAVES_N, bool VEC_W>
__global__ __launch_bounds__(64 * WAVES_M * WAVES_N) void conv2d_f32_kernel(ConvArgs p) {
    constexpr int NT = 64 * WAVES_M * WAVES_N;
    constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
    constexpr int TM = WM / 16, TN = WN / 16;
    static_assert(WM % 16 == 0 && WN % 16 == 0 && BK % 16 == 0, "tile shape");
    using WIO = TileIO<BM, BK, VEC_W, NT>;          // weights, k-contiguous
    constexpr int XPITCH = BN + LDS_PAD;            // gathered X tile [BK][BN+4]
    constexpr int VPR = BN / 4;                     // 4-wide column groups per k row
    static_assert(NT % VPR == 0, "column group must be fixed per thread");
    constexpr int ROWS_PER_PASS = NT / VPR;
    static_assert(BK % ROWS_PER_PASS == 0, "k rows per pass");
    constexpr int XPER_T = BK / ROWS_PER_PASS;

    __shared__ __attribute__((aligned(16))) float lds_w[2][BM * WIO::PITCH];
    __shared__ __attribute__((aligned(16))) float lds_x[2][BK * XPITCH];

    const int tid = threadIdx.x;
    const int lane = tid % WAVE, wave = tid / WAVE;
    const int li = lane % 16, lq = lane / 16;
    const int wm0 = (wave / WAVES_N) * WM, wn0 = (wave % WAVES_N) * WN;

    const int64_t logical = xcd_remap(blockIdx.x, p.nwg);
    const int64_t m0 = (logical / p.tiles_p) * BM;
    const int64_t p0 = (logical % p.tiles_p) * BN;

    // ---- per-thread decomposition of its four output positions -------------
    const int c4 = tid % VPR, krow0 = tid / VPR;
    int xbase[4];   // n*C*H*W + iy0*W + ix0 (may be "negative" inside the pad)
    int iy0[4], ix0[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const int64_t pp = p0 + 4 * c4 + e;
        if (pp < p.P) {
            const uint32_t n = fdiv((uint32_t)pp, p.div_ohw);
            const uint32_t q = (uint32_t)pp - n * (uint32_t)p.OHW;
            const uint32_t oy = fdiv(q, p.div_ow);
            const uint32_t ox = q - oy * (uint32_t)p.OW;
            iy0[e] = (int)oy * p.stride_h - p.pad_t;
            ix0[e] = (int)ox * p.stride_w - p.pad_l;
            xbase[e] = (int)n * p.C * p.H * p.Wd + iy0[e] * p.Wd + ix0[e];
        } else {
            iy0[e] = -(1 << 28);  // fails every bounds test
            ix0[e] = -(1 << 28);
            xbase[e] = 0;
        }
    }

    f32x4 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

    f32x4 rw[WIO::PER_T], rx[XPER_T];
    const float* __restrict__ X = p.X;
    auto load_tiles = [&](int k0) {
        WIO::load(rw, p.W, m0, k0, p.M, p.K, p.K, 1, tid);
#pragma unroll
        for (int it = 0; it < XPER_T; ++it) {
            const int k = k0 + krow0 + it * ROWS_PER_PASS;
            f32x4 v = f32x4{0.f, 0.f, 0.f, 0.f};
            if (k < p.K) {
                const uint32_t c = fdiv((uint32_t)k, p.div_khw);
                const uint32_t rs = (uint32_t)k - c * (uint32_t)(p.KH * p.KW);
                const uint32_t r = fdiv(rs, p.div_kw);
                const uint32_t s = rs - r * (uint32_t)p.KW;
                const int dy = (int)r * p.dil_h, dx = (int)s * p.dil_w;
                const int koff = (int)c * p.H * p.Wd + dy * p.Wd + dx;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const bool ok = (unsigned)(iy0[e] + dy) < (unsigned)p.H &&
                                    (unsigned)(ix0[e] + dx) < (unsigned)p.Wd;
                    if (ok) v[e] = X[xbase[e] + koff];
                }
            }
            rx[it] = v;
        }
    };
    auto store_x = [&](float* lds) {
#pragma unroll
        for (int it = 0; it < XPER_T; ++it)
            *reinterpret_cast<f32x4*>(lds + (krow0 + it * ROWS_PER_PASS) * XPITCH + 4 * c4) = rx[it];
    };

    const int ktiles = (p.K + BK - 1) / BK;
    load_tiles(0);
    WIO::store(rw, lds_w[0], tid);
    store_x(lds_x[0]);
    __syncthreads();
    for (int kt = 0; kt < ktiles; ++kt) {
        const int buf = kt & 1;
        if (kt + 1 < ktiles) load_tiles((kt + 1) * BK);
        mma_ktile<TM, TN, BK, true, false, WIO::PITCH, XPITCH>(lds_w[buf], lds_x[buf], wm0, wn0, li, lq, acc);
        if (kt + 1 < ktiles) {
            WIO::store(rw, lds_w[buf ^ 1], tid);
            store_x(lds_x[buf ^ 1]);
        }
        __syncthreads();
    }

    // ---- epilogue: acc[i][j][r] = Y[oc = m0+wm0+16i+li][p = p0+wn0+16j+4lq+r] ----
#pragma unroll
    for (int i = 0; i < TM; ++i) {
        const int64_t oc = m0 + wm0 + i * 16 + li;
        if (oc >= p.M) continue;
        const float bv = (p.epi & MI355X_EPI_BIAS) ? p.bias[oc] : 0.f;
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int64_t pp = p0 + wn0 + j * 16 + 4 * lq;
            if (pp >= p.P) continue;
            f32x4 v = acc[i][j];
            v.x = apply_epilogue(v.x, p.epi, bv);
            v.y = apply_epilogue(v.y, p.epi, bv);
            v.z = apply_epilogue(v.z, p.epi, bv);
            v.w = apply_epilogue(v.w, p.epi, bv);
            if (p.vec_y) {
                // OH*OW % 4 == 0: the four positions share an image and are adjacent
                const uint32_t n = fdiv((uint32_t)pp, p.div_ohw);
                const uint32_t q = (uint32_t)pp - n * (uint32_t)p.OHW;
                float* dst = p.Y + ((int64_t)n * p.M + oc) * p.OHW + q;
                __builtin_nontemporal_store(v, reinterpret_cast<f32x4*>(dst));
            } else {
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    if (pp + r >= p.P) break;
                    const uint32_t n = fdiv((uint32_t)(pp + r), p.div_ohw);
                    const uint32_t q = (uint32_t)(pp + r) - n * (uint32_t)p.OHW;
                    p.Y[((int64_t)n * p.M + oc) * p.OHW + q] = v[r];
                }
            }
        }
    }
}

template <int BM, int BN, int BK, int WMs, int WNs>
static void launch_conv(const ConvArgs& p, hipStream_t st) {
    const dim3 grid((unsigned)p.nwg), block(64 * WMs * WNs);
    if (p.vec_w) hipLaunchKernelGGL((conv2d_f32_kernel<BM, BN, BK, WMs, WNs, true>), grid, block, 0, st, p);
    else hipLaunchKernelGGL((conv2d_f32_kernel<BM, BN, BK, WMs, WNs, false>), grid, block, 0, st, p);
}

struct ConvTile { int bm, bn; };
static const ConvTile kConvTiles[] = {{64, 128}, {64, 64}, {32, 64}, {16, 64}, {128, 64}};
constexpr int kNumConvTiles = sizeof(kConvTiles) / sizeof(kConvTiles[0]);

static int choose_conv_tile(int64_t M, int64_t P, int cus) {
    const char* force = getenv("MI355X_CONV_CONFIG");
    if (force && force[0] >= '0' && force[0] < '0' + kNumConvTiles) return force[0] - '0';
    double best = 1e300;
    int best_cfg = 1;
    for (int c = 0; c < kNumConvTiles; ++c) {
        const ConvTile& t = kConvTiles[c];
        const int64_t nwg = ceil_div(M, t.bm) * ceil_div(P, t.bn);
        const double rounds = (double)ceil_div(nwg, (int64_t)cus * 2);
        const double cost = rounds * (double)t.bm * t.bn * (1.0 + 24.0 * (1.0 / t.bm + 1.0 / t.bn));
        if (cost < best) { best = cost; best_cfg = c; }
    }
    return best_cfg;
}

}  // namespace mi355x

extern "C" int mi355x_conv2d_f32(const float* X, const float* W, const float* bias, float* Y,
                                 int64_t N, int64_t C, int64_t H, int64_t Wd, int64_t M,
                                 int64_t KH, int64_t KW, const int64_t* pads,
                                 const int64_t* strides, const int64_t* dilations, int epilogue,
                                 void* stream) {
    using namespace mi355x;
    MI355X_REQUIRE(N >= 0 && C >= 0 && H >= 0 && Wd >= 0 && M >= 0 && KH >= 1 && KW >= 1,
                   "conv2d: bad extents N=%lld C=%lld H=%lld W=%lld M=%lld KH=%lld KW=%lld",
                   (long long)N, (long long)C, (long long)H, (long long)Wd, (long long)M,
                   (long long)KH, (long long)KW);
    MI355X_REQUIRE(pads && strides && dilations, "conv2d: null pads/strides/dilations");
    MI355X_REQUIRE((epilogue & ~(MI355X_EPI_BIAS | MI355X_EPI_RELU)) == 0,
                   "conv2d: epilogue 0x%x not supported (bias and relu only)", epilogue);
    MI355X_REQUIRE(!(epilogue & MI355X_EPI_BIAS) || bias, "conv2d: MI355X_EPI_BIAS without bias");
    for (int i = 0; i < 4; ++i) MI355X_REQUIRE(pads[i] >= 0, "conv2d: negative pad");
    for (int i = 0; i < 2; ++i)
        MI355X_REQUIRE(strides[i] >= 1 && dilations[i] >= 1, "conv2d: stride/dilation must be >= 1");
    const int64_t eff_kh = (KH - 1) * dilations[0] + 1, eff_kw = (KW - 1) * dilations[1] + 1;
    const int64_t hin = H + pads[0] + pads[2], win = Wd + pads[1] + pads[3];
    MI355X_REQUIRE(hin >= eff_kh && win >= eff_kw, "conv2d: kernel larger than padded input");
    const int64_t OH = (hin - eff_kh) / strides[0] + 1, OW = (win - eff_kw) / strides[1] + 1;
    const int64_t P = N * OH * OW, K = C * KH * KW;
    if (P == 0 || M == 0) return MI355X_OK;
    MI355X_REQUIRE(X && W && Y, "conv2d: null pointer");
    MI355X_REQUIRE(N * C * H * Wd < ((int64_t)1 << 30) && P < ((int64_t)1 << 31) && K < ((int64_t)1 << 30) &&
                       M * K < ((int64_t)1 << 40),
                   "conv2d: tensor too large for 32-bit gather offsets");

    ConvArgs p;
    p.X = X; p.W = W; p.bias = bias; p.Y = Y;
    p.N = (int)N; p.C = (int)C; p.H = (int)H; p.Wd = (int)Wd; p.M = (int)M; p.KH = (int)KH; p.KW = (int)KW;
    p.OH = (int)OH; p.OW = (int)OW; p.OHW = (int)(OH * OW);
    p.pad_t = (int)pads[0]; p.pad_l = (int)pads[1];
    p.stride_h = (int)strides[0]; p.stride_w = (int)strides[1];
    p.dil_h = (int)dilations[0]; p.dil_w = (int)dilations[1];
    p.K = (int)K; p.P = P;
    p.div_khw = make_fastdiv(KH * KW); p.div_kw = make_fastdiv(KW);
    p.div_ohw = make_fastdiv(OH * OW); p.div_ow = make_fastdiv(OW);
    p.epi = epilogue;
    auto al16 = [](const void* q) { return (reinterpret_cast<uintptr_t>(q) & 15) == 0; };
    p.vec_w = (K % 4 == 0) && al16(W);
    p.vec_y = ((OH * OW) % 4 == 0) && al16(Y);

    int cus = mi355x_device_cu_count();
    if (cus <= 0) return set_error(MI355X_ERR_NOT_INITIALIZED, "conv2d: no usable HIP device");
    const int cfg = choose_conv_tile(M, P, cus);
    p.tiles_m = ceil_div(M, kConvTiles[cfg].bm);
    p.tiles_p = ceil_div(P, kConvTiles[cfg].bn);
    p.nwg = p.tiles_m * p.tiles_p;
    MI355X_REQUIRE(p.nwg < ((int64_t)1 << 31), "conv2d: grid too large");
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (cfg) {
        case 0: launch_conv<64, 128, 16, 2, 2>(p, st); break;
        case 1: launch_conv<64, 64, 32, 2, 2>(p, st); break;
        case 2: launch_conv<32, 64, 32, 2, 2>(p, st); break;
        case 3: launch_conv<16, 64, 32, 1, 4>(p, st); break;
        default: launch_conv<128, 64, 32, 2, 2>(p, st); break;
    }
    return check_launch("conv2d_f32_kernel");
}
