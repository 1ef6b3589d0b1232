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
#include <type_traits>
#include <utility>

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

// The part of the epilogue after bias and activation: the residual (same layout as Y, hence the same
// offset) and the activation that follows it (the last two steps of a ResNet block).
__device__ __forceinline__ f32x4 conv_epilogue_tail4(f32x4 v, int epi, const float* residual, int64_t off) {
    if (epi & MI355X_EPI_RESIDUAL) v += __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(residual + off));
    if (epi & MI355X_EPI_RELU_AFTER) v = f32x4{fmaxf(v.x, 0.f), fmaxf(v.y, 0.f), fmaxf(v.z, 0.f), fmaxf(v.w, 0.f)};
    return v;
}
__device__ __forceinline__ float conv_epilogue_tail1(float v, int epi, const float* residual, int64_t off) {
    if (epi & MI355X_EPI_RESIDUAL) v += residual[off];
    if (epi & MI355X_EPI_RELU_AFTER) v = fmaxf(v, 0.f);
    return v;
}

struct ConvArgs {
    const float* X; const float* W; const float* bias; float* Y;
    const float* residual;   // laid out like Y; read only with MI355X_EPI_RESIDUAL
    int N, C, H, Wd, M, KH, KW, OH, OW;
    int pad_t, pad_l, stride_h, stride_w, dil_h, dil_w;
    int K;          // C*KH*KW
    int64_t P;      // N*OH*OW
    int OHW;
    FastDiv div_khw, div_kw, div_ohw, div_ow;
    int64_t tiles_m, tiles_p, nwg;
    int group_m;    // tile walk order, see tile_coords
    int epi;
    int vec_w;      // W tile may use 16-byte loads
    int vec_y;      // Y may use 16-byte stores (OH*OW % 4 == 0, aligned)
    int x_bytes;    // size of X (gather kernel only; below 2^31)
    // gather kernel: the first full_tiles workgroups take whole tiles, the rest 16-position slices from p_full on
    int64_t full_tiles, p_full;
    MI355X_TRACE_MEMBER
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
                const int64_t off = ((int64_t)n * p.M + oc) * p.OHW + q;
                __builtin_nontemporal_store(conv_epilogue_tail4(v, p.epi, p.residual, off), reinterpret_cast<f32x4*>(p.Y + off));
            } else {
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    if (pp + r >= p.P) break;
                    const uint32_t n = fdiv((uint32_t)(pp + r), p.div_ohw);
                    const uint32_t q = (uint32_t)(pp + r) - n * (uint32_t)p.OHW;
                    const int64_t off = ((int64_t)n * p.M + oc) * p.OHW + q;
                    p.Y[off] = conv_epilogue_tail1(v[r], p.epi, p.residual, off);
                }
            }
        }
    }
}


// ---------------------------------------------------------------------------------------------
// Kernel for K = C*KH*KW a multiple of 32 (every convolution with C % 32 == 0, and more):
// the structure of the k-contiguous GEMM kernel (gemm_f32_nt.hip), with the im2col gather
// as its B loader.
//   * W [M, K] is k-contiguous: a lane loads its MFMA operand (row oc, 4 consecutive k)
//     straight from global memory / L2, RING tiles ahead; the 4 wave rows own disjoint
//     16-row slices of the 64-row tile, nothing is shared, W never touches LDS.
//   * Xcol is gathered TRANSPOSED: a loader thread owns one output position p and one
//     k-quad (4 consecutive k = 4 different (c, r, s) taps), reads its 4 input pixels
//     with 4-byte loads -- lanes run along p, so a wave load covers 64 neighbouring
//     pixels of one (c, r, s) tap -- and writes them as ONE 16-byte LDS write into a
//     [p][k] tile. The k-quad of a unit is the same for the whole wave: tap offsets and
//     pad tests are computed once per wave on the scalar unit. Every MFMA operand read
//     is then a 16-byte LDS read (the p-contiguous layout of the generic kernel needs
//     four 4-byte reads per operand, and on this part LDS instructions, not bytes, are
//     what limits the matrix pipe).
//   * 8 waves = 4 wave rows x 2 k-split groups (group g multiplies the g-th 16-k chunk
//     of every 32-k tile, partial sums meet in LDS at the end); three LDS buffers, a
//     six-deep register ring of gathered pixels, one barrier per tile, the tile's memory
//     instructions spread between its MFMAs.
constexpr int CG_BK = 32, CG_THREADS = 512, CG_RING = 6, CG_STAGES = 3, CG_BM = 64;
constexpr int CG_PITCH = CG_BK + LDS_PAD;
constexpr int CG_MAX_K = 4608;   // e.g. 512 input channels, 3 x 3

template <int N, class F, int... I>
__device__ __forceinline__ void cg_static_for_impl(F&& f, std::integer_sequence<int, I...>) {
    (f(std::integral_constant<int, I>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void cg_static_for(F&& f) {
    cg_static_for_impl<N>(static_cast<F&&>(f), std::make_integer_sequence<int, N>{});
}

// TN: 16-position MFMA tiles per wave; BN = 16 TN output positions per workgroup: 64 or 128, or 16 for the
// slices that even out the last round of workgroups (a quarter of the loader threads fetch them, every wave still
// multiplies its 16 output channels).
constexpr int cg_lds_floats(int tn) {
    return CG_STAGES * 16 * tn * CG_PITCH > CG_BM * 16 * tn ? CG_STAGES * 16 * tn * CG_PITCH : CG_BM * 16 * tn;
}
constexpr int cg_gcd(int a, int b) { return b == 0 ? a : cg_gcd(b, a % b); }
// TAPS: 0, or KH * KW when C % 32 == 0 (K a whole number of windows of 32 channels). Then the gather needs no tap
// table and no vector arithmetic. With k = TAPS c + rs, the unit of a wave that covers k = 32 kt + 4 kq + e meets
// the taps in a pattern that repeats every WIN = TAPS / gcd(32, TAPS) steps: write 4 kq = TAPS a + rot and
// 32 i + e = TAPS n + j for step i of a window; then rs = (j + rot) mod TAPS and c = 32 window + a + n + [j + rot >= TAPS].
// rot is fixed for a wave, so the lane keeps, for j = 0 .. TAPS - 1, the byte offset of tap (j + rot) mod TAPS
// from its position's first pixel, plus one channel where j + rot wraps, with bit 31 set where that tap is
// padding: the load of (i, e) takes register j (known at compile time) as its vector offset and the running
// channel offset (a + 32 window + n) H W 4, kept on the scalar unit, as its scalar offset.
// LEAN: a three-deep register ring and one set of X operands instead of six and two (78 registers instead of 122), so
// that three workgroups share a CU. The X operands of half the position tiles are read from LDS under the MFMAs of the
// other half.
template <int TN, int TAPS = 0, bool LEAN = false>
__device__ __forceinline__ void conv2d_f32_gather_tile(const ConvArgs& p, int64_t m0, int64_t p0, float* lds, uint32_t* lds_tap) {
    constexpr int BN = 16 * TN, BK = CG_BK, RING = LEAN ? CG_STAGES : CG_RING, PITCH = CG_PITCH;
    constexpr bool STATIC_TAPS = TAPS > 0;
    constexpr int WIN = STATIC_TAPS ? TAPS / cg_gcd(BK, TAPS ? TAPS : 1) : 1;        // steps per window
    constexpr int UNROLL1 = RING * WIN / cg_gcd(RING, WIN);                          // slot and window position both fixed
    constexpr int UNROLL = UNROLL1 % 2 == 0 ? UNROLL1 : 2 * UNROLL1;                 // ... and the operand set (step parity)
    constexpr int NTAP = STATIC_TAPS ? TAPS : 1;
    constexpr int UNITS = BN * (BK / 4);                 // (position, k-quad) units of one tile
    // whole waves of loader units share their k-quad (read once, on the scalar unit); a narrow slice has four
    // k-quads per wave and only UNITS loader threads
    constexpr bool UNIFORM_KQ = BN % WAVE == 0;
    static_assert(!STATIC_TAPS || UNIFORM_KQ, "compile-time taps need one k-quad per wave");
    static_assert(UNITS % CG_THREADS == 0 || UNITS < CG_THREADS, "whole units per thread, or fewer units than threads");
    constexpr int B_PER_T = UNITS >= CG_THREADS ? UNITS / CG_THREADS : 1;
    constexpr int STAGE = BN * PITCH;
    static_assert(UNITS >= CG_THREADS || CG_STAGES * STAGE + (CG_STAGES - 1) * STAGE + 4 * CG_THREADS <= cg_lds_floats(4), "room for the idle threads' writes");

    MI355X_TRACE_STAMP(p, 0);
    MI355X_TRACE_HWID(p);
    const int tid = threadIdx.x;
    const bool loader = UNITS >= CG_THREADS || tid < UNITS;   // whole waves
    const int lane = tid % WAVE, wave = tid / WAVE;
    const int li = lane % 16, lq = lane / 16;
    const int wm = wave % 4, ks = wave / 4;   // wave row, k-split group

    if constexpr (!STATIC_TAPS) {
        for (int k = tid; k < p.K; k += CG_THREADS) {
            const uint32_t c = fdiv((uint32_t)k, p.div_khw);
            const uint32_t rs = (uint32_t)k - c * (uint32_t)(p.KH * p.KW);
            const uint32_t r = fdiv(rs, p.div_kw);
            const uint32_t t = rs - r * (uint32_t)p.KW;
            lds_tap[k] = (rs << 27) | (c * (uint32_t)(p.H * p.Wd) + r * (uint32_t)(p.dil_h * p.Wd) + t * (uint32_t)p.dil_w);
        }
    }

    // W operand of this lane: row oc (clamped), 4 floats at k = 32 kt + 16 ks + 4 lq
    int64_t am = m0 + 16 * wm + li;
    am = am < p.M ? am : p.M - 1;
    // (as a raw buffer: the lane's row and k-quad as a 32-bit byte offset, the k-tile as the scalar offset; W spans
    // less than 2^31 bytes: launch precondition)
    const __amdgpu_buffer_rsrc_t w_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(p.W), 0, 0x7fffffff, 0x00020000);
    const uint32_t a_off = (uint32_t)(am * p.K + 16 * ks + 4 * lq) * 4u;

    // loader: this thread's output position (the same for all its units): byte offset of
    // its top-left input pixel, and one bit per filter tap (r, s) saying whether that tap
    // falls outside the image (pad) for this position. KH * KW <= 32 is a launch precondition.
    const int p_local = tid % BN;
    uint32_t xbase = 0, tap_outside = 0xffffffffu;
    int iy0 = 0, ix0 = 0;
    {
        const int64_t pp = p0 + p_local;
        if (pp < p.P && loader) {
            const uint32_t n = fdiv((uint32_t)pp, p.div_ohw);
            const uint32_t q = (uint32_t)pp - n * (uint32_t)p.OHW;
            const uint32_t oy = fdiv(q, p.div_ow);
            const uint32_t ox = q - oy * (uint32_t)p.OW;
            iy0 = (int)oy * p.stride_h - p.pad_t;
            ix0 = (int)ox * p.stride_w - p.pad_l;
            // may point before the image inside the pad: only ever added to tap offsets that bring it back
            // relative to pad_t rows and pad_l pixels before X, so that it is never negative: it is the bounds-checked
            // part of the address (the tap offset goes into the load's scalar offset, which is not checked)
            xbase = (uint32_t)(((int)n * p.C * p.H * p.Wd + (iy0 + p.pad_t) * p.Wd + ix0 + p.pad_l) * 4);
            tap_outside = 0;
            for (int r = 0; r < p.KH; ++r)
                for (int t = 0; t < p.KW; ++t) {
                    const bool ok = (unsigned)(iy0 + r * p.dil_h) < (unsigned)p.H && (unsigned)(ix0 + t * p.dil_w) < (unsigned)p.Wd;
                    tap_outside |= (ok ? 0u : 1u) << (r * p.KW + t);
                }
        }
    }
    // ... and its k-quads: unit it covers k = 32 kt + 4 kq[it] .. + 3, uniform over the wave
    int kq[B_PER_T], b_lds[B_PER_T];
#pragma unroll
    for (int it = 0; it < B_PER_T; ++it) {
        kq[it] = (tid + it * CG_THREADS) / BN;
        if constexpr (UNIFORM_KQ) kq[it] = __builtin_amdgcn_readfirstlane(kq[it]);
        else kq[it] &= BK / 4 - 1;   // (threads that load nothing stay inside the table)
        b_lds[it] = p_local * PITCH + 4 * kq[it];
        // a narrow slice keeps the step free of branches: the threads without a unit load nothing (every tap counts as
        // outside) and write their zeros to a place of their own behind the three stages
        if (!loader) b_lds[it] = CG_STAGES * STAGE + 4 * tid;
    }
    // compile-time taps: the lane's offsets in the wave's rotation, and the wave's running channel offset
    const uint32_t hw4 = (uint32_t)(p.H * p.Wd) * 4u;
    const uint32_t soff_safe = (uint32_t)(p.C - 2) * hw4;   // for the look-aheads past the last step: inside X with or without the wrap
    uint32_t vtap[B_PER_T][NTAP], soff[B_PER_T];
    if constexpr (STATIC_TAPS) {
#pragma unroll
        for (int it = 0; it < B_PER_T; ++it) {
            const uint32_t a = (uint32_t)(4 * kq[it]) / (uint32_t)TAPS, rot = (uint32_t)(4 * kq[it]) - a * (uint32_t)TAPS;
            soff[it] = a * hw4;
#pragma unroll
            for (int j = 0; j < TAPS; ++j) {
                const uint32_t jj = (uint32_t)j + rot, wrap = jj >= (uint32_t)TAPS ? 1u : 0u, rs = jj - wrap * (uint32_t)TAPS;
                const uint32_t r = fdiv(rs, p.div_kw), t = rs - r * (uint32_t)p.KW;
                const uint32_t outside = (tap_outside >> rs) & 1u;
                vtap[it][j] = (xbase + (r * (uint32_t)(p.dil_h * p.Wd) + t * (uint32_t)p.dil_w) * 4u + wrap * hw4) | (outside << 31);
            }
        }
    }

    f32x4 acc[TN];
#pragma unroll
    for (int j = 0; j < TN; ++j) acc[j] = f32x4{0.f, 0.f, 0.f, 0.f};

    const int ktiles = p.K / BK;  // K % 32 == 0 is a launch precondition
    const int last_tile = ktiles - 1;
    f32x4 ra[RING];            // W operand of tile t in slot t % RING
    f32x4 rb[RING][B_PER_T];   // gathered pixels of tile t in slot t % RING
    f32x4 bf[LEAN ? 1 : 2][TN];   // X operands of tile t in set t % 2 (lean: one set, refilled pair by pair)

    auto load_a = [&](f32x4& dst, int kt) __attribute__((always_inline)) {
        dst = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(w_rsrc, (int)a_off, (kt < last_tile ? kt : last_tile) * (BK * 4), 0));
    };
    auto load_b = [&](f32x4 (&dst)[B_PER_T], int kt, auto i_tag) __attribute__((always_inline)) {
        constexpr int I = decltype(i_tag)::value;   // the step's place in its window (compile-time taps)
        const int k0 = (kt < last_tile ? kt : last_tile) * BK;
        // X as a raw buffer of 2^31 - 1 bytes: an offset with bit 31 set is out of range and loads 0.0f, so a
        // padded tap costs no branch and no select; every other tap lies inside X (which, with its leading
        // pad, is smaller than 2 GiB: checked at launch)
        const int lead = (p.pad_t * p.Wd + p.pad_l) * 4;   // bytes of the (virtual) pad rows and pixels before X
        const __amdgpu_buffer_rsrc_t x_rsrc =
            __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(reinterpret_cast<const char*>(p.X)) - lead, 0, 0x7fffffff, 0x00020000);
        if constexpr (STATIC_TAPS) {
#pragma unroll
            for (int it = 0; it < B_PER_T; ++it) {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    constexpr int S = BK * I, NEXT = BK * (I + 1);
                    const int s_now = S + e, s_next = e < 3 ? S + e + 1 : NEXT;
                    const uint32_t so = kt <= last_tile ? soff[it] : soff_safe;
                    dst[it][e] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(x_rsrc, (int)vtap[it][s_now % NTAP], (int)so, 0));
                    soff[it] += (uint32_t)(s_next / NTAP - s_now / NTAP) * hw4;
                }
            }
            return;
        }
#pragma unroll
        for (int it = 0; it < B_PER_T; ++it) {
            // the four taps of this unit's k-quad: one broadcast read (same address in every lane)
            const u32x4 taps = *reinterpret_cast<const u32x4*>(lds_tap + k0 + 4 * kq[it]);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                // Vector instructions take their time out of the matrix pipe's (measured: 3 to 5 cycles each, whatever
                // the number of waves), so what is the same for the whole wave is computed on the scalar unit: the
                // tap's offset travels as the load's scalar offset, its index selects the lane's pad bit with one
                // bit-field extract, and one shift-or marks the padded lanes out of range.
                if constexpr (UNIFORM_KQ) {
                    const uint32_t tap = (uint32_t)__builtin_amdgcn_readfirstlane((int)taps[e]);
                    const uint32_t outside = __builtin_amdgcn_ubfe(tap_outside, tap >> 27, 1u);
                    dst[it][e] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(x_rsrc, (int)(xbase | (outside << 31)), (int)((tap & 0x07ffffffu) << 2), 0));
                } else {
                    const uint32_t off = xbase + ((taps[e] & 0x07ffffffu) << 2);
                    const uint32_t outside = (tap_outside >> (taps[e] >> 27)) & 1u;
                    dst[it][e] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(x_rsrc, (int)(off | (outside << 31)), 0, 0));
                }
            }
        }
    };
    auto store_b = [&](const f32x4 (&src)[B_PER_T], int stage) __attribute__((always_inline)) {
#pragma unroll
        for (int it = 0; it < B_PER_T; ++it) *reinterpret_cast<f32x4*>(lds + stage * STAGE + b_lds[it]) = src[it];
    };
    auto read_b = [&](f32x4 (&dst)[TN], int stage) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < TN; ++j)
            dst[j] = *reinterpret_cast<const f32x4*>(lds + stage * STAGE + (16 * j + li) * PITCH + 16 * ks + 4 * lq);
    };

    auto tile_step = [&](auto u_tag, int kt) __attribute__((always_inline)) {
        constexpr int r = decltype(u_tag)::value % RING;
        constexpr int cur = LEAN ? 0 : (decltype(u_tag)::value & 1);  // UNROLL is even: tile parity == step parity
        load_b(rb[r], kt + RING, std::integral_constant<int, (decltype(u_tag)::value + RING) % WIN>{});   // slot r went to LDS two steps ago
        load_a(ra[(r + RING - 1) % RING], kt + RING - 1);   // operand consumed in the previous step
        store_b(rb[(r + 2) % RING], (r + 2) % CG_STAGES);   // tile kt + 2
        constexpr int MFMA = 0x008, VMEM_RD = 0x020, DS_RD = 0x100, DS_WR = 0x200;
        if constexpr (LEAN) {
            // Position tiles in two halves. The step starts with the reads of the second half's operands of this tile
            // (they land under the first half's MFMAs); the first half's operands of tile kt + 1, visible since the last
            // barrier, replace this step's once its MFMAs have been issued: no LDS read is outstanding at the barrier.
            constexpr int H = (TN + 1) / 2;
            auto read_half = [&](int from, int to, int stage) __attribute__((always_inline)) {
#pragma unroll
                for (int j = from; j < to; ++j)
                    bf[0][j] = *reinterpret_cast<const f32x4*>(lds + stage * STAGE + (16 * j + li) * PITCH + 16 * ks + 4 * lq);
            };
            auto mfma_half = [&](int from, int to) __attribute__((always_inline)) {
#pragma unroll
                for (int s = 0; s < 4; ++s)
#pragma unroll
                    for (int j = from; j < to; ++j)
                        acc[j] = __builtin_amdgcn_mfma_f32_16x16x4f32(bf[0][j][s], ra[r][s], acc[j], 0, 0, 0);
            };
            read_half(H, TN, r % CG_STAGES);
            mfma_half(0, H);
            read_half(0, H, (r + 1) % CG_STAGES);
            mfma_half(H, TN);
            if constexpr (UNIFORM_KQ && TN == 4) {
                __builtin_amdgcn_sched_group_barrier(DS_RD, 2, 0);
                __builtin_amdgcn_sched_group_barrier(MFMA, 1, 0);
                __builtin_amdgcn_sched_group_barrier(DS_WR, B_PER_T, 0);
                if constexpr (!STATIC_TAPS) __builtin_amdgcn_sched_group_barrier(DS_RD, B_PER_T, 0);  // tap table
#pragma unroll
                for (int v = 0; v < 4 * B_PER_T + 1; ++v) {
                    __builtin_amdgcn_sched_group_barrier(MFMA, 1, 0);
                    __builtin_amdgcn_sched_group_barrier(VMEM_RD, 1, 0);
                }
                __builtin_amdgcn_sched_group_barrier(MFMA, 8 - 1 - (4 * B_PER_T + 1), 0);
                __builtin_amdgcn_sched_group_barrier(DS_RD, 2, 0);
                __builtin_amdgcn_sched_group_barrier(MFMA, 8, 0);
            }
            __syncthreads();
            return;
        }
        read_b(bf[cur ^ 1], (r + 1) % CG_STAGES);           // tile kt + 1, visible since the last barrier
#pragma unroll
        for (int s = 0; s < 4; ++s)
#pragma unroll
            for (int j = 0; j < TN; ++j)
                acc[j] = __builtin_amdgcn_mfma_f32_16x16x4f32(bf[cur][j][s], ra[r][s], acc[j], 0, 0, 0);
        // Issue order: LDS traffic first (it must have completed at the barrier), then the
        // gather loads, each memory instruction between MFMAs so that it never queues
        // behind the other waves' requests while the matrix pipe idles.
        if constexpr (UNIFORM_KQ) {
        __builtin_amdgcn_sched_group_barrier(MFMA, 1, 0);
        __builtin_amdgcn_sched_group_barrier(DS_WR, B_PER_T, 0);
        if constexpr (!STATIC_TAPS) __builtin_amdgcn_sched_group_barrier(DS_RD, B_PER_T, 0);  // tap table
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            __builtin_amdgcn_sched_group_barrier(MFMA, 1, 0);
            __builtin_amdgcn_sched_group_barrier(DS_RD, 1, 0);
        }
#pragma unroll
        for (int v = 0; v < 4 * B_PER_T + 1; ++v) {
            __builtin_amdgcn_sched_group_barrier(MFMA, 2, 0);
            __builtin_amdgcn_sched_group_barrier(VMEM_RD, 1, 0);
        }
        __builtin_amdgcn_sched_group_barrier(MFMA, 4 * TN, 0);
        }
        __syncthreads();
    };
    static_assert(UNROLL % 2 == 0 && RING % CG_STAGES == 0, "step index fixes operand set, slot index the LDS buffer");
    static_assert(!LEAN || 4 * B_PER_T + 2 <= 8, "the lean step's memory instructions fit between the first pair's MFMAs");

#pragma unroll
    for (int r = 0; r < RING; ++r) load_a(ra[r], r);  // tiles beyond the last are clamped: no branch
    __syncthreads();  // tap table complete
    MI355X_TRACE_STAMP(p, 5);
    cg_static_for<RING>([&](auto r_tag) __attribute__((always_inline)) {
        constexpr int r = decltype(r_tag)::value;
        load_b(rb[r], r, std::integral_constant<int, r % WIN>{});
    });
    MI355X_TRACE_STAMP(p, 6);
    store_b(rb[0], 0);
    store_b(rb[1], 1);
    MI355X_TRACE_STAMP(p, 7);
    __syncthreads();
    if constexpr (LEAN) {   // (the second half of tile 0 is read by step 0 itself)
#pragma unroll
        for (int j = 0; j < (TN + 1) / 2; ++j) bf[0][j] = *reinterpret_cast<const f32x4*>(lds + (16 * j + li) * PITCH + 16 * ks + 4 * lq);
    } else {
        read_b(bf[0], 0);
    }

    // One code path for every tile: near the end of K the look-aheads are clamped to the
    // last tile, not switched off, so the step body stays branch-free.
    // Whole groups of RING steps run without a branch inside the loop (with guards in the body the
    // compiler's wait-count analysis drains every outstanding load at the loop header); the at most
    // RING - 1 remaining steps follow, guarded.
    MI355X_TRACE_STAMP(p, 1);
    MI355X_TRACE_CYCLES(p, 12);
    int kt0 = 0;
    for (; kt0 + UNROLL <= ktiles; kt0 += UNROLL) {
        cg_static_for<UNROLL>([&](auto u_tag) __attribute__((always_inline)) { tile_step(u_tag, kt0 + decltype(u_tag)::value); });
    }
    cg_static_for<UNROLL>([&](auto u_tag) __attribute__((always_inline)) {
        const int kt = kt0 + decltype(u_tag)::value;
        if (kt < ktiles) tile_step(u_tag, kt);  // uniform
    });

    MI355X_TRACE_STAMP(p, 2);
    MI355X_TRACE_CYCLES(p, 13);
    // k-split group 1 hands its partial sums to group 0 through LDS
    {
        f32x4* red = reinterpret_cast<f32x4*>(lds);
        if (ks == 1) {
#pragma unroll
            for (int j = 0; j < TN; ++j) red[(wm * TN + j) * WAVE + lane] = acc[j];
        }
        __syncthreads();
        MI355X_TRACE_STAMP(p, 8);
        if (ks == 1) return;
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[j] += red[(wm * TN + j) * WAVE + lane];
    }
    MI355X_TRACE_STAMP(p, 9);

    // epilogue: acc[j][r] = Y[oc = m0 + 16 wm + li][p = p0 + 16 j + 4 lq + r]
    const int64_t oc = m0 + 16 * wm + li;
    if (oc >= p.M) return;
    const float bv = (p.epi & MI355X_EPI_BIAS) ? p.bias[oc] : 0.f;
#ifdef MI355X_WG_TRACE
    asm volatile("" :: "v"(bv));
    MI355X_TRACE_STAMP(p, 10);
#endif
#pragma unroll
    for (int j = 0; j < TN; ++j) {
        const int64_t pp = p0 + 16 * j + 4 * lq;
        if (pp >= p.P) continue;
        f32x4 v = acc[j];
        v.x = apply_epilogue(v.x, p.epi, bv);
        v.y = apply_epilogue(v.y, p.epi, bv);
        v.z = apply_epilogue(v.z, p.epi, bv);
        v.w = apply_epilogue(v.w, p.epi, bv);
        if (p.vec_y) {
            const uint32_t n = fdiv((uint32_t)pp, p.div_ohw);
            const uint32_t q = (uint32_t)pp - n * (uint32_t)p.OHW;
            const int64_t off = ((int64_t)n * p.M + oc) * p.OHW + q;
            __builtin_nontemporal_store(conv_epilogue_tail4(v, p.epi, p.residual, off), reinterpret_cast<f32x4*>(p.Y + off));
        } else {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                if (pp + r >= p.P) break;
                const uint32_t n = fdiv((uint32_t)(pp + r), p.div_ohw);
                const uint32_t q = (uint32_t)(pp + r) - n * (uint32_t)p.OHW;
                const int64_t off = ((int64_t)n * p.M + oc) * p.OHW + q;
                p.Y[off] = conv_epilogue_tail1(v[r], p.epi, p.residual, off);
            }
        }
    }
    MI355X_TRACE_STAMP(p, 3);
}

// TN: the whole tiles; workgroups past p.full_tiles take 16-position slices (TN = 1)
template <int TN, int TAPS, bool LEAN = false>
__global__ __launch_bounds__(CG_THREADS, LEAN ? 3 : 1) void conv2d_f32_gather_kernel(ConvArgs p) {
    __shared__ __attribute__((aligned(16))) float lds[cg_lds_floats(TN)];
    // tap table: for every k = (c, r, s) the element offset of that tap relative to a
    // position's top-left input pixel (low 27 bits) and the tap index r * KW + s (high 5 bits)
    __shared__ __attribute__((aligned(16))) uint32_t lds_tap[CG_MAX_K];
    if ((int64_t)blockIdx.x < p.full_tiles) {
        const int64_t logical = xcd_remap(blockIdx.x, p.full_tiles);
        int64_t tm, tn;
        tile_coords(logical, p.tiles_m, p.tiles_p, p.group_m, tm, tn);
        conv2d_f32_gather_tile<TN, TAPS, LEAN>(p, tm * CG_BM, tn * (16 * TN), lds, lds_tap);
    } else {
        const uint32_t q = blockIdx.x - (uint32_t)p.full_tiles, tiles_m = (uint32_t)p.tiles_m;
        conv2d_f32_gather_tile<1, 0, LEAN>(p, (int64_t)(q % tiles_m) * CG_BM, p.p_full + 16 * (int64_t)(q / tiles_m), lds, lds_tap);
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

static int choose_conv_tile(int64_t M, int64_t P, int cus, int force) {
    if (force >= 0 && force < kNumConvTiles) return force;
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
    MI355X_REQUIRE((epilogue & ~(MI355X_EPI_BIAS | MI355X_EPI_RELU)) == 0,
                   "conv2d: epilogue 0x%x not supported (bias and relu only)", epilogue);
    return mi355x_conv2d_res_f32(X, W, bias, nullptr, Y, N, C, H, Wd, M, KH, KW, pads, strides, dilations, epilogue, stream);
}

extern "C" int mi355x_conv2d_res_f32(const float* X, const float* W, const float* bias, const float* residual,
                                     float* Y, int64_t N, int64_t C, int64_t H, int64_t Wd, int64_t M,
                                     int64_t KH, int64_t KW, const int64_t* pads,
                                     const int64_t* strides, const int64_t* dilations, int epilogue,
                                     void* stream) {
    using namespace mi355x;
    MI355X_REQUIRE(N >= 0 && C >= 0 && H >= 0 && Wd >= 0 && M >= 0 && KH >= 1 && KW >= 1,
                   "conv2d: bad extents N=%lld C=%lld H=%lld W=%lld M=%lld KH=%lld KW=%lld",
                   (long long)N, (long long)C, (long long)H, (long long)Wd, (long long)M,
                   (long long)KH, (long long)KW);
    MI355X_REQUIRE(pads && strides && dilations, "conv2d: null pads/strides/dilations");
    MI355X_REQUIRE((epilogue & ~(MI355X_EPI_BIAS | MI355X_EPI_RELU | MI355X_EPI_RESIDUAL | MI355X_EPI_RELU_AFTER)) == 0,
                   "conv2d: epilogue 0x%x not supported (bias, relu, residual, relu after the residual)", epilogue);
    MI355X_REQUIRE(!(epilogue & MI355X_EPI_BIAS) || bias, "conv2d: MI355X_EPI_BIAS without bias");
    MI355X_REQUIRE(!(epilogue & MI355X_EPI_RESIDUAL) || residual, "conv2d: MI355X_EPI_RESIDUAL without residual");
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
    MI355X_TRACE_INIT(p);
    p.X = X; p.W = W; p.bias = bias; p.Y = Y; p.residual = residual;
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
    p.vec_y = ((OH * OW) % 4 == 0) && al16(Y) && (!(epilogue & MI355X_EPI_RESIDUAL) || al16(residual));

    const int cus = device_cus();
    if (cus <= 0) return set_error(MI355X_ERR_NOT_INITIALIZED, "conv2d: no usable HIP device");
    const Tuning tune = tuning();
    hipStream_t st = static_cast<hipStream_t>(stream);
    p.group_m = 1;
    // K a multiple of the 32-k tile and 16-byte aligned W rows: the gather kernel
    if (K % CG_BK == 0 && K <= CG_MAX_K && KH * KW <= 32 && M * K < ((int64_t)1 << 29) && C * H * Wd < ((int64_t)1 << 27) &&
        N * C * H * Wd + pads[0] * Wd + pads[1] + H * Wd < ((int64_t)1 << 29) && al16(W) && tune.conv_config < 0) {
        p.x_bytes = (int)(N * C * H * Wd * 4);
        // 64 x 64 tiles (three workgroups share a CU) or 64 x 128 (one per CU). Time goes with the tiles a CU has
        // to run times their width; the wide tile, alone on its CU, pays its first loads and last stores in the open
        // (32 x 64 x 56 x 56 -> 64: 101.5 us as 784 wide tiles, 73.2 us as 1568 narrow ones two to a CU), hence its factor.
        auto cost = [&](int bn, double factor) {
            const int64_t tiles = ceil_div(M, (int64_t)CG_BM) * ceil_div(P, (int64_t)bn);
            return (double)ceil_div(tiles, (int64_t)cus) * bn * factor;
        };
        // The narrow tile runs as the lean kernel, three workgroups per CU (MI355X_CONV_PER_CU=2: the six-deep ring, two
        // per CU): 32 x 64 x 56 x 56 -> 64, 3 x 3, takes 67.4 against 73.2 us, 16 x 256 x 28 x 28 -> 256 129.5 against
        // 141.6 us, 16 x 64 x 28 x 28 -> 256 37.9 against 45.3 us, 1 x 1 over 32 x 64 x 56 x 56 -> 256 62.9 against 83.6 us;
        // bit-equal results (each accumulator sees the same MFMAs in the same order).
        const int per_cu = tune.conv_per_cu == 2 ? 2 : 3;
        const bool wide = tune.conv_gather_bn ? tune.conv_gather_bn == 128 : cost(128, 1.3) < cost(64, 1.0);
        const int bn = wide ? 128 : 64;
        p.tiles_m = ceil_div(M, (int64_t)CG_BM);
        p.tiles_p = ceil_div(P, (int64_t)bn);
        p.full_tiles = p.tiles_m * p.tiles_p;
        p.p_full = p.tiles_p * bn;
        int64_t slices = 0;
        // Narrow tiles in more than one round of workgroups, the last round less than half full (configuration 4:
        // 1568 tiles on 768 places): the tiles of that round run as 16-position slices, four times as many
        // workgroups of a quarter of the work each, so the places that would idle through a whole tile time
        // share its work.
        const bool lean = !wide && per_cu == 3;
        if (!wide && tune.conv_tail != 0) {
            const int64_t places = (int64_t)cus * (lean ? 3 : 2), rem = p.full_tiles % places;
            const int64_t tail_p = tune.conv_tail > 0 ? tune.conv_tail : rem / p.tiles_m;
            const bool wanted = tune.conv_tail > 0 || (p.full_tiles > places && rem > 0 && rem < places / 2);
            if (wanted && tail_p > 0 && tail_p < p.tiles_p) {
                p.tiles_p -= tail_p;
                p.full_tiles = p.tiles_m * p.tiles_p;
                p.p_full = p.tiles_p * bn;
                slices = p.tiles_m * ceil_div(P - p.p_full, (int64_t)16);
            }
        }
        p.nwg = p.full_tiles + slices;
        MI355X_REQUIRE(p.nwg < ((int64_t)1 << 31), "conv2d: grid too large");
        // 3 x 3 and 1 x 1 filters over whole windows of 32 channels: taps known at compile time
        const int taps = (C % 32 == 0 && (KH * KW == 9 || KH * KW == 1) && tune.conv_static_taps) ? (int)(KH * KW) : 0;
        const dim3 g((unsigned)p.nwg), b(CG_THREADS);
        if (wide) {
            if (taps == 9) hipLaunchKernelGGL((conv2d_f32_gather_kernel<8, 9>), g, b, 0, st, p);
            else if (taps == 1) hipLaunchKernelGGL((conv2d_f32_gather_kernel<8, 1>), g, b, 0, st, p);
            else hipLaunchKernelGGL((conv2d_f32_gather_kernel<8, 0>), g, b, 0, st, p);
        } else if (lean) {
            if (taps == 9) hipLaunchKernelGGL((conv2d_f32_gather_kernel<4, 9, true>), g, b, 0, st, p);
            else if (taps == 1) hipLaunchKernelGGL((conv2d_f32_gather_kernel<4, 1, true>), g, b, 0, st, p);
            else hipLaunchKernelGGL((conv2d_f32_gather_kernel<4, 0, true>), g, b, 0, st, p);
        } else {
            if (taps == 9) hipLaunchKernelGGL((conv2d_f32_gather_kernel<4, 9>), g, b, 0, st, p);
            else if (taps == 1) hipLaunchKernelGGL((conv2d_f32_gather_kernel<4, 1>), g, b, 0, st, p);
            else hipLaunchKernelGGL((conv2d_f32_gather_kernel<4, 0>), g, b, 0, st, p);
        }
        return check_launch("conv2d_f32_gather_kernel");
    }
    const int cfg = choose_conv_tile(M, P, cus, tune.conv_config);
    p.tiles_m = ceil_div(M, kConvTiles[cfg].bm);
    p.tiles_p = ceil_div(P, kConvTiles[cfg].bn);
    p.nwg = p.tiles_m * p.tiles_p;
    MI355X_REQUIRE(p.nwg < ((int64_t)1 << 31), "conv2d: grid too large");
    switch (cfg) {
        case 0: launch_conv<64, 128, 16, 2, 2>(p, st); break;
        case 1: launch_conv<64, 64, 32, 2, 2>(p, st); break;
        case 2: launch_conv<32, 64, 32, 2, 2>(p, st); break;
        case 3: launch_conv<16, 64, 32, 1, 4>(p, st); break;
        default: launch_conv<128, 64, 32, 2, 2>(p, st); break;
    }
    return check_launch("conv2d_f32_kernel");
}
