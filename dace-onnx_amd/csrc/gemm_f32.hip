// ONNX MatMul / Gemm, fp32, on the gfx950 matrix cores.
//
// Replaces PureMatMul -> PureEinsum -> DaCe BLAS node and PureGemm
// (daceml/onnx/op_implementations/pure_implementations.py:130-267,433-459).
//
// Design
//   * v_mfma_f32_16x16x4_f32: 64 FLOP/clk/SIMD, the fp32 matrix rate of the part.
//     The two MFMA operands are swapped (a-operand = B fragment, b-operand =
//     A fragment) so a lane's four accumulator registers are four consecutive
//     n of one output row: the epilogue is one 16-byte store per lane per tile
//     and bias / residual are 16-byte loads.
//   * A workgroup (4 waves) owns a BM x BN tile of C; the K loop stages
//     BM x BK and BK x BN through LDS, double buffered, global loads for tile
//     t+1 in flight while tile t is multiplied, one barrier per tile.
//   * LDS rows are padded by 4 floats: 16-byte fragment reads along k
//     (operands stored k-contiguous) and 4-byte reads along m/n (operands
//     stored m/n-contiguous) are both bank-conflict free. One 16-byte read along
//     k feeds four MFMA steps: lane (i, q) holds k = 4q..4q+3 of a 16-k chunk
//     for BOTH operands, so any k order is consistent.
//   * Operand layout is a template choice, not a copy: A or B may be
//     contiguous along k or along m/n (Gemm's transB=1, K^T in attention), and
//     two batch levels with arbitrary strides express a head split/merge.
//   * Workgroups are renumbered so that each XCD (own L2) gets a contiguous
//     range of tiles instead of every eighth tile.
#include "common.h"
#include "gemm_tile.h"
#include "gemm_args.h"

#include <stdlib.h>

namespace mi355x {

template <int BM, int BN, int BK, int WAVES_M, int WAVES_N, bool A_KC, bool B_KC, bool VEC>
__global__ __launch_bounds__(64 * WAVES_M * WAVES_N) void gemm_f32_kernel(GemmArgs p) {
    constexpr int NT = 64 * WAVES_M * WAVES_N;
    constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
    constexpr int TM = WM / 16, TN = WN / 16;
    static_assert(WM % 16 == 0 && WN % 16 == 0 && BK % 16 == 0, "tile shape");
    // LDS tiles: k-contiguous operands as [rows][BK+4], others as [BK][rows+4]
    using AIO = TileIO<(A_KC ? BM : BK), (A_KC ? BK : BM), VEC, NT>;
    using BIO = TileIO<(B_KC ? BN : BK), (B_KC ? BK : BN), VEC, NT>;
    constexpr int A_ROWS = A_KC ? BM : BK, B_ROWS = B_KC ? BN : BK;
    constexpr int A_TILE = A_ROWS * AIO::PITCH, B_TILE = B_ROWS * BIO::PITCH;
    __shared__ __attribute__((aligned(16))) float lds_a[2][A_TILE];
    __shared__ __attribute__((aligned(16))) float lds_b[2][B_TILE];

    const int tid = threadIdx.x;
    const int lane = tid % WAVE, wave = tid / WAVE;
    const int li = lane % 16, lq = lane / 16;
    const int wm0 = (wave / WAVES_N) * WM, wn0 = (wave % WAVES_N) * WN;

    const int64_t logical = xcd_remap(blockIdx.x, p.nwg);
    const int64_t tiles_per_batch = p.tiles_m * p.tiles_n;
    const int64_t b = logical / tiles_per_batch, t = logical % tiles_per_batch;
    const int64_t b0 = b / p.batch1, b1 = b % p.batch1;
    int64_t tm, tn;
    tile_coords(t, p.tiles_m, p.tiles_n, p.group_m, tm, tn);
    const int64_t m0 = tm * BM, n0 = tn * BN;

    const float* __restrict__ A = p.A + b0 * p.a_sb0 + b1 * p.a_sb1;
    const float* __restrict__ B = p.B + b0 * p.b_sb0 + b1 * p.b_sb1;

    f32x4 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

    f32x4 ra[AIO::PER_T], rb[BIO::PER_T];
    auto load_tiles = [&](int64_t k0) {
        if constexpr (A_KC) AIO::load(ra, A, m0, k0, p.M, p.K, p.a_sm, p.a_sk, tid);
        else AIO::load(ra, A, k0, m0, p.K, p.M, p.a_sk, p.a_sm, tid);
        if constexpr (B_KC) BIO::load(rb, B, n0, k0, p.N, p.K, p.b_sn, p.b_sk, tid);
        else BIO::load(rb, B, k0, n0, p.K, p.N, p.b_sk, p.b_sn, tid);
    };

    const int64_t ktiles = (p.K + BK - 1) / BK;
    load_tiles(0);
    AIO::store(ra, lds_a[0], tid);
    BIO::store(rb, lds_b[0], tid);
    __syncthreads();

    for (int64_t kt = 0; kt < ktiles; ++kt) {
        const int buf = (int)(kt & 1);
        if (kt + 1 < ktiles) load_tiles((kt + 1) * BK);
        const float* __restrict__ la = lds_a[buf];
        const float* __restrict__ lb = lds_b[buf];
        mma_ktile<TM, TN, BK, A_KC, B_KC, AIO::PITCH, BIO::PITCH>(la, lb, wm0, wn0, li, lq, acc);
        if (kt + 1 < ktiles) {
            AIO::store(ra, lds_a[buf ^ 1], tid);
            BIO::store(rb, lds_b[buf ^ 1], tid);
        }
        __syncthreads();
    }

    // Epilogue. acc[i][j][r] = C[m0+wm0+16i+li][n0+wn0+16j+4*lq+r].
    float* C = p.C + b0 * p.c_sb0 + b1 * p.c_sb1;
    const float* R = (p.epi & MI355X_EPI_RESIDUAL)
                                      ? p.residual + b0 * p.r_sb0 + b1 * p.r_sb1 : nullptr;
#pragma unroll
    for (int i = 0; i < TM; ++i) {
        const int64_t m = m0 + wm0 + i * 16 + li;
        if (m >= p.M) continue;
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int64_t n = n0 + wn0 + j * 16 + 4 * lq;
            if (n >= p.N) continue;
            f32x4 v = acc[i][j] * p.alpha;
            if constexpr (VEC) {
                f32x4 bv = f32x4{0.f, 0.f, 0.f, 0.f};
                if (p.epi & MI355X_EPI_BIAS) bv = *reinterpret_cast<const f32x4*>(p.bias + n);
                v.x = apply_epilogue(v.x, p.epi, bv.x);
                v.y = apply_epilogue(v.y, p.epi, bv.y);
                v.z = apply_epilogue(v.z, p.epi, bv.z);
                v.w = apply_epilogue(v.w, p.epi, bv.w);
                if (R) v += *reinterpret_cast<const f32x4*>(R + m * p.r_sm + n);
                *reinterpret_cast<f32x4*>(C + m * p.c_sm + n) = v;
            } else {
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    if (n + r >= p.N) break;
                    float o = apply_epilogue(v[r], p.epi, (p.epi & MI355X_EPI_BIAS) ? p.bias[n + r] : 0.f);
                    if (R) o += R[m * p.r_sm + n + r];
                    C[m * p.c_sm + n + r] = o;
                }
            }
        }
    }
}

// ---- host side ----------------------------------------------------------------

struct TileConfig { int bm, bn, bk; };
// index order must match the switch in launch_config()
static const TileConfig kConfigs[] = {
    {128, 128, 16},  // 0: large problems, highest reuse
    {64, 64, 32},    // 1
    {64, 48, 32},    // 2: N multiple of 48 (768, 2304, 3072) with few tiles
    {32, 64, 32},    // 3: small batched products
    {128, 64, 32},   // 4
};
constexpr int kNumConfigs = sizeof(kConfigs) / sizeof(kConfigs[0]);

template <int BM, int BN, int BK, int WMs, int WNs>
static void launch_layout(const GemmArgs& p, bool a_kc, bool b_kc, bool vec, hipStream_t st) {
    const dim3 grid((unsigned)p.nwg), block(64 * WMs * WNs);
#define MI355X_GEMM_CASE(AK, BKC, V)                                                             \
    hipLaunchKernelGGL((gemm_f32_kernel<BM, BN, BK, WMs, WNs, AK, BKC, V>), grid, block, 0, st, p)
    if (vec) {
        if (a_kc && !b_kc) MI355X_GEMM_CASE(true, false, true);
        else if (a_kc && b_kc) MI355X_GEMM_CASE(true, true, true);
        else if (!a_kc && !b_kc) MI355X_GEMM_CASE(false, false, true);
        else MI355X_GEMM_CASE(false, true, true);
    } else {
        if (a_kc && !b_kc) MI355X_GEMM_CASE(true, false, false);
        else if (a_kc && b_kc) MI355X_GEMM_CASE(true, true, false);
        else if (!a_kc && !b_kc) MI355X_GEMM_CASE(false, false, false);
        else MI355X_GEMM_CASE(false, true, false);
    }
#undef MI355X_GEMM_CASE
}

static void launch_config(int cfg, const GemmArgs& p, bool a_kc, bool b_kc, bool vec, hipStream_t st) {
    switch (cfg) {
        case 0: launch_layout<128, 128, 16, 2, 2>(p, a_kc, b_kc, vec, st); break;
        case 1: launch_layout<64, 64, 32, 2, 2>(p, a_kc, b_kc, vec, st); break;
        case 2: launch_layout<64, 48, 32, 4, 1>(p, a_kc, b_kc, vec, st); break;
        case 3: launch_layout<32, 64, 32, 2, 2>(p, a_kc, b_kc, vec, st); break;
        default: launch_layout<128, 64, 32, 2, 2>(p, a_kc, b_kc, vec, st); break;
    }
}

// Cost model: time ~ rounds of workgroups over the CUs x work per tile,
// inflated for small tiles (more LDS/L2 traffic per FLOP) and padding waste.
static int choose_config(int64_t batch, int64_t M, int64_t N, int64_t K, int cus) {
    const int force = tuning().gemm_config;
    if (force >= 0 && force < kNumConfigs) return force;
    double best = 1e300;
    int best_cfg = 1;
    for (int c = 0; c < kNumConfigs; ++c) {
        const TileConfig& t = kConfigs[c];
        const int64_t nwg = batch * ceil_div(M, t.bm) * ceil_div(N, t.bn);
        const int64_t slots = (int64_t)cus * 2;  // two resident workgroups per CU
        const double rounds = (double)ceil_div(nwg, slots);
        const double tile_flops = (double)t.bm * t.bn * (double)K;
        // bytes staged per FLOP fall with tile size; small tiles run below MFMA rate
        const double reuse_penalty = 1.0 + 24.0 * (1.0 / t.bm + 1.0 / t.bn);
        const double cost = rounds * tile_flops * reuse_penalty;
        if (cost < best) { best = cost; best_cfg = c; }
    }
    return best_cfg;
}

}  // namespace mi355x

extern "C" int mi355x_gemm_f32(const float* A, const float* B, float* C, const float* bias,
                               const float* residual, int64_t batch0, int64_t batch1, int64_t M,
                               int64_t N, int64_t K, const int64_t* a_strides,
                               const int64_t* b_strides, const int64_t* c_strides,
                               const int64_t* r_strides, float alpha, int epilogue, void* stream) {
    using namespace mi355x;
    MI355X_REQUIRE(batch0 >= 0 && batch1 >= 0 && M >= 0 && N >= 0 && K >= 0,
                   "gemm: negative extent (batch=%lldx%lld M=%lld N=%lld K=%lld)", (long long)batch0,
                   (long long)batch1, (long long)M, (long long)N, (long long)K);
    MI355X_REQUIRE(a_strides && b_strides && c_strides, "gemm: null stride array");
    MI355X_REQUIRE((epilogue & ~(MI355X_EPI_BIAS | MI355X_EPI_RELU | MI355X_EPI_GELU | MI355X_EPI_RESIDUAL)) == 0,
                   "gemm: unknown epilogue bits 0x%x", epilogue);
    MI355X_REQUIRE(!(epilogue & MI355X_EPI_BIAS) || bias, "gemm: MI355X_EPI_BIAS without bias");
    MI355X_REQUIRE(!(epilogue & MI355X_EPI_RESIDUAL) || (residual && r_strides),
                   "gemm: MI355X_EPI_RESIDUAL without residual / r_strides");
    const int64_t batch = batch0 * batch1;
    if (batch == 0 || M == 0 || N == 0) return MI355X_OK;
    MI355X_REQUIRE(C && (K == 0 || (A && B)), "gemm: null pointer");
    MI355X_REQUIRE(c_strides[2] >= N || M == 1, "gemm: C row stride %lld < N %lld", (long long)c_strides[2], (long long)N);

    GemmArgs p;
    MI355X_TRACE_INIT(p);
    p.A = A; p.B = B; p.C = C; p.bias = bias; p.residual = residual;
    p.batch = batch; p.batch1 = batch1; p.M = M; p.N = N; p.K = K;
    p.a_sb0 = a_strides[0]; p.a_sb1 = a_strides[1]; p.a_sm = a_strides[2]; p.a_sk = a_strides[3];
    p.b_sb0 = b_strides[0]; p.b_sb1 = b_strides[1]; p.b_sk = b_strides[2]; p.b_sn = b_strides[3];
    p.c_sb0 = c_strides[0]; p.c_sb1 = c_strides[1]; p.c_sm = c_strides[2];
    p.r_sb0 = r_strides ? r_strides[0] : 0; p.r_sb1 = r_strides ? r_strides[1] : 0;
    p.r_sm = r_strides ? r_strides[2] : 0;
    p.alpha = alpha; p.epi = epilogue;

    // operand layout: which direction do adjacent lanes walk when loading
    const bool a_kc = (p.a_sk == 1) || (p.a_sm != 1 && p.a_sk <= p.a_sm);
    const bool b_kc = (p.b_sk == 1 && p.b_sn != 1) || (p.b_sn != 1 && p.b_sk < p.b_sn);
    auto al16 = [](const void* q) { return (reinterpret_cast<uintptr_t>(q) & 15) == 0; };
    auto m4 = [](int64_t v) { return (v & 3) == 0; };
    bool vec = al16(A) && al16(B) && al16(C) && m4(N) && m4(p.c_sm) && m4(p.c_sb0) && m4(p.c_sb1) &&
               m4(p.a_sb0) && m4(p.a_sb1) && m4(p.b_sb0) && m4(p.b_sb1);
    vec = vec && (a_kc ? (p.a_sk == 1 && m4(K) && m4(p.a_sm)) : (p.a_sm == 1 && m4(M) && m4(p.a_sk)));
    vec = vec && (b_kc ? (p.b_sk == 1 && m4(K) && m4(p.b_sn)) : (p.b_sn == 1 && m4(N) && m4(p.b_sk)));
    if (epilogue & MI355X_EPI_BIAS) vec = vec && al16(bias);
    if (epilogue & MI355X_EPI_RESIDUAL)
        vec = vec && al16(residual) && m4(p.r_sm) && m4(p.r_sb0) && m4(p.r_sb1);

    const int cus = device_cus();
    if (cus <= 0) return set_error(MI355X_ERR_NOT_INITIALIZED, "gemm: no usable HIP device");
    // both operands contiguous along k (activations x pre-transposed weights, Q K^T):
    // the dedicated kernel reads every MFMA fragment with 16-byte accesses
    // (not for stacks of small products over a short K -- the scores of an attention head, 96 x (128 x 128 x 64): the
    // kernel's register ring is longer than their K, and 32 x 64 tiles of four waves fill the part better: 7.4 against
    // 9.1 us, 128 x 128 x 128 9.9 against 11.0 us, 128 x 128 x 32 6.1 against 8.2 us)
    const Tuning tune = tuning();
    const bool small_stack = batch > 1 && M <= 128 && N <= 128 && K <= 128 &&   // (a forced variant of that kernel is taken all the same)
                             tune.gemm_nt_bn == 0 && tune.gemm_nt_per_cu == 0 && tune.gemm_nt_bk == 0 && tune.gemm_nt_waves == 0 && tune.gemm_ksplit != 1;
    if (a_kc && b_kc && vec && tune.gemm_config < 0 && !small_stack) {
        // MI355X_GEMM_KSPLIT: 1 sends every such product to the kernel whose waves split K, 0 none
        if (tune.gemm_ksplit == 1 && launch_gemm_f32_ksplit(p, cus, static_cast<hipStream_t>(stream)))
            return check_launch("gemm_f32_ksplit_kernel");
        if (launch_gemm_f32_nt(p, cus, static_cast<hipStream_t>(stream))) return check_launch("gemm_f32_nt_kernel");
    }
    const int cfg = choose_config(batch, M, N, K, cus);
    const TileConfig& tc = kConfigs[cfg];
    p.tiles_m = ceil_div(M, tc.bm);
    p.tiles_n = ceil_div(N, tc.bn);
    p.nwg = batch * p.tiles_m * p.tiles_n;
    MI355X_REQUIRE(p.nwg < ((int64_t)1 << 31), "gemm: grid too large (%lld workgroups)", (long long)p.nwg);
    {   // about two workgroups of these tiles share a CU
        const int64_t per_xcd = ceil_div(p.nwg, (int64_t)NUM_XCD), resident = 2 * (cus / NUM_XCD);
        const int64_t per_batch = p.tiles_m * p.tiles_n;   // tiles are numbered batch entry by batch entry
        p.group_m = choose_group_m(p.tiles_m, per_xcd < per_batch ? per_xcd : per_batch, resident, tc.bm, tc.bn, K * 4);
    }
    launch_config(cfg, p, a_kc, b_kc, vec, static_cast<hipStream_t>(stream));
    return check_launch("gemm_f32_kernel");
}
