// fp32 GEMM for operands that are both contiguous along k ("NT"): activations
// times pre-transposed weights (PyTorch Linear / ONNX Gemm transB=1 layout) and
// Q K^T in attention.
//
// Why a separate kernel: on this part a wave's LDS instructions are expensive in
// latency (a 16-byte read occupies a wave's LDS queue for ~55 cycles, a 4-byte read
// ~40, a 16-byte write ~165), so the kernel that keeps the matrix pipe busy is
// the one with the fewest LDS instructions per MFMA:
//   * every MFMA fragment is a 16-byte read: with both operands k-contiguous a
//     lane's four k-values of a 16-k chunk are adjacent for A and for B;
//   * A never goes through LDS. The four wave rows of a workgroup own disjoint
//     16-row slices of the 64-row tile, so nobody shares an A fragment: each lane
//     loads its own 16 bytes straight from global memory / L2 into the register
//     the MFMA reads, RING tiles ahead;
//   * B (16*TN columns x 32 k) is staged once per workgroup: global -> register
//     ring -> LDS (three buffers, rows padded by 4 floats), one 16-byte write per
//     thread per tile;
//   * 8 waves = 4 wave rows x 2 k-split groups; group g multiplies the g-th 16-k
//     chunk of every 32-k tile, the two partial sums meet in LDS at the end. Every
//     SIMD holds two waves even when the problem has only 256 tiles
//     (1024 x 768 = 16 x 16 tiles of 64 x 48);
//   * fragments of tile t + 1 are read while tile t is multiplied (they are
//     visible since the barrier of tile t - 1); one barrier per tile.
// MFMA operands are swapped as in gemm_f32.hip: a lane's accumulator registers
// are four consecutive n of one row, stored as 16 bytes.
#include <algorithm>
#include "common.h"
#include "gemm_tile.h"
#include "gemm_args.h"

#include <stdlib.h>
#include <type_traits>
#include <utility>

namespace mi355x {

template <int N, class F, int... I>
__device__ __forceinline__ void nt_static_for_impl(F&& f, std::integer_sequence<int, I...>) {
    (f(std::integral_constant<int, I>{}), ...);
}
// f(integral_constant<0>) ... f(integral_constant<N-1>): indices usable for register arrays
template <int N, class F>
__device__ __forceinline__ void nt_static_for(F&& f) {
    nt_static_for_impl<N>(static_cast<F&&>(f), std::make_integer_sequence<int, N>{});
}

constexpr int NT_BK = 32, NT_THREADS = 512, NT_RING = 6, NT_STAGES = 3;

// TN: 16-column MFMA tiles per wave (BN = 16 TN). WAVES_M wave rows of 16 rows each
// (BM = 16 WAVES_M) times KSPLIT k-split groups make the 8 waves of a workgroup:
// (4, 2) for problems with few tiles, (8, 1) for 128-row tiles without a reduction.
// BK: k extent of a tile (32, or 64 where registers allow: half as many barriers per FLOP); RING: k-tiles in
// flight per lane (six of 32 k or three of 64 k: the same bytes).
template <int TN, int WAVES_M, int KSPLIT, int BK = NT_BK, int RING = NT_RING, int PER_CU = 1>
__global__ __launch_bounds__(WAVES_M * KSPLIT * WAVE, PER_CU) void gemm_f32_nt_kernel(GemmArgs p) {
    constexpr int THREADS = WAVES_M * KSPLIT * WAVE;   // 8 waves, or 16 (4 wave rows x 4 k-split groups)
    static_assert(THREADS == NT_THREADS || THREADS == 2 * NT_THREADS, "8 or 16 waves per workgroup");
    static_assert(RING % NT_STAGES == 0, "a tile's LDS buffer is its ring slot modulo the number of buffers");
    constexpr int BM = 16 * WAVES_M, BN = 16 * TN, NT_PITCH = BK + LDS_PAD;
    constexpr int NC = (BK / 16) / KSPLIT;  // 16-k chunks of a tile this wave multiplies
    constexpr int B_VECS = BN * (BK / 4);                       // 16-byte vectors of one B tile
    constexpr int B_PER_T = (B_VECS + THREADS - 1) / THREADS;
    constexpr int B_ROWS = B_PER_T * THREADS / (BK / 4);     // rows incl. the ones only written as padding
    constexpr int STAGE = B_ROWS * NT_PITCH;                    // floats per LDS buffer
    constexpr int RED = (KSPLIT - 1) * BM * BN;                 // partial sums of the k-split groups after the first
    constexpr int LDS_FLOATS = NT_STAGES * STAGE > RED ? NT_STAGES * STAGE : RED;
    __shared__ __attribute__((aligned(16))) float lds[LDS_FLOATS];

    const int tid = threadIdx.x;
    const int lane = tid % WAVE, wave = tid / WAVE;
    const int li = lane % 16, lq = lane / 16;
    const int wm = wave % WAVES_M, ks = wave / WAVES_M;   // wave row, k-split group
    MI355X_TRACE_STAMP(p, 0);
    MI355X_TRACE_HWID(p);

    const int64_t logical = xcd_remap(blockIdx.x, p.nwg);
    const uint32_t tiles_per_batch = (uint32_t)(p.tiles_m * p.tiles_n);
    const uint32_t b = (uint32_t)logical / tiles_per_batch, t = (uint32_t)logical % tiles_per_batch;
    const int64_t b0 = b / (uint32_t)p.batch1, b1 = b % (uint32_t)p.batch1;
    int64_t tm, tn;
    tile_coords(t, p.tiles_m, p.tiles_n, p.group_m, tm, tn);
    const int64_t m0 = tm * BM, n0 = tn * BN;

    // this lane's A fragment source: row m (clamped into the matrix), 4 floats at
    // k = 32*kt + 16*(c*KSPLIT + ks) + 4*lq for its chunks c
    int64_t am = m0 + 16 * wm + li;
    am = am < p.M ? am : p.M - 1;
    // Operands are read as raw buffers: the batch's matrix as the (scalar) base, the lane's row and column as a
    // 32-bit byte offset, the k-tile as the scalar offset. Next to a stream of MFMAs a load with a 64-bit address
    // per lane holds up the address path for about 12 cycles, one of this form for 3 or fewer, and the offset
    // arithmetic per tile leaves the vector unit (launch precondition: a matrix spans less than 2^31 bytes).
    const __amdgpu_buffer_rsrc_t a_rsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(p.A + b0 * p.a_sb0 + b1 * p.a_sb1), 0, 0x7fffffff, 0x00020000);
    const __amdgpu_buffer_rsrc_t b_rsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(p.B + b0 * p.b_sb0 + b1 * p.b_sb1), 0, 0x7fffffff, 0x00020000);
    const uint32_t a_off = (uint32_t)(am * p.a_sm + 16 * ks + 4 * lq) * 4u;
    // this thread's slice of the B tile: row n (clamped), vector c4 of the 32-k row
    uint32_t b_off[B_PER_T];
    int b_lds[B_PER_T];
#pragma unroll
    for (int it = 0; it < B_PER_T; ++it) {
        const int idx = tid + it * THREADS;
        const int row = idx / (BK / 4), c4 = idx % (BK / 4);
        int64_t bn = n0 + row;
        bn = bn < p.N ? bn : p.N - 1;
        b_off[it] = (uint32_t)(bn * p.b_sn + 4 * c4) * 4u;
        b_lds[it] = row * NT_PITCH + 4 * c4;
    }

    f32x4 acc[TN];
#pragma unroll
    for (int j = 0; j < TN; ++j) acc[j] = f32x4{0.f, 0.f, 0.f, 0.f};

    const int ktiles = (int)(p.K / BK);  // K % BK == 0 is a launch precondition
    const int last_tile = ktiles - 1;
    f32x4 ra[RING][NC];        // A fragments of tile t in slot t % RING
    f32x4 rb[RING][B_PER_T];   // B tile slice of tile t in slot t % RING
    f32x4 bf[2][TN];           // B fragments of the wave's g-th chunk in set g % 2 (g counts across tiles)

    auto load_a = [&](f32x4 (&dst)[NC], int kt) {
        const int k_bytes = (kt < last_tile ? kt : last_tile) * (BK * 4);
#pragma unroll
        for (int c = 0; c < NC; ++c)
            dst[c] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(a_rsrc, (int)(a_off + 64u * (uint32_t)(c * KSPLIT)), k_bytes, 0));
    };
    auto load_b = [&](f32x4 (&dst)[B_PER_T], int kt) {
        const int k_bytes = (kt < last_tile ? kt : last_tile) * (BK * 4);
#pragma unroll
        for (int it = 0; it < B_PER_T; ++it)
            dst[it] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(b_rsrc, (int)b_off[it], k_bytes, 0));
    };
    auto store_b = [&](const f32x4 (&src)[B_PER_T], int stage) {
        // every thread stores (rows >= BN are padding): no branch in the step body
#pragma unroll
        for (int it = 0; it < B_PER_T; ++it)
            *reinterpret_cast<f32x4*>(lds + stage * STAGE + b_lds[it]) = src[it];
    };
    auto read_b = [&](f32x4 (&dst)[TN], int stage, int c) {
#pragma unroll
        for (int j = 0; j < TN; ++j)
            dst[j] = *reinterpret_cast<const f32x4*>(lds + stage * STAGE + (16 * j + li) * NT_PITCH +
                                                     16 * (c * KSPLIT + ks) + 4 * lq);
    };

    // (u: the step's place in the unrolled group; the ring slot is u % RING, and the operand set alternates with every chunk,
    // which only repeats after RING steps when RING * NC is even: an odd ring of single-chunk tiles is unrolled twice over)
    constexpr int UNROLL = (RING * NC) % 2 == 0 ? RING : 2 * RING;
    auto tile_step = [&](auto u_tag, auto pre_tag, auto prea_tag, auto wr_tag, auto nxt_tag, int kt) {
        constexpr int u = decltype(u_tag)::value, r = u % RING;
        constexpr bool PRE = decltype(pre_tag)::value, PRE_A = decltype(prea_tag)::value;
        constexpr bool WR = decltype(wr_tag)::value, NXT = decltype(nxt_tag)::value;
        // The step's six memory instructions are spread between its MFMAs: issued
        // as one burst after the barrier they queue behind the other waves' requests
        // in the texture-address and LDS units and stall MFMA issue (measured: a
        // 16-byte LDS write costs a wave ~60 cycles of issue time, a global load up to
        // ~140 when eight waves issue together).
        if constexpr (PRE) load_b(rb[r], kt + RING);                         // slot r left for LDS two steps ago
        if constexpr (PRE_A) load_a(ra[(r + RING - 1) % RING], kt + RING - 1);  // fragments consumed in the previous step
        if constexpr (WR) store_b(rb[(r + 2) % RING], (r + 2) % NT_STAGES);  // tile kt + 2
        constexpr int MFMA = 0x008, VMEM_RD = 0x020, DS_RD = 0x100, DS_WR = 0x200;
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            constexpr int g0 = (u * NC) & 1;
            const int cur = (g0 + c) & 1;
            // fragments of the next chunk: same tile, or chunk 0 of tile kt + 1 (visible since the last barrier)
            if (c + 1 < NC) read_b(bf[cur ^ 1], r % NT_STAGES, c + 1);
            else if constexpr (NXT) read_b(bf[cur ^ 1], (r + 1) % NT_STAGES, 0);
#pragma unroll
            for (int s = 0; s < 4; ++s)
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    acc[j] = __builtin_amdgcn_mfma_f32_16x16x4f32(bf[cur][j][s], ra[r][c][s], acc[j], 0, 0, 0);
        }
        // Issue order inside the step. A wave's memory instructions are spread between
        // its MFMAs: issued as one burst after the barrier they queue behind the other
        // waves' requests in the LDS and texture-address units and hold up MFMA issue.
        // LDS traffic comes first (it must have completed at the barrier), the global
        // loads later.
        __builtin_amdgcn_sched_group_barrier(MFMA, 1, 0);
        __builtin_amdgcn_sched_group_barrier(DS_WR, B_PER_T, 0);
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            __builtin_amdgcn_sched_group_barrier(MFMA, 1, 0);
            __builtin_amdgcn_sched_group_barrier(DS_RD, 1, 0);
        }
        __builtin_amdgcn_sched_group_barrier(MFMA, 2, 0);
        __builtin_amdgcn_sched_group_barrier(VMEM_RD, B_PER_T, 0);
        __builtin_amdgcn_sched_group_barrier(MFMA, 2, 0);
        __builtin_amdgcn_sched_group_barrier(VMEM_RD, NC, 0);
        if constexpr (NC == 2) {
            __builtin_amdgcn_sched_group_barrier(MFMA, 3 * TN - 5, 0);  // rest of chunk 0
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                __builtin_amdgcn_sched_group_barrier(MFMA, 1, 0);
                __builtin_amdgcn_sched_group_barrier(DS_RD, 1, 0);
            }
        }
        __builtin_amdgcn_sched_group_barrier(MFMA, 4 * TN * NC, 0);
        __syncthreads();
    };

    MI355X_TRACE_STAMP(p, 5);
#pragma unroll
    for (int r = 0; r < RING; ++r) {  // tiles beyond the last are clamped: no branch
        load_a(ra[r], r);
        load_b(rb[r], r);
    }
    MI355X_TRACE_STAMP(p, 6);
    // The small-tile variants have registers to spare: fetch this lane's bias and residual
    // values now, so the epilogue does not wait for two more trips to memory (k-split
    // group 1 never needs them).
    constexpr bool PREFETCH_EPI = KSPLIT >= 2 && TN <= 4 && PER_CU < 3;   // (three workgroups per CU leave no registers for it)
    f32x4 pre_bias[PREFETCH_EPI ? TN : 1], pre_res[PREFETCH_EPI ? TN : 1];
    if constexpr (PREFETCH_EPI) {
        const int64_t pm = m0 + 16 * wm + li;
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int64_t n = n0 + 16 * j + 4 * lq;
            const bool in = ks == 0 && pm < p.M && n < p.N;
            pre_bias[j] = (in && (p.epi & MI355X_EPI_BIAS)) ? *reinterpret_cast<const f32x4*>(p.bias + n) : f32x4{0.f, 0.f, 0.f, 0.f};
            pre_res[j] = (in && (p.epi & MI355X_EPI_RESIDUAL))
                             ? *reinterpret_cast<const f32x4*>(p.residual + b0 * p.r_sb0 + b1 * p.r_sb1 + pm * p.r_sm + n)
                             : f32x4{0.f, 0.f, 0.f, 0.f};
        }
    }
    store_b(rb[0], 0);
    store_b(rb[1], 1);
    MI355X_TRACE_STAMP(p, 7);
    __syncthreads();
    read_b(bf[0], 0, 0);
    MI355X_TRACE_STAMP(p, 1);
    MI355X_TRACE_CYCLES(p, 12);

    // One code path for every tile: near the end of K the look-aheads are not switched
    // off but clamped to the last tile (they re-read data that is already in cache and
    // write LDS buffers nobody reads any more), so the step body stays branch-free
    // and the compiler's s_waitcnt counts stay exact from the first tile to the last.
    for (int kt0 = 0; kt0 < ktiles; kt0 += UNROLL) {
        nt_static_for<UNROLL>([&](auto u_tag) {
            const int kt = kt0 + decltype(u_tag)::value;
            if (kt < ktiles)  // uniform; only the last group can be partial
                tile_step(u_tag, std::true_type{}, std::true_type{}, std::true_type{}, std::true_type{}, kt);
        });
    }

    MI355X_TRACE_STAMP(p, 2);
    MI355X_TRACE_CYCLES(p, 13);
    // the k-split groups after the first hand their partial sums to group 0 through LDS (added in the order of the groups)
    if constexpr (KSPLIT >= 2) {
        f32x4* red = reinterpret_cast<f32x4*>(lds);
        if (ks >= 1) {
#pragma unroll
            for (int j = 0; j < TN; ++j) red[(((ks - 1) * WAVES_M + wm) * TN + j) * WAVE + lane] = acc[j];
        }
        __syncthreads();
        if (ks >= 1) return;
#pragma unroll
        for (int g = 1; g < KSPLIT; ++g)
#pragma unroll
            for (int j = 0; j < TN; ++j) acc[j] += red[(((g - 1) * WAVES_M + wm) * TN + j) * WAVE + lane];
    }

    // epilogue: acc[j][r] = C[m0 + 16*wm + li][n0 + 16*j + 4*lq + r]
    const int64_t m = m0 + 16 * wm + li;
    if (m >= p.M) return;
    float* C = p.C + b0 * p.c_sb0 + b1 * p.c_sb1;
    const float* R = (p.epi & MI355X_EPI_RESIDUAL) ? p.residual + b0 * p.r_sb0 + b1 * p.r_sb1 : nullptr;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
        const int64_t n = n0 + 16 * j + 4 * lq;
        if (n >= p.N) continue;
        f32x4 v = acc[j] * p.alpha;
        f32x4 bv = f32x4{0.f, 0.f, 0.f, 0.f};
        if constexpr (PREFETCH_EPI) bv = pre_bias[j];
        else if (p.epi & MI355X_EPI_BIAS) bv = *reinterpret_cast<const f32x4*>(p.bias + n);
        v.x = apply_epilogue(v.x, p.epi, bv.x);
        v.y = apply_epilogue(v.y, p.epi, bv.y);
        v.z = apply_epilogue(v.z, p.epi, bv.z);
        v.w = apply_epilogue(v.w, p.epi, bv.w);
        if constexpr (PREFETCH_EPI) v += pre_res[j];
        else if (R) v += *reinterpret_cast<const f32x4*>(R + m * p.r_sm + n);
        *reinterpret_cast<f32x4*>(C + m * p.c_sm + n) = v;
    }
    MI355X_TRACE_STAMP(p, 3);
}

// 128 x 48 tiles: true where the deep-ring kernel (two workgroups per CU) fills its last round and the lean one (three
// per CU) would leave most of its last round empty -- the one pattern in which the deep ring measured faster.
static bool deep_ring_rounds_fit(int64_t nwg, int cus, int64_t K) {
    const int64_t deep = 2 * (int64_t)cus, lean = 3 * (int64_t)cus;
    if (nwg <= lean || nwg > 4 * deep || K > 2048 || (nwg > 2 * deep && K < 768)) return false;   // (2048 tiles at K = 512: 99 against 110 us)
    const int64_t deep_empty = (deep - nwg % deep) % deep, lean_empty = (lean - nwg % lean) % lean;   // free places in the last round
    return deep_empty * 8 <= deep && lean_empty * 10 >= 3 * lean;
}

// and N a multiple of 4. Additionally needed here: K a multiple of the 32-k tile.
bool launch_gemm_f32_nt(GemmArgs p, int cus, hipStream_t stream) {
    if (p.K % NT_BK != 0 || p.K == 0) return false;
    // rows are addressed with 32-bit byte offsets from the start of a batch's matrix
    if (p.a_sm < 0 || p.b_sn < 0 || (p.M - 1) * p.a_sm + p.K >= ((int64_t)1 << 29) || (p.N - 1) * p.b_sn + p.K >= ((int64_t)1 << 29)) return false;
    // Candidates: 64x48, 64x64 and 64x144 tiles with two k-split groups, 128x48 and 128x96 tiles without.
    // Cost ~ rounds of workgroups over the CUs x tile area. 128 x 48 tiles run two workgroups per CU (116 registers), and
    // two workgroups that share a CU drift apart: one's first loads, last stores and barrier waits run under the other's
    // MFMAs. Measured against 128 x 96 tiles, one workgroup per CU: 1024 x 3072 x 768 (with Gelu) 42.5 against 43.7 us,
    // 2048 x 3072 x 768 78.7 against 82.6 us, 4096 x 4096 x 1024 261.8 against 297.5 us (131 TFLOP/s). A 128 x 48 tile
    // that has a CU to itself loses to two 64 x 48 tiles (512 x 3072 x 768: 24.0 against 23.4 us), hence rounds counted in
    // pairs for it. 128 x 96 stays selectable by hand (MI355X_GEMM_NT_BN=96).
    struct Cand { int bm, bn, per_cu; double weight; };
    // (1024 x 2304 x 768, measured: 768 tiles of 64 x 48, two workgroups sharing a CU, 35.2 us; 256 tiles of 64 x 144 36.1 us:
    // the wide tile gets no discount)
    const Cand cands[] = {{64, 48, 1, 1.0}, {64, 64, 1, 1.0}, {128, 96, 1, 0.8}, {64, 144, 1, 1.0}, {128, 48, 2, 0.78}};
    int best = 0;
    double best_cost = 1e300;
    const Tuning tune = tuning();
    const int force = tune.gemm_nt_bn, force_bm = tune.gemm_nt_bm;
    for (int c = 0; c < 5; ++c) {
        const int64_t nwg = p.batch * ceil_div(p.M, cands[c].bm) * ceil_div(p.N, cands[c].bn);
        double cost = (double)ceil_div(nwg, (int64_t)cus * cands[c].per_cu) * cands[c].per_cu * cands[c].bm * cands[c].bn * cands[c].weight;
        // (128 x 48 also runs three to a CU, in its lean form, 5 % faster per tile at full occupancy)
        if (c == 4) cost = std::min(cost, (double)ceil_div(nwg, (int64_t)cus * 3) * 3 * cands[c].bm * cands[c].bn * 0.74);
        // (64 x 64 tiles have no lean form: over a short K their six-tile ring is most of the work before the first MFMA.
        // 384 x 4096 x 256: 15.1 us against 13.5 us as 64 x 48; 1024 x 1024 x 256 stays with them, 8.7 against 10.5 us)
        if (c == 1 && p.K <= 512) cost *= 1.15;
        // (128 x 96 tiles, 16 waves, one workgroup per CU: over a long K and in whole rounds -- where nothing of a round is
        // wasted on them -- they are the fastest form by 1-3 %: 2048 x 3072 x 3072 270.9 against 280.3 us, 5120 x 3072 x 3072
        // 671.8 against 691.1 us; with a ragged last round they lose by up to 10 %)
        if (c == 2 && p.K >= 1536 && nwg % cus == 0) cost *= 0.75 / 0.8;
        if (force) {   // MI355X_GEMM_NT_BN picks the tile width, MI355X_GEMM_NT_BM the height where two candidates share a width
            if (force == cands[c].bn && (force_bm ? force_bm == cands[c].bm : cands[c].bm == 64 || cands[c].bn == 96)) { best = c; break; }
        } else if (cost < best_cost) {
            best = c;
            best_cost = cost;
        }
    }
    p.tiles_m = ceil_div(p.M, cands[best].bm);
    p.tiles_n = ceil_div(p.N, cands[best].bn);
    p.nwg = p.batch * p.tiles_m * p.tiles_n;
    if (p.nwg >= ((int64_t)1 << 31)) return false;
    // an XCD holds cus / 8 tiles at a time (twice that for the candidates that run in pairs)
    const int64_t per_xcd = ceil_div(p.nwg, (int64_t)NUM_XCD);
    const int64_t per_batch = p.tiles_m * p.tiles_n;   // tiles are numbered batch entry by batch entry
    // (the lean 128 x 48 kernel, chosen below, runs three workgroups per CU)
    const bool lean128 = best == 4 && tune.gemm_nt_bk == 0 && (tune.gemm_nt_per_cu ? tune.gemm_nt_per_cu == 3 : !deep_ring_rounds_fit(p.nwg, cus, p.K));
    p.group_m = choose_group_m(p.tiles_m, per_xcd < per_batch ? per_xcd : per_batch, (int64_t)(lean128 ? 3 : cands[best].per_cu) * (cus / NUM_XCD), cands[best].bm, cands[best].bn, p.K * 4);
    if (tune.gemm_group_m > 0) p.group_m = tune.gemm_group_m;
    const dim3 grid((unsigned)p.nwg), block(NT_THREADS), block16(2 * NT_THREADS);
    // The smallest variant walks K in 64-k tiles with a three-deep ring where K allows: half the barriers per FLOP
    // and the same bytes in flight as six 32-k tiles (1024 x 768 x 768: 14.0 us against 14.7 us, 1024 x 768 x 3072:
    // 41.9 us against 44.8 us with 32-k tiles and 43.9 us with six 64-k tiles in flight; the wider
    // variants lose 1-2 % with 64-k tiles)
    const bool bk64 = p.K % 64 == 0 && (tune.gemm_nt_bk ? tune.gemm_nt_bk == 64 : true);
    // ... and where K is short a lean form of it (32-k tiles, a three-deep ring, no early fetch of bias and residual: 69
    // registers) of which three workgroups share a CU: all 768 tiles of 1024 x 2304 x 768 are resident at once (32.4 against
    // 34.0 us), and a workgroup that has its CU to itself starts sooner with half the bytes in its first burst
    // (1024 x 768 x 768: 13.1 against 13.6 us). With its 64 k of look-ahead it falls behind once the operands no longer sit
    // in the L2 (1024 x 768 x 1536: 25.8 against 22.9 us; with three workgroups per CU it holds up to K = 1536).
    // MI355X_GEMM_NT_PER_CU: 3 forces it, 2 forbids it.
    const bool lean = tune.gemm_nt_per_cu ? tune.gemm_nt_per_cu == 3 : (p.K <= 1024 || (p.K <= 1536 && p.nwg > 2 * (int64_t)cus));
    // (a workgroup that has its CU to itself also has the registers to fetch its bias and residual values before the loop)
    // A workgroup that has its CU to itself over a long K runs as 16 waves, 4 wave rows x 4 k-split groups on 64-k tiles
    // (four waves per SIMD cover each other's barrier waits; 104 registers): 1024 x 768 x 3072 38.0 against 39.8 us,
    // 512 x 768 x 3072 37.2 against 39.5 us, 1024 x 768 x 1536 21.6 against 22.5 us; at K = 768 the lean kernel wins
    // (12.4 against 13.0 us), and with more than one tile per CU eight waves do (1024 x 2304 x 768: 31.0 against 35.8 us).
    // 128-k tiles or six 64-k tiles in flight (128 registers) are slower everywhere. MI355X_GEMM_NT_WAVES: 16 forces it, 8 forbids it.
    const bool waves16 = best == 0 && p.K % 64 == 0 && tune.gemm_nt_bk == 0 &&
                         (tune.gemm_nt_waves ? tune.gemm_nt_waves == 16 : (p.nwg <= cus && p.K >= 1280 && tune.gemm_nt_per_cu == 0));
    if (waves16) hipLaunchKernelGGL((gemm_f32_nt_kernel<3, 4, 4, 64, 3, 1>), grid, block16, 0, stream, p);
    else if (best == 0 && lean && tune.gemm_nt_bk == 0 && p.nwg <= cus && tune.gemm_nt_per_cu != 3) hipLaunchKernelGGL((gemm_f32_nt_kernel<3, 4, 2, 32, 3, 1>), grid, block, 0, stream, p);
    else if (best == 0 && lean && tune.gemm_nt_bk == 0) hipLaunchKernelGGL((gemm_f32_nt_kernel<3, 4, 2, 32, 3, 3>), grid, block, 0, stream, p);
    else if (best == 0 && bk64) hipLaunchKernelGGL((gemm_f32_nt_kernel<3, 4, 2, 64, 3>), grid, block, 0, stream, p);
    else if (best == 0) hipLaunchKernelGGL((gemm_f32_nt_kernel<3, 4, 2>), grid, block, 0, stream, p);
    else if (best == 1 && bk64 && p.K >= 2048) hipLaunchKernelGGL((gemm_f32_nt_kernel<4, 4, 2, 64, 3>), grid, block, 0, stream, p);  // 2.5 % at K = 3072, nothing at 1024
    else if (best == 1) hipLaunchKernelGGL((gemm_f32_nt_kernel<4, 4, 2>), grid, block, 0, stream, p);
    // (128 x 96 tiles, one workgroup per CU, are never the library's own choice any more; as 16 waves, 8 wave rows x 2 k-split
    // groups, they take 40.7 against 42.9 us on 1024 x 3072 x 768 and 288 against 302 us on 4096 x 4096 x 1024)
    else if (best == 2 && tune.gemm_nt_waves != 8) hipLaunchKernelGGL((gemm_f32_nt_kernel<6, 8, 2, 32, 3, 1>), grid, block16, 0, stream, p);
    else if (best == 2) hipLaunchKernelGGL((gemm_f32_nt_kernel<6, 8, 1>), grid, block, 0, stream, p);
    // the same for 128 x 48 tiles (80 registers, three workgroups per CU): 1024 x 3072 x 768 with Gelu takes 40.0 against
    // 42.2 us, 4096 x 4096 x 1024 246 against 262 us. Measured over 3072-wide outputs of 512 to 3328 tiles and K from 768
    // to 4096 it wins by 5-7 % at K = 768, 3-4 % at 1536 and 1-2 % from 2048 on, with one exception: where the tiles fill
    // whole rounds of two per CU but not of three (1024 tiles on 256 CUs: 88.0 against 78.3 us at K = 768, 160 against
    // 144 us at 1536, 197 against 184 us at 2048, even from K = 3072 on; 2048 tiles: even at 768, 293 against 282 us at
    // 1536) the leftover third of a round runs one or two workgroups to a CU, where the short ring cannot cover the
    // latency. MI355X_GEMM_NT_PER_CU: 3 forces it, 2 forbids it.
    else if (lean128)
        hipLaunchKernelGGL((gemm_f32_nt_kernel<3, 8, 1, 32, 3, 2>), grid, block, 0, stream, p);
    else if (best == 4 && bk64) hipLaunchKernelGGL((gemm_f32_nt_kernel<3, 8, 1, 64, 3>), grid, block, 0, stream, p);
    else if (best == 4) hipLaunchKernelGGL((gemm_f32_nt_kernel<3, 8, 1>), grid, block, 0, stream, p);
    else hipLaunchKernelGGL((gemm_f32_nt_kernel<9, 4, 2>), grid, block, 0, stream, p);
    return true;
}

}  // namespace mi355x
