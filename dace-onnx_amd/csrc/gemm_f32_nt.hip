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
#include "common.h"
#include "gemm_tile.h"
#include "gemm_args.h"

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

constexpr int NT_BM = 64, NT_BK = 32, NT_THREADS = 512, NT_RING = 6, NT_STAGES = 3;
constexpr int NT_PITCH = NT_BK + LDS_PAD;

template <int TN>
__global__ __launch_bounds__(NT_THREADS) void gemm_f32_nt_kernel(GemmArgs p) {
    constexpr int BM = NT_BM, BN = 16 * TN, BK = NT_BK, RING = NT_RING;
    constexpr int B_VECS = BN * (BK / 4);                       // 16-byte vectors of one B tile
    constexpr int B_PER_T = (B_VECS + NT_THREADS - 1) / NT_THREADS;
    constexpr int B_ROWS = B_PER_T * NT_THREADS / (BK / 4);     // rows incl. the ones only written as padding
    constexpr int STAGE = B_ROWS * NT_PITCH;                    // floats per LDS buffer
    constexpr int RED = BM * BN;                                // partial sums of k-split group 1
    constexpr int LDS_FLOATS = NT_STAGES * STAGE > RED ? NT_STAGES * STAGE : RED;
    __shared__ __attribute__((aligned(16))) float lds[LDS_FLOATS];

    const int tid = threadIdx.x;
    const int lane = tid % WAVE, wave = tid / WAVE;
    const int li = lane % 16, lq = lane / 16;
    const int wm = wave % 4, ks = wave / 4;   // wave row, k-split group

    const int64_t logical = xcd_remap(blockIdx.x, p.nwg);
    const int64_t tiles_per_batch = p.tiles_m * p.tiles_n;
    const int64_t b = logical / tiles_per_batch, t = logical % tiles_per_batch;
    const int64_t b0 = b / p.batch1, b1 = b % p.batch1;
    const int64_t m0 = (t / p.tiles_n) * BM, n0 = (t % p.tiles_n) * BN;

    // this lane's A fragment source: row m (clamped into the matrix), 4 floats at
    // k = 32*kt + 16*ks + 4*lq
    int64_t am = m0 + 16 * wm + li;
    am = am < p.M ? am : p.M - 1;
    const float* __restrict__ a_ptr = p.A + b0 * p.a_sb0 + b1 * p.a_sb1 + am * p.a_sm + 16 * ks + 4 * lq;
    // this thread's slice of the B tile: row n (clamped), vector c4 of the 32-k row
    const float* b_ptr[B_PER_T];
    int b_lds[B_PER_T];
#pragma unroll
    for (int it = 0; it < B_PER_T; ++it) {
        const int idx = tid + it * NT_THREADS;
        const int row = idx / (BK / 4), c4 = idx % (BK / 4);
        int64_t bn = n0 + row;
        bn = bn < p.N ? bn : p.N - 1;
        b_ptr[it] = p.B + b0 * p.b_sb0 + b1 * p.b_sb1 + bn * p.b_sn + 4 * c4;
        b_lds[it] = row * NT_PITCH + 4 * c4;
    }

    f32x4 acc[TN];
#pragma unroll
    for (int j = 0; j < TN; ++j) acc[j] = f32x4{0.f, 0.f, 0.f, 0.f};

    f32x4 ra[RING];            // A fragment of tile t in slot t % RING
    f32x4 rb[RING][B_PER_T];   // B tile slice of tile t in slot t % RING
    f32x4 bf[2][TN];           // B fragments of tile t in set t % 2

    auto load_a = [&](f32x4& dst, int kt) { dst = *reinterpret_cast<const f32x4*>(a_ptr + (int64_t)kt * BK); };
    auto load_b = [&](f32x4 (&dst)[B_PER_T], int kt) {
#pragma unroll
        for (int it = 0; it < B_PER_T; ++it)
            dst[it] = *reinterpret_cast<const f32x4*>(b_ptr[it] + (int64_t)kt * BK);
    };
    auto store_b = [&](const f32x4 (&src)[B_PER_T], int stage) {
        // every thread stores (rows >= BN are padding): no branch in the step body
#pragma unroll
        for (int it = 0; it < B_PER_T; ++it)
            *reinterpret_cast<f32x4*>(lds + stage * STAGE + b_lds[it]) = src[it];
    };
    auto read_b = [&](f32x4 (&dst)[TN], int stage) {
#pragma unroll
        for (int j = 0; j < TN; ++j)
            dst[j] = *reinterpret_cast<const f32x4*>(lds + stage * STAGE + (16 * j + li) * NT_PITCH + 16 * ks + 4 * lq);
    };

    auto tile_step = [&](auto r_tag, auto pre_tag, auto prea_tag, auto wr_tag, auto nxt_tag, int kt) {
        constexpr int r = decltype(r_tag)::value;
        constexpr bool PRE = decltype(pre_tag)::value, PRE_A = decltype(prea_tag)::value;
        constexpr bool WR = decltype(wr_tag)::value, NXT = decltype(nxt_tag)::value;
        // The step's six memory instructions are spread between its MFMAs: issued
        // as one burst after the barrier they queue behind the other waves' requests
        // in the texture-address and LDS units and stall MFMA issue (measured: a
        // 16-byte LDS write costs a wave ~60 cycles of issue time, a global load up to
        // ~140 when eight waves issue together).
        if constexpr (PRE) load_b(rb[r], kt + RING);                         // slot r left for LDS two steps ago
        if constexpr (PRE_A) load_a(ra[(r + RING - 1) % RING], kt + RING - 1);  // fragment consumed in the previous step
        if constexpr (WR) store_b(rb[(r + 2) % RING], (r + 2) % NT_STAGES);  // tile kt + 2
        if constexpr (NXT) read_b(bf[(r + 1) & 1], (r + 1) % NT_STAGES);     // tile kt + 1, already visible
#pragma unroll
        for (int s = 0; s < 4; ++s)
#pragma unroll
            for (int j = 0; j < TN; ++j)
                acc[j] = __builtin_amdgcn_mfma_f32_16x16x4f32(bf[r & 1][j][s], ra[r][s], acc[j], 0, 0, 0);
        // order: LDS traffic first, one instruction after each of the first MFMAs (it must
        // be complete at the barrier), the global loads later in the step
        constexpr int MFMA = 0x008, VMEM_RD = 0x020, DS_RD = 0x100, DS_WR = 0x200;
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
        __builtin_amdgcn_sched_group_barrier(VMEM_RD, 1, 0);
        __builtin_amdgcn_sched_group_barrier(MFMA, 4 * TN, 0);
        __syncthreads();
    };

    const int ktiles = (int)(p.K / BK);  // K % 32 == 0 is a launch precondition
#pragma unroll
    for (int r = 0; r < RING; ++r)
        if (r < ktiles) {
            load_a(ra[r], r);
            load_b(rb[r], r);
        }
    store_b(rb[0], 0);
    if (ktiles > 1) store_b(rb[1], 1);
    __syncthreads();
    if (ktiles > 0) read_b(bf[0], 0);

    int kt0 = 0;
    for (; kt0 + 2 * RING <= ktiles; kt0 += RING) {  // steady state: branch-free body
        nt_static_for<RING>([&](auto r_tag) {
            tile_step(r_tag, std::true_type{}, std::true_type{}, std::true_type{}, std::true_type{}, kt0 + decltype(r_tag)::value);
        });
    }
    for (; kt0 < ktiles; kt0 += RING) {              // tail: look-aheads switch off one by one
        nt_static_for<RING>([&](auto r_tag) {
            const int kt = kt0 + decltype(r_tag)::value;
            if (kt < ktiles) {
                constexpr std::true_type T{};
                constexpr std::false_type F{};
                if (kt + RING < ktiles) tile_step(r_tag, T, T, T, T, kt);
                else if (kt + RING == ktiles) tile_step(r_tag, F, T, T, T, kt);
                else if (kt + 2 < ktiles) tile_step(r_tag, F, F, T, T, kt);
                else if (kt + 1 < ktiles) tile_step(r_tag, F, F, F, T, kt);
                else tile_step(r_tag, F, F, F, F, kt);
            }
        });
    }

    // k-split group 1 hands its partial sums to group 0 through LDS
    f32x4* red = reinterpret_cast<f32x4*>(lds);
    if (ks == 1) {
#pragma unroll
        for (int j = 0; j < TN; ++j) red[(wm * TN + j) * WAVE + lane] = acc[j];
    }
    __syncthreads();
    if (ks == 1) return;
#pragma unroll
    for (int j = 0; j < TN; ++j) acc[j] += red[(wm * TN + j) * WAVE + lane];

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
        if (p.epi & MI355X_EPI_BIAS) bv = *reinterpret_cast<const f32x4*>(p.bias + n);
        v.x = apply_epilogue(v.x, p.epi, bv.x);
        v.y = apply_epilogue(v.y, p.epi, bv.y);
        v.z = apply_epilogue(v.z, p.epi, bv.z);
        v.w = apply_epilogue(v.w, p.epi, bv.w);
        if (R) v += *reinterpret_cast<const f32x4*>(R + m * p.r_sm + n);
        *reinterpret_cast<f32x4*>(C + m * p.c_sm + n) = v;
    }
}

// The caller guarantees: 16-byte aligned operands, a_sk == b_sk == 1, every stride
// and N a multiple of 4. Additionally needed here: K a multiple of the 32-k tile.
bool launch_gemm_f32_nt(GemmArgs p, int cus, hipStream_t stream) {
    if (p.K % NT_BK != 0 || p.K == 0) return false;
    // TN = 3 (48 columns) when it tiles N exactly or gives a fuller last wave of
    // workgroups than 64-column tiles do
    const int64_t tm = ceil_div(p.M, NT_BM);
    auto waste = [&](int bn) {
        const int64_t nwg = p.batch * tm * ceil_div(p.N, bn);
        const int64_t rounds = ceil_div(nwg, (int64_t)cus);
        return (double)(rounds * cus) * bn;  // column-slots of work the machine is occupied for
    };
    const bool use48 = waste(48) <= waste(64);
    const int bn = use48 ? 48 : 64;
    p.tiles_m = tm;
    p.tiles_n = ceil_div(p.N, bn);
    p.nwg = p.batch * p.tiles_m * p.tiles_n;
    if (p.nwg >= ((int64_t)1 << 31)) return false;
    const dim3 grid((unsigned)p.nwg), block(NT_THREADS);
    if (use48) hipLaunchKernelGGL(gemm_f32_nt_kernel<3>, grid, block, 0, stream, p);
    else hipLaunchKernelGGL(gemm_f32_nt_kernel<4>, grid, block, 0, stream, p);
    return true;
}

}  // namespace mi355x
