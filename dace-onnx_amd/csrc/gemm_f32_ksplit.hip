// fp32 GEMM, both operands contiguous along k, for problems with few output elements per CU and a long K
// (1024 x 768 x 3072: one 32 x 96 tile per CU): the eight waves of a workgroup split K, not the tile.
//
//   * v_mfma_f32_32x32x2_f32: a wave holds the whole 32 x 96 tile (three 32 x 32 blocks, 48 accumulator registers)
//     and multiplies every eighth 16-k slice of K. An operand register feeds 64 cycles of the matrix pipe instead of
//     the 32 of v_mfma_f32_16x16x4_f32: half the operand loads and LDS reads per FLOP.
//   * Nothing is shared between waves before the end, so there is no barrier in the K loop. A wave stages its own
//     slice of B (96 rows x 16 k, fetched with coalesced 16-byte loads: a row's 64 bytes by four neighbouring lanes)
//     through a private LDS buffer into the MFMA layout (lane = row, 16-byte reads); its slice of A (32 rows x 16 k)
//     goes from global memory straight into the operand registers. Per slice and wave: 8 loads, 6 LDS writes,
//     6 LDS reads, 24 MFMAs (1536 cycles of the matrix pipe).
//   * What this buys against 64 x 48 tiles with two k-split groups: the vector memory pipe takes a load whose
//     neighbouring lanes touch different rows (the A operand in MFMA layout) at one row per cycle, 64 cycles per
//     KB instead of 16-20. A costs (rows of the tile) x K x 4 / 16 cycles, B (coalesced) about a third of that per byte:
//     32 x 96 tiles need 0.65 cycles of that pipe per matrix-pipe cycle where 64 x 48 tiles need 0.83.
//   * The eight partial tiles meet in LDS (each wave's own staging buffer holds its 12 KB), one barrier, then every
//     wave adds up, finishes (alpha, bias, activation, residual) and stores its share of the tile.
// MFMA operands are swapped as in gemm_f32_nt.hip: a lane's accumulator registers are four consecutive n of one row.
#include "common.h"
#include "gemm_tile.h"
#include "gemm_args.h"

#include <type_traits>
#include <utility>

namespace mi355x {

template <class F, int... I>
__device__ __forceinline__ void ks_static_for_impl(F&& f, std::integer_sequence<int, I...>) {
    (f(std::integral_constant<int, I>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void ks_static_for(F&& f) {
    ks_static_for_impl(static_cast<F&&>(f), std::make_integer_sequence<int, N>{});
}

constexpr int KS_WAVES = 8, KS_THREADS = 64 * KS_WAVES, KS_BM = 32, KS_SLICE = 16;
constexpr int KS_PITCH = KS_SLICE + 4;   // floats per staged B row: 16-byte reads of 32 rows fall into distinct banks

// TN: 32-column blocks per tile (BN = 32 TN)
template <int TN>
__global__ __launch_bounds__(KS_THREADS) void gemm_f32_ksplit_kernel(GemmArgs p) {
    constexpr int BN = 32 * TN, NB = BN / 16;                 // NB: staging loads per slice (16 rows of B each)
    constexpr int STAGE = BN * KS_PITCH;                      // floats of one staged slice
    constexpr int PART = 4 * TN * 4 * WAVE;                   // floats of one wave's partial tile: 4 TN vectors per lane
    constexpr int REGION = STAGE > PART ? STAGE : PART;
    __shared__ __attribute__((aligned(16))) float lds[KS_WAVES * REGION];

    const int tid = threadIdx.x;
    const int lane = tid % WAVE, wave = __builtin_amdgcn_readfirstlane(tid / WAVE);
    const int lj = lane % 32, g = lane / 32;
    MI355X_TRACE_STAMP(p, 0);
    MI355X_TRACE_HWID(p);

    const int64_t logical = xcd_remap(blockIdx.x, p.nwg);
    const uint32_t tiles_per_batch = (uint32_t)(p.tiles_m * p.tiles_n);
    const uint32_t b = (uint32_t)logical / tiles_per_batch, t = (uint32_t)logical % tiles_per_batch;
    const int64_t b0 = b / (uint32_t)p.batch1, b1 = b % (uint32_t)p.batch1;
    int64_t tm, tn;
    tile_coords(t, p.tiles_m, p.tiles_n, p.group_m, tm, tn);
    const int64_t m0 = tm * KS_BM, n0 = tn * BN;

    // operands as raw buffers: the batch entry's matrix as the base, row and k-chunk of the lane as a 32-bit byte
    // offset, the slice as the scalar offset (launch precondition: a matrix spans less than 2^31 bytes)
    const __amdgpu_buffer_rsrc_t a_rsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(p.A + b0 * p.a_sb0 + b1 * p.a_sb1), 0, 0x7fffffff, 0x00020000);
    const __amdgpu_buffer_rsrc_t b_rsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(p.B + b0 * p.b_sb0 + b1 * p.b_sb1), 0, 0x7fffffff, 0x00020000);
    // A operand of MFMA step (h, s): A[m0 + lj][slice + 4 (2 h + g) + s]; rows past M are clamped and never stored
    int64_t am = m0 + lj;
    am = am < p.M ? am : p.M - 1;
    const uint32_t a_off = (uint32_t)(am * p.a_sm + 4 * g) * 4u;
    // staging load q of a slice: rows n0 + 16 q + lane / 4 of B, k-chunk lane % 4 (clamped past N)
    uint32_t b_off[NB];
#pragma unroll
    for (int q = 0; q < NB; ++q) {
        int64_t bn = n0 + 16 * q + lane / 4;
        bn = bn < p.N ? bn : p.N - 1;
        b_off[q] = (uint32_t)(bn * p.b_sn + 4 * (lane % 4)) * 4u;
    }
    float* const stage = lds + wave * REGION;                 // this wave's own buffer
    float* const st_wr = stage + (lane / 4) * KS_PITCH + 4 * (lane % 4);
    const float* const st_rd = stage + lj * KS_PITCH + 4 * g;

    // slices of this wave: wave, wave + 8, ... (K % 16 == 0 is a launch precondition)
    const int slices = (int)(p.K / KS_SLICE);
    const int mine = (slices - wave + KS_WAVES - 1) / KS_WAVES;
    const int last = mine > 0 ? mine - 1 : 0;

    f32x16 acc[TN];
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[j][r] = 0.f;
    f32x4 ra[4][2];        // A operands of slice i in slot i % 4
    f32x4 rb[2][NB];       // B rows of slice i on their way to LDS, slot i % 2
    f32x4 bf[2][TN][2];    // B operands of slice i, set i % 2

    // byte offset of this wave's i-th slice along k; look-aheads past its last slice (and a wave without any slice) stay inside K
    auto slice_bytes = [&](int i) {
        const int s = KS_WAVES * (i < last ? i : last) + wave;
        return (s < slices ? s : slices - 1) * (KS_SLICE * 4);
    };
    auto load_a = [&](f32x4 (&dst)[2], int i) __attribute__((always_inline)) {
#pragma unroll
        for (int h = 0; h < 2; ++h) dst[h] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(a_rsrc, (int)(a_off + 32u * h), slice_bytes(i), 0));
    };
    auto load_b = [&](f32x4 (&dst)[NB], int i) __attribute__((always_inline)) {
#pragma unroll
        for (int q = 0; q < NB; ++q) dst[q] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(b_rsrc, (int)b_off[q], slice_bytes(i), 0));
    };
    auto store_b = [&](const f32x4 (&src)[NB]) __attribute__((always_inline)) {
#pragma unroll
        for (int q = 0; q < NB; ++q) *reinterpret_cast<f32x4*>(st_wr + 16 * q * KS_PITCH) = src[q];
    };
    auto read_b = [&](f32x4 (&dst)[TN][2]) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int h = 0; h < 2; ++h) dst[j][h] = *reinterpret_cast<const f32x4*>(st_rd + 32 * j * KS_PITCH + 8 * h);
    };

    // At the top of step i: operand set i % 2 holds slice i of B, A slots i .. i + 2 (mod 4) and B slot (i + 1) % 2 are
    // loaded or on their way. The step asks for slice i + 2 of B (into the slot slice i left for LDS one step ago) and
    // i + 3 of A (into the slot slice i - 1 was multiplied from), moves slice i + 1 through LDS and multiplies slice i.
    // (A third B slot, so that a slice's loads have two steps to land, changes nothing: 41.8 us against 41.9 us on
    // 1024 x 768 x 3072, and costs the short problem its start: 15.4 us against 14.3 us at K = 768.)
    auto step = [&](auto u_tag, int i) __attribute__((always_inline)) {
        constexpr int u = decltype(u_tag)::value;   // i modulo 4
        load_b(rb[u % 2], i + 2);
        load_a(ra[(u + 3) % 4], i + 3);
        store_b(rb[(u + 1) % 2]);
        read_b(bf[(u + 1) % 2]);
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int s = 0; s < 4; ++s)
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    acc[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(bf[u % 2][j][h][s], ra[u][h][s], acc[j], 0, 0, 0);
        // one memory instruction between two MFMAs: issued as a burst they queue in the address and LDS units while
        // neither wave of the SIMD multiplies. LDS first (the next step's operands), the loads behind it.
        constexpr int MFMA = 0x008, VMEM_RD = 0x020, DS_RD = 0x100, DS_WR = 0x200;
#pragma unroll
        for (int q = 0; q < NB; ++q) {
            __builtin_amdgcn_sched_group_barrier(MFMA, 1, 0);
            __builtin_amdgcn_sched_group_barrier(DS_WR, 1, 0);
        }
#pragma unroll
        for (int q = 0; q < 2 * TN; ++q) {
            __builtin_amdgcn_sched_group_barrier(MFMA, 1, 0);
            __builtin_amdgcn_sched_group_barrier(DS_RD, 1, 0);
        }
#pragma unroll
        for (int q = 0; q < NB + 2; ++q) {
            __builtin_amdgcn_sched_group_barrier(MFMA, 1, 0);
            __builtin_amdgcn_sched_group_barrier(VMEM_RD, 1, 0);
        }
        __builtin_amdgcn_sched_group_barrier(MFMA, 8 * TN, 0);
    };

    load_a(ra[0], 0);
    load_b(rb[0], 0);
    load_a(ra[1], 1);
    load_b(rb[1], 1);
    load_a(ra[2], 2);
    store_b(rb[0]);
    read_b(bf[0]);
    MI355X_TRACE_STAMP(p, 1);
    MI355X_TRACE_CYCLES(p, 12);
    // whole groups of four steps without a branch between them (with guards inside the loop the compiler's wait counts
    // fall back to waiting for every load at the joins), then the at most three remaining steps, guarded
    int i0 = 0;
    for (; i0 + 4 <= mine; i0 += 4) ks_static_for<4>([&](auto u_tag) { step(u_tag, i0 + decltype(u_tag)::value); });
    ks_static_for<3>([&](auto u_tag) {
        const int i = i0 + decltype(u_tag)::value;
        if (i < mine) step(u_tag, i);   // uniform
    });

    MI355X_TRACE_STAMP(p, 2);
    MI355X_TRACE_CYCLES(p, 13);
    // ---- the eight partial tiles meet in LDS: vector v (0 .. 4 TN - 1) of a lane is acc[v / 4][4 (v % 4) .. + 3] =
    // C[m0 + lj][n0 + 32 (v / 4) + 8 (v % 4) + 4 g .. + 3]
    // (a wave writes its partial tile over its own staging buffer, which only it reads: no barrier before)
#pragma unroll
    for (int v = 0; v < 4 * TN; ++v)
        *reinterpret_cast<f32x4*>(stage + (v * WAVE + lane) * 4) = f32x4{acc[v / 4][4 * (v % 4)], acc[v / 4][4 * (v % 4) + 1], acc[v / 4][4 * (v % 4) + 2], acc[v / 4][4 * (v % 4) + 3]};
    __syncthreads();
    const int64_t m = m0 + lj;
    float* C = p.C + b0 * p.c_sb0 + b1 * p.c_sb1;
    const float* R = (p.epi & MI355X_EPI_RESIDUAL) ? p.residual + b0 * p.r_sb0 + b1 * p.r_sb1 : nullptr;
    // wave w finishes vectors w, w + 8, ...
#pragma unroll
    for (int vi = 0; vi < (4 * TN + KS_WAVES - 1) / KS_WAVES; ++vi) {
        const int v = wave + vi * KS_WAVES;   // uniform
        if (v >= 4 * TN) break;
        f32x4 sum = *reinterpret_cast<const f32x4*>(lds + (v * WAVE + lane) * 4);
#pragma unroll
        for (int w = 1; w < KS_WAVES; ++w) sum += *reinterpret_cast<const f32x4*>(lds + w * REGION + (v * WAVE + lane) * 4);
        const int64_t n = n0 + 32 * (v / 4) + 8 * (v % 4) + 4 * g;
        if (m >= p.M || n >= p.N) continue;
        f32x4 val = sum * p.alpha;
        f32x4 bv = f32x4{0.f, 0.f, 0.f, 0.f};
        if (p.epi & MI355X_EPI_BIAS) bv = *reinterpret_cast<const f32x4*>(p.bias + n);
        val.x = apply_epilogue(val.x, p.epi, bv.x);
        val.y = apply_epilogue(val.y, p.epi, bv.y);
        val.z = apply_epilogue(val.z, p.epi, bv.z);
        val.w = apply_epilogue(val.w, p.epi, bv.w);
        if (R) val += *reinterpret_cast<const f32x4*>(R + m * p.r_sm + n);
        *reinterpret_cast<f32x4*>(C + m * p.c_sm + n) = val;
    }
    MI355X_TRACE_STAMP(p, 3);
}

// The caller guarantees: 16-byte aligned operands, a_sk == b_sk == 1, every stride and N a multiple of 4.
// Additionally needed here: K a multiple of the 16-k slice. Returns false when nothing was launched.
bool launch_gemm_f32_ksplit(GemmArgs p, int cus, hipStream_t stream) {
    if (p.K % KS_SLICE != 0 || p.K < KS_SLICE) return false;
    if (p.a_sm < 0 || p.b_sn < 0 || (p.M - 1) * p.a_sm + p.K >= ((int64_t)1 << 29) || (p.N - 1) * p.b_sn + p.K >= ((int64_t)1 << 29)) return false;
    p.tiles_m = ceil_div(p.M, (int64_t)KS_BM);
    p.tiles_n = ceil_div(p.N, (int64_t)96);
    p.nwg = p.batch * p.tiles_m * p.tiles_n;
    if (p.nwg >= ((int64_t)1 << 31)) return false;
    const int64_t per_xcd = ceil_div(p.nwg, (int64_t)NUM_XCD), per_batch = p.tiles_m * p.tiles_n;
    p.group_m = choose_group_m(p.tiles_m, per_xcd < per_batch ? per_xcd : per_batch, cus / NUM_XCD, KS_BM, 96, p.K * 4);
    const Tuning tune = tuning();
    if (tune.gemm_group_m > 0) p.group_m = tune.gemm_group_m;
    hipLaunchKernelGGL((gemm_f32_ksplit_kernel<3>), dim3((unsigned)p.nwg), dim3(KS_THREADS), 0, stream, p);
    return true;
}

}  // namespace mi355x
