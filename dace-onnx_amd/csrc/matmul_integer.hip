// ONNX MatMulInteger, int8 x int8 -> int32, bit-exact, on the gfx950 int8 matrix cores.
//
// The reference has no expansion of its own for this node: the generated class
// (daceml/onnx/nodes/onnx_op.py:623-640) is only ever expanded through ONNX
// Runtime (onnx_op.py:686-687 -> daceml/onnx/nodes/node_codegen.py:321-573).
//
//   Y[m,n] = sum_k (A[m,k] - za)(B[k,n] - zb)
//          = sum_k A B  -  zb * rowsum_A[m]  -  za * colsum_B[n]  +  K * za * zb
// The raw product runs on v_mfma_i32_32x32x32_i8; the row/column sums are taken
// with v_dot4_i32_i8 on the very operand registers the MFMA consumes, so the
// zero points cost no extra memory traffic and (a - za) never has to fit in
// int8. All arithmetic is modulo 2^32, the same as an int32 accumulator.
//
// Data movement
//   * A [M,K] is k-contiguous: 16-byte global loads, LDS tile [128][64+16 B],
//     a lane's MFMA operand (16 consecutive k of one row) is one 16-byte read.
//   * B [K,N] is n-contiguous but the MFMA wants 16 k of one COLUMN per lane.
//     The loader transposes 4x4 byte blocks in registers (v_perm_b32) once per
//     workgroup and stores LDS words holding 4 consecutive k of one column,
//     laid out [k/4][n]: writes are 16 bytes per lane, contiguous; a lane then
//     reads columns (2j, 2j+1) of four k-quads as 8-byte reads, contiguous
//     across lanes. The k order inside an operand is the same for A and B, which
//     is all an exact integer dot product needs.
//   * A wave owns 64 x 64 of Y as 2 x 2 MFMA tiles; tile t holds columns 2j+t,
//     so a lane stores (col 2j, col 2j+1) of one row as 8 bytes and 32 lanes
//     write 256 contiguous bytes: the 50 MB int32 output (the HBM bound of this
//     op) goes out in full-line bursts.
#include "common.h"
#include "gemm_tile.h"

#include <stdlib.h>
#include <type_traits>
#include <utility>

namespace mi355x {

struct MMIArgs {
    const int8_t* A; const int8_t* B; int32_t* Y;
    int64_t M, N, K;
    const int8_t* za_ptr; const int8_t* zb_ptr;
    int64_t tiles_m, tiles_n, nwg;
    int group_m;  // tile walk order, see tile_coords
};

constexpr int MMI_BM = 128, MMI_BN = 128, MMI_BK = 64;
constexpr int MMI_A_PITCH = MMI_BK + 16;         // bytes per A row in LDS
constexpr int MMI_B_PITCH = MMI_BN + 4;          // words per k-quad row in LDS

typedef int i32x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ uint32_t perm_b32(uint32_t hi, uint32_t lo, uint32_t sel) {
    return __builtin_amdgcn_perm(hi, lo, sel);
}

// r[k] = 4 bytes (columns c..c+3) of row k  ->  o[c] = 4 bytes (rows 0..3) of column c
__device__ __forceinline__ void transpose_4x4_bytes(const uint32_t (&r)[4], uint32_t (&o)[4]) {
    const uint32_t t01_lo = perm_b32(r[1], r[0], 0x05010400u);  // r0b0 r1b0 r0b1 r1b1
    const uint32_t t01_hi = perm_b32(r[1], r[0], 0x07030602u);  // r0b2 r1b2 r0b3 r1b3
    const uint32_t t23_lo = perm_b32(r[3], r[2], 0x05010400u);
    const uint32_t t23_hi = perm_b32(r[3], r[2], 0x07030602u);
    o[0] = perm_b32(t23_lo, t01_lo, 0x05040100u);
    o[1] = perm_b32(t23_lo, t01_lo, 0x07060302u);
    o[2] = perm_b32(t23_hi, t01_hi, 0x05040100u);
    o[3] = perm_b32(t23_hi, t01_hi, 0x07060302u);
}

template <bool VEC>
__global__ __launch_bounds__(256) void matmul_integer_i8_kernel(MMIArgs p) {
    constexpr int BM = MMI_BM, BN = MMI_BN, BK = MMI_BK, NT = 256;
    __shared__ __attribute__((aligned(16))) int8_t lds_a[2][BM * MMI_A_PITCH];
    __shared__ __attribute__((aligned(16))) uint32_t lds_b[2][(BK / 4) * MMI_B_PITCH];
    __shared__ int32_t lds_rowsum[4][64];

    const int tid = threadIdx.x;
    const int lane = tid % WAVE, wave = tid / WAVE;
    const int lj = lane % 32, lg = lane / 32;
    const int wm0 = (wave / 2) * 64, wn0 = (wave % 2) * 64;

    const int64_t logical = xcd_remap(blockIdx.x, p.nwg);
    const int64_t m0 = (logical / p.tiles_n) * BM, n0 = (logical % p.tiles_n) * BN;

    // ---- loaders ----------------------------------------------------------------
    // A: 128 rows x 4 vectors of 16 bytes -> 2 vectors per thread
    // B: 16 k-quads x 32 column groups of 4 -> 2 units (4 rows x 4 cols) per thread
    i32x4 ra[2];
    uint32_t rb[2][4];
    auto load_tiles = [&](int64_t k0) {
#pragma unroll
        for (int it = 0; it < 2; ++it) {
            const int idx = tid + it * NT;
            const int row = idx / 4, c16 = idx % 4;
            const int64_t gm = m0 + row, gk = k0 + 16 * c16;
            i32x4 v = i32x4{0, 0, 0, 0};
            if (gm < p.M) {
                const int8_t* src = p.A + gm * p.K + gk;
                if constexpr (VEC) {
                    if (gk < p.K) v = *reinterpret_cast<const i32x4*>(src);
                } else {
                    uint32_t w[4] = {0, 0, 0, 0};
                    for (int e = 0; e < 16; ++e)
                        if (gk + e < p.K) w[e / 4] |= (uint32_t)(uint8_t)src[e] << (8 * (e % 4));
                    v = i32x4{(int)w[0], (int)w[1], (int)w[2], (int)w[3]};
                }
            }
            ra[it] = v;
        }
#pragma unroll
        for (int it = 0; it < 2; ++it) {
            const int idx = tid + it * NT;
            const int kq = idx / 32, cg = idx % 32;
            const int64_t gn = n0 + 4 * cg;
            uint32_t rows[4];
#pragma unroll
            for (int rr = 0; rr < 4; ++rr) {
                const int64_t gk = k0 + 4 * kq + rr;
                uint32_t w = 0;
                if (gk < p.K) {
                    const int8_t* src = p.B + gk * p.N + gn;
                    if constexpr (VEC) {
                        if (gn < p.N) w = *reinterpret_cast<const uint32_t*>(src);
                    } else {
                        for (int e = 0; e < 4; ++e)
                            if (gn + e < p.N) w |= (uint32_t)(uint8_t)src[e] << (8 * e);
                    }
                }
                rows[rr] = w;
            }
            transpose_4x4_bytes(rows, rb[it]);
        }
    };
    auto store_tiles = [&](int buf) {
#pragma unroll
        for (int it = 0; it < 2; ++it) {
            const int idx = tid + it * NT;
            const int row = idx / 4, c16 = idx % 4;
            *reinterpret_cast<i32x4*>(lds_a[buf] + row * MMI_A_PITCH + 16 * c16) = ra[it];
        }
#pragma unroll
        for (int it = 0; it < 2; ++it) {
            const int idx = tid + it * NT;
            const int kq = idx / 32, cg = idx % 32;
            *reinterpret_cast<i32x4*>(lds_b[buf] + kq * MMI_B_PITCH + 4 * cg) =
                i32x4{(int)rb[it][0], (int)rb[it][1], (int)rb[it][2], (int)rb[it][3]};
        }
    };

    i32x16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][t][r] = 0;
    int32_t rowsum[2] = {0, 0};  // partial: rows wm0+32i+lj, this lane's k half
    int32_t colsum[2] = {0, 0};  // partial: cols wn0+2*lj+t, this lane's k half
    // zero points are device scalars (wave-uniform loads); NULL means 0
    const int32_t za_i = p.za_ptr ? (int32_t)*p.za_ptr : 0, zb_i = p.zb_ptr ? (int32_t)*p.zb_ptr : 0;
    const bool need_rowsum = zb_i != 0, need_colsum = za_i != 0;

    const int64_t ktiles = (p.K + BK - 1) / BK;
    load_tiles(0);
    store_tiles(0);
    __syncthreads();
    for (int64_t kt = 0; kt < ktiles; ++kt) {
        const int buf = (int)(kt & 1);
        if (kt + 1 < ktiles) load_tiles((kt + 1) * BK);
#pragma unroll
        for (int ks = 0; ks < BK / 32; ++ks) {
            // lane (lj, lg): k-quads 8*ks + 4*lg + {0..3} of this 32-k step
            i32x4 af[2], bf[2];
#pragma unroll
            for (int i = 0; i < 2; ++i)
                af[i] = *reinterpret_cast<const i32x4*>(lds_a[buf] + (wm0 + 32 * i + lj) * MMI_A_PITCH +
                                                        32 * ks + 16 * lg);
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const i32x2 w = *reinterpret_cast<const i32x2*>(
                    lds_b[buf] + (8 * ks + 4 * lg + q) * MMI_B_PITCH + wn0 + 2 * lj);
                bf[0][q] = w.x;
                bf[1][q] = w.y;
            }
            if (need_rowsum) {
#pragma unroll
                for (int i = 0; i < 2; ++i)
#pragma unroll
                    for (int q = 0; q < 4; ++q)
                        rowsum[i] = __builtin_amdgcn_sdot4(af[i][q], 0x01010101, rowsum[i], false);
            }
            if (need_colsum) {
#pragma unroll
                for (int t = 0; t < 2; ++t)
#pragma unroll
                    for (int q = 0; q < 4; ++q)
                        colsum[t] = __builtin_amdgcn_sdot4(bf[t][q], 0x01010101, colsum[t], false);
            }
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int t = 0; t < 2; ++t)
                    acc[i][t] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[i], bf[t], acc[i][t], 0, 0, 0);
        }
        if (kt + 1 < ktiles) store_tiles(buf ^ 1);
        __syncthreads();
    }

    // ---- zero-point correction ---------------------------------------------------
    // combine the two k halves (lanes l and l^32)
#pragma unroll
    for (int i = 0; i < 2; ++i) rowsum[i] += __shfl_xor(rowsum[i], 32, WAVE);
#pragma unroll
    for (int t = 0; t < 2; ++t) colsum[t] += __shfl_xor(colsum[t], 32, WAVE);
    // a lane needs the row sums of the 16 rows its accumulator registers hold
    if (lg == 0) {
        lds_rowsum[wave][lj] = rowsum[0];
        lds_rowsum[wave][32 + lj] = rowsum[1];
    }
    __syncthreads();

    const uint32_t za = (uint32_t)za_i, zb = (uint32_t)zb_i;
    const uint32_t kzz = (uint32_t)p.K * za * zb;
    // acc[i][t][r] = Y[m0+wm0+32i + 8*(r/4)+4*lg+(r%4)][n0+wn0+2*lj+t]
    const int64_t n = n0 + wn0 + 2 * lj;
    const uint32_t c0 = kzz - za * (uint32_t)colsum[0], c1 = kzz - za * (uint32_t)colsum[1];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int row_in_tile = 8 * (r / 4) + 4 * lg + (r % 4);
            const int64_t m = m0 + wm0 + 32 * i + row_in_tile;
            if (m >= p.M || n >= p.N) continue;
            const uint32_t rs = zb * (uint32_t)lds_rowsum[wave][32 * i + row_in_tile];
            const int32_t y0 = (int32_t)((uint32_t)acc[i][0][r] - rs + c0);
            const int32_t y1 = (int32_t)((uint32_t)acc[i][1][r] - rs + c1);
            int32_t* dst = p.Y + m * p.N + n;
            if constexpr (VEC) {
                __builtin_nontemporal_store(i32x2{y0, y1}, reinterpret_cast<i32x2*>(dst));
            } else {
                dst[0] = y0;
                if (n + 1 < p.N) dst[1] = y1;
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------
// Persistent, software-pipelined kernel for the aligned case (K % 128 == 0, N % 4 == 0),
// in steps of BK = 64 or 128 along k (the description below is written for 128).
//
// The op is bound by its int32 output (4 M N bytes against M K + K N bytes of input), so
// what matters is that the stores of one tile overlap with the loads and MFMAs of the
// next, and that no workgroup ever sits waiting for its first loads. The grid is at
// most two workgroups per CU; a workgroup walks tiles blockIdx.x, blockIdx.x +
// gridDim.x, ... as ONE stream of 128-k steps: the loads for the first steps of the
// next tile are issued while the last steps of the current tile are multiplied, and a
// finished tile is stored with fire-and-forget stores before the next step starts.
//
// 128 x 128 tile, 4 waves; wave w owns rows 32 w .. 32 w + 31 and all 128 columns as
// 1 x 4 MFMA tiles (tile t holds column 4 lj + t of lane lj, so a lane stores four
// consecutive int32 of one row as 16 bytes).
//   * A never goes through LDS: no two waves share a row, so each lane loads its MFMA
//     operand (16 consecutive k of its row) straight from global memory, three steps
//     ahead.
//   * B goes through LDS k-contiguous per column ([n][k], rows of 128 k + 16 bytes):
//     a loader thread reads 16 k-rows x 4 columns (4-byte loads, 128 contiguous bytes
//     per 32 lanes), transposes 4x4 byte blocks in registers and writes the 16 k of
//     each of its columns as one 16-byte LDS write; a lane's MFMA operand is then one
//     16-byte LDS read. The 16-byte chunk index inside a row is XORed with bits 4..5
//     of the column, which keeps both the writes (lanes 4 columns apart) and the reads
//     free of bank conflicts.
//   * Three LDS buffers, one barrier per step; the B tile of step s + 2 is written while
//     step s is multiplied, operands of the next 32-k sub-step are read ahead of the
//     MFMAs that need them; B rows are loaded five steps ahead, A operands three.
// Measured limits on this part (why the kernel sits near 25 % of the int8 MFMA rate in
// steady state): per 128-k step a workgroup moves 32 KB through the vector L1, writes
// 16 KB to LDS (a 16-byte LDS write costs the CU ~15-20 cycles per wave instruction
// whatever its width) and reads 64 KB from it (~5-7 cycles per 16-byte wave read),
// against 512 cycles of MFMA: the three pipes are each about as busy as the matrix
// core, so the op stays bound by its 4 M N output bytes only for K up to ~1000.
constexpr int MMF_BM = 128, MMF_BN = 128, MMF_STAGES = 3, MMF_RING = 3;

template <int N, class F, int... I>
__device__ __forceinline__ void mmi_static_for_impl(F&& f, std::integer_sequence<int, I...>) {
    (f(std::integral_constant<int, I>{}), ...);
}
// (the lambdas passed in are marked always_inline: a kernel's register arrays must never
// be addressed through memory)
template <int N, class F>
__device__ __forceinline__ void mmi_static_for(F&& f) {
    mmi_static_for_impl<N>(static_cast<F&&>(f), std::make_integer_sequence<int, N>{});
}

// BK = 128: 250 registers, two workgroups per CU. BK = 64: three per CU.
template <int BK>
__global__ __launch_bounds__(256, BK == 128 ? 2 : 3) void matmul_integer_i8_stream_kernel(MMIArgs p) {
    constexpr int BM = MMF_BM, BN = MMF_BN, RING = MMF_RING;
    constexpr int PITCH = BK / 4 + 4;       // words per column row in LDS
    constexpr int STAGE = BN * PITCH;
    constexpr int KS = BK / 32;             // 32-k MFMA sub-steps per step
    constexpr int BROWS = BK / 8;           // k-rows per B loader unit (8 units of 32 threads cover BK)
    constexpr int BW = BROWS / 4;           // words (4 k each) a loader thread holds per column
    __shared__ __attribute__((aligned(16))) uint32_t lds[MMF_STAGES * STAGE];
    __shared__ __attribute__((aligned(16))) int32_t lds_colsum[4][WAVE][4];

    const int tid = threadIdx.x;
    const int lane = tid % WAVE, wave = tid / WAVE;
    const int lj = lane % 32, lg = lane / 32;
    const int kc = tid / 32, c4 = tid % 32;  // B loader unit: k-rows BROWS kc .. + BROWS - 1, columns 4 c4 .. 4 c4 + 3

    const int ktiles = (int)(p.K / BK);
    // tiles of this workgroup: blockIdx.x + i * gridDim.x (gridDim.x is a multiple of 8, so
    // all of them run on this workgroup's XCD and xcd_remap keeps them in its slab)
    const int my_tiles = (int)((p.nwg - blockIdx.x + gridDim.x - 1) / gridDim.x);
    const int total_steps = my_tiles * ktiles;

    // m0 / n0 of this workgroup's i-th tile
    auto tile_origin = [&](int i, int64_t& m0, int64_t& n0) __attribute__((always_inline)) {
        const int64_t logical = xcd_remap((int64_t)blockIdx.x + (int64_t)i * gridDim.x, p.nwg);
        int64_t tm, tn;
        tile_coords(logical, p.tiles_m, p.tiles_n, p.group_m, tm, tn);
        m0 = tm * BM;
        n0 = tn * BN;
    };
    // Load cursors walk the step stream ahead of the MFMAs; past the end they stay on the
    // last step (re-reading cached data) so the loop body has no branches around loads.
    struct Cursor { int tile, kt; const int8_t* ptr; };
    auto a_base = [&](int i) __attribute__((always_inline)) {
        int64_t m0, n0;
        tile_origin(i, m0, n0);
        int64_t am = m0 + 32 * wave + lj;   // row (clamped into the matrix), k = 32 ks + 16 lg + [0, 16)
        am = am < p.M ? am : p.M - 1;
        return p.A + am * p.K + 16 * lg;
    };
    auto b_base = [&](int i) __attribute__((always_inline)) {
        int64_t m0, n0;
        tile_origin(i, m0, n0);
        int64_t bn = n0 + 4 * c4;           // columns clamped as a group of four (N % 4 == 0)
        bn = bn < p.N ? bn : p.N - 4;
        return p.B + (int64_t)(BROWS * kc) * p.N + bn;
    };
    const int64_t a_step = BK, b_step = (int64_t)BK * p.N;
    static_assert(KS % 2 == 0, "operand sets alternate per sub-step across steps");
    Cursor ca{0, 0, a_base(0)}, cb{0, 0, b_base(0)};
    auto advance_a = [&]() __attribute__((always_inline)) {
        if (ca.kt + 1 < ktiles) { ++ca.kt; ca.ptr += a_step; }
        else if (ca.tile + 1 < my_tiles) { ++ca.tile; ca.kt = 0; ca.ptr = a_base(ca.tile); }
    };
    auto advance_b = [&]() __attribute__((always_inline)) {
        if (cb.kt + 1 < ktiles) { ++cb.kt; cb.ptr += b_step; }
        else if (cb.tile + 1 < my_tiles) { ++cb.tile; cb.kt = 0; cb.ptr = b_base(cb.tile); }
    };

    int b_lds[4];
#pragma unroll
    for (int c = 0; c < 4; ++c)
        b_lds[c] = (4 * c4 + c) * PITCH + 4 * ((kc * BW / 4) ^ ((c4 >> 2) & 3)) + (kc * BW) % 4;
    // operand reads: column 4 lj + t, chunk 2 ks + lg (same swizzle: (column >> 4) & 3 == (lj >> 2) & 3)
    const int f_lds = 4 * lj * PITCH, f_swz = (lj >> 2) & 3;

    i32x4 ra[RING][KS];         // A operands of step s in slot s % RING
    uint32_t rb[RING][BROWS];   // raw B rows of step s in slot s % RING
    i32x4 bf[2][4];          // B operands of 32-k sub-step q in set q % 2

    auto load_a = [&](i32x4 (&dst)[KS]) __attribute__((always_inline)) {   // at the A cursor, then advance it
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) dst[ks] = *reinterpret_cast<const i32x4*>(ca.ptr + 32 * ks);
        advance_a();
    };
    auto load_b = [&](uint32_t (&dst)[BROWS]) __attribute__((always_inline)) {
#pragma unroll
        for (int rr = 0; rr < BROWS; ++rr) dst[rr] = *reinterpret_cast<const uint32_t*>(cb.ptr + rr * p.N);
        advance_b();
    };
    auto store_b = [&](const uint32_t (&raw)[BROWS], int stage) __attribute__((always_inline)) {
        uint32_t o[BW][4];  // o[j][c]: column c, k 4 j .. 4 j + 3 of the unit's rows
#pragma unroll
        for (int j = 0; j < BW; ++j) {
            const uint32_t rows[4] = {raw[4 * j], raw[4 * j + 1], raw[4 * j + 2], raw[4 * j + 3]};
            transpose_4x4_bytes(rows, o[j]);
        }
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            if constexpr (BW == 4)
                *reinterpret_cast<i32x4*>(lds + stage * STAGE + b_lds[c]) =
                    i32x4{(int)o[0][c], (int)o[1][c], (int)o[2][c], (int)o[3][c]};
            else
                *reinterpret_cast<i32x2*>(lds + stage * STAGE + b_lds[c]) = i32x2{(int)o[0][c], (int)o[1][c]};
        }
    };
    auto read_b = [&](i32x4 (&dst)[4], int stage, int ks) __attribute__((always_inline)) {
#pragma unroll
        for (int t = 0; t < 4; ++t)
            dst[t] = *reinterpret_cast<const i32x4*>(lds + stage * STAGE + f_lds + t * PITCH + 4 * ((2 * ks + lg) ^ f_swz));
    };

    i32x16 acc[4];
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[t][r] = 0;
    int32_t rowsum = 0;                    // row 32 wave + lj, this lane's k half
    // column 4 lj + t, this lane's k half, and only the sub-steps q with q % 4 == wave: every wave
    // reads the same B operands, so the four waves share the work and add up at the end of the tile
    int32_t colsum[4] = {0, 0, 0, 0};
    const int32_t za_i = p.za_ptr ? (int32_t)*p.za_ptr : 0, zb_i = p.zb_ptr ? (int32_t)*p.zb_ptr : 0;
    const bool need_rowsum = zb_i != 0, need_colsum = za_i != 0;
    const uint32_t za = (uint32_t)za_i, zb = (uint32_t)zb_i;
    const uint32_t kzz = (uint32_t)p.K * za * zb;

    // zero-point correction and 16-byte stores of the finished tile; accumulators restart at 0
    auto finish_tile = [&](int i) __attribute__((always_inline)) {
        int64_t m0, n0;
        tile_origin(i, m0, n0);
        rowsum += __shfl_xor(rowsum, 32, WAVE);
        uint32_t cc[4] = {kzz, kzz, kzz, kzz};
        if (need_colsum) {  // uniform
#pragma unroll
            for (int t = 0; t < 4; ++t) colsum[t] += __shfl_xor(colsum[t], 32, WAVE);
            *reinterpret_cast<i32x4*>(lds_colsum[wave][lane]) = i32x4{colsum[0], colsum[1], colsum[2], colsum[3]};
            __syncthreads();  // the next write to this buffer is at least one step barrier away
            i32x4 sum = *reinterpret_cast<const i32x4*>(lds_colsum[0][lane]);
#pragma unroll
            for (int w = 1; w < 4; ++w) sum += *reinterpret_cast<const i32x4*>(lds_colsum[w][lane]);
#pragma unroll
            for (int t = 0; t < 4; ++t) cc[t] = kzz - za * (uint32_t)sum[t];
        }
        // acc[t][r] = Y[m0 + 32 wave + 8 (r / 4) + 4 lg + r % 4][n0 + 4 lj + t]
        const int64_t n = n0 + 4 * lj;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int row_in_wave = 8 * (r / 4) + 4 * lg + (r % 4);
            const int64_t m = m0 + 32 * wave + row_in_wave;
            // the row sum of that row lives in lane row_in_wave (every lane takes part in the shuffle)
            const uint32_t rs = need_rowsum ? zb * (uint32_t)__shfl(rowsum, row_in_wave, WAVE) : 0u;
            const i32x4 y = i32x4{(int32_t)((uint32_t)acc[0][r] - rs + cc[0]), (int32_t)((uint32_t)acc[1][r] - rs + cc[1]),
                                  (int32_t)((uint32_t)acc[2][r] - rs + cc[2]), (int32_t)((uint32_t)acc[3][r] - rs + cc[3])};
            if (m < p.M && n < p.N) __builtin_nontemporal_store(y, reinterpret_cast<i32x4*>(p.Y + m * p.N + n));
        }
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            colsum[t] = 0;
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[t][r] = 0;
        }
        rowsum = 0;
    };

    // ---- prologue: steps 0..2 in registers, B of steps 0 and 1 in LDS, steps 3 and 4 in flight
#pragma unroll
    for (int r = 0; r < RING; ++r) {
        load_a(ra[r]);
        load_b(rb[r]);
    }
    store_b(rb[0], 0);
    load_b(rb[0]);
    store_b(rb[1], 1);
    load_b(rb[1]);
    __syncthreads();
    read_b(bf[0], 0, 0);

    int kt = 0, tile_i = 0;  // position of the step being multiplied
    auto step = [&](auto r_tag) __attribute__((always_inline)) {
        constexpr int r = decltype(r_tag)::value;
        constexpr int nxt = (r + 2) % RING;
        store_b(rb[nxt], nxt);      // B of step s + 2, into the buffer step s - 1 was read from
        load_b(rb[nxt]);            // B of step s + 5
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            const int cur = ks & 1;
            if (ks + 1 < KS) read_b(bf[cur ^ 1], r, ks + 1);
            else read_b(bf[cur ^ 1], (r + 1) % RING, 0);  // next step's buffer: visible since the last barrier
            if (need_rowsum) {
#pragma unroll
                for (int q = 0; q < 4; ++q) rowsum = __builtin_amdgcn_sdot4(ra[r][ks][q], 0x01010101, rowsum, false);
            }
            if (need_colsum && ((kt * KS + ks) & 3) == wave) {  // uniform
#pragma unroll
                for (int t = 0; t < 4; ++t)
#pragma unroll
                    for (int q = 0; q < 4; ++q) colsum[t] = __builtin_amdgcn_sdot4(bf[cur][t][q], 0x01010101, colsum[t], false);
            }
#pragma unroll
            for (int t = 0; t < 4; ++t)
                acc[t] = __builtin_amdgcn_mfma_i32_32x32x32_i8(ra[r][ks], bf[cur][t], acc[t], 0, 0, 0);
        }
        load_a(ra[r]);              // A of step s + 3
        if (++kt == ktiles) {       // uniform
            finish_tile(tile_i);
            kt = 0;
            ++tile_i;
        }
        __syncthreads();
    };
    for (int s0 = 0; s0 < total_steps; s0 += RING) {
        mmi_static_for<RING>([&](auto r_tag) __attribute__((always_inline)) {
            if (s0 + decltype(r_tag)::value < total_steps) step(r_tag);  // uniform
        });
    }
}

}  // namespace mi355x

extern "C" int mi355x_matmul_integer_i8(const int8_t* A, const int8_t* B,
                                        const int8_t* a_zero_point, const int8_t* b_zero_point,
                                        int32_t* Y, int64_t M, int64_t N, int64_t K, void* stream) {
    using namespace mi355x;
    MI355X_REQUIRE(M >= 0 && N >= 0 && K >= 0, "matmul_integer: negative extent (M=%lld N=%lld K=%lld)",
                   (long long)M, (long long)N, (long long)K);
    if (M == 0 || N == 0) return MI355X_OK;
    MI355X_REQUIRE(A && B && Y, "matmul_integer: null pointer");
    MMIArgs p;
    p.A = A; p.B = B; p.Y = Y; p.M = M; p.N = N; p.K = K;
    p.za_ptr = a_zero_point; p.zb_ptr = b_zero_point;
    p.tiles_m = ceil_div(M, MMI_BM);
    p.tiles_n = ceil_div(N, MMI_BN);
    p.nwg = p.tiles_m * p.tiles_n;
    MI355X_REQUIRE(p.nwg < ((int64_t)1 << 31), "matmul_integer: grid too large");
    auto al = [](const void* q, int a) { return (reinterpret_cast<uintptr_t>(q) & (a - 1)) == 0; };
    // 16-byte A loads need K % 16 == 0; 4-byte B loads need N % 4 == 0; 8-byte Y stores need N % 2 == 0
    const bool vec = (K % 16 == 0) && (N % 4 == 0) && al(A, 16) && al(B, 4) && al(Y, 8);
    hipStream_t st = static_cast<hipStream_t>(stream);
    p.group_m = 1;
    if (vec && K % 128 == 0 && K > 0 && al(Y, 16) && !getenv("MI355X_MMI_GENERIC")) {
        int cus = mi355x_device_cu_count();
        if (cus <= 0) return set_error(MI355X_ERR_NOT_INITIALIZED, "matmul_integer: no usable HIP device");
        // persistent grid: two workgroups per CU (a multiple of the XCD count), fewer if there are fewer tiles
        // 64-k steps fit three workgroups on a CU (measured 22.6 us against 26.4 us with 128-k steps and
        // two workgroups on the 4096 x 3072 x 768 case); MI355X_MMI_BK=128 selects the other variant
        const bool bk64 = !(getenv("MI355X_MMI_BK") && atoi(getenv("MI355X_MMI_BK")) == 128);
        int64_t grid = (bk64 ? 3 : 2) * (int64_t)(cus / NUM_XCD) * NUM_XCD;
        if (const char* g = getenv("MI355X_MMI_WGS_PER_CU")) grid = (int64_t)atoi(g) * (cus / NUM_XCD) * NUM_XCD;
        if (grid > p.nwg || grid <= 0) grid = p.nwg;
        const int64_t per_xcd = ceil_div(p.nwg, (int64_t)NUM_XCD), resident = ceil_div(grid, (int64_t)NUM_XCD);
        p.group_m = choose_group_m(p.tiles_m, per_xcd < resident ? per_xcd : resident, MMF_BM, MMF_BN);
        if (bk64) hipLaunchKernelGGL(matmul_integer_i8_stream_kernel<64>, dim3((unsigned)grid), dim3(256), 0, st, p);
        else hipLaunchKernelGGL(matmul_integer_i8_stream_kernel<128>, dim3((unsigned)grid), dim3(256), 0, st, p);
        return check_launch("matmul_integer_i8_stream_kernel");
    }
    if (vec) hipLaunchKernelGGL(matmul_integer_i8_kernel<true>, dim3((unsigned)p.nwg), dim3(256), 0, st, p);
    else hipLaunchKernelGGL(matmul_integer_i8_kernel<false>, dim3((unsigned)p.nwg), dim3(256), 0, st, p);
    return check_launch("matmul_integer_i8_kernel");
}
