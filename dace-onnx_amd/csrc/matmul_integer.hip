// ONNX MatMulInteger, (u)int8 x (u)int8 -> int32, bit-exact, on the gfx950 int8 matrix cores.
//
// The reference has no expansion of its own for this node: the generated class
// (daceml/onnx/nodes/onnx_op.py:623-640) is only ever expanded through ONNX
// Runtime (onnx_op.py:686-687 -> daceml/onnx/nodes/node_codegen.py:321-573).
//
//   Y[m,n] = sum_k (A[m,k] - za[m])(B[k,n] - zb[n])
//          = sum_k A B  -  zb[n] * rowsum_A[m]  -  za[m] * colsum_B[n]  +  K * za[m] * zb[n]
// The raw product runs on v_mfma_i32_32x32x32_i8; the row/column sums are taken
// with v_dot4_i32_i8 on the very operand registers the MFMA consumes, so the
// zero points cost no extra memory traffic and (a - za) never has to fit in
// int8. All arithmetic is modulo 2^32, the same as an int32 accumulator.
// An unsigned operand u is multiplied as the signed byte u ^ 0x80 = u - 128 with
// its zero point moved by the same 128.
#include "common.h"
#include "gemm_tile.h"

#include <stdlib.h>
#include <type_traits>

namespace mi355x {

struct MMIArgs {
    const int8_t* A; const int8_t* B; int32_t* Y;
    int64_t M, N, K;
    const int8_t* za_ptr; const int8_t* zb_ptr;   // NULL: zero
    int za_stride, zb_stride;                     // 0: one value, 1: one per row of A / per column of B
    int a_unsigned, b_unsigned;
    int64_t tiles_m, tiles_n, nwg;
    int group_m;  // tile walk order, see tile_coords
    MI355X_TRACE_MEMBER
};

typedef int i32x2 __attribute__((ext_vector_type(2)));

// zero point of row m of A / column n of B as the kernels use it: that of the signed bytes they multiply
__device__ __forceinline__ int32_t a_zero_point(const MMIArgs& p, int64_t m) {
    const int32_t bias = p.a_unsigned ? 128 : 0;
    if (!p.za_ptr) return -bias;
    const int64_t i = m * p.za_stride;
    return (p.a_unsigned ? (int32_t)reinterpret_cast<const uint8_t*>(p.za_ptr)[i] : (int32_t)p.za_ptr[i]) - bias;
}
__device__ __forceinline__ int32_t b_zero_point(const MMIArgs& p, int64_t n) {
    const int32_t bias = p.b_unsigned ? 128 : 0;
    if (!p.zb_ptr) return -bias;
    const int64_t i = n * p.zb_stride;
    return (p.b_unsigned ? (int32_t)reinterpret_cast<const uint8_t*>(p.zb_ptr)[i] : (int32_t)p.zb_ptr[i]) - bias;
}

// ---------------------------------------------------------------------------------------------
// Any shape and alignment: 128 x 128 tile, register-staged loads, B transposed with byte permutes.
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
//     so a lane stores (col 2j, col 2j+1) of one row as 8 bytes.
constexpr int MMI_BM = 128, MMI_BN = 128, MMI_BK = 64;
constexpr int MMI_A_PITCH = MMI_BK + 16;         // bytes per A row in LDS
constexpr int MMI_B_PITCH = MMI_BN + 4;          // words per k-quad row in LDS

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
    // unsigned bytes become signed ones (u ^ 0x80 = u - 128) as they are loaded; bytes outside the matrix stay 0,
    // so a padded k adds 0 to the product and to both sums
    const uint32_t a_flip = p.a_unsigned ? 0x80808080u : 0u, b_flip = p.b_unsigned ? 0x80808080u : 0u;

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
                    if (gk < p.K) v = *reinterpret_cast<const i32x4*>(src) ^ (int)a_flip;
                } else {
                    uint32_t w[4] = {0, 0, 0, 0};
                    for (int e = 0; e < 16; ++e)
                        if (gk + e < p.K) w[e / 4] |= (uint32_t)((uint8_t)src[e] ^ (uint8_t)a_flip) << (8 * (e % 4));
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
                        if (gn < p.N) w = *reinterpret_cast<const uint32_t*>(src) ^ b_flip;
                    } else {
                        for (int e = 0; e < 4; ++e)
                            if (gn + e < p.N) w |= (uint32_t)((uint8_t)src[e] ^ (uint8_t)b_flip) << (8 * e);
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
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int q = 0; q < 4; ++q)
                    rowsum[i] = __builtin_amdgcn_sdot4(af[i][q], 0x01010101, rowsum[i], false);
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int q = 0; q < 4; ++q)
                    colsum[t] = __builtin_amdgcn_sdot4(bf[t][q], 0x01010101, colsum[t], false);
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

    // acc[i][t][r] = Y[m0+wm0+32i + 8*(r/4)+4*lg+(r%4)][n0+wn0+2*lj+t]
    const int64_t n = n0 + wn0 + 2 * lj;
    uint32_t zbn[2], c2[2];   // zero point of the lane's two columns; colsum - K zb
#pragma unroll
    for (int t = 0; t < 2; ++t) {
        zbn[t] = n + t < p.N ? (uint32_t)b_zero_point(p, n + t) : 0u;
        c2[t] = (uint32_t)colsum[t] - (uint32_t)p.K * zbn[t];
    }
#pragma unroll
    for (int i = 0; i < 2; ++i) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int row_in_tile = 8 * (r / 4) + 4 * lg + (r % 4);
            const int64_t m = m0 + wm0 + 32 * i + row_in_tile;
            if (m >= p.M || n >= p.N) continue;
            const uint32_t rs = (uint32_t)lds_rowsum[wave][32 * i + row_in_tile];
            const uint32_t zam = (uint32_t)a_zero_point(p, m);
            const int32_t y0 = (int32_t)((uint32_t)acc[i][0][r] - zbn[0] * rs - zam * c2[0]);
            const int32_t y1 = (int32_t)((uint32_t)acc[i][1][r] - zbn[1] * rs - zam * c2[1]);
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
// Aligned shapes (K % 64 == 0, N % 16 == 0, 16-byte aligned pointers): persistent kernel, three workgroups
// per CU, each walking its 128 x 128 tiles as one stream of 64-k steps.
//
// What bounds this operator on the part, measured: a 50 MB int32 result takes ~9 us to store however the stores
// are shaped (5.6 TB/s), and the vector memory pipe of a CU accepts one cache line per cycle per four lanes: an
// operand load whose four neighbouring lanes touch four different lines (A rows read straight into the MFMA
// layout, 32 rows x 32 bytes per instruction) costs 64 cycles per wave instruction, a 4-byte-per-lane load of
// B rows 13 cycles per 256 bytes, a fully coalesced 16-byte-per-lane load 20 cycles per KB. So both operands
// are fetched with coalesced 16-byte loads that write straight into LDS (global_load_lds_dwordx4: no staging
// registers, no LDS write instructions), and the MFMA layouts are produced on the LDS read side:
//   * A stage [128 rows][64 k]: the 16-byte chunk c of row r lives in slot c ^ ((r >> 2) & 3) of the row, so
//     the 16 rows a quarter-wave reads together fall into distinct banks (a lane's operand is one 16-byte read).
//   * B stage [64 k][128 columns] as it is in memory, 16-byte chunk c of k-row k in slot c ^ (2 ((k >> 1) & 3));
//     the k-contiguous operand comes from the transposing LDS read (ds_read_b64_tr_b8: within 16 lanes, result
//     byte j of lane i is byte i % 8 of the 8 bytes addressed by lane 2 j + i / 8), two per 16-byte operand.
//   * 4 waves as 2 x 2 of 64 x 64 (2 x 2 MFMA tiles); MFMA tile t holds columns 32 t + lane % 32, so a store
//     instruction writes two rows of 128 contiguous bytes (4-byte stores of that shape drain exactly as fast as
//     16-byte ones: the stores are bound by HBM, not by instruction count).
//   * Three LDS stages; the transfer of step s + 2 is issued at the top of step s and awaited at its end, one
//     barrier per step, operands of the next 32-k sub-step are read ahead of the MFMAs of the current one.
//   * Row sums of A are needed by both waves of a wave row, column sums of B by both of a wave column: each
//     wave sums one of its two A operands and one of its two B operands and the results meet in LDS.
// The transfers are written as assembly: through the builtin the compiler would wait for vmcnt(0) before every
// LDS read that follows one. Completion is tracked by hand (each thread issues 4 transfers per step).
constexpr int MMF_BM = 128, MMF_BN = 128, MMF_BK = 64, MMF_STAGES = 3;
constexpr int MMF_A_STAGE = MMF_BM * MMF_BK, MMF_B_STAGE = MMF_BK * MMF_BN, MMF_STAGE = MMF_A_STAGE + MMF_B_STAGE;

__device__ __forceinline__ i32x2 lds_read_tr8(const uint8_t* p) {
    return __builtin_amdgcn_ds_read_tr8_b64_v2i32((__attribute__((address_space(3))) i32x2*)(p));
}
// 16 bytes per lane from global memory (base + offset: a wave-uniform pointer in scalar registers and the lane's
// 32-bit byte offset) into LDS at lds_addr + 16 * lane (lds_addr is wave-uniform). The form matters: with a 64-bit
// address per lane the same transfer occupies the CU's address path three to five times as long (measured next to
// an MFMA stream: about 50 to 80 cycles per instruction against 16, which is the 64 bytes per cycle of the L1).
__device__ __forceinline__ void global_to_lds_16(const int8_t* base, uint32_t offset, uint32_t lds_addr) {
    // the pointer is wave-uniform by construction; saying so keeps it in scalar registers whatever the compiler can prove
    // (a no-op where it already holds it there)
    const uint64_t b64 = reinterpret_cast<uint64_t>(base);
    base = reinterpret_cast<const int8_t*>(((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(b64 >> 32)) << 32) |
                                           (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)b64));
    lds_addr = (uint32_t)__builtin_amdgcn_readfirstlane((int)lds_addr);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_addr), "v"(offset), "s"(base) : "memory", "m0");
}
__device__ __forceinline__ uint32_t lds_address(const void* p) {
    return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const void*)p;
}
// s_waitcnt vmcnt(n) alone: vmcnt[3:0] | expcnt[6:4] | lgkmcnt[11:8] | vmcnt[5:4] in bits 15:14
#define MI355X_WAIT_VMCNT(n) __builtin_amdgcn_s_waitcnt(((n) & 0xF) | (((n) >> 4) << 14) | (0x7 << 4) | (0xF << 8))

template <bool ZP, bool AU, bool BU>
__global__ __launch_bounds__(256, (AU && BU) ? 2 : 3) void matmul_integer_i8_stream_kernel(MMIArgs p) {
    constexpr int BM = MMF_BM, BN = MMF_BN, BK = MMF_BK, STAGES = MMF_STAGES, STAGE = MMF_STAGE, A_STAGE = MMF_A_STAGE;
    __shared__ __attribute__((aligned(1024))) uint8_t lds[STAGES * STAGE];
    __shared__ __attribute__((aligned(16))) int32_t lds_rows[2][2][2][64];   // [tile parity][wave row][summed by wave column][row]
    __shared__ int32_t lds_cols[2][2][2][64];   // [tile parity][wave column][summed by wave row][column]
    const int tid = threadIdx.x;
    const int lane = tid % WAVE;
    const int wave = __builtin_amdgcn_readfirstlane(tid / WAVE);
    const int lj = lane % 32, lg = lane / 32;
    const int wm = wave / 2, wn = wave % 2;
    const int wm0 = wm * 64, wn0 = wn * 64;

    MI355X_TRACE_STAMP(p, 0);
    MI355X_TRACE_HWID(p);
    const int ktiles = (int)(p.K / BK);
    // tiles of this workgroup: blockIdx.x + i * gridDim.x (gridDim.x is a multiple of 8 or the whole tile
    // count, so all of them run on this workgroup's XCD and xcd_remap keeps them in its slab)
    const int my_tiles = (int)((p.nwg - blockIdx.x + gridDim.x - 1) / gridDim.x);
    const int total_steps = my_tiles * ktiles;

    auto tile_origin = [&](int i, int64_t& m0, int64_t& n0) __attribute__((always_inline)) {
        const int64_t logical = xcd_remap((int64_t)blockIdx.x + (int64_t)i * gridDim.x, p.nwg);
        int64_t tm, tn;
        tile_coords(logical, p.tiles_m, p.tiles_n, p.group_m, tm, tn);
        m0 = tm * BM;
        n0 = tn * BN;
    };

    // ---- loader: per step and thread two 16-byte chunks of A and two of B
    //   A: instruction j of wave w fills rows 16 (2 w + j) .. + 15: lane i -> row + i / 4, slot i % 4
    //   B: instruction j of wave w fills k-rows 8 (2 w + j) .. + 7: lane i -> row + i / 8, slot i % 8
    // Rows past M and columns past N are clamped into the matrix (what they produce is never stored).
    const int a_row = lane / 4, a_chunk = (lane % 4) ^ ((lane >> 4) & 3);
    const int b_row = lane / 8, b_chunk = (lane % 8) ^ (2 * ((lane >> 4) & 3));
    // (a tile's operands as a wave-uniform pointer to its first element plus 32-bit offsets: 127 K + 48 and
    // 63 N + 112 at most, launch preconditions keep them below 2^31)
    const int64_t b_step = (int64_t)BK * p.N;
    struct Cursor { int tile, kt; const int8_t* a_base; const int8_t* b_base; uint32_t a[2], b[2]; } cur;
    auto set_tile = [&](int i) __attribute__((always_inline)) {
        int64_t m0, n0;
        tile_origin(i, m0, n0);
        int64_t bn = n0 + 16 * b_chunk;
        bn = bn < p.N ? bn : p.N - 16;
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            int64_t am = m0 + 16 * (2 * wave + j) + a_row;
            am = am < p.M ? am : p.M - 1;
            cur.a[j] = (uint32_t)((am - m0) * p.K) + 16u * (uint32_t)a_chunk;
            cur.b[j] = (uint32_t)(8 * (2 * wave + j) + b_row) * (uint32_t)p.N + (uint32_t)(bn - n0);
        }
        cur.a_base = p.A + m0 * p.K;
        cur.b_base = p.B + n0;
        cur.tile = i;
        cur.kt = 0;
    };
    const uint32_t lds_base = lds_address(lds);
    set_tile(0);
    auto issue_loads = [&](int stage) __attribute__((always_inline)) {
        const uint32_t sa = lds_base + stage * STAGE + 1024 * (2 * wave), sb = sa + A_STAGE;
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            global_to_lds_16(cur.a_base, cur.a[j], sa + 1024 * j);
            global_to_lds_16(cur.b_base, cur.b[j], sb + 1024 * j);
        }
        if (cur.kt + 1 < ktiles) {
            ++cur.kt;
            cur.a_base += BK;
            cur.b_base += b_step;
        } else if (cur.tile + 1 < my_tiles) {
            set_tile(cur.tile + 1);
        }
    };

    // ---- operand reads
    // A operand i: row wm0 + 32 i + lj, chunk 2 ks + lg; (2 ks + lg) ^ s = (lg ^ s) ^ 2 ks for a swizzle s < 4,
    // so the sub-step enters as an XOR of the byte address with 32 ks
    int a_off[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int row = wm0 + 32 * i + lj;
        a_off[i] = row * BK + 16 * (lg ^ ((row >> 2) & 3));
    }
    // B operand t: columns wn0 + 32 t + lane % 32; lane i16 of a group of 16 addresses k-row 32 ks + 16 lg +
    // i16 / 2 (+ 8 for the second read), 8 columns from 16 (lane / 16 % 2) + 8 (i16 % 2)
    const int i16 = lane & 15, half = (lane >> 4) & 1;
    const int rib = i16 >> 1;
    int b_off[2];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
        const int cc = (wn0 + 32 * t) / 16 + half;
        b_off[t] = 1024 * (2 * lg) + 16 * (8 * rib + (cc ^ (2 * ((rib >> 1) & 3)))) + 8 * (i16 & 1);
    }

    i32x16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][t][r] = 0;
    // this wave sums its A operands in the sub-steps ks == wn and its B operands in the sub-steps ks == wm (the
    // wave next to it takes the others), its lane's k half
    int32_t rowsum[2] = {0, 0}, colsum[2] = {0, 0};

    i32x4 fa[2][2], fb[2][2];
    auto read_frags = [&](int set, int stage, int ks) __attribute__((always_inline)) {
        const uint8_t* sa = lds + stage * STAGE;
        const uint8_t* sb = sa + A_STAGE;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            fa[set][i] = *reinterpret_cast<const i32x4*>(sa + (a_off[i] ^ (32 * ks)));
            if constexpr (AU) fa[set][i] ^= (int)0x80808080u;
        }
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const i32x2 lo = lds_read_tr8(sb + 4096 * ks + b_off[t]);
            const i32x2 hi = lds_read_tr8(sb + 4096 * ks + 1024 + b_off[t]);
            fb[set][t] = i32x4{lo[0], lo[1], hi[0], hi[1]};
            if constexpr (BU) fb[set][t] ^= (int)0x80808080u;
        }
    };
    auto multiply = [&](auto ks_tag) __attribute__((always_inline)) {
        constexpr int ks = decltype(ks_tag)::value;   // operand set ks holds sub-step ks
        if constexpr (ZP) {
            if (wn == ks) {   // wave-uniform
#pragma unroll
                for (int i = 0; i < 2; ++i)
#pragma unroll
                    for (int q = 0; q < 4; ++q) rowsum[i] = __builtin_amdgcn_sdot4(fa[ks][i][q], 0x01010101, rowsum[i], false);
            }
            if (wm == ks) {
#pragma unroll
                for (int t = 0; t < 2; ++t)
#pragma unroll
                    for (int q = 0; q < 4; ++q) colsum[t] = __builtin_amdgcn_sdot4(fb[ks][t][q], 0x01010101, colsum[t], false);
            }
        }
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int t = 0; t < 2; ++t) acc[i][t] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[ks][i], fb[ks][t], acc[i][t], 0, 0, 0);
    };
    auto publish_sums = [&](int parity) __attribute__((always_inline)) {
        if constexpr (ZP) {
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                const int32_t r = rowsum[i] + __shfl_xor(rowsum[i], 32, WAVE), c = colsum[i] + __shfl_xor(colsum[i], 32, WAVE);
                if (lg == 0) {
                    lds_rows[parity][wm][wn][32 * i + lj] = r;
                    lds_cols[parity][wn][wm][32 * i + lj] = c;
                }
                rowsum[i] = 0;
                colsum[i] = 0;
            }
        }
    };
    // zero points when there is one value per operand (read once, wave-uniform)
    // First zero point of each operand, as the aligned 32-bit word that holds it: loaded behind the first operand transfers (below) and
    // not looked at before the first tile is finished, so the load (a cold page, typically) never stalls the
    // pipeline's start. A missing zero point reads a byte of the operand instead (any valid address).
    uint32_t za_raw = 0u, zb_raw = 0u;

    // Y = acc - zb[n] rowsum[m] - za[m] (colsum[n] - K zb[n]); accumulators restart at 0
    auto finish_tile = [&](int ti) __attribute__((always_inline)) {
        int64_t m0, n0;
        tile_origin(ti, m0, n0);
        const int parity = ti & 1;
        // the tile's rows as a raw buffer: stores past the last row fall outside it and are dropped, columns
        // past N are dropped through offset bit 31 (128 rows of N int32 stay below 2^31 bytes: launch precondition)
        const int64_t rows_left = p.M - m0 < BM ? p.M - m0 : BM;
        const __amdgpu_buffer_rsrc_t y_rsrc =
            __builtin_amdgcn_make_buffer_rsrc(p.Y + m0 * p.N + n0, 0, (int)((rows_left * p.N - n0) * 4), 0x00020000);
        const bool one_each = p.za_stride == 0 && p.zb_stride == 0;   // wave-uniform
        uint32_t za_one = 0u, zb_one = 0u;
        if constexpr (ZP) {
            asm volatile("" : "+v"(za_raw), "+v"(zb_raw));   // keeps the conversion (and the wait for the load) here
            const int32_t a_bias = AU ? 128 : 0, b_bias = BU ? 128 : 0;
            const uint32_t za_byte = (za_raw >> (8 * (reinterpret_cast<uintptr_t>(p.za_ptr) & 3))) & 0xffu;
            const uint32_t zb_byte = (zb_raw >> (8 * (reinterpret_cast<uintptr_t>(p.zb_ptr) & 3))) & 0xffu;
            za_one = (uint32_t)((p.za_ptr ? (AU ? (int32_t)za_byte : (int32_t)(int8_t)za_byte) : 0) - a_bias);
            zb_one = (uint32_t)((p.zb_ptr ? (BU ? (int32_t)zb_byte : (int32_t)(int8_t)zb_byte) : 0) - b_bias);
        }
        const uint32_t row_bytes = (uint32_t)p.N * 4u;
        uint32_t voff[2], zbn[2] = {0u, 0u}, c2[2] = {0u, 0u};
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const int col = wn0 + 32 * t + lj;
            const bool inside = n0 + col < p.N;
            voff[t] = (uint32_t)(wm0 + 4 * lg) * row_bytes + (inside ? (uint32_t)col * 4u : 0x80000000u);
            if constexpr (ZP) {
                zbn[t] = p.zb_stride == 0 ? zb_one : (inside ? (uint32_t)b_zero_point(p, n0 + col) : 0u);
                c2[t] = (uint32_t)(lds_cols[parity][wn][0][32 * t + lj] + lds_cols[parity][wn][1][32 * t + lj]) - (uint32_t)p.K * zbn[t];
            }
        }
        // 32-bit integer multiplies run at a quarter of the rate of adds: with one zero point per operand the
        // correction of an element is two subtractions, y = acc - zb rowsum[m] - za (colsum[n] - K zb)
        uint32_t d_col[2] = {0u, 0u};
        if constexpr (ZP) {
#pragma unroll
            for (int t = 0; t < 2; ++t) d_col[t] = za_one * c2[t];
        }
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            int32_t za_lane = 0;   // zero point of row wm0 + 32 i + lj when there is one per row
            if constexpr (ZP) {
                if (p.za_stride != 0) {
                    const int64_t m = m0 + wm0 + 32 * i + lj;
                    za_lane = a_zero_point(p, m < p.M ? m : p.M - 1);
                }
            }
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                // row sums of the four rows 32 i + 8 q + 4 lg + e that registers 4 q + e hold
                i32x4 rs4 = {};
                if constexpr (ZP)
                    rs4 = *reinterpret_cast<const i32x4*>(&lds_rows[parity][wm][0][32 * i + 8 * q + 4 * lg]) +
                          *reinterpret_cast<const i32x4*>(&lds_rows[parity][wm][1][32 * i + 8 * q + 4 * lg]);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int r = 4 * q + e;
                    const uint32_t roff = (uint32_t)(32 * i + 8 * q + e) * row_bytes;
                    uint32_t y[2] = {(uint32_t)acc[i][0][r], (uint32_t)acc[i][1][r]};
                    if constexpr (ZP) {
                        const uint32_t rs = (uint32_t)rs4[e];
                        if (one_each) {
                            const uint32_t e_row = zb_one * rs;
#pragma unroll
                            for (int t = 0; t < 2; ++t) y[t] = y[t] - e_row - d_col[t];
                        } else {
                            const uint32_t zam = p.za_stride == 0 ? za_one : (uint32_t)__shfl(za_lane, 8 * q + 4 * lg + e, WAVE);
#pragma unroll
                            for (int t = 0; t < 2; ++t) y[t] = y[t] - zbn[t] * rs - zam * c2[t];
                        }
                    }
#pragma unroll
                    for (int t = 0; t < 2; ++t) {
                        __builtin_amdgcn_raw_buffer_store_b32((int32_t)y[t], y_rsrc, (int)(voff[t] + roff), 0, 0);
                        acc[i][t][r] = 0;
                    }
                }
            }
        }
    };

    // ---- software pipeline. At the top of step s: stages s and s + 1 are in LDS and visible to every wave,
    // operand set 0 holds (stage s, first 32 k). A stage is overwritten two steps after it was read.
    issue_loads(0);
    if (total_steps > 1) issue_loads(1);
    if constexpr (ZP) {
        // (the aligned word that holds the byte: no conversion instruction, hence no wait, at this point)
        za_raw = *reinterpret_cast<const uint32_t*>(reinterpret_cast<uintptr_t>(p.za_ptr ? p.za_ptr : p.A) & ~(uintptr_t)3);
        zb_raw = *reinterpret_cast<const uint32_t*>(reinterpret_cast<uintptr_t>(p.zb_ptr ? p.zb_ptr : p.B) & ~(uintptr_t)3);
        MI355X_WAIT_VMCNT(2);   // operations complete in order: the transfers have landed, these two loads may not have
    } else {
        MI355X_WAIT_VMCNT(0);
    }
    __syncthreads();
    MI355X_TRACE_STAMP(p, 1);   // the first operands are in LDS
    MI355X_TRACE_CYCLES(p, 12);
    read_frags(0, 0, 0);

    int kt = 0, tile_i = 0, stage = 0;
    bool pending = false;   // the tile that ended with the previous step still has to be stored
    for (int s = 0; s < total_steps; ++s) {
        const int stage1 = stage + 1 == STAGES ? 0 : stage + 1;
        const int stage2 = stage1 + 1 == STAGES ? 0 : stage1 + 1;
        if (s + 2 < total_steps) issue_loads(stage2);
        const bool stored = pending;
        if (pending) {   // its sums are in LDS since that step's barrier
            finish_tile(tile_i - 1);
            pending = false;
        }
        read_frags(1, stage, 1);
        multiply(std::integral_constant<int, 0>{});
        read_frags(0, stage1, 0);
        multiply(std::integral_constant<int, 1>{});
        // the transfers of this step have to land before the barrier. Memory operations complete in order and
        // the tile's 64 stores were issued after them: once at most 63 operations are outstanding the transfers
        // are among the completed ones, without waiting for the stores to drain.
        if (stored) MI355X_WAIT_VMCNT(63);
        else MI355X_WAIT_VMCNT(0);
        if (++kt == ktiles) {
            publish_sums(tile_i & 1);
            pending = true;
            kt = 0;
            ++tile_i;
        }
        __syncthreads();
        stage = stage1;
    }
    MI355X_TRACE_STAMP(p, 2);
    MI355X_TRACE_CYCLES(p, 13);
    if (pending) finish_tile(tile_i - 1);
#ifdef MI355X_WG_TRACE
    if (p.trace) MI355X_WAIT_VMCNT(0);   // slot 3: the last store is acknowledged
#endif
    MI355X_TRACE_STAMP(p, 3);
}

template <bool ZP>
static void launch_stream(const MMIArgs& p, int64_t grid, hipStream_t st) {
    const dim3 g((unsigned)grid), b(256);
    if (p.a_unsigned) {
        if (p.b_unsigned) hipLaunchKernelGGL((matmul_integer_i8_stream_kernel<true, true, true>), g, b, 0, st, p);
        else hipLaunchKernelGGL((matmul_integer_i8_stream_kernel<true, true, false>), g, b, 0, st, p);
    } else if (p.b_unsigned) {
        hipLaunchKernelGGL((matmul_integer_i8_stream_kernel<true, false, true>), g, b, 0, st, p);
    } else {
        hipLaunchKernelGGL((matmul_integer_i8_stream_kernel<ZP, false, false>), g, b, 0, st, p);
    }
}

}  // namespace mi355x

extern "C" int mi355x_matmul_integer(const void* A, const void* B, const void* a_zero_point, const void* b_zero_point,
                                     int32_t* Y, int64_t M, int64_t N, int64_t K, int a_unsigned, int b_unsigned,
                                     int64_t a_zero_point_count, int64_t b_zero_point_count, void* stream) {
    using namespace mi355x;
    MI355X_REQUIRE(M >= 0 && N >= 0 && K >= 0, "matmul_integer: negative extent (M=%lld N=%lld K=%lld)",
                   (long long)M, (long long)N, (long long)K);
    MI355X_REQUIRE(!a_zero_point || a_zero_point_count == 1 || a_zero_point_count == M,
                   "matmul_integer: a_zero_point holds %lld values, expected 1 or M=%lld", (long long)a_zero_point_count, (long long)M);
    MI355X_REQUIRE(!b_zero_point || b_zero_point_count == 1 || b_zero_point_count == N,
                   "matmul_integer: b_zero_point holds %lld values, expected 1 or N=%lld", (long long)b_zero_point_count, (long long)N);
    if (M == 0 || N == 0) return MI355X_OK;
    MI355X_REQUIRE(A && B && Y, "matmul_integer: null pointer");
    MMIArgs p;
    p.A = static_cast<const int8_t*>(A); p.B = static_cast<const int8_t*>(B); p.Y = Y; p.M = M; p.N = N; p.K = K;
    p.za_ptr = static_cast<const int8_t*>(a_zero_point); p.zb_ptr = static_cast<const int8_t*>(b_zero_point);
    p.za_stride = a_zero_point && a_zero_point_count != 1 ? 1 : 0;
    p.zb_stride = b_zero_point && b_zero_point_count != 1 ? 1 : 0;
    p.a_unsigned = a_unsigned != 0; p.b_unsigned = b_unsigned != 0;
    p.tiles_m = ceil_div(M, MMI_BM);
    p.tiles_n = ceil_div(N, MMI_BN);
    p.nwg = p.tiles_m * p.tiles_n;
    MI355X_REQUIRE(p.nwg < ((int64_t)1 << 31), "matmul_integer: grid too large");
    auto al = [](const void* q, int a) { return (reinterpret_cast<uintptr_t>(q) & (a - 1)) == 0; };
    hipStream_t st = static_cast<hipStream_t>(stream);
    p.group_m = 1;
    MI355X_TRACE_INIT(p);
    const Tuning tune = tuning();

    const int cus = device_cus();
    // 16-byte transfers of A rows and B rows; a tile's 128 rows of Y are addressed with 31-bit byte offsets
    if (K > 0 && K % MMF_BK == 0 && N % 16 == 0 && al(A, 16) && al(B, 16) && al(Y, 4) && N < ((int64_t)1 << 21) &&
        K < ((int64_t)1 << 24) && !tune.mmi_generic) {
        if (cus <= 0) return set_error(MI355X_ERR_NOT_INITIALIZED, "matmul_integer: no usable HIP device");
        // persistent grid: three workgroups per CU (a multiple of the XCD count), fewer if there are fewer tiles
        int64_t grid = (int64_t)(tune.mmi_wgs_per_cu > 0 ? tune.mmi_wgs_per_cu : 3) * (cus / NUM_XCD) * NUM_XCD;
        if (grid > p.nwg || grid <= 0) grid = p.nwg;
        const int64_t per_xcd = ceil_div(p.nwg, (int64_t)NUM_XCD), resident = ceil_div(grid, (int64_t)NUM_XCD);
        p.group_m = choose_group_m(p.tiles_m, per_xcd < resident ? per_xcd : resident, MMF_BM, MMF_BN);
        if (a_zero_point || b_zero_point) launch_stream<true>(p, grid, st);
        else launch_stream<false>(p, grid, st);
        return check_launch("matmul_integer_i8_stream_kernel");
    }
    // 16-byte A loads need K % 16 == 0; 4-byte B loads need N % 4 == 0; 8-byte Y stores need N % 2 == 0
    const bool vec = (K % 16 == 0) && (N % 4 == 0) && al(A, 16) && al(B, 4) && al(Y, 8);
    if (vec) hipLaunchKernelGGL(matmul_integer_i8_kernel<true>, dim3((unsigned)p.nwg), dim3(256), 0, st, p);
    else hipLaunchKernelGGL(matmul_integer_i8_kernel<false>, dim3((unsigned)p.nwg), dim3(256), 0, st, p);
    return check_launch("matmul_integer_i8_kernel");
}

extern "C" int mi355x_matmul_integer_i8(const int8_t* A, const int8_t* B,
                                        const int8_t* a_zero_point, const int8_t* b_zero_point,
                                        int32_t* Y, int64_t M, int64_t N, int64_t K, void* stream) {
    return mi355x_matmul_integer(A, B, a_zero_point, b_zero_point, Y, M, N, K, 0, 0, 1, 1, stream);
}
