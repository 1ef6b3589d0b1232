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
#include <utility>

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

template <class F, int... I>
__device__ __forceinline__ void mmi_static_for_impl(F&& f, std::integer_sequence<int, I...>) {
    (f(std::integral_constant<int, I>{}), ...);
}
// f(integral_constant<0>) ... f(integral_constant<N-1>)
template <int N, class F>
__device__ __forceinline__ void mmi_static_for(F&& f) {
    mmi_static_for_impl(static_cast<F&&>(f), std::make_integer_sequence<int, N>{});
}

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
        // (the aligned word that holds the byte; written as assembly like the transfers, so that exactly two vector
        // memory operations follow them whatever the compiler would have selected for a wave-uniform address)
        const uint32_t* za_word = reinterpret_cast<const uint32_t*>(reinterpret_cast<uintptr_t>(p.za_ptr ? p.za_ptr : p.A) & ~(uintptr_t)3);
        const uint32_t* zb_word = reinterpret_cast<const uint32_t*>(reinterpret_cast<uintptr_t>(p.zb_ptr ? p.zb_ptr : p.B) & ~(uintptr_t)3);
        const uint32_t zero = 0u;
        asm volatile("global_load_dword %0, %1, %2" : "=v"(za_raw) : "v"(zero), "s"(za_word) : "memory");
        asm volatile("global_load_dword %0, %1, %2" : "=v"(zb_raw) : "v"(zero), "s"(zb_word) : "memory");
        // operations complete in order: with at most these 2 outstanding the transfers have landed. The two values are first
        // looked at in finish_tile, behind its own fence and at least one wait of the loop (vmcnt(0), or vmcnt(63) with 64
        // stores issued after them).
        MI355X_WAIT_VMCNT(2);
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

// ---------------------------------------------------------------------------------------------
// The same data path with one tile per workgroup and a loop the compiler can count: waves in a WAVES_M x WAVES_N
// grid, a wave multiplies 64 rows x 32 TNF columns (2 x 2 waves and TNF = 2: 128 x 128 tiles, three workgroups
// per CU; 4 x 2 waves and TNF = 3: 256 x 192 tiles, one workgroup per CU). What differs from the persistent kernel
// above is the shape of the code, not of the data: the K loop is unrolled over the NS LDS stages, so every LDS
// address is a register set up before the loop plus an immediate (no vector arithmetic per step besides the
// zero-point sums), the loop body has no tile bookkeeping in it, and the result is stored once, behind the loop.
// The compiler's s_waitcnt for the operand reads is then a count (the reads of the next sub-step stay in flight
// under the current one's MFMAs) instead of the wait for everything it falls back to in a loop with the stores inside.
constexpr int mmt_b_swizzle(int krow, int pos, int cpr) {
    return cpr == 8 ? pos ^ (2 * ((krow >> 1) & 3)) : pos ^ (((krow >> 2) & 1) | (((krow >> 4) & 1) << 1));
}

template <bool ZP, bool AU, bool BU, int WAVES_M, int WAVES_N, int TNF, int NS, bool A_DIRECT = false>
__global__ __launch_bounds__(64 * WAVES_M * WAVES_N, WAVES_M * WAVES_N == 4 ? ((AU && BU) ? 2 : 3) : 1) void matmul_integer_i8_tile_kernel(MMIArgs p) {
    constexpr int BM = 64 * WAVES_M, BN = 32 * TNF * WAVES_N, BK = 64;
    constexpr int A_STAGE = A_DIRECT ? 0 : BM * BK, STAGE = A_STAGE + BK * BN, NW = WAVES_M * WAVES_N;
    constexpr int CPR = BN / 16;                              // 16-byte chunks of a B row
    constexpr int NA = A_DIRECT ? 0 : BM / 16, NT = NA + BN / 16;            // transfer instructions of a step: 1 KB each, A first
    constexpr int PER_WAVE = (NT + NW - 1) / NW;
    static_assert(WAVES_N == 2, "row sums are shared by the two waves of a wave row, one sub-step each");
    static_assert(WAVES_M == 2 || WAVES_M == 4, "column sums are shared by the waves of a wave column, one sub-step in WAVES_M each");
    static_assert(CPR == 8 || CPR == 12, "swizzle of the B stage");
    static_assert(NS >= 3, "a stage is overwritten NS - 1 steps after it was read");
    __shared__ __attribute__((aligned(1024))) uint8_t lds[NS * STAGE];
    __shared__ __attribute__((aligned(16))) int32_t lds_rows[WAVES_M][2][64];   // [wave row][summed by wave column][row]
    __shared__ int32_t lds_cols[WAVES_N][WAVES_M][32 * TNF];                    // [wave column][summed by wave row][column]
    const int tid = threadIdx.x;
    const int lane = tid % WAVE;
    const int wave = __builtin_amdgcn_readfirstlane(tid / WAVE);
    const int lj = lane % 32, lg = lane / 32;
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;
    const int wm0 = wm * 64, wn0 = wn * (32 * TNF);

    MI355X_TRACE_STAMP(p, 0);
    MI355X_TRACE_HWID(p);
    const int ktiles = (int)(p.K / BK);
    const int last_tile = ktiles - 1;
    int64_t m0, n0;
    {
        int64_t tm, tn;
        tile_coords(xcd_remap(blockIdx.x, p.nwg), p.tiles_m, p.tiles_n, p.group_m, tm, tn);
        m0 = tm * BM;
        n0 = tn * BN;
    }

    // ---- loader: transfer instruction q of a step moves 1 KB, 16 bytes per lane: q < NA fills A rows 16 q .. + 15
    //   (lane i -> row + i / 4, slot i % 4 swizzled), the others fill the B stage (instruction q' = q - NA: chunks
    //   64 q' .. + 63, chunk c = k-row c / CPR, position c % CPR). Wave w issues q = w, w + NW, ...; where that runs
    //   past the last instruction, the wave repeats its previous one (same bytes to the same place).
    // Rows past M and columns past N are clamped into the matrix (what they produce is never stored).
    const int8_t* const a_tile = p.A + m0 * p.K;
    const int8_t* const b_tile = p.B + n0;
    const int64_t b_step = (int64_t)BK * p.N;
    uint32_t t_off[PER_WAVE];
    int q_of[PER_WAVE];
#pragma unroll
    for (int i = 0; i < PER_WAVE; ++i) {
        const int q0 = wave + i * NW;
        const int q = q0 < NT ? q0 : q0 - NW;   // wave-uniform
        q_of[i] = q;
        if (q < NA) {
            int64_t am = m0 + 16 * q + lane / 4;
            am = am < p.M ? am : p.M - 1;
            t_off[i] = (uint32_t)((am - m0) * p.K) + 16u * (uint32_t)((lane % 4) ^ ((lane >> 4) & 3));
        } else {
            const int c = 64 * (q - NA) + lane, krow = c / CPR, pos = c - CPR * krow;
            int64_t bn = n0 + 16 * mmt_b_swizzle(krow, pos, CPR);
            bn = bn < p.N ? bn : p.N - 16;
            t_off[i] = (uint32_t)krow * (uint32_t)p.N + (uint32_t)(bn - n0);
        }
    }
    const uint32_t lds_base = lds_address(lds);
    uint32_t t_lds[PER_WAVE];   // where in a stage instruction i of this wave writes (wave-uniform)
#pragma unroll
    for (int i = 0; i < PER_WAVE; ++i) t_lds[i] = (uint32_t)__builtin_amdgcn_readfirstlane((int)(lds_base + 1024u * (uint32_t)q_of[i]));
    // k-tile kt of the tile's operands; look-aheads past the end of K fetch the last k-tile again
    auto issue_loads = [&](int stage, int kt) __attribute__((always_inline)) {
        const int k = kt < last_tile ? kt : last_tile;
        const int8_t* const a_base = a_tile + (int64_t)k * BK;
        const int8_t* const b_base = b_tile + (int64_t)k * b_step;
#pragma unroll
        for (int i = 0; i < PER_WAVE; ++i) global_to_lds_16(q_of[i] < NA ? a_base : b_base, t_off[i], t_lds[i] + (uint32_t)(stage * STAGE));
    };

    // ---- operand reads: A operand i is row wm0 + 32 i + lj, chunk 2 ks + lg at (chunk ^ swizzle); B operand t is
    // columns wn0 + 32 t + lane % 32, lane i16 of a group of 16 addresses k-row 32 ks + 16 lg + i16 / 2 (+ 8 for the
    // second read), 8 columns from 16 (lane / 16 % 2) + 8 (i16 % 2). One pointer per operand and sub-step, set up here.
    const uint8_t* a_ptr[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int row = wm0 + 32 * i + lj;
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) a_ptr[i][ks] = lds + row * BK + 16 * ((2 * ks + lg) ^ ((row >> 2) & 3));
    }
    const int i16 = lane & 15, half = (lane >> 4) & 1, rib = i16 >> 1;
    const uint8_t* b_ptr[TNF];
#pragma unroll
    for (int t = 0; t < TNF; ++t) {
        const int cc = (wn0 + 32 * t) / 16 + half, krow = 16 * lg + rib;
        b_ptr[t] = lds + A_STAGE + krow * BN + 16 * mmt_b_swizzle(krow, cc, CPR) + 8 * (i16 & 1);
    }

    i32x16 acc[2][TNF];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int t = 0; t < TNF; ++t)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][t][r] = 0;
    int32_t rowsum[2] = {0, 0}, colsum[TNF] = {};
    i32x4 fa[2][2], fb[2][TNF];
    // A_DIRECT (measurement variant): A never enters LDS; a lane's operand (16 consecutive k of one row) is one raw-buffer
    // load straight into the register the MFMA reads, NS - 1 steps ahead; the two waves of a wave row fetch the same bytes
    i32x4 ra[A_DIRECT ? NS : 1][2][2];
    const int64_t a_rows_left = p.M - m0 - wm0;
    const __amdgpu_buffer_rsrc_t a_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<int8_t*>(p.A + (m0 + wm0) * p.K), 0, a_rows_left > 0 ? (int)((a_rows_left < 64 ? a_rows_left : 64) * p.K) : 0, 0x00020000);
    uint32_t a_voff[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) a_voff[i] = (uint32_t)(32 * i + lj) * (uint32_t)p.K + 16u * (uint32_t)lg;
    auto load_a = [&](auto slot_tag, int kt) __attribute__((always_inline)) {
        constexpr int slot = decltype(slot_tag)::value;
        if constexpr (A_DIRECT) {
            const int k = kt < last_tile ? kt : last_tile;
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int ks = 0; ks < 2; ++ks)
                    ra[slot][i][ks] = __builtin_bit_cast(i32x4, __builtin_amdgcn_raw_buffer_load_b128(a_rsrc, (int)(a_voff[i] + 32u * ks), k * BK, 0));
        }
    };
    auto read_frags = [&](auto set_tag, int stage, auto ks_tag) __attribute__((always_inline)) {
        constexpr int set = decltype(set_tag)::value, ks = decltype(ks_tag)::value;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            if constexpr (!A_DIRECT) {
                fa[set][i] = *reinterpret_cast<const i32x4*>(a_ptr[i][ks] + stage * STAGE);
                if constexpr (AU) fa[set][i] ^= (int)0x80808080u;
            }
        }
#pragma unroll
        for (int t = 0; t < TNF; ++t) {
            const i32x2 lo = lds_read_tr8(b_ptr[t] + stage * STAGE + 32 * BN * ks);
            const i32x2 hi = lds_read_tr8(b_ptr[t] + stage * STAGE + 32 * BN * ks + 8 * BN);
            fb[set][t] = i32x4{lo[0], lo[1], hi[0], hi[1]};
            if constexpr (BU) fb[set][t] ^= (int)0x80808080u;
        }
    };
    // (wm_tag, wn_tag: this wave's place in the wave grid as constants, see the dispatch below; r = step % NS)
    auto multiply = [&](auto ks_tag, auto r_tag, auto wm_tag, auto wn_tag) __attribute__((always_inline)) {
        constexpr int ks = decltype(ks_tag)::value;   // operand set ks holds sub-step ks
        constexpr int r = decltype(r_tag)::value, WM = decltype(wm_tag)::value, WN = decltype(wn_tag)::value;
        if constexpr (A_DIRECT) {
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                fa[ks][i] = ra[r][i][ks];
                if constexpr (AU) fa[ks][i] ^= (int)0x80808080u;
            }
        }
        if constexpr (ZP && WN == ks) {   // the two waves of a wave row sum one sub-step each
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int q = 0; q < 4; ++q) rowsum[i] = __builtin_amdgcn_sdot4(fa[ks][i][q], 0x01010101, rowsum[i], false);
        }
        if constexpr (ZP && WM == ((2 * r + ks) & (WAVES_M - 1))) {   // sub-step 2 kt + ks of the tile, one wave of the column in turn
#pragma unroll
            for (int t = 0; t < TNF; ++t)
#pragma unroll
                for (int q = 0; q < 4; ++q) colsum[t] = __builtin_amdgcn_sdot4(fb[ks][t][q], 0x01010101, colsum[t], false);
        }
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int t = 0; t < TNF; ++t) acc[i][t] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[ks][i], fb[ks][t], acc[i][t], 0, 0, 0);
    };

    // ---- prologue: stages 0 .. NS - 2 on their way, then the aligned 32-bit words that hold the first zero points
    // (behind the operand transfers, so that a cold page never delays the first step; they are looked at after the
    // loop). Both as assembly, so that the number of memory operations in flight is what is written here: the waits
    // below count them.
    mmi_static_for<NS - 1>([&](auto s_tag) {
        issue_loads(decltype(s_tag)::value, decltype(s_tag)::value);
        load_a(s_tag, decltype(s_tag)::value);
    });
    uint32_t za_raw = 0u, zb_raw = 0u;
    if constexpr (ZP) {
        const uint32_t* za_word = reinterpret_cast<const uint32_t*>(reinterpret_cast<uintptr_t>(p.za_ptr ? p.za_ptr : p.A) & ~(uintptr_t)3);
        const uint32_t* zb_word = reinterpret_cast<const uint32_t*>(reinterpret_cast<uintptr_t>(p.zb_ptr ? p.zb_ptr : p.B) & ~(uintptr_t)3);
        const uint32_t zero = 0u;
        asm volatile("global_load_dword %0, %1, %2" : "=v"(za_raw) : "v"(zero), "s"(za_word) : "memory");
        asm volatile("global_load_dword %0, %1, %2" : "=v"(zb_raw) : "v"(zero), "s"(zb_word) : "memory");
    }
    // operations complete in order: once all but the (NS - 3) youngest transfer groups and the two zero-point loads
    // have completed, stages 0 and 1 are in LDS
    constexpr int GROUP = PER_WAVE + (A_DIRECT ? 4 : 0);   // memory operations a wave issues per step: transfers, then A loads
    MI355X_WAIT_VMCNT((NS - 3) * GROUP + (A_DIRECT ? 4 : 0) + (ZP ? 2 : 0));
    __syncthreads();
    MI355X_TRACE_STAMP(p, 1);   // the first operands are in LDS
    MI355X_TRACE_CYCLES(p, 12);
    read_frags(std::integral_constant<int, 0>{}, 0, std::integral_constant<int, 0>{});

    // ---- K loop. At the top of step kt: stages kt and kt + 1 (mod NS) are in LDS and visible to every wave, operand
    // set 0 holds (stage kt, first 32 k). The transfer of step kt + NS - 1 goes into the stage step kt - 1 read.
    // The loop exists once per wave of the wave grid, with the wave's row and column as constants: which operands a
    // wave adds up for the zero points is then decided at compile time, and a step is straight-line code.
    static_assert((2 * NS) % WAVES_M == 0, "the wave whose turn it is to sum B depends on the step modulo NS only");
    auto k_loop = [&](auto wm_tag, auto wn_tag) __attribute__((always_inline)) {
        auto step = [&](auto r_tag, int kt) __attribute__((always_inline)) {
            constexpr int r = decltype(r_tag)::value;   // kt % NS
            issue_loads((r + NS - 1) % NS, kt + NS - 1);
            load_a(std::integral_constant<int, (r + NS - 1) % NS>{}, kt + NS - 1);
            read_frags(std::integral_constant<int, 1>{}, r, std::integral_constant<int, 1>{});
            multiply(std::integral_constant<int, 0>{}, r_tag, wm_tag, wn_tag);
            read_frags(std::integral_constant<int, 0>{}, (r + 1) % NS, std::integral_constant<int, 0>{});
            multiply(std::integral_constant<int, 1>{}, r_tag, wm_tag, wn_tag);
            // the transfer of step kt + 2 has to be in LDS behind the barrier: everything but the NS - 3 youngest groups
            MI355X_WAIT_VMCNT((NS - 3) * GROUP + (A_DIRECT ? 4 : 0));
            __syncthreads();
        };
        for (int kt0 = 0; kt0 < ktiles; kt0 += NS) {
            mmi_static_for<NS>([&](auto r_tag) {
                const int kt = kt0 + decltype(r_tag)::value;
                if (kt < ktiles) step(r_tag, kt);   // uniform; only the last group can be partial
            });
        }
    };
    mmi_static_for<NW>([&](auto w_tag) {
        constexpr int w = decltype(w_tag)::value;
        if (wave == w) k_loop(std::integral_constant<int, w / WAVES_N>{}, std::integral_constant<int, w % WAVES_N>{});
    });
    MI355X_TRACE_STAMP(p, 2);
    MI355X_TRACE_CYCLES(p, 13);
    MI355X_WAIT_VMCNT(0);   // look-ahead transfers past the end of K, and the zero points
    if constexpr (ZP) asm volatile("" : "+v"(za_raw), "+v"(zb_raw));   // nothing derived from them is computed before this wait

    // ---- the sums meet in LDS
    if constexpr (ZP) {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int32_t rs = rowsum[i] + __shfl_xor(rowsum[i], 32, WAVE);
            if (lg == 0) lds_rows[wm][wn][32 * i + lj] = rs;
        }
#pragma unroll
        for (int t = 0; t < TNF; ++t) {
            const int32_t cs = colsum[t] + __shfl_xor(colsum[t], 32, WAVE);
            if (lg == 0) lds_cols[wn][wm][32 * t + lj] = cs;
        }
        __syncthreads();
    }

    // ---- Y = acc - zb[n] rowsum[m] - za[m] (colsum[n] - K zb[n])
    // the tile's rows as a raw buffer: stores past the last row fall outside it and are dropped, columns
    // past N are dropped through offset bit 31 (BM rows of N int32 stay below 2^31 bytes: launch precondition)
    const int64_t rows_left = p.M - m0 < BM ? p.M - m0 : BM;
    const __amdgpu_buffer_rsrc_t y_rsrc =
        __builtin_amdgcn_make_buffer_rsrc(p.Y + m0 * p.N + n0, 0, (int)((rows_left * p.N - n0) * 4), 0x00020000);
    const bool one_each = p.za_stride == 0 && p.zb_stride == 0;   // wave-uniform
    uint32_t za_one = 0u, zb_one = 0u;
    if constexpr (ZP) {
        const int32_t a_bias = AU ? 128 : 0, b_bias = BU ? 128 : 0;
        const uint32_t za_byte = (za_raw >> (8 * (reinterpret_cast<uintptr_t>(p.za_ptr) & 3))) & 0xffu;
        const uint32_t zb_byte = (zb_raw >> (8 * (reinterpret_cast<uintptr_t>(p.zb_ptr) & 3))) & 0xffu;
        za_one = (uint32_t)((p.za_ptr ? (AU ? (int32_t)za_byte : (int32_t)(int8_t)za_byte) : 0) - a_bias);
        zb_one = (uint32_t)((p.zb_ptr ? (BU ? (int32_t)zb_byte : (int32_t)(int8_t)zb_byte) : 0) - b_bias);
    }
    const uint32_t row_bytes = (uint32_t)p.N * 4u;
    uint32_t voff[TNF], zbn[TNF] = {}, c2[TNF] = {};
#pragma unroll
    for (int t = 0; t < TNF; ++t) {
        const int col = wn0 + 32 * t + lj;
        const bool inside = n0 + col < p.N;
        voff[t] = (uint32_t)(wm0 + 4 * lg) * row_bytes + (inside ? (uint32_t)col * 4u : 0x80000000u);
        if constexpr (ZP) {
            zbn[t] = p.zb_stride == 0 ? zb_one : (inside ? (uint32_t)b_zero_point(p, n0 + col) : 0u);
            int32_t cs = 0;
#pragma unroll
            for (int w = 0; w < WAVES_M; ++w) cs += lds_cols[wn][w][32 * t + lj];
            c2[t] = (uint32_t)cs - (uint32_t)p.K * zbn[t];
        }
    }
    // 32-bit integer multiplies run at a quarter of the rate of adds: with one zero point per operand the
    // correction of an element is two subtractions, y = acc - zb rowsum[m] - za (colsum[n] - K zb)
    uint32_t d_col[TNF] = {};
    if constexpr (ZP) {
#pragma unroll
        for (int t = 0; t < TNF; ++t) d_col[t] = za_one * c2[t];
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
                rs4 = *reinterpret_cast<const i32x4*>(&lds_rows[wm][0][32 * i + 8 * q + 4 * lg]) +
                      *reinterpret_cast<const i32x4*>(&lds_rows[wm][1][32 * i + 8 * q + 4 * lg]);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int r = 4 * q + e;
                const uint32_t roff = (uint32_t)(32 * i + 8 * q + e) * row_bytes;
                uint32_t y[TNF];
#pragma unroll
                for (int t = 0; t < TNF; ++t) y[t] = (uint32_t)acc[i][t][r];
                if constexpr (ZP) {
                    const uint32_t rs = (uint32_t)rs4[e];
                    if (one_each) {
                        const uint32_t e_row = zb_one * rs;
#pragma unroll
                        for (int t = 0; t < TNF; ++t) y[t] = y[t] - e_row - d_col[t];
                    } else {
                        const uint32_t zam = p.za_stride == 0 ? za_one : (uint32_t)__shfl(za_lane, 8 * q + 4 * lg + e, WAVE);
#pragma unroll
                        for (int t = 0; t < TNF; ++t) y[t] = y[t] - zbn[t] * rs - zam * c2[t];
                    }
                }
#pragma unroll
                for (int t = 0; t < TNF; ++t)
                    __builtin_amdgcn_raw_buffer_store_b32((int32_t)y[t], y_rsrc, (int)(voff[t] + roff), 0, 0);
            }
        }
    }
#ifdef MI355X_WG_TRACE
    if (p.trace) MI355X_WAIT_VMCNT(0);   // slot 3: the last store is acknowledged
#endif
    MI355X_TRACE_STAMP(p, 3);
}

template <bool ZP, int WAVES_M, int WAVES_N, int TNF, int NS, bool A_DIRECT = false>
static void launch_tile(const MMIArgs& p, hipStream_t st) {
    const dim3 g((unsigned)p.nwg), b(64 * WAVES_M * WAVES_N);
    if (p.a_unsigned) {
        if (p.b_unsigned) hipLaunchKernelGGL((matmul_integer_i8_tile_kernel<true, true, true, WAVES_M, WAVES_N, TNF, NS>), g, b, 0, st, p);
        else hipLaunchKernelGGL((matmul_integer_i8_tile_kernel<true, true, false, WAVES_M, WAVES_N, TNF, NS>), g, b, 0, st, p);
    } else if (p.b_unsigned) {
        hipLaunchKernelGGL((matmul_integer_i8_tile_kernel<true, false, true, WAVES_M, WAVES_N, TNF, NS>), g, b, 0, st, p);
    } else {
        hipLaunchKernelGGL((matmul_integer_i8_tile_kernel<ZP, false, false, WAVES_M, WAVES_N, TNF, NS, A_DIRECT>), g, b, 0, st, p);
    }
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
        // Three forms of the same data path. Long K: 256 x 192 tiles, one workgroup of eight waves per CU (0.72 us per 64-k
        // step of the whole 4096 x 3072 problem against 0.87 us: less LDS traffic per MFMA and 14 instead of 16 zero-point
        // instructions per wave and step), where such tiles fill the CUs as evenly as 128 x 128 tiles in threes do. Short K:
        // the persistent kernel below, whose three workgroups per CU hide each other's start and stores (K = 768: 19.2 us
        // against 19.7 us). MI355X_MMI_TILE forces 128 (one 128 x 128 tile per workgroup) or 256; 129 and 257 are the same
        // two with A read straight from global memory into the MFMA registers, kept as a measurement (signed operands only):
        // the vector memory pipe takes a load whose neighbouring lanes touch different rows at one row per cycle, 64 cycles
        // per instruction instead of 16, and a step takes 1.63 us / 1.06 us.
        const int64_t wide_tiles = ceil_div(M, (int64_t)256) * ceil_div(N, (int64_t)192);
        const double narrow_cost = (double)ceil_div(p.nwg, (int64_t)3 * cus) * 3 * 128 * 128;
        const double wide_cost = (double)ceil_div(wide_tiles, (int64_t)cus) * 256 * 192;
        const int tile = tune.mmi_tile ? tune.mmi_tile :   // (1: none of the tile kernels)
                         (K >= 1536 && wide_cost <= narrow_cost && N < ((int64_t)1 << 20)) ? 256 : 0;
        if (tile == 128 || tile == 256 || tile == 129 || tile == 257) {
            const bool a_direct = (tile & 1) && !p.a_unsigned && !p.b_unsigned && p.M * p.K < ((int64_t)1 << 31);
            const int bm = tile >= 256 ? 256 : 128, bn = tile >= 256 ? 192 : 128;
            p.tiles_m = ceil_div(M, (int64_t)bm);
            p.tiles_n = ceil_div(N, (int64_t)bn);
            p.nwg = p.tiles_m * p.tiles_n;
            const int64_t per_xcd = ceil_div(p.nwg, (int64_t)NUM_XCD), resident = (int64_t)(bm == 256 ? 1 : 3) * (cus / NUM_XCD);
            p.group_m = choose_group_m(p.tiles_m, per_xcd, resident, bm, bn, K);
            const bool zp = a_zero_point || b_zero_point;
            if (a_direct) {
                if (bm == 256) { if (zp) launch_tile<true, 4, 2, 3, 4, true>(p, st); else launch_tile<false, 4, 2, 3, 4, true>(p, st); }
                else { if (zp) launch_tile<true, 2, 2, 2, 3, true>(p, st); else launch_tile<false, 2, 2, 2, 3, true>(p, st); }
            } else if (bm == 256) {
                if (zp) launch_tile<true, 4, 2, 3, 4>(p, st); else launch_tile<false, 4, 2, 3, 4>(p, st);
            } else {
                if (zp) launch_tile<true, 2, 2, 2, 3>(p, st); else launch_tile<false, 2, 2, 2, 3>(p, st);
            }
            return check_launch("matmul_integer_i8_tile_kernel");
        }
        // persistent grid: three workgroups per CU (a multiple of the XCD count), fewer if there are fewer tiles
        int64_t grid = (int64_t)(tune.mmi_wgs_per_cu > 0 ? tune.mmi_wgs_per_cu : 3) * (cus / NUM_XCD) * NUM_XCD;
        if (grid > p.nwg || grid <= 0) grid = p.nwg;
        const int64_t per_xcd = ceil_div(p.nwg, (int64_t)NUM_XCD), resident = ceil_div(grid, (int64_t)NUM_XCD);
        p.group_m = choose_group_m(p.tiles_m, per_xcd, resident, MMF_BM, MMF_BN, K);
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
