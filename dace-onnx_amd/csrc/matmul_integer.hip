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

namespace mi355x {

struct MMIArgs {
    const int8_t* A; const int8_t* B; int32_t* Y;
    int64_t M, N, K;
    const int8_t* za_ptr; const int8_t* zb_ptr;
    int64_t tiles_m, tiles_n, nwg;
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
    if (vec) hipLaunchKernelGGL(matmul_integer_i8_kernel<true>, dim3((unsigned)p.nwg), dim3(256), 0, st, p);
    else hipLaunchKernelGGL(matmul_integer_i8_kernel<false>, dim3((unsigned)p.nwg), dim3(256), 0, st, p);
    return check_launch("matmul_integer_i8_kernel");
}
