// Building blocks shared by the MFMA contraction kernels (GEMM and implicit-GEMM
// convolution): XCD-aware workgroup numbering, global->LDS tile staging, and the
// LDS->MFMA inner product over one staged k-tile.
#pragma once

#include "common.h"

namespace mi355x {

constexpr int NUM_XCD = 8;
constexpr int LDS_PAD = 4;

// Hardware places workgroup w on XCD w % 8. Give XCD x the contiguous logical
// range it would own if the tile space were cut into eight slabs.
// (Grids are below 2^31 workgroups: 32-bit arithmetic, a 64-bit division costs
// every wave several hundred instructions before its first load.)
__device__ __forceinline__ int64_t xcd_remap(int64_t wg, int64_t nwg) {
    const uint32_t w = (uint32_t)wg, n = (uint32_t)nwg;
    const uint32_t full = n / NUM_XCD, rem = n % NUM_XCD;
    const uint32_t xcd = w % NUM_XCD, slot = w / NUM_XCD;
    return (int64_t)(xcd * full + (xcd < rem ? xcd : rem) + slot);
}

// Tile t of a tiles_m x tiles_n grid, walked in panels of group_m tile rows, down
// the panel's rows first. Consecutive t (the slab one XCD works on at a time, see
// xcd_remap) then cover a group_m x (slab / group_m) block of tiles instead of a
// single tile row, so the XCD's L2 fetches far fewer distinct operand rows.
__device__ __forceinline__ void tile_coords(int64_t t64, int64_t tiles_m64, int64_t tiles_n64, int group_m,
                                            int64_t& tm, int64_t& tn) {
    const uint32_t t = (uint32_t)t64, tiles_m = (uint32_t)tiles_m64, tiles_n = (uint32_t)tiles_n64;
    const uint32_t panel = (uint32_t)group_m * tiles_n;
    const uint32_t first_m = (t / panel) * (uint32_t)group_m;
    const uint32_t rows = tiles_m - first_m < (uint32_t)group_m ? tiles_m - first_m : (uint32_t)group_m;
    const uint32_t in_panel = t % panel;
    tm = first_m + in_panel % rows;
    tn = in_panel / rows;
}

// Panel height for tile_coords. An XCD works on a slab of `per_xcd` consecutive tiles, `resident` of them at a time
// (bm x bn each, K k-values of `elem` bytes per operand row). The rows of A and of B a block of g x c tiles needs are
// g bm + c bn; every XCD fetches its own copy of them through its own L2 (4 MB). If the panels of the whole slab fit
// that L2 the slab is shaped (a later round of workgroups then finds the operand rows of the earlier ones: QKV
// projection as 768 tiles, 96 per XCD in three rounds: 25.9 MiB through the L2-to-fabric counters with panels of 8
// tile rows against 33.3 MiB with 4), otherwise the block that is resident at one time. Measured on the four GEMMs
// of a BERT-base layer: the walk changes the fetched bytes by up to 3x (one tile row at a time: 100 MiB for the QKV
// projection) and the run time by 1-2 %.
inline int choose_group_m(int64_t tiles_m, int64_t per_xcd, int64_t resident, int bm, int bn, int64_t k_bytes) {
    auto best_for = [&](int64_t tiles, double& cost_out) {
        int best = 1;
        double best_cost = 1e300;
        for (int g = 1; g <= 16 && g <= tiles_m; ++g) {
            const int64_t cols = (tiles + g - 1) / g;
            // a block that leaves its last column ragged touches the rows of all g anyway: whole columns are cheaper
            const double cost = g * (double)bm + cols * (double)bn;
            if (cost < best_cost) { best_cost = cost; best = g; }
        }
        cost_out = best_cost;
        return best;
    };
    constexpr double L2_BYTES = 3.5 * 1024 * 1024;   // of the 4 MB, leaving room for the results on their way out
    double slab_rows = 0, block_rows = 0;
    const int g_slab = best_for(per_xcd, slab_rows);
    const int g_block = best_for(resident < per_xcd ? resident : per_xcd, block_rows);
    return slab_rows * (double)k_bytes <= L2_BYTES ? g_slab : g_block;
}

// Global -> registers for a ROWS x COLS tile whose COLS direction is the
// operand's contiguous one. VEC: 16-byte loads (extent along COLS is a multiple
// of 4 and 16-byte aligned, so a vector is entirely inside or outside).
template <int ROWS, int COLS, bool VEC, int NT>
struct TileIO {
    static constexpr int VPR = COLS / 4;
    static constexpr int NVEC = ROWS * VPR;
    static constexpr int PER_T = (NVEC + NT - 1) / NT;
    static constexpr int PITCH = COLS + LDS_PAD;

    __device__ static __forceinline__ void load(f32x4 (&r)[PER_T], const float* __restrict__ base,
                                                int64_t r0, int64_t c0, int64_t r_lim,
                                                int64_t c_lim, int64_t s_r, int64_t s_c, int tid) {
#pragma unroll
        for (int it = 0; it < PER_T; ++it) {
            const int idx = tid + it * NT;
            const int row = idx / VPR, c4 = idx % VPR;
            const int64_t gr = r0 + row, gc = c0 + 4 * c4;
            f32x4 v = f32x4{0.f, 0.f, 0.f, 0.f};
            if ((NVEC % NT == 0 || idx < NVEC) && gr < r_lim) {
                if constexpr (VEC) {
                    if (gc < c_lim) v = *reinterpret_cast<const f32x4*>(base + gr * s_r + gc);
                } else {
                    const float* p = base + gr * s_r + gc * s_c;
                    if (gc + 0 < c_lim) v.x = p[0];
                    if (gc + 1 < c_lim) v.y = p[s_c];
                    if (gc + 2 < c_lim) v.z = p[2 * s_c];
                    if (gc + 3 < c_lim) v.w = p[3 * s_c];
                }
            }
            r[it] = v;
        }
    }
    __device__ static __forceinline__ void store(const f32x4 (&r)[PER_T], float* lds, int tid) {
#pragma unroll
        for (int it = 0; it < PER_T; ++it) {
            const int idx = tid + it * NT;
            const int row = idx / VPR, c4 = idx % VPR;
            if (NVEC % NT == 0 || idx < NVEC)
                *reinterpret_cast<f32x4*>(lds + row * PITCH + 4 * c4) = r[it];
        }
    }
};


// Multiply the staged k-tile: acc[i][j] += A(16 rows at wm0+16i) x B(16 cols at wn0+16j).
// Operands stored k-contiguous ([rows][BK+4]) are read 16 bytes at a time: lane
// (li, lq) gets k = kc+4*lq .. +3, which feeds four MFMA steps; operands stored
// m/n-contiguous ([BK][rows+4]) are read 4 bytes at a time at the same k. The
// MFMA operands are swapped so acc[i][j][r] = C[wm0+16i+li][wn0+16j+4*lq+r].
template <int TM, int TN, int BK, bool A_KC, bool B_KC, int A_PITCH, int B_PITCH>
__device__ __forceinline__ void mma_ktile(const float* __restrict__ la, const float* __restrict__ lb,
                                          int wm0, int wn0, int li, int lq, f32x4 (&acc)[TM][TN]) {
#pragma unroll
    for (int kc = 0; kc < BK; kc += 16) {
        float af[TM][4], bf[TN][4];
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            if constexpr (A_KC) {
                const f32x4 v = *reinterpret_cast<const f32x4*>(la + (wm0 + i * 16 + li) * A_PITCH + kc + 4 * lq);
                af[i][0] = v.x; af[i][1] = v.y; af[i][2] = v.z; af[i][3] = v.w;
            } else {
#pragma unroll
                for (int s = 0; s < 4; ++s) af[i][s] = la[(kc + 4 * lq + s) * A_PITCH + wm0 + i * 16 + li];
            }
        }
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            if constexpr (B_KC) {
                const f32x4 v = *reinterpret_cast<const f32x4*>(lb + (wn0 + j * 16 + li) * B_PITCH + kc + 4 * lq);
                bf[j][0] = v.x; bf[j][1] = v.y; bf[j][2] = v.z; bf[j][3] = v.w;
            } else {
#pragma unroll
                for (int s = 0; s < 4; ++s) bf[j][s] = lb[(kc + 4 * lq + s) * B_PITCH + wn0 + j * 16 + li];
            }
        }
#pragma unroll
        for (int s = 0; s < 4; ++s)
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(bf[j][s], af[i][s], acc[i][j], 0, 0, 0);
    }
}

}  // namespace mi355x
