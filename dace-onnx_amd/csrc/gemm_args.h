// Argument block shared by the fp32 GEMM kernels.
#pragma once

#include "common.h"

namespace mi355x {

struct GemmArgs {
    const float* A; const float* B; float* C; const float* bias; const float* residual;
    int64_t batch, batch1;  // total batch entries, and the extent of the inner batch level
    int64_t M, N, K;
    int64_t a_sb0, a_sb1, a_sm, a_sk;
    int64_t b_sb0, b_sb1, b_sk, b_sn;
    int64_t c_sb0, c_sb1, c_sm;
    int64_t r_sb0, r_sb1, r_sm;
    int64_t tiles_m, tiles_n, nwg;
    int group_m;  // tile walk order, see tile_coords
    float alpha;
    int epi;
    MI355X_TRACE_MEMBER
};

// GEMM with both operands contiguous along k (gemm_f32_nt.hip). Returns false when
// the problem is outside what that kernel handles (nothing launched).
bool launch_gemm_f32_nt(GemmArgs p, int cus, hipStream_t stream);

// GEMM with both operands contiguous along k whose eight waves split K (gemm_f32_ksplit.hip): 32 x 96 tiles.
bool launch_gemm_f32_ksplit(GemmArgs p, int cus, hipStream_t stream);

}  // namespace mi355x
