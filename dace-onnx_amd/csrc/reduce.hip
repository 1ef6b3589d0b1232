// ONNX ReduceMean along one (collapsed) axis, fp32.
//
// Replaces PureReduceMean.forward (daceml/onnx/op_implementations/
// pure_implementations.py:97-109). X is viewed as [outer, axis_len, inner]:
//   reduce_mean_rows     inner == 1: one wave per row, 16-byte loads when the row
//                        length allows, DPP wave reduction, no LDS;
//   reduce_mean_strided  otherwise: one thread per (outer, inner) column, lanes
//                        adjacent along `inner` so every access is coalesced.
// The node only appears in graphs that spell LayerNormalization out (opset < 17
// exports); the fusion pass turns that pattern back into one LayerNormalization
// kernel, so this kernel serves what is left over and is written for
// correctness at full bandwidth on long rows, not for tiny launches.
#include "common.h"

namespace mi355x {

template <bool VEC>
__global__ __launch_bounds__(256) void reduce_mean_rows(const float* __restrict__ X, float* __restrict__ Y,
                                                        int64_t rows, int64_t cols, float inv_n) {
    const int lane = threadIdx.x % WAVE;
    const int64_t row = (int64_t)blockIdx.x * (256 / WAVE) + threadIdx.x / WAVE;
    if (row >= rows) return;  // whole wave
    const float* x = X + row * cols;
    float s = 0.0f;
    if constexpr (VEC) {
        const f32x4* x4 = reinterpret_cast<const f32x4*>(x);
        for (int64_t c = lane; c < cols / 4; c += WAVE) {
            const f32x4 v = x4[c];
            s += (v.x + v.y) + (v.z + v.w);
        }
    } else {
        for (int64_t c = lane; c < cols; c += WAVE) s += x[c];
    }
    s = wave_sum(s);
    if (lane == 0) Y[row] = s * inv_n;
}

__global__ __launch_bounds__(256) void reduce_mean_strided(const float* __restrict__ X, float* __restrict__ Y,
                                                           int64_t outer, int64_t axis_len, int64_t inner,
                                                           float inv_n) {
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= outer * inner) return;
    const int64_t o = idx / inner, i = idx % inner;
    const float* x = X + o * axis_len * inner + i;
    // independent chains for the loads; in double, because one thread adds up a whole column
    double s[8] = {0., 0., 0., 0., 0., 0., 0., 0.};
    int64_t a = 0;
    for (; a + 8 <= axis_len; a += 8) {
#pragma unroll
        for (int u = 0; u < 8; ++u) s[u] += (double)x[(a + u) * inner];
    }
    for (int u = 0; a < axis_len; ++a, ++u) s[u] += (double)x[a * inner];
    Y[idx] = (float)((((s[0] + s[1]) + (s[2] + s[3])) + ((s[4] + s[5]) + (s[6] + s[7]))) / (double)axis_len);
}

}  // namespace mi355x

extern "C" int mi355x_reduce_mean_f32(const float* X, float* Y, int64_t outer, int64_t axis_len,
                                      int64_t inner, void* stream) {
    using namespace mi355x;
    MI355X_REQUIRE(outer >= 0 && axis_len >= 1 && inner >= 0,
                   "reduce_mean: bad extents outer=%lld axis_len=%lld inner=%lld",
                   (long long)outer, (long long)axis_len, (long long)inner);
    if (outer == 0 || inner == 0) return MI355X_OK;
    MI355X_REQUIRE(X && Y, "reduce_mean: null pointer");
    hipStream_t st = static_cast<hipStream_t>(stream);
    const float inv_n = 1.0f / (float)axis_len;
    if (inner == 1) {
        const int64_t blocks = ceil_div(outer, (int64_t)(256 / WAVE));
        MI355X_REQUIRE(blocks < ((int64_t)1 << 31), "reduce_mean: grid too large");
        const bool vec = axis_len % 4 == 0 && (reinterpret_cast<uintptr_t>(X) & 15) == 0;
        if (vec) hipLaunchKernelGGL(reduce_mean_rows<true>, dim3((unsigned)blocks), dim3(256), 0, st, X, Y, outer, axis_len, inv_n);
        else hipLaunchKernelGGL(reduce_mean_rows<false>, dim3((unsigned)blocks), dim3(256), 0, st, X, Y, outer, axis_len, inv_n);
        return check_launch("reduce_mean_rows");
    }
    const int64_t blocks = ceil_div(outer * inner, (int64_t)256);
    MI355X_REQUIRE(blocks < ((int64_t)1 << 31), "reduce_mean: grid too large");
    hipLaunchKernelGGL(reduce_mean_strided, dim3((unsigned)blocks), dim3(256), 0, st, X, Y, outer, axis_len, inner, inv_n);
    return check_launch("reduce_mean_strided");
}
