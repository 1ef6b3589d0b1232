// ONNX LayerNormalization over the last axis, fp32, one pass over HBM.
//
// The reference reaches this op only as the exporter's nine-node chain
// ReduceMean, Sub, Pow, ReduceMean, Add(eps), Sqrt, Div, Mul(gamma), Add(beta)
// (daceml/onnx/op_implementations/pure_implementations.py:97-109,82-84,59-74,
// 77-79,41-56,92-94), each with a materialised intermediate. Here a row stays
// in registers: mean, then the biased variance of the centred values (the same
// two-step order as the chain, not E[x^2]-E[x]^2), then the affine output.
//
// Kernels:
//   layernorm_rows_reg<NV>  cols % 4 == 0, cols <= 256*NV: one wave per row,
//       NV float4 per lane (768 columns = 3 loads of 16 bytes per lane), DPP +
//       readlane reductions, no LDS.
//   layernorm_rows_loop     any cols: one wave per row, three sweeps.
#include "common.h"

namespace mi355x {

template <int NV>
__global__ __launch_bounds__(256) void layernorm_rows_reg(const float* __restrict__ X,
                                                          const float* __restrict__ gamma,
                                                          const float* __restrict__ beta,
                                                          float* __restrict__ Y, int64_t rows,
                                                          int cols, float eps) {
    const int lane = threadIdx.x % WAVE;
    const int64_t row = (int64_t)blockIdx.x * (256 / WAVE) + threadIdx.x / WAVE;
    if (row >= rows) return;  // wave-uniform
    const int cols4 = cols >> 2;
    const f32x4* src = reinterpret_cast<const f32x4*>(X + row * cols);

    f32x4 v[NV];
#pragma unroll
    for (int j = 0; j < NV; ++j) {
        const int c4 = lane + j * WAVE;
        v[j] = (c4 < cols4) ? __builtin_nontemporal_load(src + c4) : f32x4{0.f, 0.f, 0.f, 0.f};
    }
    // gamma / beta are shared by every row: ordinary (cached) loads
    f32x4 g[NV], b[NV];
#pragma unroll
    for (int j = 0; j < NV; ++j) {
        const int c4 = lane + j * WAVE;
        g[j] = (c4 < cols4) ? reinterpret_cast<const f32x4*>(gamma)[c4] : f32x4{0.f, 0.f, 0.f, 0.f};
        b[j] = (beta != nullptr && c4 < cols4) ? reinterpret_cast<const f32x4*>(beta)[c4]
                                               : f32x4{0.f, 0.f, 0.f, 0.f};
    }

    float s = 0.0f;
#pragma unroll
    for (int j = 0; j < NV; ++j) s += (v[j].x + v[j].y) + (v[j].z + v[j].w);
    const float inv_n = 1.0f / (float)cols;
    const float mean = wave_sum(s) * inv_n;

    float q = 0.0f;
#pragma unroll
    for (int j = 0; j < NV; ++j) {
        const int c4 = lane + j * WAVE;
        if (c4 < cols4) {
            v[j] -= mean;
            q += (v[j].x * v[j].x + v[j].y * v[j].y) + (v[j].z * v[j].z + v[j].w * v[j].w);
        }
    }
    const float var = wave_sum(q) * inv_n;
    const float inv_std = 1.0f / sqrtf(var + eps);

    f32x4* dst = reinterpret_cast<f32x4*>(Y + row * cols);
#pragma unroll
    for (int j = 0; j < NV; ++j) {
        const int c4 = lane + j * WAVE;
        if (c4 < cols4) {
            f32x4 o = (v[j] * inv_std) * g[j] + b[j];
            __builtin_nontemporal_store(o, dst + c4);
        }
    }
}

__global__ __launch_bounds__(256) void layernorm_rows_loop(const float* __restrict__ X,
                                                           const float* __restrict__ gamma,
                                                           const float* __restrict__ beta,
                                                           float* __restrict__ Y, int64_t rows,
                                                           int64_t cols, float eps) {
    const int lane = threadIdx.x % WAVE;
    const int64_t row = (int64_t)blockIdx.x * (256 / WAVE) + threadIdx.x / WAVE;
    if (row >= rows) return;
    const float* x = X + row * cols;
    float* y = Y + row * cols;
    float s = 0.0f;
    for (int64_t c = lane; c < cols; c += WAVE) s += x[c];
    const float mean = wave_sum(s) / (float)cols;
    float q = 0.0f;
    for (int64_t c = lane; c < cols; c += WAVE) {
        const float d = x[c] - mean;
        q += d * d;
    }
    const float var = wave_sum(q) / (float)cols;
    const float inv_std = 1.0f / sqrtf(var + eps);
    for (int64_t c = lane; c < cols; c += WAVE) {
        const float bb = beta ? beta[c] : 0.0f;
        y[c] = ((x[c] - mean) * inv_std) * gamma[c] + bb;
    }
}

}  // namespace mi355x

extern "C" int mi355x_layernorm_f32(const float* X, const float* gamma, const float* beta,
                                    float* Y, int64_t rows, int64_t cols, float eps,
                                    void* stream) {
    using namespace mi355x;
    MI355X_REQUIRE(rows >= 0 && cols >= 0, "layernorm: negative extent (rows=%lld cols=%lld)",
                   (long long)rows, (long long)cols);
    if (rows == 0 || cols == 0) return MI355X_OK;
    MI355X_REQUIRE(X && Y && gamma, "layernorm: null pointer (X, Y and gamma are required)");
    MI355X_REQUIRE(ceil_div(rows, 256 / WAVE) < ((int64_t)1 << 31), "layernorm: too many rows");
    hipStream_t st = static_cast<hipStream_t>(stream);
    const dim3 grid((unsigned)ceil_div(rows, 256 / WAVE)), block(256);
    auto aligned = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
    const bool vec_ok = (cols % 4 == 0) && aligned(X) && aligned(Y) && aligned(gamma) &&
                        (beta == nullptr || aligned(beta));
    const int c = (int)cols;
    if (vec_ok && cols <= 256) hipLaunchKernelGGL(layernorm_rows_reg<1>, grid, block, 0, st, X, gamma, beta, Y, rows, c, eps);
    else if (vec_ok && cols <= 512) hipLaunchKernelGGL(layernorm_rows_reg<2>, grid, block, 0, st, X, gamma, beta, Y, rows, c, eps);
    else if (vec_ok && cols <= 768) hipLaunchKernelGGL(layernorm_rows_reg<3>, grid, block, 0, st, X, gamma, beta, Y, rows, c, eps);
    else if (vec_ok && cols <= 1024) hipLaunchKernelGGL(layernorm_rows_reg<4>, grid, block, 0, st, X, gamma, beta, Y, rows, c, eps);
    else if (vec_ok && cols <= 2048) hipLaunchKernelGGL(layernorm_rows_reg<8>, grid, block, 0, st, X, gamma, beta, Y, rows, c, eps);
    else if (vec_ok && cols <= 4096) hipLaunchKernelGGL(layernorm_rows_reg<16>, grid, block, 0, st, X, gamma, beta, Y, rows, c, eps);
    else hipLaunchKernelGGL(layernorm_rows_loop, grid, block, 0, st, X, gamma, beta, Y, rows, cols, eps);
    return check_launch("layernorm_rows");
}
