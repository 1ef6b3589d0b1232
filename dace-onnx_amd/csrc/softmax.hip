// ONNX Softmax and LogSoftmax, fp32, one pass over HBM.
//
// The reference expansion (daceml/onnx/op_implementations/pure_implementations.py:346-366)
// runs max, subtract, exp, sum and divide as five maps with three full-size
// temporaries. Here a row lives in registers between the read and the write,
// so HBM traffic is the algorithmic minimum: one read and one write per element.
// LogSoftmax (PureLogSoftmax, :594-616: (x - max) - log(sum(exp(x - max)))) is the same
// kernels with a different last step (template parameter LOG).
//
// Kernels:
//   softmax_rows_reg<L, NV, UNR>  last axis, cols % 4 == 0, cols <= L*4*NV.
//       A row is owned by L lanes (16, 32 or 64) holding NV float4 each, so a
//       128-column row is one 16-byte load per lane of a half wave and the two
//       reductions are DPP row operations, no LDS. Each group handles UNR rows
//       with all loads issued before the first reduction to keep HBM requests
//       in flight.
//   softmax_rows_loop   last axis, any cols: one wave per row, three sweeps
//       (max, sum, write); sweeps two and three hit in L2.
//   softmax_strided     axis is not last: one thread per (outer, inner) column,
//       lanes adjacent along `inner` so every access is coalesced.
#include "common.h"

namespace mi355x {

template <int L>
__device__ __forceinline__ float group_sum(float v) {
    if constexpr (L == 16) return row16_sum(v);
    else if constexpr (L == 32) return half32_sum(v);
    else return wave_sum(v);
}
template <int L>
__device__ __forceinline__ float group_max(float v) {
    if constexpr (L == 16) return row16_max(v);
    else if constexpr (L == 32) return half32_max(v);
    else return wave_max(v);
}

template <int L, int NV, int UNR, bool LOG>
__global__ __launch_bounds__(256) void softmax_rows_reg(const float* __restrict__ X,
                                                        float* __restrict__ Y,
                                                        int64_t rows, int cols) {
    constexpr int GROUPS_PER_BLOCK = 256 / L;
    const int lane = threadIdx.x % L;
    const int group = threadIdx.x / L;
    const int64_t row0 = ((int64_t)blockIdx.x * GROUPS_PER_BLOCK + group) * UNR;
    const int cols4 = cols >> 2;

    f32x4 v[UNR][NV];
#pragma unroll
    for (int u = 0; u < UNR; ++u) {
        const int64_t row = row0 + u;
        const f32x4* src = reinterpret_cast<const f32x4*>(X + row * cols);
#pragma unroll
        for (int j = 0; j < NV; ++j) {
            const int c4 = lane + j * L;
            if (row < rows && c4 < cols4) {
                v[u][j] = __builtin_nontemporal_load(src + c4);
            } else {
                v[u][j] = f32x4{-INFINITY, -INFINITY, -INFINITY, -INFINITY};
            }
        }
    }

#pragma unroll
    for (int u = 0; u < UNR; ++u) {
        const int64_t row = row0 + u;
        float m = -INFINITY;
#pragma unroll
        for (int j = 0; j < NV; ++j)
            m = fmaxf(m, fmaxf(fmaxf(v[u][j].x, v[u][j].y), fmaxf(v[u][j].z, v[u][j].w)));
        m = group_max<L>(m);
        constexpr float LOG2E = 1.4426950408889634f;
        float s = 0.0f;
#pragma unroll
        for (int j = 0; j < NV; ++j) {
            // padded lanes hold -inf: exp(-inf - m) == 0 contributes nothing
            if constexpr (LOG) {
                v[u][j] = v[u][j] - m;   // kept for the result; the exponentials only feed the sum
                s += (expf(v[u][j].x) + expf(v[u][j].y)) + (expf(v[u][j].z) + expf(v[u][j].w));
            } else {
                // exp(x - m) as 2^((x - m) log2 e): one v_exp_f32 per element instead of the library routine.
                // The argument t is <= 0 (no overflow); its rounding error |t| 2^-24 shows as a relative error of
                // the result below 1.3e-6 for every element that is at least 2^-30 of the row maximum.
                v[u][j].x = __builtin_amdgcn_exp2f((v[u][j].x - m) * LOG2E);
                v[u][j].y = __builtin_amdgcn_exp2f((v[u][j].y - m) * LOG2E);
                v[u][j].z = __builtin_amdgcn_exp2f((v[u][j].z - m) * LOG2E);
                v[u][j].w = __builtin_amdgcn_exp2f((v[u][j].w - m) * LOG2E);
                s += (v[u][j].x + v[u][j].y) + (v[u][j].z + v[u][j].w);
            }
        }
        s = group_sum<L>(s);
        const float inv = 1.0f / s, log_s = LOG ? logf(s) : 0.0f;
        f32x4* dst = reinterpret_cast<f32x4*>(Y + row * cols);
#pragma unroll
        for (int j = 0; j < NV; ++j) {
            const int c4 = lane + j * L;
            if (row < rows && c4 < cols4) {
                f32x4 o = LOG ? v[u][j] - log_s : v[u][j] * inv;
                __builtin_nontemporal_store(o, dst + c4);
            }
        }
    }
}

template <bool LOG>
__global__ __launch_bounds__(256) void softmax_rows_loop(const float* __restrict__ X,
                                                         float* __restrict__ Y,
                                                         int64_t rows, int64_t cols) {
    const int lane = threadIdx.x % WAVE;
    const int64_t row = (int64_t)blockIdx.x * (256 / WAVE) + threadIdx.x / WAVE;
    if (row >= rows) return;  // whole wave leaves together
    const float* x = X + row * cols;
    float* y = Y + row * cols;
    float m = -INFINITY;
    for (int64_t c = lane; c < cols; c += WAVE) m = fmaxf(m, x[c]);
    m = wave_max(m);
    float s = 0.0f;
    for (int64_t c = lane; c < cols; c += WAVE) s += expf(x[c] - m);
    s = wave_sum(s);
    const float inv = 1.0f / s, log_s = LOG ? logf(s) : 0.0f;
    for (int64_t c = lane; c < cols; c += WAVE) y[c] = LOG ? (x[c] - m) - log_s : expf(x[c] - m) * inv;
}

template <bool LOG>
__global__ __launch_bounds__(256) void softmax_strided(const float* __restrict__ X,
                                                       float* __restrict__ Y,
                                                       int64_t outer, int64_t axis_len,
                                                       int64_t inner) {
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= outer * inner) return;
    const int64_t o = idx / inner, i = idx % inner;
    const float* x = X + o * axis_len * inner + i;
    float* y = Y + o * axis_len * inner + i;
    float m = -INFINITY;
    for (int64_t a = 0; a < axis_len; ++a) m = fmaxf(m, x[a * inner]);
    // eight running sums (independent chains for the loads), kept in double: a thread adds up a whole
    // column by itself, and in float the rounding error of the denominator would grow with axis_len
    // (3e-6 relative at 4100 elements); the kernel waits on strided loads, the wider adds are free
    double s[8] = {0., 0., 0., 0., 0., 0., 0., 0.};
    int64_t a = 0;
    for (; a + 8 <= axis_len; a += 8) {
#pragma unroll
        for (int u = 0; u < 8; ++u) s[u] += (double)expf(x[(a + u) * inner] - m);
    }
    for (int u = 0; a < axis_len; ++a, ++u) s[u] += (double)expf(x[a * inner] - m);
    const double total = ((s[0] + s[1]) + (s[2] + s[3])) + ((s[4] + s[5]) + (s[6] + s[7]));
    const float inv = (float)(1.0 / total), log_s = LOG ? (float)log(total) : 0.0f;
    for (a = 0; a < axis_len; ++a) y[a * inner] = LOG ? (x[a * inner] - m) - log_s : expf(x[a * inner] - m) * inv;
}

template <int L, int NV, int UNR, bool LOG>
static void launch_reg(const float* X, float* Y, int64_t rows, int cols, hipStream_t st) {
    constexpr int rows_per_block = (256 / L) * UNR;
    const int64_t blocks = ceil_div(rows, rows_per_block);
    hipLaunchKernelGGL((softmax_rows_reg<L, NV, UNR, LOG>), dim3((unsigned)blocks), dim3(256), 0, st,
                       X, Y, rows, cols);
}

// Rows per lane group. Inputs of a few MB are one round trip to memory per CU and finish sooner the more
// workgroups share it (12288 rows of 128: 3.1 us with 2 rows per group, 3.6 us with 3, 4.4 us with 6, against
// 2.8 us for a plain copy of the same bytes and 1.8 us for an empty kernel); inputs that stream for many
// rounds run faster with three rows of loads in flight per lane.
template <int L, int NV, bool LOG>
static void launch_reg_unr(const float* X, float* Y, int64_t rows, int cols, hipStream_t st) {
    constexpr int groups = 256 / L;
    const bool streams = rows * (int64_t)cols * 4 >= ((int64_t)64 << 20);
    if (NV <= 2 && streams)
        launch_reg<L, NV, (NV <= 2 ? 3 : 1), LOG>(X, Y, rows, cols, st);
    else if (NV <= 2 && rows >= (int64_t)groups * 2 * 512)
        launch_reg<L, NV, (NV <= 2 ? 2 : 1), LOG>(X, Y, rows, cols, st);
    else
        launch_reg<L, NV, 1, LOG>(X, Y, rows, cols, st);
}

template <bool LOG>
static int softmax_dispatch(const float* X, float* Y, int64_t outer, int64_t axis_len, int64_t inner, void* stream) {
    MI355X_REQUIRE(outer >= 0 && axis_len >= 0 && inner >= 0,
                   "softmax: negative extent (outer=%lld axis_len=%lld inner=%lld)",
                   (long long)outer, (long long)axis_len, (long long)inner);
    if (outer == 0 || axis_len == 0 || inner == 0) return MI355X_OK;
    MI355X_REQUIRE(X != nullptr && Y != nullptr, "softmax: null pointer");
    hipStream_t st = static_cast<hipStream_t>(stream);

    if (inner == 1) {
        const int64_t rows = outer, cols = axis_len;
        MI355X_REQUIRE(rows < ((int64_t)1 << 31), "softmax: too many rows (%lld)", (long long)rows);
        const bool vec_ok = (cols % 4 == 0) && ((reinterpret_cast<uintptr_t>(X) & 15) == 0) &&
                            ((reinterpret_cast<uintptr_t>(Y) & 15) == 0);
        if (vec_ok && cols <= 64) launch_reg_unr<16, 1, LOG>(X, Y, rows, (int)cols, st);
        else if (vec_ok && cols <= 128) launch_reg_unr<32, 1, LOG>(X, Y, rows, (int)cols, st);
        else if (vec_ok && cols <= 256) launch_reg_unr<64, 1, LOG>(X, Y, rows, (int)cols, st);
        else if (vec_ok && cols <= 512) launch_reg_unr<64, 2, LOG>(X, Y, rows, (int)cols, st);
        else if (vec_ok && cols <= 1024) launch_reg_unr<64, 4, LOG>(X, Y, rows, (int)cols, st);
        else if (vec_ok && cols <= 2048) launch_reg_unr<64, 8, LOG>(X, Y, rows, (int)cols, st);
        else
            hipLaunchKernelGGL(softmax_rows_loop<LOG>, dim3((unsigned)ceil_div(rows, 256 / WAVE)),
                               dim3(256), 0, st, X, Y, rows, cols);
        return check_launch("softmax_rows");
    }
    const int64_t n = outer * inner;
    MI355X_REQUIRE(ceil_div(n, 256) < ((int64_t)1 << 31), "softmax: grid too large");
    hipLaunchKernelGGL(softmax_strided<LOG>, dim3((unsigned)ceil_div(n, 256)), dim3(256), 0, st, X, Y,
                       outer, axis_len, inner);
    return check_launch("softmax_strided");
}

}  // namespace mi355x

extern "C" int mi355x_softmax_f32(const float* X, float* Y, int64_t outer, int64_t axis_len,
                                  int64_t inner, void* stream) {
    return mi355x::softmax_dispatch<false>(X, Y, outer, axis_len, inner, stream);
}

extern "C" int mi355x_log_softmax_f32(const float* X, float* Y, int64_t outer, int64_t axis_len,
                                      int64_t inner, void* stream) {
    return mi355x::softmax_dispatch<true>(X, Y, outer, axis_len, inner, stream);
}
