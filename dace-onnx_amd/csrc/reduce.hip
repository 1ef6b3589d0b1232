// ONNX ReduceMean / ReduceSum / ReduceMax / ReduceMin along one (collapsed) axis, fp32.
//
// Replaces PureReduceMean.forward, PureReduceSum, PureReduceMax and PureReduceMin
// (daceml/onnx/op_implementations/pure_implementations.py:97-109, 301-343). X is viewed
// as [outer, axis_len, inner]:
//   reduce_rows     inner == 1: one wave per row, 16-byte loads when the row
//                   length allows, DPP wave reduction, no LDS;
//   reduce_strided  otherwise: one thread per (outer, inner) column, lanes
//                   adjacent along `inner` so every access is coalesced.
// ReduceMean only appears in graphs that spell LayerNormalization out (opset < 17
// exports); the fusion pass turns that pattern back into one LayerNormalization
// kernel, so these kernels serve what is left over and are written for
// correctness at full bandwidth on long rows, not for tiny launches.
#include "common.h"

#include <type_traits>

namespace mi355x {

// KIND is one of MI355X_REDUCE_*; sums are kept in T (float per lane of a row, double where a single
// thread adds up a whole column), maxima and minima in float.
template <int KIND, class T>
struct Reducer {
    static constexpr bool SUM = KIND == MI355X_REDUCE_MEAN || KIND == MI355X_REDUCE_SUM;
    static __device__ __forceinline__ T identity() {
        return SUM ? (T)0 : KIND == MI355X_REDUCE_MAX ? (T)-INFINITY : (T)INFINITY;
    }
    static __device__ __forceinline__ T combine(T a, T b) {
        if constexpr (SUM) return a + b;
        else if constexpr (KIND == MI355X_REDUCE_MAX) return a > b ? a : (b > a ? b : (a != a ? a : b));  // NaN wins, as in numpy
        else return a < b ? a : (b < a ? b : (a != a ? a : b));
    }
    static __device__ __forceinline__ float finish(T v, int64_t axis_len) {
        return KIND == MI355X_REDUCE_MEAN ? (float)(v / (T)axis_len) : (float)v;
    }
};

template <int KIND>
__device__ __forceinline__ float wave_combine(float v) {
    using R = Reducer<KIND, float>;
    if constexpr (R::SUM) return wave_sum(v);
    else {
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) v = R::combine(v, __shfl_xor(v, off, WAVE));
        return v;
    }
}

template <int KIND, bool VEC>
__global__ __launch_bounds__(256) void reduce_rows(const float* __restrict__ X, float* __restrict__ Y,
                                                   int64_t rows, int64_t cols) {
    using R = Reducer<KIND, float>;
    const int lane = threadIdx.x % WAVE;
    const int64_t row = (int64_t)blockIdx.x * (256 / WAVE) + threadIdx.x / WAVE;
    if (row >= rows) return;  // whole wave
    const float* x = X + row * cols;
    float s = R::identity();
    if constexpr (VEC) {
        const f32x4* x4 = reinterpret_cast<const f32x4*>(x);
        for (int64_t c = lane; c < cols / 4; c += WAVE) {
            const f32x4 v = x4[c];
            s = R::combine(s, R::combine(R::combine(v.x, v.y), R::combine(v.z, v.w)));
        }
    } else {
        for (int64_t c = lane; c < cols; c += WAVE) s = R::combine(s, x[c]);
    }
    s = wave_combine<KIND>(s);
    if (lane == 0) Y[row] = KIND == MI355X_REDUCE_MEAN ? s * (1.0f / (float)cols) : s;
}

template <int KIND>
__global__ __launch_bounds__(256) void reduce_strided(const float* __restrict__ X, float* __restrict__ Y,
                                                      int64_t outer, int64_t axis_len, int64_t inner) {
    // sums in double, because one thread adds up a whole column
    using T = typename std::conditional<KIND == MI355X_REDUCE_MEAN || KIND == MI355X_REDUCE_SUM, double, float>::type;
    using R = Reducer<KIND, T>;
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= outer * inner) return;
    const int64_t o = idx / inner, i = idx % inner;
    const float* x = X + o * axis_len * inner + i;
    // independent chains for the loads
    T s[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) s[u] = R::identity();
    int64_t a = 0;
    for (; a + 8 <= axis_len; a += 8) {
#pragma unroll
        for (int u = 0; u < 8; ++u) s[u] = R::combine(s[u], (T)x[(a + u) * inner]);
    }
    for (int u = 0; a < axis_len; ++a, ++u) s[u] = R::combine(s[u], (T)x[a * inner]);
    const T all = R::combine(R::combine(R::combine(s[0], s[1]), R::combine(s[2], s[3])),
                             R::combine(R::combine(s[4], s[5]), R::combine(s[6], s[7])));
    Y[idx] = R::finish(all, axis_len);
}

// Reduced axes that are not adjacent (ReduceSum over axes 0 and 2 of [2, 4, 10]): one wave per output element.
// The kept and the reduced axes are given separately, each with its extents and element strides in X; a lane
// walks the reduced index space with stride 64 and decomposes its index over the reduced axes.
struct ReduceNdArgs {
    int n_keep, n_red;
    int64_t keep_shape[8], keep_strides[8], red_shape[8], red_strides[8];
    int64_t n_out, n_red_total;
};

template <int KIND>
__global__ __launch_bounds__(256) void reduce_nd(const float* __restrict__ X, float* __restrict__ Y, ReduceNdArgs p) {
    using R = Reducer<KIND, float>;
    const int lane = threadIdx.x % WAVE;
    const int64_t out = (int64_t)blockIdx.x * (256 / WAVE) + threadIdx.x / WAVE;
    if (out >= p.n_out) return;  // whole wave
    int64_t rem = out, base = 0;
    for (int d = p.n_keep - 1; d >= 0; --d) {
        base += (rem % p.keep_shape[d]) * p.keep_strides[d];
        rem /= p.keep_shape[d];
    }
    float s = R::identity();
    for (int64_t r = lane; r < p.n_red_total; r += WAVE) {
        int64_t q = r, off = base;
        for (int d = p.n_red - 1; d >= 0; --d) {
            off += (q % p.red_shape[d]) * p.red_strides[d];
            q /= p.red_shape[d];
        }
        s = R::combine(s, X[off]);
    }
    s = wave_combine<KIND>(s);
    if (lane == 0) Y[out] = KIND == MI355X_REDUCE_MEAN ? s / (float)p.n_red_total : s;
}

template <int KIND>
static int launch_reduce(const float* X, float* Y, int64_t outer, int64_t axis_len, int64_t inner, hipStream_t st) {
    if (inner == 1) {
        const int64_t blocks = ceil_div(outer, (int64_t)(256 / WAVE));
        MI355X_REQUIRE(blocks < ((int64_t)1 << 31), "reduce: grid too large");
        const bool vec = axis_len % 4 == 0 && (reinterpret_cast<uintptr_t>(X) & 15) == 0;
        if (vec) hipLaunchKernelGGL((reduce_rows<KIND, true>), dim3((unsigned)blocks), dim3(256), 0, st, X, Y, outer, axis_len);
        else hipLaunchKernelGGL((reduce_rows<KIND, false>), dim3((unsigned)blocks), dim3(256), 0, st, X, Y, outer, axis_len);
        return check_launch("reduce_rows");
    }
    const int64_t blocks = ceil_div(outer * inner, (int64_t)256);
    MI355X_REQUIRE(blocks < ((int64_t)1 << 31), "reduce: grid too large");
    hipLaunchKernelGGL(reduce_strided<KIND>, dim3((unsigned)blocks), dim3(256), 0, st, X, Y, outer, axis_len, inner);
    return check_launch("reduce_strided");
}

}  // namespace mi355x

extern "C" int mi355x_reduce_f32(int kind, const float* X, float* Y, int64_t outer, int64_t axis_len,
                                 int64_t inner, void* stream) {
    using namespace mi355x;
    MI355X_REQUIRE(outer >= 0 && axis_len >= 1 && inner >= 0,
                   "reduce: bad extents outer=%lld axis_len=%lld inner=%lld",
                   (long long)outer, (long long)axis_len, (long long)inner);
    MI355X_REQUIRE(kind >= MI355X_REDUCE_MEAN && kind <= MI355X_REDUCE_MIN, "reduce: unknown kind %d", kind);
    if (outer == 0 || inner == 0) return MI355X_OK;
    MI355X_REQUIRE(X && Y, "reduce: null pointer");
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (kind) {
        case MI355X_REDUCE_MEAN: return launch_reduce<MI355X_REDUCE_MEAN>(X, Y, outer, axis_len, inner, st);
        case MI355X_REDUCE_SUM: return launch_reduce<MI355X_REDUCE_SUM>(X, Y, outer, axis_len, inner, st);
        case MI355X_REDUCE_MAX: return launch_reduce<MI355X_REDUCE_MAX>(X, Y, outer, axis_len, inner, st);
        default: return launch_reduce<MI355X_REDUCE_MIN>(X, Y, outer, axis_len, inner, st);
    }
}

extern "C" int mi355x_reduce_mean_f32(const float* X, float* Y, int64_t outer, int64_t axis_len,
                                      int64_t inner, void* stream) {
    return mi355x_reduce_f32(MI355X_REDUCE_MEAN, X, Y, outer, axis_len, inner, stream);
}

extern "C" int mi355x_reduce_nd_f32(int kind, const float* X, float* Y, int ndim, const int64_t* shape,
                                    const int64_t* x_strides, const int64_t* reduced, void* stream) {
    using namespace mi355x;
    MI355X_REQUIRE(kind >= MI355X_REDUCE_MEAN && kind <= MI355X_REDUCE_MIN, "reduce_nd: unknown kind %d", kind);
    MI355X_REQUIRE(ndim >= 1 && ndim <= 8 && shape && x_strides && reduced, "reduce_nd: ndim %d outside [1, 8] or null arrays", ndim);
    ReduceNdArgs p = {};
    p.n_out = 1;
    p.n_red_total = 1;
    for (int d = 0; d < ndim; ++d) {
        MI355X_REQUIRE(shape[d] >= 0, "reduce_nd: negative extent");
        if (reduced[d]) {
            p.red_shape[p.n_red] = shape[d]; p.red_strides[p.n_red++] = x_strides[d]; p.n_red_total *= shape[d];
        } else {
            p.keep_shape[p.n_keep] = shape[d]; p.keep_strides[p.n_keep++] = x_strides[d]; p.n_out *= shape[d];
        }
    }
    MI355X_REQUIRE(p.n_red_total >= 1, "reduce_nd: empty reduction");
    if (p.n_out == 0) return MI355X_OK;
    MI355X_REQUIRE(X && Y, "reduce_nd: null pointer");
    const int64_t blocks = ceil_div(p.n_out, (int64_t)(256 / WAVE));
    MI355X_REQUIRE(blocks < ((int64_t)1 << 31), "reduce_nd: grid too large");
    hipStream_t st = static_cast<hipStream_t>(stream);
    const dim3 grid((unsigned)blocks), block(256);
    switch (kind) {
        case MI355X_REDUCE_MEAN: hipLaunchKernelGGL(reduce_nd<MI355X_REDUCE_MEAN>, grid, block, 0, st, X, Y, p); break;
        case MI355X_REDUCE_SUM: hipLaunchKernelGGL(reduce_nd<MI355X_REDUCE_SUM>, grid, block, 0, st, X, Y, p); break;
        case MI355X_REDUCE_MAX: hipLaunchKernelGGL(reduce_nd<MI355X_REDUCE_MAX>, grid, block, 0, st, X, Y, p); break;
        default: hipLaunchKernelGGL(reduce_nd<MI355X_REDUCE_MIN>, grid, block, 0, st, X, Y, p); break;
    }
    return check_launch("reduce_nd");
}
