// Elementwise ONNX ops (Add/Sub/Mul/Div/Pow, Relu, Gelu, Erf, Sqrt, Log, Tanh,
// Sigmoid, Softplus, Reciprocal, Exp, Neg, Abs) and the Transpose copy, fp32 /
// 4-byte elements.
//
// Each of these is one map in the reference (daceml/onnx/op_implementations/
// pure_implementations.py:23-56,77-94,112-127,275-298,369-379,462-474,696-712). They are HBM
// bound: the kernels below move 16 bytes per lane per access wherever the
// layout allows and otherwise fall back to an index-decomposing gather.
//
// The host collapses adjacent dimensions whose strides are contiguous for
// every operand, so [8,128,768] + [768] becomes a 2-D (rows, cols) problem
// with a row-broadcast operand, and same-shape operands become 1-D.
#include "common.h"

namespace mi355x {

constexpr int MAX_DIMS = 8;

struct IndexMap {
    int ndim;
    int64_t shape[MAX_DIMS];
    int64_t a_strides[MAX_DIMS];
    int64_t b_strides[MAX_DIMS];
};

template <int OP>
__device__ __forceinline__ float apply_op(float a, float b) {
    if constexpr (OP == MI355X_OP_ADD) return a + b;
    else if constexpr (OP == MI355X_OP_SUB) return a - b;
    else if constexpr (OP == MI355X_OP_MUL) return a * b;
    else if constexpr (OP == MI355X_OP_DIV) return a / b;
    else if constexpr (OP == MI355X_OP_POW) return b == 2.0f ? a * a : powf(a, b);
    else if constexpr (OP == MI355X_OP_RELU) return fmaxf(a, 0.0f);
    else if constexpr (OP == MI355X_OP_GELU) return gelu_erf(a);
    else if constexpr (OP == MI355X_OP_ERF) return erff(a);
    else if constexpr (OP == MI355X_OP_SQRT) return sqrtf(a);
    else return unary_math(OP, a);
}
template <int OP>
__device__ __forceinline__ f32x4 apply_op4(f32x4 a, f32x4 b) {
    return f32x4{apply_op<OP>(a.x, b.x), apply_op<OP>(a.y, b.y), apply_op<OP>(a.z, b.z),
                 apply_op<OP>(a.w, b.w)};
}
constexpr bool is_binary(int op) { return op < MI355X_OP_RELU; }

// MODE 0: A and B contiguous (or unary). MODE 1: B is a row vector broadcast
// over rows (index = i % cols). MODE 2: A is the row vector.
template <int OP, int MODE>
__global__ __launch_bounds__(256) void eltwise_vec4(const f32x4* __restrict__ A,
                                                    const f32x4* __restrict__ B,
                                                    f32x4* __restrict__ C, int64_t n4,
                                                    int64_t cols4) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += stride) {
        f32x4 a, b = f32x4{0.f, 0.f, 0.f, 0.f};
        if constexpr (MODE == 2) a = A[i % cols4];
        else a = __builtin_nontemporal_load(A + i);
        if constexpr (is_binary(OP)) {
            if constexpr (MODE == 1) b = B[i % cols4];
            else b = __builtin_nontemporal_load(B + i);
        }
        __builtin_nontemporal_store(apply_op4<OP>(a, b), C + i);
    }
}

template <int OP>
__global__ __launch_bounds__(256) void eltwise_generic(const float* __restrict__ A,
                                                       const float* __restrict__ B,
                                                       float* __restrict__ C, int64_t n,
                                                       IndexMap map) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        int64_t rem = i, ao = 0, bo = 0;
        for (int d = map.ndim - 1; d >= 0; --d) {
            const int64_t idx = rem % map.shape[d];
            rem /= map.shape[d];
            ao += idx * map.a_strides[d];
            bo += idx * map.b_strides[d];
        }
        const float a = A[ao];
        const float b = is_binary(OP) ? B[bo] : 0.0f;
        C[i] = apply_op<OP>(a, b);
    }
}

// Y[i] = X[gather(i)] for 4-byte elements. The innermost output dimension is
// walked by adjacent lanes, so stores are always coalesced; loads are coalesced
// whenever the innermost input stride is 1.
__global__ __launch_bounds__(256) void permute_generic(const uint32_t* __restrict__ X,
                                                       uint32_t* __restrict__ Y, int64_t n,
                                                       IndexMap map) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        int64_t rem = i, xo = 0;
        for (int d = map.ndim - 1; d >= 0; --d) {
            const int64_t idx = rem % map.shape[d];
            rem /= map.shape[d];
            xo += idx * map.a_strides[d];
        }
        Y[i] = X[xo];
    }
}

// Tiled 2-level transpose: output [.., R, C] from input where the output's last
// dim has input stride `s_c` != 1 and some other output dim `R` has input
// stride 1. A 64x64 tile goes through LDS so both sides are coalesced.
__global__ __launch_bounds__(256) void permute_tiled(const uint32_t* __restrict__ X,
                                                     uint32_t* __restrict__ Y, IndexMap map,
                                                     int rdim, int64_t tiles_r, int64_t tiles_c) {
    __shared__ uint32_t tile[64][65];
    const int cdim = map.ndim - 1;
    const int64_t R = map.shape[rdim], Cn = map.shape[cdim];
    int64_t t = blockIdx.x;
    const int64_t tc = t % tiles_c; t /= tiles_c;
    const int64_t tr = t % tiles_r; t /= tiles_r;
    // remaining dims (all except rdim and cdim) decoded from t
    int64_t xo = 0, yo = 0, ystride = 1;
    int64_t y_strides[MAX_DIMS];
    for (int d = map.ndim - 1; d >= 0; --d) { y_strides[d] = ystride; ystride *= map.shape[d]; }
    for (int d = map.ndim - 2; d >= 0; --d) {
        if (d == rdim) continue;
        const int64_t idx = t % map.shape[d];
        t /= map.shape[d];
        xo += idx * map.a_strides[d];
        yo += idx * y_strides[d];
    }
    const int64_t r0 = tr * 64, c0 = tc * 64;
    const int lx = threadIdx.x % 64, ly = threadIdx.x / 64;  // 64 x 4
    // load: adjacent lanes walk r (input stride 1)
    for (int j = ly; j < 64; j += 4) {
        const int64_t r = r0 + lx, c = c0 + j;
        if (r < R && c < Cn) tile[j][lx] = X[xo + r * map.a_strides[rdim] + c * map.a_strides[cdim]];
    }
    __syncthreads();
    // store: adjacent lanes walk c (output stride 1)
    for (int j = ly; j < 64; j += 4) {
        const int64_t r = r0 + j, c = c0 + lx;
        if (r < R && c < Cn) Y[yo + r * y_strides[rdim] + c] = tile[lx][j];
    }
}

// ONNX Cast: Y[i] = (TO)X[i]; to bool is X[i] != 0 (stored as one byte). VEC: four elements per lane and
// access (both pointers aligned to four elements), the last n % 4 elements one by one.
template <class T> using Vec4 = T __attribute__((ext_vector_type(4)));

template <class FROM, class TO, bool TO_BOOL>
__device__ __forceinline__ TO cast_one(FROM v) {
    if constexpr (TO_BOOL) return (TO)(v != (FROM)0);
    else return (TO)v;
}

template <class FROM, class TO, bool TO_BOOL, bool VEC>
__global__ __launch_bounds__(256) void cast_kernel(const FROM* __restrict__ X, TO* __restrict__ Y, int64_t n) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x, first = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if constexpr (VEC) {
        const Vec4<FROM>* x4 = reinterpret_cast<const Vec4<FROM>*>(X);
        Vec4<TO>* y4 = reinterpret_cast<Vec4<TO>*>(Y);
        for (int64_t i = first; i < n / 4; i += stride) {
            const Vec4<FROM> v = x4[i];
            y4[i] = Vec4<TO>{cast_one<FROM, TO, TO_BOOL>(v.x), cast_one<FROM, TO, TO_BOOL>(v.y),
                             cast_one<FROM, TO, TO_BOOL>(v.z), cast_one<FROM, TO, TO_BOOL>(v.w)};
        }
        for (int64_t i = (n / 4) * 4 + first; i < n; i += stride) Y[i] = cast_one<FROM, TO, TO_BOOL>(X[i]);
    } else {
        for (int64_t i = first; i < n; i += stride) Y[i] = cast_one<FROM, TO, TO_BOOL>(X[i]);
    }
}

// Merge adjacent dims (d, d+1) when both operands step through them as one.
static void collapse(IndexMap& m, bool use_b) {
    // drop size-1 dims
    int k = 0;
    for (int d = 0; d < m.ndim; ++d) {
        if (m.shape[d] == 1) continue;
        m.shape[k] = m.shape[d]; m.a_strides[k] = m.a_strides[d]; m.b_strides[k] = m.b_strides[d];
        ++k;
    }
    if (k == 0) { m.shape[0] = 1; m.a_strides[0] = 0; m.b_strides[0] = 0; k = 1; }
    m.ndim = k;
    // merge
    int w = 0;
    for (int d = 1; d < m.ndim; ++d) {
        const bool a_ok = m.a_strides[w] == m.a_strides[d] * m.shape[d];
        const bool b_ok = !use_b || m.b_strides[w] == m.b_strides[d] * m.shape[d];
        if (a_ok && b_ok) {
            m.shape[w] *= m.shape[d];
            m.a_strides[w] = m.a_strides[d];
            m.b_strides[w] = m.b_strides[d];
        } else {
            ++w;
            m.shape[w] = m.shape[d]; m.a_strides[w] = m.a_strides[d]; m.b_strides[w] = m.b_strides[d];
        }
    }
    m.ndim = w + 1;
}

static inline unsigned grid_for(int64_t work_items) {
    // grid-stride loops: enough blocks for >= 8 per CU on a 256-CU part, never more than needed
    const int64_t want = ceil_div(work_items, 256);
    return (unsigned)(want < 1 ? 1 : (want > 65536 ? 65536 : want));
}

template <int OP>
static int launch_eltwise(const float* A, const float* B, float* C, IndexMap m, hipStream_t st) {
    int64_t n = 1;
    for (int d = 0; d < m.ndim; ++d) n *= m.shape[d];
    if (n == 0) return MI355X_OK;
    const bool bin = is_binary(OP);
    collapse(m, bin);
    auto aligned = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
    const bool al = aligned(A) && aligned(C) && (!bin || aligned(B));
    const f32x4* A4 = reinterpret_cast<const f32x4*>(A);
    const f32x4* B4 = reinterpret_cast<const f32x4*>(B);
    f32x4* C4 = reinterpret_cast<f32x4*>(C);
    if (al && m.ndim == 1 && m.a_strides[0] == 1 && (!bin || m.b_strides[0] == 1) && n % 4 == 0) {
        hipLaunchKernelGGL((eltwise_vec4<OP, 0>), dim3(grid_for(n / 4)), dim3(256), 0, st, A4, B4, C4, n / 4, (int64_t)1);
    } else if (bin && al && m.ndim == 2 && m.shape[1] % 4 == 0 && m.a_strides[1] == 1 &&
               m.b_strides[1] == 1 && m.a_strides[0] == m.shape[1] && m.b_strides[0] == 0) {
        hipLaunchKernelGGL((eltwise_vec4<OP, 1>), dim3(grid_for(n / 4)), dim3(256), 0, st, A4, B4, C4, n / 4, m.shape[1] / 4);
    } else if (bin && al && m.ndim == 2 && m.shape[1] % 4 == 0 && m.a_strides[1] == 1 &&
               m.b_strides[1] == 1 && m.b_strides[0] == m.shape[1] && m.a_strides[0] == 0) {
        hipLaunchKernelGGL((eltwise_vec4<OP, 2>), dim3(grid_for(n / 4)), dim3(256), 0, st, A4, B4, C4, n / 4, m.shape[1] / 4);
    } else {
        hipLaunchKernelGGL((eltwise_generic<OP>), dim3(grid_for(n)), dim3(256), 0, st, A, B, C, n, m);
    }
    return check_launch("eltwise");
}

}  // namespace mi355x

extern "C" int mi355x_eltwise_f32(int op, const float* A, const float* B, float* C, int ndim,
                                  const int64_t* shape, const int64_t* a_strides,
                                  const int64_t* b_strides, void* stream) {
    using namespace mi355x;
    MI355X_REQUIRE(ndim >= 0 && ndim <= MAX_DIMS, "eltwise: ndim %d outside [0, %d]", ndim, MAX_DIMS);
    const bool bin = is_binary(op);
    MI355X_REQUIRE(ndim == 0 || (shape && a_strides && (!bin || b_strides)), "eltwise: null shape/strides");
    int64_t total = 1;
    for (int d = 0; d < ndim; ++d) total *= shape[d] > 0 ? shape[d] : 0;
    if (total == 0) {
        for (int d = 0; d < ndim; ++d) MI355X_REQUIRE(shape[d] >= 0, "eltwise: negative extent");
        return MI355X_OK;
    }
    MI355X_REQUIRE(A && C, "eltwise: null pointer");
    MI355X_REQUIRE(!bin || B, "eltwise: binary op %d needs B", op);
    IndexMap m;
    m.ndim = ndim == 0 ? 1 : ndim;
    for (int d = 0; d < MAX_DIMS; ++d) { m.shape[d] = 1; m.a_strides[d] = 0; m.b_strides[d] = 0; }
    for (int d = 0; d < ndim; ++d) {
        MI355X_REQUIRE(shape[d] >= 0, "eltwise: negative extent");
        m.shape[d] = shape[d];
        m.a_strides[d] = a_strides[d];
        m.b_strides[d] = bin ? b_strides[d] : 0;
    }
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (op) {
        case MI355X_OP_ADD: return launch_eltwise<MI355X_OP_ADD>(A, B, C, m, st);
        case MI355X_OP_SUB: return launch_eltwise<MI355X_OP_SUB>(A, B, C, m, st);
        case MI355X_OP_MUL: return launch_eltwise<MI355X_OP_MUL>(A, B, C, m, st);
        case MI355X_OP_DIV: return launch_eltwise<MI355X_OP_DIV>(A, B, C, m, st);
        case MI355X_OP_POW: return launch_eltwise<MI355X_OP_POW>(A, B, C, m, st);
        case MI355X_OP_RELU: return launch_eltwise<MI355X_OP_RELU>(A, B, C, m, st);
        case MI355X_OP_GELU: return launch_eltwise<MI355X_OP_GELU>(A, B, C, m, st);
        case MI355X_OP_ERF: return launch_eltwise<MI355X_OP_ERF>(A, B, C, m, st);
        case MI355X_OP_SQRT: return launch_eltwise<MI355X_OP_SQRT>(A, B, C, m, st);
        case MI355X_OP_LOG: return launch_eltwise<MI355X_OP_LOG>(A, B, C, m, st);
        case MI355X_OP_TANH: return launch_eltwise<MI355X_OP_TANH>(A, B, C, m, st);
        case MI355X_OP_SIGMOID: return launch_eltwise<MI355X_OP_SIGMOID>(A, B, C, m, st);
        case MI355X_OP_SOFTPLUS: return launch_eltwise<MI355X_OP_SOFTPLUS>(A, B, C, m, st);
        case MI355X_OP_RECIPROCAL: return launch_eltwise<MI355X_OP_RECIPROCAL>(A, B, C, m, st);
        case MI355X_OP_EXP: return launch_eltwise<MI355X_OP_EXP>(A, B, C, m, st);
        case MI355X_OP_NEG: return launch_eltwise<MI355X_OP_NEG>(A, B, C, m, st);
        case MI355X_OP_ABS: return launch_eltwise<MI355X_OP_ABS>(A, B, C, m, st);
        default: return set_error(MI355X_ERR_INVALID_ARGUMENT, "eltwise: unknown op %d", op);
    }
}

namespace mi355x {

template <class FROM, class TO, bool TO_BOOL>
static void launch_cast_to(const void* X, void* Y, int64_t n, hipStream_t st) {
    const FROM* x = static_cast<const FROM*>(X);
    TO* y = static_cast<TO*>(Y);
    const bool vec = reinterpret_cast<uintptr_t>(X) % (4 * sizeof(FROM)) == 0 && reinterpret_cast<uintptr_t>(Y) % (4 * sizeof(TO)) == 0 && n >= 4;
    if (vec) hipLaunchKernelGGL((cast_kernel<FROM, TO, TO_BOOL, true>), dim3(grid_for(n / 4)), dim3(256), 0, st, x, y, n);
    else hipLaunchKernelGGL((cast_kernel<FROM, TO, TO_BOOL, false>), dim3(grid_for(n)), dim3(256), 0, st, x, y, n);
}

template <class FROM>
static int launch_cast_from(const void* X, void* Y, int to_type, int64_t n, hipStream_t st) {
    switch (to_type) {
        case MI355X_TYPE_FLOAT: launch_cast_to<FROM, float, false>(X, Y, n, st); break;
        case MI355X_TYPE_DOUBLE: launch_cast_to<FROM, double, false>(X, Y, n, st); break;
        case MI355X_TYPE_INT32: launch_cast_to<FROM, int32_t, false>(X, Y, n, st); break;
        case MI355X_TYPE_INT64: launch_cast_to<FROM, int64_t, false>(X, Y, n, st); break;
        case MI355X_TYPE_INT8: launch_cast_to<FROM, int8_t, false>(X, Y, n, st); break;
        case MI355X_TYPE_UINT8: launch_cast_to<FROM, uint8_t, false>(X, Y, n, st); break;
        case MI355X_TYPE_BOOL: launch_cast_to<FROM, uint8_t, true>(X, Y, n, st); break;
        default: return set_error(MI355X_ERR_INVALID_ARGUMENT, "cast: unsupported target type %d", to_type);
    }
    return check_launch("cast");
}

}  // namespace mi355x

extern "C" int mi355x_cast(const void* X, int from_type, void* Y, int to_type, int64_t n, void* stream) {
    using namespace mi355x;
    MI355X_REQUIRE(n >= 0, "cast: negative element count %lld", (long long)n);
    if (n == 0) return MI355X_OK;
    MI355X_REQUIRE(X && Y, "cast: null pointer");
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (from_type) {
        case MI355X_TYPE_FLOAT: return launch_cast_from<float>(X, Y, to_type, n, st);
        case MI355X_TYPE_DOUBLE: return launch_cast_from<double>(X, Y, to_type, n, st);
        case MI355X_TYPE_INT32: return launch_cast_from<int32_t>(X, Y, to_type, n, st);
        case MI355X_TYPE_INT64: return launch_cast_from<int64_t>(X, Y, to_type, n, st);
        case MI355X_TYPE_INT8: return launch_cast_from<int8_t>(X, Y, to_type, n, st);
        case MI355X_TYPE_UINT8:
        case MI355X_TYPE_BOOL: return launch_cast_from<uint8_t>(X, Y, to_type, n, st);
        default: return set_error(MI355X_ERR_INVALID_ARGUMENT, "cast: unsupported source type %d", from_type);
    }
}

extern "C" int mi355x_permute_b32(const void* X, void* Y, int ndim, const int64_t* shape,
                                  const int64_t* x_strides, void* stream) {
    using namespace mi355x;
    MI355X_REQUIRE(ndim >= 0 && ndim <= MAX_DIMS, "permute: ndim %d outside [0, %d]", ndim, MAX_DIMS);
    MI355X_REQUIRE(ndim == 0 || (shape && x_strides), "permute: null shape/strides");
    IndexMap m;
    m.ndim = ndim == 0 ? 1 : ndim;
    for (int d = 0; d < MAX_DIMS; ++d) { m.shape[d] = 1; m.a_strides[d] = 0; m.b_strides[d] = 0; }
    int64_t n = 1;
    for (int d = 0; d < ndim; ++d) {
        MI355X_REQUIRE(shape[d] >= 0, "permute: negative extent");
        m.shape[d] = shape[d];
        m.a_strides[d] = x_strides[d];
        n *= shape[d];
    }
    if (n == 0) return MI355X_OK;
    MI355X_REQUIRE(X && Y, "permute: null pointer");
    collapse(m, false);
    hipStream_t st = static_cast<hipStream_t>(stream);
    const uint32_t* x = static_cast<const uint32_t*>(X);
    uint32_t* y = static_cast<uint32_t*>(Y);
    // a dim with input stride 1 that is not the output's last dim -> tiled transpose
    int rdim = -1;
    if (m.ndim >= 2 && m.a_strides[m.ndim - 1] != 1) {
        for (int d = 0; d < m.ndim - 1; ++d)
            if (m.a_strides[d] == 1 && m.shape[d] >= 16) rdim = d;
    }
    if (rdim >= 0 && m.shape[m.ndim - 1] >= 16) {
        const int64_t tiles_r = ceil_div(m.shape[rdim], 64), tiles_c = ceil_div(m.shape[m.ndim - 1], 64);
        int64_t blocks = tiles_r * tiles_c;
        for (int d = 0; d < m.ndim - 1; ++d) if (d != rdim) blocks *= m.shape[d];
        MI355X_REQUIRE(blocks < ((int64_t)1 << 31), "permute: grid too large");
        hipLaunchKernelGGL(permute_tiled, dim3((unsigned)blocks), dim3(256), 0, st, x, y, m, rdim, tiles_r, tiles_c);
    } else {
        hipLaunchKernelGGL(permute_generic, dim3(grid_for(n)), dim3(256), 0, st, x, y, n, m);
    }
    return check_launch("permute");
}
