// A chain (or small DAG) of elementwise ONNX nodes as one launch, fp32.
//
// The reference runs every elementwise node as its own map with a materialised result
// (daceml/onnx/op_implementations/pure_implementations.py:41-127, 462-474) and relies on DaCe's
// map / tasklet fusion (daceml/transformation/tasklet_fusion.py) to merge them afterwards. Here the
// fusion pass hands the whole group to this kernel as a short program: every tensor operand is read
// once, the result is written once, intermediates live in registers.
//
// Operands of an instruction are registers (results of earlier instructions), tensor inputs (same
// shape as the result, contiguous), vector inputs (one value per position of the last axis, broadcast
// over the rest) or immediates (scalar constants). The program is the same for every element, so all
// decoding is scalar control flow; per 16 bytes of every operand a lane executes the program once.
#include "common.h"

namespace mi355x {

struct ProgramArgs {
    const float* tensors[MI355X_PROGRAM_MAX_TENSORS];
    const float* vectors[MI355X_PROGRAM_MAX_VECTORS];
    float* Y;
    int64_t n, last_dim;
    int n_tensors, n_vectors, n_instr;
    uint32_t col_step;   // (grid stride in floats) mod last_dim
    uint32_t program[MI355X_PROGRAM_MAX_INSTR];
    float imm[MI355X_PROGRAM_MAX_IMM];
};

template <class V> struct Lanes;
template <> struct Lanes<float> {
    static constexpr int W = 1;
    static __device__ __forceinline__ float splat(float v) { return v; }
    template <class F> static __device__ __forceinline__ float map(F f, float a, float b) { return f(a, b); }
};
template <> struct Lanes<f32x4> {
    static constexpr int W = 4;
    static __device__ __forceinline__ f32x4 splat(float v) { return f32x4{v, v, v, v}; }
    template <class F> static __device__ __forceinline__ f32x4 map(F f, f32x4 a, f32x4 b) {
        return f32x4{f(a.x, b.x), f(a.y, b.y), f(a.z, b.z), f(a.w, b.w)};
    }
};

template <class V>
__device__ __forceinline__ V program_op(int op, V a, V b) {
    using L = Lanes<V>;
    switch (op) {  // uniform
        case MI355X_OP_ADD: return a + b;
        case MI355X_OP_SUB: return a - b;
        case MI355X_OP_MUL: return a * b;
        case MI355X_OP_DIV: return L::map([](float x, float y) { return x / y; }, a, b);
        case MI355X_OP_POW: return L::map([](float x, float y) { return powf(x, y); }, a, b);
        case MI355X_OP_RELU: return L::map([](float x, float) { return fmaxf(x, 0.0f); }, a, b);
        case MI355X_OP_GELU: return L::map([](float x, float) { return gelu_erf(x); }, a, b);
        case MI355X_OP_ERF: return L::map([](float x, float) { return erff(x); }, a, b);
        case MI355X_OP_SQRT: return L::map([](float x, float) { return sqrtf(x); }, a, b);
        case MI355X_OP_LOG: return L::map([](float x, float) { return unary_math(MI355X_OP_LOG, x); }, a, b);
        case MI355X_OP_TANH: return L::map([](float x, float) { return unary_math(MI355X_OP_TANH, x); }, a, b);
        case MI355X_OP_SIGMOID: return L::map([](float x, float) { return unary_math(MI355X_OP_SIGMOID, x); }, a, b);
        case MI355X_OP_SOFTPLUS: return L::map([](float x, float) { return unary_math(MI355X_OP_SOFTPLUS, x); }, a, b);
        case MI355X_OP_RECIPROCAL: return L::map([](float x, float) { return unary_math(MI355X_OP_RECIPROCAL, x); }, a, b);
        case MI355X_OP_EXP: return L::map([](float x, float) { return unary_math(MI355X_OP_EXP, x); }, a, b);
        case MI355X_OP_NEG: return L::map([](float x, float) { return unary_math(MI355X_OP_NEG, x); }, a, b);
        case MI355X_OP_ABS: return L::map([](float x, float) { return unary_math(MI355X_OP_ABS, x); }, a, b);
        default: return a;  // MI355X_OP_COPY
    }
}

// NT / NV / NR: how many tensor, vector and register slots this instantiation keeps. Registers that are never
// used still cost occupancy (the loop lives on loads in flight), so short programs -- most of them -- run a
// variant with 2 / 2 / 4 slots at twice the occupancy of the full 4 / 4 / 8 one.
template <class V, int NT, int NV, int NR>
__global__ __launch_bounds__(256) void eltwise_program_kernel(ProgramArgs p) {
    using L = Lanes<V>;
    constexpr int W = L::W;
    const int64_t count = p.n / W, stride = (int64_t)gridDim.x * blockDim.x;
    const int64_t first = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    // position along the last axis, advanced by (stride W) mod last_dim per trip instead of a 64-bit modulo per trip
    uint32_t col = p.n_vectors > 0 ? (uint32_t)((first * W) % p.last_dim) : 0u;
    for (int64_t i = first; i < count; i += stride) {
        V t[NT], v[NV], r[NR];   // only ever indexed with constants
#pragma unroll
        for (int k = 0; k < NT; ++k) t[k] = L::splat(0.f);
#pragma unroll
        for (int k = 0; k < NV; ++k) v[k] = L::splat(0.f);
#pragma unroll
        for (int k = 0; k < NR; ++k) r[k] = L::splat(0.f);
#pragma unroll
        for (int k = 0; k < NT; ++k)
            if (k < p.n_tensors) t[k] = __builtin_nontemporal_load(reinterpret_cast<const V*>(p.tensors[k]) + i);   // uniform
#pragma unroll
        for (int k = 0; k < NV; ++k)
            if (k < p.n_vectors) v[k] = *reinterpret_cast<const V*>(p.vectors[k] + col);                              // uniform
        col += p.col_step;
        col = col >= (uint32_t)p.last_dim ? col - (uint32_t)p.last_dim : col;
        // Operand fetch and register write are chains of selects / scalar branches over named registers.
        // (Indexing one register file with the uniform index instead -- which the compiler turns into indexed
        // register addressing -- was measured 25 % slower.)
        auto fetch = [&](uint32_t enc) __attribute__((always_inline)) -> V {
            const uint32_t idx = enc & 63u;
            V out = L::splat(0.f);
            // scalar branches, one taken: the empty asm keeps the compiler from turning the cases into a chain of
            // per-lane selects over every candidate register
#define MI355X_PICK(arr, n)                                                   \
            _Pragma("unroll") for (int k = 0; k < (n); ++k)                   \
                if (idx == (uint32_t)k) { out = arr[k]; asm volatile(""); }
            switch (enc >> 6) {  // uniform
                case MI355X_PROGRAM_REG: MI355X_PICK(r, NR) break;
                case MI355X_PROGRAM_TENSOR: MI355X_PICK(t, NT) break;
                case MI355X_PROGRAM_VECTOR: MI355X_PICK(v, NV) break;
                default: out = L::splat(p.imm[idx & (MI355X_PROGRAM_MAX_IMM - 1)]);
            }
#undef MI355X_PICK
            return out;
        };
        V result = L::splat(0.f);
        for (int pc = 0; pc < p.n_instr; ++pc) {
            const uint32_t ins = p.program[pc];
            result = program_op<V>((int)(ins & 255u), fetch((ins >> 16) & 255u), fetch(ins >> 24));
            const uint32_t dst = (ins >> 8) & 255u;
#pragma unroll
            for (int k = 0; k < NR; ++k) if (dst == (uint32_t)k) { r[k] = result; asm volatile(""); }   // uniform
        }
        __builtin_nontemporal_store(result, reinterpret_cast<V*>(p.Y) + i);
    }
}

}  // namespace mi355x

extern "C" int mi355x_eltwise_program_f32(const float* const* tensors, int n_tensors,
                                          const float* const* vectors, int n_vectors, float* Y, int64_t n,
                                          int64_t last_dim, const uint32_t* program, int n_instr,
                                          const float* immediates, int n_immediates, void* stream) {
    using namespace mi355x;
    MI355X_REQUIRE(n >= 0 && last_dim >= 1 && last_dim < ((int64_t)1 << 31), "eltwise_program: bad extents n=%lld last_dim=%lld",
                   (long long)n, (long long)last_dim);
    MI355X_REQUIRE(n_tensors >= 0 && n_tensors <= MI355X_PROGRAM_MAX_TENSORS && n_vectors >= 0 &&
                       n_vectors <= MI355X_PROGRAM_MAX_VECTORS && n_instr >= 1 && n_instr <= MI355X_PROGRAM_MAX_INSTR &&
                       n_immediates >= 0 && n_immediates <= MI355X_PROGRAM_MAX_IMM,
                   "eltwise_program: %d tensors, %d vectors, %d instructions, %d immediates exceed the limits",
                   n_tensors, n_vectors, n_instr, n_immediates);
    MI355X_REQUIRE(n_tensors + n_vectors >= 1, "eltwise_program: no input");
    if (n == 0) return MI355X_OK;
    MI355X_REQUIRE(n % last_dim == 0, "eltwise_program: n=%lld is not a multiple of last_dim=%lld", (long long)n,
                   (long long)last_dim);
    MI355X_REQUIRE(Y && program && (n_tensors == 0 || tensors) && (n_vectors == 0 || vectors) &&
                       (n_immediates == 0 || immediates), "eltwise_program: null pointer");
    ProgramArgs p = {};
    p.Y = Y; p.n = n; p.last_dim = last_dim;
    p.n_tensors = n_tensors; p.n_vectors = n_vectors; p.n_instr = n_instr;
    bool vec = n % 4 == 0 && last_dim % 4 == 0 && (reinterpret_cast<uintptr_t>(Y) & 15) == 0;
    for (int k = 0; k < n_tensors; ++k) {
        MI355X_REQUIRE(tensors[k], "eltwise_program: null tensor %d", k);
        p.tensors[k] = tensors[k];
        vec = vec && (reinterpret_cast<uintptr_t>(tensors[k]) & 15) == 0;
    }
    for (int k = 0; k < n_vectors; ++k) {
        MI355X_REQUIRE(vectors[k], "eltwise_program: null vector %d", k);
        p.vectors[k] = vectors[k];
        vec = vec && (reinterpret_cast<uintptr_t>(vectors[k]) & 15) == 0;
    }
    for (int k = 0; k < n_immediates; ++k) p.imm[k] = immediates[k];
    int written = 0;   // registers written so far, as a bit mask: an instruction may only read those
    uint32_t max_reg = 0;
    for (int pc = 0; pc < n_instr; ++pc) {
        const uint32_t ins = program[pc], op = ins & 255u, dst = (ins >> 8) & 255u;
        const bool known = op <= MI355X_OP_POW || (op >= MI355X_OP_RELU && op <= MI355X_OP_LAST);
        MI355X_REQUIRE(known && dst < 8, "eltwise_program: instruction %d (0x%08x) has an unknown op or register", pc, ins);
        const uint32_t operands[2] = {(ins >> 16) & 255u, ins >> 24};
        for (int k = 0; k < (op <= MI355X_OP_POW ? 2 : 1); ++k) {
            const uint32_t kind = operands[k] >> 6, idx = operands[k] & 63u;
            const bool ok = kind == MI355X_PROGRAM_REG ? (idx < 8 && (written >> idx & 1)) :
                            kind == MI355X_PROGRAM_TENSOR ? (int)idx < n_tensors :
                            kind == MI355X_PROGRAM_VECTOR ? (int)idx < n_vectors : (int)idx < n_immediates;
            MI355X_REQUIRE(ok, "eltwise_program: instruction %d (0x%08x) reads an operand that does not exist", pc, ins);
        }
        written |= 1 << dst;
        max_reg = dst > max_reg ? dst : max_reg;
        // unary ops never look at their second operand: point it at a register that exists
        p.program[pc] = op > MI355X_OP_POW ? (ins & 0x00ffffffu) : ins;
    }
    const int64_t count = vec ? n / 4 : n;
    int64_t blocks = ceil_div(count, (int64_t)256);
    const int64_t max_blocks = (int64_t)device_cus() * 16;
    if (max_blocks > 0 && blocks > max_blocks) blocks = max_blocks;
    p.col_step = (uint32_t)((blocks * 256 * (vec ? 4 : 1)) % last_dim);
    hipStream_t st = static_cast<hipStream_t>(stream);
    const bool small = n_tensors <= 2 && n_vectors <= 2 && max_reg < 4;
    if (vec && small) hipLaunchKernelGGL((eltwise_program_kernel<f32x4, 2, 2, 4>), dim3((unsigned)blocks), dim3(256), 0, st, p);
    else if (vec) hipLaunchKernelGGL((eltwise_program_kernel<f32x4, 4, 4, 8>), dim3((unsigned)blocks), dim3(256), 0, st, p);
    else hipLaunchKernelGGL((eltwise_program_kernel<float, 4, 4, 8>), dim3((unsigned)blocks), dim3(256), 0, st, p);
    return check_launch("eltwise_program_kernel");
}
