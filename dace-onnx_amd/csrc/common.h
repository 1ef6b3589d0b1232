// Shared device/host helpers for the gfx950 kernels of libmi355x_onnx.so.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdarg.h>
#include <stdio.h>

#include "../../include/mi355x_onnx.h"

namespace mi355x {

// ---- host side: per-thread error channel -----------------------------------
int set_error(int code, const char* fmt, ...);
int check_launch(const char* kernel_name);

#define MI355X_REQUIRE(cond, ...)                                              \
    do {                                                                       \
        if (!(cond)) return ::mi355x::set_error(MI355X_ERR_INVALID_ARGUMENT, __VA_ARGS__); \
    } while (0)

static inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Kernel-variant overrides from the MI355X_* environment variables (0 / -1 / false: not set), parsed once
// and again on mi355x_reload_tuning(); CU count of the current device, asked of the runtime once per device.
struct Tuning {
    int gemm_config = -1, gemm_nt_bn = 0, gemm_nt_bm = 0, gemm_nt_bk = 0, gemm_nt_per_cu = 0, gemm_nt_waves = 0, gemm_group_m = 0, gemm_ksplit = -1;
    int conv_config = -1, conv_gather_bn = 0, conv_tail = -1, conv_static_taps = 1, conv_per_cu = 0;
    bool mmi_generic = false;
    int mmi_wgs_per_cu = 0, mmi_tile = 0;
    int attn_waves = 0;
};
Tuning tuning();   // a copy taken under the lock: a reload never changes what a launch in progress reads
int device_cus();

// Workgroup trace, compiled in only with -DMI355X_WG_TRACE (`make trace` builds libmi355x_onnx_trace.so): the contraction
// kernels stamp the wall clock (100 MHz) at the start of a workgroup, at the first and after the last step of its main
// loop and at its end, plus the hardware id of the CU it runs on, into the buffer whose device address the environment
// variable MI355X_WG_TRACE_BUFFER holds (16 x 64-bit words per workgroup: slots 0-3 the four stamps, 4 the hardware id,
// 5 to 11 kernel-specific stamps, 12 and 13 the shader cycle counter at the loop's first and after its last step; unset: no
// stamps). MI355X_WG_TRACE_CAPACITY holds the number of workgroups the buffer has room for: workgroups beyond it write
// nothing, and without it no stamp is written at all. The normal build carries neither the arguments nor the code.
#ifdef MI355X_WG_TRACE
#define MI355X_TRACE_MEMBER unsigned long long* trace; unsigned trace_capacity;
#define MI355X_TRACE_INIT(args) (args).trace = ::mi355x::trace_buffer(&(args).trace_capacity)
#define MI355X_TRACE_ON(args) ((args).trace && threadIdx.x == 0 && blockIdx.x < (args).trace_capacity)
#define MI355X_TRACE_STAMP(args, slot)                                                          \
    do {                                                                                        \
        if (MI355X_TRACE_ON(args)) (args).trace[16 * blockIdx.x + (slot)] = wall_clock64(); \
    } while (0)
#define MI355X_TRACE_CYCLES(args, slot)                                                         \
    do {                                                                                        \
        if (MI355X_TRACE_ON(args)) (args).trace[16 * blockIdx.x + (slot)] = __builtin_readcyclecounter(); \
    } while (0)
#define MI355X_TRACE_HWID(args)                                                                 \
    do {                                                                                        \
        if (MI355X_TRACE_ON(args)) {                                                 \
            unsigned hw_, xcc_;                                                                 \
            asm volatile("s_getreg_b32 %0, hwreg(HW_REG_HW_ID)" : "=s"(hw_));                   \
            asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(xcc_));                 \
            (args).trace[16 * blockIdx.x + 4] = ((unsigned long long)xcc_ << 32) | hw_;          \
        }                                                                                       \
    } while (0)
unsigned long long* trace_buffer(unsigned* capacity);
#else
#define MI355X_TRACE_MEMBER
#define MI355X_TRACE_INIT(args) do {} while (0)
#define MI355X_TRACE_STAMP(args, slot) do {} while (0)
#define MI355X_TRACE_CYCLES(args, slot) do {} while (0)
#define MI355X_TRACE_HWID(args) do {} while (0)
#endif

// ---- device side -------------------------------------------------------------
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef int i32x16 __attribute__((ext_vector_type(16)));

constexpr int WAVE = 64;  // CDNA wavefront width

// DPP lane permutations inside a 16-lane row (no LDS traffic).
template <int CTRL>
__device__ __forceinline__ float dpp_f32(float v) {
    return __builtin_bit_cast(
        float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, false));
}
constexpr int DPP_QUAD_XOR1 = 0xB1;        // quad_perm:[1,0,3,2]
constexpr int DPP_QUAD_XOR2 = 0x4E;        // quad_perm:[2,3,0,1]
constexpr int DPP_ROW_HALF_MIRROR = 0x141; // lane i <-> 7-i inside 8 lanes
constexpr int DPP_ROW_MIRROR = 0x140;      // lane i <-> 15-i inside 16 lanes

__device__ __forceinline__ float readlane_f32(float v, int lane) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
}

// After row16_*: every lane holds the reduction over its 16-lane DPP row.
__device__ __forceinline__ float row16_sum(float v) {
    v += dpp_f32<DPP_QUAD_XOR1>(v);
    v += dpp_f32<DPP_QUAD_XOR2>(v);
    v += dpp_f32<DPP_ROW_HALF_MIRROR>(v);
    v += dpp_f32<DPP_ROW_MIRROR>(v);
    return v;
}
__device__ __forceinline__ float row16_max(float v) {
    v = fmaxf(v, dpp_f32<DPP_QUAD_XOR1>(v));
    v = fmaxf(v, dpp_f32<DPP_QUAD_XOR2>(v));
    v = fmaxf(v, dpp_f32<DPP_ROW_HALF_MIRROR>(v));
    v = fmaxf(v, dpp_f32<DPP_ROW_MIRROR>(v));
    return v;
}
// Reduction over 32 lanes (lanes 0-31 and 32-63 each get their own result).
__device__ __forceinline__ float half32_sum(float v) {
    v = row16_sum(v);
    const int base = (int)(threadIdx.x & 32);
    // the two rows of this half: lanes base and base+16 hold the row totals
    float lo = readlane_f32(v, 0), hi = readlane_f32(v, 16);
    float lo2 = readlane_f32(v, 32), hi2 = readlane_f32(v, 48);
    return base ? (lo2 + hi2) : (lo + hi);
}
__device__ __forceinline__ float half32_max(float v) {
    v = row16_max(v);
    const int base = (int)(threadIdx.x & 32);
    float lo = readlane_f32(v, 0), hi = readlane_f32(v, 16);
    float lo2 = readlane_f32(v, 32), hi2 = readlane_f32(v, 48);
    return base ? fmaxf(lo2, hi2) : fmaxf(lo, hi);
}
// Reduction over the whole 64-lane wave; result is wave-uniform.
__device__ __forceinline__ float wave_sum(float v) {
    v = row16_sum(v);
    return (readlane_f32(v, 0) + readlane_f32(v, 16)) + (readlane_f32(v, 32) + readlane_f32(v, 48));
}
__device__ __forceinline__ float wave_max(float v) {
    v = row16_max(v);
    return fmaxf(fmaxf(readlane_f32(v, 0), readlane_f32(v, 16)),
                 fmaxf(readlane_f32(v, 32), readlane_f32(v, 48)));
}

// erf(x) = sign(x) (1 - 2^q(|x|)), q = t r(t) a degree-8 fit of log2(erfc(t)) on [0, 3.92] weighted by
// erfc (beyond 3.92, erf rounds to +-1 in fp32). Absolute error <= 1.2e-7 over the whole line (checked on
// 2 million points against the double-precision erf), i.e. one fp32 rounding of the "1 + erf" it is used
// in; branch-free, 8 FMAs and one v_exp_f32 instead of the library routine's two-branch evaluation.
__device__ __forceinline__ float erf_f32(float x) {
    const float t = fminf(fabsf(x), 3.92f);
    float q = -4.586598749e-05f;
    q = fmaf(q, t, 4.494983512e-04f);
    q = fmaf(q, t, -1.501731449e-03f);
    q = fmaf(q, t, -7.556890470e-04f);
    q = fmaf(q, t, 2.823820188e-02f);
    q = fmaf(q, t, -1.484750841e-01f);
    q = fmaf(q, t, -9.184176589e-01f);
    q = fmaf(q, t, -1.627908512e+00f);
    return copysignf(1.0f - __builtin_amdgcn_exp2f(q * t), x);
}

// erf Gelu, same formula as the exporter's Div, Erf, Add, Mul, Mul chain
__device__ __forceinline__ float gelu_erf(float v) {
    return 0.5f * v * (1.0f + erf_f32(v * 0.70710678118654752440f));
}

// The unary maps beyond Relu / Gelu / Erf / Sqrt; `op` is a constant at every call site. Softplus and
// Sigmoid are written the way the reference writes them (log(1 + exp(x)), 1 / (1 + exp(-x)):
// pure_implementations.py:696-712), so they also overflow where the reference's do.
__device__ __forceinline__ float unary_math(int op, float x) {
    switch (op) {
        case MI355X_OP_LOG: return logf(x);
        case MI355X_OP_TANH: return tanhf(x);
        case MI355X_OP_SIGMOID: return 1.0f / (1.0f + expf(-x));
        case MI355X_OP_SOFTPLUS: return logf(1.0f + expf(x));
        case MI355X_OP_RECIPROCAL: return 1.0f / x;
        case MI355X_OP_EXP: return expf(x);
        case MI355X_OP_NEG: return -x;
        default: return fabsf(x);   // MI355X_OP_ABS
    }
}

__device__ __forceinline__ float apply_epilogue(float v, int epi, float bias_v) {
    if (epi & MI355X_EPI_BIAS) v += bias_v;
    if (epi & MI355X_EPI_RELU) v = fmaxf(v, 0.0f);
    if (epi & MI355X_EPI_GELU) v = gelu_erf(v);
    return v;
}

}  // namespace mi355x
