/*
 * C restatement of the reference's CPU ("pure") expansions -- TEST INFRASTRUCTURE
 * ONLY: the checker for the HIP kernels and the CPU baseline timed next to them.
 * Nothing in the product library links or calls this file.
 *
 * Each function keeps the PASS STRUCTURE of the SDFG the reference generates
 * (one loop nest per map, materialised temporaries between them, OpenMP over
 * the outer map dimensions as DaCe's CPU codegen does), so its run time is a
 * fair stand-in for the reference's CPU path.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* PureConv2D, daceml/onnx/op_implementations/img_op_implementations.py:246-293:
 * zero_init / broadcast(bias) map, then one 7-dimensional map accumulating
 * filter*image into Y with a "+" write-conflict resolution; outer map
 * (b, m, out_y, out_x) parallel, inner (cin, hx, hy) serial (:312-324).
 * The stride / pad / dilation terms of the ONNX specification are included
 * (the reference drops the stride at :278 and refuses pads at :201-203). */
void oracle_conv2d_f32(const float* X, const float* W, const float* B, float* Y,
                       int64_t N, int64_t C, int64_t H, int64_t Wd, int64_t M, int64_t KH, int64_t KW,
                       const int64_t* pads, const int64_t* strides, const int64_t* dil) {
    const int64_t OH = (H + pads[0] + pads[2] - ((KH - 1) * dil[0] + 1)) / strides[0] + 1;
    const int64_t OW = (Wd + pads[1] + pads[3] - ((KW - 1) * dil[1] + 1)) / strides[1] + 1;
#pragma omp parallel for collapse(4) schedule(static)
    for (int64_t b = 0; b < N; ++b)
        for (int64_t m = 0; m < M; ++m)
            for (int64_t oy = 0; oy < OH; ++oy)
                for (int64_t ox = 0; ox < OW; ++ox)
                    Y[((b * M + m) * OH + oy) * OW + ox] = B ? B[m] : 0.0f;
#pragma omp parallel for collapse(4) schedule(static)
    for (int64_t b = 0; b < N; ++b)
        for (int64_t m = 0; m < M; ++m)
            for (int64_t oy = 0; oy < OH; ++oy)
                for (int64_t ox = 0; ox < OW; ++ox) {
                    float* out = &Y[((b * M + m) * OH + oy) * OW + ox];
                    for (int64_t cin = 0; cin < C; ++cin)
                        for (int64_t hx = 0; hx < KH; ++hx)
                            for (int64_t hy = 0; hy < KW; ++hy) {
                                const int64_t iy = oy * strides[0] - pads[0] + hx * dil[0];
                                const int64_t ix = ox * strides[1] - pads[1] + hy * dil[1];
                                if (iy < 0 || iy >= H || ix < 0 || ix >= Wd) continue;
                                *out += W[((m * C + cin) * KH + hx) * KW + hy] *
                                        X[((b * C + cin) * H + iy) * Wd + ix];
                            }
                }
}

/* PureSoftmax, pure_implementations.py:358-364, last axis: five maps
 * (max, subtract+exp, sum, divide) with the temporaries max[], exp_arr[], sum[]. */
void oracle_softmax_f32(const float* X, float* Y, int64_t rows, int64_t cols) {
    float* mx = (float*)malloc(sizeof(float) * (size_t)rows);
    float* sm = (float*)malloc(sizeof(float) * (size_t)rows);
    float* ex = (float*)malloc(sizeof(float) * (size_t)(rows * cols));
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; ++r) {
        float m = -INFINITY;
        for (int64_t c = 0; c < cols; ++c) m = fmaxf(m, X[r * cols + c]);
        mx[r] = m;
    }
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; ++r)
        for (int64_t c = 0; c < cols; ++c) ex[r * cols + c] = expf(X[r * cols + c] - mx[r]);
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; ++r) {
        float s = 0.0f;
        for (int64_t c = 0; c < cols; ++c) s += ex[r * cols + c];
        sm[r] = s;
    }
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; ++r)
        for (int64_t c = 0; c < cols; ++c) Y[r * cols + c] = ex[r * cols + c] / sm[r];
    free(mx); free(sm); free(ex);
}

/* LayerNormalization as the exporter's chain, one loop nest and one temporary per
 * node: ReduceMean, Sub, Pow, ReduceMean, Add, Sqrt, Div, Mul, Add
 * (pure_implementations.py:97-109,82-84,59-74,77-79,41-56,92-94). */
void oracle_layernorm_f32(const float* X, const float* gamma, const float* beta, float* Y,
                          int64_t rows, int64_t cols, float eps) {
    const size_t n = (size_t)(rows * cols);
    float* mean = (float*)malloc(sizeof(float) * (size_t)rows);
    float* var = (float*)malloc(sizeof(float) * (size_t)rows);
    float* cen = (float*)malloc(sizeof(float) * n);
    float* sq = (float*)malloc(sizeof(float) * n);
    float* t = (float*)malloc(sizeof(float) * n);
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; ++r) { float s = 0; for (int64_t c = 0; c < cols; ++c) s += X[r * cols + c]; mean[r] = s / (float)cols; }
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; ++r) for (int64_t c = 0; c < cols; ++c) cen[r * cols + c] = X[r * cols + c] - mean[r];
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < (int64_t)n; ++i) sq[i] = powf(cen[i], 2.0f);
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; ++r) { float s = 0; for (int64_t c = 0; c < cols; ++c) s += sq[r * cols + c]; var[r] = s / (float)cols; }
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; ++r) var[r] = var[r] + eps;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; ++r) var[r] = sqrtf(var[r]);
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; ++r) for (int64_t c = 0; c < cols; ++c) t[r * cols + c] = cen[r * cols + c] / var[r];
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; ++r) for (int64_t c = 0; c < cols; ++c) t[r * cols + c] = t[r * cols + c] * gamma[c];
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; ++r) for (int64_t c = 0; c < cols; ++c) Y[r * cols + c] = t[r * cols + c] + (beta ? beta[c] : 0.0f);
    free(mean); free(var); free(cen); free(sq); free(t);
}

/* Gelu as the exporter's chain Div(sqrt 2), Erf, Add(1), Mul(x), Mul(0.5): five maps. */
void oracle_gelu_f32(const float* X, float* Y, int64_t n) {
    float* t = (float*)malloc(sizeof(float) * (size_t)n);
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; ++i) t[i] = X[i] / 1.41421356237309504880f;
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; ++i) t[i] = erff(t[i]);
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; ++i) t[i] = t[i] + 1.0f;
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; ++i) t[i] = X[i] * t[i];
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; ++i) Y[i] = t[i] * 0.5f;
    free(t);
}

/* ONNX MatMulInteger per the operator specification (the reference delegates the
 * node to ONNX Runtime): int32 GEMM of the zero-point-shifted operands. */
void oracle_matmul_integer_i8(const int8_t* A, const int8_t* B, int32_t za, int32_t zb, int32_t* Y,
                              int64_t M, int64_t N, int64_t K) {
#pragma omp parallel for schedule(static)
    for (int64_t m = 0; m < M; ++m) {
        int32_t* y = &Y[m * N];
        memset(y, 0, sizeof(int32_t) * (size_t)N);
        for (int64_t k = 0; k < K; ++k) {
            const int32_t a = (int32_t)A[m * K + k] - za;
            const int8_t* b = &B[k * N];
            for (int64_t n = 0; n < N; ++n) y[n] += a * ((int32_t)b[n] - zb);
        }
    }
}

/* The same for int8 or uint8 operands and zero points given per row of A (za_stride 1) and per column
 * of B (zb_stride 1) or as one value (stride 0); int32 accumulation wraps modulo 2^32 like the node's
 * int32 output. */
void oracle_matmul_integer(const void* A, const void* B, const int32_t* za, const int32_t* zb, int32_t* Y,
                           int64_t M, int64_t N, int64_t K, int a_unsigned, int b_unsigned,
                           int64_t za_stride, int64_t zb_stride) {
    const int8_t* As = (const int8_t*)A;
    const uint8_t* Au = (const uint8_t*)A;
    const int8_t* Bs = (const int8_t*)B;
    const uint8_t* Bu = (const uint8_t*)B;
#pragma omp parallel for schedule(static)
    for (int64_t m = 0; m < M; ++m) {
        uint32_t* y = (uint32_t*)&Y[m * N];
        memset(y, 0, sizeof(int32_t) * (size_t)N);
        for (int64_t k = 0; k < K; ++k) {
            const int32_t a = (a_unsigned ? (int32_t)Au[m * K + k] : (int32_t)As[m * K + k]) - za[m * za_stride];
            for (int64_t n = 0; n < N; ++n) {
                const int32_t b = (b_unsigned ? (int32_t)Bu[k * N + n] : (int32_t)Bs[k * N + n]) - zb[n * zb_stride];
                y[n] += (uint32_t)(a * b);
            }
        }
    }
}

/* MatMul without a BLAS library: DaCe's pure map-reduce GEMM, what
 * create_einsum_sdfg falls back to (pure_implementations.py:260-266). */
void oracle_matmul_f32(const float* A, const float* B, float* Y, int64_t M, int64_t N, int64_t K) {
#pragma omp parallel for schedule(static)
    for (int64_t m = 0; m < M; ++m) {
        float* y = &Y[m * N];
        memset(y, 0, sizeof(float) * (size_t)N);
        for (int64_t k = 0; k < K; ++k) {
            const float a = A[m * K + k];
            const float* b = &B[k * N];
            for (int64_t n = 0; n < N; ++n) y[n] += a * b[n];
        }
    }
}
