/*
 * mi355x_onnx.h -- C ABI of libmi355x_onnx.so: hand-written gfx950 (MI355X)
 * kernels for the ONNX library nodes that DaCeML expands
 * (MatMul/Gemm, Conv, MatMulInteger, Softmax, LayerNormalization,
 * Add/Relu/Gelu and the Transpose copy that sits between them).
 *
 * Conventions (all entry points):
 *   - every pointer is a DEVICE pointer owned by the caller; nothing is
 *     allocated, freed or retained by the library (reference ownership rule:
 *     daceml/pytorch/module_codegen.py:74-84,143-145 -- inputs are
 *     .contiguous() data_ptr()s, outputs are pre-allocated by the caller);
 *   - shapes and strides are int64 ELEMENT counts (not bytes);
 *   - `stream` is a hipStream_t passed as void*; kernels are enqueued on it
 *     and the call returns without synchronising (reference threading rule:
 *     daceml/pytorch/module_codegen.py:461-463 sets state.nosync = True and
 *     daceml/onnx/environments/cudnn.py:44 binds __dace_current_stream);
 *   - return value 0 = enqueued; non-zero = nothing was launched and
 *     mi355x_last_error() holds a message for the calling thread
 *     (the reference's vendor-library glue prints and continues,
 *     daceml/onnx/include/daceml_cudnn.h:15-22, or prints and exit(1)s,
 *     daceml/onnx/include/dace_onnx.h:7-15; here the caller decides).
 *
 * A DaCe C++ tasklet links this library the way cuDNN is linked in
 * daceml/onnx/environments/cudnn.py:11-67; Python loads it with ctypes the way
 * the reference loads its ORT bridge (daceml/ort_api/raw_api_bindings.py:305-321).
 */
#ifndef MI355X_ONNX_H
#define MI355X_ONNX_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MI355X_ONNX_VERSION 100 /* major*10000 + minor*100 + patch */

/* status codes */
#define MI355X_OK 0
#define MI355X_ERR_INVALID_ARGUMENT 1 /* shape/stride/attribute outside what the kernel supports */
#define MI355X_ERR_LAUNCH 2           /* hipLaunchKernel reported an error */
#define MI355X_ERR_NOT_INITIALIZED 3  /* no gfx950 device / runtime not usable */

/* Library identity and error channel.
 * Counterpart of the per-process handle object of the reference's cuDNN glue
 * (daceml/onnx/include/daceml_cudnn.h:38-64): there is no handle here, the
 * only per-thread state is the last error string. */
int mi355x_version(void);
const char* mi355x_last_error(void);

/* Number of compute units of the current device (0 when no device is usable).
 * Used by callers that size grids or report occupancy; no reference counterpart. */
int mi355x_device_cu_count(void);

/* Launches one workgroup of a kernel that does nothing, on `stream`. What such a launch costs is the floor under every
 * kernel duration on the part; a benchmark measures it to say how much of a small kernel's time is the launch itself.
 * No reference counterpart (the reference times whole programs, daceml/testing/profiling/event_profiler.py:87-143). */
int mi355x_launch_empty_kernel(void* stream);

/* The MI355X_* environment variables that force a kernel variant (MI355X_GEMM_CONFIG, MI355X_GEMM_NT_BN,
 * MI355X_GEMM_NT_BM, MI355X_GEMM_NT_BK, MI355X_GEMM_NT_PER_CU, MI355X_GEMM_NT_WAVES, MI355X_GEMM_GROUP_M, MI355X_GEMM_KSPLIT, MI355X_CONV_CONFIG, MI355X_CONV_GATHER_BN, MI355X_CONV_PER_CU, MI355X_CONV_TAIL, MI355X_CONV_STATIC_TAPS, MI355X_MMI_GENERIC,
 * MI355X_MMI_WGS_PER_CU, MI355X_MMI_TILE, MI355X_ATTN_WAVES) are read on the first launch only; call this after changing them. The role of
 * CudnnConvolution.default_algorithm / node._algorithm in the reference (cudnn_implementations.py:119-131):
 * a way to pick the algorithm by hand. */
void mi355x_reload_tuning(void);

/* ---- epilogue flags shared by GEMM and Conv (bitwise OR) ------------------
 * Applied per output element in this order:
 *   v = alpha * acc; if BIAS v += bias[n]; if RELU v = max(v,0);
 *   if GELU v = 0.5*v*(1+erf(v/sqrt(2))); if RESIDUAL v += residual[m,n].
 * Replaces the separate Add / Relu / (Div,Erf,Add,Mul,Mul) nodes that follow a
 * contraction in the reference's graphs (daceml/onnx/op_implementations/
 * pure_implementations.py:77-79,112-127,462-474); the reference fuses only by
 * graph transformation (daceml/transformation/tasklet_fusion.py:35). */
#define MI355X_EPI_NONE 0
#define MI355X_EPI_BIAS 1
#define MI355X_EPI_RELU 2
#define MI355X_EPI_GELU 4
#define MI355X_EPI_RESIDUAL 8
/* convolution only: v = max(v, 0) once more after the residual (the end of a ResNet block) */
#define MI355X_EPI_RELU_AFTER 16

/* ONNX MatMul / Gemm, fp32, on MFMA.
 *   C[b0,b1,m,n] = epilogue(alpha * sum_k A[b0,b1,m,k] * B[b0,b1,k,n])
 * Replaces PureMatMul.forward -> PureEinsum.forward -> DaCe BLAS node
 * (daceml/onnx/op_implementations/pure_implementations.py:130-267) and
 * PureGemm.forward (pure_implementations.py:433-459, transB=1 is expressed by
 * swapping the two B strides).
 *   a_strides = {batch0, batch1, m, k}; b_strides = {batch0, batch1, k, n};
 *   c_strides = {batch0, batch1, m} (n stride is 1); r_strides like c_strides
 *   for `residual` (ignored unless MI355X_EPI_RESIDUAL). A batch stride of 0
 *   broadcasts that operand (numpy broadcasting of leading dims,
 *   pure_implementations.py:189-208). Two batch levels let a head split/merge
 *   ([B,S,H*D] <-> [B,H,S,D]) be expressed as strides instead of the
 *   Reshape+Transpose copies of pure_implementations.py:369-379,477-513.
 *   bias is [N] (ignored unless MI355X_EPI_BIAS). */
int mi355x_gemm_f32(const float* A, const float* B, float* C,
                    const float* bias, const float* residual,
                    int64_t batch0, int64_t batch1,
                    int64_t M, int64_t N, int64_t K,
                    const int64_t* a_strides, const int64_t* b_strides,
                    const int64_t* c_strides, const int64_t* r_strides,
                    float alpha, int epilogue, void* stream);

/* ONNX Conv, 2-D, NCHW, group 1, fp32, implicit GEMM on MFMA.
 *   Y[n,m,oy,ox] = epilogue(sum_{c,r,s} W[m,c,r,s] *
 *        X[n,c,oy*stride_h - pad_top + r*dil_h, ox*stride_w - pad_left + s*dil_w])
 * with out-of-range X taken as 0. Replaces PureConv2D
 * (daceml/onnx/op_implementations/img_op_implementations.py:164-326; that
 * expansion requires zero pads and drops the stride term at :278,:291) and the
 * cudnnConvolutionForward call of cudnn_implementations.py:303-322.
 *   pads = {top, left, bottom, right} (ONNX order), strides = {h, w},
 *   dilations = {h, w}. X, W, Y are C-contiguous; bias is [M] or NULL.
 *   epilogue accepts MI355X_EPI_BIAS and MI355X_EPI_RELU. */
int mi355x_conv2d_f32(const float* X, const float* W, const float* bias, float* Y,
                      int64_t N, int64_t C, int64_t H, int64_t Wd,
                      int64_t M, int64_t KH, int64_t KW,
                      const int64_t* pads, const int64_t* strides,
                      const int64_t* dilations, int epilogue, void* stream);

/* The same convolution with a residual: `residual` has the shape and layout of Y and is added after
 * bias and activation (MI355X_EPI_RESIDUAL); MI355X_EPI_RELU_AFTER applies max(v, 0) to the sum. Stands
 * for Conv -> Add -> Relu, three nodes (and two more passes over the result) in the reference's graphs
 * (img_op_implementations.py:164-326, pure_implementations.py:77-79, 462-474). */
int mi355x_conv2d_res_f32(const float* X, const float* W, const float* bias, const float* residual,
                          float* Y, int64_t N, int64_t C, int64_t H, int64_t Wd,
                          int64_t M, int64_t KH, int64_t KW,
                          const int64_t* pads, const int64_t* strides,
                          const int64_t* dilations, int epilogue, void* stream);

/* ONNX MaxPool, 2-D, fp32, NCHW: Y[n,c,oh,ow] = max over the KH x KW window at
 * (oh * strides[0] - pads[0] + kh * dilations[0], ow * strides[1] - pads[1] + kw * dilations[1]);
 * positions in the padding do not take part. pads = {top, left, bottom, right}, floor output size
 * (ceil_mode 0). Replaces PureMaxPool2D.forward (img_op_implementations.py:28-161), which accepts
 * neither pads nor dilations. */
int mi355x_maxpool2d_f32(const float* X, float* Y, int64_t N, int64_t C, int64_t H, int64_t W,
                         int64_t KH, int64_t KW, const int64_t* pads, const int64_t* strides,
                         const int64_t* dilations, void* stream);

/* ONNX BatchNormalization in inference form, fp32, X and Y are [N, C, HW]:
 * Y = (X - mean[c]) * (1 / sqrt(var[c] + eps)) * scale[c] + B[c], the arithmetic of
 * PureBatchNormalization.forward (img_op_implementations.py:362-375) with the stored statistics in
 * place of the batch's (the reference expands the training form only and leaves inference to ONNX
 * Runtime). */
int mi355x_batchnorm_f32(const float* X, const float* scale, const float* B, const float* mean,
                         const float* var, float* Y, int64_t N, int64_t C, int64_t HW, float eps,
                         void* stream);

/* ONNX MatMulInteger (opset 10), 8-bit operands -> int32 on int8 MFMA, bit-exact against the formula below
 * evaluated in 64-bit integers (wrapped to 32 bits); parity with the reference is unpinned: it has no
 * implementation of its own to compare with.
 *   Y[m,n] = sum_k (A[m,k] - a_zero_point[m]) * (B[k,n] - b_zero_point[n])
 * The reference has no expansion of its own for this node: the generated class
 * (daceml/onnx/nodes/onnx_op.py:623-640, built from the ONNX schema: T1, T2 in
 * {int8, uint8}, optional zero points of the operand's type) only has the
 * "onnxruntime" implementation (onnx_op.py:686-687 -> node_codegen.py:321-573).
 * A is [M,K], B is [K,N], Y is [M,N], all C-contiguous; a stack of A matrices
 * against one B is the same call with the stack folded into M.
 * a_unsigned / b_unsigned: the operand (and its zero point) is uint8, else int8.
 * The zero points are DEVICE pointers read by the kernel (no host
 * synchronisation); NULL means 0. a_zero_point_count is 1 (one value) or M (one
 * per row of A), b_zero_point_count is 1 or N (one per column of B). */
int mi355x_matmul_integer(const void* A, const void* B,
                          const void* a_zero_point, const void* b_zero_point,
                          int32_t* Y, int64_t M, int64_t N, int64_t K,
                          int a_unsigned, int b_unsigned,
                          int64_t a_zero_point_count, int64_t b_zero_point_count,
                          void* stream);

/* The same with int8 operands and one zero point each (or NULL). */
int mi355x_matmul_integer_i8(const int8_t* A, const int8_t* B,
                             const int8_t* a_zero_point, const int8_t* b_zero_point,
                             int32_t* Y, int64_t M, int64_t N, int64_t K,
                             void* stream);

/* ONNX Softmax along one axis, fp32. X viewed as [outer, axis_len, inner]
 * (C-contiguous): y = exp(x - max) / sum(exp(x - max)) over axis_len.
 * Replaces the five maps of PureSoftmax.forward
 * (pure_implementations.py:346-366) with one pass. inner == 1 is the
 * last-axis case. */
int mi355x_softmax_f32(const float* X, float* Y,
                       int64_t outer, int64_t axis_len, int64_t inner,
                       void* stream);

/* ONNX LogSoftmax along one axis, fp32, same view of X:
 * y = (x - max) - log(sum(exp(x - max))). Replaces the eight steps of
 * PureLogSoftmax.forward (pure_implementations.py:594-616) with one pass. */
int mi355x_log_softmax_f32(const float* X, float* Y,
                           int64_t outer, int64_t axis_len, int64_t inner,
                           void* stream);

/* Scaled-dot-product attention core, fp32, one launch:
 *   O[b0,b1] = softmax(scale * Q[b0,b1] K[b0,b1]^T, over keys) V[b0,b1]
 * Q, O are [Sq, D], K, V are [Sk, D] per (b0, b1) slice; the last dimension is
 * contiguous, *_strides = {batch0, batch1, row} element strides (multiples of 4,
 * operands 16-byte aligned), so the head split/merge of a [B, S, H*D] projection is
 * expressed without a copy. Replaces the node sequence MatMul -> (Div | Mul by a
 * scalar) -> Softmax(last axis) -> MatMul that the reference expands one node at a
 * time (pure_implementations.py:130-235, 346-366); the score tensor never reaches
 * memory. Supported: D == 64 and any Sk >= 1 (128 keys in one pass, any other
 * number in blocks of 128 with a running row maximum and sum); another head size
 * returns MI355X_ERR_INVALID_ARGUMENT and launches nothing (the caller keeps the
 * three separate nodes). */
int mi355x_attention_f32(const float* Q, const float* K, const float* V, float* O,
                         int64_t batch0, int64_t batch1, int64_t Sq, int64_t Sk, int64_t D,
                         const int64_t* q_strides, const int64_t* k_strides,
                         const int64_t* v_strides, const int64_t* o_strides,
                         float scale, void* stream);

/* ONNX LayerNormalization over the last axis, fp32, X is [rows, cols]:
 *   y = (x - mean) / sqrt(var + eps) * gamma + beta, biased variance.
 * The reference has no such node (opset 12); it runs the exporter's
 * decomposition ReduceMean, Sub, Pow, ReduceMean, Add, Sqrt, Div, Mul, Add
 * (pure_implementations.py:97-109,82-84,59-74,77-79,41-56,92-94).
 * gamma/beta are [cols]; beta may be NULL. */
int mi355x_layernorm_f32(const float* X, const float* gamma, const float* beta,
                         float* Y, int64_t rows, int64_t cols, float eps,
                         void* stream);

/* ONNX ReduceMean along one axis, fp32. X viewed as [outer, axis_len, inner]
 * (C-contiguous); Y is [outer, inner] (keepdims only changes the shape the
 * caller gives it). Replaces PureReduceMean.forward
 * (pure_implementations.py:97-109), which the reference meets in every
 * exported LayerNorm (opset 12 has no LayerNormalization node). Several
 * adjacent reduced axes are one axis of the product length. */
int mi355x_reduce_mean_f32(const float* X, float* Y,
                           int64_t outer, int64_t axis_len, int64_t inner,
                           void* stream);

/* ONNX ReduceMean / ReduceSum / ReduceMax / ReduceMin along one axis, fp32, same
 * view of X and Y as mi355x_reduce_mean_f32 (which is kind MI355X_REDUCE_MEAN).
 * Replaces PureReduceSum, PureReduceMax and PureReduceMin
 * (pure_implementations.py:301-343: np.sum / np.max / np.min over `axes`). A
 * NaN in a reduced slice makes its maximum and minimum NaN, as numpy does. */
#define MI355X_REDUCE_MEAN 0
#define MI355X_REDUCE_SUM 1
#define MI355X_REDUCE_MAX 2
#define MI355X_REDUCE_MIN 3
int mi355x_reduce_f32(int kind, const float* X, float* Y,
                      int64_t outer, int64_t axis_len, int64_t inner,
                      void* stream);

/* The same reductions over any set of axes (ReduceSum over axes 0 and 2 of a [2, 4, 10] tensor, as in the
 * reference's tests/pure_expansions/test_expansions.py:176-230): `reduced[d]` != 0 marks the axes of
 * X[shape] (element strides x_strides) that are reduced; Y holds the kept axes in order, C-contiguous. One
 * wave per output element; adjacent axes are served faster by mi355x_reduce_f32. ndim <= 8. */
int mi355x_reduce_nd_f32(int kind, const float* X, float* Y, int ndim, const int64_t* shape,
                         const int64_t* x_strides, const int64_t* reduced, void* stream);

/* Elementwise ops, fp32, with numpy broadcasting.
 * Replaces the one-map expansions Add/Sub/Mul/Div
 * (pure_implementations.py:77-94), PurePow (:59-74), PureRelu (:462-474),
 * PureErf (:112-127), PureSqrt (:41-56), the Gelu decomposition
 * Div,Erf,Add,Mul,Mul, and the unary maps PureLog (:23-38), PureReciprocal
 * (:275-293), Tanh (:296-298), Softplus (:696-698, log(1 + exp(x)) as written
 * there) and PureSigmoid (:701-712, 1 / (1 + exp(-x))); Exp, Neg and Abs have
 * no pure expansion in the reference (ONNX Runtime runs them there).
 *   binary ops: C = A op B; unary ops ignore B (pass NULL).
 *   ndim <= 8; shape is the OUTPUT shape; a_strides / b_strides are element
 *   strides of each operand in the output's index space (0 on broadcast dims).
 *   C is C-contiguous. */
#define MI355X_OP_ADD 0
#define MI355X_OP_SUB 1
#define MI355X_OP_MUL 2
#define MI355X_OP_DIV 3
#define MI355X_OP_POW 4
#define MI355X_OP_RELU 16
#define MI355X_OP_GELU 17
#define MI355X_OP_ERF 18
#define MI355X_OP_SQRT 19
/* 20 is MI355X_OP_COPY, see the program kernel below */
#define MI355X_OP_LOG 21
#define MI355X_OP_TANH 22
#define MI355X_OP_SIGMOID 23
#define MI355X_OP_SOFTPLUS 24
#define MI355X_OP_RECIPROCAL 25
#define MI355X_OP_EXP 26
#define MI355X_OP_NEG 27
#define MI355X_OP_ABS 28
#define MI355X_OP_LAST 28
int mi355x_eltwise_f32(int op, const float* A, const float* B, float* C,
                       int ndim, const int64_t* shape,
                       const int64_t* a_strides, const int64_t* b_strides,
                       void* stream);

/* A group of elementwise nodes as one launch, fp32: every tensor operand is read once, the result
 * written once, intermediates stay in registers. In the reference each of these nodes is its own map with
 * a materialised result (pure_implementations.py:41-127, 462-474) and merging them is left to DaCe's map /
 * tasklet fusion (daceml/transformation/tasklet_fusion.py); here the fusion pass emits a short program.
 *   tensors[n_tensors]  inputs of the result's shape, C-contiguous (n elements each)
 *   vectors[n_vectors]  inputs of last_dim elements, broadcast along every other axis
 *   immediates          scalar constants (host memory, copied into the launch)
 *   program[n_instr]    host memory; one 32-bit word per instruction:
 *                         op | dst register << 8 | operand a << 16 | operand b << 24
 *                       op is one of MI355X_OP_* (unary ops ignore b); registers are 0..7; an operand byte is
 *                       kind << 6 | index with the kinds below. Y receives the last instruction's result.
 * Limits are the MI355X_PROGRAM_MAX_* below; a register must be written before it is read. */
#define MI355X_OP_COPY 20
#define MI355X_PROGRAM_REG 0
#define MI355X_PROGRAM_TENSOR 1
#define MI355X_PROGRAM_VECTOR 2
#define MI355X_PROGRAM_IMMEDIATE 3
#define MI355X_PROGRAM_MAX_INSTR 16
#define MI355X_PROGRAM_MAX_TENSORS 4
#define MI355X_PROGRAM_MAX_VECTORS 4
#define MI355X_PROGRAM_MAX_IMM 8
int mi355x_eltwise_program_f32(const float* const* tensors, int n_tensors,
                               const float* const* vectors, int n_vectors, float* Y, int64_t n,
                               int64_t last_dim, const uint32_t* program, int n_instr,
                               const float* immediates, int n_immediates, void* stream);

/* ONNX Transpose (and any strided gather), 4-byte elements:
 *   Y (C-contiguous, `shape`) [i0..] = X[sum_d i_d * x_strides[d]].
 * Replaces PureTranspose.forward (pure_implementations.py:369-379), and
 * PureSlice.forward (:619-693) with X pointing at the first selected element
 * and x_strides = stride * step per axis. ndim <= 8. */
int mi355x_permute_b32(const void* X, void* Y, int ndim, const int64_t* shape,
                       const int64_t* x_strides, void* stream);

/* ONNX Cast between float, double, int32, int64, int8, uint8 and bool, one pass.
 * Replaces PureCast.forward (pure_implementations.py:382-430: one map of
 * `__output = __input`, i.e. the C conversion, which truncates toward zero
 * from floating point to integers); to bool is `x != 0`.
 * `from_type` / `to_type` are ONNX TensorProto data types (the values of the
 * node's `to` attribute): 1 float, 2 uint8, 3 int8, 6 int32, 7 int64, 9 bool,
 * 11 double. n elements, both buffers C-contiguous. */
#define MI355X_TYPE_FLOAT 1
#define MI355X_TYPE_UINT8 2
#define MI355X_TYPE_INT8 3
#define MI355X_TYPE_INT32 6
#define MI355X_TYPE_INT64 7
#define MI355X_TYPE_BOOL 9
#define MI355X_TYPE_DOUBLE 11
int mi355x_cast(const void* X, int from_type, void* Y, int to_type, int64_t n,
                void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MI355X_ONNX_H */
