// The convolution network ops around Conv: MaxPool (2-D), BatchNormalization in inference form,
// fp32, NCHW. GlobalAveragePool needs no kernel of its own: it is the row mean of [N*C, H*W].
//
// The reference's PureMaxPool2D (daceml/onnx/op_implementations/img_op_implementations.py:28-161)
// initialises Y to the smallest float and folds every window element in with a max write-conflict
// resolution; it accepts no pads, no dilation, no ceil_mode and ignores nothing else. Its
// PureBatchNormalization (:329-407) is the training form only (batch statistics, running-mean
// update); the inference form -- what an exported eval() network contains -- goes to ONNX
// Runtime there. Both kernels are one pass over HBM: every input element is read (MaxPool: at
// most ceil(KH / SH) * ceil(KW / SW) times, from cache) and every output element written once.
#include "common.h"

namespace mi355x {

struct PoolArgs {
    const float* X; float* Y;
    int64_t total;               // N * C * OH * OW
    int H, W, OH, OW, KH, KW, pad_t, pad_l, sh, sw, dh, dw;
};

// One thread per output element, adjacent lanes adjacent along OW. Padded positions do not take part in the
// maximum (ONNX MaxPool pads with -inf); NaN propagates like numpy's max.
__global__ __launch_bounds__(256) void maxpool2d_kernel(PoolArgs p) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < p.total; i += stride) {
        const int ow = (int)(i % p.OW);
        const int64_t t = i / p.OW;
        const int oh = (int)(t % p.OH);
        const int64_t plane = t / p.OH;                      // n * C + c
        const float* x = p.X + plane * p.H * p.W;
        float m = -INFINITY;
        bool nan = false;
        for (int kh = 0; kh < p.KH; ++kh) {
            const int ih = oh * p.sh - p.pad_t + kh * p.dh;
            if (ih < 0 || ih >= p.H) continue;
            for (int kw = 0; kw < p.KW; ++kw) {
                const int iw = ow * p.sw - p.pad_l + kw * p.dw;
                if (iw < 0 || iw >= p.W) continue;
                const float v = x[(int64_t)ih * p.W + iw];
                nan |= v != v;
                m = fmaxf(m, v);
            }
        }
        p.Y[i] = nan ? NAN : m;
    }
}

// Y = (X - mean[c]) * (1 / sqrt(var[c] + eps)) * scale[c] + B[c], in the reference's order of operations
// (img_op_implementations.py:362-375 with the stored statistics in place of the batch's).
template <bool VEC>
__global__ __launch_bounds__(256) void batchnorm_kernel(const float* __restrict__ X, const float* __restrict__ scale,
                                                        const float* __restrict__ B, const float* __restrict__ mean,
                                                        const float* __restrict__ var, float* __restrict__ Y,
                                                        int64_t planes, int C, int64_t hw, float eps) {
    // one workgroup walks planes blockIdx.x, blockIdx.x + gridDim.x, ...: the four per-channel values are uniform
    for (int64_t plane = blockIdx.x; plane < planes; plane += gridDim.x) {
        const int c = (int)(plane % C);
        const float mu = mean[c], inv = 1.0f / sqrtf(var[c] + eps), g = scale[c], b = B[c];
        const float* x = X + plane * hw;
        float* y = Y + plane * hw;
        if constexpr (VEC) {
            const f32x4* x4 = reinterpret_cast<const f32x4*>(x);
            f32x4* y4 = reinterpret_cast<f32x4*>(y);
            for (int64_t i = threadIdx.x; i < hw / 4; i += blockDim.x) {
                const f32x4 v = __builtin_nontemporal_load(x4 + i);
                __builtin_nontemporal_store((v - mu) * inv * g + b, y4 + i);
            }
        } else {
            for (int64_t i = threadIdx.x; i < hw; i += blockDim.x) y[i] = (x[i] - mu) * inv * g + b;
        }
    }
}

}  // namespace mi355x

extern "C" int mi355x_maxpool2d_f32(const float* X, float* Y, int64_t N, int64_t C, int64_t H, int64_t W,
                                    int64_t KH, int64_t KW, const int64_t* pads, const int64_t* strides,
                                    const int64_t* dilations, void* stream) {
    using namespace mi355x;
    MI355X_REQUIRE(N >= 0 && C >= 0 && H >= 1 && W >= 1 && KH >= 1 && KW >= 1, "maxpool: bad extents");
    MI355X_REQUIRE(pads && strides && dilations, "maxpool: null pads / strides / dilations");
    MI355X_REQUIRE(strides[0] >= 1 && strides[1] >= 1 && dilations[0] >= 1 && dilations[1] >= 1 && pads[0] >= 0 &&
                       pads[1] >= 0 && pads[2] >= 0 && pads[3] >= 0, "maxpool: bad pads / strides / dilations");
    // a window that starts inside the padding must still reach the image (ONNX requires pads < kernel extent)
    MI355X_REQUIRE(pads[0] < (KH - 1) * dilations[0] + 1 && pads[2] < (KH - 1) * dilations[0] + 1 &&
                       pads[1] < (KW - 1) * dilations[1] + 1 && pads[3] < (KW - 1) * dilations[1] + 1,
                   "maxpool: pads must be smaller than the window");
    const int64_t eh = (KH - 1) * dilations[0] + 1, ew = (KW - 1) * dilations[1] + 1;
    const int64_t OH = (H + pads[0] + pads[2] - eh) / strides[0] + 1, OW = (W + pads[1] + pads[3] - ew) / strides[1] + 1;
    MI355X_REQUIRE(H + pads[0] + pads[2] >= eh && W + pads[1] + pads[3] >= ew, "maxpool: window larger than the padded image");
    MI355X_REQUIRE(H < (1 << 30) && W < (1 << 30) && KH < (1 << 15) && KW < (1 << 15), "maxpool: extent too large");
    const int64_t total = N * C * OH * OW;
    if (total == 0) return MI355X_OK;
    MI355X_REQUIRE(X && Y, "maxpool: null pointer");
    PoolArgs p;
    p.X = X; p.Y = Y; p.total = total;
    p.H = (int)H; p.W = (int)W; p.OH = (int)OH; p.OW = (int)OW; p.KH = (int)KH; p.KW = (int)KW;
    p.pad_t = (int)pads[0]; p.pad_l = (int)pads[1]; p.sh = (int)strides[0]; p.sw = (int)strides[1];
    p.dh = (int)dilations[0]; p.dw = (int)dilations[1];
    int64_t blocks = ceil_div(total, (int64_t)256);
    if (blocks > 65536) blocks = 65536;
    hipLaunchKernelGGL(maxpool2d_kernel, dim3((unsigned)blocks), dim3(256), 0, static_cast<hipStream_t>(stream), p);
    return check_launch("maxpool2d_kernel");
}

extern "C" int mi355x_batchnorm_f32(const float* X, const float* scale, const float* B, const float* mean,
                                    const float* var, float* Y, int64_t N, int64_t C, int64_t HW, float eps,
                                    void* stream) {
    using namespace mi355x;
    MI355X_REQUIRE(N >= 0 && C >= 0 && HW >= 0 && C < ((int64_t)1 << 31), "batchnorm: bad extents");
    if (N * C * HW == 0) return MI355X_OK;
    MI355X_REQUIRE(X && scale && B && mean && var && Y, "batchnorm: null pointer");
    const int64_t planes = N * C;
    int64_t blocks = planes < 65536 ? planes : 65536;
    const bool vec = HW % 4 == 0 && (reinterpret_cast<uintptr_t>(X) & 15) == 0 && (reinterpret_cast<uintptr_t>(Y) & 15) == 0;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (vec) hipLaunchKernelGGL(batchnorm_kernel<true>, dim3((unsigned)blocks), dim3(256), 0, st, X, scale, B, mean, var, Y, planes, (int)C, HW, eps);
    else hipLaunchKernelGGL(batchnorm_kernel<false>, dim3((unsigned)blocks), dim3(256), 0, st, X, scale, B, mean, var, Y, planes, (int)C, HW, eps);
    return check_launch("batchnorm_kernel");
}
