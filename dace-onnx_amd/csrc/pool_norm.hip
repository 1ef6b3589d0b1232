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

// IEEE-754-2019 maximum: a NaN in either operand gives NaN (numpy's max does the same); one v_maximum3_f32.
__device__ __forceinline__ float max_nan(float a, float b) { return __builtin_elementwise_maximum(a, b); }

// One thread per output element, adjacent lanes adjacent along OW. Padded positions do not take part in the
// maximum (ONNX MaxPool pads with -inf).
__global__ __launch_bounds__(256) void maxpool2d_kernel(PoolArgs p) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < p.total; i += stride) {
        const int ow = (int)(i % p.OW);
        const int64_t t = i / p.OW;
        const int oh = (int)(t % p.OH);
        const int64_t plane = t / p.OH;                      // n * C + c
        const float* x = p.X + plane * p.H * p.W;
        float m = -INFINITY;
        for (int kh = 0; kh < p.KH; ++kh) {
            const int ih = oh * p.sh - p.pad_t + kh * p.dh;
            if (ih < 0 || ih >= p.H) continue;
            for (int kw = 0; kw < p.KW; ++kw) {
                const int iw = ow * p.sw - p.pad_l + kw * p.dw;
                if (iw < 0 || iw >= p.W) continue;
                m = max_nan(m, x[(int64_t)ih * p.W + iw]);
            }
        }
        p.Y[i] = m;
    }
}

// The same pooling with the input staged through LDS: a workgroup owns `band` consecutive output rows of one
// (n, c) plane. The input rows they need are one contiguous piece of the plane, so it is fetched with fully
// coalesced loads (16 bytes per lane when the piece is aligned) and every element crosses HBM / L2 once, instead of
// once per window that covers it with stride-`sw` accesses; the band's outputs are one contiguous piece of Y.
// KH_ / KW_: window extents known at compile time (0: taken from the arguments). A thread walks outputs
// tid, tid + 256, ... of the band; (oh, ow) advance by (step_oh, step_ow) = divmod(256, OW) without dividing.
// Windows that lie inside the image -- all but the border -- skip the bounds checks.
template <bool VEC, int KH_, int KW_>
__global__ __launch_bounds__(256) void maxpool2d_lds_kernel(PoolArgs p, int band, int bands_per_plane, int step_oh, int step_ow) {
    extern __shared__ __attribute__((aligned(16))) float rows[];
    const int KH = KH_ ? KH_ : p.KH, KW = KW_ ? KW_ : p.KW;
    const int64_t plane = blockIdx.x / bands_per_plane;
    const int oh0 = (int)(blockIdx.x % bands_per_plane) * band;
    const int n_oh = min(band, p.OH - oh0);
    // input rows [ih_lo, ih_hi) of the plane cover every window of the band
    const int ih_lo = max(oh0 * p.sh - p.pad_t, 0);
    const int ih_hi = min((oh0 + n_oh - 1) * p.sh - p.pad_t + (KH - 1) * p.dh + 1, p.H);
    const float* x = p.X + (plane * p.H + ih_lo) * p.W;
    const int count = (ih_hi - ih_lo) * p.W;
    if constexpr (VEC) {      // count % 4 == 0 and x 16-byte aligned (checked on the host for every band)
        const f32x4* x4 = reinterpret_cast<const f32x4*>(x);
        f32x4* r4 = reinterpret_cast<f32x4*>(rows);
        for (int i = threadIdx.x; i < count / 4; i += 256) r4[i] = __builtin_nontemporal_load(x4 + i);
    } else {
        for (int i = threadIdx.x; i < count; i += 256) rows[i] = x[i];
    }
    __syncthreads();
    float* y = p.Y + (plane * p.OH + oh0) * p.OW;
    const int eh = (KH - 1) * p.dh + 1, ew = (KW - 1) * p.dw + 1;
    int oh = oh0 + (int)threadIdx.x / p.OW, ow = (int)threadIdx.x % p.OW;
    for (int i = threadIdx.x; i < n_oh * p.OW; i += 256) {
        const int ih0 = oh * p.sh - p.pad_t, iw0 = ow * p.sw - p.pad_l;
        float m = -INFINITY;
        if (ih0 >= 0 && ih0 + eh <= p.H && iw0 >= 0 && iw0 + ew <= p.W) {
            const float* win = rows + (ih0 - ih_lo) * p.W + iw0;
            if constexpr (KH_ != 0) {
#pragma unroll
                for (int kh = 0; kh < KH_; ++kh)
#pragma unroll
                    for (int kw = 0; kw < KW_; ++kw) m = max_nan(m, win[kh * p.dh * p.W + kw * p.dw]);
            } else {
                for (int kh = 0; kh < KH; ++kh)
                    for (int kw = 0; kw < KW; ++kw) m = max_nan(m, win[kh * p.dh * p.W + kw * p.dw]);
            }
        } else {
            for (int kh = 0; kh < KH; ++kh) {
                const int ih = ih0 + kh * p.dh;
                if (ih < 0 || ih >= p.H) continue;
                for (int kw = 0; kw < KW; ++kw) {
                    const int iw = iw0 + kw * p.dw;
                    if (iw >= 0 && iw < p.W) m = max_nan(m, rows[(ih - ih_lo) * p.W + iw]);
                }
            }
        }
        y[i] = m;
        ow += step_ow;
        oh += step_oh;
        if (ow >= p.OW) { ow -= p.OW; ++oh; }
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
    hipStream_t st = static_cast<hipStream_t>(stream);
    // Staged variant: bands of output rows whose input rows fit 32 KB of LDS and hold about 1024 outputs
    // (four per thread); planes too wide for that, and launches too small to fill the machine in bands, go direct.
    constexpr int64_t LDS_FLOATS = 8192;
    int64_t band = ceil_div((int64_t)1024, OW);
    band = band < OH ? band : OH;
    auto rows_needed = [&](int64_t b) { return (b - 1) * strides[0] + eh; };
    while (band > 1 && rows_needed(band) * W > LDS_FLOATS) --band;
    const int64_t bands_per_plane = ceil_div(OH, band);
    const int64_t nwg = N * C * bands_per_plane;
    if (rows_needed(band) * W <= LDS_FLOATS && nwg < ((int64_t)1 << 31) && total >= 65536) {
        // 16-byte loads need every band's first input row at a 16-byte boundary: that holds when X is aligned
        // and W is a multiple of 4 (then any row offset is)
        const bool vec = W % 4 == 0 && (reinterpret_cast<uintptr_t>(X) & 15) == 0;
        const size_t lds = (size_t)(rows_needed(band) < H ? rows_needed(band) : H) * W * sizeof(float);
        const dim3 grid((unsigned)nwg), block(256);
        const int b = (int)band, bpp = (int)bands_per_plane, q = (int)(256 / OW), r = (int)(256 % OW);
        const int shape = KH == 3 && KW == 3 ? 3 : KH == 2 && KW == 2 ? 2 : 0;
        if (vec && shape == 3) hipLaunchKernelGGL((maxpool2d_lds_kernel<true, 3, 3>), grid, block, lds, st, p, b, bpp, q, r);
        else if (vec && shape == 2) hipLaunchKernelGGL((maxpool2d_lds_kernel<true, 2, 2>), grid, block, lds, st, p, b, bpp, q, r);
        else if (vec) hipLaunchKernelGGL((maxpool2d_lds_kernel<true, 0, 0>), grid, block, lds, st, p, b, bpp, q, r);
        else if (shape == 3) hipLaunchKernelGGL((maxpool2d_lds_kernel<false, 3, 3>), grid, block, lds, st, p, b, bpp, q, r);
        else if (shape == 2) hipLaunchKernelGGL((maxpool2d_lds_kernel<false, 2, 2>), grid, block, lds, st, p, b, bpp, q, r);
        else hipLaunchKernelGGL((maxpool2d_lds_kernel<false, 0, 0>), grid, block, lds, st, p, b, bpp, q, r);
        return check_launch("maxpool2d_lds_kernel");
    }
    int64_t blocks = ceil_div(total, (int64_t)256);
    if (blocks > 65536) blocks = 65536;
    hipLaunchKernelGGL(maxpool2d_kernel, dim3((unsigned)blocks), dim3(256), 0, st, p);
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
