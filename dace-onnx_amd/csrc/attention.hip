// Fused scaled-dot-product attention core, fp32:  O = softmax(scale * Q K^T) V
// for one (batch, head) per slice, head size = 64; 128 keys (BERT-base) in one pass, any other number of
// keys in blocks of 128 with a running maximum and sum.
//
// The reference runs this as three library nodes -- MatMul, Softmax, MatMul
// (daceml/onnx/op_implementations/pure_implementations.py:130-235, 346-366) -- with
// the [B, H, S, S] score tensor written to and read from memory twice. Here a
// workgroup of 4 waves owns 64 query rows of one (batch, head): scores and
// probabilities never leave registers.
//
//   * K and V of the slice (128 x 64 each) are staged once in LDS, rows padded by 4
//     floats; Q operands come straight from global memory (16 query rows per wave,
//     nobody shares them).
//   * S = Q K^T uses the swapped-operand form of v_mfma_f32_16x16x4_f32: afterwards
//     lane (li, lq) holds S[q = li][key = 16 j + 4 lq + r] in acc[j][r] -- a query
//     row's 128 scores sit in 4 lanes x 32 registers. Row max and row sum are 31
//     register operations plus two cross-lane steps (lanes li, li+16, li+32, li+48).
//   * That register layout is exactly the A-operand layout of the second product
//     when the four keys of an MFMA step are taken as {16 j + r + 4 lq, lq = 0..3}:
//     acc[j][r] is used as the operand as it stands, no shuffle, no LDS round trip.
//     The matching V operand of lane (li, lq) is V[key = 16 j + 4 lq + r][4 li .. 4 li + 3]:
//     one 16-byte LDS read feeds four MFMAs (output tile t holds columns 4 li + t),
//     and a lane ends up with four consecutive output columns of a row: 16-byte stores.
#include "common.h"
#include "gemm_tile.h"

namespace mi355x {

constexpr int AT_SK = 128, AT_D = 64, AT_BQ = 64, AT_PITCH = AT_D + LDS_PAD;

struct AttnArgs {
    const float* Q; const float* K; const float* V; float* O;
    int64_t batch1, Sq, Sk, q_blocks, nwg;
    int64_t q_sb0, q_sb1, q_sr, k_sb0, k_sb1, k_sr, v_sb0, v_sb1, v_sr, o_sb0, o_sb1, o_sr;
    float scale;
};

__device__ __forceinline__ float quad_lanes_max(float v) {  // over lanes li, li+16, li+32, li+48
    v = fmaxf(v, __shfl_xor(v, 16, WAVE));
    return fmaxf(v, __shfl_xor(v, 32, WAVE));
}
__device__ __forceinline__ float quad_lanes_sum(float v) {
    v += __shfl_xor(v, 16, WAVE);
    return v + __shfl_xor(v, 32, WAVE);
}

// WAVES waves of 16 query rows each per workgroup: 4 (64 rows, two workgroups per 128-row slice) is what the library
// uses; 3 and 2 (48 and 32 rows: three and four workgroups per slice, the last one of three with two working waves)
// exist to measure whether more, smaller workgroups help, see MI355X_ATTN_WAVES in the launcher.
template <int WAVES>
__global__ __launch_bounds__(64 * WAVES) void attention_f32_kernel(AttnArgs p) {
    constexpr int SK = AT_SK, D = AT_D, PITCH = AT_PITCH, NJ = SK / 16, NC = D / 16;
    constexpr int NT = 64 * WAVES, VECS = SK * D / 4, PER_T = (VECS + NT - 1) / NT;   // K / V tile: 16-byte vectors per thread
    __shared__ __attribute__((aligned(16))) float lds_k[SK * PITCH];
    __shared__ __attribute__((aligned(16))) float lds_v[SK * PITCH];

    const int tid = threadIdx.x;
    const int lane = tid % WAVE, wave = tid / WAVE;
    const int li = lane % 16, lq = lane / 16;

    // consecutive logical ids (the query blocks of one slice, neighbouring heads) share an XCD's L2
    const int64_t logical = xcd_remap(blockIdx.x, p.nwg);
    const int64_t slice = logical / p.q_blocks, qb = logical % p.q_blocks;
    const int64_t b0 = slice / p.batch1, b1 = slice % p.batch1;
    const float* __restrict__ Q = p.Q + b0 * p.q_sb0 + b1 * p.q_sb1;
    const float* __restrict__ K = p.K + b0 * p.k_sb0 + b1 * p.k_sb1;
    const float* __restrict__ V = p.V + b0 * p.v_sb0 + b1 * p.v_sb1;
    float* __restrict__ O = p.O + b0 * p.o_sb0 + b1 * p.o_sb1;
    const int64_t q0 = qb * (16 * WAVES) + 16 * wave;   // first query row of this wave

    // ---- loads: K and V tiles (PER_T + PER_T vectors per thread), Q operands (4 per lane) ----------------
    f32x4 rk[PER_T], rv[PER_T], rq[NC];
#pragma unroll
    for (int it = 0; it < PER_T; ++it) {
        const int idx = tid + it * NT, row = idx / (D / 4), c4 = idx % (D / 4);
        if (VECS % NT == 0 || idx < VECS) rk[it] = *reinterpret_cast<const f32x4*>(K + row * p.k_sr + 4 * c4);
    }
    {
        int64_t qrow = q0 + li;
        qrow = qrow < p.Sq ? qrow : p.Sq - 1;   // clamped; rows beyond Sq are computed and not stored
#pragma unroll
        for (int c = 0; c < NC; ++c) rq[c] = *reinterpret_cast<const f32x4*>(Q + qrow * p.q_sr + 16 * c + 4 * lq);
    }
#pragma unroll
    for (int it = 0; it < PER_T; ++it) {
        const int idx = tid + it * NT, row = idx / (D / 4), c4 = idx % (D / 4);
        if (VECS % NT == 0 || idx < VECS) rv[it] = *reinterpret_cast<const f32x4*>(V + row * p.v_sr + 4 * c4);
    }
#pragma unroll
    for (int it = 0; it < PER_T; ++it) {
        const int idx = tid + it * NT, row = idx / (D / 4), c4 = idx % (D / 4);
        if (VECS % NT == 0 || idx < VECS) *reinterpret_cast<f32x4*>(lds_k + row * PITCH + 4 * c4) = rk[it];
    }
#pragma unroll
    for (int it = 0; it < PER_T; ++it) {
        const int idx = tid + it * NT, row = idx / (D / 4), c4 = idx % (D / 4);
        if (VECS % NT == 0 || idx < VECS) *reinterpret_cast<f32x4*>(lds_v + row * PITCH + 4 * c4) = rv[it];
    }
    __syncthreads();
    if (q0 >= p.Sq) return;  // whole wave beyond the last query row (after the only barrier)

    // ---- S = Q K^T: acc[j][r] = S[q0 + li][16 j + 4 lq + r] -------------------------------------------
    f32x4 acc[NJ];
#pragma unroll
    for (int j = 0; j < NJ; ++j) acc[j] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int c = 0; c < NC; ++c) {
        f32x4 kf[NJ];
#pragma unroll
        for (int j = 0; j < NJ; ++j)
            kf[j] = *reinterpret_cast<const f32x4*>(lds_k + (16 * j + li) * PITCH + 16 * c + 4 * lq);
#pragma unroll
        for (int s = 0; s < 4; ++s)
#pragma unroll
            for (int j = 0; j < NJ; ++j)
                acc[j] = __builtin_amdgcn_mfma_f32_16x16x4f32(kf[j][s], rq[c][s], acc[j], 0, 0, 0);
    }

    // ---- softmax over the 128 keys of each query row ------------------------------------------------
    // exp(scale s - max) as 2^(c s - max'), c = scale log2(e): one multiply per score and the bare v_exp_f32
    // (the library expf costs half a dozen more instructions per value; 32 values per lane)
    const float c = p.scale * 1.44269504088896340736f;
    float m = -INFINITY;
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
        acc[j] *= c;
        m = fmaxf(m, fmaxf(fmaxf(acc[j].x, acc[j].y), fmaxf(acc[j].z, acc[j].w)));
    }
    m = quad_lanes_max(m);
    float sum = 0.f;
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
        acc[j].x = __builtin_amdgcn_exp2f(acc[j].x - m);
        acc[j].y = __builtin_amdgcn_exp2f(acc[j].y - m);
        acc[j].z = __builtin_amdgcn_exp2f(acc[j].z - m);
        acc[j].w = __builtin_amdgcn_exp2f(acc[j].w - m);
        sum += (acc[j].x + acc[j].y) + (acc[j].z + acc[j].w);
    }
    const float inv = 1.0f / quad_lanes_sum(sum);
#pragma unroll
    for (int j = 0; j < NJ; ++j) acc[j] *= inv;

    // ---- O = P V: out[t][r] = O[q0 + 4 lq + r][4 li + t] -------------------------------------------------
    f32x4 out[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) out[t] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
        f32x4 vf[4];
#pragma unroll
        for (int r = 0; r < 4; ++r)
            vf[r] = *reinterpret_cast<const f32x4*>(lds_v + (16 * j + 4 * lq + r) * PITCH + 4 * li);
#pragma unroll
        for (int r = 0; r < 4; ++r)
#pragma unroll
            for (int t = 0; t < 4; ++t)
                out[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(acc[j][r], vf[r][t], out[t], 0, 0, 0);
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int64_t qrow = q0 + 4 * lq + r;
        if (qrow < p.Sq)
            *reinterpret_cast<f32x4*>(O + qrow * p.o_sr + 4 * li) = f32x4{out[0][r], out[1][r], out[2][r], out[3][r]};
    }
}

// Any number of keys: the same workgroup walks the keys in blocks of 128 with a running row maximum and
// row sum (the probabilities of a block are exp(s - running max); when the maximum grows, the sums and the
// output accumulators are rescaled by exp(old max - new max); the division by the row sum happens once, at
// the end). Keys beyond Sk in the last block are loaded from the last valid row and their scores set to
// -inf. Every wave takes part in the barriers of every block, so there is no early exit for query rows
// beyond Sq: they are computed on the clamped last row and not stored.
__global__ __launch_bounds__(256) void attention_f32_blocks_kernel(AttnArgs p) {
    constexpr int SK = AT_SK, D = AT_D, PITCH = AT_PITCH, NJ = SK / 16, NC = D / 16;
    __shared__ __attribute__((aligned(16))) float lds_k[SK * PITCH];
    __shared__ __attribute__((aligned(16))) float lds_v[SK * PITCH];

    const int tid = threadIdx.x;
    const int lane = tid % WAVE, wave = tid / WAVE;
    const int li = lane % 16, lq = lane / 16;

    const int64_t logical = xcd_remap(blockIdx.x, p.nwg);
    const int64_t slice = logical / p.q_blocks, qb = logical % p.q_blocks;
    const int64_t b0 = slice / p.batch1, b1 = slice % p.batch1;
    const float* __restrict__ Q = p.Q + b0 * p.q_sb0 + b1 * p.q_sb1;
    const float* __restrict__ K = p.K + b0 * p.k_sb0 + b1 * p.k_sb1;
    const float* __restrict__ V = p.V + b0 * p.v_sb0 + b1 * p.v_sb1;
    float* __restrict__ O = p.O + b0 * p.o_sb0 + b1 * p.o_sb1;
    const int64_t q0 = qb * AT_BQ + 16 * wave;   // first query row of this wave

    f32x4 rq[NC];
    {
        int64_t qrow = q0 + li;
        qrow = qrow < p.Sq ? qrow : p.Sq - 1;
#pragma unroll
        for (int c = 0; c < NC; ++c) rq[c] = *reinterpret_cast<const f32x4*>(Q + qrow * p.q_sr + 16 * c + 4 * lq);
    }
    f32x4 out[4];                       // out[t][r] = O[q0 + 4 lq + r][4 li + t], not yet divided by the row sum
#pragma unroll
    for (int t = 0; t < 4; ++t) out[t] = f32x4{0.f, 0.f, 0.f, 0.f};
    float m_run = -INFINITY, l_run = 0.f;   // of query row q0 + li (the same value in its four lanes)
    const float c = p.scale * 1.44269504088896340736f;   // scores in units of log2: exp(scale s - m) = 2^(c s - m')

    for (int64_t key0 = 0; key0 < p.Sk; key0 += SK) {
        f32x4 rk[8], rv[8];
#pragma unroll
        for (int it = 0; it < 8; ++it) {
            const int idx = tid + it * 256, c4 = idx % (D / 4);
            int64_t row = key0 + idx / (D / 4);
            row = row < p.Sk ? row : p.Sk - 1;
            rk[it] = *reinterpret_cast<const f32x4*>(K + row * p.k_sr + 4 * c4);
            rv[it] = *reinterpret_cast<const f32x4*>(V + row * p.v_sr + 4 * c4);
        }
        if (key0 > 0) __syncthreads();   // the previous block's operands have been read by everyone
#pragma unroll
        for (int it = 0; it < 8; ++it) {
            const int idx = tid + it * 256, row = idx / (D / 4), c4 = idx % (D / 4);
            *reinterpret_cast<f32x4*>(lds_k + row * PITCH + 4 * c4) = rk[it];
            *reinterpret_cast<f32x4*>(lds_v + row * PITCH + 4 * c4) = rv[it];
        }
        __syncthreads();

        // ---- S = Q K^T of this block: acc[j][r] = S[q0 + li][key0 + 16 j + 4 lq + r]
        f32x4 acc[NJ];
#pragma unroll
        for (int j = 0; j < NJ; ++j) acc[j] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            f32x4 kf[NJ];
#pragma unroll
            for (int j = 0; j < NJ; ++j)
                kf[j] = *reinterpret_cast<const f32x4*>(lds_k + (16 * j + li) * PITCH + 16 * c + 4 * lq);
#pragma unroll
            for (int s = 0; s < 4; ++s)
#pragma unroll
                for (int j = 0; j < NJ; ++j)
                    acc[j] = __builtin_amdgcn_mfma_f32_16x16x4f32(kf[j][s], rq[c][s], acc[j], 0, 0, 0);
        }
        const bool ragged = key0 + SK > p.Sk;   // uniform
        float m_blk = -INFINITY;
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            acc[j] *= c;
            if (ragged) {
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    if (key0 + 16 * j + 4 * lq + r >= p.Sk) acc[j][r] = -INFINITY;
            }
            m_blk = fmaxf(m_blk, fmaxf(fmaxf(acc[j].x, acc[j].y), fmaxf(acc[j].z, acc[j].w)));
        }
        const float m_new = fmaxf(m_run, quad_lanes_max(m_blk));
        const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);    // 0 for the first block
        float sum = 0.f;
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            acc[j].x = __builtin_amdgcn_exp2f(acc[j].x - m_new);
            acc[j].y = __builtin_amdgcn_exp2f(acc[j].y - m_new);
            acc[j].z = __builtin_amdgcn_exp2f(acc[j].z - m_new);
            acc[j].w = __builtin_amdgcn_exp2f(acc[j].w - m_new);
            sum += (acc[j].x + acc[j].y) + (acc[j].z + acc[j].w);
        }
        l_run = l_run * alpha + quad_lanes_sum(sum);
        m_run = m_new;
        // the accumulators hold rows 4 lq + r: that row's factor lives in lane 4 lq + r
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const float a = __shfl(alpha, 4 * lq + r, WAVE);
#pragma unroll
            for (int t = 0; t < 4; ++t) out[t][r] *= a;
        }
        // ---- out += P V of this block
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            f32x4 vf[4];
#pragma unroll
            for (int r = 0; r < 4; ++r)
                vf[r] = *reinterpret_cast<const f32x4*>(lds_v + (16 * j + 4 * lq + r) * PITCH + 4 * li);
#pragma unroll
            for (int r = 0; r < 4; ++r)
#pragma unroll
                for (int t = 0; t < 4; ++t)
                    out[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(acc[j][r], vf[r][t], out[t], 0, 0, 0);
        }
    }
    const float inv = 1.0f / l_run;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const float a = __shfl(inv, 4 * lq + r, WAVE);
        const int64_t qrow = q0 + 4 * lq + r;
        if (qrow < p.Sq)
            *reinterpret_cast<f32x4*>(O + qrow * p.o_sr + 4 * li) = f32x4{out[0][r] * a, out[1][r] * a, out[2][r] * a, out[3][r] * a};
    }
}

}  // namespace mi355x

extern "C" int mi355x_attention_f32(const float* Q, const float* K, const float* V, float* O,
                                    int64_t batch0, int64_t batch1, int64_t Sq, int64_t Sk, int64_t D,
                                    const int64_t* q_strides, const int64_t* k_strides,
                                    const int64_t* v_strides, const int64_t* o_strides,
                                    float scale, void* stream) {
    using namespace mi355x;
    MI355X_REQUIRE(batch0 >= 0 && batch1 >= 0 && Sq >= 0, "attention: negative extent");
    MI355X_REQUIRE(Sk >= 1 && D == AT_D, "attention: head size 64 and at least one key are required (got %lld keys x %lld)",
                   (long long)Sk, (long long)D);
    if (batch0 * batch1 == 0 || Sq == 0) return MI355X_OK;
    MI355X_REQUIRE(Q && K && V && O && q_strides && k_strides && v_strides && o_strides, "attention: null pointer");
    auto al16 = [](const void* q) { return (reinterpret_cast<uintptr_t>(q) & 15) == 0; };
    bool ok = al16(Q) && al16(K) && al16(V) && al16(O);
    for (int i = 0; i < 3; ++i)
        ok = ok && q_strides[i] % 4 == 0 && k_strides[i] % 4 == 0 && v_strides[i] % 4 == 0 && o_strides[i] % 4 == 0 &&
             q_strides[i] >= 0 && k_strides[i] >= 0 && v_strides[i] >= 0 && o_strides[i] >= 0;
    MI355X_REQUIRE(ok, "attention: operands must be 16-byte aligned with strides that are multiples of 4 floats");
    AttnArgs p;
    p.Q = Q; p.K = K; p.V = V; p.O = O;
    p.batch1 = batch1; p.Sq = Sq; p.Sk = Sk;
    p.q_blocks = ceil_div(Sq, (int64_t)AT_BQ);
    p.nwg = batch0 * batch1 * p.q_blocks;
    MI355X_REQUIRE(p.nwg < ((int64_t)1 << 31), "attention: grid too large");
    p.q_sb0 = q_strides[0]; p.q_sb1 = q_strides[1]; p.q_sr = q_strides[2];
    p.k_sb0 = k_strides[0]; p.k_sb1 = k_strides[1]; p.k_sr = k_strides[2];
    p.v_sb0 = v_strides[0]; p.v_sb1 = v_strides[1]; p.v_sr = v_strides[2];
    p.o_sb0 = o_strides[0]; p.o_sb1 = o_strides[1]; p.o_sr = o_strides[2];
    p.scale = scale;
    if (Sk == AT_SK) {
        // MI355X_ATTN_WAVES = 2 / 3: 32 / 48 query rows per workgroup instead of 64 (measured on 8 x 12 slices of 128 rows:
        // 384 / 288 workgroups instead of 192 -- no faster, the time is one wave's chain of loads, 256 MFMAs and stores)
        const int waves = tuning().attn_waves == 2 || tuning().attn_waves == 3 ? tuning().attn_waves : 4;
        p.q_blocks = ceil_div(Sq, (int64_t)16 * waves);
        p.nwg = batch0 * batch1 * p.q_blocks;
        MI355X_REQUIRE(p.nwg < ((int64_t)1 << 31), "attention: grid too large");
        const dim3 g((unsigned)p.nwg);
        hipStream_t st = static_cast<hipStream_t>(stream);
        if (waves == 2) hipLaunchKernelGGL(attention_f32_kernel<2>, g, dim3(128), 0, st, p);
        else if (waves == 3) hipLaunchKernelGGL(attention_f32_kernel<3>, g, dim3(192), 0, st, p);
        else hipLaunchKernelGGL(attention_f32_kernel<4>, g, dim3(256), 0, st, p);
        return check_launch("attention_f32_kernel");
    }
    hipLaunchKernelGGL(attention_f32_blocks_kernel, dim3((unsigned)p.nwg), dim3(256), 0, static_cast<hipStream_t>(stream), p);
    return check_launch("attention_f32_blocks_kernel");
}
