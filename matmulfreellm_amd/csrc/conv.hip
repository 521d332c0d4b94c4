// ShortConvolution: the causal depthwise convolution (kernel size W <= 8, one filter per channel) with an optional SiLU that
// mmfreelm/modules/convolution.py:45-162 builds on nn.Conv1d / causal_conv1d, as three small HIP kernels: the whole-sequence
// forward, the one-token step on a cache of the last W inputs, and the backward.
//
// Arithmetic (restated on the CPU by oracle/conv.py, bit for bit): fp32, one rounding per operation, no FMA;
//   acc = 0;  for w = 0 .. W-1 with s = t - (W-1) + w >= 0:  acc = acc + weight[d, w] * x[b, s, d]     (oldest input first)
//   acc = acc + bias[d];  pre = T(acc)  (the convolution's output tensor in the activation dtype)
//   y = T(pre / (1 + exp(-pre)))  with the deterministic exp of mmf_common.h, or y = pre without an activation.
// The cache [B, D, W] holds the last W inputs of every channel, oldest first, in the activation dtype; a step drops the
// oldest, appends the new token and evaluates the same sum, so a prefill of T tokens followed by a step equals a prefill of
// T + 1 tokens bit for bit (a zero input contributes an exact zero).
#include "mmf_common.h"

namespace {

constexpr int kConvMaxW = 8;
#pragma clang fp contract(off)

__device__ __forceinline__ float conv_act(float pre, int activation) {
    return activation ? __fdiv_rn(pre, __fadd_rn(1.0f, mmf_exp(-pre))) : pre;
}

// One thread per (b, t, d); d runs fastest, so the W loads of a thread are coalesced across the wave.
template <typename T>
__global__ __launch_bounds__(256) void short_conv_fwd_kernel(const T* __restrict__ x, const T* __restrict__ weight,
                                                             const T* __restrict__ bias, T* __restrict__ y,
                                                             T* __restrict__ cache, int64_t B, int64_t Tlen, int64_t D, int W,
                                                             int activation) {
    const int64_t n = B * Tlen * D;
    for (int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x; idx < n; idx += (int64_t)gridDim.x * 256) {
        const int64_t d = idx % D, bt = idx / D, t = bt % Tlen, b = bt / Tlen;
        float acc = 0.0f;
        for (int w = 0; w < W; ++w) {
            const int64_t s = t - (W - 1) + w;
            if (s >= 0) acc = __fadd_rn(acc, __fmul_rn(mmf_to_float(weight[d * W + w]), mmf_to_float(x[(b * Tlen + s) * D + d])));
        }
        if (bias) acc = __fadd_rn(acc, mmf_to_float(bias[d]));
        const float pre = mmf_round_to<T>(acc);
        y[idx] = mmf_from_float<T>(conv_act(pre, activation));
        // the cache receives the last W inputs (zeros where the sequence is shorter)
        if (cache && t >= Tlen - W) cache[(b * D + d) * W + (W - (Tlen - t))] = x[idx];
    }
    if (cache && Tlen < W) {
        const int64_t m = B * D * (W - Tlen);
        for (int64_t j = (int64_t)blockIdx.x * 256 + threadIdx.x; j < m; j += (int64_t)gridDim.x * 256) {
            const int64_t w = j % (W - Tlen), bd = j / (W - Tlen);
            cache[bd * W + w] = mmf_from_float<T>(0.0f);
        }
    }
}

// One thread per (b, d): shift the cache, append, evaluate.
template <typename T>
__global__ __launch_bounds__(256) void short_conv_step_kernel(const T* __restrict__ x, const T* __restrict__ weight,
                                                              const T* __restrict__ bias, T* __restrict__ cache,
                                                              T* __restrict__ y, int64_t B, int64_t D, int W, int activation) {
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= B * D) return;
    const int64_t d = idx % D;
    T* c = cache + idx * W;
    float acc = 0.0f;
    for (int w = 0; w < W; ++w) {
        const T v = w + 1 < W ? c[w + 1] : x[idx];
        c[w] = v;
        acc = __fadd_rn(acc, __fmul_rn(mmf_to_float(weight[d * W + w]), mmf_to_float(v)));
    }
    if (bias) acc = __fadd_rn(acc, mmf_to_float(bias[d]));
    const float pre = mmf_round_to<T>(acc);
    y[idx] = mmf_from_float<T>(conv_act(pre, activation));
}

// Backward, first half: dpre[b, t, d] = dy * act'(pre) (fp32, pre recomputed as in the forward) and this workgroup's partial
// sums of dweight[d, w] = sum dpre[b, t, d] * x[b, t - (W-1) + w, d] and dbias[d] = sum dpre.  A thread owns a channel and
// walks the rows blockIdx.y, + gridDim.y, ...; partial row layout [(W + 1) * D]: entry w * D + d, the bias sums at w = W.
template <typename T>
__global__ __launch_bounds__(256) void short_conv_bwd_pre_kernel(const T* __restrict__ x, const T* __restrict__ weight,
                                                                 const T* __restrict__ bias, const T* __restrict__ dy,
                                                                 float* __restrict__ dpre, float* __restrict__ part, int64_t B,
                                                                 int64_t Tlen, int64_t D, int W, int activation) {
    const int64_t d = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (d >= D) return;
    float wv[kConvMaxW], dw[kConvMaxW + 1];
    for (int w = 0; w < kConvMaxW; ++w) { wv[w] = w < W ? mmf_to_float(weight[d * W + w]) : 0.0f; dw[w] = 0.0f; }
    dw[kConvMaxW] = 0.0f;
    const float bv = bias ? mmf_to_float(bias[d]) : 0.0f;
    for (int64_t r = blockIdx.y; r < B * Tlen; r += gridDim.y) {
        const int64_t t = r % Tlen;
        float xv[kConvMaxW], acc = 0.0f;
        for (int w = 0; w < W; ++w) {
            const int64_t s = t - (W - 1) + w;
            xv[w] = s >= 0 ? mmf_to_float(x[(r - (W - 1) + w) * D + d]) : 0.0f;
            if (s >= 0) acc = __fadd_rn(acc, __fmul_rn(wv[w], xv[w]));
        }
        if (bias) acc = __fadd_rn(acc, bv);
        const float pre = mmf_round_to<T>(acc);
        float g = mmf_to_float(dy[r * D + d]);
        if (activation) {
            const float sg = 1.0f / (1.0f + __expf(-pre));
            g *= sg * (1.0f + pre * (1.0f - sg));
        }
        dpre[r * D + d] = g;
        for (int w = 0; w < W; ++w) dw[w] += g * xv[w];
        dw[kConvMaxW] += g;
    }
    float* p = part + (int64_t)blockIdx.y * (W + 1) * D;
    for (int w = 0; w < W; ++w) p[w * D + d] = dw[w];
    p[W * D + d] = dw[kConvMaxW];
}

// Backward, second half: dx[b, s, d] = sum_w weight[d, w] * dpre[b, s + (W-1) - w, d] over the positions inside the sequence.
template <typename T>
__global__ __launch_bounds__(256) void short_conv_bwd_dx_kernel(const float* __restrict__ dpre, const T* __restrict__ weight,
                                                                T* __restrict__ dx, int64_t B, int64_t Tlen, int64_t D, int W) {
    const int64_t n = B * Tlen * D;
    for (int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x; idx < n; idx += (int64_t)gridDim.x * 256) {
        const int64_t d = idx % D, bt = idx / D, s = bt % Tlen;
        float acc = 0.0f;
        for (int w = 0; w < W; ++w) {
            const int64_t t = s + (W - 1) - w;
            if (t < Tlen) acc += mmf_to_float(weight[d * W + w]) * dpre[(bt + (W - 1) - w) * D + d];
        }
        dx[idx] = mmf_from_float<T>(acc);
    }
}

// out[k] = sum over the groups of part[g, k], groups in index order (a few thousand entries: one thread per entry).
__global__ __launch_bounds__(256) void short_conv_colsum_kernel(const float* __restrict__ part, int groups, int64_t K,
                                                                float* __restrict__ out) {
    const int64_t k = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (k >= K) return;
    float s = 0.0f;
    for (int g = 0; g < groups; ++g) s += part[(int64_t)g * K + k];
    out[k] = s;
}

unsigned grid_for(int64_t n) {
    const int64_t g = mmf_ceil_div(n, 256);
    return (unsigned)(g < 1 ? 1 : g > 65536 ? 65536 : g);
}

}  // namespace

extern "C" {

int mmf_short_conv_max_kernel_size(void) { return kConvMaxW; }

int mmf_short_conv_fwd(const void* x, const void* weight, const void* bias, void* y, void* cache, int64_t B, int64_t T,
                       int64_t D, int W, int activation, int dtype, void* stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (B < 0 || T < 0 || D <= 0 || W < 1 || activation < 0 || activation > 1) return MMF_ERR_ARG;
    if (W > kConvMaxW) return MMF_ERR_WIDE;
    if (B == 0 || T == 0) return 0;
    if (!x || !weight || !y) return MMF_ERR_ARG;
#define MMF_CF(T_) short_conv_fwd_kernel<T_><<<grid_for(B * T * D), 256, 0, stream>>>(static_cast<const T_*>(x), \
        static_cast<const T_*>(weight), static_cast<const T_*>(bias), static_cast<T_*>(y), static_cast<T_*>(cache), B, T, D, W, activation)
    switch (dtype) {
        case MMF_F32: MMF_CF(float); break;
        case MMF_BF16: MMF_CF(bf16_t); break;
        case MMF_F16: MMF_CF(f16_t); break;
        default: return MMF_ERR_ARG;
    }
#undef MMF_CF
    MMF_CHECK_LAUNCH();
    return 0;
}

int mmf_short_conv_step(const void* x, const void* weight, const void* bias, void* cache, void* y, int64_t B, int64_t D, int W,
                        int activation, int dtype, void* stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (B < 0 || D <= 0 || W < 1 || activation < 0 || activation > 1) return MMF_ERR_ARG;
    if (W > kConvMaxW) return MMF_ERR_WIDE;
    if (B == 0) return 0;
    if (!x || !weight || !cache || !y) return MMF_ERR_ARG;
#define MMF_CS(T_) short_conv_step_kernel<T_><<<grid_for(B * D), 256, 0, stream>>>(static_cast<const T_*>(x), \
        static_cast<const T_*>(weight), static_cast<const T_*>(bias), static_cast<T_*>(cache), static_cast<T_*>(y), B, D, W, activation)
    switch (dtype) {
        case MMF_F32: MMF_CS(float); break;
        case MMF_BF16: MMF_CS(bf16_t); break;
        case MMF_F16: MMF_CS(f16_t); break;
        default: return MMF_ERR_ARG;
    }
#undef MMF_CS
    MMF_CHECK_LAUNCH();
    return 0;
}

int mmf_short_conv_bwd_groups(int64_t rows) { return (int)(rows < 1 ? 1 : rows < 256 ? rows : 256); }

int mmf_short_conv_bwd(const void* x, const void* weight, const void* bias, const void* dy, void* dx, float* dpre, float* partial,
                       float* dweight_bias, int64_t B, int64_t T, int64_t D, int W, int activation, int dtype, void* stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (B < 0 || T < 0 || D <= 0 || W < 1 || activation < 0 || activation > 1) return MMF_ERR_ARG;
    if (W > kConvMaxW) return MMF_ERR_WIDE;
    if (!dweight_bias) return MMF_ERR_ARG;
    const int64_t entries = (int64_t)(W + 1) * D;
    if (B == 0 || T == 0) {                                      // no rows: the sums are zero
        short_conv_colsum_kernel<<<grid_for(entries), 256, 0, stream>>>(nullptr, 0, entries, dweight_bias);
        MMF_CHECK_LAUNCH();
        return 0;
    }
    if (!x || !weight || !dy || !dx || !dpre || !partial) return MMF_ERR_ARG;
    const int groups = mmf_short_conv_bwd_groups(B * T);
    dim3 grid((unsigned)mmf_ceil_div(D, 256), (unsigned)groups);
#define MMF_CB(T_) do { \
        short_conv_bwd_pre_kernel<T_><<<grid, 256, 0, stream>>>(static_cast<const T_*>(x), static_cast<const T_*>(weight), \
            static_cast<const T_*>(bias), static_cast<const T_*>(dy), dpre, partial, B, T, D, W, activation); \
        short_conv_bwd_dx_kernel<T_><<<grid_for(B * T * D), 256, 0, stream>>>(dpre, static_cast<const T_*>(weight), \
            static_cast<T_*>(dx), B, T, D, W); } while (0)
    switch (dtype) {
        case MMF_F32: MMF_CB(float); break;
        case MMF_BF16: MMF_CB(bf16_t); break;
        case MMF_F16: MMF_CB(f16_t); break;
        default: return MMF_ERR_ARG;
    }
#undef MMF_CB
    MMF_CHECK_LAUNCH();
    short_conv_colsum_kernel<<<grid_for(entries), 256, 0, stream>>>(partial, groups, entries, dweight_bias);
    MMF_CHECK_LAUNCH();
    return 0;
}

}  // extern "C"
