// HGRN recurrence  h_t = g_t * h_{t-1} + x_t  and the gate math in front of it.
//
//   mmf_hgrn_recurrent : g is the decay itself (linear domain); strictly sequential
//                        arithmetic (multiply, round, add, round) like
//                        mmfreelm/ops/hgrn/recurrent_fuse.py:32-68 / ops/hgrn/naive.py:8-31.
//   mmf_hgrn_chunk     : g is the log decay; the two-pass chunked algorithm of
//                        mmfreelm/ops/hgrn/chunk.py:49-116 in ONE kernel without the two
//                        fp32 [B,H,T,D] scratch tensors of chunk.py:232-233.
//   mmf_hgrn_gate      : sigmoid / lower bound / swiglu / mask of
//                        mmfreelm/layers/hgrn_bit.py:113-120 as one elementwise pass.
//   mmf_hgrn_step      : the same gate math fused with one recurrence step (decode, T = 1).
//
// Layout: x, g, o are [BH, T, D] contiguous; a lane owns one channel d, a wave 64
// consecutive channels (128 B per time step in bf16), a workgroup of NW waves one
// 64-channel column of one (b, h).  Time is cut into chunks of 64 steps; a wave holds a
// whole chunk of x and g in registers, so all of a chunk's loads are in flight together
// and NW chunks per workgroup overlap.
//   recurrent: the waves take turns ("baton" = running state in LDS): on its turn a wave
//              runs its 64 dependent steps from registers, hands the state on, and only
//              then converts/stores its outputs and issues the loads of its next chunk,
//              so the serial chain sees no memory latency.
//   chunk    : every wave scans its chunk from zero state in parallel, publishes the chunk
//              summary (last h, sum of g), every wave replays the short carry chain over
//              the NW summaries, then fixes its chunk up from registers.
#include "mmf_common.h"
#include "../../include/mmf.h"

namespace {

constexpr int kCH = 64;   // time steps per register-resident chunk

template <typename T> struct Raw;
template <> struct Raw<float> {
    using type = float;
    static __device__ __forceinline__ float get(float v) { return v; }
};
template <> struct Raw<bf16_t> {
    using type = uint16_t;
    static __device__ __forceinline__ float get(uint16_t v) { return __uint_as_float(((uint32_t)v) << 16); }
};
template <> struct Raw<f16_t> {
    using type = _Float16;
    static __device__ __forceinline__ float get(_Float16 v) { return (float)v; }
};

template <typename T>
__device__ __forceinline__ void store_one(T* p, float v) { *p = mmf_from_float<T>(v); }

// -------------------------------------------------------------------------- recurrent
template <typename T, int NW>
__global__ __launch_bounds__(64 * NW) void hgrn_recurrent_kernel(const T* __restrict__ x, const T* __restrict__ g,
                                                                 const float* __restrict__ h0, T* __restrict__ o,
                                                                 float* __restrict__ ht, int64_t Tlen, int64_t D) {
    using R = typename Raw<T>::type;
    __shared__ float baton[64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t bh = blockIdx.y;
    const int64_t d = (int64_t)blockIdx.x * 64 + lane;
    const bool active = d < D;
    const int64_t base = bh * Tlen * D + d;
    const R* xr_p = reinterpret_cast<const R*>(x);
    const R* gr_p = reinterpret_cast<const R*>(g);

    const int64_t NC = (Tlen + kCH - 1) / kCH;
    const int64_t rounds = (NC + NW - 1) / NW * NW;

    R xr[kCH], gr[kCH];
    float hs[kCH];

    auto load_chunk = [&](int64_t c) {
        const int64_t t0 = c * kCH;
#pragma unroll
        for (int t = 0; t < kCH; ++t) {
            if (active && t0 + t < Tlen) {
                xr[t] = xr_p[base + (t0 + t) * D];
                gr[t] = gr_p[base + (t0 + t) * D];
            }
        }
    };

    if (wave == 0) baton[lane] = (h0 && active) ? h0[bh * D + d] : 0.0f;
    if (wave < NC) load_chunk(wave);
    __syncthreads();

    for (int64_t r = 0; r < rounds; ++r) {
        const bool mine = (r % NW) == wave && r < NC;
        const int64_t t0 = r * kCH;
        if (mine) {
            float h = baton[lane];
#pragma unroll
            for (int t = 0; t < kCH; ++t) {
                if (t0 + t < Tlen) {
                    h = __fadd_rn(__fmul_rn(Raw<T>::get(gr[t]), h), Raw<T>::get(xr[t]));
                    hs[t] = h;
                }
            }
            baton[lane] = h;
        }
        __syncthreads();
        if (mine) {
#pragma unroll
            for (int t = 0; t < kCH; ++t)
                if (active && t0 + t < Tlen) store_one<T>(o + base + (t0 + t) * D, hs[t]);
            if (r + NW < NC) load_chunk(r + NW);
        }
    }
    if (ht && wave == 0 && active) ht[bh * D + d] = baton[lane];
}

// -------------------------------------------------------------------------- chunk
template <typename T, int NW>
__global__ __launch_bounds__(64 * NW) void hgrn_chunk_kernel(const T* __restrict__ x, const T* __restrict__ g,
                                                             const float* __restrict__ h0, T* __restrict__ o,
                                                             float* __restrict__ ht, int64_t Tlen, int64_t D, int chunk) {
    using R = typename Raw<T>::type;
    __shared__ float sum_h[2][NW][64];
    __shared__ float sum_g[2][NW][64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t bh = blockIdx.y;
    const int64_t d = (int64_t)blockIdx.x * 64 + lane;
    const bool active = d < D;
    const int64_t base = bh * Tlen * D + d;
    const R* xr_p = reinterpret_cast<const R*>(x);
    const R* gr_p = reinterpret_cast<const R*>(g);

    const int64_t NC = (Tlen + chunk - 1) / chunk;
    const int64_t supers = (NC + NW - 1) / NW;

    R xr[kCH], gr[kCH];
    float hl[kCH], gc[kCH];
    float carry = 0.0f;   // fixed-up last output of the chunk before this super-step

    for (int64_t sidx = 0; sidx < supers; ++sidx) {
        const int64_t c = sidx * NW + wave;
        const int64_t t0 = c * chunk;
        const bool have = c < NC;
        const int pb = (int)(sidx & 1);
        if (have) {
#pragma unroll
            for (int t = 0; t < kCH; ++t)
                if (active && t < chunk && t0 + t < Tlen) {
                    xr[t] = xr_p[base + (t0 + t) * D];
                    gr[t] = gr_p[base + (t0 + t) * D];
                }
            float h = (c == 0 && h0 && active) ? h0[bh * D + d] : 0.0f;
            float a = 0.0f;
#pragma unroll
            for (int t = 0; t < kCH; ++t)
                if (t < chunk && t0 + t < Tlen) {
                    const float gv = Raw<T>::get(gr[t]);
                    h = __fadd_rn(__fmul_rn(__expf(gv), h), Raw<T>::get(xr[t]));
                    a = __fadd_rn(a, gv);
                    hl[t] = h;
                    gc[t] = a;
                }
            sum_h[pb][wave][lane] = h;
            sum_g[pb][wave][lane] = a;
        }
        __syncthreads();
        // carry chain over the chunks of this super-step that precede this wave's chunk
        float prev = carry;          // fixed-up last output of chunk sidx*NW - 1
        float mine_prev = carry;
#pragma unroll
        for (int w = 0; w < NW; ++w) {
            if (w == wave) mine_prev = prev;
            const int64_t cw = sidx * NW + w;
            if (cw < NC) {
                const float hw = sum_h[pb][w][lane], gw = sum_g[pb][w][lane];
                prev = (cw == 0) ? hw : __fadd_rn(hw, __fmul_rn(__expf(gw), prev));
            }
        }
        carry = prev;
        if (have) {
#pragma unroll
            for (int t = 0; t < kCH; ++t)
                if (active && t < chunk && t0 + t < Tlen) {
                    const float v = (c == 0) ? hl[t] : __fadd_rn(hl[t], __fmul_rn(__expf(gc[t]), mine_prev));
                    store_one<T>(o + base + (t0 + t) * D, v);
                }
        }
        // sum_* buffers alternate between super-steps, so one barrier per super-step is enough
    }
    if (ht && wave == 0 && active) ht[bh * D + d] = carry;
}

// -------------------------------------------------------------------------- gate math
// g_out = T( lb + (1 - lb) * sigmoid(f) )   (lb == null: T(sigmoid(f)))
// x_out = T( (i * (1 - g_out)) / (1 + exp(-i)) ), zeroed where mask == 0
template <typename T>
__device__ __forceinline__ void gate_math(float iv, float fv, bool has_lb, float lb, float& xo, float& go) {
    float s = mmf_sigmoid(fv);
    if (has_lb) s = __fadd_rn(lb, __fmul_rn(__fsub_rn(1.0f, lb), s));
    go = mmf_round_to<T>(s);
    const float u = __fsub_rn(1.0f, go);
    xo = mmf_round_to<T>(__fdiv_rn(__fmul_rn(iv, u), __fadd_rn(1.0f, mmf_exp(-iv))));
}

template <typename T>
__global__ __launch_bounds__(256) void hgrn_gate_kernel(const T* __restrict__ i_in, int64_t ldi, const T* __restrict__ f_in,
                                                        int64_t ldf, const float* __restrict__ lb,
                                                        const uint8_t* __restrict__ mask, T* __restrict__ x_out,
                                                        T* __restrict__ g_out, int64_t rows, int64_t D) {
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= rows * D) return;
    const int64_t r = idx / D, d = idx % D;
    float xo, go;
    gate_math<T>(mmf_to_float(i_in[r * ldi + d]), mmf_to_float(f_in[r * ldf + d]), lb != nullptr, lb ? lb[d] : 0.0f, xo, go);
    if (mask && mask[r] == 0) xo = 0.0f;
    x_out[idx] = mmf_from_float<T>(xo);
    g_out[idx] = mmf_from_float<T>(go);
}

template <typename T>
__global__ __launch_bounds__(256) void hgrn_step_kernel(const T* __restrict__ i_in, int64_t ldi, const T* __restrict__ f_in,
                                                        int64_t ldf, const float* __restrict__ lb,
                                                        const uint8_t* __restrict__ mask, float* __restrict__ state,
                                                        T* __restrict__ o, int64_t rows, int64_t D) {
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= rows * D) return;
    const int64_t r = idx / D, d = idx % D;
    float xo, go;
    gate_math<T>(mmf_to_float(i_in[r * ldi + d]), mmf_to_float(f_in[r * ldf + d]), lb != nullptr, lb ? lb[d] : 0.0f, xo, go);
    if (mask && mask[r] == 0) xo = 0.0f;
    const float h = __fadd_rn(__fmul_rn(go, state[idx]), xo);
    state[idx] = h;
    o[idx] = mmf_from_float<T>(h);
}

// ht = h0 (or zeros) for an empty sequence; a kernel, not a memset, so it can be graph captured.
__global__ __launch_bounds__(256) void state_init_kernel(const float* __restrict__ h0, float* __restrict__ ht, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) ht[i] = h0 ? h0[i] : 0.0f;
}

template <typename T>
int launch_recurrent(const void* x, const void* g, const float* h0, void* o, float* ht, int64_t BH, int64_t Tlen,
                     int64_t D, hipStream_t s) {
    dim3 grid((unsigned)mmf_ceil_div(D, 64), (unsigned)BH);
    const int64_t NC = mmf_ceil_div(Tlen, kCH);
    if (NC >= 8)
        hgrn_recurrent_kernel<T, 8><<<grid, 512, 0, s>>>(static_cast<const T*>(x), static_cast<const T*>(g), h0,
                                                         static_cast<T*>(o), ht, Tlen, D);
    else if (NC >= 2)
        hgrn_recurrent_kernel<T, 2><<<grid, 128, 0, s>>>(static_cast<const T*>(x), static_cast<const T*>(g), h0,
                                                         static_cast<T*>(o), ht, Tlen, D);
    else
        hgrn_recurrent_kernel<T, 1><<<grid, 64, 0, s>>>(static_cast<const T*>(x), static_cast<const T*>(g), h0,
                                                        static_cast<T*>(o), ht, Tlen, D);
    MMF_CHECK_LAUNCH();
    return 0;
}

template <typename T>
int launch_chunk(const void* x, const void* g, const float* h0, void* o, float* ht, int64_t BH, int64_t Tlen,
                 int64_t D, int chunk, hipStream_t s) {
    dim3 grid((unsigned)mmf_ceil_div(D, 64), (unsigned)BH);
    const int64_t NC = mmf_ceil_div(Tlen, chunk);
    if (NC >= 8)
        hgrn_chunk_kernel<T, 8><<<grid, 512, 0, s>>>(static_cast<const T*>(x), static_cast<const T*>(g), h0,
                                                     static_cast<T*>(o), ht, Tlen, D, chunk);
    else if (NC >= 2)
        hgrn_chunk_kernel<T, 2><<<grid, 128, 0, s>>>(static_cast<const T*>(x), static_cast<const T*>(g), h0,
                                                     static_cast<T*>(o), ht, Tlen, D, chunk);
    else
        hgrn_chunk_kernel<T, 1><<<grid, 64, 0, s>>>(static_cast<const T*>(x), static_cast<const T*>(g), h0,
                                                    static_cast<T*>(o), ht, Tlen, D, chunk);
    MMF_CHECK_LAUNCH();
    return 0;
}

template <typename T>
int launch_gate(const void* i_in, int64_t ldi, const void* f_in, int64_t ldf, const float* lb, const uint8_t* mask,
                void* x_out, void* g_out, float* state, int64_t rows, int64_t D, bool step, hipStream_t s) {
    const int64_t n = rows * D;
    if (n == 0) return 0;
    const unsigned blocks = (unsigned)mmf_ceil_div(n, 256);
    if (step)
        hgrn_step_kernel<T><<<blocks, 256, 0, s>>>(static_cast<const T*>(i_in), ldi, static_cast<const T*>(f_in), ldf, lb,
                                                   mask, state, static_cast<T*>(x_out), rows, D);
    else
        hgrn_gate_kernel<T><<<blocks, 256, 0, s>>>(static_cast<const T*>(i_in), ldi, static_cast<const T*>(f_in), ldf, lb,
                                                   mask, static_cast<T*>(x_out), static_cast<T*>(g_out), rows, D);
    MMF_CHECK_LAUNCH();
    return 0;
}

}  // namespace

extern "C" {

int mmf_hgrn_recurrent(const void* x, const void* g, const float* h0, void* o, float* ht, int64_t BH, int64_t T,
                       int64_t D, int dtype, void* stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (BH < 0 || T < 0 || D <= 0 || BH > 65535) return MMF_ERR_ARG;
    if (BH == 0) return 0;
    if (T == 0) {   // nothing to scan: the final state is the initial one
        if (ht) {
            state_init_kernel<<<(unsigned)mmf_ceil_div(BH * D, 256), 256, 0, stream>>>(h0, ht, BH * D);
            MMF_CHECK_LAUNCH();
        }
        return 0;
    }
    if (!x || !g || !o) return MMF_ERR_ARG;
    switch (dtype) {
        case MMF_F32: return launch_recurrent<float>(x, g, h0, o, ht, BH, T, D, stream);
        case MMF_BF16: return launch_recurrent<bf16_t>(x, g, h0, o, ht, BH, T, D, stream);
        case MMF_F16: return launch_recurrent<f16_t>(x, g, h0, o, ht, BH, T, D, stream);
    }
    return MMF_ERR_ARG;
}

int mmf_hgrn_chunk(const void* x, const void* g, const float* h0, void* o, float* ht, int64_t BH, int64_t T, int64_t D,
                   int chunk, int dtype, void* stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (BH < 0 || T < 0 || D <= 0 || BH > 65535 || chunk < 1 || chunk > kCH) return MMF_ERR_ARG;
    if (BH == 0) return 0;
    if (T == 0) {
        if (ht) {
            state_init_kernel<<<(unsigned)mmf_ceil_div(BH * D, 256), 256, 0, stream>>>(h0, ht, BH * D);
            MMF_CHECK_LAUNCH();
        }
        return 0;
    }
    if (!x || !g || !o) return MMF_ERR_ARG;
    switch (dtype) {
        case MMF_F32: return launch_chunk<float>(x, g, h0, o, ht, BH, T, D, chunk, stream);
        case MMF_BF16: return launch_chunk<bf16_t>(x, g, h0, o, ht, BH, T, D, chunk, stream);
        case MMF_F16: return launch_chunk<f16_t>(x, g, h0, o, ht, BH, T, D, chunk, stream);
    }
    return MMF_ERR_ARG;
}

int mmf_hgrn_gate(const void* i_in, int64_t ldi, const void* f_in, int64_t ldf, const float* lower_bound,
                  const uint8_t* mask, void* x_out, void* g_out, int64_t rows, int64_t D, int dtype, void* stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (rows < 0 || D <= 0 || ldi < D || ldf < D) return MMF_ERR_ARG;
    if (rows > 0 && (!i_in || !f_in || !x_out || !g_out)) return MMF_ERR_ARG;
    switch (dtype) {
        case MMF_F32: return launch_gate<float>(i_in, ldi, f_in, ldf, lower_bound, mask, x_out, g_out, nullptr, rows, D, false, stream);
        case MMF_BF16: return launch_gate<bf16_t>(i_in, ldi, f_in, ldf, lower_bound, mask, x_out, g_out, nullptr, rows, D, false, stream);
        case MMF_F16: return launch_gate<f16_t>(i_in, ldi, f_in, ldf, lower_bound, mask, x_out, g_out, nullptr, rows, D, false, stream);
    }
    return MMF_ERR_ARG;
}

int mmf_hgrn_step(const void* i_in, int64_t ldi, const void* f_in, int64_t ldf, const float* lower_bound,
                  const uint8_t* mask, float* state, void* o, int64_t rows, int64_t D, int dtype, void* stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (rows < 0 || D <= 0 || ldi < D || ldf < D) return MMF_ERR_ARG;
    if (rows > 0 && (!i_in || !f_in || !state || !o)) return MMF_ERR_ARG;
    switch (dtype) {
        case MMF_F32: return launch_gate<float>(i_in, ldi, f_in, ldf, lower_bound, mask, o, nullptr, state, rows, D, true, stream);
        case MMF_BF16: return launch_gate<bf16_t>(i_in, ldi, f_in, ldf, lower_bound, mask, o, nullptr, state, rows, D, true, stream);
        case MMF_F16: return launch_gate<f16_t>(i_in, ldi, f_in, ldf, lower_bound, mask, o, nullptr, state, rows, D, true, stream);
    }
    return MMF_ERR_ARG;
}

}  // extern "C"
