// Backward kernels of the training side of the path (the reference's Triton backward kernels and its fused loss).
//
//   mmf_rmsnorm_bwd          mmfreelm/modules/layernorm.py:245-330 (RMSNorm), mmfreelm/modules/fused_norm_gate.py:210-300
//                            (swish-gated), mmfreelm/ops/fusedbitnet.py:209-317 (BitLinear's norm with the quantised
//                            output recomputed for the weight gradient; the straight-through estimator of :556-581 passes
//                            the gradient through both quantisers unchanged)
//   mmf_swiglu_bwd           mmfreelm/modules/activations.py:121-126
//   mmf_hgrn_gate_bwd        autograd of mmfreelm/layers/hgrn_bit.py:113-120 (sigmoid, lower bound, swiglu(i, 1 - f), mask)
//   mmf_hgrn_recurrent_bwd   mmfreelm/ops/hgrn/recurrent_fuse.py:89-133 (and, with log gates, the gradient that
//                            mmfreelm/ops/hgrn/chunk.py:137-220 computes chunk-wise)
//   mmf_cross_entropy_train_fwd / _bwd   mmfreelm/modules/fused_cross_entropy.py:26-98 / :98-160 (label smoothing, logit
//                            scale, z-loss)
//
// Gradients are fp32 arithmetic with hardware exp / log, checked against autograd
// through the CPU restatement to a tolerance: unlike the forward path nothing downstream re-quantises them, so there
// is no bit-level contract to keep.  The one exception is the recomputed quantised output of the BitLinear norm: it
// follows the forward arithmetic exactly (fp64 sum of squares, separately rounded products, round-half-to-even), so the
// weight gradient sees the codes the forward pass used.
// Per-column sums over rows (norm weight, lower bound) are accumulated per workgroup in registers, written as
// [groups, K] partials and added up in a fixed order by a second small kernel: no atomics, same bits every run.
#include "mmf_common.h"

namespace {

constexpr int kBT = 512;

__device__ __forceinline__ float block_sum_f(float v, float* red) {
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    const int w = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) red[w] = v;
    __syncthreads();
    float s = 0.0f;
#pragma unroll
    for (int i = 0; i < kBT / 64; ++i) s += red[i];
    __syncthreads();
    return s;
}
__device__ __forceinline__ float fast_sigmoid(float x) { return 1.0f / (1.0f + __expf(-x)); }

// ------------------------------------------------------------------------------------------ norms
enum BwdMode : int { BWD_PLAIN = 0, BWD_GATED = 1, BWD_QUANT = 2 };

struct NormBwdArgs {
    const void* x;       // [M, K] what the norm normalised (the summed residual stream where there was a residual)
    const void* gate;    // GATED: the swish gate o [M, K]
    const void* w;       // [K] or null
    const void* dy;      // [M, K]
    const void* dres;    // [M, K] or null: gradient that arrives through the residual output (prenorm)
    void* dx;            // [M, K]
    void* dgate;         // GATED: [M, K]
    void* y;             // QUANT: the quantised (de-quantised values) output recomputed, [M, K]
    float* dw_part;      // [gridDim.x, K] or null
    int64_t M, ldx, ldg, lddy;
    int K;
    float eps;
    double inv_K;
};

// VEC: K, the row strides and the base addresses allow 4-element vector accesses (a thread's 4 channels are then all inside
// the row or all outside it).
template <typename T, typename TW, int NV, int MODE, bool VEC>
__global__ __launch_bounds__(kBT) void rmsnorm_bwd_kernel(NormBwdArgs a) {
    __shared__ double red_d[kBT / 64];
    __shared__ float red_f[kBT / 64];
    const int K = a.K;
    const TW* w = static_cast<const TW*>(a.w);
    float wv[NV][4], dwacc[NV][4];
#pragma unroll
    for (int v = 0; v < NV; ++v) {
        const int k0 = (v * kBT + (int)threadIdx.x) * 4;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            wv[v][i] = (w && k0 + i < K) ? mmf_to_float(w[k0 + i]) : 1.0f;
            dwacc[v][i] = 0.0f;
        }
    }
    for (int64_t row = blockIdx.x; row < a.M; row += gridDim.x) {
        const T* x = static_cast<const T*>(a.x) + row * a.ldx;
        const T* dy = static_cast<const T*>(a.dy) + row * a.lddy;
        const T* gt = MODE == BWD_GATED ? static_cast<const T*>(a.gate) + row * a.ldg : nullptr;
        const T* dr = a.dres ? static_cast<const T*>(a.dres) + row * (int64_t)K : nullptr;
        float xv[NV][4], dv[NV][4], gv[MODE == BWD_GATED ? NV : 1][4], rv[NV][4];
        double ss = 0.0;
        // every load of the row is issued before anything is converted
        Raw4<T> xr[NV], dyr[NV], gr[MODE == BWD_GATED ? NV : 1], rr[NV];
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            const int k0 = (v * kBT + (int)threadIdx.x) * 4;
            if (k0 < K) {
                xr[v] = raw4_load<T, VEC>(x, k0, K);
                dyr[v] = raw4_load<T, VEC>(dy, k0, K);
                if constexpr (MODE == BWD_GATED) gr[v] = raw4_load<T, VEC>(gt, k0, K);
                if (dr) rr[v] = raw4_load<T, VEC>(dr, k0, K);
            }
        }
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            const int k0 = (v * kBT + (int)threadIdx.x) * 4;
            if (k0 < K) {
                raw4_unpack<T>(xr[v], xv[v]);
                raw4_unpack<T>(dyr[v], dv[v]);
                if constexpr (MODE == BWD_GATED) raw4_unpack<T>(gr[v], gv[v]);
                if (dr) raw4_unpack<T>(rr[v], rv[v]);
            }
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const bool in = k0 + i < K;
                xv[v][i] = in ? xv[v][i] : 0.0f;
                dv[v][i] = in ? dv[v][i] : 0.0f;
                if constexpr (MODE == BWD_GATED) gv[v][i] = in ? gv[v][i] : 0.0f;
                rv[v][i] = (dr && in) ? rv[v][i] : 0.0f;
                ss = mmf_add_square(ss, xv[v][i]);
            }
        }
        ss = mmf_block_sum<kBT / 64>(ss, red_d);
        const float rstd = mmf_rstd(ss, K, a.inv_K, a.eps);      // the forward's rstd, bit for bit
        float xh[NV][4], wdy[NV][4], dot = 0.0f, amax = 0.0f;
#pragma unroll
        for (int v = 0; v < NV; ++v)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                xh[v][i] = __fmul_rn(xv[v][i], rstd);
                float d = dv[v][i];
                if constexpr (MODE == BWD_GATED) {
                    const float yv = xh[v][i] * wv[v][i], o = gv[v][i], sg = fast_sigmoid(o);
                    gv[v][i] = d * yv * (sg + o * sg * (1.0f - sg));     // gradient of the gate
                    d = d * o * sg;
                }
                if constexpr (MODE == BWD_QUANT) amax = fmaxf(amax, fabsf(__fmul_rn(xh[v][i], wv[v][i])));
                dwacc[v][i] += d * xh[v][i];
                wdy[v][i] = d * wv[v][i];
                dot += xh[v][i] * wdy[v][i];
            }
        const float c1 = block_sum_f(dot, red_f) / (float)K;
        T* dx = static_cast<T*>(a.dx) + row * (int64_t)K;
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            const int k0 = (v * kBT + (int)threadIdx.x) * 4;
            float o[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) o[i] = (wdy[v][i] - xh[v][i] * c1) * rstd + rv[v][i];
            raw4_store<T, VEC>(dx, k0, K, o);
            if constexpr (MODE == BWD_GATED) raw4_store<T, VEC>(static_cast<T*>(a.dgate) + row * (int64_t)K, k0, K, gv[v]);
        }
        if constexpr (MODE == BWD_QUANT) {
            amax = mmf_block_max<kBT / 64>(amax, red_f);
            const float scale = __fdiv_rn(127.0f, fmaxf(amax, 1e-5f)), deq = __fdiv_rn(1.0f, scale);
            T* y = static_cast<T*>(a.y) + row * (int64_t)K;
#pragma unroll
            for (int v = 0; v < NV; ++v) {
                const int k0 = (v * kBT + (int)threadIdx.x) * 4;
                float o[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) o[i] = __fmul_rn((float)mmf_code(__fmul_rn(xh[v][i], wv[v][i]), scale), deq);
                raw4_store<T, VEC>(y, k0, K, o);
            }
        }
    }
    if (a.dw_part) {
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            const int k0 = (v * kBT + (int)threadIdx.x) * 4;
#pragma unroll
            for (int i = 0; i < 4; ++i)
                if (k0 + i < K) a.dw_part[(int64_t)blockIdx.x * K + k0 + i] = dwacc[v][i];
        }
    }
}

// out[k] = T(sum_g part[g, k]).  A workgroup owns 32 columns; its 32 lanes per column each add every 32nd group in index order and
// the 32 lane sums are then added in lane order, so the result depends on the shape only.
constexpr int kColsumCols = 32, kColsumLanes = 32;
template <typename T>
__global__ __launch_bounds__(kColsumCols * kColsumLanes) void colsum_kernel(const float* __restrict__ part, int groups, int K,
                                                                            T* __restrict__ out) {
    __shared__ float lane_sum[kColsumLanes][kColsumCols + 1];
    const int c = (int)threadIdx.x % kColsumCols, l = (int)threadIdx.x / kColsumCols;
    const int k = (int)blockIdx.x * kColsumCols + c;
    float s0 = 0.0f, s1 = 0.0f, s2 = 0.0f, s3 = 0.0f;
    if (k < K) {
        int g = l;
        for (; g + 3 * kColsumLanes < groups; g += 4 * kColsumLanes) {
            const float a0 = part[(int64_t)g * K + k], a1 = part[(int64_t)(g + kColsumLanes) * K + k];
            const float a2 = part[(int64_t)(g + 2 * kColsumLanes) * K + k], a3 = part[(int64_t)(g + 3 * kColsumLanes) * K + k];
            s0 += a0; s1 += a1; s2 += a2; s3 += a3;
        }
        for (; g < groups; g += kColsumLanes) s0 += part[(int64_t)g * K + k];
    }
    lane_sum[l][c] = (s0 + s1) + (s2 + s3);
    __syncthreads();
    if (l == 0 && k < K) {
        float s = 0.0f;
#pragma unroll
        for (int i = 0; i < kColsumLanes; ++i) s += lane_sum[i][c];
        out[k] = mmf_from_float<T>(s);
    }
}
template <typename T>
void launch_colsum(const float* part, int groups, int64_t K, T* out, hipStream_t s) {
    colsum_kernel<T><<<(unsigned)mmf_ceil_div(K, kColsumCols), kColsumCols * kColsumLanes, 0, s>>>(part, groups, (int)K, out);
}

template <typename T, typename TW, int MODE, bool VEC>
int launch_norm_bwd_v(const NormBwdArgs& a, int groups, hipStream_t s) {
    const int nv = (int)mmf_ceil_div(a.K, kBT * 4);
    if (nv <= 1) rmsnorm_bwd_kernel<T, TW, 1, MODE, VEC><<<groups, kBT, 0, s>>>(a);
    else if (nv <= 2) rmsnorm_bwd_kernel<T, TW, 2, MODE, VEC><<<groups, kBT, 0, s>>>(a);
    else if (nv <= 4) rmsnorm_bwd_kernel<T, TW, 4, MODE, VEC><<<groups, kBT, 0, s>>>(a);
    else return MMF_ERR_WIDE;
    MMF_CHECK_LAUNCH();
    return 0;
}
template <typename T, typename TW, int MODE>
int launch_norm_bwd(const NormBwdArgs& a, int groups, hipStream_t s) {
    const uintptr_t al = 4 * sizeof(T) - 1;
    auto ok = [&](const void* p) { return (reinterpret_cast<uintptr_t>(p) & al) == 0; };
    const bool vec = a.K % 4 == 0 && a.ldx % 4 == 0 && a.ldg % 4 == 0 && a.lddy % 4 == 0 && ok(a.x) && ok(a.gate) && ok(a.dy) &&
                     ok(a.dres) && ok(a.dx) && ok(a.dgate) && ok(a.y);
    return vec ? launch_norm_bwd_v<T, TW, MODE, true>(a, groups, s) : launch_norm_bwd_v<T, TW, MODE, false>(a, groups, s);
}
template <typename T, typename TW>
int dispatch_norm_bwd(const NormBwdArgs& a, int mode, int groups, hipStream_t s) {
    switch (mode) {
        case BWD_PLAIN: return launch_norm_bwd<T, TW, BWD_PLAIN>(a, groups, s);
        case BWD_GATED: return launch_norm_bwd<T, TW, BWD_GATED>(a, groups, s);
        case BWD_QUANT: return launch_norm_bwd<T, TW, BWD_QUANT>(a, groups, s);
    }
    return MMF_ERR_ARG;
}

// ------------------------------------------------------------------------------------------ swiglu
template <typename T>
__global__ __launch_bounds__(256) void swiglu_bwd_kernel(const T* __restrict__ x, int64_t ldx, const T* __restrict__ y, int64_t ldy,
                                                         const T* __restrict__ g, int64_t ldg, T* __restrict__ dx, int64_t lddx,
                                                         T* __restrict__ dy, int64_t lddy, int64_t rows, int64_t cols) {
    const int64_t n = rows * cols;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) {
        const int64_t r = i / cols, c = i % cols;
        const float xv = mmf_to_float(x[r * ldx + c]), yv = mmf_to_float(y[r * ldy + c]), gv = mmf_to_float(g[r * ldg + c]);
        const float sg = fast_sigmoid(xv);
        dx[r * lddx + c] = mmf_from_float<T>(sg * (1.0f + xv * (1.0f - sg)) * gv * yv);
        dy[r * lddy + c] = mmf_from_float<T>(xv * sg * gv);
    }
}

// ------------------------------------------------------------------------------------------ gate math
// forward: s = sigmoid(f); g = lb + (1 - lb) s; x = i sigmoid(i) (1 - g), 0 on masked rows.  A thread owns 4 channels and walks rows.
template <typename T, bool VEC>
__global__ __launch_bounds__(256) void hgrn_gate_bwd_kernel(const T* __restrict__ i_in, int64_t ldi, const T* __restrict__ f_in,
                                                            int64_t ldf, const float* __restrict__ lb,
                                                            const uint8_t* __restrict__ mask, const T* __restrict__ gx,
                                                            const T* __restrict__ gg, T* __restrict__ di, int64_t lddi,
                                                            T* __restrict__ df, int64_t lddf, float* __restrict__ dlb_part,
                                                            int64_t rows, int D) {
    const int d0 = ((int)blockIdx.x * 256 + (int)threadIdx.x) * 4;
    if (d0 >= D) return;
    float lbv[4], acc[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        lbv[e] = (lb && d0 + e < D) ? lb[d0 + e] : 0.0f;
        acc[e] = 0.0f;
    }
    for (int64_t r = blockIdx.y; r < rows; r += gridDim.y) {
        const bool keep = !(mask && mask[r] == 0);
        float iv4[4], fv4[4], dx4[4], dg4[4], di4[4], df4[4];
        const Raw4<T> ir = raw4_load<T, VEC>(i_in + r * ldi, d0, D), fr = raw4_load<T, VEC>(f_in + r * ldf, d0, D);
        const Raw4<T> xr = raw4_load<T, VEC>(gx + r * (int64_t)D, d0, D), gr = raw4_load<T, VEC>(gg + r * (int64_t)D, d0, D);
        raw4_unpack<T>(ir, iv4); raw4_unpack<T>(fr, fv4); raw4_unpack<T>(xr, dx4); raw4_unpack<T>(gr, dg4);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float iv = iv4[e], fv = fv4[e];
            const float dX = keep ? dx4[e] : 0.0f, dG = dg4[e];
            const float s = fast_sigmoid(fv), g = lb ? lbv[e] + (1.0f - lbv[e]) * s : s;
            const float si = fast_sigmoid(iv), sw = iv * si, u = 1.0f - g;
            const float dgt = dG - dX * sw;                        // u = 1 - g
            const float ds = lb ? dgt * (1.0f - lbv[e]) : dgt;
            if (d0 + e < D) acc[e] += dgt * (1.0f - s);
            di4[e] = dX * u * si * (1.0f + iv * (1.0f - si));
            df4[e] = ds * s * (1.0f - s);
        }
        raw4_store<T, VEC>(di + r * lddi, d0, D, di4);
        raw4_store<T, VEC>(df + r * lddf, d0, D, df4);
    }
    if (dlb_part) {
#pragma unroll
        for (int e = 0; e < 4; ++e)
            if (d0 + e < D) dlb_part[(int64_t)blockIdx.y * D + d0 + e] = acc[e];
    }
}

// ------------------------------------------------------------------------------------------ recurrence
// dh += do_t; dx_t = dh; dg_t = dh * h_{t-1} (* exp(g_t) for log gates); dh *= g_t (exp(g_t)).  A lane owns a channel and a
// workgroup 64 channels of one sequence; its NW waves split the time axis.  Every wave first walks its segment from a zero carry
// and keeps the carry L it would hand to the earlier segment and the product P of its gates, then folds the (L, P) of the later
// segments (carry = L + P * carry, last segment first) into the carry it really starts from, and walks its segment again to
// write the gradients.  Time runs backwards in register blocks of 32 steps whose loads are issued together.
constexpr int kScanBwdBlock = 32, kScanBwdMaxWaves = 8;
template <typename T, bool LOG>
__global__ __launch_bounds__(64 * kScanBwdMaxWaves) void hgrn_recurrent_bwd_kernel(const T* __restrict__ g, const T* __restrict__ o,
                                                                                   const T* __restrict__ dout,
                                                                                   const float* __restrict__ h0, T* __restrict__ dx,
                                                                                   T* __restrict__ dg, int64_t Tlen, int64_t D,
                                                                                   int64_t seg) {
    constexpr int BL = kScanBwdBlock;
    __shared__ float carry_l[kScanBwdMaxWaves][64], carry_p[kScanBwdMaxWaves][64];
    const int lane = (int)threadIdx.x & 63, wave = (int)threadIdx.x >> 6, nw = (int)blockDim.x >> 6;
    const int64_t d = (int64_t)blockIdx.x * 64 + lane, bh = blockIdx.y;
    const bool live = d < D;
    const int64_t base = bh * Tlen * D + (live ? d : 0);
    const int64_t ta = (int64_t)wave * seg, tb = ta + seg < Tlen ? ta + seg : Tlen;   // this wave's steps ta .. tb - 1 (may be none)
    float dh = 0.0f;
    if (nw > 1) {
        float prod = 1.0f;
        if (live)
            for (int64_t t1 = tb; t1 > ta; t1 -= BL) {
                const int64_t t0 = t1 - BL;
                float gv[BL], dv[BL];
#pragma unroll
                for (int j = 0; j < BL; ++j) {
                    const int64_t t = t0 + j;
                    if (t >= ta) {
                        gv[j] = mmf_to_float(g[base + t * D]);
                        dv[j] = mmf_to_float(dout[base + t * D]);
                    }
                }
#pragma unroll
                for (int j = BL - 1; j >= 0; --j)
                    if (t0 + j >= ta) {
                        const float gl = LOG ? __expf(gv[j]) : gv[j];
                        dh = (dh + dv[j]) * gl;
                        prod *= gl;
                    }
            }
        carry_l[wave][lane] = dh;
        carry_p[wave][lane] = prod;
        __syncthreads();
        dh = 0.0f;
        for (int w = nw - 1; w > wave; --w) dh = carry_l[w][lane] + carry_p[w][lane] * dh;
    }
    if (!live) return;
    const float hinit = h0 ? h0[bh * D + d] : 0.0f;
    for (int64_t t1 = tb; t1 > ta; t1 -= BL) {
        const int64_t t0 = t1 - BL;                              // block covers steps max(t0, ta) .. t1 - 1
        float gv[BL], dv[BL], hv[BL];
#pragma unroll
        for (int j = 0; j < BL; ++j) {
            const int64_t t = t0 + j;
            if (t >= ta) {
                gv[j] = mmf_to_float(g[base + t * D]);
                dv[j] = mmf_to_float(dout[base + t * D]);
                hv[j] = t > 0 ? mmf_to_float(o[base + (t - 1) * D]) : hinit;
            }
        }
#pragma unroll
        for (int j = BL - 1; j >= 0; --j) {
            const int64_t t = t0 + j;
            if (t >= ta) {
                const float gl = LOG ? __expf(gv[j]) : gv[j];
                dh += dv[j];
                dx[base + t * D] = mmf_from_float<T>(dh);
                dg[base + t * D] = mmf_from_float<T>(LOG ? dh * hv[j] * gl : dh * hv[j]);
                dh *= gl;
            }
        }
    }
}

// ------------------------------------------------------------------------------------------ cross entropy (training)
// forward: lse, the loss with label smoothing and z-loss, and the z-loss alone, per row (fp32); 512 threads per row.
template <typename T>
__global__ __launch_bounds__(512) void ce_train_fwd_kernel(const T* __restrict__ logits, int64_t ld, int64_t V,
                                                           const int64_t* __restrict__ labels, int64_t ignore_index,
                                                           float smoothing, float logit_scale, float lse_square_scale,
                                                           float* __restrict__ loss, float* __restrict__ lse_out,
                                                           float* __restrict__ z_out) {
    __shared__ float red_m[8], red_s[8], red_t[8];
    const int64_t r = blockIdx.x;
    const T* row = logits + r * ld;
    float mx = -INFINITY, sum = 0.0f, tot = 0.0f;
    for (int64_t c = threadIdx.x; c < V; c += 512) {
        const float v = mmf_to_float(row[c]) * logit_scale;
        tot += v;
        if (v > mx) { sum = mx == -INFINITY ? 0.0f : sum * __expf(mx - v); mx = v; }
        sum += __expf(v - mx);
    }
    for (int o = 32; o > 0; o >>= 1) {
        const float om = __shfl_xor(mx, o, 64), os = __shfl_xor(sum, o, 64);
        const float nm = fmaxf(mx, om);
        if (nm != -INFINITY) sum = (mx == -INFINITY ? 0.0f : sum * __expf(mx - nm)) + (om == -INFINITY ? 0.0f : os * __expf(om - nm));
        mx = nm;
        tot += __shfl_xor(tot, o, 64);
    }
    const int w = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) { red_m[w] = mx; red_s[w] = sum; red_t[w] = tot; }
    __syncthreads();
    if (threadIdx.x == 0) {
        float m = red_m[0], s = red_s[0], t = red_t[0];
        for (int i = 1; i < 8; ++i) {
            const float om = red_m[i], os = red_s[i];
            const float nm = fmaxf(m, om);
            if (nm != -INFINITY) s = (m == -INFINITY ? 0.0f : s * __expf(m - nm)) + (om == -INFINITY ? 0.0f : os * __expf(om - nm));
            m = nm;
            t += red_t[i];
        }
        const float lse = __logf(s) + m;
        lse_out[r] = lse;
        const int64_t label = labels[r];
        float l = 0.0f, z = 0.0f;
        if (label != ignore_index) {
            if (label >= 0 && label < V) {
                const float picked = mmf_to_float(row[label]) * logit_scale;
                l = smoothing > 0.0f ? lse - smoothing * t / (float)V - (1.0f - smoothing) * picked : lse - picked;
            } else if (smoothing > 0.0f) {
                l = smoothing * (lse - t / (float)V);
            }
            z = lse_square_scale * lse * lse;
            l += z;
        }
        loss[r] = l;
        if (z_out) z_out[r] = z;
    }
}

// backward: dlogits = dloss * logit_scale * ( p (1 + 2 zs lse) - onehot (1 - smoothing) - smoothing / V ), p = exp(l - lse)
template <typename T>
__global__ __launch_bounds__(256) void ce_train_bwd_kernel(const T* __restrict__ logits, int64_t ld, int64_t V,
                                                           const int64_t* __restrict__ labels, int64_t ignore_index,
                                                           const float* __restrict__ lse, const float* __restrict__ dloss,
                                                           float smoothing, float logit_scale, float lse_square_scale,
                                                           T* __restrict__ dlogits, int64_t ldd) {
    const int64_t r = blockIdx.y;
    const int64_t label = labels[r];
    const float dl = label == ignore_index ? 0.0f : dloss[r] * logit_scale;
    const float l = lse[r], zf = 1.0f + 2.0f * lse_square_scale * l, neg = smoothing > 0.0f ? smoothing / (float)V : 0.0f;
    const float hot = smoothing > 0.0f ? 1.0f - smoothing : 1.0f;
    for (int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x; c < V; c += (int64_t)gridDim.x * 256) {
        float p = __expf(mmf_to_float(logits[r * ld + c]) * logit_scale - l) * zf;
        if (c == label) p -= hot;
        dlogits[r * ldd + c] = mmf_from_float<T>(dl * (p - neg));
    }
}

}  // namespace

extern "C" {

int mmf_backward_groups(int64_t rows) { return (int)(rows < 1 ? 1 : rows < 1024 ? rows : 1024); }

int mmf_rmsnorm_bwd(int mode, const void* x, int64_t ldx, const void* gate, int64_t ldg, const void* weight, const void* dy,
                    int64_t lddy, const void* dresidual, void* dx, void* dgate, void* y_quant, float* dw_partial, void* dweight,
                    int64_t M, int64_t K, float eps, int x_dtype, int weight_dtype, void* stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (M < 0 || K <= 0 || ldx < K || lddy < K || mode < BWD_PLAIN || mode > BWD_QUANT) return MMF_ERR_ARG;
    if (M == 0) return 0;
    if (!x || !dy || !dx) return MMF_ERR_ARG;
    if (mode == BWD_GATED && (!gate || !dgate || ldg < K)) return MMF_ERR_ARG;
    if (mode == BWD_QUANT && !y_quant) return MMF_ERR_ARG;
    if (weight && dweight && !dw_partial) return MMF_ERR_ARG;
    if (K > kBT * 4 * 4) return MMF_ERR_WIDE;
    const int groups = mmf_backward_groups(M);
    NormBwdArgs a{};
    a.x = x; a.gate = gate; a.w = weight; a.dy = dy; a.dres = dresidual; a.dx = dx; a.dgate = dgate; a.y = y_quant;
    a.dw_part = (weight && dweight) ? dw_partial : nullptr; a.M = M; a.ldx = ldx; a.ldg = ldg; a.lddy = lddy; a.K = (int)K;
    a.eps = eps; a.inv_K = 1.0 / (double)K;
    const bool wf32 = weight_dtype == MMF_F32 || !weight;
    if (!wf32 && weight_dtype != x_dtype) return MMF_ERR_ARG;
    int rc = MMF_ERR_ARG;
    switch (x_dtype) {
        case MMF_F32: rc = dispatch_norm_bwd<float, float>(a, mode, groups, stream); break;
        case MMF_BF16: rc = wf32 ? dispatch_norm_bwd<bf16_t, float>(a, mode, groups, stream) : dispatch_norm_bwd<bf16_t, bf16_t>(a, mode, groups, stream); break;
        case MMF_F16: rc = wf32 ? dispatch_norm_bwd<f16_t, float>(a, mode, groups, stream) : dispatch_norm_bwd<f16_t, f16_t>(a, mode, groups, stream); break;
    }
    if (rc != 0 || !a.dw_part) return rc;
    switch (weight_dtype) {
        case MMF_F32: launch_colsum(dw_partial, groups, K, static_cast<float*>(dweight), stream); break;
        case MMF_BF16: launch_colsum(dw_partial, groups, K, static_cast<bf16_t*>(dweight), stream); break;
        case MMF_F16: launch_colsum(dw_partial, groups, K, static_cast<f16_t*>(dweight), stream); break;
        default: return MMF_ERR_ARG;
    }
    MMF_CHECK_LAUNCH();
    return 0;
}

int mmf_swiglu_bwd(const void* x, int64_t ldx, const void* y, int64_t ldy, const void* g, int64_t ldg, void* dx, int64_t lddx,
                   void* dy, int64_t lddy, int64_t rows, int64_t cols, int dtype, void* stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (rows < 0 || cols < 0) return MMF_ERR_ARG;
    if (rows * cols == 0) return 0;
    if (!x || !y || !g || !dx || !dy || ldx < cols || ldy < cols || ldg < cols || lddx < cols || lddy < cols) return MMF_ERR_ARG;
    const int64_t n = rows * cols;
    const unsigned grid = (unsigned)(mmf_ceil_div(n, 256) < 65536 ? mmf_ceil_div(n, 256) : 65536);
#define MMF_SWB(T) swiglu_bwd_kernel<T><<<grid, 256, 0, stream>>>(static_cast<const T*>(x), ldx, static_cast<const T*>(y), ldy, \
        static_cast<const T*>(g), ldg, static_cast<T*>(dx), lddx, static_cast<T*>(dy), lddy, rows, cols)
    switch (dtype) {
        case MMF_F32: MMF_SWB(float); break;
        case MMF_BF16: MMF_SWB(bf16_t); break;
        case MMF_F16: MMF_SWB(f16_t); break;
        default: return MMF_ERR_ARG;
    }
#undef MMF_SWB
    MMF_CHECK_LAUNCH();
    return 0;
}

int mmf_hgrn_gate_bwd(const void* i_in, int64_t ldi, const void* f_in, int64_t ldf, const float* lower_bound, const uint8_t* mask,
                      const void* grad_x, const void* grad_g, void* di, int64_t lddi, void* df, int64_t lddf, float* dlb_partial,
                      float* dlb, int64_t rows, int64_t D, int dtype, void* stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (rows < 0 || D <= 0 || ldi < D || ldf < D || lddi < D || lddf < D || D > 0x7ffffff0) return MMF_ERR_ARG;
    if (rows == 0) return 0;
    if (!i_in || !f_in || !grad_x || !grad_g || !di || !df) return MMF_ERR_ARG;
    if (lower_bound && dlb && !dlb_partial) return MMF_ERR_ARG;
    const int groups = mmf_backward_groups(rows);
    float* part = (lower_bound && dlb) ? dlb_partial : nullptr;
    dim3 grid((unsigned)mmf_ceil_div(D, 1024), (unsigned)groups);
    const uintptr_t al = (dtype == MMF_F32 ? 16 : 8) - 1;
    auto ok = [&](const void* p) { return (reinterpret_cast<uintptr_t>(p) & al) == 0; };
    const bool vec = D % 4 == 0 && ldi % 4 == 0 && ldf % 4 == 0 && lddi % 4 == 0 && lddf % 4 == 0 && ok(i_in) && ok(f_in) &&
                     ok(grad_x) && ok(grad_g) && ok(di) && ok(df);
#define MMF_GB(T, V) hgrn_gate_bwd_kernel<T, V><<<grid, 256, 0, stream>>>(static_cast<const T*>(i_in), ldi, static_cast<const T*>(f_in), ldf, \
        lower_bound, mask, static_cast<const T*>(grad_x), static_cast<const T*>(grad_g), static_cast<T*>(di), lddi, static_cast<T*>(df), \
        lddf, part, rows, (int)D)
    switch (dtype) {
        case MMF_F32: if (vec) MMF_GB(float, true); else MMF_GB(float, false); break;
        case MMF_BF16: if (vec) MMF_GB(bf16_t, true); else MMF_GB(bf16_t, false); break;
        case MMF_F16: if (vec) MMF_GB(f16_t, true); else MMF_GB(f16_t, false); break;
        default: return MMF_ERR_ARG;
    }
#undef MMF_GB
    MMF_CHECK_LAUNCH();
    if (part) {
        launch_colsum(part, groups, D, dlb, stream);
        MMF_CHECK_LAUNCH();
    }
    return 0;
}

int mmf_hgrn_recurrent_bwd(const void* g, const void* o, const void* grad_o, const float* h0, void* dx, void* dg, int64_t BH,
                           int64_t T, int64_t D, int log_gates, int dtype, void* stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (BH < 0 || T < 0 || D <= 0 || BH > 65535) return MMF_ERR_ARG;
    if (BH == 0 || T == 0) return 0;
    if (!g || !o || !grad_o || !dx || !dg) return MMF_ERR_ARG;
    dim3 grid((unsigned)mmf_ceil_div(D, 64), (unsigned)BH);
    // segments of at least 64 steps, a whole number of register blocks each, at most 8 waves
    int64_t nw = T / 64 < 1 ? 1 : T / 64 > kScanBwdMaxWaves ? kScanBwdMaxWaves : T / 64;
    const int64_t seg = mmf_ceil_div(mmf_ceil_div(T, nw), kScanBwdBlock) * kScanBwdBlock;
    nw = mmf_ceil_div(T, seg);
#define MMF_RB(T_, L_) hgrn_recurrent_bwd_kernel<T_, L_><<<grid, (unsigned)(64 * nw), 0, stream>>>(static_cast<const T_*>(g), \
        static_cast<const T_*>(o), static_cast<const T_*>(grad_o), h0, static_cast<T_*>(dx), static_cast<T_*>(dg), T, D, seg)
    switch (dtype) {
        case MMF_F32: if (log_gates) MMF_RB(float, true); else MMF_RB(float, false); break;
        case MMF_BF16: if (log_gates) MMF_RB(bf16_t, true); else MMF_RB(bf16_t, false); break;
        case MMF_F16: if (log_gates) MMF_RB(f16_t, true); else MMF_RB(f16_t, false); break;
        default: return MMF_ERR_ARG;
    }
#undef MMF_RB
    MMF_CHECK_LAUNCH();
    return 0;
}

int mmf_cross_entropy_train_fwd(const void* logits, int64_t ld, const int64_t* labels, int64_t ignore_index, float smoothing,
                                float logit_scale, float lse_square_scale, float* loss, float* lse, float* z_loss, int64_t rows,
                                int64_t V, int dtype, void* stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (rows < 0 || V <= 0 || ld < V || rows > 0x7fffffff || smoothing < 0.0f || smoothing > 1.0f) return MMF_ERR_ARG;
    if (rows == 0) return 0;
    if (!logits || !labels || !loss || !lse) return MMF_ERR_ARG;
#define MMF_CF(T) ce_train_fwd_kernel<T><<<(unsigned)rows, 512, 0, stream>>>(static_cast<const T*>(logits), ld, V, labels, ignore_index, \
        smoothing, logit_scale, lse_square_scale, loss, lse, z_loss)
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

int mmf_cross_entropy_train_bwd(const void* logits, int64_t ld, const int64_t* labels, int64_t ignore_index, const float* lse,
                                const float* dloss, float smoothing, float logit_scale, float lse_square_scale, void* dlogits,
                                int64_t ldd, int64_t rows, int64_t V, int dtype, void* stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (rows < 0 || V <= 0 || ld < V || ldd < V) return MMF_ERR_ARG;
    if (rows == 0) return 0;
    if (!logits || !labels || !lse || !dloss || !dlogits) return MMF_ERR_ARG;
    if (dtype != MMF_F32 && dtype != MMF_BF16 && dtype != MMF_F16) return MMF_ERR_ARG;
    const int64_t esz = dtype == MMF_F32 ? 4 : 2;
    for (int64_t r0 = 0; r0 < rows; r0 += 65535) {                // rows ride on grid.y
        const int64_t nr = rows - r0 < 65535 ? rows - r0 : 65535;
        dim3 grid((unsigned)mmf_ceil_div(V, 256 * 8), (unsigned)nr);
        const char* lg = static_cast<const char*>(logits) + r0 * ld * esz;
        char* dl = static_cast<char*>(dlogits) + r0 * ldd * esz;
#define MMF_CB(T) ce_train_bwd_kernel<T><<<grid, 256, 0, stream>>>(reinterpret_cast<const T*>(lg), ld, V, labels + r0, ignore_index, lse + r0, \
        dloss + r0, smoothing, logit_scale, lse_square_scale, reinterpret_cast<T*>(dl), ldd)
        switch (dtype) {
            case MMF_F32: MMF_CB(float); break;
            case MMF_BF16: MMF_CB(bf16_t); break;
            case MMF_F16: MMF_CB(f16_t); break;
        }
#undef MMF_CB
        MMF_CHECK_LAUNCH();
    }
    return 0;
}

}  // extern "C"
