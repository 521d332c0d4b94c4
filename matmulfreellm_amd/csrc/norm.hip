// One-pass row kernels: RMSNorm, RMSNorm * swish-gate, RMSNorm + int8 quantiser, swiglu.
//
// One workgroup of 256 threads owns one row; the row lives in registers (8-element
// vectors, up to NV per thread), sums of squares are reduced in fp64 with a wave64
// butterfly plus a 4-entry LDS exchange, so HBM sees each input once and each output
// once.  Replaces the Triton row kernels at mmfreelm/modules/layernorm.py:104-165,
// mmfreelm/modules/fused_norm_gate.py:68-131, mmfreelm/ops/fusedbitnet.py:63-131 and
// the jiterator kernel at mmfreelm/modules/activations.py:115-119.
#include "mmf_common.h"
#include "../../include/mmf.h"

namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / 64;

enum RowMode : int { ROW_NORM = 0, ROW_GATE = 1, ROW_QUANT = 2 };

struct RowArgs {
    const void* x;          // [M, K]
    const void* residual;   // [M, K] or null            (dtype TR)
    const void* gate;       // [M, K] or null            (ROW_GATE, dtype T)
    const void* weight;     // [K] or null               (dtype TW)
    const void* bias;       // [K] or null: added after the weight (dtype TW)
    int center;             // LayerNorm: subtract the row mean before the variance (else RMSNorm)
    void* y;                // [M, K] T                  (ROW_NORM / ROW_GATE)
    void* residual_out;     // [M, K] TR or null
    int8_t* q;              // codes                     (ROW_QUANT)
    float* deq;             // [M]
    int* qsum;              // [M]
    int64_t M, K, Kp, ldx;   // ldx: row stride of x in elements
    double inv_K;            // RN(1 / K)
    float eps;
    int q_tiled;            // 0: row-major [M, Kp]; 1: [ceil32(M)/32][Kp/16][32][16]
};

template <typename T, typename TR, typename TW, int MODE, int NV>
__global__ __launch_bounds__(kThreads) void row_kernel(RowArgs a) {
    __shared__ double red_d[kWaves];
    __shared__ float red_f[kWaves];
    __shared__ int red_i[kWaves];

    const int64_t row = blockIdx.x;
    const int64_t K = a.K;
    const bool vec_ok = (K % 8) == 0;
    const T* x = static_cast<const T*>(a.x) + row * a.ldx;
    const TR* res = a.residual ? static_cast<const TR*>(a.residual) + row * K : nullptr;
    TR* res_out = a.residual_out ? static_cast<TR*>(a.residual_out) + row * K : nullptr;
    const TW* w = static_cast<const TW*>(a.weight);

    // Every global load of the row is issued up front (x, residual, norm weight, gate) so
    // their latencies overlap; the reductions below then run on registers only.
    float xv[NV][8];
    float wv[NV][8];
    float ov[MODE == ROW_GATE ? NV : 1][8];
    double ss = 0.0;
#pragma unroll
    for (int v = 0; v < NV; ++v) {
        const int64_t k0 = ((int64_t)v * kThreads + threadIdx.x) * 8;
        if (k0 < K) {
            if (w) mmf_load8<TW>(w, k0, K, vec_ok, wv[v]);
            if constexpr (MODE == ROW_GATE)
                mmf_load8<T>(static_cast<const T*>(a.gate) + row * K, k0, K, vec_ok, ov[v]);
        }
    }
#pragma unroll
    for (int v = 0; v < NV; ++v) {
        const int64_t k0 = ((int64_t)v * kThreads + threadIdx.x) * 8;
        if (k0 < K) {
            mmf_load8<T>(x, k0, K, vec_ok, xv[v]);
            if (res) {
                float rv[8];
                mmf_load8<TR>(res, k0, K, vec_ok, rv);
#pragma unroll
                for (int i = 0; i < 8; ++i) xv[v][i] = __fadd_rn(xv[v][i], rv[i]);
            }
            if (res_out) mmf_store8<TR>(res_out, k0, K, vec_ok, xv[v]);
#pragma unroll
            for (int i = 0; i < 8; ++i) ss = mmf_add_square(ss, xv[v][i]);
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i) xv[v][i] = 0.0f;
        }
    }
    if (a.center) {
        // LayerNorm: mean = fp32(sum / K) with the sum in fp64; the variance is that of the fp32 differences
        double sx = 0.0;
#pragma unroll
        for (int v = 0; v < NV; ++v)
#pragma unroll
            for (int i = 0; i < 8; ++i) sx += (double)xv[v][i];
        sx = mmf_block_sum<kWaves>(sx, red_d);
        const float mean = (float)mmf_quotient_by_count(sx, K, a.inv_K);
        ss = 0.0;
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            const int64_t k0 = ((int64_t)v * kThreads + threadIdx.x) * 8;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                xv[v][i] = k0 + i < K ? __fsub_rn(xv[v][i], mean) : 0.0f;
                ss = mmf_add_square(ss, xv[v][i]);
            }
        }
    }
    ss = mmf_block_sum<kWaves>(ss, red_d);
    const float rstd = mmf_rstd(ss, K, a.inv_K, a.eps);

    float amax = 0.0f;
#pragma unroll
    for (int v = 0; v < NV; ++v) {
        const int64_t k0 = ((int64_t)v * kThreads + threadIdx.x) * 8;
        if (k0 < K) {
            float bv[8];
            if (a.bias) mmf_load8<TW>(static_cast<const TW*>(a.bias), k0, K, vec_ok, bv);
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                float y = __fmul_rn(xv[v][i], rstd);
                if (w) y = __fmul_rn(y, wv[v][i]);
                if (a.bias) y = k0 + i < K ? __fadd_rn(y, bv[i]) : 0.0f;
                xv[v][i] = y;
                amax = fmaxf(amax, fabsf(y));
            }
            if constexpr (MODE == ROW_GATE) {
                float sg[8];
                mmf_sigmoid_n<8>(ov[v], sg);
#pragma unroll
                for (int i = 0; i < 8; ++i) xv[v][i] = __fmul_rn(__fmul_rn(xv[v][i], ov[v][i]), sg[i]);
            }
            if constexpr (MODE != ROW_QUANT)
                mmf_store8<T>(static_cast<T*>(a.y) + row * K, k0, K, vec_ok, xv[v]);
        }
    }
    if constexpr (MODE != ROW_QUANT) return;

    amax = mmf_block_max<kWaves>(amax, red_f);
    const float amaxc = fmaxf(amax, 1e-5f);
    const float scale = mmf_127_over(amaxc);
    int qs = 0;
    const int64_t Kp = a.Kp;
#pragma unroll
    for (int v = 0; v < NV; ++v) {
        const int64_t k0 = ((int64_t)v * kThreads + threadIdx.x) * 8;
        if (k0 < Kp) {
            uint32_t lo = 0, hi = 0;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                int c = (k0 + i < K) ? mmf_code(xv[v][i], scale) : 0;   // xv is 0 beyond K
                qs += c;
                uint32_t b = (uint32_t)(c & 0xff) << (8 * (i & 3));
                if (i < 4) lo |= b; else hi |= b;
            }
            int64_t off;
            if (a.q_tiled)
                off = ((row >> 5) * (Kp >> 4) + (k0 >> 4)) * 512 + (row & 31) * 16 + (k0 & 15);
            else
                off = row * Kp + k0;
            *reinterpret_cast<uint2*>(a.q + off) = make_uint2(lo, hi);
        }
    }
    qs = mmf_block_sum<kWaves>(qs, red_i);
    if (threadIdx.x == 0) {
        a.deq[row] = mmf_rcp_pos(scale);
        a.qsum[row] = qs;
    }
}

template <typename T, typename TR, typename TW, int MODE>
int launch_row(const RowArgs& a, hipStream_t s) {
    if (a.M == 0) return 0;
    const int64_t width = (MODE == ROW_QUANT) ? a.Kp : a.K;   // the quantiser also zero-fills the padding
    const int64_t nv = mmf_ceil_div(width, (int64_t)kThreads * 8);
    dim3 grid((unsigned)a.M), block(kThreads);
    if (nv <= 1) row_kernel<T, TR, TW, MODE, 1><<<grid, block, 0, s>>>(a);
    else if (nv <= 2) row_kernel<T, TR, TW, MODE, 2><<<grid, block, 0, s>>>(a);
    else if (nv <= 4) row_kernel<T, TR, TW, MODE, 4><<<grid, block, 0, s>>>(a);
    else if (nv <= 8) row_kernel<T, TR, TW, MODE, 8><<<grid, block, 0, s>>>(a);
    else return MMF_ERR_WIDE;
    MMF_CHECK_LAUNCH();
    return 0;
}

template <typename T, typename TR, int MODE>
int dispatch_w(const RowArgs& a, int x_dtype, int w_dtype, hipStream_t s) {
    // The norm weight is either fp32 or the activation dtype.
    if (w_dtype == MMF_F32) return launch_row<T, TR, float, MODE>(a, s);
    if (w_dtype == x_dtype) return launch_row<T, TR, T, MODE>(a, s);
    return MMF_ERR_ARG;
}

template <typename T, int MODE>
int dispatch_r(const RowArgs& a, int x_dtype, int r_dtype, int w_dtype, hipStream_t s) {
    // The residual stream is either the activation dtype or fp32 (residual_in_fp32).
    if (r_dtype == MMF_F32) return dispatch_w<T, float, MODE>(a, x_dtype, w_dtype, s);
    return dispatch_w<T, T, MODE>(a, x_dtype, w_dtype, s);
}

template <int MODE>
int dispatch_x(const RowArgs& a, int x_dtype, int r_dtype, int w_dtype, hipStream_t s) {
    const bool uses_res = a.residual || a.residual_out;
    if (uses_res && r_dtype != MMF_F32 && r_dtype != x_dtype) return MMF_ERR_ARG;
    if (!uses_res) r_dtype = x_dtype;
    if (!a.weight) w_dtype = MMF_F32;
    switch (x_dtype) {
        case MMF_F32: return dispatch_r<float, MODE>(a, x_dtype, r_dtype, w_dtype, s);
        case MMF_BF16: return dispatch_r<bf16_t, MODE>(a, x_dtype, r_dtype, w_dtype, s);
        case MMF_F16: return dispatch_r<f16_t, MODE>(a, x_dtype, r_dtype, w_dtype, s);
    }
    return MMF_ERR_ARG;
}

// ---------------------------------------------------------------- fused prologue + quantiser
// The int8 quantiser with the elementwise op that precedes each BitLinear of a decode step
// folded in (batch sizes that go to the matrix cores, where the codes must exist in memory):
//   QPRO_PLAIN      v = x                                                  (nothing in front: many-row form of ROW_QUANT)
//   QPRO_NORM       v = T(RMSNorm(x; w1, eps1))                            (block norm)
//   QPRO_RESNORM    s = x + aux; res_out = s; v = T(RMSNorm(s; w1, eps1))  (fused residual norm)
//   QPRO_STEP_GATE  i = x, f = aux, g = aux2 (raw projections of one token): gate math, one recurrence
//                   step on the fp32 state (in place), o = T(h); v = T(RMSNorm(g; w1, eps1) * o * sigmoid(o))
//   QPRO_SWIGLU     v = T((x * aux) / (1 + exp(-x)))                       (MLP activation)
//   QPRO_GATEDNORM  v = T(RMSNorm(x; w1, eps1) * aux * sigmoid(aux))       (g_norm in front of o_proj, any T)
// then  y = RMSNorm(v; norm_w, eps),  q = int8 absmax codes of y  (tiled operand layout).
enum QPro : int { QPRO_PLAIN = 0, QPRO_NORM = 1, QPRO_RESNORM = 2, QPRO_STEP_GATE = 3, QPRO_SWIGLU = 4, QPRO_GATEDNORM = 5 };

struct FusedQuantArgs {
    const void* x; const void* aux; const void* aux2;
    int64_t ldx, ldaux, ldaux2;
    void* res_out;
    const void* w1; const void* norm_w;
    const float* lb; float* state;
    int8_t* q; float* deq; int* qsum;
    int64_t M, K, Kp;
    double inv_K;            // RN(1 / K)
    float eps1, eps;
};

constexpr int kQWaves = 8, kQThreads = kQWaves * 64;

// RPW rows per workgroup, 512 / RPW threads per row, NV passes of (512 / RPW) * 4 elements.
//   RPW = 1 : a decode batch has few rows and each launch is a step of a dependent chain, so all
//             8 waves share one row (shortest latency);
//   RPW = 8 : prefill has thousands of rows and the kernel should stream: one wave per row, whose
//             reductions are DPP folds only - no LDS exchange and no barrier anywhere.
// VEC: K, the strides and every pointer allow 4-element accesses.
template <typename T, typename TW, int NV, int PRO, bool VEC, int RPW>
__global__ __launch_bounds__(kQThreads) void row_quant_fused_kernel(FusedQuantArgs a) {
    constexpr int TPR = kQThreads / RPW, WPR = TPR / 64;        // threads / waves per row
    __shared__ double red_a[kQWaves], red_b[kQWaves];
    __shared__ float red_f[kQWaves];
    __shared__ int red_i[kQWaves];
    constexpr bool HAS_AUX = PRO >= QPRO_RESNORM, STEP = PRO == QPRO_STEP_GATE, HAS_W1 = PRO != QPRO_SWIGLU && PRO != QPRO_PLAIN;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int w0 = (wave / WPR) * WPR;                          // first wave of this row
    const int tr = (int)threadIdx.x % TPR;                      // thread within the row
    const int64_t row_raw = (int64_t)blockIdx.x * RPW + (int)threadIdx.x / TPR;
    const bool live = row_raw < a.M;                            // rows past M compute on row M-1 and store nothing
    const int64_t row = live ? row_raw : a.M - 1;
    const int K = (int)a.K, Kp = (int)a.Kp;
    // element k0 + i of the row exists; with vector accesses (K a multiple of 4) a thread's 4 elements stand or fall together
    auto inb = [&](int k0, int i) { return VEC ? k0 < K : k0 + i < K; };
    const T* x = static_cast<const T*>(a.x) + row * a.ldx;
    const T* aux = static_cast<const T*>(a.aux) + row * a.ldaux;
    const T* aux2 = static_cast<const T*>(a.aux2) + row * a.ldaux2;
    const TW* w1 = static_cast<const TW*>(a.w1);
    const TW* nw = static_cast<const TW*>(a.norm_w);
    float* st = a.state + row * K;

    // every load of the kernel first, raw; conversions only after the last one is issued
    Raw4<T> xraw[NV], araw[HAS_AUX ? NV : 1], graw[STEP ? NV : 1];
    Raw4<float> straw[STEP ? NV : 1], lbraw[STEP ? NV : 1];
    Raw4<TW> w1raw[HAS_W1 ? NV : 1], nwraw[NV];
#pragma unroll
    for (int v = 0; v < NV; ++v) {
        const int k0 = (v * TPR + tr) * 4;
        xraw[v] = raw4_load<T, VEC>(x, k0, K);
        if constexpr (HAS_AUX) araw[v] = raw4_load<T, VEC>(aux, k0, K);
        if constexpr (STEP) {
            graw[v] = raw4_load<T, VEC>(aux2, k0, K);
            straw[v] = raw4_load<float, VEC>(st, k0, K);
            if (a.lb) lbraw[v] = raw4_load<float, VEC>(a.lb, k0, K);
        }
        if constexpr (HAS_W1) w1raw[v] = raw4_load<TW, VEC>(w1, k0, K);
        if (nw) nwraw[v] = raw4_load<TW, VEC>(nw, k0, K);
    }
    float xv[NV][4], av[HAS_AUX ? NV : 1][4];
#pragma unroll
    for (int v = 0; v < NV; ++v) {
        const int k0 = (v * TPR + tr) * 4;
        raw4_unpack<T>(xraw[v], xv[v]);
        if constexpr (HAS_AUX) raw4_unpack<T>(araw[v], av[v]);
#pragma unroll
        for (int i = 0; i < 4; ++i)
            if (!inb(k0, i)) xv[v][i] = 0.0f;
    }
    if constexpr (PRO == QPRO_RESNORM) {
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            const int k0 = (v * TPR + tr) * 4;
#pragma unroll
            for (int i = 0; i < 4; ++i) xv[v][i] = inb(k0, i) ? __fadd_rn(xv[v][i], av[v][i]) : 0.0f;
            if (a.res_out && live) raw4_store<T, VEC>(static_cast<T*>(a.res_out) + row * K, k0, K, xv[v]);
        }
    }
    if constexpr (STEP) {
        // gate math + one recurrence step per channel; xv becomes the raw g projection, av the new o
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            const int k0 = (v * TPR + tr) * 4;
            float gv[4], stv[4], lbv[4];
            raw4_unpack<T>(graw[v], gv);
            raw4_unpack<float>(straw[v], stv);
            if (a.lb) raw4_unpack<float>(lbraw[v], lbv);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float iv = xv[v][i], fv = av[v][i];
                float s = mmf_sigmoid(fv);
                if (a.lb) s = __fadd_rn(lbv[i], __fmul_rn(__fsub_rn(1.0f, lbv[i]), s));
                const float go = mmf_round_to<T>(s);
                const float xo = mmf_round_to<T>(__fdiv_rn(__fmul_rn(iv, __fsub_rn(1.0f, go)), __fadd_rn(1.0f, mmf_exp(-iv))));
                const float h = __fadd_rn(__fmul_rn(go, stv[i]), xo);
                stv[i] = h;
                av[v][i] = mmf_round_to<T>(h);          // o, the swish gate of the gated norm
                xv[v][i] = inb(k0, i) ? gv[i] : 0.0f;   // the gated norm normalises the g projection
            }
            if (live) raw4_store<float, VEC>(st, k0, K, stv);
        }
    }
    if constexpr (HAS_W1) {
        double s1 = 0.0;
#pragma unroll
        for (int v = 0; v < NV; ++v)
#pragma unroll
            for (int i = 0; i < 4; ++i) s1 = mmf_add_square(s1, xv[v][i]);
        s1 = mmf_wave_sum(s1);
        if constexpr (WPR > 1) {
            if ((threadIdx.x & 63) == 0) red_a[wave] = s1;
            __syncthreads();
            s1 = red_a[w0];
#pragma unroll
            for (int w = 1; w < WPR; ++w) s1 += red_a[w0 + w];
        }
        const float rstd1 = mmf_rstd(s1, K, a.inv_K, a.eps1);
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            const int k0 = (v * TPR + tr) * 4;
            float w1v[4], sg[4] = {0.0f, 0.0f, 0.0f, 0.0f};
            raw4_unpack<TW>(w1raw[v], w1v);
            if constexpr (STEP || PRO == QPRO_GATEDNORM) mmf_sigmoid_n<4>(av[v], sg);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                float y = __fmul_rn(__fmul_rn(xv[v][i], rstd1), w1v[i]);
                if constexpr (STEP || PRO == QPRO_GATEDNORM) y = __fmul_rn(__fmul_rn(y, av[v][i]), sg[i]);
                xv[v][i] = inb(k0, i) ? mmf_round_to<T>(y) : 0.0f;
            }
        }
    } else if constexpr (PRO == QPRO_SWIGLU) {
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            const int k0 = (v * TPR + tr) * 4;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float g = xv[v][i];
                const float z = __fdiv_rn(__fmul_rn(g, av[v][i]), __fadd_rn(1.0f, mmf_exp(-g)));
                xv[v][i] = inb(k0, i) ? mmf_round_to<T>(z) : 0.0f;
            }
        }
    }
    // BitLinear's own norm + absmax codes
    double ss = 0.0;
#pragma unroll
    for (int v = 0; v < NV; ++v)
#pragma unroll
        for (int i = 0; i < 4; ++i) ss = mmf_add_square(ss, xv[v][i]);
    ss = mmf_wave_sum(ss);
    if constexpr (WPR > 1) {
        if ((threadIdx.x & 63) == 0) red_b[wave] = ss;
        __syncthreads();
        ss = red_b[w0];
#pragma unroll
        for (int w = 1; w < WPR; ++w) ss += red_b[w0 + w];
    }
    const float rstd = mmf_rstd(ss, K, a.inv_K, a.eps);
    float amax = 0.0f;
#pragma unroll
    for (int v = 0; v < NV; ++v) {
        float wv[4];
        if (nw) raw4_unpack<TW>(nwraw[v], wv);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            float y = __fmul_rn(xv[v][i], rstd);
            if (nw) y = __fmul_rn(y, wv[i]);
            xv[v][i] = y;                                       // elements past K are exact zeros and stay so
            amax = fmaxf(amax, fabsf(y));
        }
    }
    amax = mmf_wave_max(amax);
    if constexpr (WPR > 1) {
        if ((threadIdx.x & 63) == 0) red_f[wave] = amax;
        __syncthreads();
        amax = red_f[w0];
#pragma unroll
        for (int w = 1; w < WPR; ++w) amax = fmaxf(amax, red_f[w0 + w]);
    }
    const float scale = mmf_127_over(fmaxf(amax, 1e-5f));
    int qs = 0;
#pragma unroll
    for (int v = 0; v < NV; ++v) {
        const int k0 = (v * TPR + tr) * 4;
        if (k0 < Kp) {
            uint32_t packed4 = 0;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int c = inb(k0, i) ? mmf_code(xv[v][i], scale) : 0;
                qs += c;
                packed4 |= (uint32_t)(c & 0xff) << (8 * i);
            }
            const int64_t off = ((row >> 5) * (Kp >> 4) + (k0 >> 4)) * 512 + (row & 31) * 16 + (k0 & 15);
            if (live) *reinterpret_cast<uint32_t*>(a.q + off) = packed4;
        }
    }
    qs = mmf_wave_sum(qs);
    if constexpr (WPR > 1) {
        if ((threadIdx.x & 63) == 0) red_i[wave] = qs;
        __syncthreads();
        qs = 0;
#pragma unroll
        for (int w = 0; w < WPR; ++w) qs += red_i[w0 + w];
    }
    if (tr == 0 && live) {
        a.deq[row] = mmf_rcp_pos(scale);
        a.qsum[row] = qs;
    }
}

template <typename T, typename TW, int PRO, int RPW>
int launch_fused_quant_rpw(const FusedQuantArgs& a, hipStream_t s) {
    constexpr int TPR = kQThreads / RPW;
    const int64_t nv = mmf_ceil_div(a.Kp, (int64_t)TPR * 4);
    dim3 grid((unsigned)mmf_ceil_div(a.M, (int64_t)RPW)), block(kQThreads);
    if (nv <= 1) row_quant_fused_kernel<T, TW, 1, PRO, true, RPW><<<grid, block, 0, s>>>(a);
    else if (nv <= 2) row_quant_fused_kernel<T, TW, 2, PRO, true, RPW><<<grid, block, 0, s>>>(a);
    else if (nv <= 3) row_quant_fused_kernel<T, TW, 3, PRO, true, RPW><<<grid, block, 0, s>>>(a);
    else if (nv <= 4) row_quant_fused_kernel<T, TW, 4, PRO, true, RPW><<<grid, block, 0, s>>>(a);
    else if (nv <= 6) row_quant_fused_kernel<T, TW, 6, PRO, true, RPW><<<grid, block, 0, s>>>(a);
    else if (nv <= 8) row_quant_fused_kernel<T, TW, 8, PRO, true, RPW><<<grid, block, 0, s>>>(a);
    else if constexpr (PRO == QPRO_PLAIN && RPW == 4) {
        if (nv > 12) return MMF_ERR_WIDE;
        row_quant_fused_kernel<T, TW, 12, PRO, true, RPW><<<grid, block, 0, s>>>(a);
    } else return MMF_ERR_WIDE;
    MMF_CHECK_LAUNCH();
    return 0;
}

template <typename T, typename TW, int PRO>
int launch_fused_quant(const FusedQuantArgs& a, bool vec, hipStream_t s) {
    if (mmf_ceil_div(a.Kp, (int64_t)kQThreads * 4) > 8) return MMF_ERR_WIDE;
    if (!vec) {                                                 // ragged rows: one generic build
        row_quant_fused_kernel<T, TW, 8, PRO, false, 1><<<dim3((unsigned)a.M), dim3(kQThreads), 0, s>>>(a);
        MMF_CHECK_LAUNCH();
        return 0;
    }
    // decode: latency (the recurrence-step prologue only exists there: one token per row)
    if (a.M <= 256 || PRO == QPRO_STEP_GATE) return launch_fused_quant_rpw<T, TW, PRO, 1>(a, s);
    // prefill: as many rows per workgroup as 8 passes of 4 elements per thread allow
    if constexpr (PRO != QPRO_STEP_GATE) {
        if (a.Kp <= 64 * 4 * 8) return launch_fused_quant_rpw<T, TW, PRO, 8>(a, s);
        if (a.Kp <= 128 * 4 * 8) return launch_fused_quant_rpw<T, TW, PRO, 4>(a, s);
        // the 5632- and 6912-wide rows in front of down_proj (nothing folded in: few registers per element): two waves
        // per row and 12 passes measured 12 % faster than four waves and 6
        if constexpr (PRO == QPRO_PLAIN) {
            if (a.Kp <= 128 * 4 * 12) return launch_fused_quant_rpw<T, TW, PRO, 4>(a, s);
        }
        if (a.Kp <= 256 * 4 * 8) return launch_fused_quant_rpw<T, TW, PRO, 2>(a, s);
    }
    return launch_fused_quant_rpw<T, TW, PRO, 1>(a, s);
}

template <typename T, typename TW>
int dispatch_fused_quant(const FusedQuantArgs& a, int pro, bool vec, hipStream_t s) {
    switch (pro) {
        case QPRO_PLAIN: return launch_fused_quant<T, TW, QPRO_PLAIN>(a, vec, s);
        case QPRO_NORM: return launch_fused_quant<T, TW, QPRO_NORM>(a, vec, s);
        case QPRO_RESNORM: return launch_fused_quant<T, TW, QPRO_RESNORM>(a, vec, s);
        case QPRO_STEP_GATE: return launch_fused_quant<T, TW, QPRO_STEP_GATE>(a, vec, s);
        case QPRO_SWIGLU: return launch_fused_quant<T, TW, QPRO_SWIGLU>(a, vec, s);
        case QPRO_GATEDNORM: return launch_fused_quant<T, TW, QPRO_GATEDNORM>(a, vec, s);
    }
    return MMF_ERR_ARG;
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// ---------------------------------------------------------------- swiglu (elementwise)
template <typename T>
__global__ __launch_bounds__(256) void swiglu_kernel(const T* __restrict__ x, int64_t ldx, const T* __restrict__ y,
                                                     int64_t ldy, T* __restrict__ out, int64_t rows, int64_t cols) {
    // cols % 8 == 0; one 8-vector per thread.
    const int64_t vpr = cols / 8;
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= rows * vpr) return;
    const int64_t r = idx / vpr, c0 = (idx % vpr) * 8;
    float xv[8], yv[8];
    mmf_load8<T>(x + r * ldx, c0, cols, true, xv);
    mmf_load8<T>(y + r * ldy, c0, cols, true, yv);
#pragma unroll
    for (int i = 0; i < 8; ++i)
        xv[i] = __fdiv_rn(__fmul_rn(xv[i], yv[i]), __fadd_rn(1.0f, mmf_exp(-xv[i])));
    mmf_store8<T>(out + r * cols, c0, cols, true, xv);
}

template <typename T>
__global__ __launch_bounds__(256) void swiglu_scalar_kernel(const T* __restrict__ x, int64_t ldx, const T* __restrict__ y,
                                                            int64_t ldy, T* __restrict__ out, int64_t rows, int64_t cols) {
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= rows * cols) return;
    const int64_t r = idx / cols, c = idx % cols;
    const float xv = mmf_to_float(x[r * ldx + c]), yv = mmf_to_float(y[r * ldy + c]);
    out[r * cols + c] = mmf_from_float<T>(__fdiv_rn(__fmul_rn(xv, yv), __fadd_rn(1.0f, mmf_exp(-xv))));
}

template <typename T>
int launch_swiglu(const void* x, int64_t ldx, const void* y, int64_t ldy, void* out, int64_t rows, int64_t cols,
                  hipStream_t s) {
    if (rows == 0 || cols == 0) return 0;
    const int esz = sizeof(T);
    const bool vec = cols % 8 == 0 && ldx % 8 == 0 && ldy % 8 == 0 && aligned16(x) && aligned16(y) && aligned16(out);
    (void)esz;
    if (vec) {
        const int64_t n = rows * (cols / 8);
        swiglu_kernel<T><<<(unsigned)mmf_ceil_div(n, 256), 256, 0, s>>>(static_cast<const T*>(x), ldx,
                                                                       static_cast<const T*>(y), ldy,
                                                                       static_cast<T*>(out), rows, cols);
    } else {
        const int64_t n = rows * cols;
        swiglu_scalar_kernel<T><<<(unsigned)mmf_ceil_div(n, 256), 256, 0, s>>>(static_cast<const T*>(x), ldx,
                                                                              static_cast<const T*>(y), ldy,
                                                                              static_cast<T*>(out), rows, cols);
    }
    MMF_CHECK_LAUNCH();
    return 0;
}

}  // namespace

extern "C" {

int mmf_rmsnorm(const void* x, const void* residual, const void* weight, void* y, void* residual_out, int64_t M,
                int64_t K, float eps, int x_dtype, int residual_dtype, int weight_dtype, void* stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (M < 0 || K <= 0 || (M > 0 && (!x || !y))) return MMF_ERR_ARG;
    if (K % 8 == 0 && !(aligned16(x) && aligned16(y) && aligned16(residual) && aligned16(residual_out) && aligned16(weight)))
        return MMF_ERR_ALIGN;
    RowArgs a{};
    a.x = x; a.residual = residual; a.weight = weight; a.y = y; a.residual_out = residual_out;
    a.M = M; a.K = K; a.inv_K = 1.0 / (double)K; a.Kp = K; a.ldx = K; a.eps = eps;
    return dispatch_x<ROW_NORM>(a, x_dtype, residual_dtype, weight_dtype, stream);
}

int mmf_rmsnorm_swishgate(const void* x, int64_t ldx, const void* gate, const void* residual, const void* weight, void* y,
                          void* residual_out, int64_t M, int64_t K, float eps, int x_dtype, int residual_dtype,
                          int weight_dtype, void* stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (M < 0 || K <= 0 || ldx < K || (M > 0 && (!x || !y || !gate))) return MMF_ERR_ARG;
    if (K % 8 == 0 && ldx % 8 != 0) return MMF_ERR_ALIGN;
    if (K % 8 == 0 && !(aligned16(x) && aligned16(y) && aligned16(gate) && aligned16(residual) &&
                        aligned16(residual_out) && aligned16(weight)))
        return MMF_ERR_ALIGN;
    RowArgs a{};
    a.x = x; a.gate = gate; a.residual = residual; a.weight = weight; a.y = y; a.residual_out = residual_out;
    a.M = M; a.K = K; a.inv_K = 1.0 / (double)K; a.Kp = K; a.ldx = ldx; a.eps = eps;
    return dispatch_x<ROW_GATE>(a, x_dtype, residual_dtype, weight_dtype, stream);
}

int64_t mmf_codes_bytes(int64_t M, int64_t K, int tiled) {
    const int64_t Kp = mmf_round_up(K, 128);
    return (tiled ? mmf_round_up(M, 32) : M) * Kp;
}

int mmf_rmsnorm_quant(const void* x, const void* residual, const void* weight, int8_t* q, float* deq, int* qsum,
                      void* residual_out, int64_t M, int64_t K, float eps, int x_dtype, int residual_dtype,
                      int weight_dtype, int tiled, void* stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (M < 0 || K <= 0 || (M > 0 && (!x || !q || !deq || !qsum))) return MMF_ERR_ARG;
    if (!aligned16(q)) return MMF_ERR_ALIGN;
    if (K % 8 == 0 && !(aligned16(x) && aligned16(residual) && aligned16(residual_out) && aligned16(weight)))
        return MMF_ERR_ALIGN;
    RowArgs a{};
    a.x = x; a.residual = residual; a.weight = weight; a.residual_out = residual_out;
    a.q = q; a.deq = deq; a.qsum = qsum;
    a.M = M; a.K = K; a.inv_K = 1.0 / (double)K; a.Kp = mmf_round_up(K, 128); a.ldx = K; a.eps = eps; a.q_tiled = tiled;
    return dispatch_x<ROW_QUANT>(a, x_dtype, residual_dtype, weight_dtype, stream);
}

int mmf_layernorm_quant(const void* x, const void* residual, const void* weight, const void* bias, int8_t* q, float* deq,
                        int* qsum, void* residual_out, int64_t M, int64_t K, float eps, int x_dtype, int residual_dtype,
                        int weight_dtype, int tiled, void* stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (M < 0 || K <= 0 || (M > 0 && (!x || !q || !deq || !qsum))) return MMF_ERR_ARG;
    if (bias && !weight) return MMF_ERR_ARG;                     // the bias shares the weight's dtype
    if (!aligned16(q)) return MMF_ERR_ALIGN;
    if (K % 8 == 0 && !(aligned16(x) && aligned16(residual) && aligned16(residual_out) && aligned16(weight) && aligned16(bias)))
        return MMF_ERR_ALIGN;
    RowArgs a{};
    a.x = x; a.residual = residual; a.weight = weight; a.bias = bias; a.center = 1; a.residual_out = residual_out;
    a.q = q; a.deq = deq; a.qsum = qsum;
    a.M = M; a.K = K; a.inv_K = 1.0 / (double)K; a.Kp = mmf_round_up(K, 128); a.ldx = K; a.eps = eps; a.q_tiled = tiled;
    return dispatch_x<ROW_QUANT>(a, x_dtype, residual_dtype, weight_dtype, stream);
}

int mmf_rmsnorm_quant_fused(int prologue, const void* x, int64_t ldx, const void* aux, int64_t ldaux, const void* aux2,
                            int64_t ldaux2, void* res_out, const void* w1, float eps1, const void* norm_weight, float eps,
                            const float* lower_bound, float* state, int8_t* q, float* deq, int* qsum, int64_t M, int64_t K,
                            int x_dtype, int weight_dtype, void* stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (M < 0 || K <= 0 || ldx < K) return MMF_ERR_ARG;
    if (M == 0) return 0;
    if (!x || !q || !deq || !qsum) return MMF_ERR_ARG;
    if (prologue < QPRO_PLAIN || prologue > QPRO_GATEDNORM) return MMF_ERR_ARG;
    if (prologue >= QPRO_RESNORM && (!aux || ldaux < K)) return MMF_ERR_ARG;
    if (prologue == QPRO_STEP_GATE && (!aux2 || ldaux2 < K || !state)) return MMF_ERR_ARG;
    if (prologue != QPRO_SWIGLU && prologue != QPRO_PLAIN && !w1) return MMF_ERR_ARG;
    FusedQuantArgs a{};
    a.x = x; a.aux = aux ? aux : x; a.aux2 = aux2 ? aux2 : x; a.ldx = ldx; a.ldaux = aux ? ldaux : ldx;
    a.ldaux2 = aux2 ? ldaux2 : ldx; a.res_out = res_out; a.w1 = w1; a.norm_w = norm_weight; a.lb = lower_bound; a.state = state;
    a.q = q; a.deq = deq; a.qsum = qsum; a.M = M; a.K = K; a.inv_K = 1.0 / (double)K; a.Kp = mmf_round_up(K, 128); a.eps1 = eps1; a.eps = eps;
    if (!aligned16(q)) return MMF_ERR_ALIGN;
    if (!norm_weight && !w1) weight_dtype = MMF_F32;
    const uintptr_t xa = 4 * (x_dtype == MMF_F32 ? 4 : 2), wa = 4 * (weight_dtype == MMF_F32 ? 4 : 2);
    auto al = [](const void* ptr, uintptr_t n) { return (reinterpret_cast<uintptr_t>(ptr) % n) == 0; };
    const bool vec = K % 4 == 0 && ldx % 4 == 0 && a.ldaux % 4 == 0 && a.ldaux2 % 4 == 0;
    if (vec && !(al(x, xa) && al(a.aux, xa) && al(a.aux2, xa) && al(res_out, xa) && al(w1, wa) && al(norm_weight, wa) &&
                 al(lower_bound, 16) && al(state, 16)))
        return MMF_ERR_ALIGN;
    const bool wf32 = weight_dtype == MMF_F32;
    if (!wf32 && weight_dtype != x_dtype) return MMF_ERR_ARG;
    switch (x_dtype) {
        case MMF_F32: return dispatch_fused_quant<float, float>(a, prologue, vec, stream);
        case MMF_BF16: return wf32 ? dispatch_fused_quant<bf16_t, float>(a, prologue, vec, stream)
                                   : dispatch_fused_quant<bf16_t, bf16_t>(a, prologue, vec, stream);
        case MMF_F16: return wf32 ? dispatch_fused_quant<f16_t, float>(a, prologue, vec, stream)
                                  : dispatch_fused_quant<f16_t, f16_t>(a, prologue, vec, stream);
    }
    return MMF_ERR_ARG;
}

int mmf_swiglu(const void* x, int64_t ldx, const void* y, int64_t ldy, void* out, int64_t rows, int64_t cols,
               int dtype, void* stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (rows < 0 || cols < 0 || (rows * cols > 0 && (!x || !y || !out))) return MMF_ERR_ARG;
    switch (dtype) {
        case MMF_F32: return launch_swiglu<float>(x, ldx, y, ldy, out, rows, cols, stream);
        case MMF_BF16: return launch_swiglu<bf16_t>(x, ldx, y, ldy, out, rows, cols, stream);
        case MMF_F16: return launch_swiglu<f16_t>(x, ldx, y, ldy, out, rows, cols, stream);
    }
    return MMF_ERR_ARG;
}

}  // extern "C"
