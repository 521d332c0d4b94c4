// Fused BitLinear for decode-sized M: [elementwise / norm prologue] -> RMSNorm -> int8 absmax
// codes -> ternary GEMV -> [epilogue], one launch, weights streamed 2-bit packed from HBM
// exactly once per row of x.
//
// Replaces, for one token, the whole of LayerNormLinearQuantFn.forward
// (mmfreelm/ops/fusedbitnet.py:416-468): the Triton norm/quant row kernel (:63-131), the
// per-call weight_quant (:456) and the dense F.linear (:458) -- and, through the prologue /
// epilogue variants, the elementwise kernels the model runs around each BitLinear
// (mmfreelm/models/hgrn_bit/modeling_hgrn_bit.py:55-59,97-109, mmfreelm/layers/hgrn_bit.py:113-139).
// A decode step is a chain of dependent launches whose cost is latency, not bandwidth, so
// every elementwise op is folded into the GEMV that consumes or produces it.
//
// Grid = (row groups of 32 outputs, M).  A workgroup of 8 waves owns R n-blocks of one row of x.
//   prologue : every workgroup recomputes the row's input itself (the row is <= 16 KiB and L2
//              resident) and leaves the int8 codes in LDS:
//                PRO_PLAIN      v = x
//                PRO_NORM       v = T(RMSNorm(x; w1, eps1))                    (block norm)
//                PRO_RESNORM    s = x + aux; res_out = s; v = T(RMSNorm(s))    (fused residual)
//                PRO_GATEDNORM  v = T(RMSNorm(x; w1) * aux * sigmoid(aux))     (g_norm)
//                PRO_SWIGLU     v = T((x * aux) / (1 + exp(-x)))               (MLP activation)
//              then  y = RMSNorm(v; norm_w, eps),  q = int8 absmax codes of y.
//              The packed weight loads of the wave are issued before any of it.
//   main     : wave w takes the 1 KiB weight blocks kb = w, w+8, ... of each of its R n-blocks;
//              a lane holds 64 weights of one output row, expands each dword to four
//              byte-wide code dwords (shift + mask) and accumulates with v_dot4_i32_i8
//              against the broadcast activation bytes read from LDS.
//   epilogue : halves of the wave are folded with one cross-lane move, the 8 wave partials
//              through LDS;  r = T(fp32(acc - sum(q)) * deq_row * deq_weight (+ bias)), then
//                EPI_PLAIN   out = r, or T(r + addend)                          (residual add)
//                EPI_STEP    R = 3 (i, f, g rows of the same 32 channels): gate math, one
//                            recurrence step on the fp32 state, writes o and g
//                EPI_SWIGLU  R = 2 (gate, up rows of the same 32 channels): out = swiglu
#include "mmf_common.h"

namespace {

constexpr int kGemvWaves = 8;
constexpr int kGemvThreads = kGemvWaves * 64;
constexpr int kGemvMaxBlocksPerWave = 8;                        // Kp <= 8 * 8 * 128 = 8192
constexpr int64_t kGemvMaxK = (int64_t)kGemvWaves * kGemvMaxBlocksPerWave * 128;

enum Pro : int { PRO_PLAIN = 0, PRO_NORM = 1, PRO_RESNORM = 2, PRO_GATEDNORM = 3, PRO_SWIGLU = 4 };
enum Epi : int { EPI_PLAIN = 0, EPI_STEP = 1, EPI_SWIGLU = 2 };

struct GemvArgs {
    const void* x;        // [M, K], row stride ldx
    const void* aux;      // residual / gate / up operand of the prologue, row stride ldaux
    void* res_out;        // PRO_RESNORM: summed residual stream [M, K] (written by the first workgroup of a row)
    const void* w1;       // weight of the prologue's own norm [K]
    const void* norm_w;   // BitLinear's inner norm weight [K] or null
    const uint4* packed;  // [Np/32][Kp/128][64] uint4
    const float* wdeq;    // one scale per segment of seg_rows output rows
    const void* bias;     // [N] or null
    const void* addend;   // [M, N] or null: out = T(T(o) + addend)
    void* out;            // EPI_PLAIN [M, N]; EPI_SWIGLU [M, N/2]; EPI_STEP: o [M, N/3]
    void* g_out;          // EPI_STEP: raw g projection [M, N/3]
    const float* lb;      // EPI_STEP: lower bound [N/3] or null
    float* state;         // EPI_STEP: recurrent state [M, N/3] fp32, updated in place
    int64_t K, Kp, N, seg_rows, ldx, ldaux;
    float eps, eps1;
};

template <int NW>
__device__ __forceinline__ double block_sum_once(double v, double* slot) {
    v = mmf_wave_sum(v);
    if ((threadIdx.x & 63) == 0) slot[threadIdx.x >> 6] = v;
    __syncthreads();
    double s = slot[0];
#pragma unroll
    for (int i = 1; i < NW; ++i) s += slot[i];
    return s;
}
template <int NW>
__device__ __forceinline__ float block_max_once(float v, float* slot) {
    v = mmf_wave_max(v);
    if ((threadIdx.x & 63) == 0) slot[threadIdx.x >> 6] = v;
    __syncthreads();
    float s = slot[0];
#pragma unroll
    for (int i = 1; i < NW; ++i) s = fmaxf(s, slot[i]);
    return s;
}

template <typename T, typename TW, int NV, int PRO, int EPI>
__global__ __launch_bounds__(kGemvThreads) void bitlinear_gemv_kernel(GemvArgs a) {
    constexpr int R = EPI == EPI_STEP ? 3 : EPI == EPI_SWIGLU ? 2 : 1;
    extern __shared__ __align__(16) unsigned char smem[];
    int8_t* q_lds = reinterpret_cast<int8_t*>(smem);            // Kp bytes
    // one slot array per reduction, so each costs a single barrier
    __shared__ double red_a[kGemvWaves], red_b[kGemvWaves];
    __shared__ float red_f[kGemvWaves];
    __shared__ int red_q[kGemvWaves];
    __shared__ int part[R][kGemvWaves][32];

    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);   // wave-uniform: keep it in a scalar register
    const int64_t nb = blockIdx.x, row = blockIdx.y;
    const int64_t K = a.K, Kp = a.Kp, KB = Kp >> 7;
    const int64_t NBseg = (a.N / R + 31) >> 5;                  // n-blocks per stacked segment (R > 1)

    // ---- issue this wave's weight loads first (independent of the prologue)
    uint4 wreg[R][kGemvMaxBlocksPerWave];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int i = 0; i < kGemvMaxBlocksPerWave; ++i) {
            const int64_t kb = wave + (int64_t)i * kGemvWaves;
            if (kb < KB) wreg[r][i] = a.packed[((nb + r * NBseg) * KB + kb) * 64 + lane];
        }

    // ---- all other global loads the kernel will need, back to back
    const bool vec_ok = (K % 8) == 0 && (a.ldx % 8) == 0 && (a.ldaux % 8) == 0;
    const T* x = static_cast<const T*>(a.x) + row * a.ldx;
    const T* aux = static_cast<const T*>(a.aux) + row * a.ldaux;
    const TW* w1 = static_cast<const TW*>(a.w1);
    const TW* nw = static_cast<const TW*>(a.norm_w);
    float xv[NV][8], av[PRO >= PRO_RESNORM ? NV : 1][8], w1v[(PRO >= PRO_NORM && PRO <= PRO_GATEDNORM) ? NV : 1][8], wv[NV][8];
#pragma unroll
    for (int v = 0; v < NV; ++v) {
        const int64_t k0 = ((int64_t)v * kGemvThreads + threadIdx.x) * 8;
        if (k0 < K) {
            mmf_load8<T>(x, k0, K, vec_ok, xv[v]);
            if constexpr (PRO >= PRO_RESNORM) mmf_load8<T>(aux, k0, K, vec_ok, av[v]);
            if constexpr (PRO >= PRO_NORM && PRO <= PRO_GATEDNORM) mmf_load8<TW>(w1, k0, K, vec_ok, w1v[v]);
            if (nw) mmf_load8<TW>(nw, k0, K, vec_ok, wv[v]);
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i) xv[v][i] = 0.0f;
        }
    }
    float ep_wdeq[R], ep_bias = 0.0f, ep_add = 0.0f, ep_lb = 0.0f, ep_state = 0.0f;
    const int64_t ch = nb * 32 + (threadIdx.x & 31);            // output column / channel of the epilogue lanes
    const int64_t Nseg = a.N / R;
    if (threadIdx.x < 32 && ch < Nseg) {
#pragma unroll
        for (int r = 0; r < R; ++r) ep_wdeq[r] = a.wdeq[(ch + r * NBseg * 32) / a.seg_rows];
        if constexpr (EPI == EPI_PLAIN) {
            if (a.bias) ep_bias = mmf_to_float(static_cast<const T*>(a.bias)[ch]);
            if (a.addend) ep_add = mmf_to_float(static_cast<const T*>(a.addend)[row * a.N + ch]);
        }
        if constexpr (EPI == EPI_STEP) {
            if (a.lb) ep_lb = a.lb[ch];
            ep_state = a.state[row * Nseg + ch];
        }
    }

    // ---- prologue stage 1: the value the BitLinear sees, v (rounded to T like the tensor it replaces)
    if constexpr (PRO == PRO_RESNORM) {
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            const int64_t k0 = ((int64_t)v * kGemvThreads + threadIdx.x) * 8;
            if (k0 < K) {
#pragma unroll
                for (int i = 0; i < 8; ++i) xv[v][i] = __fadd_rn(xv[v][i], av[v][i]);
                if (a.res_out && blockIdx.x == 0)
                    mmf_store8<T>(static_cast<T*>(a.res_out) + row * K, k0, K, (K % 8) == 0, xv[v]);
            }
        }
    }
    if constexpr (PRO == PRO_NORM || PRO == PRO_RESNORM || PRO == PRO_GATEDNORM) {
        double s1 = 0.0;
#pragma unroll
        for (int v = 0; v < NV; ++v)
#pragma unroll
            for (int i = 0; i < 8; ++i) s1 += (double)xv[v][i] * (double)xv[v][i];
        s1 = block_sum_once<kGemvWaves>(s1, red_a);
        const float rstd1 = mmf_rstd(s1, K, a.eps1);
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            const int64_t k0 = ((int64_t)v * kGemvThreads + threadIdx.x) * 8;
            if (k0 < K) {
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    float y = __fmul_rn(__fmul_rn(xv[v][i], rstd1), w1v[v][i]);
                    if constexpr (PRO == PRO_GATEDNORM) y = __fmul_rn(__fmul_rn(y, av[v][i]), mmf_sigmoid(av[v][i]));
                    xv[v][i] = (k0 + i < K) ? mmf_round_to<T>(y) : 0.0f;
                }
            }
        }
    }
    if constexpr (PRO == PRO_SWIGLU) {
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            const int64_t k0 = ((int64_t)v * kGemvThreads + threadIdx.x) * 8;
            if (k0 < K) {
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const float g = xv[v][i];
                    const float z = __fdiv_rn(__fmul_rn(g, av[v][i]), __fadd_rn(1.0f, mmf_exp(-g)));
                    xv[v][i] = (k0 + i < K) ? mmf_round_to<T>(z) : 0.0f;
                }
            }
        }
    }

    // ---- prologue stage 2: BitLinear's own RMSNorm + absmax int8 codes into LDS
    double ss = 0.0;
#pragma unroll
    for (int v = 0; v < NV; ++v)
#pragma unroll
        for (int i = 0; i < 8; ++i) ss += (double)xv[v][i] * (double)xv[v][i];
    ss = block_sum_once<kGemvWaves>(ss, red_b);
    const float rstd = mmf_rstd(ss, K, a.eps);
    float amax = 0.0f;
#pragma unroll
    for (int v = 0; v < NV; ++v) {
        const int64_t k0 = ((int64_t)v * kGemvThreads + threadIdx.x) * 8;
        if (k0 < K) {
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                float y = __fmul_rn(xv[v][i], rstd);
                if (nw) y = __fmul_rn(y, wv[v][i]);
                xv[v][i] = y;
                amax = fmaxf(amax, fabsf(y));
            }
        }
    }
    amax = block_max_once<kGemvWaves>(amax, red_f);
    const float scale = __fdiv_rn(127.0f, fmaxf(amax, 1e-5f));
    int qs = 0;
#pragma unroll
    for (int v = 0; v < NV; ++v) {
        const int64_t k0 = ((int64_t)v * kGemvThreads + threadIdx.x) * 8;
        if (k0 < Kp) {
            uint32_t lo = 0, hi = 0;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int c = (k0 + i < K) ? mmf_code(xv[v][i], scale) : 0;
                qs += c;
                const uint32_t b = (uint32_t)(c & 0xff) << (8 * (i & 3));
                if (i < 4) lo |= b; else hi |= b;
            }
            *reinterpret_cast<uint2*>(q_lds + k0) = make_uint2(lo, hi);
        }
    }
    qs = mmf_wave_sum(qs);
    if (lane == 0) red_q[wave] = qs;
    __syncthreads();                                            // publishes q_lds and red_q

    // ---- main: sum_k q[k] * (t[n,k] + 1) for n = (nb + r*NBseg)*32 + lane%32 over this wave's blocks
    const int half = lane >> 5;
    int acc[R];
#pragma unroll
    for (int r = 0; r < R; ++r) acc[r] = 0;
#pragma unroll
    for (int i = 0; i < kGemvMaxBlocksPerWave; ++i) {
        const int64_t kb = wave + (int64_t)i * kGemvWaves;
        if (kb < KB) {
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                const int4 qv = *reinterpret_cast<const int4*>(q_lds + kb * 128 + s * 32 + half * 16);
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    const uint32_t w = s == 0 ? wreg[r][i].x : s == 1 ? wreg[r][i].y : s == 2 ? wreg[r][i].z : wreg[r][i].w;
                    acc[r] = __builtin_amdgcn_sdot4((int)(w & 0x03030303u), qv.x, acc[r], false);
                    acc[r] = __builtin_amdgcn_sdot4((int)((w >> 2) & 0x03030303u), qv.y, acc[r], false);
                    acc[r] = __builtin_amdgcn_sdot4((int)((w >> 4) & 0x03030303u), qv.z, acc[r], false);
                    acc[r] = __builtin_amdgcn_sdot4((int)((w >> 6) & 0x03030303u), qv.w, acc[r], false);
                }
            }
        }
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
        acc[r] += __shfl_xor(acc[r], 32, 64);
        if (lane < 32) part[r][wave][lane] = acc[r];
    }
    __syncthreads();
    if (threadIdx.x < 32 && ch < Nseg) {
        int qtot = 0;
#pragma unroll
        for (int w = 0; w < kGemvWaves; ++w) qtot += red_q[w];
        const float deq = __fdiv_rn(1.0f, scale);
        float res[R];
#pragma unroll
        for (int r = 0; r < R; ++r) {
            int tot = 0;
#pragma unroll
            for (int w = 0; w < kGemvWaves; ++w) tot += part[r][w][threadIdx.x];
            res[r] = __fmul_rn(__fmul_rn((float)(tot - qtot), deq), ep_wdeq[r]);
        }
        if constexpr (EPI == EPI_PLAIN) {
            float o = res[0];
            if (a.bias) o = __fadd_rn(o, ep_bias);
            if (a.addend) o = __fadd_rn(mmf_round_to<T>(o), ep_add);
            static_cast<T*>(a.out)[row * a.N + ch] = mmf_from_float<T>(o);
        } else if constexpr (EPI == EPI_STEP) {
            // res = raw i, f, g projections of channel ch (each rounded to T like the tensors they replace)
            const float iv = mmf_round_to<T>(res[0]), fv = mmf_round_to<T>(res[1]);
            float s = mmf_sigmoid(fv);
            if (a.lb) s = __fadd_rn(ep_lb, __fmul_rn(__fsub_rn(1.0f, ep_lb), s));
            const float go = mmf_round_to<T>(s);
            const float xo = mmf_round_to<T>(__fdiv_rn(__fmul_rn(iv, __fsub_rn(1.0f, go)), __fadd_rn(1.0f, mmf_exp(-iv))));
            const float h = __fadd_rn(__fmul_rn(go, ep_state), xo);
            a.state[row * Nseg + ch] = h;
            static_cast<T*>(a.out)[row * Nseg + ch] = mmf_from_float<T>(h);
            static_cast<T*>(a.g_out)[row * Nseg + ch] = mmf_from_float<T>(res[2]);
        } else {
            const float g = mmf_round_to<T>(res[0]), u = mmf_round_to<T>(res[1]);
            static_cast<T*>(a.out)[row * Nseg + ch] =
                mmf_from_float<T>(__fdiv_rn(__fmul_rn(g, u), __fadd_rn(1.0f, mmf_exp(-g))));
        }
    }
}

template <typename T, typename TW, int PRO, int EPI>
int launch_gemv(const GemvArgs& a, int64_t M, hipStream_t s) {
    constexpr int R = EPI == EPI_STEP ? 3 : EPI == EPI_SWIGLU ? 2 : 1;
    const int64_t nv = mmf_ceil_div(a.Kp, (int64_t)kGemvThreads * 8);
    dim3 grid((unsigned)mmf_ceil_div(a.N / R, 32), (unsigned)M), block(kGemvThreads);
    const size_t lds = (size_t)a.Kp;
    if (nv <= 1) bitlinear_gemv_kernel<T, TW, 1, PRO, EPI><<<grid, block, lds, s>>>(a);
    else if (nv <= 2) bitlinear_gemv_kernel<T, TW, 2, PRO, EPI><<<grid, block, lds, s>>>(a);
    else return MMF_ERR_WIDE;
    MMF_CHECK_LAUNCH();
    return 0;
}

template <typename T, typename TW>
int dispatch_gemv_kind(const GemvArgs& a, int64_t M, int pro, int epi, hipStream_t s) {
    // the combinations a decode step uses
    if (epi == EPI_PLAIN) {
        switch (pro) {
            case PRO_PLAIN: return launch_gemv<T, TW, PRO_PLAIN, EPI_PLAIN>(a, M, s);
            case PRO_NORM: return launch_gemv<T, TW, PRO_NORM, EPI_PLAIN>(a, M, s);
            case PRO_RESNORM: return launch_gemv<T, TW, PRO_RESNORM, EPI_PLAIN>(a, M, s);
            case PRO_GATEDNORM: return launch_gemv<T, TW, PRO_GATEDNORM, EPI_PLAIN>(a, M, s);
            case PRO_SWIGLU: return launch_gemv<T, TW, PRO_SWIGLU, EPI_PLAIN>(a, M, s);
        }
    } else if (epi == EPI_STEP) {
        if (pro == PRO_NORM) return launch_gemv<T, TW, PRO_NORM, EPI_STEP>(a, M, s);
        if (pro == PRO_PLAIN) return launch_gemv<T, TW, PRO_PLAIN, EPI_STEP>(a, M, s);
    } else if (epi == EPI_SWIGLU) {
        if (pro == PRO_RESNORM) return launch_gemv<T, TW, PRO_RESNORM, EPI_SWIGLU>(a, M, s);
        if (pro == PRO_PLAIN) return launch_gemv<T, TW, PRO_PLAIN, EPI_SWIGLU>(a, M, s);
    }
    return MMF_ERR_ARG;
}

template <typename T>
int dispatch_gemv_w(const GemvArgs& a, int64_t M, int pro, int epi, int x_dtype, int w_dtype, hipStream_t s) {
    if (w_dtype == MMF_F32) return dispatch_gemv_kind<T, float>(a, M, pro, epi, s);
    if (w_dtype == x_dtype) return dispatch_gemv_kind<T, T>(a, M, pro, epi, s);
    return MMF_ERR_ARG;
}

bool al16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

}  // namespace

extern "C" {

int64_t mmf_bitlinear_gemv_max_k(void) { return kGemvMaxK; }

int mmf_bitlinear_gemv_fused(int prologue, int epilogue, const void* x, int64_t ldx, const void* aux, int64_t ldaux,
                             void* res_out, const void* w1, float eps1, const void* norm_weight, float eps,
                             const void* packed, const float* wdeq, int64_t seg_rows, const void* bias,
                             const void* addend, void* out, void* g_out, const float* lower_bound, float* state,
                             int64_t M, int64_t K, int64_t N, int x_dtype, int weight_dtype, void* stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (M < 0 || K <= 0 || N <= 0 || seg_rows <= 0 || ldx < K) return MMF_ERR_ARG;
    if (M == 0) return 0;
    if (M > 65535 || !x || !packed || !wdeq || !out) return MMF_ERR_ARG;
    if (prologue < PRO_PLAIN || prologue > PRO_SWIGLU || epilogue < EPI_PLAIN || epilogue > EPI_SWIGLU) return MMF_ERR_ARG;
    if (prologue >= PRO_RESNORM && (!aux || ldaux < K)) return MMF_ERR_ARG;
    if (prologue >= PRO_NORM && prologue <= PRO_GATEDNORM && !w1) return MMF_ERR_ARG;
    if (epilogue == EPI_STEP && (N % 96 != 0 || !g_out || !state || bias || addend)) return MMF_ERR_ARG;
    if (epilogue == EPI_SWIGLU && (N % 64 != 0 || bias || addend)) return MMF_ERR_ARG;
    GemvArgs a{};
    a.x = x; a.aux = aux ? aux : x; a.res_out = res_out; a.w1 = w1; a.norm_w = norm_weight;
    a.packed = static_cast<const uint4*>(packed); a.wdeq = wdeq; a.bias = bias; a.addend = addend; a.out = out;
    a.g_out = g_out; a.lb = lower_bound; a.state = state;
    a.K = K; a.Kp = mmf_round_up(K, 128); a.N = N; a.seg_rows = seg_rows; a.ldx = ldx; a.ldaux = aux ? ldaux : ldx;
    a.eps = eps; a.eps1 = eps1;
    if (a.Kp > kGemvMaxK) return MMF_ERR_WIDE;
    if (!al16(packed)) return MMF_ERR_ALIGN;
    if (K % 8 == 0 && ldx % 8 == 0 && a.ldaux % 8 == 0 &&
        !(al16(x) && al16(a.aux) && al16(w1) && al16(norm_weight) && al16(res_out)))
        return MMF_ERR_ALIGN;
    if (!norm_weight && !w1) weight_dtype = MMF_F32;
    switch (x_dtype) {
        case MMF_F32: return dispatch_gemv_w<float>(a, M, prologue, epilogue, x_dtype, weight_dtype, stream);
        case MMF_BF16: return dispatch_gemv_w<bf16_t>(a, M, prologue, epilogue, x_dtype, weight_dtype, stream);
        case MMF_F16: return dispatch_gemv_w<f16_t>(a, M, prologue, epilogue, x_dtype, weight_dtype, stream);
    }
    return MMF_ERR_ARG;
}

int mmf_bitlinear_gemv(const void* x, const void* norm_weight, const void* packed, const float* wdeq,
                       int64_t seg_rows, const void* bias, const void* addend, void* out, int64_t M, int64_t K, int64_t N,
                       float eps, int x_dtype, int norm_weight_dtype, void* stream_) {
    return mmf_bitlinear_gemv_fused(PRO_PLAIN, EPI_PLAIN, x, K, nullptr, 0, nullptr, nullptr, 0.0f, norm_weight, eps, packed,
                                    wdeq, seg_rows, bias, addend, out, nullptr, nullptr, nullptr, M, K, N, x_dtype,
                                    norm_weight_dtype, stream_);
}

}  // extern "C"
