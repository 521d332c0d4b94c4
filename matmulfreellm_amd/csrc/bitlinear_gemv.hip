// Fused BitLinear for decode-sized M: RMSNorm -> int8 absmax codes -> ternary GEMV,
// one launch, weights streamed 2-bit packed from HBM exactly once per row of x.
//
// Replaces, for one token, the whole of LayerNormLinearQuantFn.forward
// (mmfreelm/ops/fusedbitnet.py:416-468): the Triton norm/quant row kernel (:63-131), the
// per-call weight_quant (:456) and the dense F.linear (:458).
//
// Grid = (Np/32, M).  A workgroup of 8 waves owns 32 output features of one row of x.
//   prologue : every workgroup normalises and quantises the row itself (the row is
//              <= 16 KiB and L2 resident; recomputing it is cheaper than a second launch)
//              and leaves the int8 codes in LDS.  The packed weight loads of the wave are
//              issued before the prologue so HBM latency hides behind it.
//   main     : wave w takes the 1 KiB weight blocks kb = w, w+8, ...; a lane holds 64
//              weights of one output row, expands each dword to four byte-wide code
//              dwords (shift + mask) and accumulates with v_dot4_i32_i8 against the
//              broadcast activation bytes read from LDS.
//   epilogue : halves of the wave are folded with one cross-lane move, the 8 wave partials
//              through LDS; out = fp32(acc - sum(q)) * deq_row * deq_weight (+ bias).
#include "mmf_common.h"
#include "../../include/mmf.h"

namespace {

constexpr int kGemvWaves = 8;
constexpr int kGemvThreads = kGemvWaves * 64;
constexpr int kGemvMaxBlocksPerWave = 8;                        // Kp <= 8 * 8 * 128 = 8192
constexpr int64_t kGemvMaxK = (int64_t)kGemvWaves * kGemvMaxBlocksPerWave * 128;

struct GemvArgs {
    const void* x;        // [M, K]
    const void* norm_w;   // [K] or null
    const uint4* packed;  // [Np/32][Kp/128][64] uint4
    const float* wdeq;    // one scale per segment of seg_rows output rows
    const void* bias;     // [N] or null (dtype T)
    const void* addend;   // [M, N] or null (dtype T): out = T(T(o) + addend)
    void* out;            // [M, N]
    int64_t K, Kp, N, seg_rows;
    float eps;
};

template <typename T, typename TW, int NV>
__global__ __launch_bounds__(kGemvThreads) void bitlinear_gemv_kernel(GemvArgs a) {
    extern __shared__ __align__(16) unsigned char smem[];
    int8_t* q_lds = reinterpret_cast<int8_t*>(smem);            // Kp bytes
    __shared__ double red_d[kGemvWaves];
    __shared__ float red_f[kGemvWaves];
    __shared__ int red_i[kGemvWaves];
    __shared__ int part[kGemvWaves][32];

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t nb = blockIdx.x, row = blockIdx.y;
    const int64_t K = a.K, Kp = a.Kp, KB = Kp >> 7;

    // ---- issue this wave's weight loads first (independent of the prologue)
    uint4 wreg[kGemvMaxBlocksPerWave];
#pragma unroll
    for (int i = 0; i < kGemvMaxBlocksPerWave; ++i) {
        const int64_t kb = wave + (int64_t)i * kGemvWaves;
        if (kb < KB) wreg[i] = a.packed[(nb * KB + kb) * 64 + lane];
    }

    // ---- prologue: RMSNorm + absmax int8 codes of row `row` into LDS.  All global loads the
    // kernel will ever need (x, norm weight, and the epilogue's scale / bias / addend) are
    // issued here, back to back, so the kernel pays one memory round trip, not four.
    const bool vec_ok = (K % 8) == 0;
    const T* x = static_cast<const T*>(a.x) + row * K;
    const TW* nw = static_cast<const TW*>(a.norm_w);
    float xv[NV][8];
    float wv[NV][8];
    float ep_wdeq = 0.0f, ep_bias = 0.0f, ep_add = 0.0f;
    if (threadIdx.x < 32) {
        const int64_t n = nb * 32 + threadIdx.x;
        if (n < a.N) {
            ep_wdeq = a.wdeq[n / a.seg_rows];
            if (a.bias) ep_bias = mmf_to_float(static_cast<const T*>(a.bias)[n]);
            if (a.addend) ep_add = mmf_to_float(static_cast<const T*>(a.addend)[row * a.N + n]);
        }
    }
    double ss = 0.0;
#pragma unroll
    for (int v = 0; v < NV; ++v) {
        const int64_t k0 = ((int64_t)v * kGemvThreads + threadIdx.x) * 8;
        if (k0 < K && nw) mmf_load8<TW>(nw, k0, K, vec_ok, wv[v]);
    }
#pragma unroll
    for (int v = 0; v < NV; ++v) {
        const int64_t k0 = ((int64_t)v * kGemvThreads + threadIdx.x) * 8;
        if (k0 < K) {
            mmf_load8<T>(x, k0, K, vec_ok, xv[v]);
#pragma unroll
            for (int i = 0; i < 8; ++i) ss += (double)xv[v][i] * (double)xv[v][i];
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i) xv[v][i] = 0.0f;
        }
    }
    ss = mmf_block_sum<kGemvWaves>(ss, red_d);
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
    amax = mmf_block_max<kGemvWaves>(amax, red_f);
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
    qs = mmf_block_sum<kGemvWaves>(qs, red_i);   // its barriers also publish q_lds

    // ---- main: sum_k q[k] * (t[n,k] + 1) for n = nb*32 + lane%32 over this wave's blocks
    const int half = lane >> 5;
    int acc = 0;
#pragma unroll
    for (int i = 0; i < kGemvMaxBlocksPerWave; ++i) {
        const int64_t kb = wave + (int64_t)i * kGemvWaves;
        if (kb < KB) {
            const uint32_t wd[4] = {wreg[i].x, wreg[i].y, wreg[i].z, wreg[i].w};
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                const int4 qv = *reinterpret_cast<const int4*>(q_lds + kb * 128 + s * 32 + half * 16);
                const uint32_t w = wd[s];
                acc = __builtin_amdgcn_sdot4((int)(w & 0x03030303u), qv.x, acc, false);
                acc = __builtin_amdgcn_sdot4((int)((w >> 2) & 0x03030303u), qv.y, acc, false);
                acc = __builtin_amdgcn_sdot4((int)((w >> 4) & 0x03030303u), qv.z, acc, false);
                acc = __builtin_amdgcn_sdot4((int)((w >> 6) & 0x03030303u), qv.w, acc, false);
            }
        }
    }
    acc += __shfl_xor(acc, 32, 64);
    if (lane < 32) part[wave][lane] = acc;
    __syncthreads();
    if (threadIdx.x < 32) {
        int tot = 0;
#pragma unroll
        for (int w = 0; w < kGemvWaves; ++w) tot += part[w][threadIdx.x];
        const int64_t n = nb * 32 + threadIdx.x;
        if (n < a.N) {
            const float deq = __fdiv_rn(1.0f, scale);
            float o = __fmul_rn(__fmul_rn((float)(tot - qs), deq), ep_wdeq);
            if (a.bias) o = __fadd_rn(o, ep_bias);
            if (a.addend) o = __fadd_rn(mmf_round_to<T>(o), ep_add);
            static_cast<T*>(a.out)[row * a.N + n] = mmf_from_float<T>(o);
        }
    }
}

template <typename T, typename TW>
int launch_gemv(const GemvArgs& a, int64_t M, hipStream_t s) {
    const int64_t nv = mmf_ceil_div(a.Kp, (int64_t)kGemvThreads * 8);
    dim3 grid((unsigned)mmf_ceil_div(a.N, 32), (unsigned)M), block(kGemvThreads);
    const size_t lds = (size_t)a.Kp;
    if (nv <= 1) bitlinear_gemv_kernel<T, TW, 1><<<grid, block, lds, s>>>(a);
    else if (nv <= 2) bitlinear_gemv_kernel<T, TW, 2><<<grid, block, lds, s>>>(a);
    else return MMF_ERR_WIDE;
    MMF_CHECK_LAUNCH();
    return 0;
}

template <typename T>
int dispatch_gemv_w(const GemvArgs& a, int64_t M, int x_dtype, int w_dtype, hipStream_t s) {
    if (!a.norm_w || w_dtype == MMF_F32) return launch_gemv<T, float>(a, M, s);
    if (w_dtype == x_dtype) return launch_gemv<T, T>(a, M, s);
    return MMF_ERR_ARG;
}

}  // namespace

extern "C" {

int64_t mmf_bitlinear_gemv_max_k(void) { return kGemvMaxK; }

int mmf_bitlinear_gemv(const void* x, const void* norm_weight, const void* packed, const float* wdeq,
                       int64_t seg_rows, const void* bias, const void* addend, void* out, int64_t M, int64_t K, int64_t N,
                       float eps,
                       int x_dtype, int norm_weight_dtype, void* stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (M < 0 || K <= 0 || N <= 0 || seg_rows <= 0 || (M > 0 && (!x || !packed || !wdeq || !out))) return MMF_ERR_ARG;
    if (M == 0) return 0;
    if (M > 65535) return MMF_ERR_ARG;
    GemvArgs a{};
    a.x = x; a.norm_w = norm_weight; a.packed = static_cast<const uint4*>(packed); a.wdeq = wdeq; a.bias = bias; a.addend = addend;
    a.out = out; a.K = K; a.Kp = mmf_round_up(K, 128); a.N = N; a.seg_rows = seg_rows; a.eps = eps;
    if (a.Kp > kGemvMaxK) return MMF_ERR_WIDE;
    if ((reinterpret_cast<uintptr_t>(packed) & 15u) ||
        (K % 8 == 0 && ((reinterpret_cast<uintptr_t>(x) & 15u) || (reinterpret_cast<uintptr_t>(norm_weight) & 15u))))
        return MMF_ERR_ALIGN;
    switch (x_dtype) {
        case MMF_F32: return dispatch_gemv_w<float>(a, M, x_dtype, norm_weight_dtype, stream);
        case MMF_BF16: return dispatch_gemv_w<bf16_t>(a, M, x_dtype, norm_weight_dtype, stream);
        case MMF_F16: return dispatch_gemv_w<f16_t>(a, M, x_dtype, norm_weight_dtype, stream);
    }
    return MMF_ERR_ARG;
}

}  // extern "C"
