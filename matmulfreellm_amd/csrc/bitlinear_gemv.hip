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
// Grid = (groups of 32 - or, for small launches, 8 - output rows, M).  A workgroup of 8 to 16 waves owns R
// n-blocks (or 8 rows of each) of one row of x.
//   prologue : every workgroup recomputes the row's input itself (the row is <= 16 KiB and L2
//              resident) and leaves the int8 codes in LDS:
//                PRO_PLAIN      v = x
//                PRO_NORM       v = T(RMSNorm(x; w1, eps1))                    (block norm)
//                PRO_RESNORM    s = x + aux; res_out = s; v = T(RMSNorm(s))    (fused residual)
//                PRO_GATEDNORM  v = T(RMSNorm(x; w1) * aux * sigmoid(aux))     (g_norm)
//                PRO_SWIGLU     v = T((x * aux) / (1 + exp(-x)))               (MLP activation)
//              then  y = RMSNorm(v; norm_w, eps),  q = int8 absmax codes of y.
//              A launch costs what its instruction stream and its dependent memory round
//              trips cost, so every global load of the kernel (row, norm weights, the wave's
//              packed weight blocks, the epilogue's operands) is issued up front, raw, and
//              converted only where it is used; a thread owns 4 elements of the row per pass.
//   main     : wave w takes the 1 KiB weight blocks kb = w, w+NW, ... of each of its R n-blocks
//              (8-row mode: groups of four k-blocks, two 128-byte runs of each);
//              a lane holds 64 weights of one output row, expands each dword to four
//              byte-wide code dwords (shift + mask) and accumulates with v_dot4_i32_i8
//              against the broadcast activation bytes read from LDS.
//   epilogue : the lanes' partial sums (k-halves, waves or k-groups) meet in LDS;
//              r = T(fp32(acc - sum(q)) * deq_row * deq_weight (+ bias)), then
//                EPI_PLAIN   out = r, or T(r + addend)                          (residual add)
//                EPI_STEP    R = 3 (i, f, g rows of the same 32 channels): gate math, one
//                            recurrence step on the fp32 state, writes o and g
//                EPI_SWIGLU  R = 2 (gate, up rows of the same 32 channels): out = swiglu
#include "mmf_common.h"
#include <stdlib.h>

namespace {

constexpr int kGemvEl = 4;                                      // elements of x per thread and pass
constexpr int64_t kGemvMaxK = 8192;                             // 16 waves x 2 passes (or 8 waves x 4)

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
    int64_t ldx, ldaux;
    int K, Kp, N, seg_rows;                                     // all < 2^31 (checked by the entry point)
    float eps, eps1;
    double inv_K;         // RN(1 / K)
};

// NW waves per workgroup, NV passes over the row (Kp <= NV * NW * 256); a wave then owns at most
// 2 * NV of the row's 1 KiB weight blocks per n-block.  The launcher takes the fewest passes, then
// the fewest waves, that cover K: a thread's instruction stream, not bandwidth, sets the time.  VEC: K, the row strides and every pointer allow 4-element accesses.
// S: row split.  S = 1: a workgroup owns whole n-blocks (32 output rows; lane = (k-half, row)).
// S = 4: it owns 8 of the 32 rows, so that a 2048-row projection fills 256 CUs instead of 64; a
// lane is (k-block of a group of four, k-half, row of 8), a wave-load covers four k-blocks (two
// 128-byte runs of each 1 KiB block), and the waves share out the (n-block, k-group) items.
// WALK (S = 1, plain epilogue): a launch with many more n-blocks than CUs (a vocabulary-sized projection) runs on a
// grid of as many workgroups as are resident at once; workgroup b of a row of x takes the n-blocks b, b + grid, ... behind ONE
// prologue, the next block's packed weights in flight while the current one is contracted -- otherwise every 16 KiB of
// weights would wait behind a re-quantisation of the whole row.
template <typename T, typename TW, int NW, int NV, int PRO, int EPI, bool VEC, int S, bool WALK = false>
__global__ __launch_bounds__(64 * NW) void bitlinear_gemv_kernel(GemvArgs a) {
    static_assert(!WALK || (S == 1 && EPI == EPI_PLAIN), "the n-block walk is built for whole n-blocks and the plain epilogue");
    constexpr int kGemvWaves = NW, kGemvThreads = 64 * NW;
    constexpr int R = EPI == EPI_STEP ? 3 : EPI == EPI_SWIGLU ? 2 : 1;
    constexpr int BPW = 2 * NV;
    constexpr int GMAX = NV * NW / 2;                           // k-groups of four blocks (S = 4)
    constexpr int ITEMS = (R * GMAX + kGemvWaves - 1) / kGemvWaves;   // (n-block, k-group) items per wave (S = 4)
    constexpr int CHN = 32 / S;                                 // output channels per workgroup and n-block
    constexpr bool HAS_AUX = PRO >= PRO_RESNORM;
    constexpr bool HAS_W1 = PRO >= PRO_NORM && PRO <= PRO_GATEDNORM;
    extern __shared__ __align__(16) unsigned char smem[];
    int8_t* q_lds = reinterpret_cast<int8_t*>(smem);            // Kp bytes
    // one slot array per reduction, so each costs a single barrier
    __shared__ double red_a[kGemvWaves], red_b[kGemvWaves];
    __shared__ float red_f[kGemvWaves];
    __shared__ int red_q[kGemvWaves];
    __shared__ int2 part[S == 1 ? R * kGemvWaves * 32 : R * GMAX * 8];   // S = 1: [r][wave][row], S = 4: [item][row8]; .x/.y: lane halves

    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int nb = blockIdx.x / S, sub = blockIdx.x % S, row = blockIdx.y;
    const int K = a.K, Kp = a.Kp, KB = Kp >> 7;
    const int Nseg = a.N / R;
    const int NBseg = (Nseg + 31) >> 5;                         // n-blocks per stacked segment (R > 1)

    // ---- every global load of the kernel, back to back: the row first (the prologue's
    // reductions wait for it), then this wave's packed weights, then the epilogue's operands
    const T* x = static_cast<const T*>(a.x) + (int64_t)row * a.ldx;
    const T* aux = static_cast<const T*>(a.aux) + (int64_t)row * a.ldaux;
    const TW* w1 = static_cast<const TW*>(a.w1);
    const TW* nw = static_cast<const TW*>(a.norm_w);
    Raw4<T> xraw[NV], araw[HAS_AUX ? NV : 1];
    Raw4<TW> w1raw[HAS_W1 ? NV : 1], nwraw[NV];
#pragma unroll
    for (int v = 0; v < NV; ++v) {
        const int k0 = (v * kGemvThreads + (int)threadIdx.x) * kGemvEl;
        xraw[v] = raw4_load<T, VEC>(x, k0, K);
        if constexpr (HAS_AUX) araw[v] = raw4_load<T, VEC>(aux, k0, K);
        if constexpr (HAS_W1) w1raw[v] = raw4_load<TW, VEC>(w1, k0, K);
        if (nw) nwraw[v] = raw4_load<TW, VEC>(nw, k0, K);
    }
    constexpr int NWREG = S == 1 ? R * BPW : ITEMS;
    uint4 wreg[NWREG];
    const int G = (KB + 3) >> 2;                                // k-groups in this row (S = 4)
    const int kbi = lane >> 4, half = S == 1 ? lane >> 5 : (lane >> 3) & 1;
    if constexpr (S == 1) {
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int i = 0; i < BPW; ++i) {
                const int kb = wave + i * kGemvWaves;
                if (kb < KB) wreg[r * BPW + i] = a.packed[((int64_t)(nb + r * NBseg) * KB + kb) * 64 + lane];
            }
    } else {
#pragma unroll
        for (int i = 0; i < ITEMS; ++i) {
            const int item = wave + i * kGemvWaves;             // wave-uniform
            wreg[i] = make_uint4(0u, 0u, 0u, 0u);               // code 0 against any activation adds nothing
            if (item < R * G) {
                const int r = item / G, kb = (item % G) * 4 + kbi;
                if (kb < KB)
                    wreg[i] = a.packed[((int64_t)(nb + r * NBseg) * KB + kb) * 64 + half * 32 + sub * CHN + (lane & 7)];
            }
        }
    }
    float ep_wdeq[R], ep_bias = 0.0f, ep_add = 0.0f, ep_lb = 0.0f, ep_state = 0.0f;
    const int ch = nb * 32 + sub * CHN + (lane & (CHN - 1));    // output column / channel of the epilogue lanes
    const bool ep_lane = wave == 0 && lane < CHN && ch < Nseg;
    if (wave == 0) {
        // the 32 outputs of an n-block share a scale (segments are multiples of 32 rows)
#pragma unroll
        for (int r = 0; r < R; ++r) ep_wdeq[r] = a.wdeq[(uint32_t)((nb + r * NBseg) * 32) / (uint32_t)a.seg_rows];
        if (ep_lane) {
            if constexpr (EPI == EPI_PLAIN) {
                if (a.bias) ep_bias = mmf_to_float(static_cast<const T*>(a.bias)[ch]);
                if (a.addend) ep_add = mmf_to_float(static_cast<const T*>(a.addend)[(int64_t)row * a.N + ch]);
            }
            if constexpr (EPI == EPI_STEP) {
                if (a.lb) ep_lb = a.lb[ch];
                ep_state = a.state[(int64_t)row * Nseg + ch];
            }
        }
    }

    // ---- prologue stage 1: the value the BitLinear sees, v (rounded to T like the tensor it replaces)
    float xv[NV][4], av[HAS_AUX ? NV : 1][4];
#pragma unroll
    for (int v = 0; v < NV; ++v) {
        const int k0 = (v * kGemvThreads + (int)threadIdx.x) * kGemvEl;
        raw4_unpack<T>(xraw[v], xv[v]);
        if constexpr (HAS_AUX) raw4_unpack<T>(araw[v], av[v]);
#pragma unroll
        for (int i = 0; i < 4; ++i)
            if (k0 + i >= K) xv[v][i] = 0.0f;
    }
    if constexpr (PRO == PRO_RESNORM) {
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            const int k0 = (v * kGemvThreads + (int)threadIdx.x) * kGemvEl;
#pragma unroll
            for (int i = 0; i < 4; ++i) xv[v][i] = k0 + i < K ? __fadd_rn(xv[v][i], av[v][i]) : 0.0f;
            if (a.res_out && blockIdx.x == 0) raw4_store<T, VEC>(static_cast<T*>(a.res_out) + (int64_t)row * K, k0, K, xv[v]);
        }
    }
    if constexpr (PRO == PRO_NORM || PRO == PRO_RESNORM || PRO == PRO_GATEDNORM) {
        double s1 = 0.0;
#pragma unroll
        for (int v = 0; v < NV; ++v)
#pragma unroll
            for (int i = 0; i < 4; ++i) s1 = mmf_add_square(s1, xv[v][i]);
        s1 = mmf_block_sum_once<kGemvWaves>(s1, red_a);
        const float rstd1 = mmf_rstd(s1, K, a.inv_K, a.eps1);
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            const int k0 = (v * kGemvThreads + (int)threadIdx.x) * kGemvEl;
            float w1v[4], sg[4] = {0.0f, 0.0f, 0.0f, 0.0f};
            raw4_unpack<TW>(w1raw[v], w1v);
            if constexpr (PRO == PRO_GATEDNORM) mmf_sigmoid_n<4>(av[v], sg);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                float y = __fmul_rn(__fmul_rn(xv[v][i], rstd1), w1v[i]);
                if constexpr (PRO == PRO_GATEDNORM) y = __fmul_rn(__fmul_rn(y, av[v][i]), sg[i]);
                xv[v][i] = (k0 + i < K) ? mmf_round_to<T>(y) : 0.0f;
            }
        }
    }
    if constexpr (PRO == PRO_SWIGLU) {
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            const int k0 = (v * kGemvThreads + (int)threadIdx.x) * kGemvEl;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float g = xv[v][i];
                const float z = __fdiv_rn(__fmul_rn(g, av[v][i]), __fadd_rn(1.0f, mmf_exp(-g)));
                xv[v][i] = (k0 + i < K) ? mmf_round_to<T>(z) : 0.0f;
            }
        }
    }

    // ---- prologue stage 2: BitLinear's own RMSNorm + absmax int8 codes into LDS
    double ss = 0.0;
#pragma unroll
    for (int v = 0; v < NV; ++v)
#pragma unroll
        for (int i = 0; i < 4; ++i) ss = mmf_add_square(ss, xv[v][i]);
    ss = mmf_block_sum_once<kGemvWaves>(ss, red_b);
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
    amax = mmf_block_max_once<kGemvWaves>(amax, red_f);
    const float scale = mmf_127_over(fmaxf(amax, 1e-5f));
    const float deq = mmf_rcp_pos(scale);                 // needed by the epilogue only: computed here, in the shadow of the barriers
    int qs = 0;
#pragma unroll
    for (int v = 0; v < NV; ++v) {
        const int k0 = (v * kGemvThreads + (int)threadIdx.x) * kGemvEl;
        if (k0 < Kp) {
            uint32_t packed4 = 0;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int c = (k0 + i < K) ? mmf_code(xv[v][i], scale) : 0;
                qs += c;
                packed4 |= (uint32_t)(c & 0xff) << (8 * i);
            }
            *reinterpret_cast<uint32_t*>(q_lds + k0) = packed4;
        }
    }
    __syncthreads();                                            // publishes q_lds
    // the code sum is only needed by the epilogue: fold it after the barrier, off the critical path
    // (red_q is read behind the next barrier)
    qs = mmf_wave_sum(qs);
    if (lane == 0) red_q[wave] = qs;

    // ---- main + epilogue of one n-block (R stacked ones): weights `wr`, epilogue operands as loaded for that block
    auto contract = [&](const uint4 (&wr)[NWREG], int nbc, const float (&wdq)[R], float bias_v, float add_v) {
        const int chc = nbc * 32 + sub * CHN + (lane & (CHN - 1));
        const bool epl = wave == 0 && lane < CHN && chc < Nseg;
        auto dot_block = [&](const uint4& wq, int kb, int acc) { return mmf_dot_block(q_lds, wq, kb, half, acc); };
        if constexpr (S == 1) {
            int acc[R];
#pragma unroll
            for (int r = 0; r < R; ++r) acc[r] = 0;
#pragma unroll
            for (int i = 0; i < BPW; ++i) {
                const int kb = wave + i * kGemvWaves;
                if (kb < KB) {
#pragma unroll
                    for (int r = 0; r < R; ++r) acc[r] = dot_block(wr[r * BPW + i], kb, acc[r]);
                }
            }
#pragma unroll
            for (int r = 0; r < R; ++r) reinterpret_cast<int*>(&part[(r * kGemvWaves + wave) * 32 + (lane & 31)])[half] = acc[r];
        } else {
#pragma unroll
            for (int i = 0; i < ITEMS; ++i) {
                const int item = wave + i * kGemvWaves;
                if (item < R * G) {
                    const int kb = (item % G) * 4 + kbi;
                    int acc = dot_block(wr[i], kb < KB ? kb : 0, 0);   // blocks past the end carry zero codes
                    acc += mmf_dpp<0x128>(acc);                      // row_ror:8 -> the other k-half
                    acc += __builtin_amdgcn_ds_swizzle(acc, 0x401F);   // xor 16 -> the neighbouring k-block
                    if ((lane & 31) < 8) reinterpret_cast<int*>(&part[item * 8 + (lane & 7)])[lane >> 5] = acc;
                }
            }
        }
        __syncthreads();
        if (epl) {
            int qtot = 0;
#pragma unroll
            for (int w = 0; w < kGemvWaves; ++w) qtot += red_q[w];
            float res[R];
#pragma unroll
            for (int r = 0; r < R; ++r) {
                int tot = 0;
                if constexpr (S == 1) {
#pragma unroll
                    for (int w = 0; w < kGemvWaves; ++w) {
                        const int2 pr = part[(r * kGemvWaves + w) * 32 + lane];
                        tot += pr.x + pr.y;
                    }
                } else {
#pragma unroll
                    for (int gi = 0; gi < GMAX; ++gi) {                 // compile-time bound: the reads are issued together
                        const int2 pr = part[(r * G + (gi < G ? gi : 0)) * 8 + lane];
                        tot += gi < G ? pr.x + pr.y : 0;
                    }
                }
                res[r] = __fmul_rn(__fmul_rn((float)(tot - qtot), deq), wdq[r]);
            }
            if constexpr (EPI == EPI_PLAIN) {
                float o = res[0];
                if (a.bias) o = __fadd_rn(o, bias_v);
                if (a.addend) o = __fadd_rn(mmf_round_to<T>(o), add_v);
                static_cast<T*>(a.out)[(int64_t)row * a.N + chc] = mmf_from_float<T>(o);
            } else if constexpr (EPI == EPI_STEP) {
                // res = raw i, f, g projections of channel ch (each rounded to T like the tensors they replace)
                const float iv = mmf_round_to<T>(res[0]), fv = mmf_round_to<T>(res[1]);
                float s = mmf_sigmoid(fv);
                if (a.lb) s = __fadd_rn(ep_lb, __fmul_rn(__fsub_rn(1.0f, ep_lb), s));
                const float go = mmf_round_to<T>(s);
                const float xo = mmf_round_to<T>(__fdiv_rn(__fmul_rn(iv, __fsub_rn(1.0f, go)), __fadd_rn(1.0f, mmf_exp(-iv))));
                const float h = __fadd_rn(__fmul_rn(go, ep_state), xo);
                a.state[(int64_t)row * Nseg + chc] = h;
                static_cast<T*>(a.out)[(int64_t)row * Nseg + chc] = mmf_from_float<T>(h);
                static_cast<T*>(a.g_out)[(int64_t)row * Nseg + chc] = mmf_from_float<T>(res[2]);
            } else {
                const float g = mmf_round_to<T>(res[0]), u = mmf_round_to<T>(res[1]);
                static_cast<T*>(a.out)[(int64_t)row * Nseg + chc] =
                    mmf_from_float<T>(__fdiv_rn(__fmul_rn(g, u), __fadd_rn(1.0f, mmf_exp(-g))));
            }
        }
    };
    if constexpr (!WALK) {
        contract(wreg, nb, ep_wdeq, ep_bias, ep_add);
    } else {
        // One n-block ahead: deeper (two blocks in flight through a ring of three register sets) measured 15 % slower.
        const int NBall = (a.N + 31) >> 5, stride = (int)gridDim.x;
        for (int nbc = nb; nbc < NBall; nbc += stride) {
            // the next block's weights and epilogue operands travel under this block's contraction
            const int nbn = nbc + stride < NBall ? nbc + stride : nbc;
            uint4 wnext[NWREG];
#pragma unroll
            for (int i = 0; i < BPW; ++i) {
                const int kb = wave + i * kGemvWaves;
                if (kb < KB) wnext[i] = a.packed[((int64_t)nbn * KB + kb) * 64 + lane];
            }
            float wdq_n[R], bias_n = 0.0f, add_n = 0.0f;
            const int chn = nbn * 32 + (lane & 31);
            wdq_n[0] = a.wdeq[(uint32_t)(nbn * 32) / (uint32_t)a.seg_rows];
            if (wave == 0 && lane < 32 && chn < a.N) {
                if (a.bias) bias_n = mmf_to_float(static_cast<const T*>(a.bias)[chn]);
                if (a.addend) add_n = mmf_to_float(static_cast<const T*>(a.addend)[(int64_t)row * a.N + chn]);
            }
            contract(wreg, nbc, ep_wdeq, ep_bias, ep_add);
            __syncthreads();                                    // part[] is free again
#pragma unroll
            for (int i = 0; i < NWREG; ++i) wreg[i] = wnext[i];
            ep_wdeq[0] = wdq_n[0]; ep_bias = bias_n; ep_add = add_n;
        }
    }
}

template <typename T, typename TW, int PRO, int EPI, int NW, int NV>
void launch_gemv_shape(const GemvArgs& a, dim3 grid, bool split, bool walk, hipStream_t s) {
    if constexpr (EPI == EPI_PLAIN) {
        if (walk) {
            bitlinear_gemv_kernel<T, TW, NW, NV, PRO, EPI, true, 1, true><<<grid, dim3(64 * NW), (size_t)a.Kp, s>>>(a);
            return;
        }
    }
    if (split) bitlinear_gemv_kernel<T, TW, NW, NV, PRO, EPI, true, 4><<<grid, dim3(64 * NW), (size_t)a.Kp, s>>>(a);
    else bitlinear_gemv_kernel<T, TW, NW, NV, PRO, EPI, true, 1><<<grid, dim3(64 * NW), (size_t)a.Kp, s>>>(a);
}

// Workgroups that a launch keeps resident at once on this build's target (256 CUs, 2048 threads each): the n-block walk
// sizes its grid to them.  MMF_GEMV_WALK_GRID overrides the per-launch total (0 = never walk): a measuring aid.
inline int gemv_walk_slots(int threads) {
    static const int env = [] {
        const char* e = getenv("MMF_GEMV_WALK_GRID");
        return e ? atoi(e) : -1;
    }();
    return env >= 0 ? env : 256 * (2048 / threads);
}

template <typename T, typename TW, int PRO, int EPI>
int launch_gemv(const GemvArgs& a, int64_t M, bool vec, hipStream_t s) {
    constexpr int R = EPI == EPI_STEP ? 3 : EPI == EPI_SWIGLU ? 2 : 1;
    const int64_t nblocks = mmf_ceil_div(a.N / R, 32);
    // few n-blocks (a 2048-row projection has 64): give each workgroup 8 rows, not 32, to reach every CU
    const bool split = vec && nblocks * M <= 64;             // at most 256 workgroups after the split: one per CU
    // waves per workgroup and passes over the row: the fewest passes, then the fewest waves, that cover K
    const int nw = a.Kp <= 2048 ? 8 : a.Kp <= 3072 ? 12 : a.Kp <= 4096 ? 16 : a.Kp <= 6144 ? 12 : 16;
    // many more n-blocks than resident workgroups (vocabulary-sized N): a grid of resident workgroups walks them
    const int64_t per_row = gemv_walk_slots(64 * nw) / M;
    const bool walk = vec && EPI == EPI_PLAIN && per_row >= 32 && nblocks > per_row;
    dim3 grid((unsigned)(walk ? per_row : nblocks * (split ? 4 : 1)), (unsigned)M);
    if (!vec) bitlinear_gemv_kernel<T, TW, 8, 4, PRO, EPI, false, 1><<<grid, dim3(512), (size_t)a.Kp, s>>>(a);   // ragged shapes: one generic build
    else if (a.Kp <= 2048) launch_gemv_shape<T, TW, PRO, EPI, 8, 1>(a, grid, split, walk, s);
    else if (a.Kp <= 3072) launch_gemv_shape<T, TW, PRO, EPI, 12, 1>(a, grid, split, walk, s);
    else if (a.Kp <= 4096) launch_gemv_shape<T, TW, PRO, EPI, 16, 1>(a, grid, split, walk, s);
    else if (a.Kp <= 6144) launch_gemv_shape<T, TW, PRO, EPI, 12, 2>(a, grid, split, walk, s);
    else launch_gemv_shape<T, TW, PRO, EPI, 16, 2>(a, grid, split, walk, s);
    MMF_CHECK_LAUNCH();
    return 0;
}

template <typename T, typename TW>
int dispatch_gemv_kind(const GemvArgs& a, int64_t M, int pro, int epi, bool vec, hipStream_t s) {
    // the combinations a decode step uses
    if (epi == EPI_PLAIN) {
        switch (pro) {
            case PRO_PLAIN: return launch_gemv<T, TW, PRO_PLAIN, EPI_PLAIN>(a, M, vec, s);
            case PRO_NORM: return launch_gemv<T, TW, PRO_NORM, EPI_PLAIN>(a, M, vec, s);
            case PRO_RESNORM: return launch_gemv<T, TW, PRO_RESNORM, EPI_PLAIN>(a, M, vec, s);
            case PRO_GATEDNORM: return launch_gemv<T, TW, PRO_GATEDNORM, EPI_PLAIN>(a, M, vec, s);
            case PRO_SWIGLU: return launch_gemv<T, TW, PRO_SWIGLU, EPI_PLAIN>(a, M, vec, s);
        }
    } else if (epi == EPI_STEP) {
        if (pro == PRO_NORM) return launch_gemv<T, TW, PRO_NORM, EPI_STEP>(a, M, vec, s);
        if (pro == PRO_PLAIN) return launch_gemv<T, TW, PRO_PLAIN, EPI_STEP>(a, M, vec, s);
    } else if (epi == EPI_SWIGLU) {
        if (pro == PRO_RESNORM) return launch_gemv<T, TW, PRO_RESNORM, EPI_SWIGLU>(a, M, vec, s);
        if (pro == PRO_PLAIN) return launch_gemv<T, TW, PRO_PLAIN, EPI_SWIGLU>(a, M, vec, s);
    }
    return MMF_ERR_ARG;
}

template <typename T>
int dispatch_gemv_w(const GemvArgs& a, int64_t M, int pro, int epi, int x_dtype, int w_dtype, bool vec, hipStream_t s) {
    if (w_dtype == MMF_F32) return dispatch_gemv_kind<T, float>(a, M, pro, epi, vec, s);
    if (w_dtype == x_dtype) return dispatch_gemv_kind<T, T>(a, M, pro, epi, vec, s);
    return MMF_ERR_ARG;
}

bool aligned(const void* p, size_t n) { return (reinterpret_cast<uintptr_t>(p) % n) == 0; }

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
    if (K > INT32_MAX - 128 || N > INT32_MAX - 96 || seg_rows > INT32_MAX) return MMF_ERR_WIDE;
    if (seg_rows % 32 != 0 && seg_rows < N) return MMF_ERR_ARG;   // stacked segments are whole n-blocks
    GemvArgs a{};
    a.x = x; a.aux = aux ? aux : x; a.res_out = res_out; a.w1 = w1; a.norm_w = norm_weight;
    a.packed = static_cast<const uint4*>(packed); a.wdeq = wdeq; a.bias = bias; a.addend = addend; a.out = out;
    a.g_out = g_out; a.lb = lower_bound; a.state = state;
    a.K = (int)K; a.Kp = (int)mmf_round_up(K, 128); a.N = (int)N; a.seg_rows = (int)seg_rows; a.ldx = ldx;
    a.ldaux = aux ? ldaux : ldx;
    a.eps = eps; a.eps1 = eps1; a.inv_K = 1.0 / (double)K;
    if (a.Kp > kGemvMaxK) return MMF_ERR_WIDE;
    if (!aligned(packed, 16)) return MMF_ERR_ALIGN;
    if (!norm_weight && !w1) weight_dtype = MMF_F32;
    const size_t xa = 4 * (x_dtype == MMF_F32 ? 4 : 2), wa = 4 * (weight_dtype == MMF_F32 ? 4 : 2);
    const bool vec = K % 4 == 0 && ldx % 4 == 0 && a.ldaux % 4 == 0;
    if (vec && !(aligned(x, xa) && aligned(a.aux, xa) && aligned(res_out, xa) && aligned(w1, wa) && aligned(norm_weight, wa)))
        return MMF_ERR_ALIGN;
    switch (x_dtype) {
        case MMF_F32: return dispatch_gemv_w<float>(a, M, prologue, epilogue, x_dtype, weight_dtype, vec, stream);
        case MMF_BF16: return dispatch_gemv_w<bf16_t>(a, M, prologue, epilogue, x_dtype, weight_dtype, vec, stream);
        case MMF_F16: return dispatch_gemv_w<f16_t>(a, M, prologue, epilogue, x_dtype, weight_dtype, vec, stream);
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
