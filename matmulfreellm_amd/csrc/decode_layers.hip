// One batch-1 decode step -- embedding row, all layers, final norm + lm_head, greedy argmax -- in ONE persistent launch.
//
// A decode step is a chain of 4 dependent fused BitLinears per layer (mmfreelm/models/hgrn_bit/
// modeling_hgrn_bit.py:97-109 around mmfreelm/layers/hgrn_bit.py:83-162): block norm -> i/f/g -> gate math +
// recurrence step; gated norm -> o_proj; residual + norm -> gate_proj -> swiglu; down_proj + residual.
// As separate launches each link costs a kernel boundary (about 1.3 us) plus a cold read of the
// previous link's output (about 1 us).  Here 256 workgroups stay resident and walk the 4L links
// ("phases") themselves.  Activations travel between workgroups as self-validating words: a 16-bit
// value in the high half, a 16-bit tag naming the producing phase in the low half, written and
// polled with relaxed device-scope accesses, so a consumer's poll is both the synchronisation and the
// data transfer and no fence or grid barrier is needed.  The arithmetic of every phase is
// that of bitlinear_gemv_kernel with the same prologue / epilogue, operation for operation.
// With a head record the launch goes on with final norm -> lm_head (each workgroup walks several 32-row blocks behind
// one prologue, writes plain logits and keeps its best candidate) and the greedy argmax (workgroup 0 combines the
// workgroups' candidates and writes the token the next launch embeds; mmfreelm/models/hgrn_bit/
// modeling_hgrn_bit.py:386 followed by the argmax of greedy decoding).
//
// Why a buffer is never rewritten under a reader: a workgroup stores a link's outputs only after it has polled that
// link's whole input, i.e. after every producer of the previous link has finished that link -- and a producer reads
// its inputs before it stores.  Every buffer is rewritten at the earliest two links after it was read (the residual
// stream alternates between two buffers), and the chain of polls between those links passes through every reader.
//
// Every wait is bounded: a poll gives up after `spin` rounds, raises the error word and carries on
// with whatever it read, so the grid always drains.  The host must make sure all 256 workgroups can
// be resident at once (one per CU) and checks the error word.
#include "mmf_common.h"

namespace {

constexpr int kNW = 8, kNT = 64 * kNW, kEl = 4;
constexpr int kWGs = 256;

enum Pro : int { PRO_PLAIN = 0, PRO_NORM = 1, PRO_RESNORM = 2, PRO_GATEDNORM = 3 };
enum Epi : int { EPI_PLAIN = 0, EPI_STEP = 1, EPI_SWIGLU = 2 };

struct Phase {                // one fused BitLinear; four per layer: i/f/g, o, gate, down
    const void* w1;           // weight of the norm in front of the BitLinear (null for down)
    const void* norm_w;       // the BitLinear's own norm weight
    const uint4* packed;
    const float* wdeq;
    const float* lb;          // i/f/g: lower bound [D] or null
    float* state;             // i/f/g: recurrent state [D] fp32
    double inv_K;
    float eps, eps1;
    int K, N, seg_rows, pad_;
};

struct LayersArgs {
    const Phase* phases;      // [4 * n_layers], device memory
    const void* table;        // embedding table [vocab, H]
    const int64_t* tok;       // the token to embed
    int64_t vocab;
    uint32_t* hb[2];          // tagged words: residual stream after a layer (ping-pong)
    uint32_t* ob;             //   recurrence output [D]
    uint32_t* gb;             //   raw g projection [D]
    uint32_t* ab;             //   attention output [H]
    uint32_t* rb;             //   summed residual [H]
    uint32_t* zb;             //   swiglu output [I]
    void* h_out;              // plain copy of the final residual stream [H]
    const Phase* head;        // final norm + lm_head (device record) or null: stop after the layers
    void* logits;             // head: plain logits [V]
    uint64_t* am_words;       // head: one (index | value | tag) record per workgroup
    int64_t* tok_out;         // head: the greedy token
    uint32_t* epoch;          // tag base; advanced by 4 * n_layers at the end of the launch
    int* err;                 // set to 1 when a poll ran out of rounds
    long long* trace;         // null, or kTraceWGs * kTraceLinks * kTraceStamps cycle stamps (see MMF_STAMP)
    int n_layers, H, D, I, spin;
};

// Optional cycle trace: thread 0 of three workgroups notes the shader clock at ten points of every link (entry, row
// arrived, block norm done, sum of squares, rstd, absmax, codes in LDS, dot done, partials met, epilogue done).
constexpr int kTraceWGs = 3, kTraceLinks = 128, kTraceStamps = 12;
#define MMF_STAMP(i)                                                                                              \
    do {                                                                                                          \
        if (a.trace && threadIdx.x == 0 && tr_link < kTraceLinks) {                                               \
            const int slot_ = blockIdx.x == 0 ? 0 : blockIdx.x == 37 ? 1 : blockIdx.x == 200 ? 2 : -1;            \
            if (slot_ >= 0) a.trace[(slot_ * kTraceLinks + tr_link) * kTraceStamps + (i)] = __builtin_amdgcn_s_memtime(); \
        }                                                                                                         \
    } while (0)

// A row as a phase reads it: plain elements (layer 0 reads the embedding row) or tagged words.
struct RowSrc {
    const void* plain;
    const uint32_t* words;
    uint32_t tag;
};

// Running greedy choice of one epilogue lane: lowest index of the largest value seen; NaNs never win.
struct Best {
    float v;
    uint32_t i;               // 0xffffffff: nothing yet
};
constexpr uint32_t kNone = 0xffffffffu;
__device__ __forceinline__ void best_take(Best& b, float v, uint32_t i) {
    if (i != kNone && (b.i == kNone || v > b.v || (v == b.v && i < b.i))) { b.v = v; b.i = i; }
}

struct Smem {
    int8_t q[4 * kNT * kEl];                  // int8 codes of the row (K <= 8192)
    double red_a[kNW], red_b[kNW];
    float red_f[kNW];
    int red_q[kNW];
    int2 part[3 * kNW * 32];                  // S = 1: [r][wave][row];  S = 4: [item][row8]
};

__device__ __forceinline__ uint64_t ll_ld8(const uint64_t* p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ uint32_t ll_ld4(const uint32_t* p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void ll_st8(uint64_t* p, uint64_t v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void ll_st4(uint32_t* p, uint32_t v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }

template <typename T> __device__ __forceinline__ float word_value(uint32_t w) {
    return mmf_to_float(mmf_from_bits16<T>((uint16_t)(w >> 16)));
}
template <typename T> __device__ __forceinline__ uint32_t make_word(float v, uint32_t tag) {
    return ((uint32_t)mmf_bits16(mmf_from_float<T>(v)) << 16) | tag;
}

// Four consecutive plain elements k0..k0+3 of a row (k0 a multiple of 4, k0 < K).
template <typename T>
__device__ __forceinline__ void plain_load4(const RowSrc& s, int k0, float (&out)[4]) {
    Raw4<T> r = raw4_load<T, true>(static_cast<const T*>(s.plain), k0, k0 + 4);
    raw4_unpack<T>(r, out);
}

// One word whose first read `w` was issued long before (at the start of the phase): usually it already carries the tag.
template <typename T>
__device__ __forceinline__ float word_finish1(uint32_t w, const uint32_t* p, uint32_t tag, int spin, int* err) {
    int n = 0;
    while ((w & 0xffffu) != tag && n++ < spin) w = ll_ld4(p);
    if ((w & 0xffffu) != tag) *err = 1;
    return word_value<T>(w);
}

// One phase.  NV passes over the row (K <= NV * 2048); S = 4: a virtual block owns 8 of an n-block's 32 rows.
// Virtual block vb -> (n-block vb / S, row group vb % S); a workgroup takes vb = blockIdx.x, + gridDim.x, ...
// The prologue (the row's int8 codes) is computed once per workgroup, whatever the number of virtual blocks.
// PF: the workgroup walks several virtual blocks (the lm_head link): request the next block's weights as soon as the
// dot of the current one has consumed its registers, so they travel under the epilogue.
template <typename T, int NV, int PRO, int EPI, int S, bool PF = false>
__device__ __forceinline__ void run_phase(const Phase& ph, const LayersArgs& a, Smem& sm, const RowSrc& xs, const RowSrc& auxs,
                                          const uint32_t* add_words, uint32_t add_tag, uint32_t* res_words,
                                          uint32_t* out_words, uint32_t* g_words, T* plain_out, uint32_t tag_out, int tr_link,
                                          Best* am = nullptr) {
    constexpr int R = EPI == EPI_STEP ? 3 : EPI == EPI_SWIGLU ? 2 : 1;
    constexpr int BPW = 2 * NV;
    constexpr int GMAX = NV * kNW / 2;
    constexpr int ITEMS = (R * GMAX + kNW - 1) / kNW;
    constexpr int CHN = 32 / S;
    constexpr bool HAS_AUX = PRO >= PRO_RESNORM;
    constexpr bool HAS_W1 = PRO >= PRO_NORM;
    constexpr int NWREG = S == 1 ? R * BPW : ITEMS;

    MMF_STAMP(0);
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int K = ph.K, KB = (K + 127) >> 7, Kp = KB << 7;
    const int Nseg = ph.N / R;
    const int NBseg = (Nseg + 31) >> 5;
    const int nvb = NBseg * S;
    if ((int)blockIdx.x >= nvb) return;                         // nothing of this phase falls to this workgroup
    const int G = (KB + 3) >> 2;
    const int kbi = lane >> 4, half = S == 1 ? lane >> 5 : (lane >> 3) & 1;

    // ---- loads that do not depend on the previous phase go first: norm weights, the first virtual block's
    // packed weights and epilogue operands.  They are in flight while the row is polled.
    const T* w1 = static_cast<const T*>(ph.w1);
    const T* nw = static_cast<const T*>(ph.norm_w);
    Raw4<T> w1raw[HAS_W1 ? NV : 1], nwraw[NV];
#pragma unroll
    for (int v = 0; v < NV; ++v) {
        const int k0 = (v * kNT + (int)threadIdx.x) * kEl;
        if constexpr (HAS_W1) w1raw[v] = raw4_load<T, true>(w1, k0, K);
        nwraw[v] = raw4_load<T, true>(nw, k0, K);
    }
    float ep_wdeq[R], ep_lb = 0.0f, ep_state = 0.0f;
    uint32_t ep_add = 0u;
    auto load_weights = [&](int vb, uint4 (&wreg)[NWREG]) {
        const int nb = vb / S, sub = vb % S;
        if constexpr (S == 1) {
#pragma unroll
            for (int r = 0; r < R; ++r)
#pragma unroll
                for (int i = 0; i < BPW; ++i) {
                    const int kb = wave + i * kNW;
                    if (kb < KB) wreg[r * BPW + i] = ph.packed[((int64_t)(nb + r * NBseg) * KB + kb) * 64 + lane];
                }
        } else {
#pragma unroll
            for (int i = 0; i < ITEMS; ++i) {
                const int item = wave + i * kNW;
                wreg[i] = make_uint4(0u, 0u, 0u, 0u);
                if (item < R * G) {
                    const int r = item / G, kb = (item % G) * 4 + kbi;
                    if (kb < KB)
                        wreg[i] = ph.packed[((int64_t)(nb + r * NBseg) * KB + kb) * 64 + half * 32 + sub * CHN + (lane & 7)];
                }
            }
        }
    };
    auto load_ep = [&](int vb) {
        const int nb = vb / S, sub = vb % S;
        if (wave == 0) {
#pragma unroll
            for (int r = 0; r < R; ++r) ep_wdeq[r] = ph.wdeq[(uint32_t)((nb + r * NBseg) * 32) / (uint32_t)ph.seg_rows];
            const int ch = nb * 32 + sub * CHN + (lane & (CHN - 1));
            if constexpr (EPI == EPI_STEP) {
                if (lane < (S == 4 ? 2 * CHN : CHN) && ch < Nseg) {   // S = 4: lanes 8..15 run the f rows of the same channels
                    if (ph.lb) ep_lb = ph.lb[ch];
                    ep_state = ph.state[ch];
                }
            }
            if constexpr (EPI == EPI_PLAIN) {
                if (add_words && lane < CHN && ch < Nseg) ep_add = ll_ld4(add_words + ch);   // checked (and re-read if early) in the epilogue
            }
        }
    };
    // PF: the weights of this workgroup's first four virtual blocks are requested now, together (one block in
    // flight at a time would stream them at a fraction of the CU's share of the bandwidth)
    constexpr int NPF = PF ? 4 : 1;
    uint4 wpf[NPF][NWREG];
#pragma unroll
    for (int j = 0; j < NPF; ++j)
        if ((int)blockIdx.x + j * (int)gridDim.x < nvb) load_weights((int)blockIdx.x + j * (int)gridDim.x, wpf[j]);
    load_ep((int)blockIdx.x);

    // ---- the row (and the prologue's second operand): poll until every word carries the producer's tag.  The first
    // read of every piece of both rows is issued before anything is examined, so an operand that was produced links
    // ago (the residual stream) costs no round trip of its own, and the passes over a wide row do not queue up.
    float xv[NV][4], av[HAS_AUX ? NV : 1][4];
    {
        uint64_t xw[NV][2], aw[HAS_AUX ? NV : 1][2];
        const bool x_tagged = xs.plain == nullptr, a_tagged = HAS_AUX && auxs.plain == nullptr;
        auto issue = [&](const RowSrc& src, int k0, uint64_t (&w)[2]) {
            const uint64_t* p = reinterpret_cast<const uint64_t*>(src.words + k0);
            w[0] = ll_ld8(p);
            w[1] = ll_ld8(p + 1);
        };
        auto valid = [&](const RowSrc& src, const uint64_t (&w)[2]) {
            const uint64_t want = ((uint64_t)src.tag << 32) | src.tag, mask = 0x0000ffff0000ffffull;
            return ((w[0] & mask) == want) && ((w[1] & mask) == want);
        };
        auto unpack = [&](const uint64_t (&w)[2], float (&out)[4]) {
            out[0] = word_value<T>((uint32_t)w[0]);
            out[1] = word_value<T>((uint32_t)(w[0] >> 32));
            out[2] = word_value<T>((uint32_t)w[1]);
            out[3] = word_value<T>((uint32_t)(w[1] >> 32));
        };
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            const int k0 = (v * kNT + (int)threadIdx.x) * kEl;
#pragma unroll
            for (int i = 0; i < 4; ++i) xv[v][i] = 0.0f;
            if constexpr (HAS_AUX) {
#pragma unroll
                for (int i = 0; i < 4; ++i) av[v][i] = 0.0f;
            }
            if (k0 < K) {
                if (x_tagged) issue(xs, k0, xw[v]);
                else plain_load4<T>(xs, k0, xv[v]);
                if constexpr (HAS_AUX) {
                    if (a_tagged) issue(auxs, k0, aw[v]);
                    else plain_load4<T>(auxs, k0, av[v]);
                }
            }
        }
        for (int n = 0;; ++n) {
            bool all = true;
#pragma unroll
            for (int v = 0; v < NV; ++v) {
                const int k0 = (v * kNT + (int)threadIdx.x) * kEl;
                if (k0 < K) {
                    if (x_tagged && !valid(xs, xw[v])) { all = false; issue(xs, k0, xw[v]); }
                    if constexpr (HAS_AUX) {
                        if (a_tagged && !valid(auxs, aw[v])) { all = false; issue(auxs, k0, aw[v]); }
                    }
                }
            }
            if (all) break;
            if (n >= a.spin) { *a.err = 1; break; }
        }
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            const int k0 = (v * kNT + (int)threadIdx.x) * kEl;
            if (k0 < K) {
                if (x_tagged) unpack(xw[v], xv[v]);
                if constexpr (HAS_AUX) {
                    if (a_tagged) unpack(aw[v], av[v]);
                }
            }
        }
    }

    MMF_STAMP(1);
    // ---- prologue stage 1
    if constexpr (PRO == PRO_RESNORM) {
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            const int k0 = (v * kNT + (int)threadIdx.x) * kEl;
            if (k0 < K) {
#pragma unroll
                for (int i = 0; i < 4; ++i) xv[v][i] = __fadd_rn(xv[v][i], av[v][i]);
                if (blockIdx.x == 0) {
                    uint64_t* p = reinterpret_cast<uint64_t*>(res_words + k0);
                    ll_st8(p, (uint64_t)make_word<T>(xv[v][0], tag_out) | ((uint64_t)make_word<T>(xv[v][1], tag_out) << 32));
                    ll_st8(p + 1, (uint64_t)make_word<T>(xv[v][2], tag_out) | ((uint64_t)make_word<T>(xv[v][3], tag_out) << 32));
                }
            }
        }
    }
    if constexpr (HAS_W1) {
        double s1 = 0.0;
#pragma unroll
        for (int v = 0; v < NV; ++v)
#pragma unroll
            for (int i = 0; i < 4; ++i) s1 = mmf_add_square(s1, xv[v][i]);
        s1 = mmf_block_sum_once<kNW>(s1, sm.red_a);
        const float rstd1 = mmf_rstd(s1, K, ph.inv_K, ph.eps1);
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            const int k0 = (v * kNT + (int)threadIdx.x) * kEl;
            float w1v[4];
            raw4_unpack<T>(w1raw[v], w1v);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                float y = __fmul_rn(__fmul_rn(xv[v][i], rstd1), w1v[i]);
                if constexpr (PRO == PRO_GATEDNORM) y = __fmul_rn(__fmul_rn(y, av[v][i]), mmf_sigmoid(av[v][i]));
                xv[v][i] = (k0 < K) ? mmf_round_to<T>(y) : 0.0f;
            }
        }
    }

    MMF_STAMP(2);
    // ---- prologue stage 2: the BitLinear's own norm, absmax int8 codes into LDS
    double ss = 0.0;
#pragma unroll
    for (int v = 0; v < NV; ++v)
#pragma unroll
        for (int i = 0; i < 4; ++i) ss = mmf_add_square(ss, xv[v][i]);
    ss = mmf_block_sum_once<kNW>(ss, sm.red_b);
    MMF_STAMP(3);
    const float rstd = mmf_rstd(ss, K, ph.inv_K, ph.eps);
    MMF_STAMP(4);
    float amax = 0.0f;
#pragma unroll
    for (int v = 0; v < NV; ++v) {
        float wv[4];
        raw4_unpack<T>(nwraw[v], wv);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float y = __fmul_rn(__fmul_rn(xv[v][i], rstd), wv[i]);
            xv[v][i] = y;
            amax = fmaxf(amax, fabsf(y));
        }
    }
    amax = mmf_block_max_once<kNW>(amax, sm.red_f);
    MMF_STAMP(5);
    const float scale = __fdiv_rn(127.0f, fmaxf(amax, 1e-5f));
    const float deq = __fdiv_rn(1.0f, scale);                 // needed by the epilogue only: computed here, in the shadow of the barriers
    int qs = 0;
#pragma unroll
    for (int v = 0; v < NV; ++v) {
        const int k0 = (v * kNT + (int)threadIdx.x) * kEl;
        if (k0 < Kp) {
            uint32_t packed4 = 0;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int c = (k0 < K) ? mmf_code(xv[v][i], scale) : 0;
                qs += c;
                packed4 |= (uint32_t)(c & 0xff) << (8 * i);
            }
            *reinterpret_cast<uint32_t*>(sm.q + k0) = packed4;
        }
    }
    __syncthreads();
    MMF_STAMP(6);
    qs = mmf_wave_sum(qs);
    if (lane == 0) sm.red_q[wave] = qs;

    auto dot_block = [&](const uint4& wq, int kb, int acc) { return mmf_dot_block(sm.q, wq, kb, half, acc); };

    auto process = [&](int vb, const uint4 (&wreg)[NWREG]) {
        const int nb = vb / S, sub = vb % S;
        if constexpr (S == 1) {
            int acc[R];
#pragma unroll
            for (int r = 0; r < R; ++r) acc[r] = 0;
#pragma unroll
            for (int i = 0; i < BPW; ++i) {
                const int kb = wave + i * kNW;
                if (kb < KB) {
#pragma unroll
                    for (int r = 0; r < R; ++r) acc[r] = dot_block(wreg[r * BPW + i], kb, acc[r]);
                }
            }
#pragma unroll
            for (int r = 0; r < R; ++r) reinterpret_cast<int*>(&sm.part[(r * kNW + wave) * 32 + (lane & 31)])[half] = acc[r];
        } else {
#pragma unroll
            for (int i = 0; i < ITEMS; ++i) {
                const int item = wave + i * kNW;
                if (item < R * G) {
                    const int kb = (item % G) * 4 + kbi;
                    int acc = dot_block(wreg[i], kb < KB ? kb : 0, 0);
                    acc += mmf_dpp<0x128>(acc);
                    acc += __builtin_amdgcn_ds_swizzle(acc, 0x401F);
                    if ((lane & 31) < 8) reinterpret_cast<int*>(&sm.part[item * 8 + (lane & 7)])[lane >> 5] = acc;
                }
            }
        }
        MMF_STAMP(7);
        __syncthreads();
        MMF_STAMP(8);
        const int ch = nb * 32 + sub * CHN + (lane & (CHN - 1));
        if constexpr (EPI == EPI_STEP && S == 4) {
            // Lanes 0-7 take the i rows, 8-15 the f rows, 16-23 the g rows of the same 8 channels, so the two exp /
            // divide chains of the gate math run side by side instead of one after the other.  Every lane executes
            // the same instructions (1 + exp(-v), then its reciprocal); the f lanes' gate reaches the i lanes by a
            // rotate within the 16-lane row.  Operation for operation the arithmetic of the single-lane form.
            if (wave == 0 && lane < 24) {
                const int r3 = lane >> 3;
                int qtot = 0;
#pragma unroll
                for (int w = 0; w < kNW; ++w) qtot += sm.red_q[w];
                int tot = 0;
#pragma unroll
                for (int gi = 0; gi < GMAX; ++gi) {                 // compile-time bound: the reads are issued together
                    const int2 pr = sm.part[(r3 * G + (gi < G ? gi : 0)) * 8 + (lane & 7)];
                    tot += gi < G ? pr.x + pr.y : 0;
                }
                const float wd = r3 == 0 ? ep_wdeq[0] : r3 == 1 ? ep_wdeq[1] : ep_wdeq[2];
                const float res = __fmul_rn(__fmul_rn((float)(tot - qtot), deq), wd);
                const float v16 = mmf_round_to<T>(res);                       // iv on the i lanes, fv on the f lanes
                const float ex = __fadd_rn(1.0f, mmf_exp(-v16));
                float sg = __fdiv_rn(1.0f, ex);                               // sigmoid(fv) on the f lanes
                if (ph.lb) sg = __fadd_rn(ep_lb, __fmul_rn(__fsub_rn(1.0f, ep_lb), sg));
                const float go = mmf_dpp<0x128>(mmf_round_to<T>(sg));         // lanes 0-7 read lanes 8-15
                const float xo = mmf_round_to<T>(__fdiv_rn(__fmul_rn(v16, __fsub_rn(1.0f, go)), ex));
                const float h = __fadd_rn(__fmul_rn(go, ep_state), xo);
                if (ch < Nseg) {
                    if (r3 == 0) {
                        ph.state[ch] = h;
                        ll_st4(out_words + ch, make_word<T>(h, tag_out));
                    } else if (r3 == 2) {
                        ll_st4(g_words + ch, make_word<T>(res, tag_out));
                    }
                }
            }
        } else if (wave == 0 && lane < CHN && ch < Nseg) {
            int qtot = 0;
#pragma unroll
            for (int w = 0; w < kNW; ++w) qtot += sm.red_q[w];
            float res[R];
#pragma unroll
            for (int r = 0; r < R; ++r) {
                int tot = 0;
                if constexpr (S == 1) {
#pragma unroll
                    for (int w = 0; w < kNW; ++w) {
                        const int2 pr = sm.part[(r * kNW + w) * 32 + lane];
                        tot += pr.x + pr.y;
                    }
                } else {
#pragma unroll
                    for (int gi = 0; gi < GMAX; ++gi) {             // compile-time bound: the reads are issued together
                        const int2 pr = sm.part[(r * G + (gi < G ? gi : 0)) * 8 + lane];
                        tot += gi < G ? pr.x + pr.y : 0;
                    }
                }
                res[r] = __fmul_rn(__fmul_rn((float)(tot - qtot), deq), ep_wdeq[r]);
            }
            if constexpr (EPI == EPI_PLAIN) {
                float o = res[0];
                if (add_words) o = __fadd_rn(mmf_round_to<T>(o), word_finish1<T>(ep_add, add_words + ch, add_tag, a.spin, a.err));
                if (out_words) ll_st4(out_words + ch, make_word<T>(o, tag_out));
                if (plain_out) plain_out[ch] = mmf_from_float<T>(o);
                if (am) {
                    const float ov = mmf_round_to<T>(o);
                    if (ov == ov) best_take(*am, ov, (uint32_t)ch);
                }
            } else if constexpr (EPI == EPI_STEP) {
                const float iv = mmf_round_to<T>(res[0]), fv = mmf_round_to<T>(res[1]);
                float s = mmf_sigmoid(fv);
                if (ph.lb) s = __fadd_rn(ep_lb, __fmul_rn(__fsub_rn(1.0f, ep_lb), s));
                const float go = mmf_round_to<T>(s);
                const float xo = mmf_round_to<T>(__fdiv_rn(__fmul_rn(iv, __fsub_rn(1.0f, go)), __fadd_rn(1.0f, mmf_exp(-iv))));
                const float h = __fadd_rn(__fmul_rn(go, ep_state), xo);
                ph.state[ch] = h;
                ll_st4(out_words + ch, make_word<T>(h, tag_out));
                ll_st4(g_words + ch, make_word<T>(res[2], tag_out));
            } else {
                const float g = mmf_round_to<T>(res[0]), u = mmf_round_to<T>(res[1]);
                ll_st4(out_words + ch, make_word<T>(__fdiv_rn(__fmul_rn(g, u), __fadd_rn(1.0f, mmf_exp(-g))), tag_out));
            }
        }
        MMF_STAMP(9);
        __syncthreads();                                        // part[] and the wave-0 registers are reused by the next block
    };
#pragma unroll
    for (int j = 0; j < NPF; ++j) {
        const int vb = (int)blockIdx.x + j * (int)gridDim.x;
        if (vb < nvb) {
            if (j > 0) load_ep(vb);
            process(vb, wpf[j]);
        }
    }
    for (int vb = (int)blockIdx.x + NPF * (int)gridDim.x; vb < nvb; vb += (int)gridDim.x) {
        load_weights(vb, wpf[0]);
        load_ep(vb);
        process(vb, wpf[0]);
    }
}

// NVH / NVI: passes over a row of width H (= D) / I.  A phase takes 8-row virtual blocks when that still leaves at
// most one per workgroup.
template <typename T, int NVH, int NVI>
__global__ __launch_bounds__(kNT) void decode_layers_kernel(LayersArgs a) {
    __shared__ Smem sm;
    const uint32_t e = *a.epoch;
    int64_t id = *a.tok;
    if (id < 0 || id >= a.vocab) id = 0;
    const T* emb_row = static_cast<const T*>(a.table) + id * a.H;
    auto tag_of = [&](int gp) { return (e + (uint32_t)gp + 1u) & 0xffffu; };
    for (int l = 0; l < a.n_layers; ++l) {
        const Phase* ph = a.phases + 4 * l;
        const RowSrc h_in = l == 0 ? RowSrc{emb_row, nullptr, 0u} : RowSrc{nullptr, a.hb[(l - 1) & 1], tag_of(4 * (l - 1) + 3)};
        const RowSrc none{nullptr, nullptr, 0u};
        const bool last = l == a.n_layers - 1;
        // i/f/g: block norm -> stacked projection -> gate math + recurrence step
        {
            const Phase p = ph[0];
            if ((p.N / 3 + 31) / 32 <= 64)
                run_phase<T, NVH, PRO_NORM, EPI_STEP, 4>(p, a, sm, h_in, none, nullptr, 0u, nullptr, a.ob, a.gb, nullptr, tag_of(4 * l), 4 * l);
            else
                run_phase<T, NVH, PRO_NORM, EPI_STEP, 1>(p, a, sm, h_in, none, nullptr, 0u, nullptr, a.ob, a.gb, nullptr, tag_of(4 * l), 4 * l);
        }
        // gated norm -> o_proj
        {
            const Phase p = ph[1];
            const RowSrc g_in{nullptr, a.gb, tag_of(4 * l)}, o_in{nullptr, a.ob, tag_of(4 * l)};
            if ((p.N + 31) / 32 <= 64)
                run_phase<T, NVH, PRO_GATEDNORM, EPI_PLAIN, 4>(p, a, sm, g_in, o_in, nullptr, 0u, nullptr, a.ab, nullptr, nullptr, tag_of(4 * l + 1), 4 * l + 1);
            else
                run_phase<T, NVH, PRO_GATEDNORM, EPI_PLAIN, 1>(p, a, sm, g_in, o_in, nullptr, 0u, nullptr, a.ab, nullptr, nullptr, tag_of(4 * l + 1), 4 * l + 1);
        }
        // residual + norm -> gate_proj -> swiglu
        {
            const Phase p = ph[2];
            const RowSrc a_in{nullptr, a.ab, tag_of(4 * l + 1)};
            if ((p.N / 2 + 31) / 32 <= 64)
                run_phase<T, NVH, PRO_RESNORM, EPI_SWIGLU, 4>(p, a, sm, a_in, h_in, nullptr, 0u, a.rb, a.zb, nullptr, nullptr, tag_of(4 * l + 2), 4 * l + 2);
            else
                run_phase<T, NVH, PRO_RESNORM, EPI_SWIGLU, 1>(p, a, sm, a_in, h_in, nullptr, 0u, a.rb, a.zb, nullptr, nullptr, tag_of(4 * l + 2), 4 * l + 2);
        }
        // down_proj + residual
        {
            const Phase p = ph[3];
            const RowSrc z_in{nullptr, a.zb, tag_of(4 * l + 2)};
            T* plain = last ? static_cast<T*>(a.h_out) : nullptr;
            if ((p.N + 31) / 32 <= 64)
                run_phase<T, NVI, PRO_PLAIN, EPI_PLAIN, 4>(p, a, sm, z_in, none, a.rb, tag_of(4 * l + 2), nullptr, a.hb[l & 1], nullptr, plain, tag_of(4 * l + 3), 4 * l + 3);
            else
                run_phase<T, NVI, PRO_PLAIN, EPI_PLAIN, 1>(p, a, sm, z_in, none, a.rb, tag_of(4 * l + 2), nullptr, a.hb[l & 1], nullptr, plain, tag_of(4 * l + 3), 4 * l + 3);
        }
    }
    if (a.head) {
        // final norm -> lm_head: plain logits, and this workgroup's candidate for the greedy token
        const int L = a.n_layers;
        const Phase p = *a.head;
        const RowSrc h_last{nullptr, a.hb[(L - 1) & 1], tag_of(4 * (L - 1) + 3)}, none{nullptr, nullptr, 0u};
        const uint32_t tag_h = tag_of(4 * L);
        Best best{0.0f, kNone};
        run_phase<T, NVH, PRO_NORM, EPI_PLAIN, 1, true>(p, a, sm, h_last, none, nullptr, 0u, nullptr, nullptr, nullptr,
                                                  static_cast<T*>(a.logits), tag_h, 4 * L, &best);
        const int lane = threadIdx.x & 63;
        if (threadIdx.x < 64) {                                  // wave 0 holds the candidates of its 32 epilogue lanes
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) {
                const float ov = __shfl_xor(best.v, o, 64);
                const uint32_t oi = (uint32_t)__shfl_xor((int)best.i, o, 64);
                best_take(best, ov, oi);
            }
            if (lane == 0)
                ll_st8(a.am_words + blockIdx.x, ((uint64_t)best.i << 32) | (uint64_t)make_word<T>(best.i == kNone ? 0.0f : best.v, tag_h));
        }
        if (blockIdx.x == 0) {
            // the greedy token: lowest index of the largest logit over the workgroups' candidates
            __syncthreads();                                    // run_phase is done with the shared arrays
            Best b{0.0f, kNone};
            if (threadIdx.x < gridDim.x) {
                uint64_t w;
                int n = 0;
                do { w = ll_ld8(a.am_words + threadIdx.x); } while (((uint32_t)w & 0xffffu) != tag_h && ++n < a.spin);
                if (((uint32_t)w & 0xffffu) != tag_h) *a.err = 1;
                b.i = (uint32_t)(w >> 32);
                b.v = word_value<T>((uint32_t)w);
            }
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) {
                const float ov = __shfl_xor(b.v, o, 64);
                const uint32_t oi = (uint32_t)__shfl_xor((int)b.i, o, 64);
                best_take(b, ov, oi);
            }
            if (lane == 0) { sm.red_f[threadIdx.x >> 6] = b.v; sm.red_q[threadIdx.x >> 6] = (int)b.i; }
            __syncthreads();
            if (threadIdx.x == 0) {
                for (int w = 1; w < kNW; ++w) best_take(b, sm.red_f[w], (uint32_t)sm.red_q[w]);
                *a.tok_out = b.i == kNone ? 0 : (int64_t)b.i;
            }
        }
    }
    // Every workgroup read the tag base (and the token) before any workgroup could get here (the last link's inputs
    // depend, through the chain, on an output of every workgroup that takes part), so the next launch's base can be
    // published now.
    if (blockIdx.x == 0 && threadIdx.x == 0) *a.epoch = e + 4u * (uint32_t)a.n_layers + 2u;
}

template <typename T>
int launch_layers(const LayersArgs& a, hipStream_t s) {
    const int nvh = (int)mmf_ceil_div(a.H > a.D ? a.H : a.D, 2048), nvi = (int)mmf_ceil_div(a.I, 2048);
    if (nvh == 1 && nvi <= 3) decode_layers_kernel<T, 1, 3><<<kWGs, kNT, 0, s>>>(a);
    else if (nvh <= 2 && nvi <= 4) decode_layers_kernel<T, 2, 4><<<kWGs, kNT, 0, s>>>(a);
    else return MMF_ERR_WIDE;
    MMF_CHECK_LAUNCH();
    return 0;
}

}  // namespace

extern "C" {

int mmf_decode_layers_phase_bytes(void) { return (int)sizeof(Phase); }

int mmf_decode_layers_trace_words(void) { return kTraceWGs * kTraceLinks * kTraceStamps; }

int mmf_decode_layers(const void* phases, int n_layers, const void* table, const int64_t* tok, int64_t vocab,
                      uint32_t* h0, uint32_t* h1, uint32_t* o, uint32_t* g, uint32_t* attn, uint32_t* res, uint32_t* z,
                      void* h_out, const void* head, void* logits, uint64_t* am_words, int64_t* tok_out, uint32_t* epoch, int* err,
                      int64_t* trace, int H, int D, int I, int spin, int dtype, void* stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (!phases || n_layers <= 0 || !table || !tok || vocab <= 0 || !h0 || !h1 || !o || !g || !attn || !res || !z || !h_out ||
        !epoch || !err || H <= 0 || D <= 0 || I <= 0 || spin <= 0)
        return MMF_ERR_ARG;
    if (head && (!logits || !am_words || !tok_out)) return MMF_ERR_ARG;
    if (H % 128 != 0 || D != H || I % 128 != 0) return MMF_ERR_ARG;      // rows are whole k-blocks: no ragged tail in a phase
    if (dtype != MMF_BF16 && dtype != MMF_F16) return MMF_ERR_ARG;        // a tagged word carries a 16-bit value
    if (H > 4096 || I > 8192) return MMF_ERR_WIDE;                        // at most two passes over an H-wide row, four over an I-wide one
    for (const void* p : {(const void*)h0, (const void*)h1, (const void*)o, (const void*)g, (const void*)attn, (const void*)res,
                          (const void*)z, (const void*)table, (const void*)h_out})
        if (reinterpret_cast<uintptr_t>(p) & 15u) return MMF_ERR_ALIGN;
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess)
        return MMF_ERR_ARG;
    if (cus < kWGs) return MMF_ERR_ARG;                                       // the resident grid needs one CU per workgroup
    LayersArgs a{};
    a.phases = static_cast<const Phase*>(phases); a.n_layers = n_layers; a.table = table; a.tok = tok; a.vocab = vocab;
    a.hb[0] = h0; a.hb[1] = h1; a.ob = o; a.gb = g; a.ab = attn; a.rb = res; a.zb = z; a.h_out = h_out; a.head = static_cast<const Phase*>(head); a.logits = logits; a.am_words = am_words; a.tok_out = tok_out;
    a.epoch = epoch;
    a.err = err; a.trace = reinterpret_cast<long long*>(trace); a.H = H; a.D = D; a.I = I; a.spin = spin;
    switch (dtype) {
        case MMF_BF16: return launch_layers<bf16_t>(a, stream);
        case MMF_F16: return launch_layers<f16_t>(a, stream);
    }
    return MMF_ERR_ARG;
}

}  // extern "C"
