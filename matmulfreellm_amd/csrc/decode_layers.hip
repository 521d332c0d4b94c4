// One batch-1 decode step -- embedding row, all layers, final norm + lm_head, greedy argmax -- in ONE persistent launch.
//
// A decode step is a chain of 4 dependent fused BitLinears per layer (mmfreelm/models/hgrn_bit/
// modeling_hgrn_bit.py:97-109 around mmfreelm/layers/hgrn_bit.py:83-162): block norm -> i/f/g -> gate math +
// recurrence step; gated norm -> o_proj; residual + norm -> gate_proj -> swiglu; down_proj + residual.
// 256 workgroups of 4 waves stay resident (one per CU, one wave per SIMD) and walk the 4L links themselves.
//
// Hand-off.  Activations travel between workgroups as self-validating 32-bit words: a 16-bit value in the high half,
// a 16-bit tag naming the producing link in the low half.  A producer stores its words to 8 replicas of the row (one
// per XCD: a row polled by 256 workgroups at once is a hot spot in the memory-side cache, 32 pollers per copy are
// not); a consumer polls the copy of its XCD with 16-byte device-coherent loads until every word carries the tag.
// The poll is both the synchronisation and the transfer: no fence, no grid barrier.  The first poll of a link is
// held back a little so that it reaches memory after the producers' stores rather than just before them (a poll that
// comes back stale costs a whole round trip).
//
// Body of a link.  A wave owns a contiguous slice of the row's k-blocks from the poll to the dot products: it polls
// that slice, takes part in the row statistics (per-wave partial -> LDS -> barrier: sum of squares of the block norm,
// sum of squares of the BitLinear's own norm, absmax), quantises its slice into LDS and multiplies it with its slice
// of the packed weights -- the codes never cross waves, so no barrier sits between quantiser and dot.  The per-wave
// partial dot products meet in LDS for the epilogue (one more barrier).  A workgroup owns row-groups of 8 output rows
// (row-group g of a segment belongs to workgroup g mod 256); 16 lanes = (2 halves x 8 rows) read the 2-bit weights of
// one k-block, so a wave load covers 4 k-blocks.  The packed weights, norm weights and epilogue operands of link n+1
// are requested as soon as link n's row has arrived, so they stream from HBM under link n's arithmetic and the
// hand-off (loads return in order: requested before the poll they would delay it).
//
// The arithmetic of every link is that of bitlinear_gemv_kernel with the same prologue / epilogue, operation for
// operation (sums of squares in fp64 are order-insensitive to rounding, integer sums exact).
//
// With a head record the launch goes on with final norm -> lm_head (plain logits; each workgroup keeps its best
// candidate) and the greedy argmax (workgroup 0 combines the candidates and writes the token the next launch embeds;
// mmfreelm/models/hgrn_bit/modeling_hgrn_bit.py:386 followed by the argmax of greedy decoding).
//
// Why a buffer is never rewritten under a reader: a workgroup stores a link's outputs only after it has polled that
// link's whole input, i.e. after every producer of the previous link has finished that link -- and a producer reads
// its inputs before it stores.  Every buffer is rewritten at the earliest two links after it was last read (the
// residual stream alternates between two buffers), and the chain of polls between those links passes through every
// reader.
//
// Every wait is bounded: a poll gives up after `spin` rounds, raises the error word and carries on with whatever it
// read, so the grid always drains.  The host must make sure all 256 workgroups can be resident at once and checks the
// error word.
#include "mmf_common.h"
#include <stdlib.h>

namespace {

constexpr int kNW = 4, kNT = 64 * kNW;
constexpr int kWGs = 256, kRep = 8;
constexpr int kHeadChunk = 16;                 // row-groups of the lm_head a workgroup takes per pass

#define MMF_AS_GLOBAL __attribute__((address_space(1)))
#define MMF_AS_CONST __attribute__((address_space(4)))

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
    const Phase* phases;      // [4 * n_layers], device memory, not written during the launch
    const void* table;        // embedding table [vocab, H]
    const int64_t* tok;       // the token to embed
    int64_t vocab;
    uint32_t* words;          // tagged words, kRep copies each: h0 [H], h1 [H], o [D], g [D], attn [H], z [I]
    void* h_out;              // plain copy of the final residual stream [H]
    const Phase* head;        // final norm + lm_head (device record) or null: stop after the layers
    void* logits;             // head: plain logits [V]
    uint64_t* am_words;       // head: one (index | value | tag) record per workgroup
    int64_t* tok_out;         // head: the greedy token
    uint32_t* epoch;          // tag base; advanced by 4 * n_layers + 2 at the end of the launch
    int* err;                 // set to 1 when a poll ran out of rounds
    long long* trace;         // TRACE builds: kTraceWGs * kTraceLinks * kTraceStamps cycle stamps
    int n_layers, H, D, I, spin, delay;
};

constexpr int kTraceWGs = 3, kTraceLinks = 128, kTraceStamps = 12;

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// Loads through the global address space (pointers read from the phase table are generic to the compiler; these keep
// the accesses off the flat path).  Builtin vector types only: they can be read from any address space.
__device__ __forceinline__ uint4 gload16(const void* base, uint32_t byte_off) {
    const u32x4 v = *reinterpret_cast<const MMF_AS_GLOBAL u32x4*>((const MMF_AS_GLOBAL char*)(base) + byte_off);
    return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ uint2 gload8(const void* base, uint32_t byte_off) {
    const u32x2 v = *reinterpret_cast<const MMF_AS_GLOBAL u32x2*>((const MMF_AS_GLOBAL char*)(base) + byte_off);
    return make_uint2(v.x, v.y);
}
__device__ __forceinline__ float gloadf(const void* base, int i) { return ((const MMF_AS_GLOBAL float*)base)[i]; }
__device__ __forceinline__ uint16_t gload2(const void* base, int i) { return ((const MMF_AS_GLOBAL uint16_t*)base)[i]; }

enum Pro : int { PRO_PLAIN = 0, PRO_NORM = 1, PRO_RESNORM = 2, PRO_GATEDNORM = 3 };
enum Epi : int { EPI_PLAIN = 0, EPI_STEP = 1, EPI_SWIGLU = 2, EPI_HEAD = 3 };

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
    int8_t q[8192];                          // int8 codes of the row; a wave reads and writes its own slice only
    double sum1[kNW], sum2[kNW];             // per-wave partial sums of squares
    float amax[kNW];
    int qs[kNW];                             // per-wave sums of codes
    int part[kHeadChunk][8][2 * kNW];        // [row-group x segment][row][wave x lane half] partial dot products
    float best_v[kNW];
    uint32_t best_i[kNW];
};

__device__ __forceinline__ uint64_t ll_ld8(const uint64_t* p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void ll_st8(uint64_t* p, uint64_t v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }

// Four tagged words as two 8-byte device-coherent loads (relaxed atomics: the compiler keeps track of them, so a whole
// row's loads are in flight before the one wait it inserts in front of the first tag test).
__device__ __forceinline__ u32x4 poll_issue(const uint32_t* p) {
    const uint64_t* q = reinterpret_cast<const uint64_t*>(p);
    const uint64_t lo = ll_ld8(q), hi = ll_ld8(q + 1);
    u32x4 r;
    r.x = (uint32_t)lo; r.y = (uint32_t)(lo >> 32); r.z = (uint32_t)hi; r.w = (uint32_t)(hi >> 32);
    return r;
}
__device__ __forceinline__ bool words_valid(const u32x4& w, uint32_t tag) {
    return ((w.x & 0xffffu) == tag) & ((w.y & 0xffffu) == tag) & ((w.z & 0xffffu) == tag) & ((w.w & 0xffffu) == tag);
}
template <typename T> __device__ __forceinline__ float word_value(uint32_t w) {
    return mmf_to_float(mmf_from_bits16<T>((uint16_t)(w >> 16)));
}
template <typename T> __device__ __forceinline__ uint32_t make_word(float v, uint32_t tag) {
    return ((uint32_t)mmf_bits16(mmf_from_float<T>(v)) << 16) | tag;
}

// A row as a link reads it: plain 16-bit elements (layer 0 reads the embedding row) or tagged words of this XCD's copy.
struct RowSrc {
    const void* plain;
    const uint32_t* words;
    uint32_t tag;
};

// Geometry of a link for this wave and workgroup (all wave-uniform).
struct Geo {
    int K, KB, kb0, nkb, nq;                 // row width, its k-blocks, this wave's slice [kb0, kb0 + nkb), k-quads per item
    int Nseg, NBseg, RG, NG;                 // rows / n-blocks / row-groups per segment, row-groups of this workgroup
};
template <int R>
__device__ __forceinline__ Geo make_geo(int K, int N, int wave) {
    Geo g;
    g.K = K;
    g.KB = K >> 7;
    const int kbw = (g.KB + kNW - 1) / kNW;
    g.kb0 = wave * kbw;
    g.nkb = g.KB - g.kb0 < 0 ? 0 : (g.KB - g.kb0 < kbw ? g.KB - g.kb0 : kbw);
    if (g.nkb == 0) g.kb0 = 0;
    g.nq = (kbw + 3) >> 2;
    g.Nseg = N / R;
    g.NBseg = (g.Nseg + 31) >> 5;
    g.RG = (g.Nseg + 7) >> 3;
    g.NG = g.RG > (int)blockIdx.x ? (g.RG - (int)blockIdx.x + kWGs - 1) / kWGs : 0;
    return g;
}

// Everything a link needs that does not depend on the link before it: requested one link ahead.
template <typename T, int NP, int MAXLD, int R, int NGE = 1>
struct Pre {
    uint4 w[MAXLD];                          // packed weights: load j = (row-group, segment, k-quad), 4 k-blocks x 16 lanes
    Raw4<T> w1raw[NP], nwraw[NP];            // norm weights of this wave's slice
    float wdeq[R];
    float lb[NGE], state[NGE];               // i/f/g epilogue: lower bound and recurrent state of this lane's channel, per row-group
                                             // (read here, before any wave's epilogue writes the new state)
    uint32_t add0, add1;                     // down epilogue: the two operands of the residual (tagged words or plain)
};

// The weights of row-groups [g0, g0 + ng) of this workgroup (at most MAXLD loads; the rest is left alone).
template <int R, int MAXLD>
__device__ __forceinline__ void load_weights(const Phase& ph, const Geo& g, int g0, int ng, int lane, uint4 (&w)[MAXLD]) {
    if (g.nkb == 0) return;
    const int slot = lane >> 4;
    const uint32_t lane_off = (uint32_t)(((lane >> 3) & 1) * 512 + (lane & 7) * 16);
    int gi = 0, r = 0, q = 0;
#pragma unroll
    for (int j = 0; j < MAXLD; ++j) {
        if (gi < ng) {
            const int rg = (int)blockIdx.x + kWGs * (g0 + gi);
            const int nb = (rg >> 2) + r * g.NBseg;
            const uint32_t s_off = (uint32_t)(nb * g.KB + g.kb0) * 1024u + (uint32_t)(rg & 3) * 128u;
            int kbl = 4 * q + slot;
            kbl = kbl < g.nkb ? kbl : g.nkb - 1;
            w[j] = gload16(ph.packed, s_off + (uint32_t)kbl * 1024u + lane_off);
        }
        if (++q == g.nq) { q = 0; if (++r == R) { r = 0; ++gi; } }
    }
}

// Element index (within the row) of the first of the four elements lane `lane` holds in pass v of this wave's slice.
__device__ __forceinline__ int slice_elem(const Geo& g, int v, int lane) { return g.kb0 * 128 + 4 * (64 * v + lane); }
__device__ __forceinline__ bool slice_has(const Geo& g, int v, int lane) { return 4 * (64 * v + lane) < g.nkb * 128; }

template <typename T, int NP>
__device__ __forceinline__ void load_norm_weights(const void* wp, const Geo& g, int lane, Raw4<T> (&raw)[NP]) {
    static_assert(sizeof(T) == 2, "16-bit activations");
#pragma unroll
    for (int v = 0; v < NP; ++v) {
        const int k0 = slice_has(g, v, lane) ? slice_elem(g, v, lane) : 0;
        raw[v].v = gload8(wp, (uint32_t)k0 * 2u);
    }
}

template <typename T, int NPH, int NPI, int NQH, int NQI, int NGH, int NGI, bool TRACE>
struct Chain {
    // loads per wave and link kind
    static constexpr int LD_IFG = NGH * 3 * NQH, LD_O = NGH * NQH, LD_GATE = NGI * 2 * NQH, LD_DOWN = NGH * NQI,
                         LD_HEAD = kHeadChunk * NQH;
    using PreIfg = Pre<T, NPH, LD_IFG, 3, NGH>;
    using PreO = Pre<T, NPH, LD_O, 1>;
    using PreGate = Pre<T, NPH, LD_GATE, 2>;
    using PreDown = Pre<T, NPI, LD_DOWN, 1>;
    using PreHead = Pre<T, NPH, LD_HEAD, 1>;

    const LayersArgs& a;
    Smem& sm;
    const int lane, wave;
    const uint32_t e;
    uint32_t* const hb0;                      // bases of the word buffers (copy 0)
    uint32_t* const hb1;
    uint32_t* const ob;
    uint32_t* const gb;
    uint32_t* const ab;
    uint32_t* const zb;
    const int rep;                            // the copy this workgroup polls

    __device__ Chain(const LayersArgs& a_, Smem& sm_, uint32_t e_)
        : a(a_), sm(sm_), lane(threadIdx.x & 63), wave(__builtin_amdgcn_readfirstlane(threadIdx.x >> 6)), e(e_),
          hb0(a_.words), hb1(a_.words + kRep * a_.H), ob(a_.words + 2 * kRep * a_.H), gb(a_.words + 2 * kRep * a_.H + kRep * a_.D),
          ab(a_.words + 2 * kRep * a_.H + 2 * kRep * a_.D), zb(a_.words + 3 * kRep * a_.H + 2 * kRep * a_.D), rep((int)blockIdx.x & (kRep - 1)) {}

    __device__ __forceinline__ uint32_t tag_of(int link) const { return (e + (uint32_t)link + 1u) & 0xffffu; }

    __device__ __forceinline__ void stamp(int link, int i) const {
        if constexpr (TRACE) {
            if (threadIdx.x == 0 && link < kTraceLinks) {
                const int slot = blockIdx.x == 0 ? 0 : blockIdx.x == 37 ? 1 : blockIdx.x == 200 ? 2 : -1;
                if (slot >= 0) a.trace[(slot * kTraceLinks + link) * kTraceStamps + i] = __builtin_amdgcn_s_memtime();
            }
        }
    }

    // ---- what a link requests one link ahead
    template <int NP, int MAXLD, int R, int PRO, int EPI, int NGE>
    __device__ __forceinline__ void prefetch(const Phase& ph, const Geo& g, Pre<T, NP, MAXLD, R, NGE>& pre, const RowSrc& add0, const RowSrc& add1) {
        if (g.NG == 0) return;
        load_weights<R, MAXLD>(ph, g, 0, g.NG < kHeadChunk ? g.NG : kHeadChunk, lane, pre.w);
        if constexpr (PRO >= PRO_NORM) load_norm_weights<T, NP>(ph.w1, g, lane, pre.w1raw);
        load_norm_weights<T, NP>(ph.norm_w, g, lane, pre.nwraw);
#pragma unroll
        for (int r = 0; r < R; ++r) pre.wdeq[r] = gloadf(ph.wdeq, ph.seg_rows == g.Nseg ? r : 0);
        if constexpr (EPI == EPI_STEP) {
            // lanes of a 32-lane half: 0-7 the i rows, 8-15 the f rows, 16-23 the g rows of one row-group
#pragma unroll
            for (int gi = 0; gi < NGE; ++gi) {
                const int ch = ((int)blockIdx.x + kWGs * gi) * 8 + (lane & 7);
                pre.lb[gi] = 0.0f;
                pre.state[gi] = 0.0f;
                if (gi < g.NG && ch < g.Nseg) {
                    if (ph.lb) pre.lb[gi] = gloadf(ph.lb, ch);
                    pre.state[gi] = gloadf(ph.state, ch);
                }
            }
        }
        if constexpr (EPI == EPI_PLAIN && PRO == PRO_PLAIN) {
            // down: the residual operands of this lane's channel (lane = copy x row; wave = row-group)
            const int ch = ((int)blockIdx.x + kWGs * wave) * 8 + (lane & 7);
            pre.add0 = pre.add1 = 0u;
            if (wave < g.NG && ch < g.Nseg) {
                pre.add0 = fetch_word(add0, ch);
                pre.add1 = fetch_word(add1, ch);
            }
        }
    }

    // One element of a row as a tagged word (a plain element gets the tag it is expected to carry).
    __device__ __forceinline__ uint32_t fetch_word(const RowSrc& s, int ch) const {
        if (s.plain) return ((uint32_t)gload2(s.plain, ch) << 16) | s.tag;
        return __hip_atomic_load(s.words + ch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __device__ __forceinline__ float finish_word(uint32_t w, const RowSrc& s, int ch) const {
        int n = 0;
        while ((w & 0xffffu) != s.tag && n++ < a.spin) w = __hip_atomic_load(s.words + ch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if ((w & 0xffffu) != s.tag) *a.err = 1;
        return word_value<T>(w);
    }

    // ---- the row (and the prologue's second operand) of this wave's slice: poll until every word carries the tag
    template <int NP, bool HAS_AUX>
    __device__ __forceinline__ void poll(const Geo& g, const RowSrc& xs, const RowSrc& as, u32x4 (&X)[NP], u32x4 (&A)[HAS_AUX ? NP : 1]) {
        auto plain4 = [&](const RowSrc& s, int k0) {
            const uint2 r = gload8(s.plain, (uint32_t)k0 * 2u);
            u32x4 w;
            w.x = (r.x << 16) | s.tag; w.y = (r.x & 0xffff0000u) | s.tag; w.z = (r.y << 16) | s.tag; w.w = (r.y & 0xffff0000u) | s.tag;
            return w;
        };
        const bool x_tagged = xs.plain == nullptr, a_tagged = HAS_AUX && as.plain == nullptr;
        int k0[NP];
#pragma unroll
        for (int v = 0; v < NP; ++v) k0[v] = slice_has(g, v, lane) ? slice_elem(g, v, lane) : g.kb0 * 128;
        if (x_tagged || a_tagged)
            for (int d = 0; d < a.delay; ++d) __builtin_amdgcn_s_sleep(1);
#pragma unroll
        for (int v = 0; v < NP; ++v) {
            if (x_tagged) X[v] = poll_issue(xs.words + k0[v]);
            else X[v] = plain4(xs, k0[v]);
            if constexpr (HAS_AUX) {
                if (a_tagged) A[v] = poll_issue(as.words + k0[v]);
                else A[v] = plain4(as, k0[v]);
            }
        }
        if (!(x_tagged || a_tagged)) return;
        for (int n = 0;; ++n) {
            bool all = true;
#pragma unroll
            for (int v = 0; v < NP; ++v) {
                if (x_tagged && __builtin_amdgcn_ballot_w64(!words_valid(X[v], xs.tag)) != 0) { all = false; X[v] = poll_issue(xs.words + k0[v]); }
                if constexpr (HAS_AUX) {
                    if (a_tagged && __builtin_amdgcn_ballot_w64(!words_valid(A[v], as.tag)) != 0) { all = false; A[v] = poll_issue(as.words + k0[v]); }
                }
            }
            if (all) break;
            if (n >= a.spin) {
                if (lane == 0) *a.err = 1;
                break;
            }
        }
    }

    // ---- prologue: norms, absmax int8 codes of this wave's slice into LDS.  Returns deq (1 / scale).
    template <int NP, int PRO>
    __device__ __forceinline__ float prologue(const Phase& ph, const Geo& g, const u32x4 (&X)[NP], const u32x4 (&A)[PRO >= PRO_RESNORM ? NP : 1],
                                              const Raw4<T> (&w1raw)[NP], const Raw4<T> (&nwraw)[NP], int link) {
        constexpr bool HAS_AUX = PRO >= PRO_RESNORM, HAS_W1 = PRO >= PRO_NORM;
        float xv[NP][4], av[HAS_AUX ? NP : 1][4];
        bool has[NP];
#pragma unroll
        for (int v = 0; v < NP; ++v) {
            has[v] = slice_has(g, v, lane);
            xv[v][0] = has[v] ? word_value<T>(X[v].x) : 0.0f; xv[v][1] = has[v] ? word_value<T>(X[v].y) : 0.0f;
            xv[v][2] = has[v] ? word_value<T>(X[v].z) : 0.0f; xv[v][3] = has[v] ? word_value<T>(X[v].w) : 0.0f;
            if constexpr (HAS_AUX) {
                av[v][0] = has[v] ? word_value<T>(A[v].x) : 0.0f; av[v][1] = has[v] ? word_value<T>(A[v].y) : 0.0f;
                av[v][2] = has[v] ? word_value<T>(A[v].z) : 0.0f; av[v][3] = has[v] ? word_value<T>(A[v].w) : 0.0f;
            }
        }
        if constexpr (PRO == PRO_RESNORM) {
#pragma unroll
            for (int v = 0; v < NP; ++v)
#pragma unroll
                for (int i = 0; i < 4; ++i) xv[v][i] = __fadd_rn(xv[v][i], av[v][i]);
        }
        if constexpr (HAS_W1) {
            double s1 = 0.0;
#pragma unroll
            for (int v = 0; v < NP; ++v)
#pragma unroll
                for (int i = 0; i < 4; ++i) s1 = mmf_add_square(s1, xv[v][i]);
            s1 = mmf_wave_sum(s1);
            if (lane == 0) sm.sum1[wave] = s1;
            float sg[PRO == PRO_GATEDNORM ? NP : 1][4];
            if constexpr (PRO == PRO_GATEDNORM) {             // the swish gate does not wait for the statistics
#pragma unroll
                for (int v = 0; v < NP; ++v)
#pragma unroll
                    for (int i = 0; i < 4; ++i) sg[v][i] = mmf_sigmoid(av[v][i]);
            }
            __syncthreads();
            const double tot = (sm.sum1[0] + sm.sum1[1]) + (sm.sum1[2] + sm.sum1[3]);
            const float rstd1 = mmf_rstd(tot, g.K, ph.inv_K, ph.eps1);
#pragma unroll
            for (int v = 0; v < NP; ++v) {
                float w1v[4];
                raw4_unpack<T>(w1raw[v], w1v);
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    float y = __fmul_rn(__fmul_rn(xv[v][i], rstd1), w1v[i]);
                    if constexpr (PRO == PRO_GATEDNORM) y = __fmul_rn(__fmul_rn(y, av[v][i]), sg[v][i]);
                    xv[v][i] = has[v] ? mmf_round_to<T>(y) : 0.0f;
                }
            }
        }
        stamp(link, 2);
        // the BitLinear's own norm
        double ss = 0.0;
#pragma unroll
        for (int v = 0; v < NP; ++v)
#pragma unroll
            for (int i = 0; i < 4; ++i) ss = mmf_add_square(ss, xv[v][i]);
        ss = mmf_wave_sum(ss);
        if (lane == 0) sm.sum2[wave] = ss;
        __syncthreads();
        const double tot2 = (sm.sum2[0] + sm.sum2[1]) + (sm.sum2[2] + sm.sum2[3]);
        const float rstd = mmf_rstd(tot2, g.K, ph.inv_K, ph.eps);
        stamp(link, 3);
        float amax = 0.0f;
#pragma unroll
        for (int v = 0; v < NP; ++v) {
            float wv[4];
            raw4_unpack<T>(nwraw[v], wv);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float y = has[v] ? __fmul_rn(__fmul_rn(xv[v][i], rstd), wv[i]) : 0.0f;
                xv[v][i] = y;
                amax = fmaxf(amax, fabsf(y));
            }
        }
        amax = mmf_wave_max(amax);
        if (lane == 0) sm.amax[wave] = amax;
        __syncthreads();
        amax = fmaxf(fmaxf(sm.amax[0], sm.amax[1]), fmaxf(sm.amax[2], sm.amax[3]));
        stamp(link, 4);
        const float scale = __fdiv_rn(127.0f, fmaxf(amax, 1e-5f));
        int qs = 0;
#pragma unroll
        for (int v = 0; v < NP; ++v) {
            uint32_t packed4 = 0;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int c = mmf_code(xv[v][i], scale);
                qs += c;
                packed4 |= (uint32_t)(c & 0xff) << (8 * i);
            }
            if (has[v]) *reinterpret_cast<uint32_t*>(sm.q + slice_elem(g, v, lane)) = packed4;
        }
        qs = mmf_wave_sum(qs);
        if (lane == 0) sm.qs[wave] = qs;
        // the codes are read back by this wave only: LDS operations of a wave execute in order, no barrier needed
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        stamp(link, 5);
        return __fdiv_rn(1.0f, scale);       // needed by the epilogue only
    }

    // ---- dot products of this wave's slice with the weights of row-groups [0, ng) x R segments; partial sums to LDS
    template <int R, int MAXLD>
    __device__ __forceinline__ void dot(const Geo& g, int ng, const uint4 (&w)[MAXLD]) {
        if (g.nkb == 0) {
            // nothing of this row belongs to the wave: its partial sums are zero
            for (int it = lane >> 4; it < ng * R; it += 4)
                if ((lane & 15) < 8) { sm.part[it][lane & 7][2 * wave] = 0; sm.part[it][lane & 7][2 * wave + 1] = 0; }
            return;
        }
        const int slot = lane >> 4, half = (lane >> 3) & 1;
        int gi = 0, r = 0, q = 0, acc = 0;
#pragma unroll
        for (int j = 0; j < MAXLD; ++j) {
            if (gi < ng) {
                const int kraw = 4 * q + slot;
                const bool live = kraw < g.nkb;
                const int kb = g.kb0 + (live ? kraw : g.nkb - 1);
                uint4 wq = w[j];
                if (!live) wq = make_uint4(0u, 0u, 0u, 0u);
                acc = mmf_dot_block(sm.q, wq, kb, half, acc);
                if (q == g.nq - 1) {
                    acc += mmf_dpp<0x128>(acc);                              // the other half of the 16 lanes (rotate by 8)
                    acc += __builtin_amdgcn_ds_swizzle(acc, 0x401F);         // lane ^ 16: the neighbouring k-block
                    if ((lane & 31) < 8) sm.part[gi * R + r][lane & 7][2 * wave + (lane >> 5)] = acc;
                    acc = 0;
                }
            }
            if (++q == g.nq) { q = 0; if (++r == R) { r = 0; ++gi; } }
        }
    }

    // the integer result of item `it`, row `row`: the waves' partial sums less the row's code sum (weights are stored as t + 1)
    __device__ __forceinline__ int total(int it, int row) const {
        const int4 p0 = *reinterpret_cast<const int4*>(&sm.part[it][row][0]);
        const int4 p1 = *reinterpret_cast<const int4*>(&sm.part[it][row][4]);
        const int4 qv = *reinterpret_cast<const int4*>(&sm.qs[0]);
        return ((p0.x + p0.y) + (p0.z + p0.w)) + ((p1.x + p1.y) + (p1.z + p1.w)) - ((qv.x + qv.y) + (qv.z + qv.w));
    }

    // Two neighbouring rows' words become one 8-byte store by the even row (fewer, wider stores travel faster).
    __device__ __forceinline__ void store_pair(uint32_t* base, int ch, uint32_t word, bool active) const {
        const uint32_t next = (uint32_t)mmf_dpp<kDppXor1>((int)word);
        if (active && !(lane & 1)) ll_st8(reinterpret_cast<uint64_t*>(base + ch), (uint64_t)word | ((uint64_t)next << 32));
    }

    // ================================================================ the four links of a layer
    // i/f/g: block norm -> stacked projection -> gate math + recurrence step
    template <class PreNext, class FNext>
    __device__ __forceinline__ void link_ifg(const Phase& ph, const Geo& g, PreIfg& pre, const RowSrc& h_in, int link, FNext&& next) {
        stamp(link, 0);
        if (g.NG == 0) { next(); return; }
        u32x4 X[NPH], A[1];
        poll<NPH, false>(g, h_in, h_in, X, A);
        stamp(link, 1);
        next();
        const float deq = prologue<NPH, PRO_NORM>(ph, g, X, A, pre.w1raw, pre.nwraw, link);
        dot<3, LD_IFG>(g, g.NG, pre.w);
        stamp(link, 6);
        __syncthreads();
        stamp(link, 7);
        const uint32_t tag = tag_of(link);
        // a wave serves two copies: lanes 0-23 of each 32-lane half run the i, f and g rows of the 8 channels side by
        // side, so the two exp / divide chains of the gate math run in parallel; the f lanes' gate reaches the i lanes by
        // a rotate within the 16-lane row.  Operation for operation the arithmetic of the single-lane form.
        const int r3 = (lane & 31) >> 3, row = lane & 7, copy = 2 * wave + (lane >> 5);
#pragma unroll
        for (int gi = 0; gi < NGH; ++gi) {
            if (gi >= g.NG) break;
            const int ch = ((int)blockIdx.x + kWGs * gi) * 8 + row;
            const float lb = pre.lb[gi], st = pre.state[gi];
            const int tot = total(gi * 3 + (r3 < 3 ? r3 : 0), row);
            const float wd = r3 == 0 ? pre.wdeq[0] : r3 == 1 ? pre.wdeq[1] : pre.wdeq[2];
            const float res = __fmul_rn(__fmul_rn((float)tot, deq), wd);
            const float v16 = mmf_round_to<T>(res);                       // iv on the i lanes, fv on the f lanes
            const float ex = __fadd_rn(1.0f, mmf_exp(-v16));
            float sg = __fdiv_rn(1.0f, ex);                               // sigmoid(fv) on the f lanes
            if (ph.lb) sg = __fadd_rn(lb, __fmul_rn(__fsub_rn(1.0f, lb), sg));
            const float go = mmf_dpp<0x128>(mmf_round_to<T>(sg));         // lanes 0-7 read lanes 8-15
            const float xo = mmf_round_to<T>(__fdiv_rn(__fmul_rn(v16, __fsub_rn(1.0f, go)), ex));
            const float h = __fadd_rn(__fmul_rn(go, st), xo);
            const bool live = ch < g.Nseg;
            if (live && r3 == 0 && copy == 0) ((MMF_AS_GLOBAL float*)ph.state)[ch] = h;
            store_pair(ob + copy * a.D, ch, make_word<T>(h, tag), live && r3 == 0);
            store_pair(gb + copy * a.D, ch, make_word<T>(res, tag), live && r3 == 2);
        }
        stamp(link, 8);
    }

    // a link whose 8 x 8 epilogue lanes are copy x row, one row-group per wave: o_proj, gate/up, down
    template <int NP, int MAXLD, int R, int PRO, int EPI, class FNext>
    __device__ __forceinline__ void link_plain(const Phase& ph, const Geo& g, Pre<T, NP, MAXLD, R, 1>& pre, const RowSrc& xs, const RowSrc& as,
                                               const RowSrc& add0, const RowSrc& add1, uint32_t* out, int out_n, T* plain_out, int link,
                                               FNext&& next) {
        stamp(link, 0);
        if (g.NG == 0) { next(); return; }
        constexpr bool HAS_AUX = PRO >= PRO_RESNORM;
        u32x4 X[NP], A[HAS_AUX ? NP : 1];
        poll<NP, HAS_AUX>(g, xs, as, X, A);
        stamp(link, 1);
        next();
        const float deq = prologue<NP, PRO>(ph, g, X, A, pre.w1raw, pre.nwraw, link);
        dot<R, MAXLD>(g, g.NG, pre.w);
        stamp(link, 6);
        __syncthreads();
        stamp(link, 7);
        const uint32_t tag = tag_of(link);
        const int row = lane & 7, copy = lane >> 3;
        for (int gi = wave; gi < g.NG; gi += kNW) {
            const int ch = ((int)blockIdx.x + kWGs * gi) * 8 + row;
            const bool live = ch < g.Nseg;
            float res[R];
#pragma unroll
            for (int r = 0; r < R; ++r) res[r] = __fmul_rn(__fmul_rn((float)total(gi * R + r, row), deq), pre.wdeq[r]);
            float o;
            if constexpr (EPI == EPI_SWIGLU) {
                const float gt = mmf_round_to<T>(res[0]), u = mmf_round_to<T>(res[1]);
                o = __fdiv_rn(__fmul_rn(gt, u), __fadd_rn(1.0f, mmf_exp(-gt)));
            } else {
                o = res[0];
                if constexpr (PRO == PRO_PLAIN) {
                    // down: the residual it adds is T(attn + h), formed here from its two operands
                    uint32_t w0 = pre.add0, w1 = pre.add1;
                    if (gi != wave && live) { w0 = fetch_word(add0, ch); w1 = fetch_word(add1, ch); }
                    float r0 = 0.0f, r1 = 0.0f;
                    if (live) {
                        r0 = add0.plain ? word_value<T>(w0) : finish_word(w0, add0, ch);
                        r1 = add1.plain ? word_value<T>(w1) : finish_word(w1, add1, ch);
                    }
                    o = __fadd_rn(mmf_round_to<T>(o), mmf_round_to<T>(__fadd_rn(r0, r1)));
                }
            }
            store_pair(out + copy * out_n, ch, make_word<T>(o, tag), live);
            if (plain_out && live && copy == 0) plain_out[ch] = mmf_from_float<T>(o);
        }
        stamp(link, 8);
    }

    // final norm -> lm_head: plain logits, and this lane's running candidate for the greedy token
    template <class FNext>
    __device__ __forceinline__ void link_head(const Phase& ph, const Geo& g, PreHead& pre, const RowSrc& h_last, int link, Best& best, FNext&& next) {
        stamp(link, 0);
        if (g.NG == 0) { next(); return; }
        u32x4 X[NPH], A[1];
        poll<NPH, false>(g, h_last, h_last, X, A);
        stamp(link, 1);
        next();
        const float deq = prologue<NPH, PRO_NORM>(ph, g, X, A, pre.w1raw, pre.nwraw, link);
        T* logits = static_cast<T*>(a.logits);
        for (int c0 = 0; c0 < g.NG; c0 += kHeadChunk) {
            const int ng = g.NG - c0 < kHeadChunk ? g.NG - c0 : kHeadChunk;
            if (c0 > 0) load_weights<1, LD_HEAD>(ph, g, c0, ng, lane, pre.w);
            dot<1, LD_HEAD>(g, ng, pre.w);
            __syncthreads();
            const int gl = wave * 8 + (lane >> 3), row = lane & 7;        // a wave takes 8 row-groups of the chunk
            if (gl < ng) {
                const int ch = ((int)blockIdx.x + kWGs * (c0 + gl)) * 8 + row;
                if (ch < g.Nseg) {
                    const float o = __fmul_rn(__fmul_rn((float)total(gl, row), deq), pre.wdeq[0]);
                    logits[ch] = mmf_from_float<T>(o);
                    const float ov = mmf_round_to<T>(o);
                    if (ov == ov) best_take(best, ov, (uint32_t)ch);
                }
            }
            if (c0 + kHeadChunk < g.NG) __syncthreads();                  // part[] is reused by the next chunk
        }
        stamp(link, 8);
    }
};

// A record of the phase table, read with scalar loads (the table is not written during the launch).
__device__ __forceinline__ Phase load_phase(const Phase* table, int i) {
    const MMF_AS_CONST Phase* p = (const MMF_AS_CONST Phase*)table + i;
    Phase r;
    r.w1 = p->w1; r.norm_w = p->norm_w; r.packed = p->packed; r.wdeq = p->wdeq; r.lb = p->lb; r.state = p->state;
    r.inv_K = p->inv_K; r.eps = p->eps; r.eps1 = p->eps1; r.K = p->K; r.N = p->N; r.seg_rows = p->seg_rows; r.pad_ = 0;
    return r;
}

template <typename T, int NPH, int NPI, int NQH, int NQI, int NGH, int NGI, bool TRACE>
__global__ __launch_bounds__(kNT) void decode_layers_kernel(LayersArgs a) {
    using C = Chain<T, NPH, NPI, NQH, NQI, NGH, NGI, TRACE>;
    __shared__ Smem sm;
    const uint32_t e = *a.epoch;
    int64_t id = *a.tok;
    if (id < 0 || id >= a.vocab) id = 0;
    const T* emb_row = static_cast<const T*>(a.table) + id * a.H;
    C c(a, sm, e);
    const int L = a.n_layers;
    const RowSrc none{nullptr, nullptr, 0u};

    typename C::PreIfg pa;
    typename C::PreO pb;
    typename C::PreGate pc;
    typename C::PreDown pd;
    typename C::PreHead phd;

    auto h_src = [&](int l) {        // the residual stream that enters layer l (this XCD's copy)
        return l == 0 ? RowSrc{emb_row, nullptr, c.tag_of(-1)} : RowSrc{nullptr, ((l - 1) & 1 ? c.hb1 : c.hb0) + c.rep * a.H, c.tag_of(4 * (l - 1) + 3)};
    };

    Phase p0 = load_phase(a.phases, 0);
    Geo g0 = make_geo<3>(p0.K, p0.N, c.wave);
    c.template prefetch<NPH, C::LD_IFG, 3, PRO_NORM, EPI_STEP, NGH>(p0, g0, pa, none, none);
    for (int l = 0; l < L; ++l) {
        const bool last = l == L - 1;
        const RowSrc h_in = h_src(l);
        const Phase p1 = load_phase(a.phases, 4 * l + 1), p2 = load_phase(a.phases, 4 * l + 2), p3 = load_phase(a.phases, 4 * l + 3);
        const Geo g1 = make_geo<1>(p1.K, p1.N, c.wave), g2 = make_geo<2>(p2.K, p2.N, c.wave), g3 = make_geo<1>(p3.K, p3.N, c.wave);
        const RowSrc g_in{nullptr, c.gb + c.rep * a.D, c.tag_of(4 * l)}, o_in{nullptr, c.ob + c.rep * a.D, c.tag_of(4 * l)};
        const RowSrc a_in{nullptr, c.ab + c.rep * a.H, c.tag_of(4 * l + 1)};
        const RowSrc z_in{nullptr, c.zb + c.rep * a.I, c.tag_of(4 * l + 2)};
        c.template link_ifg<typename C::PreO>(p0, g0, pa, h_in, 4 * l,
                                              [&] { c.template prefetch<NPH, C::LD_O, 1, PRO_GATEDNORM, EPI_PLAIN, 1>(p1, g1, pb, none, none); });
        c.template link_plain<NPH, C::LD_O, 1, PRO_GATEDNORM, EPI_PLAIN>(p1, g1, pb, g_in, o_in, none, none, c.ab, a.H, nullptr, 4 * l + 1,
                                              [&] { c.template prefetch<NPH, C::LD_GATE, 2, PRO_RESNORM, EPI_SWIGLU, 1>(p2, g2, pc, none, none); });
        c.template link_plain<NPH, C::LD_GATE, 2, PRO_RESNORM, EPI_SWIGLU>(p2, g2, pc, a_in, h_in, none, none, c.zb, a.I, nullptr, 4 * l + 2,
                                              [&] { c.template prefetch<NPI, C::LD_DOWN, 1, PRO_PLAIN, EPI_PLAIN, 1>(p3, g3, pd, a_in, h_in); });
        T* plain = last ? static_cast<T*>(a.h_out) : nullptr;
        Phase pn = p0;
        Geo gn = g0;
        if (!last) {
            pn = load_phase(a.phases, 4 * l + 4);
            gn = make_geo<3>(pn.K, pn.N, c.wave);
        } else if (a.head) {
            pn = load_phase(a.head, 0);
            gn = make_geo<1>(pn.K, pn.N, c.wave);
        }
        c.template link_plain<NPI, C::LD_DOWN, 1, PRO_PLAIN, EPI_PLAIN>(p3, g3, pd, z_in, none, a_in, h_in, (l & 1) ? c.hb1 : c.hb0, a.H, plain, 4 * l + 3,
                                              [&] {
                                                  if (!last) c.template prefetch<NPH, C::LD_IFG, 3, PRO_NORM, EPI_STEP, NGH>(pn, gn, pa, none, none);
                                                  else if (a.head) c.template prefetch<NPH, C::LD_HEAD, 1, PRO_NORM, EPI_HEAD, 1>(pn, gn, phd, none, none);
                                              });
        p0 = pn;
        g0 = gn;
    }
    if (a.head) {
        // final norm -> lm_head: plain logits, and this workgroup's candidate for the greedy token
        const RowSrc h_last{nullptr, ((L - 1) & 1 ? c.hb1 : c.hb0) + c.rep * a.H, c.tag_of(4 * (L - 1) + 3)};
        const uint32_t tag_h = c.tag_of(4 * L);
        Best best{0.0f, kNone};
        c.link_head(p0, g0, phd, h_last, 4 * L, best, [] {});
        const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            const float ov = __shfl_xor(best.v, o, 64);
            const uint32_t oi = (uint32_t)__shfl_xor((int)best.i, o, 64);
            best_take(best, ov, oi);
        }
        __syncthreads();                                        // the links are done with the shared arrays
        if (lane == 0) { sm.best_v[wave] = best.v; sm.best_i[wave] = best.i; }
        __syncthreads();
        if (threadIdx.x == 0) {
            for (int w = 1; w < kNW; ++w) best_take(best, sm.best_v[w], sm.best_i[w]);
            ll_st8(a.am_words + blockIdx.x, ((uint64_t)best.i << 32) | (uint64_t)make_word<T>(best.i == kNone ? 0.0f : best.v, tag_h));
        }
        if (blockIdx.x == 0) {
            // the greedy token: lowest index of the largest logit over the workgroups' candidates
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
            __syncthreads();                                    // thread 0 is done with best_v / best_i
            if (lane == 0) { sm.best_v[wave] = b.v; sm.best_i[wave] = b.i; }
            __syncthreads();
            if (threadIdx.x == 0) {
                for (int w = 1; w < kNW; ++w) best_take(b, sm.best_v[w], sm.best_i[w]);
                *a.tok_out = b.i == kNone ? 0 : (int64_t)b.i;
            }
        }
    }
    // Every workgroup that takes part in a link read the tag base (and the token) before workgroup 0 could get here
    // (the last link's inputs depend, through the chain, on an output of every such workgroup), so the next launch's
    // base can be published now.
    if (blockIdx.x == 0 && threadIdx.x == 0) *a.epoch = e + 4u * (uint32_t)a.n_layers + 2u;
}

template <typename T, bool TRACE>
int launch_layers(const LayersArgs& a, hipStream_t s) {
    if (a.H <= 2048 && a.I <= 6144) decode_layers_kernel<T, 2, 6, 1, 3, 1, 3, TRACE><<<kWGs, kNT, 0, s>>>(a);
    else if (a.H <= 4096 && a.I <= 8192) decode_layers_kernel<T, 4, 8, 2, 4, 2, 4, TRACE><<<kWGs, kNT, 0, s>>>(a);
    else return MMF_ERR_WIDE;
    MMF_CHECK_LAUNCH();
    return 0;
}

int decode_layers_entry(const void* phases, int n_layers, const void* table, const int64_t* tok, int64_t vocab, uint32_t* words,
                        void* h_out, const void* head, void* logits, uint64_t* am_words, int64_t* tok_out, uint32_t* epoch, int* err,
                        int64_t* trace, int H, int D, int I, int spin, int delay, int dtype, void* stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (!phases || n_layers <= 0 || !table || !tok || vocab <= 0 || !words || !h_out || !epoch || !err || H <= 0 || D <= 0 || I <= 0 ||
        spin <= 0 || delay < 0 || delay > 64)
        return MMF_ERR_ARG;
    if (head && (!logits || !am_words || !tok_out)) return MMF_ERR_ARG;
    if (H % 128 != 0 || D != H || I % 128 != 0) return MMF_ERR_ARG;      // rows are whole k-blocks: no ragged tail in a link
    if (dtype != MMF_BF16 && dtype != MMF_F16) return MMF_ERR_ARG;        // a tagged word carries a 16-bit value
    if (H > 4096 || I > 8192) return MMF_ERR_WIDE;
    for (const void* p : {(const void*)words, (const void*)table, (const void*)h_out})
        if (reinterpret_cast<uintptr_t>(p) & 15u) return MMF_ERR_ALIGN;
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess)
        return MMF_ERR_ARG;
    if (cus < kWGs) return MMF_ERR_ARG;                                       // the resident grid needs one CU per workgroup
    LayersArgs a{};
    a.phases = static_cast<const Phase*>(phases); a.n_layers = n_layers; a.table = table; a.tok = tok; a.vocab = vocab;
    a.words = words; a.h_out = h_out; a.head = static_cast<const Phase*>(head); a.logits = logits; a.am_words = am_words;
    a.tok_out = tok_out; a.epoch = epoch; a.err = err; a.trace = reinterpret_cast<long long*>(trace);
    a.H = H; a.D = D; a.I = I; a.spin = spin; a.delay = delay;
    if (trace) {
        switch (dtype) {
            case MMF_BF16: return launch_layers<bf16_t, true>(a, stream);
            case MMF_F16: return launch_layers<f16_t, true>(a, stream);
        }
    } else {
        switch (dtype) {
            case MMF_BF16: return launch_layers<bf16_t, false>(a, stream);
            case MMF_F16: return launch_layers<f16_t, false>(a, stream);
        }
    }
    return MMF_ERR_ARG;
}

}  // namespace

extern "C" {

int mmf_decode_layers_phase_bytes(void) { return (int)sizeof(Phase); }

int64_t mmf_decode_layers_words(int H, int D, int I) { return (int64_t)kRep * (3 * (int64_t)H + 2 * (int64_t)D + (int64_t)I); }

int mmf_decode_layers_copies(void) { return kRep; }

int mmf_decode_layers(const void* phases, int n_layers, const void* table, const int64_t* tok, int64_t vocab, uint32_t* words,
                      void* h_out, const void* head, void* logits, uint64_t* am_words, int64_t* tok_out, uint32_t* epoch, int* err,
                      int H, int D, int I, int spin, int dtype, void* stream) {
    static const int delay = [] {
        const char* v = getenv("MMF_DECODE_POLL_DELAY");
        return v ? atoi(v) : 6;
    }();
    return decode_layers_entry(phases, n_layers, table, tok, vocab, words, h_out, head, logits, am_words, tok_out, epoch, err, nullptr,
                               H, D, I, spin, delay, dtype, stream);
}

int mmf_decode_layers_trace_words(void) { return kTraceWGs * kTraceLinks * kTraceStamps; }

int mmf_decode_layers_traced(const void* phases, int n_layers, const void* table, const int64_t* tok, int64_t vocab, uint32_t* words,
                             void* h_out, const void* head, void* logits, uint64_t* am_words, int64_t* tok_out, uint32_t* epoch, int* err,
                             int64_t* trace, int H, int D, int I, int spin, int delay, int dtype, void* stream) {
    if (!trace) return MMF_ERR_ARG;
    return decode_layers_entry(phases, n_layers, table, tok, vocab, words, h_out, head, logits, am_words, tok_out, epoch, err, trace, H, D,
                               I, spin, delay, dtype, stream);
}

}  // extern "C"
