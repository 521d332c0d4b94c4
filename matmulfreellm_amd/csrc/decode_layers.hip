// One batch-1 decode step -- embedding row, all layers, final norm + lm_head, greedy argmax -- in ONE persistent launch.
//
// A decode step is a chain of 4 dependent fused BitLinears per layer (mmfreelm/models/hgrn_bit/
// modeling_hgrn_bit.py:97-109 around mmfreelm/layers/hgrn_bit.py:83-162): block norm -> i/f/g -> gate math +
// recurrence step; gated norm -> o_proj; residual + norm -> gate_proj -> swiglu; down_proj + residual.
// 256 workgroups of 4 waves stay resident (one per CU, one wave per SIMD) and walk the 4L links themselves, all
// through ONE loop body (a single wave per SIMD has nobody to hide instruction fetch behind: the code stays small).
//
// Hand-off.  Activations travel between workgroups as self-validating 32-bit words: a 16-bit value in the high half,
// a 16-bit tag naming the producing link in the low half.  A producer stores its words to 8 copies of the row (one
// per XCD: a row polled by 256 workgroups at once is a hot spot in the memory-side cache, 32 pollers per copy are
// not); a consumer polls the copy of its XCD with device-coherent loads until every word carries the tag.  The poll
// is both the synchronisation and the transfer: no fence, no grid barrier.  The first poll of a link is held back a
// little so that it reaches memory after the producers' stores rather than just before them (a poll that comes back
// stale costs a whole round trip).
//
// Body of a link.  A wave owns a contiguous slice of the row's k-blocks from the poll to the dot products: it polls
// that slice, takes part in the row statistics (per-wave partial -> LDS -> barrier: sum of squares of the block norm,
// sum of squares of the BitLinear's own norm, absmax), quantises its slice into LDS and multiplies it with its slice
// of the packed weights -- the codes never cross waves, so no barrier sits between quantiser and dot.  The per-wave
// partial dot products meet in LDS for the epilogue (one more barrier).  A workgroup owns row-groups of 8 output rows
// (row-group g of a segment belongs to workgroup g mod 256); 16 lanes = (2 halves x 8 rows) read the 2-bit weights of
// one k-block, so a wave load covers 4 k-blocks.
//
// Nothing a link needs besides its input row is waited for inside the link: the phase table is copied to LDS when the
// launch starts; the packed weights and the norm weights of link n+1 are brought into LDS by the DMA path
// (global_load_lds, no registers) while link n computes, each wave fetching exactly the slices it will read itself;
// the few epilogue operands (recurrent state, lower bound, scales, residual operands) are loaded into registers one
// link ahead.  All of these are requested after link n's row has arrived (requested before the poll they would
// delay it) and are waited for, with everything else in flight, right after link n+1's poll.
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
#include <type_traits>

namespace {

constexpr int kNW = 4, kNT = 64 * kNW;
constexpr int kWGs = 256, kRep = 8;
constexpr int kMaxLayers = 96;
constexpr int kItems = 8;                      // (row-group, segment) items of a pass over a link's outputs

#define MMF_AS_GLOBAL __attribute__((address_space(1)))
#define MMF_AS_LDS __attribute__((address_space(3)))

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
static_assert(sizeof(Phase) == 80, "five 16-byte pieces per record");

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
    int n_layers, H, D, I, spin;
    int delay[5];             // hold-back of a link's first poll, per kind of link, in units of about 64 cycles
    int nqmax;                // k-quads of the widest wave slice: a wave's norm-weight region in LDS is nqmax KiB
    int itemsA, itemsB;       // 1 KiB weight loads per wave the two weight buffers hold
    uint32_t off_q, off_nrm, off_w;   // dynamic LDS: codes, norm weights (w1 regions, then the BitLinear's), weight buffers
};

constexpr int kTraceWGs = 256, kTraceLinks = 128, kTraceStamps = 12;

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// Loads through the global address space (pointers read from the phase table are generic to the compiler; these keep
// the accesses off the flat path).  Builtin vector types only: they can be read from any address space.
__device__ __forceinline__ uint2 gload8(const void* base, uint32_t byte_off) {
    const u32x2 v = *reinterpret_cast<const MMF_AS_GLOBAL u32x2*>((const MMF_AS_GLOBAL char*)(base) + byte_off);
    return make_uint2(v.x, v.y);
}
__device__ __forceinline__ float gloadf(const void* base, int i) { return ((const MMF_AS_GLOBAL float*)base)[i]; }
__device__ __forceinline__ uint16_t gload2(const void* base, int i) { return ((const MMF_AS_GLOBAL uint16_t*)base)[i]; }

// 64 lanes x 16 bytes from global memory straight into 1 KiB of LDS at `lds` (wave-uniform), lane order.
// Issued by hand: told about a transfer into LDS, the compiler makes every later LDS read (the statistics exchanged a
// few hundred cycles on, the partial sums) wait for it -- a trip to HBM in the middle of every link.  The data is
// only read after the next link's input row has arrived, behind a wait for ALL vector-memory traffic (a count that
// left younger loads in flight would not do: transfers into LDS and ordinary loads complete in no fixed order).
__device__ __forceinline__ void dma16(const void* gbase, uint32_t byte_off, unsigned char* lds) {
    const uint32_t l = (uint32_t)(uintptr_t)(MMF_AS_LDS unsigned char*)lds;
    const uint64_t b = (uint64_t)gbase;
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(l), "v"(byte_off), "s"(b) : "memory");
}

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also waits for every outstanding vector-memory
// operation -- here that would be the DMA of the NEXT link's weights, requested a moment ago, i.e. a trip to HBM in
// the middle of every link.  Those requests are waited for where their data is needed (the next link's poll).
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

enum Kind : int { K_IFG = 0, K_O = 1, K_GATE = 2, K_DOWN = 3, K_HEAD = 4 };

// Running greedy choice of one epilogue lane: lowest index of the largest value seen; NaNs never win.
struct Best {
    float v;
    uint32_t i;               // 0xffffffff: nothing yet
};
constexpr uint32_t kNone = 0xffffffffu;
__device__ __forceinline__ void best_take(Best& b, float v, uint32_t i) {
    if (i != kNone && (b.i == kNone || v > b.v || (v == b.v && i < b.i))) { b.v = v; b.i = i; }
}

struct Small {
    double sum1[kNW], sum2[kNW];             // per-wave partial sums of squares
    float amax[kNW];
    int qs[kNW];                             // per-wave sums of codes
    int part[kItems][8][2 * kNW];            // [row-group x segment][row][wave x lane half] partial dot products
    float best_v[kNW];
    uint32_t best_i[kNW];
};

__device__ __forceinline__ uint64_t ll_ld8(const uint64_t* p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ uint32_t ll_ld4(const uint32_t* p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
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

// Wave-uniform values read from the LDS copy of the phase table, as scalars.
__device__ __forceinline__ uint32_t uni32(const void* lds) { return (uint32_t)__builtin_amdgcn_readfirstlane(*reinterpret_cast<const int*>(lds)); }
__device__ __forceinline__ uint64_t uni64(const void* lds) {
    const int* p = reinterpret_cast<const int*>(lds);
    return (uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane(p[0]) | ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane(p[1]) << 32);
}
// Shape of the model a kernel instantiation serves.  Static: hidden and intermediate width are compile-time constants,
// so every link's geometry (k-blocks per wave, passes, loads, masks) folds into the code -- with one wave per SIMD a
// wave issues one instruction every four cycles, scalar or vector, so bookkeeping instructions cost as much as
// arithmetic and are worth compiling away.  Dynamic: the same source with the widths read from the arguments.
template <int H_, int I_>
struct StaticShape {
    static constexpr bool kStatic = true;
    static constexpr int H = H_, I = I_;
};
struct DynShape {
    static constexpr bool kStatic = false;
    static constexpr int H = 0, I = 0;
};
constexpr int ceil_div_c(int a, int b) { return (a + b - 1) / b; }
// passes of 256 elements over a wave's slice of a K-wide row, k-quads of that slice
constexpr int passes_of(int K) { return ceil_div_c(ceil_div_c(K / 128, kNW), 2); }
constexpr int quads_of(int K) { return ceil_div_c(ceil_div_c(K / 128, kNW), 4); }

// Geometry of a link for this wave and workgroup (all wave-uniform; constants when the shape is static).
struct Geo {
    int K, KB, kb0, nkb, nq, np;             // row width, its k-blocks, this wave's slice [kb0, kb0 + nkb), k-quads and 256-element passes of a slice
    int R, Nseg, NBseg, NG;                  // segments, rows / n-blocks per segment, row-groups of this workgroup
    bool even;                               // every wave's slice is nq whole k-quads: no clamps, no masks
};
__device__ __forceinline__ Geo make_geo(int K, int N, int kind, int wave) {
    Geo g;
    g.K = K;
    g.KB = K >> 7;
    const int kbw = (g.KB + kNW - 1) / kNW;
    g.kb0 = wave * kbw;
    g.nkb = g.KB - g.kb0 < 0 ? 0 : (g.KB - g.kb0 < kbw ? g.KB - g.kb0 : kbw);
    if (g.KB % kNW == 0) g.nkb = kbw;        // (folds when K is a constant)
    if (g.nkb == 0) g.kb0 = 0;
    g.nq = (kbw + 3) >> 2;
    g.np = (kbw + 1) >> 1;
    g.even = g.KB % (4 * kNW) == 0;
    g.R = kind == K_IFG ? 3 : kind == K_GATE ? 2 : 1;
    g.Nseg = kind == K_IFG ? N / 3 : kind == K_GATE ? N >> 1 : N;
    g.NBseg = (g.Nseg + 31) >> 5;
    const int RG = (g.Nseg + 7) >> 3;
    g.NG = RG > (int)blockIdx.x ? (RG - (int)blockIdx.x + kWGs - 1) / kWGs : 0;
    return g;
}

template <typename T, class S, bool TRACE>
__global__ __launch_bounds__(kNT) void decode_layers_kernel(LayersArgs a) {
    extern __shared__ __align__(16) unsigned char dyn[];
    __shared__ Small sm;
    const uint32_t e = *a.epoch;
    int64_t id = *a.tok;
    if (id < 0 || id >= a.vocab) id = 0;
    const int L = a.n_layers;
    const T* emb_row = static_cast<const T*>(a.table) + id * (S::kStatic ? S::H : a.H);

    // ---- the phase table into LDS: a record is then an LDS read away, not a cold trip to memory in front of every link
    {
        const int n16 = 4 * L * 5;
        for (int i = threadIdx.x; i < n16; i += kNT) reinterpret_cast<uint4*>(dyn)[i] = reinterpret_cast<const uint4*>(a.phases)[i];
        if (a.head && threadIdx.x < 5) reinterpret_cast<uint4*>(dyn)[n16 + threadIdx.x] = reinterpret_cast<const uint4*>(a.head)[threadIdx.x];
    }
    __syncthreads();

    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int slot = lane >> 4, half = (lane >> 3) & 1;
    const uint32_t lane_off = (uint32_t)(half * 512 + (lane & 7) * 16);       // this lane's 16 bytes within a 1 KiB weight block, less the k-block
    const int rep = (int)blockIdx.x & (kRep - 1);                             // the copy this workgroup polls
    constexpr int NP = S::kStatic ? (passes_of(S::H) > passes_of(S::I) ? passes_of(S::H) : passes_of(S::I)) : 8;   // passes of the widest row
    constexpr int NPH = S::kStatic ? passes_of(S::H) : 4;                                                           // passes of a hidden-wide row
    using KIfg = std::integral_constant<int, K_IFG>;
    using KO = std::integral_constant<int, K_O>;
    using KGate = std::integral_constant<int, K_GATE>;
    using KDown = std::integral_constant<int, K_DOWN>;
    using KHead = std::integral_constant<int, K_HEAD>;
    Best best{0.0f, kNone};
    // epilogue operands of this lane, loaded one link ahead; a set per kind of link, so that the request for the next
    // link does not replace what the current link's epilogue is about to use
    float wdk[5][3] = {};
    float lb[2] = {0.0f, 0.0f}, st[2] = {0.0f, 0.0f};     // i/f/g: lower bound and recurrent state of this lane's channel, per row-group
    uint32_t a0 = 0u, a1 = 0u;                             // down: the two operands of the residual
    u32x4 auxH[NPH] = {};                                  // gate/up: the residual stream of this wave's slice (stored links ago: fetched a link ahead)
    const int Hh = S::kStatic ? S::H : a.H, Ii = S::kStatic ? S::I : a.I;
    int8_t* const qbuf = reinterpret_cast<int8_t*>(dyn + a.off_q);
    unsigned char* const nrm_w1 = dyn + a.off_nrm;                                   // kNW regions of nqmax KiB
    unsigned char* const nrm_nw = dyn + a.off_nrm + kNW * a.nqmax * 1024;
    unsigned char* const wbufA = dyn + a.off_w;                                      // weights of i/f/g and gate/up (and the lm_head's even passes)
    unsigned char* const wbufB = dyn + a.off_w + kNW * a.itemsA * 1024;              // weights of o_proj and down_proj (and the lm_head's odd passes)
    uint32_t* const hb0 = a.words;
    uint32_t* const hb1 = a.words + kRep * Hh;
    uint32_t* const ob = a.words + 2 * kRep * Hh;
    uint32_t* const gb = a.words + 3 * kRep * Hh;
    uint32_t* const ab = a.words + 4 * kRep * Hh;
    uint32_t* const zb = a.words + 5 * kRep * Hh;
    auto tag_of = [&](int link) -> uint32_t { return (e + (uint32_t)link + 1u) & 0xffffu; };
    auto stamp = [&](int link, int i) {
        if constexpr (TRACE) {
            if (threadIdx.x == 0 && link < kTraceLinks) {
                long long* t = a.trace + ((int)blockIdx.x * kTraceLinks + link) * kTraceStamps;
                t[i] = __builtin_amdgcn_s_memtime();
                // entry, arrival and end of the link also on the 100 MHz clock all XCDs share (slots 9-11)
                if (i == 0 || i == 1 || i == 8) t[i == 0 ? 9 : i == 1 ? 10 : 11] = __builtin_amdgcn_s_memrealtime();
            }
        }
    };
    // the record of link ln in the LDS copy of the phase table
    auto rec = [&](int ln) -> const unsigned char* { return dyn + ln * (int)sizeof(Phase); };
    auto geo = [&](auto kc, int ln) -> Geo {
        constexpr int KIND = decltype(kc)::value;
        if constexpr (S::kStatic) {
            constexpr int K = KIND == K_DOWN ? S::I : S::H;
            const int N = KIND == K_IFG ? 3 * S::H : KIND == K_O ? S::H : KIND == K_GATE ? 2 * S::I : KIND == K_DOWN ? S::H : (int)uni32(rec(ln) + 68);
            return make_geo(K, N, KIND, wave);
        } else {
            return make_geo((int)uni32(rec(ln) + 64), (int)uni32(rec(ln) + 68), KIND, wave);
        }
    };
    auto h_src = [&](int l) -> RowSrc {        // the residual stream that enters layer l (this XCD's copy)
        return l == 0 ? RowSrc{emb_row, nullptr, tag_of(-1)} : RowSrc{nullptr, ((l - 1) & 1 ? hb1 : hb0) + rep * Hh, tag_of(4 * (l - 1) + 3)};
    };
    // Four plain elements of a row as tagged words / one element as a tagged word (a plain element gets the tag it is
    // expected to carry).
    auto plain_words = [&](const RowSrc& s, int k) -> u32x4 {
        const uint2 r = gload8(s.plain, (uint32_t)k * 2u);
        u32x4 w;
        w.x = (r.x << 16) | s.tag; w.y = (r.x & 0xffff0000u) | s.tag; w.z = (r.y << 16) | s.tag; w.w = (r.y & 0xffff0000u) | s.tag;
        return w;
    };
    auto fetch_word = [&](const RowSrc& s, int ch) -> uint32_t {
        if (s.plain) return ((uint32_t)gload2(s.plain, ch) << 16) | s.tag;
        return ll_ld4(s.words + ch);
    };
    auto finish_word = [&](uint32_t w, const RowSrc& s, int ch) -> float {
        if (!s.plain) {
            int n = 0;
            while ((w & 0xffffu) != s.tag && n++ < a.spin) w = ll_ld4(s.words + ch);
            if ((w & 0xffffu) != s.tag) *a.err = 1;
        }
        return word_value<T>(w);
    };
    auto wbuf_of = [&](auto kc, int pass) -> unsigned char* {
        constexpr int KIND = decltype(kc)::value;
        const bool useA = KIND == K_HEAD ? !(pass & 1) : (KIND == K_IFG || KIND == K_GATE);
        return (useA ? wbufA + wave * a.itemsA * 1024 : wbufB + wave * a.itemsB * 1024);
    };

    // ---- requests made one link ahead
    // packed weights of row-groups [g0, g0 + ng) of this workgroup, this wave's k-slice, into dst
    auto dma_weights = [&](const void* packed, const Geo& g, int g0, int ng, unsigned char* dst) {
        if (g.nkb == 0) return;
        int j = 0;
        for (int gi = 0; gi < ng; ++gi) {
            const int rg = (int)blockIdx.x + kWGs * (g0 + gi);
#pragma unroll
            for (int r = 0; r < 3; ++r) {
                if (r < g.R) {
                    const int nb = (rg >> 2) + r * g.NBseg;
                    const uint32_t s_off = (uint32_t)(nb * g.KB + g.kb0) * 1024u + (uint32_t)(rg & 3) * 128u + lane_off;
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        if (q < g.nq) {
                            int kbl = 4 * q + slot;
                            if (!g.even) kbl = kbl < g.nkb ? kbl : g.nkb - 1;
                            dma16(packed, s_off + (uint32_t)kbl * 1024u, dst + j * 1024);
                            ++j;
                        }
                    }
                }
            }
        }
    };
    // norm weights of this wave's slice (the region of a wave is written and read by that wave only)
    auto dma_norm = [&](auto kc, const unsigned char* rc, const Geo& g) {
        constexpr int KIND = decltype(kc)::value;
        if (g.nkb == 0 || g.NG == 0) return;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            if (q < g.nq) {
                const int el = q * 512 + lane * 8;
                const uint32_t off = (uint32_t)(g.kb0 * 128 + (g.even || el < g.nkb * 128 ? el : 0)) * 2u;
                if constexpr (KIND != K_DOWN) dma16(reinterpret_cast<const void*>(uni64(rc)), off, nrm_w1 + (wave * a.nqmax + q) * 1024);
                dma16(reinterpret_cast<const void*>(uni64(rc + 8)), off, nrm_nw + (wave * a.nqmax + q) * 1024);
            }
        }
    };
    // epilogue operands of this lane for the link that comes next
    auto load_ep = [&](auto kc, const unsigned char* rc, const Geo& g, const RowSrc& add0, const RowSrc& add1) {
        constexpr int KIND = decltype(kc)::value;
        const void* wdeq = reinterpret_cast<const void*>(uni64(rc + 24));
        const bool per_seg = (int)uni32(rc + 72) == g.Nseg;
#pragma unroll
        for (int r = 0; r < 3; ++r)
            if (r < g.R) wdk[KIND][r] = gloadf(wdeq, per_seg ? r : 0);
        if constexpr (KIND == K_IFG) {
            const void* lbp = reinterpret_cast<const void*>(uni64(rc + 32));
            const void* stp = reinterpret_cast<const void*>(uni64(rc + 40));
#pragma unroll
            for (int gi = 0; gi < 2; ++gi) {
                // read here, one link ahead, so that no wave reads a state another wave's epilogue has already replaced
                const int ch = ((int)blockIdx.x + kWGs * gi) * 8 + (lane & 7);
                lb[gi] = 0.0f;
                st[gi] = 0.0f;
                if (gi < g.NG && ch < g.Nseg) {
                    if (lbp) lb[gi] = gloadf(lbp, ch);
                    st[gi] = gloadf(stp, ch);
                }
            }
        }
        if constexpr (KIND == K_DOWN) {
            const int ch = ((int)blockIdx.x + kWGs * wave) * 8 + (lane & 7);
            a0 = a1 = 0u;
            if (wave < g.NG && ch < g.Nseg) { a0 = fetch_word(add0, ch); a1 = fetch_word(add1, ch); }
        }
    };
    // everything link ln (of kind KIND) needs besides its row; called while the link before it computes
    auto request = [&](auto kc, int ln) {
        constexpr int KIND = decltype(kc)::value;
        const Geo g = geo(kc, ln);
        if (g.NG == 0) return;
        const unsigned char* rc = rec(ln);
        const int cap = (KIND == K_IFG || KIND == K_GATE || KIND == K_HEAD ? a.itemsA : a.itemsB) / (g.R * g.nq);   // row-groups a buffer holds
        dma_weights(reinterpret_cast<const void*>(uni64(rc + 16)), g, 0, g.NG < cap ? g.NG : cap, wbuf_of(kc, 0));
        const int l = ln >> 2;
        const RowSrc none{nullptr, nullptr, 0u};
        if constexpr (KIND == K_DOWN) load_ep(kc, rc, g, RowSrc{nullptr, ab + rep * Hh, tag_of(4 * l + 1)}, h_src(l));
        else load_ep(kc, rc, g, none, none);
        if constexpr (KIND == K_GATE) {
            // its second operand, the residual stream, was stored three links ago: read it now, off the link's poll
            const RowSrc hs = h_src(l);
#pragma unroll
            for (int v = 0; v < NPH; ++v) {
                if (v < g.np) {
                    const bool in = g.even || 4 * (64 * v + lane) < g.nkb * 128;
                    const int k = g.kb0 * 128 + (in ? 4 * (64 * v + lane) : 0);
                    auxH[v] = hs.plain ? plain_words(hs, k) : poll_issue(hs.words + k);
                }
            }
        }
    };

    // the integer result of item `it`, row `row`: the waves' partial sums less the row's code sum (weights are stored as t + 1)
    auto total = [&](int it, int row) -> int {
        const int4 p0 = *reinterpret_cast<const int4*>(&sm.part[it][row][0]);
        const int4 p1 = *reinterpret_cast<const int4*>(&sm.part[it][row][4]);
        const int4 qv = *reinterpret_cast<const int4*>(&sm.qs[0]);
        return ((p0.x + p0.y) + (p0.z + p0.w)) + ((p1.x + p1.y) + (p1.z + p1.w)) - ((qv.x + qv.y) + (qv.z + qv.w));
    };
    // Two neighbouring rows' words become one 8-byte store by the even row (fewer, wider stores travel faster); `even_active`:
    // this lane holds an even row that is to be stored.
    auto store_pair = [&](uint32_t* base, int ch, uint32_t word, bool even_active) {
        const uint32_t next = (uint32_t)mmf_dpp<kDppXor1>((int)word);
        if (even_active) ll_st8(reinterpret_cast<uint64_t*>(base + ch), (uint64_t)word | ((uint64_t)next << 32));
    };

    // ---- one link.  NEXT: the kind of the link that follows (its requests are made here, once this link's row is in).
    // kc: the kind of this link; nc: the kind of the link that follows (its requests are made here, once this link's row
    // is in); nc2: the kind that follows instead when `alt` is set (the lm_head after the last down_proj)
    auto link = [&](auto kc, auto nc, auto nc2, bool alt, int ln, bool more) {
        constexpr int KIND = decltype(kc)::value;
        // The lane index as this link sees it.  Made opaque per link: tests on it (lane 0, the epilogue lanes, the even rows)
        // are then a compare where they are used, not masks kept in scalar registers across the whole layer loop, where
        // there are too many of them and they end up spilled and reloaded lane by lane.
        int pl = lane;
        asm volatile("" : "+v"(pl));
        auto request_next = [&] {
            if constexpr (decltype(nc)::value != decltype(nc2)::value) {
                if (alt) { request(nc2, ln + 1); return; }
            }
            request(nc, ln + 1);
        };
        auto dma_norm_next = [&] {
            if constexpr (decltype(nc)::value != decltype(nc2)::value) {
                if (alt) { dma_norm(nc2, rec(ln + 1), geo(nc2, ln + 1)); return; }
            }
            dma_norm(nc, rec(ln + 1), geo(nc, ln + 1));
        };
        constexpr bool HAS_AUX = KIND == K_O || KIND == K_GATE, HAS_W1 = KIND != K_DOWN;
        constexpr int NPK = KIND == K_DOWN ? NP : NPH;                       // passes this link's row can take
        const int l = ln >> 2;
        const Geo g = geo(kc, ln);
        stamp(ln, 0);
        if (g.NG == 0) {
            // nothing of this link falls to this workgroup; it still requests what its next link needs
            if (more) { request_next(); dma_norm_next(); }
            return;
        }
        const unsigned char* rc = rec(ln);
        const RowSrc none{nullptr, nullptr, 0u};
        RowSrc xs = none, as = none, add0 = none, add1 = none;
        if constexpr (KIND == K_IFG) xs = h_src(l);
        if constexpr (KIND == K_O) { xs = RowSrc{nullptr, gb + rep * Hh, tag_of(4 * l)}; as = RowSrc{nullptr, ob + rep * Hh, tag_of(4 * l)}; }
        if constexpr (KIND == K_GATE) { xs = RowSrc{nullptr, ab + rep * Hh, tag_of(4 * l + 1)}; as = h_src(l); }
        if constexpr (KIND == K_DOWN) { xs = RowSrc{nullptr, zb + rep * Ii, tag_of(4 * l + 2)}; add0 = RowSrc{nullptr, ab + rep * Hh, tag_of(4 * l + 1)}; add1 = h_src(l); }
        if constexpr (KIND == K_HEAD) xs = h_src(L);

        // ---- the row (and the prologue's second operand) of this wave's slice: poll until every word carries the tag
        u32x4 X[NPK], A[HAS_AUX ? NPK : 1];
        bool has[NPK];
        int k0[NPK];
#pragma unroll
        for (int v = 0; v < NPK; ++v) {
            has[v] = g.even || 4 * (64 * v + lane) < g.nkb * 128;
            k0[v] = g.kb0 * 128 + (has[v] ? 4 * (64 * v + lane) : 0);
        }
        {
            const bool x_tagged = xs.plain == nullptr, a_tagged = HAS_AUX && as.plain == nullptr;
            if (x_tagged || a_tagged)
                for (int d = 0; d < a.delay[KIND]; ++d) __builtin_amdgcn_s_sleep(1);
#pragma unroll
            for (int v = 0; v < NPK; ++v) {
                if (v < g.np) {
                    X[v] = x_tagged ? poll_issue(xs.words + k0[v]) : plain_words(xs, k0[v]);
                    if constexpr (KIND == K_GATE) A[v] = auxH[v];
                    else if constexpr (HAS_AUX) A[v] = a_tagged ? poll_issue(as.words + k0[v]) : plain_words(as, k0[v]);
                }
            }
            if (x_tagged || a_tagged) {
                for (int n = 0;; ++n) {
                    bool ok = true;
#pragma unroll
                    for (int v = 0; v < NPK; ++v) {
                        if (v < g.np) {
                            if (x_tagged) ok = ok & words_valid(X[v], xs.tag);
                            if constexpr (HAS_AUX) {
                                if (a_tagged) ok = ok & words_valid(A[v], as.tag);
                            }
                        }
                    }
                    if (__builtin_amdgcn_ballot_w64(!ok) == 0) break;
                    if (n >= a.spin) {
                        if (pl == 0) *a.err = 1;
                        break;
                    }
#pragma unroll
                    for (int v = 0; v < NPK; ++v) {
                        if (v < g.np) {
                            if (x_tagged) X[v] = poll_issue(xs.words + k0[v]);
                            if constexpr (HAS_AUX) {
                                if (a_tagged) A[v] = poll_issue(as.words + k0[v]);
                            }
                        }
                    }
                }
            }
        }
        // every load made so far has been waited for (said explicitly: the requests below are not to be waited for here)
        __builtin_amdgcn_s_waitcnt(0x0F70);
        stamp(ln, 1);
        // ---- the row is here: from now on what the next link needs may be requested (it is, below, in the shadow of the
        // first exchange of partial sums)

        // ---- prologue: norms, absmax int8 codes of this wave's slice into LDS
        float xv[NPK][4], av[HAS_AUX ? NPK : 1][4];
#pragma unroll
        for (int v = 0; v < NPK; ++v) {
            const bool on = v < g.np && has[v];
            xv[v][0] = on ? word_value<T>(X[v].x) : 0.0f; xv[v][1] = on ? word_value<T>(X[v].y) : 0.0f;
            xv[v][2] = on ? word_value<T>(X[v].z) : 0.0f; xv[v][3] = on ? word_value<T>(X[v].w) : 0.0f;
            if constexpr (HAS_AUX) {
                av[v][0] = on ? word_value<T>(A[v].x) : 0.0f; av[v][1] = on ? word_value<T>(A[v].y) : 0.0f;
                av[v][2] = on ? word_value<T>(A[v].z) : 0.0f; av[v][3] = on ? word_value<T>(A[v].w) : 0.0f;
            }
        }
        const unsigned char* my_w1 = nrm_w1 + wave * a.nqmax * 1024 + lane * 8;
        const unsigned char* my_nw = nrm_nw + wave * a.nqmax * 1024 + lane * 8;
        const double inv_K = __longlong_as_double((long long)uni64(rc + 48));
        if constexpr (KIND == K_GATE) {
#pragma unroll
            for (int v = 0; v < NPK; ++v)
#pragma unroll
                for (int i = 0; i < 4; ++i) xv[v][i] = __fadd_rn(xv[v][i], av[v][i]);
        }
        if constexpr (HAS_W1) {
            double s1 = 0.0, s1b = 0.0;                         // two chains: half the dependent fp64 operations
#pragma unroll
            for (int v = 0; v < NPK; ++v) {
                s1 = mmf_add_square(mmf_add_square(s1, xv[v][0]), xv[v][1]);
                s1b = mmf_add_square(mmf_add_square(s1b, xv[v][2]), xv[v][3]);
            }
            s1 = mmf_wave_sum(s1 + s1b);
            if (pl == 0) sm.sum1[wave] = s1;
            float sg[KIND == K_O ? NPK : 1][4];
            if constexpr (KIND == K_O) {                          // the swish gate does not wait for the statistics
                // one range test for all of this lane's gate values, then straight-line code whose chains interleave
                bool mid = true;
#pragma unroll
                for (int v = 0; v < NPK; ++v)
#pragma unroll
                    for (int i = 0; i < 4; ++i) mid = mid & (v >= g.np || mmf_sigmoid_mid_ok(av[v][i]));
                if (__builtin_expect(mid, 1)) {
#pragma unroll
                    for (int v = 0; v < NPK; ++v)
#pragma unroll
                        for (int i = 0; i < 4; ++i) sg[v][i] = v < g.np ? mmf_sigmoid_mid(av[v][i]) : 0.0f;
                } else {
#pragma unroll
                    for (int v = 0; v < NPK; ++v)
#pragma unroll
                        for (int i = 0; i < 4; ++i) sg[v][i] = v < g.np ? mmf_sigmoid(av[v][i]) : 0.0f;
                }
            }
            if (more) request_next();                             // while the partial sums settle in LDS
            lds_barrier();
            const double tot = (sm.sum1[0] + sm.sum1[1]) + (sm.sum1[2] + sm.sum1[3]);
            const float rstd1 = mmf_rstd(tot, g.K, inv_K, __uint_as_float(uni32(rc + 60)));
#pragma unroll
            for (int v = 0; v < NPK; ++v) {
                if (v < g.np) {
                    Raw4<T> raw;
                    raw.v = *reinterpret_cast<const uint2*>(my_w1 + v * 512);
                    float w1v[4];
                    raw4_unpack<T>(raw, w1v);
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        float y = __fmul_rn(__fmul_rn(xv[v][i], rstd1), w1v[i]);
                        if constexpr (KIND == K_O) y = __fmul_rn(__fmul_rn(y, av[v][i]), sg[v][i]);
                        xv[v][i] = has[v] ? mmf_round_to<T>(y) : 0.0f;
                    }
                }
            }
        }
        stamp(ln, 2);
        // the BitLinear's own norm
        double ss = 0.0, ssb = 0.0;
#pragma unroll
        for (int v = 0; v < NPK; ++v) {
            ss = mmf_add_square(mmf_add_square(ss, xv[v][0]), xv[v][1]);
            ssb = mmf_add_square(mmf_add_square(ssb, xv[v][2]), xv[v][3]);
        }
        ss = mmf_wave_sum(ss + ssb);
        if (pl == 0) sm.sum2[wave] = ss;
        if constexpr (!HAS_W1) {
            if (more) request_next();
        }
        lds_barrier();
        const double tot2 = (sm.sum2[0] + sm.sum2[1]) + (sm.sum2[2] + sm.sum2[3]);
        const float rstd = mmf_rstd(tot2, g.K, inv_K, __uint_as_float(uni32(rc + 56)));
        stamp(ln, 3);
        float amax = 0.0f;
#pragma unroll
        for (int v = 0; v < NPK; ++v) {
            if (v < g.np) {
                Raw4<T> raw;
                raw.v = *reinterpret_cast<const uint2*>(my_nw + v * 512);
                float wv[4];
                raw4_unpack<T>(raw, wv);
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const float y = has[v] ? __fmul_rn(__fmul_rn(xv[v][i], rstd), wv[i]) : 0.0f;
                    xv[v][i] = y;
                    amax = fmaxf(amax, fabsf(y));
                }
            }
        }
        // this wave is done with its norm-weight regions: the next link's may come in
        if (more) dma_norm_next();
        amax = mmf_wave_max(amax);
        if (pl == 0) sm.amax[wave] = amax;
        lds_barrier();
        amax = fmaxf(fmaxf(sm.amax[0], sm.amax[1]), fmaxf(sm.amax[2], sm.amax[3]));
        stamp(ln, 4);
        const float scale = mmf_127_over(fmaxf(amax, 1e-5f));
        int qs = 0;
#pragma unroll
        for (int v = 0; v < NPK; ++v) {
            if (v < g.np) {
                uint32_t packed4 = 0;
#pragma unroll
                for (int i = 0; i < 4; ++i) packed4 |= (uint32_t)(mmf_code(xv[v][i], scale) & 0xff) << (8 * i);
                qs = __builtin_amdgcn_sdot4((int)packed4, 0x01010101, qs, false);      // the sum of the four codes
                if (has[v]) *reinterpret_cast<uint32_t*>(qbuf + k0[v]) = packed4;
            }
        }
        qs = mmf_wave_sum(qs);
        if (pl == 0) sm.qs[wave] = qs;
        const float deq = mmf_rcp_pos(scale);       // needed by the epilogue only
        stamp(ln, 5);

        const uint32_t tag = tag_of(ln);
        const int rq = g.R * g.nq;
        const int capA = a.itemsA / rq, capB = a.itemsB / rq;
        const int cap0 = (KIND == K_IFG || KIND == K_GATE || KIND == K_HEAD) ? capA : capB;       // row-groups of the first pass
        int g0 = 0;
        for (int pass = 0; g0 < g.NG; ++pass) {
            const int cap = KIND == K_HEAD ? ((pass & 1) ? capB : capA) : cap0;
            const int ng = g.NG - g0 < cap ? g.NG - g0 : cap;
            if (pass > 0) {
                __builtin_amdgcn_s_waitcnt(0x0F70);                   // vmcnt(0): this pass's weights, requested a pass ago, have landed
                lds_barrier();                                        // part[] of the pass before has been read
            }
            if (KIND == K_HEAD || !S::kStatic) {
                // more row-groups than a buffer holds (the lm_head): the next pass's weights travel under this one
                const int gn = g0 + ng;
                if (gn < g.NG) {
                    const int capn = KIND == K_HEAD ? ((pass & 1) ? capA : capB) : cap0;
                    dma_weights(reinterpret_cast<const void*>(uni64(rc + 16)), g, gn, g.NG - gn < capn ? g.NG - gn : capn, wbuf_of(kc, pass + 1));
                }
            }
            // ---- dot products of this wave's slice with the weights of this pass; partial sums to LDS.  The weights were
            // requested a link (or a pass) ago; the wait for everything in flight behind the row's poll (or the one above)
            // has seen them land.  The codes are read back by this wave only: LDS operations of a wave execute in order.
            __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
            if (g.nkb == 0) {
                for (int it = lane >> 4; it < ng * g.R; it += 4)
                    if ((pl & 15) < 8) { sm.part[it][pl & 7][2 * wave] = 0; sm.part[it][pl & 7][2 * wave + 1] = 0; }
            } else if constexpr (S::kStatic && KIND != K_HEAD) {
                // the shape is known: every LDS read of the pass (weights, codes) is issued before the first product
                constexpr int KK = KIND == K_DOWN ? S::I : S::H;
                constexpr int NQ = quads_of(KK);
                constexpr int MAXIT = ceil_div_c((KIND == K_GATE ? S::I : S::H) / 8, kWGs) * (KIND == K_IFG ? 3 : KIND == K_GATE ? 2 : 1);
                const unsigned char* src = wbuf_of(kc, pass) + lane * 16;
                const int nit = ng * g.R;
                uint4 wq[MAXIT][NQ];
                int4 qv[NQ][4];
#pragma unroll
                for (int q = 0; q < NQ; ++q) {
                    const int kraw = 4 * q + slot;
                    const int kb = g.kb0 + (g.even || kraw < g.nkb ? kraw : g.nkb - 1);
#pragma unroll
                    for (int s4 = 0; s4 < 4; ++s4) qv[q][s4] = *reinterpret_cast<const int4*>(qbuf + kb * 128 + s4 * 32 + half * 16);
                }
#pragma unroll
                for (int it = 0; it < MAXIT; ++it)
#pragma unroll
                    for (int q = 0; q < NQ; ++q) {
                        wq[it][q] = make_uint4(0u, 0u, 0u, 0u);
                        if (it < nit && (g.even || 4 * q + slot < g.nkb)) wq[it][q] = *reinterpret_cast<const uint4*>(src + (it * NQ + q) * 1024);
                    }
                int acc[MAXIT];
#pragma unroll
                for (int it = 0; it < MAXIT; ++it) {
                    acc[it] = 0;
#pragma unroll
                    for (int q = 0; q < NQ; ++q) acc[it] = mmf_dot_block_regs(qv[q], wq[it][q], acc[it]);
                    acc[it] += mmf_dpp<0x128>(acc[it]);                      // the other half of the 16 lanes (rotate by 8)
                }
#pragma unroll
                for (int it = 0; it < MAXIT; ++it) acc[it] += __builtin_amdgcn_ds_swizzle(acc[it], 0x401F);   // lane ^ 16: the neighbouring k-block
#pragma unroll
                for (int it = 0; it < MAXIT; ++it)
                    if (it < nit && (pl & 31) < 8) sm.part[it][pl & 7][2 * wave + (pl >> 5)] = acc[it];
            } else {
                const unsigned char* src = wbuf_of(kc, pass) + lane * 16;
                const int nit = ng * g.R;
                for (int it = 0; it < nit; ++it) {
                    int acc = 0;
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        if (q < g.nq) {
                            const int kraw = 4 * q + slot;
                            const bool live = g.even || kraw < g.nkb;
                            const int kb = g.kb0 + (live ? kraw : g.nkb - 1);
                            uint4 wq = *reinterpret_cast<const uint4*>(src + (it * g.nq + q) * 1024);
                            if (!live) wq = make_uint4(0u, 0u, 0u, 0u);
                            acc = mmf_dot_block(qbuf, wq, kb, half, acc);
                        }
                    }
                    acc += mmf_dpp<0x128>(acc);                              // the other half of the 16 lanes (rotate by 8)
                    acc += __builtin_amdgcn_ds_swizzle(acc, 0x401F);         // lane ^ 16: the neighbouring k-block
                    if ((pl & 31) < 8) sm.part[it][pl & 7][2 * wave + (pl >> 5)] = acc;
                }
            }
            stamp(ln, 6);
            lds_barrier();
            stamp(ln, 7);
            // ---- epilogue
            if constexpr (KIND == K_IFG) {
                // a wave serves two copies: lanes 0-23 of each 32-lane half run the i, f and g rows of the 8 channels side
                // by side, so the two exp / divide chains of the gate math run in parallel; the f lanes' gate reaches the i
                // lanes by a rotate within the 16-lane row.  Operation for operation the arithmetic of the single-lane form.
                const int r3 = (pl & 31) >> 3, row = pl & 7, copy = 2 * wave + (pl >> 5);
                const void* lbp = reinterpret_cast<const void*>(uni64(rc + 32));
                float* stp = reinterpret_cast<float*>(uni64(rc + 40));
#pragma unroll
                for (int gl = 0; gl < 2; ++gl) {
                    if (gl >= ng) break;
                    const int ch = ((int)blockIdx.x + kWGs * (g0 + gl)) * 8 + row;
                    const float lbv = g0 + gl == 0 ? lb[0] : lb[1], stv = g0 + gl == 0 ? st[0] : st[1];
                    const int tot = total(gl * 3 + (r3 < 3 ? r3 : 0), row);
                    const float wdv = r3 == 0 ? wdk[KIND][0] : r3 == 1 ? wdk[KIND][1] : wdk[KIND][2];
                    const float res = __fmul_rn(__fmul_rn((float)tot, deq), wdv);
                    const float v16 = mmf_round_to<T>(res);                       // iv on the i lanes, fv on the f lanes
                    const float ex = __fadd_rn(1.0f, mmf_exp(-v16));
                    float sgm = mmf_rcp_pos(ex);                                 // sigmoid(fv) on the f lanes
                    if (lbp) sgm = __fadd_rn(lbv, __fmul_rn(__fsub_rn(1.0f, lbv), sgm));
                    const float go = mmf_dpp<0x128>(mmf_round_to<T>(sgm));        // lanes 0-7 read lanes 8-15
                    const float xo = mmf_round_to<T>(__fdiv_rn(__fmul_rn(v16, __fsub_rn(1.0f, go)), ex));
                    const float h = __fadd_rn(__fmul_rn(go, stv), xo);
                    const bool live = ch < g.Nseg;
                    if (live && r3 == 0 && copy == 0) ((MMF_AS_GLOBAL float*)stp)[ch] = h;
                    store_pair(ob + copy * Hh, ch, make_word<T>(h, tag), live && r3 == 0 && !(pl & 1));
                    store_pair(gb + copy * Hh, ch, make_word<T>(res, tag), live && r3 == 2 && !(pl & 1));
                }
            } else if constexpr (KIND == K_HEAD) {
                const int row = pl & 7;                                   // a wave takes 8 row-groups of a pass
                for (int gl = wave * 8 + (pl >> 3); gl < ng; gl += 8 * kNW) {
                    const int ch = ((int)blockIdx.x + kWGs * (g0 + gl)) * 8 + row;
                    if (ch < g.Nseg) {
                        const float o = __fmul_rn(__fmul_rn((float)total(gl, row), deq), wdk[KIND][0]);
                        static_cast<T*>(a.logits)[ch] = mmf_from_float<T>(o);
                        const float ov = mmf_round_to<T>(o);
                        if (ov == ov) best_take(best, ov, (uint32_t)ch);
                    }
                }
            } else {
                // 8 x 8 lanes are copy x row, one row-group per wave: o_proj, gate/up, down
                const int row = pl & 7, copy = pl >> 3;
                uint32_t* out = KIND == K_O ? ab : KIND == K_GATE ? zb : ((l & 1) ? hb1 : hb0);
                const int out_n = KIND == K_GATE ? Ii : Hh;
                for (int gl = wave; gl < ng; gl += kNW) {
                    const int ch = ((int)blockIdx.x + kWGs * (g0 + gl)) * 8 + row;
                    const bool live = ch < g.Nseg;
                    float o = __fmul_rn(__fmul_rn((float)total(gl * g.R, row), deq), wdk[KIND][0]);
                    if constexpr (KIND == K_GATE) {
                        const float u = mmf_round_to<T>(__fmul_rn(__fmul_rn((float)total(gl * 2 + 1, row), deq), wdk[KIND][1]));
                        const float gt = mmf_round_to<T>(o);
                        o = __fdiv_rn(__fmul_rn(gt, u), __fadd_rn(1.0f, mmf_exp(-gt)));
                    }
                    if constexpr (KIND == K_DOWN) {
                        // the residual it adds is T(attn + h), formed here from its two operands
                        uint32_t w0 = a0, w1 = a1;
                        if (g0 + gl != wave && live) { w0 = fetch_word(add0, ch); w1 = fetch_word(add1, ch); }
                        float r0 = 0.0f, r1 = 0.0f;
                        if (live) { r0 = finish_word(w0, add0, ch); r1 = finish_word(w1, add1, ch); }
                        o = __fadd_rn(mmf_round_to<T>(o), mmf_round_to<T>(__fadd_rn(r0, r1)));
                    }
                    store_pair(out + copy * out_n, ch, make_word<T>(o, tag), live && !(pl & 1));
                    if (KIND == K_DOWN && l == L - 1 && live && copy == 0) static_cast<T*>(a.h_out)[ch] = mmf_from_float<T>(o);
                }
            }
            stamp(ln, 8);
            g0 += ng;
        }
    };
    request(KIfg{}, 0);
    dma_norm(KIfg{}, rec(0), geo(KIfg{}, 0));
    for (int l = 0; l < L; ++l) {
        const bool last = l == L - 1;
        link(KIfg{}, KO{}, KO{}, false, 4 * l, true);
        link(KO{}, KGate{}, KGate{}, false, 4 * l + 1, true);
        link(KGate{}, KDown{}, KDown{}, false, 4 * l + 2, true);
        link(KDown{}, KIfg{}, KHead{}, last, 4 * l + 3, !last || a.head != nullptr);
    }
    if (a.head) {
        link(KHead{}, KHead{}, KHead{}, false, 4 * L, false);
        // this workgroup's candidate for the greedy token, then workgroup 0 combines the candidates
        const uint32_t tag_h = tag_of(4 * L);
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

template <typename T, class S, bool TRACE>
int launch_one(const LayersArgs& a, size_t lds, hipStream_t s) {
    auto kern = decode_layers_kernel<T, S, TRACE>;
    static size_t allowed = 0;                                   // per instantiation; the attribute only ever grows
    if (lds > allowed) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return (int)e;
        allowed = lds;
    }
    kern<<<kWGs, kNT, lds, s>>>(a);
    MMF_CHECK_LAUNCH();
    return 0;
}

template <typename T, bool TRACE>
int launch_layers(LayersArgs a, hipStream_t s) {
    const int kmax = a.H > a.I ? a.H : a.I;
    a.nqmax = quads_of(kmax);
    // weight loads (1 KiB each) per wave a link kind needs when all its row-groups are resident: buffer A serves i/f/g
    // and gate/up, buffer B o_proj and down_proj; the lm_head takes what they hold, pass by pass
    const int nqh = quads_of(a.H), nqi = quads_of(a.I);
    const int ngh = ceil_div_c(a.D / 8, kWGs), ngi = ceil_div_c(a.I / 8, kWGs);
    const int ifg = ngh * 3 * nqh, gate = ngi * 2 * nqh, o = ngh * nqh, down = ngh * nqi;
    a.itemsA = ifg > gate ? ifg : gate;
    a.itemsB = o > down ? o : down;
    if (a.itemsA > 16 || a.itemsB > 16 || ngh > 2 || ngi * 2 > kItems) return MMF_ERR_WIDE;
    const uint32_t tab = (uint32_t)mmf_round_up((4 * a.n_layers + 1) * (int64_t)sizeof(Phase), 16);
    a.off_q = tab;
    a.off_nrm = a.off_q + (uint32_t)mmf_round_up(kmax, 16);
    a.off_w = a.off_nrm + 2u * kNW * (uint32_t)a.nqmax * 1024u;
    const size_t lds = a.off_w + (size_t)kNW * (a.itemsA + a.itemsB) * 1024u;
    if (a.H == 2048 && a.I == 5632) return launch_one<T, StaticShape<2048, 5632>, TRACE>(a, lds, s);
    if (a.H == 2560 && a.I == 6912) return launch_one<T, StaticShape<2560, 6912>, TRACE>(a, lds, s);
    return launch_one<T, DynShape, TRACE>(a, lds, s);
}

int decode_layers_entry(const void* phases, int n_layers, const void* table, const int64_t* tok, int64_t vocab, uint32_t* words,
                        void* h_out, const void* head, void* logits, uint64_t* am_words, int64_t* tok_out, uint32_t* epoch, int* err,
                        int64_t* trace, int H, int D, int I, int spin, const int* delay, int dtype, void* stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (!phases || n_layers <= 0 || !table || !tok || vocab <= 0 || !words || !h_out || !epoch || !err || H <= 0 || D <= 0 || I <= 0 ||
        spin <= 0 || !delay)
        return MMF_ERR_ARG;
    for (int k = 0; k < 5; ++k)
        if (delay[k] < 0 || delay[k] > 64) return MMF_ERR_ARG;
    if (head && (!logits || !am_words || !tok_out)) return MMF_ERR_ARG;
    if (H % 128 != 0 || D != H || I % 128 != 0) return MMF_ERR_ARG;      // rows are whole k-blocks: no ragged tail in a link
    if (dtype != MMF_BF16 && dtype != MMF_F16) return MMF_ERR_ARG;        // a tagged word carries a 16-bit value
    if (H > 4096 || I > 8192 || n_layers > kMaxLayers) return MMF_ERR_WIDE;
    for (const void* p : {(const void*)words, (const void*)table, (const void*)h_out, phases, head})
        if (reinterpret_cast<uintptr_t>(p) & 15u) return MMF_ERR_ALIGN;
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess)
        return MMF_ERR_ARG;
    if (cus < kWGs) return MMF_ERR_ARG;                                       // the resident grid needs one CU per workgroup
    LayersArgs a{};
    a.phases = static_cast<const Phase*>(phases); a.n_layers = n_layers; a.table = table; a.tok = tok; a.vocab = vocab;
    a.words = words; a.h_out = h_out; a.head = static_cast<const Phase*>(head); a.logits = logits; a.am_words = am_words;
    a.tok_out = tok_out; a.epoch = epoch; a.err = err; a.trace = reinterpret_cast<long long*>(trace);
    a.H = H; a.D = D; a.I = I; a.spin = spin;
    for (int k = 0; k < 5; ++k) a.delay[k] = delay[k];
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
    // hold-back of the first poll per kind of link (i/f/g, o_proj, gate/up, down_proj, lm_head); MMF_DECODE_POLL_DELAY
    // ("a" or "a,b,c,d,e") overrides the tuned values
    static const struct Delays {
        int d[5] = {8, 14, 22, 22, 8};
        Delays() {
            const char* v = getenv("MMF_DECODE_POLL_DELAY");
            if (!v) return;
            int k = 0, last = 6;
            while (*v && k < 5) {
                last = atoi(v);
                d[k++] = last < 0 ? 0 : last > 64 ? 64 : last;
                while (*v && *v != ',') ++v;
                if (*v == ',') ++v;
            }
            for (; k < 5; ++k) d[k] = last < 0 ? 0 : last > 64 ? 64 : last;
        }
    } delays;
    const int* delay = delays.d;
    return decode_layers_entry(phases, n_layers, table, tok, vocab, words, h_out, head, logits, am_words, tok_out, epoch, err, nullptr,
                               H, D, I, spin, delay, dtype, stream);
}

int mmf_decode_layers_trace_words(void) { return kTraceWGs * kTraceLinks * kTraceStamps; }

int mmf_decode_layers_traced(const void* phases, int n_layers, const void* table, const int64_t* tok, int64_t vocab, uint32_t* words,
                             void* h_out, const void* head, void* logits, uint64_t* am_words, int64_t* tok_out, uint32_t* epoch, int* err,
                             int64_t* trace, int H, int D, int I, int spin, int delay, int dtype, void* stream) {
    if (!trace) return MMF_ERR_ARG;
    const int d[5] = {delay, delay, delay, delay, delay};
    return decode_layers_entry(phases, n_layers, table, tok, vocab, words, h_out, head, logits, am_words, tok_out, epoch, err, trace, H, D,
                               I, spin, d, dtype, stream);
}

}  // extern "C"
