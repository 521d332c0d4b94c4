// Top-p (nucleus) sampling of one token per row of logits, in one launch and without a sort.
//
// Replaces, for the loop that mmfreelm's generate.py:11 runs (model.generate(do_sample=True, top_p=0.4,
// temperature=0.6)), the per-token chain temperature scaling -> softmax -> descending sort -> cumulative sum ->
// nucleus mask -> renormalise -> multinomial draw that transformers' sampling path performs on the logits of
// HGRNBitForCausalLM.forward (mmfreelm/models/hgrn_bit/modeling_hgrn_bit.py:386).
//
// Every decision is made on integers, so the result does not depend on any summation order and a CPU restatement
// reproduces it exactly:
//   l_i   = logit_i / temperature                      (fp32 division; NaN counts as -inf)
//   p_i   = 1 if l_i == max l, else exp(l_i - max l)   (the deterministic fp32 exp of mmf_common.h)
//   top_k > 0:  l_i = -inf unless l_i >= the top_k-th largest l        (transformers' TopKLogitsWarper, which the
//               reference's call gets from the default generation parameters, top_k = 50; equal values stay together)
//   m_i   = trunc(p_i * 2^31)                          (uint32 probability mass; the row maximum has 2^31)
//   Z     = sum m_i,  P = max(1, trunc(double(top_p) * double(Z)))
//   keep i  iff  m_i > 0 and  sum{ m_j : m_j > m_i } < P     (the smallest set of most probable tokens whose mass
//                                                             reaches top_p; tokens of equal mass stay together)
//   S     = sum of kept m_i,  target = trunc(double(u) * double(S)),  u in [0, 1) supplied by the caller
//   token = the lowest index whose running sum of kept masses (in index order) exceeds target.
//
// One workgroup of 1024 threads per row; a thread owns NPT consecutive vocabulary entries and keeps their masses in
// registers.  The nucleus threshold (the smallest kept mass) is found by a radix descent over the 32-bit mass, 8 bits
// a pass: a 256-bin histogram of mass (LDS atomics on 64-bit integers, 16 interleaved copies of every bin so that
// neighbouring lanes hit different banks; a thread merges runs of equal bins before it touches LDS), a suffix scan of
// the bins by one wave, and the digit whose bin straddles P.  The top_k-th largest scaled logit comes from the same
// descent on token counts over an order-preserving integer image of the floats, BEFORE the exp: only the kept tokens
// (some 50 of 32000) then pay for it.
#include "mmf_common.h"

namespace {

typedef unsigned long long u64;
constexpr int kSampThreads = 1024, kSampWaves = 16, kSampBins = 256, kSampCopies = 16;
constexpr int64_t kSampMaxV = 65536;

struct SampleArgs {
    const void* logits;
    int64_t ld;
    int V;
    float temperature, top_p;
    int top_k;              // 0: no limit
    const float* u;
    int64_t* out;
};

__device__ __forceinline__ u64 samp_shfl_down(u64 v, int o) {
    const unsigned lo = (unsigned)__shfl_down((int)(unsigned)v, o, 64), hi = (unsigned)__shfl_down((int)(unsigned)(v >> 32), o, 64);
    return ((u64)hi << 32) | lo;
}
__device__ __forceinline__ u64 samp_shfl_up(u64 v, int o) {
    const unsigned lo = (unsigned)__shfl_up((int)(unsigned)v, o, 64), hi = (unsigned)__shfl_up((int)(unsigned)(v >> 32), o, 64);
    return ((u64)hi << 32) | lo;
}

// Radix descent over the 32-bit masses, 8 bits a pass.  With W(S) the mass (COUNT false) or the number (COUNT true) of
// the non-zero entries in S, returns the lowest v with W({m > v}) < limit: the smallest kept mass of the nucleus, or the
// limit-th largest mass.  prefix = the high digits found so far, above = W of everything larger than any mass with that prefix.
template <bool COUNT, int NPT>
__device__ __forceinline__ unsigned samp_descent(const unsigned (&m)[NPT], u64 limit, u64* hist, u64* hsum, u64* sel) {
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const u64 P = limit;
    unsigned prefix = 0;
    u64 above = 0;
#pragma unroll
    for (int pass = 0; pass < 4; ++pass) {
        const int shift = 24 - 8 * pass;
        int cur = -1;
        u64 acc = 0;
#pragma unroll
        for (int j = 0; j < NPT; ++j) {
            const unsigned mj = m[j];
            const bool match = mj != 0 && (pass == 0 || (mj >> ((shift + 8) & 31)) == prefix);
            if (match) {
                const int b = (int)((mj >> shift) & 255u);
                if (b != cur) {
                    if (cur >= 0) atomicAdd(&hist[cur * kSampCopies + (lane & (kSampCopies - 1))], acc);
                    cur = b;
                    acc = 0;
                }
                acc += COUNT ? 1u : mj;
            }
        }
        if (cur >= 0) atomicAdd(&hist[cur * kSampCopies + (lane & (kSampCopies - 1))], acc);
        __syncthreads();
        if (t < kSampBins) {
            u64 h = 0;
#pragma unroll
            for (int c = 0; c < kSampCopies; ++c) {
                const int s = t * kSampCopies + ((c + t) & (kSampCopies - 1));   // rotated: lanes start on different banks
                h += hist[s];
                hist[s] = 0;                                                     // ready for the next pass
            }
            hsum[t] = h;
        }
        __syncthreads();
        if (wave == 0) {
            // lane owns bins 4*lane .. 4*lane+3; A(d) = above + mass of the bins over d; take the lowest d with A(d) < P
            u64 h[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) h[i] = hsum[lane * 4 + i];
            const u64 mine = h[0] + h[1] + h[2] + h[3];
            u64 suf = mine;                                       // inclusive suffix sum over the lanes
#pragma unroll
            for (int o = 1; o < 64; o <<= 1) {
                const u64 y = samp_shfl_down(suf, o);
                if (lane + o < 64) suf += y;
            }
            u64 A = above + (suf - mine);                         // mass over this lane's bins
            int best = 256;
            u64 bestA = 0;
#pragma unroll
            for (int i = 3; i >= 0; --i) {
                if (A < P) { best = lane * 4 + i; bestA = A; }
                A += h[i];
            }
            int lowest = best;
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) lowest = min(lowest, __shfl_xor(lowest, o, 64));
            if (best == lowest && best < 256) { sel[0] = bestA; sel[1] = (u64)best; }
        }
        __syncthreads();
        above = sel[0];
        prefix = (prefix << 8) | (unsigned)sel[1];
    }
    return prefix;
}

template <typename T, int NPT>
__global__ __launch_bounds__(kSampThreads) void sample_top_p_kernel(SampleArgs a) {
    __shared__ u64 hist[kSampBins * kSampCopies];                // 32 KiB
    __shared__ u64 hsum[kSampBins];
    __shared__ u64 wtot[kSampWaves], wtot2[kSampWaves];
    __shared__ u64 sel[2];
    __shared__ float wmax[kSampWaves];
    __shared__ int wcand[kSampWaves];
    __shared__ int few_n, few_i[64];
    __shared__ unsigned few_m[64];
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int V = a.V;
    const T* row = static_cast<const T*>(a.logits) + (int64_t)blockIdx.x * a.ld;
    const int base = t * NPT;
    const bool vec_ok = (V % 8) == 0 && (a.ld % 8) == 0 && (reinterpret_cast<uintptr_t>(a.logits) & 15u) == 0;

    Raw8<T> raw[NPT / 8];
#pragma unroll
    for (int c = 0; c < NPT / 8; ++c) raw[c] = mmf_load8_raw<T>(row, (int64_t)base + c * 8, V, vec_ok);
#pragma unroll
    for (int i = 0; i < kSampBins * kSampCopies / kSampThreads; ++i) hist[i * kSampThreads + t] = 0;

    float l[NPT];
    float mx = -INFINITY;
#pragma unroll
    for (int c = 0; c < NPT / 8; ++c) {
        float v[8];
        mmf_unpack8<T>(raw[c], v);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int idx = base + c * 8 + i;
            float x = v[i];
            x = (idx < V && x == x) ? __fdiv_rn(x, a.temperature) : -INFINITY;
            l[c * 8 + i] = x;
            mx = fmaxf(mx, x);
        }
    }
    mx = mmf_wave_max(mx);
    if (lane == 0) wmax[wave] = mx;
    __syncthreads();                                              // also publishes the zeroed histogram
#pragma unroll
    for (int w = 0; w < kSampWaves; ++w) mx = fmaxf(mx, wmax[w]);

    unsigned m[NPT];
    if (a.top_k > 0 && a.top_k < V && mx != -INFINITY) {          // a row without a finite logit has no top_k-th largest: it is drawn
                                                                   // uniformly like without the limit (every mass is 2^31)
        // order-preserving image of the scaled logits: non-negative floats above the negative ones, -inf and the slots
        // past V at 0 (which the descent ignores)
#pragma unroll
        for (int j = 0; j < NPT; ++j) {
            const unsigned b = __float_as_uint(__fadd_rn(l[j], 0.0f));       // -0 counts as +0, as the comparison of floats does
            m[j] = l[j] == -INFINITY ? 0u : (b & 0x80000000u) ? ~b : (b | 0x80000000u);
        }
        const unsigned kth = samp_descent<true, NPT>(m, (u64)a.top_k, hist, hsum, sel);
        // the kept tokens (top_k of them, more on ties) with their masses, in any order, for one wave to finish
        if (t == 0) few_n = 0;
        __syncthreads();
#pragma unroll
        for (int j = 0; j < NPT; ++j) {
            const bool keep = m[j] != 0u && m[j] >= kth;
            float p = 0.0f;
            if (__builtin_amdgcn_ballot_w64(keep) != 0) {         // wave-uniform: most waves skip the exp for most slots
                p = l[j] == mx ? 1.0f : mmf_exp(__fsub_rn(l[j], mx));
                p = keep ? p : 0.0f;
            }
            m[j] = (unsigned)__fmul_rn(p, 2147483648.0f);
            if (keep) {
                const int pos = atomicAdd(&few_n, 1);
                if (pos < 64) { few_m[pos] = m[j]; few_i[pos] = base + j; }
            }
        }
        __syncthreads();
        const int n = few_n;
        if (n <= 64) {
            // Few enough for one lane each: the nucleus and the draw by direct comparison (64 x 64), same rule as below.
            if (wave == 0) {
                const unsigned mi = lane < n ? few_m[lane] : 0u;
                const int ii = lane < n ? few_i[lane] : 0x7fffffff;
                u64 Zf = mi;
#pragma unroll
                for (int o = 32; o > 0; o >>= 1) Zf += samp_shfl_down(Zf, o);
                Zf = ((u64)(unsigned)__builtin_amdgcn_readfirstlane((int)(Zf >> 32)) << 32) | (unsigned)__builtin_amdgcn_readfirstlane((int)Zf);
                u64 Pf = (u64)((double)a.top_p * (double)Zf);
                if (Pf < 1) Pf = 1;
                u64 heavier = 0;
#pragma unroll
                for (int j = 0; j < 64; ++j) {
                    const unsigned mj = (unsigned)__builtin_amdgcn_readlane((int)mi, j);
                    heavier += mj > mi ? mj : 0u;
                }
                const unsigned kept = (mi != 0u && heavier < Pf) ? mi : 0u;
                u64 Sf = kept;
#pragma unroll
                for (int o = 32; o > 0; o >>= 1) Sf += samp_shfl_down(Sf, o);
                Sf = ((u64)(unsigned)__builtin_amdgcn_readfirstlane((int)(Sf >> 32)) << 32) | (unsigned)__builtin_amdgcn_readfirstlane((int)Sf);
                float uf = a.u[blockIdx.x];
                uf = uf >= 0.0f ? uf : 0.0f;
                u64 target = (u64)((double)uf * (double)Sf);
                if (target >= Sf) target = Sf - 1;
                u64 before = 0;                                   // kept mass at lower vocabulary indices
#pragma unroll
                for (int j = 0; j < 64; ++j) {
                    const unsigned kj = (unsigned)__builtin_amdgcn_readlane((int)kept, j);
                    const int ij = __builtin_amdgcn_readlane(ii, j);
                    before += ij < ii ? kj : 0u;
                }
                if (kept != 0u && before <= target && target < before + kept) a.out[blockIdx.x] = ii;
            }
            return;
        }
    } else {
#pragma unroll
        for (int j = 0; j < NPT; ++j) {
            const float p = l[j] == mx ? 1.0f : mmf_exp(__fsub_rn(l[j], mx));
            m[j] = base + j < V ? (unsigned)__fmul_rn(p, 2147483648.0f) : 0u;
        }
    }
    u64 zs = 0;
#pragma unroll
    for (int j = 0; j < NPT; ++j) zs += m[j];
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) zs += samp_shfl_down(zs, o);
    if (lane == 0) wtot[wave] = zs;
    __syncthreads();
    u64 Z = 0;
#pragma unroll
    for (int w = 0; w < kSampWaves; ++w) Z += wtot[w];
    u64 P = (u64)((double)a.top_p * (double)Z);
    if (P < 1) P = 1;

    // ---- the nucleus: the smallest kept mass
    const unsigned thr = samp_descent<false, NPT>(m, P, hist, hsum, sel);

    // ---- the draw: inverse CDF over the kept masses in index order
    u64 s = 0;
#pragma unroll
    for (int j = 0; j < NPT; ++j) s += m[j] >= thr ? m[j] : 0u;
    u64 inc = s;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
        const u64 y = samp_shfl_up(inc, o);
        if (lane >= o) inc += y;
    }
    if (lane == 63) wtot2[wave] = inc;
    __syncthreads();
    u64 S = 0, before = 0;
#pragma unroll
    for (int w = 0; w < kSampWaves; ++w) {
        const u64 x = wtot2[w];
        S += x;
        if (w < wave) before += x;
    }
    float u = a.u[blockIdx.x];
    u = u >= 0.0f ? u : 0.0f;                                     // NaN and negatives draw the first kept token
    u64 target = (u64)((double)u * (double)S);
    if (target >= S) target = S - 1;                              // u >= 1
    u64 run = before + inc - s;
    int cand = 0x7fffffff;
#pragma unroll
    for (int j = 0; j < NPT; ++j) {
        if (m[j] >= thr) {
            run += m[j];
            if (run > target && cand == 0x7fffffff) cand = base + j;
        }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) cand = min(cand, __shfl_xor(cand, o, 64));
    if (lane == 0) wcand[wave] = cand;
    __syncthreads();
    if (t == 0) {
#pragma unroll
        for (int w = 0; w < kSampWaves; ++w) cand = min(cand, wcand[w]);
        a.out[blockIdx.x] = cand < V ? cand : 0;
    }
}

template <typename T>
int launch_sample(const SampleArgs& a, int64_t rows, hipStream_t s) {
    if (a.V <= 32 * kSampThreads) sample_top_p_kernel<T, 32><<<(unsigned)rows, kSampThreads, 0, s>>>(a);
    else sample_top_p_kernel<T, 64><<<(unsigned)rows, kSampThreads, 0, s>>>(a);
    MMF_CHECK_LAUNCH();
    return 0;
}

}  // namespace

extern "C" {

int64_t mmf_sample_top_p_max_vocab(void) { return kSampMaxV; }

int mmf_sample_top_p(const void* logits, int64_t ld, int64_t rows, int64_t V, float temperature, float top_p,
                     int64_t top_k, const float* u, int64_t* out, int dtype, void* stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (rows < 0 || V <= 0 || ld < V || rows > 0x7fffffff || top_k < 0) return MMF_ERR_ARG;
    if (!(temperature > 0.0f) || !(top_p == top_p)) return MMF_ERR_ARG;
    if (rows == 0) return 0;
    if (!logits || !u || !out) return MMF_ERR_ARG;
    if (V > kSampMaxV) return MMF_ERR_WIDE;
    SampleArgs a{};
    a.logits = logits; a.ld = ld; a.V = (int)V; a.temperature = temperature;
    a.top_p = top_p < 0.0f ? 0.0f : top_p > 1.0f ? 1.0f : top_p;
    a.top_k = top_k >= V ? 0 : (int)top_k;
    a.u = u; a.out = out;
    switch (dtype) {
        case MMF_F32: return launch_sample<float>(a, rows, stream);
        case MMF_BF16: return launch_sample<bf16_t>(a, rows, stream);
        case MMF_F16: return launch_sample<f16_t>(a, rows, stream);
    }
    return MMF_ERR_ARG;
}

}  // extern "C"
