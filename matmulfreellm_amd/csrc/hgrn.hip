// HGRN recurrence  h_t = g_t * h_{t-1} + x_t  and the gate math in front of it.
//
//   mmf_hgrn_recurrent : g is the decay itself (linear domain); strictly sequential
//                        arithmetic (multiply, round, add, round) like
//                        mmfreelm/ops/hgrn/recurrent_fuse.py:32-68 / ops/hgrn/naive.py:8-31.
//   mmf_hgrn_chunk     : g is the log decay; the chunked evaluation of
//                        mmfreelm/ops/hgrn/chunk.py:49-116, 223-254 (per chunk a scan from zero and the
//                        running sum of log gates, then o_t += exp(gc_t) * (last output of the chunk
//                        before)) in one pass with the chunk's values in registers instead of
//                        chunk.py:232-233's two fp32 [B,H,T,D] scratch tensors; the time axis is cut into
//                        segments that run in parallel when batch * channels alone do not fill the chip.
//   mmf_hgrn_gate      : sigmoid / lower bound / swiglu / mask of
//                        mmfreelm/layers/hgrn_bit.py:113-120 as one elementwise pass.
//   mmf_hgrn_step      : the same gate math fused with one recurrence step (decode, T = 1).
//
// Layout: x, g, o are [BH, T, D] contiguous; a lane owns one channel d, a wave 64
// consecutive channels (128 B per time step in bf16), a workgroup of 8 waves one
// 64-channel column of one (b, h).  Time is cut into chunks of 64 steps; a wave holds a
// whole chunk of x and g in registers, and the waves take turns ("baton" = running state
// in LDS): on its turn a wave runs its 64 dependent steps from registers and hands the
// state on, so the serial chain sees no memory latency while the other waves' loads and
// stores are in flight.
#include <type_traits>
#include "mmf_common.h"
#include "../../include/mmf.h"

namespace {

constexpr int kCH = 64;   // time steps per register-resident chunk

// -------------------------------------------------------------------------- recurrence
// A wave's memory work is spread over the rounds between its turns.  Issuing a chunk's 64
// stores and the next chunk's 128 loads in one go overruns the 64-deep vector-memory queue and
// puts a full memory round trip inside every round; here each of the four rounds after a turn
// issues 16 stores and 32 loads, so a round lasts as long as one wave's 64 dependent steps and
// the waiting waves keep ~40 KiB in flight.
//
// Every wave runs the same straight-line iteration (turn, four memory rounds, three idle
// rounds: eight barriers), entered `wave` barriers late, so the register arrays are never
// assigned under a branch and stay where they are.  Memory goes through buffer instructions:
// the resource holds the chunk base, the lane's byte offset sits in one VGPR and the row offset
// in one SGPR.  What must not happen is switched off without a branch: a resource of zero
// records turns the loads past the last chunk into zeros and drops the stores of the padding
// chunks, lanes past D carry an out-of-range offset, the tail chunk clamps its row index for
// loads and feeds the missing steps (g, x) = (1, -0), which leaves the state bit for bit.
template <typename R>
__device__ __forceinline__ R buf_load(__amdgpu_buffer_rsrc_t r, uint32_t voff, uint32_t soff) {
    if constexpr (sizeof(R) == 4) return __uint_as_float((uint32_t)__builtin_amdgcn_raw_buffer_load_b32(r, voff, soff, 0));
    else return (R)__builtin_amdgcn_raw_buffer_load_b16(r, voff, soff, 0);
}
template <typename T>
__device__ __forceinline__ void buf_store(float v, __amdgpu_buffer_rsrc_t r, uint32_t voff, uint32_t soff) {
    if constexpr (sizeof(T) == 4) {
        __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(v), r, voff, soff, 0);
    } else {
        T t = mmf_from_float<T>(v);
        __builtin_amdgcn_raw_buffer_store_b16(mmf_bits16(t), r, voff, soff, 0);
    }
}
template <typename T, typename R>
__device__ __forceinline__ float raw_get(R v) {
    if constexpr (sizeof(T) == 4) return v;
    else return mmf_to_float(mmf_from_bits16<T>((uint16_t)v));
}

// Compile-time loop: the body sees its index as a constant from the front end on, so the
// register arrays below are split into scalars before any pass can turn a 16-bit array into
// packed pairs (packing would make every load wait for its neighbour inside the memory rounds).
template <int V> struct IntC { static constexpr int value = V; };
template <int B, int E, typename F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (B < E) { f(IntC<B>{}); static_for<B + 1, E>(f); }
}

// Requires (checked by the launcher): 64 rows of D elements span < 2^31 bytes, Tlen / 64 < 2^30.
// NW waves per workgroup: 8 for long sequences (the schedule above); 4 or 2 when the sequence has
// at most 4 or 2 chunks, where more waves would only idle through the barriers - the memory
// rounds then carry two or all four quarters each.
template <typename T, int NW>
__global__ __launch_bounds__(64 * NW) void hgrn_recurrent_pipelined_kernel(const T* __restrict__ x, const T* __restrict__ g,
                                                                       const float* __restrict__ h0, T* __restrict__ o,
                                                                       float* __restrict__ ht, int64_t Tlen, int64_t D) {
    using R = typename std::conditional<sizeof(T) == 4, float, uint16_t>::type;
    constexpr int MR = NW >= 8 ? 4 : NW / 2;                    // memory rounds per iteration
    constexpr int QPR = 4 / MR;                                 // quarters per memory round
    constexpr int kRsrcFlags = 0x00020000;                      // raw buffer, 32-bit data format, no swizzle
    constexpr int kAll = 0x7fffffff;
    __shared__ float baton[64];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int64_t bh = blockIdx.y;
    const uint32_t d = blockIdx.x * 64u + lane;
    const bool active = d < D;
    const uint32_t voff = active ? d * (uint32_t)sizeof(T) : 0x80000000u;   // lanes past D: always out of range
    const int NC = (int)((Tlen + kCH - 1) / kCH);
    const int iters = (NC + NW - 1) / NW;
    const uint32_t rowb = (uint32_t)D * (uint32_t)sizeof(T);
    const int64_t chunkb = (int64_t)kCH * rowb;
    const char* xb = reinterpret_cast<const char*>(x + bh * Tlen * D);
    const char* gb = reinterpret_cast<const char*>(g + bh * Tlen * D);
    char* ob = reinterpret_cast<char*>(o + bh * Tlen * D);

    R xr[kCH], gr[kCH];
    float hs[kCH];

    auto rem_of = [&](int c) {                                  // steps of chunk c inside the sequence, as a scalar int
        return __builtin_amdgcn_readfirstlane((int)max((int64_t)0, min((int64_t)kCH, Tlen - (int64_t)c * kCH)));
    };

#define MMF_LOAD_QUARTER(c_, q_)                                                                                       \
    {                                                                                                                  \
        const int cc = (c_);                                                                                           \
        const int rem = rem_of(cc);                                                                                    \
        const int recs = cc < NC ? kAll : 0;                                                                           \
        const __amdgpu_buffer_rsrc_t rx = __builtin_amdgcn_make_buffer_rsrc((void*)(xb + cc * chunkb), 0, recs, kRsrcFlags); \
        const __amdgpu_buffer_rsrc_t rg = __builtin_amdgcn_make_buffer_rsrc((void*)(gb + cc * chunkb), 0, recs, kRsrcFlags); \
        static_for<16 * (q_), 16 * (q_) + 16>([&](auto I) __attribute__((always_inline)) {                             \
            constexpr int t = decltype(I)::value;                                                                      \
            const uint32_t so = (uint32_t)max(0, min(t, rem - 1)) * rowb; /* rows past the end re-read the last one */ \
            xr[t] = buf_load<R>(rx, voff, so);                                                                         \
            gr[t] = buf_load<R>(rg, voff, so);                                                                         \
        });                                                                                                            \
    }
#define MMF_STORE_QUARTER(c_, q_)                                                                                      \
    {                                                                                                                  \
        const int cc = (c_);                                                                                           \
        const int rem = rem_of(cc);                                                                                    \
        const __amdgpu_buffer_rsrc_t ro = __builtin_amdgcn_make_buffer_rsrc((void*)(ob + cc * chunkb), 0, cc < NC ? kAll : 0, kRsrcFlags); \
        static_for<16 * (q_), 16 * (q_) + 16>([&](auto I) __attribute__((always_inline)) {                             \
            constexpr int t = decltype(I)::value;                                                                      \
            if (t < rem) buf_store<T>(hs[t], ro, voff, (uint32_t)t * rowb);                                            \
        });                                                                                                            \
    }

    if (wave == 0) baton[lane] = (h0 && active) ? h0[bh * D + d] : 0.0f;
    MMF_LOAD_QUARTER(wave, 0) MMF_LOAD_QUARTER(wave, 1) MMF_LOAD_QUARTER(wave, 2) MMF_LOAD_QUARTER(wave, 3)
    __syncthreads();
    for (int i = 0; i < wave; ++i) __syncthreads();              // wave w takes its first turn in round w

    for (int it = 0; it < iters; ++it) {
        const int c = it * NW + wave;
        {                                                        // my turn: chunk c, 64 dependent steps
            const int rem = rem_of(c);
            float h = baton[lane];
            if (rem == kCH) {                                    // full chunk: no selects on the serial chain's inputs
                static_for<0, kCH>([&](auto I) __attribute__((always_inline)) {
                    constexpr int t = decltype(I)::value;
                    const float gl = raw_get<T, R>(gr[t]);
                    h = __fadd_rn(__fmul_rn(gl, h), raw_get<T, R>(xr[t]));
                    hs[t] = h;
                });
            } else {
                static_for<0, kCH>([&](auto I) __attribute__((always_inline)) {
                    constexpr int t = decltype(I)::value;
                    const float gl = raw_get<T, R>(gr[t]);
                    const float gv = t < rem ? gl : 1.0f;
                    const float xv = t < rem ? raw_get<T, R>(xr[t]) : -0.0f;
                    h = __fadd_rn(__fmul_rn(gv, h), xv);
                    hs[t] = h;
                });
            }
            baton[lane] = h;
        }
        __syncthreads();
        static_for<0, MR>([&](auto RI) __attribute__((always_inline)) {
            static_for<0, QPR>([&](auto QI) __attribute__((always_inline)) {
                constexpr int q = decltype(RI)::value * QPR + decltype(QI)::value;
                MMF_STORE_QUARTER(c, q) MMF_LOAD_QUARTER(c + NW, q)
            });
            __syncthreads();
        });
#pragma unroll
        for (int i = 0; i < NW - 1 - MR; ++i) __syncthreads();   // idle rounds
    }
    for (int i = wave; i < NW - 1; ++i) __syncthreads();         // every wave passes the same number of barriers
    __syncthreads();
    if (ht && wave == 0 && active) ht[bh * D + d] = baton[lane];
#undef MMF_LOAD_QUARTER
#undef MMF_STORE_QUARTER
}

// -------------------------------------------------------------------------- chunked scan
// One workgroup = 64 channels (a lane owns one) x one segment [seg * seg_len, ...) of one (b, h).  The segment is cut
// into register blocks of CB steps (whole chunks of C steps, at most 8 of them and at most 64 steps).  Wave w takes
// blocks w, w + NW, ...:
//   1. loads the block's x and g (128 loads in flight per lane);
//   2. local pass, per chunk from zero (the first chunk of the sequence from h0), mmfreelm/ops/hgrn/chunk.py:69-85:
//        l_t = exp(g_t) * l_{t-1} + x_t,  gc_t = gc_{t-1} + g_t;  keeps l_t and E_t = exp(gc_t) in the registers that held
//        x_t and g_t.  The waves do this concurrently: nothing here depends on an earlier block;
//   3. its turn (blocks in order; the running state h sits in LDS): per chunk of the block ONE dependent step,
//        h = l_last + E_last * h  (chunk.py:108-114 applied to the chunk's last row) -- this is all that is serial
//        across chunks, so a turn is a handful of instructions, not 64 dependent steps;
//   4. after passing the turn on: o_t = l_t + E_t * (h before the chunk) for the whole block, stores.
//      (The first chunk of the sequence takes h = 0 here: the reference leaves it as the local pass made it.)
// Waves are not in lockstep (no barrier in the loop): a wave waiting for memory leaves the SIMDs to the others.
// CT > 0: the chunk length is the compile-time CT = CB = 64 and a full block runs straight-line code; CT = 0 (any
// chunk length) and tail blocks take the general path, whose chunk boundaries are bit masks tested per step.
// Segments: with NS > 1 a first launch (AGG) runs steps 1-3 only and leaves per segment the pair
// (A, b) = (product of the chunks' E_last, state at the segment's end when entered with zero) in `agg`; the second
// launch enters segment s with the fold h = A_j * h + b_j over the segments before it.  exp is the hardware one.
template <typename T, int NW, bool AGG, int CT>
__global__ __launch_bounds__(64 * NW) void hgrn_chunk_kernel(const T* __restrict__ x, const T* __restrict__ g,
                                                             const float* __restrict__ h0, T* __restrict__ o,
                                                             float* __restrict__ ht, float* __restrict__ agg, int64_t Tlen,
                                                             int64_t D, int CB, int64_t seg_len, int NS, uint64_t smask,
                                                             uint64_t emask) {
    constexpr int kRsrcFlags = 0x00020000;
    constexpr int kAll = 0x7fffffff;
    constexpr bool W16 = sizeof(T) == 2;
    __shared__ float baton_h[64], baton_a[64];
    __shared__ int turn;
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int64_t bh = blockIdx.y;
    const int seg = blockIdx.z;
    const uint32_t d = blockIdx.x * 64u + lane;
    const bool active = d < D;
    const uint32_t voff = active ? d * (uint32_t)sizeof(T) : 0x80000000u;
    const uint32_t rowb = (uint32_t)D * (uint32_t)sizeof(T);
    const int64_t t0 = (int64_t)seg * seg_len;
    const int64_t t1 = t0 + seg_len < Tlen ? t0 + seg_len : Tlen;
    const int nblk = (int)((t1 - t0 + CB - 1) / CB);
    const float h0v = (h0 && active && seg == 0) ? h0[bh * D + d] : 0.0f;   // enters through the first chunk's local pass

    if (wave == 0) {
        float hin = 0.0f;
        if (!AGG && seg > 0) {                                   // fold the segments before this one
            const float* ag = agg + bh * NS * 2 * D;
            hin = active ? ag[D + d] : 0.0f;                    // segment 0 carries h0: its b is its end state
            for (int j = 1; j < seg; ++j) {
                const float A = active ? ag[(int64_t)(2 * j) * D + d] : 0.0f;
                const float b = active ? ag[(int64_t)(2 * j + 1) * D + d] : 0.0f;
                hin = __fadd_rn(__fmul_rn(A, hin), b);
            }
        }
        baton_h[lane] = hin;
        baton_a[lane] = 1.0f;
        if (lane == 0) turn = 0;
    }
    __syncthreads();

    uint32_t a[kCH], q[kCH];                                     // x_t -> l_t and g_t -> E_t (raw bits, then float bits)
    auto val = [](uint32_t v) __attribute__((always_inline)) {
        if constexpr (W16) return mmf_to_float(mmf_from_bits16<T>((uint16_t)v));
        else return __uint_as_float(v);
    };
    auto wait_turn = [&](int b) __attribute__((always_inline)) {
        while (__hip_atomic_load(&turn, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_WORKGROUP) != b) __builtin_amdgcn_s_sleep(1);
    };

    for (int b = wave; b < nblk; b += NW) {
        const int64_t tb = t0 + (int64_t)b * CB;
        const int rem = __builtin_amdgcn_readfirstlane((int)((t1 - tb) < (int64_t)CB ? (t1 - tb) : (int64_t)CB));
        const float lin0 = (seg == 0 && b == 0) ? h0v : 0.0f;   // what the block's first chunk starts from
        const __amdgpu_buffer_rsrc_t rx = __builtin_amdgcn_make_buffer_rsrc((void*)(x + (bh * Tlen + tb) * D), 0, kAll, kRsrcFlags);
        const __amdgpu_buffer_rsrc_t rg = __builtin_amdgcn_make_buffer_rsrc((void*)(g + (bh * Tlen + tb) * D), 0, kAll, kRsrcFlags);
        const __amdgpu_buffer_rsrc_t ro = __builtin_amdgcn_make_buffer_rsrc((void*)(o + (bh * Tlen + tb) * D), 0, kAll, kRsrcFlags);
        if (CT > 0 && rem == kCH) {
            // ---- a full block that is one chunk: no boundary tests
            static_for<0, kCH>([&](auto I) __attribute__((always_inline)) {
                constexpr int t = decltype(I)::value;
                if constexpr (W16) {
                    a[t] = (uint32_t)(uint16_t)__builtin_amdgcn_raw_buffer_load_b16(rx, voff, (uint32_t)t * rowb, 0);
                    q[t] = (uint32_t)(uint16_t)__builtin_amdgcn_raw_buffer_load_b16(rg, voff, (uint32_t)t * rowb, 0);
                } else {
                    a[t] = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(rx, voff, (uint32_t)t * rowb, 0);
                    q[t] = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(rg, voff, (uint32_t)t * rowb, 0);
                }
            });
            float l = lin0, gc = 0.0f;
            static_for<0, kCH>([&](auto I) __attribute__((always_inline)) {
                constexpr int t = decltype(I)::value;
                const float gl = val(q[t]);
                l = __fadd_rn(__fmul_rn(__expf(gl), l), val(a[t]));
                gc = __fadd_rn(gc, gl);
                a[t] = __float_as_uint(l);
                if constexpr (!AGG || t == kCH - 1) q[t] = __float_as_uint(__expf(gc));   // AGG: only the chunk's last E is used
            });
            wait_turn(b);
            const float h_in = baton_h[lane];
            baton_h[lane] = __fadd_rn(__uint_as_float(a[kCH - 1]), __fmul_rn(__uint_as_float(q[kCH - 1]), h_in));
            if constexpr (AGG) baton_a[lane] = __fmul_rn(baton_a[lane], __uint_as_float(q[kCH - 1]));
            __hip_atomic_store(&turn, b + 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
            if constexpr (!AGG) {
                static_for<0, kCH>([&](auto I) __attribute__((always_inline)) {
                    constexpr int t = decltype(I)::value;
                    buf_store<T>(__fadd_rn(__uint_as_float(a[t]), __fmul_rn(__uint_as_float(q[t]), h_in)), ro, voff, (uint32_t)t * rowb);
                });
            }
            continue;
        }
        // ---- general path: chunk boundaries from the masks, tail blocks
        const uint64_t low = rem >= 64 ? ~0ull : ((1ull << rem) - 1ull);
        const uint64_t sm = smask & low, em = (emask | (1ull << (rem - 1))) & low;
        static_for<0, kCH>([&](auto I) __attribute__((always_inline)) {
            constexpr int t = decltype(I)::value;
            const uint32_t so = (uint32_t)(t < rem ? t : rem - 1) * rowb;     // rows past the end re-read the last one
            if constexpr (W16) {
                a[t] = (uint32_t)(uint16_t)__builtin_amdgcn_raw_buffer_load_b16(rx, voff, so, 0);
                q[t] = (uint32_t)(uint16_t)__builtin_amdgcn_raw_buffer_load_b16(rg, voff, so, 0);
            } else {
                a[t] = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(rx, voff, so, 0);
                q[t] = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(rg, voff, so, 0);
            }
        });
        {                                                        // local pass
            float l = 0.0f, gc = 0.0f;
            static_for<0, kCH>([&](auto I) __attribute__((always_inline)) {
                constexpr int t = decltype(I)::value;
                const bool st = (sm >> t) & 1ull;                // a chunk starts here (uniform)
                const bool live = t < rem;                       // steps past the end: (g, x) = (0, -0) change nothing
                const float gl = live ? val(q[t]) : 0.0f;
                const float xv = live ? val(a[t]) : -0.0f;
                const float lin = st ? (t == 0 ? lin0 : 0.0f) : l;
                const float gin = st ? 0.0f : gc;
                l = __fadd_rn(__fmul_rn(__expf(gl), lin), xv);
                gc = __fadd_rn(gin, gl);
                a[t] = __float_as_uint(l);
                q[t] = __float_as_uint(__expf(gc));
            });
        }
        wait_turn(b);
        float h = baton_h[lane];
        const float h_in = h;
        {
            float A = AGG ? baton_a[lane] : 1.0f;
            static_for<0, kCH>([&](auto I) __attribute__((always_inline)) {
                constexpr int t = decltype(I)::value;
                if ((em >> t) & 1ull) {                          // last step of a chunk (uniform)
                    const float Et = __uint_as_float(q[t]);
                    h = __fadd_rn(__uint_as_float(a[t]), __fmul_rn(Et, h));
                    if constexpr (AGG) A = __fmul_rn(A, Et);
                }
            });
            baton_h[lane] = h;
            if constexpr (AGG) baton_a[lane] = A;
        }
        __hip_atomic_store(&turn, b + 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
        if constexpr (!AGG) {                                    // the block's outputs
            float h2 = h_in;
            static_for<0, kCH>([&](auto I) __attribute__((always_inline)) {
                constexpr int t = decltype(I)::value;
                const float ot = __fadd_rn(__uint_as_float(a[t]), __fmul_rn(__uint_as_float(q[t]), h2));
                if ((em >> t) & 1ull) h2 = ot;
                if (t < rem) buf_store<T>(ot, ro, voff, (uint32_t)t * rowb);
            });
        }
    }
    if (wave == 0) {
        wait_turn(nblk);
        if constexpr (AGG) {
            if (active) {
                float* ag = agg + (bh * NS + seg) * 2 * D;
                ag[d] = baton_a[lane];
                ag[D + d] = baton_h[lane];
            }
        } else if (ht && seg == NS - 1 && active) {
            ht[bh * D + d] = baton_h[lane];
        }
    }
}

// -------------------------------------------------------------------------- gate math
// g_out = T( lb + (1 - lb) * sigmoid(f) )   (lb == null: T(sigmoid(f)))
// x_out = T( (i * (1 - g_out)) / (1 + exp(-i)) ), zeroed where mask == 0
// sf = sigmoid(f), taken by the caller for all its elements at once (mmf_sigmoid_n)
template <typename T>
__device__ __forceinline__ void gate_math(float iv, float sf, bool has_lb, float lb, float& xo, float& go) {
    float s = sf;
    if (has_lb) s = __fadd_rn(lb, __fmul_rn(__fsub_rn(1.0f, lb), s));
    go = mmf_round_to<T>(s);
    const float u = __fsub_rn(1.0f, go);
    xo = mmf_round_to<T>(__fdiv_rn(__fmul_rn(iv, u), __fadd_rn(1.0f, mmf_exp(-iv))));
}

// One kernel for both forms: STEP = false writes (x, g); STEP = true runs one recurrence step on the
// fp32 state in place and writes o.  grid = (ceil(D / 1024), rows): a thread owns 4 consecutive
// channels of one row, so there is no index division and the loads are 8- / 16-byte vectors
// (VEC: D, the row strides and every pointer allow that; otherwise element accesses).
template <typename T, bool STEP, bool VEC>
__global__ __launch_bounds__(256) void hgrn_gate_kernel(const T* __restrict__ i_in, int64_t ldi, const T* __restrict__ f_in,
                                                        int64_t ldf, const float* __restrict__ lb,
                                                        const uint8_t* __restrict__ mask, float* __restrict__ state,
                                                        T* __restrict__ x_out, T* __restrict__ g_out, int D) {
    const int64_t r = blockIdx.y;
    const int d0 = ((int)blockIdx.x * 256 + (int)threadIdx.x) * 4;
    if (d0 >= D) return;
    const Raw4<T> iraw = raw4_load<T, VEC>(i_in + r * ldi, d0, D);
    const Raw4<T> fraw = raw4_load<T, VEC>(f_in + r * ldf, d0, D);
    Raw4<float> lbraw, straw;
    if (lb) lbraw = raw4_load<float, VEC>(lb, d0, D);
    if constexpr (STEP) straw = raw4_load<float, VEC>(state + r * D, d0, D);
    const bool keep = !(mask && mask[r] == 0);
    float iv[4], fv[4], lbv[4] = {0.0f, 0.0f, 0.0f, 0.0f}, stv[4], xo[4], go[4];
    raw4_unpack<T>(iraw, iv);
    raw4_unpack<T>(fraw, fv);
    if (lb) raw4_unpack<float>(lbraw, lbv);
    if constexpr (STEP) raw4_unpack<float>(straw, stv);
    float sf[4];
    mmf_sigmoid_n<4>(fv, sf);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        gate_math<T>(iv[e], sf[e], lb != nullptr, lbv[e], xo[e], go[e]);
        if (!keep) xo[e] = 0.0f;
        if constexpr (STEP) {
            stv[e] = __fadd_rn(__fmul_rn(go[e], stv[e]), xo[e]);
            xo[e] = stv[e];                                     // o = T(h)
        }
    }
    if constexpr (STEP) raw4_store<float, VEC>(state + r * D, d0, D, stv);
    raw4_store<T, VEC>(x_out + r * D, d0, D, xo);
    if constexpr (!STEP) raw4_store<T, VEC>(g_out + r * D, d0, D, go);
}

// ht = h0 (or zeros) for an empty sequence; a kernel, not a memset, so it can be graph captured.
__global__ __launch_bounds__(256) void state_init_kernel(const float* __restrict__ h0, float* __restrict__ ht, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) ht[i] = h0 ? h0[i] : 0.0f;
}

// The kernel addresses a 64-step chunk with 32-bit offsets and counts chunks in an int.
template <typename T>
bool scan_fits(int64_t Tlen, int64_t D) {
    return mmf_ceil_div(Tlen, (int64_t)kCH) < (1 << 30) && (int64_t)kCH * D * (int64_t)sizeof(T) < (1ll << 31);
}

template <typename T>
int launch_scan(const void* x, const void* g, const float* h0, void* o, float* ht, int64_t BH, int64_t Tlen, int64_t D,
                hipStream_t s) {
    if (!scan_fits<T>(Tlen, D)) return MMF_ERR_WIDE;
    dim3 grid((unsigned)mmf_ceil_div(D, 64), (unsigned)BH);
    const int64_t NC = mmf_ceil_div(Tlen, (int64_t)kCH);
    const T* xp = static_cast<const T*>(x);
    const T* gp = static_cast<const T*>(g);
    T* op = static_cast<T*>(o);
    if (NC <= 2) hgrn_recurrent_pipelined_kernel<T, 2><<<grid, 128, 0, s>>>(xp, gp, h0, op, ht, Tlen, D);
    else if (NC <= 4) hgrn_recurrent_pipelined_kernel<T, 4><<<grid, 256, 0, s>>>(xp, gp, h0, op, ht, Tlen, D);
    else hgrn_recurrent_pipelined_kernel<T, 8><<<grid, 512, 0, s>>>(xp, gp, h0, op, ht, Tlen, D);
    MMF_CHECK_LAUNCH();
    return 0;
}

// How mmf_hgrn_chunk cuts the time axis: register blocks of CB steps (whole chunks), NS segments of seg_len steps.
// One segment when batch * channels already give every CU a workgroup; otherwise enough segments for about two
// workgroups per CU, each at least four blocks long.
struct ChunkPlan {
    int CB, NS;
    int64_t seg_len;
    uint64_t smask, emask;
};
ChunkPlan chunk_plan(int64_t BH, int64_t Tlen, int64_t D, int chunk) {
    ChunkPlan p{};
    p.CB = (kCH / chunk > 8 ? 8 : kCH / chunk) * chunk;        // whole chunks, at most 8 and at most 64 steps
    const int64_t wgs = BH * mmf_ceil_div(D, 64);
    int64_t ns = 1;
    if (wgs < 256 && Tlen > 0) {
        const int64_t want = mmf_ceil_div(512, wgs), most = Tlen / (4 * p.CB);
        ns = want < most ? want : most;
        ns = ns < 1 ? 1 : ns > 64 ? 64 : ns;
    }
    p.seg_len = mmf_round_up(mmf_ceil_div(Tlen > 0 ? Tlen : 1, ns), p.CB);
    p.NS = (int)mmf_ceil_div(Tlen > 0 ? Tlen : 1, p.seg_len);
    for (int t = 0; t < p.CB; ++t) {
        if (t % chunk == 0) p.smask |= 1ull << t;
        if (t % chunk == chunk - 1) p.emask |= 1ull << t;
    }
    return p;
}

template <typename T>
int launch_chunk(const void* x, const void* g, const float* h0, void* o, float* ht, float* agg, int64_t BH, int64_t Tlen,
                 int64_t D, int chunk, hipStream_t s) {
    if (!scan_fits<T>(Tlen, D)) return MMF_ERR_WIDE;
    const ChunkPlan p = chunk_plan(BH, Tlen, D, chunk);
    if (p.NS > 1 && !agg) return MMF_ERR_ARG;
    const T* xp = static_cast<const T*>(x);
    const T* gp = static_cast<const T*>(g);
    T* op = static_cast<T*>(o);
    const unsigned gx = (unsigned)mmf_ceil_div(D, 64);
    const dim3 grid_agg(gx, (unsigned)BH, (unsigned)(p.NS > 1 ? p.NS - 1 : 1)), grid(gx, (unsigned)BH, (unsigned)p.NS);
    if (chunk == kCH) {
        if (p.NS > 1) {
            hgrn_chunk_kernel<T, 8, true, kCH><<<grid_agg, 512, 0, s>>>(xp, gp, h0, op, ht, agg, Tlen, D, p.CB, p.seg_len, p.NS,
                                                                        p.smask, p.emask);
            MMF_CHECK_LAUNCH();
        }
        hgrn_chunk_kernel<T, 8, false, kCH><<<grid, 512, 0, s>>>(xp, gp, h0, op, ht, agg, Tlen, D, p.CB, p.seg_len, p.NS, p.smask,
                                                                 p.emask);
    } else {
        if (p.NS > 1) {
            hgrn_chunk_kernel<T, 8, true, 0><<<grid_agg, 512, 0, s>>>(xp, gp, h0, op, ht, agg, Tlen, D, p.CB, p.seg_len, p.NS,
                                                                      p.smask, p.emask);
            MMF_CHECK_LAUNCH();
        }
        hgrn_chunk_kernel<T, 8, false, 0><<<grid, 512, 0, s>>>(xp, gp, h0, op, ht, agg, Tlen, D, p.CB, p.seg_len, p.NS, p.smask,
                                                               p.emask);
    }
    MMF_CHECK_LAUNCH();
    return 0;
}

template <typename T>
int launch_gate(const void* i_in, int64_t ldi, const void* f_in, int64_t ldf, const float* lb, const uint8_t* mask,
                void* x_out, void* g_out, float* state, int64_t rows, int64_t D, bool step, hipStream_t s) {
    if (rows * D == 0) return 0;
    if (rows > 65535 * (int64_t)32768 || D > INT32_MAX - 4) return MMF_ERR_WIDE;
    auto al = [](const void* p, uintptr_t n) { return (reinterpret_cast<uintptr_t>(p) % n) == 0; };
    const uintptr_t ea = 4 * sizeof(T);
    const bool vec = D % 4 == 0 && ldi % 4 == 0 && ldf % 4 == 0 && al(i_in, ea) && al(f_in, ea) && al(x_out, ea) &&
                     al(g_out, ea) && al(lb, 16) && al(state, 16);
    const T* ip = static_cast<const T*>(i_in);
    const T* fp = static_cast<const T*>(f_in);
    T* xp = static_cast<T*>(x_out);
    T* gp = static_cast<T*>(g_out);
    const unsigned gx = (unsigned)mmf_ceil_div(D, (int64_t)1024);
    // rows go on grid.y (<= 65535 per launch)
    for (int64_t r0 = 0; r0 < rows; r0 += 65535) {
        const int64_t nr = rows - r0 < 65535 ? rows - r0 : 65535;
        dim3 grid(gx, (unsigned)nr);
        const T* ipr = ip + r0 * ldi;
        const T* fpr = fp + r0 * ldf;
        const uint8_t* mk = mask ? mask + r0 : nullptr;
        float* st = state ? state + r0 * D : nullptr;
        T* xpr = xp + r0 * D;
        T* gpr = gp ? gp + r0 * D : nullptr;
        if (step) {
            if (vec) hgrn_gate_kernel<T, true, true><<<grid, 256, 0, s>>>(ipr, ldi, fpr, ldf, lb, mk, st, xpr, gpr, (int)D);
            else hgrn_gate_kernel<T, true, false><<<grid, 256, 0, s>>>(ipr, ldi, fpr, ldf, lb, mk, st, xpr, gpr, (int)D);
        } else {
            if (vec) hgrn_gate_kernel<T, false, true><<<grid, 256, 0, s>>>(ipr, ldi, fpr, ldf, lb, mk, st, xpr, gpr, (int)D);
            else hgrn_gate_kernel<T, false, false><<<grid, 256, 0, s>>>(ipr, ldi, fpr, ldf, lb, mk, st, xpr, gpr, (int)D);
        }
        MMF_CHECK_LAUNCH();
    }
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
        case MMF_F32: return launch_scan<float>(x, g, h0, o, ht, BH, T, D, stream);
        case MMF_BF16: return launch_scan<bf16_t>(x, g, h0, o, ht, BH, T, D, stream);
        case MMF_F16: return launch_scan<f16_t>(x, g, h0, o, ht, BH, T, D, stream);
    }
    return MMF_ERR_ARG;
}

int64_t mmf_hgrn_chunk_workspace_bytes(int64_t BH, int64_t T, int64_t D, int chunk) {
    if (BH <= 0 || T <= 0 || D <= 0 || chunk < 1 || chunk > kCH) return 0;
    const ChunkPlan p = chunk_plan(BH, T, D, chunk);
    return p.NS > 1 ? BH * p.NS * 2 * D * (int64_t)sizeof(float) : 0;
}

int mmf_hgrn_chunk(const void* x, const void* g, const float* h0, void* o, float* ht, int64_t BH, int64_t T, int64_t D,
                   int chunk, int dtype, void* workspace, void* stream_) {
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
    float* agg = static_cast<float*>(workspace);
    switch (dtype) {
        case MMF_F32: return launch_chunk<float>(x, g, h0, o, ht, agg, BH, T, D, chunk, stream);
        case MMF_BF16: return launch_chunk<bf16_t>(x, g, h0, o, ht, agg, BH, T, D, chunk, stream);
        case MMF_F16: return launch_chunk<f16_t>(x, g, h0, o, ht, agg, BH, T, D, chunk, stream);
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
