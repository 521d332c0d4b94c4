// Shared device helpers for the MatMul-free LM hot-path kernels (gfx950, wave64).
//
// Arithmetic contract used by every kernel in this directory:
//  * all floating-point math is fp32 (fp64 only for sums of squares / |w|), one
//    IEEE-rounded operation at a time: the files are compiled with
//    -ffp-contract=off and the helpers below use the __f*_rn intrinsics, so no
//    multiply-add is ever fused;
//  * division and sqrt are the correctly rounded ones;
//  * rounding to integer codes is round-half-to-even (rintf);
//  * exp is mmf_exp() below, built from add/mul only, so a CPU restatement can
//    reproduce every result bit for bit.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

// Keep every multiply and add separately rounded in all code that includes this header,
// whatever -ffp-contract the translation unit is built with.
#pragma clang fp contract(off)

#include "../../include/mmf.h"        // dtype ids, error codes, entry-point declarations
#include "../../include/mmf_diag.h"   // measuring aids

#define MMF_CHECK_LAUNCH()                          \
    do {                                            \
        hipError_t e__ = hipGetLastError();         \
        if (e__ != hipSuccess) return (int)e__;     \
    } while (0)

struct bf16_t { uint16_t v; };
struct f16_t { _Float16 v; };

// ---------------------------------------------------------------- scalar conversions
__device__ __forceinline__ float mmf_to_float(float x) { return x; }
__device__ __forceinline__ float mmf_to_float(bf16_t x) { return __uint_as_float(((uint32_t)x.v) << 16); }
__device__ __forceinline__ float mmf_to_float(f16_t x) { return (float)x.v; }

__device__ __forceinline__ uint16_t mmf_f32_to_bf16_bits(float f) {
    // round to nearest even; gfx950 has a hardware convert (v_cvt_pk_bf16_f32) the compiler selects
    const __bf16 b = (__bf16)f;
    return __builtin_bit_cast(uint16_t, b);
}

// The 16 bits of a bf16_t / f16_t value and back (no pointer punning: _Float16 and uint16_t do not alias).
template <typename T> __device__ __forceinline__ uint16_t mmf_bits16(T t) {
    static_assert(sizeof(T) == 2, "16-bit types only");
    return __builtin_bit_cast(uint16_t, t);
}
template <typename T> __device__ __forceinline__ T mmf_from_bits16(uint16_t b) {
    static_assert(sizeof(T) == 2, "16-bit types only");
    return __builtin_bit_cast(T, b);
}

template <typename T> __device__ __forceinline__ T mmf_from_float(float f);
template <> __device__ __forceinline__ float mmf_from_float<float>(float f) { return f; }
template <> __device__ __forceinline__ bf16_t mmf_from_float<bf16_t>(float f) { bf16_t r; r.v = mmf_f32_to_bf16_bits(f); return r; }
template <> __device__ __forceinline__ f16_t mmf_from_float<f16_t>(float f) { f16_t r; r.v = (_Float16)f; return r; }

// Round an fp32 value to T and bring it back (what a materialised tensor would hold).
template <typename T> __device__ __forceinline__ float mmf_round_to(float f) { return mmf_to_float(mmf_from_float<T>(f)); }

// ---------------------------------------------------------------- 8-element vectors
// Rows are processed 8 elements at a time: one 16-byte load for bf16/f16, two for fp32.
template <typename T> struct Vec8;
template <> struct Vec8<float> { float4 a, b; };
template <> struct Vec8<bf16_t> { uint4 a; };
template <> struct Vec8<f16_t> { uint4 a; };

template <typename T>
__device__ __forceinline__ void mmf_load8(const T* __restrict__ p, int64_t k0, int64_t K, bool vec_ok, float (&out)[8]) {
    if (vec_ok) {
        if constexpr (sizeof(T) == 4) {
            const float4* q = reinterpret_cast<const float4*>(p + k0);
            float4 a = q[0], b = q[1];
            out[0] = a.x; out[1] = a.y; out[2] = a.z; out[3] = a.w;
            out[4] = b.x; out[5] = b.y; out[6] = b.z; out[7] = b.w;
        } else {
            const uint4 a = *reinterpret_cast<const uint4*>(p + k0);
            T e[8];
            __builtin_memcpy(e, &a, 16);
#pragma unroll
            for (int i = 0; i < 8; ++i) out[i] = mmf_to_float(e[i]);
        }
    } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) out[i] = (k0 + i < K) ? mmf_to_float(p[k0 + i]) : 0.0f;
    }
}

// The same eight elements as they sit in memory.  Kernels whose cost is latency issue all of
// their loads as raw vectors first and unpack them where they are used, so that no conversion
// waits for one load before the next is issued.  Lanes with k0 >= K read the row start (vector
// path) or zeros (element path); the caller discards them.
template <typename T> struct Raw8 { uint4 a; };
template <> struct Raw8<float> { float4 a, b; };

template <typename T>
__device__ __forceinline__ Raw8<T> mmf_load8_raw(const T* __restrict__ p, int64_t k0, int64_t K, bool vec_ok) {
    Raw8<T> r;
    if (vec_ok) {
        const T* q = p + (k0 < K ? k0 : 0);
        if constexpr (sizeof(T) == 4) {
            r.a = reinterpret_cast<const float4*>(q)[0];
            r.b = reinterpret_cast<const float4*>(q)[1];
        } else {
            r.a = *reinterpret_cast<const uint4*>(q);
        }
    } else {
        T e[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) e[i] = p[k0 + i < K ? k0 + i : 0];
        __builtin_memcpy(&r, e, sizeof(r));
    }
    return r;
}
template <typename T>
__device__ __forceinline__ void mmf_unpack8(const Raw8<T>& r, float (&out)[8]) {
    T e[8];
    __builtin_memcpy(e, &r, sizeof(r));
#pragma unroll
    for (int i = 0; i < 8; ++i) out[i] = mmf_to_float(e[i]);
}

// Four consecutive elements as they sit in memory; unpacked to fp32 only where they are used, so
// that all of a thread's loads are in flight before the first conversion waits for one.
template <typename T> struct Raw4 { uint2 v; };
template <> struct Raw4<float> { float4 v; };

template <typename T, bool VEC>
__device__ __forceinline__ Raw4<T> raw4_load(const T* p, int k0, int K) {
    Raw4<T> r;
    if constexpr (VEC) {
        const int kk = k0 < K ? k0 : 0;                         // lanes past K re-read the row start; zeroed on unpack
        r.v = *reinterpret_cast<const decltype(r.v)*>(p + kk);
    } else {
        T e[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) e[i] = p[k0 + i < K ? k0 + i : 0];
        __builtin_memcpy(&r.v, e, sizeof(r.v));
    }
    return r;
}
template <typename T>
__device__ __forceinline__ void raw4_unpack(const Raw4<T>& r, float (&f)[4]) {
    if constexpr (sizeof(T) == 4) {
        f[0] = r.v.x; f[1] = r.v.y; f[2] = r.v.z; f[3] = r.v.w;
    } else {
        T e[4];
        __builtin_memcpy(e, &r.v, sizeof(r.v));
#pragma unroll
        for (int i = 0; i < 4; ++i) f[i] = mmf_to_float(e[i]);
    }
}
template <typename T, bool VEC>
__device__ __forceinline__ void raw4_store(T* p, int k0, int K, const float (&f)[4]) {
    T e[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) e[i] = mmf_from_float<T>(f[i]);
    if constexpr (VEC) {
        if (k0 < K) __builtin_memcpy(p + k0, e, sizeof(e));
    } else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
            if (k0 + i < K) p[k0 + i] = e[i];
    }
}

template <typename T>
__device__ __forceinline__ void mmf_store8(T* __restrict__ p, int64_t k0, int64_t K, bool vec_ok, const float (&in)[8]) {
    if (vec_ok) {
        if constexpr (sizeof(T) == 4) {
            float4* q = reinterpret_cast<float4*>(p + k0);
            q[0] = make_float4(in[0], in[1], in[2], in[3]);
            q[1] = make_float4(in[4], in[5], in[6], in[7]);
        } else {
            uint4 a;
            T e[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) e[i] = mmf_from_float<T>(in[i]);
            __builtin_memcpy(&a, e, 16);
            *reinterpret_cast<uint4*>(p + k0) = a;
        }
    } else {
#pragma unroll
        for (int i = 0; i < 8; ++i)
            if (k0 + i < K) p[k0 + i] = mmf_from_float<T>(in[i]);
    }
}

// ---------------------------------------------------------------- deterministic exp
// Cody-Waite reduction by ln2, degree-5 Horner polynomial, two-step 2^n scaling.
// Every operation is a separately rounded fp32 add or multiply.  This is the DEFINITION of the function (the CPU
// restatement follows it operation by operation); the kernels call mmf_exp() below, which returns the same bits.
__device__ __forceinline__ float mmf_exp_definition(float x) {
    float xc = fminf(fmaxf(x, -104.0f), 89.0f);                 // a NaN argument is clamped like any other and put back at the end
    float n = rintf(__fmul_rn(xc, 1.44269504088896341f));
    float r = __fsub_rn(xc, __fmul_rn(n, 0.693359375f));
    r = __fsub_rn(r, __fmul_rn(n, -2.12194440e-4f));
    float z = __fmul_rn(r, r);
    float p = 1.9875691500e-4f;
    p = __fadd_rn(__fmul_rn(p, r), 1.3981999507e-3f);
    p = __fadd_rn(__fmul_rn(p, r), 8.3334519073e-3f);
    p = __fadd_rn(__fmul_rn(p, r), 4.1665795894e-2f);
    p = __fadd_rn(__fmul_rn(p, r), 1.6666665459e-1f);
    p = __fadd_rn(__fmul_rn(p, r), 5.0000001201e-1f);
    float y = __fmul_rn(p, z);
    y = __fadd_rn(y, r);
    y = __fadd_rn(y, 1.0f);
    int ni = (int)n;
    int n1 = ni >> 1;
    int n2 = ni - n1;
    y = __fmul_rn(y, __int_as_float((n1 + 127) << 23));
    y = __fmul_rn(y, __int_as_float((n2 + 127) << 23));
    return x != x ? x : y;                                       // a select, not a branch
}

// The same function with the two-step scaling as ONE ldexp: the first of the two multiplications by a power of two is
// exact (y is in [0.7, 1.5] and 2^n1 keeps it normal), so only the second rounds -- once, like ldexp(y, n).  Equal to the
// definition for every one of the 2^32 arguments (mmf_diag_check_exact_forms runs them all on the device).
__device__ __forceinline__ float mmf_exp(float x) {
    float xc = fminf(fmaxf(x, -104.0f), 89.0f);
    float n = rintf(__fmul_rn(xc, 1.44269504088896341f));
    float r = __fsub_rn(xc, __fmul_rn(n, 0.693359375f));
    r = __fsub_rn(r, __fmul_rn(n, -2.12194440e-4f));
    float z = __fmul_rn(r, r);
    float p = 1.9875691500e-4f;
    p = __fadd_rn(__fmul_rn(p, r), 1.3981999507e-3f);
    p = __fadd_rn(__fmul_rn(p, r), 8.3334519073e-3f);
    p = __fadd_rn(__fmul_rn(p, r), 4.1665795894e-2f);
    p = __fadd_rn(__fmul_rn(p, r), 1.6666665459e-1f);
    p = __fadd_rn(__fmul_rn(p, r), 5.0000001201e-1f);
    float y = __fmul_rn(p, z);
    y = __fadd_rn(y, r);
    y = __fadd_rn(y, 1.0f);
    y = __builtin_ldexpf(y, (int)n);
    return x != x ? x : y;
}

// Short forms of the correctly rounded reciprocal, square root and quotient 127 / a: the hardware's approximation and
// one (two) Newton steps with fused multiply-adds, three to seven dependent instructions where the general correctly
// rounded sequences take eleven to fifteen.  Outside the range where that is exact (results or intermediates near the
// subnormals or overflow, zero, infinities, NaN) they branch to the general sequence -- no wave of a real activation
// does.  Each is equal to the general sequence for EVERY float argument: mmf_diag_check_exact_forms runs all 2^32
// through both on the device (a GPU test asserts zero differences).
__device__ __forceinline__ bool mmf_mid_range(float d) {         // 2^-100 <= d < 2^100 (false for NaN)
    return d >= 0x1p-100f && d < 0x1p100f;
}
__device__ __forceinline__ float mmf_rcp_pos(float d) {          // == __fdiv_rn(1.0f, d)
    if (__builtin_expect(!mmf_mid_range(d), 0)) return __fdiv_rn(1.0f, d);
    const float r0 = __builtin_amdgcn_rcpf(d);
    const float e = __builtin_fmaf(-d, r0, 1.0f);
    return __builtin_fmaf(e, r0, r0);
}
__device__ __forceinline__ float mmf_rcp_ge1(float d) { return mmf_rcp_pos(d); }
__device__ __forceinline__ float mmf_sqrt_pos(float v) {         // == sqrtf(v), the correctly rounded one
    if (__builtin_expect(!mmf_mid_range(v), 0)) return sqrtf(v);
    const float rs = __builtin_amdgcn_rsqf(v);
    const float s0 = __fmul_rn(v, rs), h = __fmul_rn(0.5f, rs);
    const float s1 = __builtin_fmaf(__builtin_fmaf(-s0, s0, v), h, s0);
    return __builtin_fmaf(__builtin_fmaf(-s1, s1, v), h, s1);
}
__device__ __forceinline__ float mmf_127_over(float a) {         // == __fdiv_rn(127.0f, a)
    if (__builtin_expect(!mmf_mid_range(a), 0)) return __fdiv_rn(127.0f, a);
    const float r0 = __builtin_amdgcn_rcpf(a);
    const float y = __builtin_fmaf(__builtin_fmaf(-a, r0, 1.0f), r0, r0);
    const float q0 = __fmul_rn(127.0f, y);
    return __builtin_fmaf(__builtin_fmaf(-a, q0, 127.0f), y, q0);
}

// 1 / (1 + exp(-x))
__device__ __forceinline__ float mmf_sigmoid_definition(float x) {
    return __fdiv_rn(1.0f, __fadd_rn(1.0f, mmf_exp_definition(-x)));
}
__device__ __forceinline__ float mmf_sigmoid(float x) {
    return mmf_rcp_ge1(__fadd_rn(1.0f, mmf_exp(-x)));
}
// The same without a branch and without the NaN test, for x >= -69 (then 1 + exp(-x) stays below 2^100, where the short
// reciprocal is exact; NaN fails the test).  A kernel that takes many sigmoids in a row tests its arguments once
// (mmf_sigmoid_n) and runs straight-line code, whose independent chains the compiler can interleave; with a test per
// element every sigmoid is a basic block of its own.  Equal to the definition for every float that passes the test
// (mmf_diag_check_exact_forms).
__device__ __forceinline__ bool mmf_sigmoid_mid_ok(float x) { return x >= -69.0f; }
__device__ __forceinline__ float mmf_sigmoid_mid(float x) {
    const float xn = -x;
    float xc = fminf(fmaxf(xn, -104.0f), 89.0f);
    float n = rintf(__fmul_rn(xc, 1.44269504088896341f));
    float r = __fsub_rn(xc, __fmul_rn(n, 0.693359375f));
    r = __fsub_rn(r, __fmul_rn(n, -2.12194440e-4f));
    float z = __fmul_rn(r, r);
    float p = 1.9875691500e-4f;
    p = __fadd_rn(__fmul_rn(p, r), 1.3981999507e-3f);
    p = __fadd_rn(__fmul_rn(p, r), 8.3334519073e-3f);
    p = __fadd_rn(__fmul_rn(p, r), 4.1665795894e-2f);
    p = __fadd_rn(__fmul_rn(p, r), 1.6666665459e-1f);
    p = __fadd_rn(__fmul_rn(p, r), 5.0000001201e-1f);
    float y = __fmul_rn(p, z);
    y = __fadd_rn(y, r);
    y = __fadd_rn(y, 1.0f);
    y = __builtin_ldexpf(y, (int)n);
    const float d = __fadd_rn(1.0f, y);
    const float r0 = __builtin_amdgcn_rcpf(d);
    return __builtin_fmaf(__builtin_fmaf(-d, r0, 1.0f), r0, r0);
}
// N sigmoids: one range test for all of them, then straight-line code (or, for an argument below -69 or a NaN among
// them, the general form for all).
template <int N>
__device__ __forceinline__ void mmf_sigmoid_n(const float (&x)[N], float (&s)[N]) {
    bool ok = true;
#pragma unroll
    for (int i = 0; i < N; ++i) ok = ok & mmf_sigmoid_mid_ok(x[i]);
    if (__builtin_expect(ok, 1)) {
#pragma unroll
        for (int i = 0; i < N; ++i) s[i] = mmf_sigmoid_mid(x[i]);
    } else {
#pragma unroll
        for (int i = 0; i < N; ++i) s[i] = mmf_sigmoid(x[i]);
    }
}

// ---------------------------------------------------------------- reductions (wave64)
// Rows of 16 lanes are folded with four DPP moves (quad swaps, half-row mirror, row mirror: a few
// cycles each, where a generic cross-lane shuffle goes through the LDS crossbar); the four row
// results are then read as scalars and combined in row order.  Every lane ends with the same bits.
template <int CTRL>
__device__ __forceinline__ int mmf_dpp(int v) { return __builtin_amdgcn_mov_dpp(v, CTRL, 0xf, 0xf, true); }
template <int CTRL>
__device__ __forceinline__ float mmf_dpp(float v) { return __int_as_float(mmf_dpp<CTRL>(__float_as_int(v))); }
template <int CTRL>
__device__ __forceinline__ double mmf_dpp(double v) {
    return __hiloint2double(mmf_dpp<CTRL>(__double2hiint(v)), mmf_dpp<CTRL>(__double2loint(v)));
}
__device__ __forceinline__ int mmf_readlane(int v, int l) { return __builtin_amdgcn_readlane(v, l); }
__device__ __forceinline__ float mmf_readlane(float v, int l) { return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), l)); }
__device__ __forceinline__ double mmf_readlane(double v, int l) {
    return __hiloint2double(__builtin_amdgcn_readlane(__double2hiint(v), l), __builtin_amdgcn_readlane(__double2loint(v), l));
}
constexpr int kDppXor1 = 0xB1, kDppXor2 = 0x4E, kDppHalfMirror = 0x141, kDppMirror = 0x140;

__device__ __forceinline__ double mmf_wave_sum(double v) {
    v += mmf_dpp<kDppXor1>(v);
    v += mmf_dpp<kDppXor2>(v);
    v += mmf_dpp<kDppHalfMirror>(v);
    v += mmf_dpp<kDppMirror>(v);
    return (mmf_readlane(v, 0) + mmf_readlane(v, 16)) + (mmf_readlane(v, 32) + mmf_readlane(v, 48));
}
__device__ __forceinline__ float mmf_wave_max(float v) {
    v = fmaxf(v, mmf_dpp<kDppXor1>(v));
    v = fmaxf(v, mmf_dpp<kDppXor2>(v));
    v = fmaxf(v, mmf_dpp<kDppHalfMirror>(v));
    v = fmaxf(v, mmf_dpp<kDppMirror>(v));
    return fmaxf(fmaxf(mmf_readlane(v, 0), mmf_readlane(v, 16)), fmaxf(mmf_readlane(v, 32), mmf_readlane(v, 48)));
}
__device__ __forceinline__ int mmf_wave_sum(int v) {
    v += mmf_dpp<kDppXor1>(v);
    v += mmf_dpp<kDppXor2>(v);
    v += mmf_dpp<kDppHalfMirror>(v);
    v += mmf_dpp<kDppMirror>(v);
    return mmf_readlane(v, 0) + mmf_readlane(v, 16) + mmf_readlane(v, 32) + mmf_readlane(v, 48);
}

// Block-wide reductions for blocks of NW waves; `red` is LDS scratch of >= NW entries
// that the caller does not otherwise touch between the two barriers.  The per-wave
// partials are combined in index order by every thread, so all threads (and all
// blocks reducing the same data) see the same bits.
template <int NW>
__device__ __forceinline__ double mmf_block_sum(double v, double* red) {
    v = mmf_wave_sum(v);
    if constexpr (NW == 1) return v;
    const int w = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) red[w] = v;
    __syncthreads();
    double s = red[0];
#pragma unroll
    for (int i = 1; i < NW; ++i) s += red[i];
    __syncthreads();
    return s;
}
template <int NW>
__device__ __forceinline__ float mmf_block_max(float v, float* red) {
    v = mmf_wave_max(v);
    if constexpr (NW == 1) return v;
    const int w = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) red[w] = v;
    __syncthreads();
    float s = red[0];
#pragma unroll
    for (int i = 1; i < NW; ++i) s = fmaxf(s, red[i]);
    __syncthreads();
    return s;
}
template <int NW>
__device__ __forceinline__ int mmf_block_sum(int v, int* red) {
    v = mmf_wave_sum(v);
    if constexpr (NW == 1) return v;
    const int w = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) red[w] = v;
    __syncthreads();
    int s = red[0];
#pragma unroll
    for (int i = 1; i < NW; ++i) s += red[i];
    __syncthreads();
    return s;
}

// One 1 KiB packed weight block (a lane holds 64 weights of one output row: 4 dwords = 4 k-steps of 16) against the
// int8 codes of k-block kb in LDS: each dword expands to four byte-wide code dwords (shift + mask), v_dot4_i32_i8
// accumulates.  `half` selects the lane's 16 of each k-step's 32 inputs.
__device__ __forceinline__ int mmf_dot_block(const int8_t* q_lds, const uint4& wq, int kb, int half, int acc) {
#pragma unroll
    for (int s4 = 0; s4 < 4; ++s4) {
        const int4 qv = *reinterpret_cast<const int4*>(q_lds + kb * 128 + s4 * 32 + half * 16);
        const uint32_t w = s4 == 0 ? wq.x : s4 == 1 ? wq.y : s4 == 2 ? wq.z : wq.w;
        acc = __builtin_amdgcn_sdot4((int)(w & 0x03030303u), qv.x, acc, false);
        acc = __builtin_amdgcn_sdot4((int)((w >> 2) & 0x03030303u), qv.y, acc, false);
        acc = __builtin_amdgcn_sdot4((int)((w >> 4) & 0x03030303u), qv.z, acc, false);
        acc = __builtin_amdgcn_sdot4((int)((w >> 6) & 0x03030303u), qv.w, acc, false);
    }
    return acc;
}

// The same with the 128 codes of the k-block already in registers (qv[s] = the lane's 16 codes of k-step s).
__device__ __forceinline__ int mmf_dot_block_regs(const int4 (&qv)[4], const uint4& wq, int acc) {
#pragma unroll
    for (int s4 = 0; s4 < 4; ++s4) {
        const uint32_t w = s4 == 0 ? wq.x : s4 == 1 ? wq.y : s4 == 2 ? wq.z : wq.w;
        acc = __builtin_amdgcn_sdot4((int)(w & 0x03030303u), qv[s4].x, acc, false);
        acc = __builtin_amdgcn_sdot4((int)((w >> 2) & 0x03030303u), qv[s4].y, acc, false);
        acc = __builtin_amdgcn_sdot4((int)((w >> 4) & 0x03030303u), qv[s4].z, acc, false);
        acc = __builtin_amdgcn_sdot4((int)((w >> 6) & 0x03030303u), qv[s4].w, acc, false);
    }
    return acc;
}

// One-barrier block reductions of the decode kernels: the NW per-wave results meet in `slot` (LDS, NW entries,
// one array per reduction so that no second barrier is needed before its reuse) and every thread combines them
// pairwise in the same order: log2(NW) dependent additions instead of NW - 1.
template <int N>
__device__ __forceinline__ double mmf_tree_sum(const double* v) {
    if constexpr (N == 1) return v[0];
    else return mmf_tree_sum<N / 2>(v) + mmf_tree_sum<N - N / 2>(v + N / 2);
}
template <int NW>
__device__ __forceinline__ double mmf_block_sum_once(double v, double* slot) {
    v = mmf_wave_sum(v);
    if ((threadIdx.x & 63) == 0) slot[threadIdx.x >> 6] = v;
    __syncthreads();
    double t[NW];
#pragma unroll
    for (int i = 0; i < NW; ++i) t[i] = slot[i];
    return mmf_tree_sum<NW>(t);
}
template <int NW>
__device__ __forceinline__ float mmf_block_max_once(float v, float* slot) {
    v = mmf_wave_max(v);
    if ((threadIdx.x & 63) == 0) slot[threadIdx.x >> 6] = v;
    __syncthreads();
    float s = slot[0];
#pragma unroll
    for (int i = 1; i < NW; ++i) s = fmaxf(s, slot[i]);
    return s;
}

// rstd = 1 / sqrt( fp32(sumsq / K) + eps ).
// sumsq / K is the correctly rounded fp64 quotient without the division sequence: with
// inv_K = RN(1 / K) from the host, q0 = sumsq * inv_K is within two ulps, one residual step
// makes it faithful, and a second one (r exact through the fused multiply-add) lands on the
// correctly rounded quotient (Markstein's theorem; K is a small integer, 0 <= sumsq < 2^200).
// s + v * v in fp64.  The square of an fp32 value is exact in fp64 (48 significant bits), so the fused multiply-add rounds
// exactly what the separate multiply and add would: same result, one fp64 operation instead of two.
__device__ __forceinline__ double mmf_add_square(double s, float v) {
    const double d = (double)v;
    return __builtin_fma(d, d, s);
}
__device__ __forceinline__ double mmf_quotient_by_count(double sum, int64_t K, double inv_K) {
    const double Kd = (double)K;
    double q = sum * inv_K;
    q = fma(fma(-q, Kd, sum), inv_K, q);
    q = fma(fma(-q, Kd, sum), inv_K, q);
    return q;
}
__device__ __forceinline__ float mmf_rstd(double sumsq, int64_t K, double inv_K, float eps) {
    const float var = (float)mmf_quotient_by_count(sumsq, K, inv_K);
    return mmf_rcp_pos(mmf_sqrt_pos(__fadd_rn(var, eps)));   // == 1 / sqrtf(var + eps), both correctly rounded
}

// int8 code of one normalised value:  clamp(rint(y * scale), -128, 127)
__device__ __forceinline__ int mmf_code(float y, float scale) {
    float r = rintf(__fmul_rn(y, scale));
    r = fminf(fmaxf(r, -128.0f), 127.0f);
    return (int)r;
}

__host__ __device__ static inline int64_t mmf_ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }
__host__ __device__ static inline int64_t mmf_round_up(int64_t a, int64_t b) { return mmf_ceil_div(a, b) * b; }
