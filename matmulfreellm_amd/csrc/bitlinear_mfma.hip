// Ternary-weight contraction on the int8 matrix cores (v_mfma_i32_32x32x32_i8, gfx950).
//
//   out[m, n] = T( fp32( sum_k q[m,k] * t[n,k] ) * deq[m] * wdeq[seg(n)] (+ bias[n]) )
//
// Replaces the dense F.linear on de-quantised weights at mmfreelm/ops/fusedbitnet.py:458
// (and the weight_quant at :456, done once at pack time instead).
//
// Operands
//   A  int8 activation codes in the fragment-tiled layout the quantiser writes:
//      [ceil32(M)/32][Kp/16][32 rows][16 bytes]; the 1 KiB at (mb, 2*ks .. 2*ks+1) is one
//      32x32 A fragment in lane order (lane l: row l%32, k = 16*(l/32) .. +15).
//   B  2-bit packed ternary codes (t+1), block layout [Np/32][Kp/128][64 lanes][4 dwords];
//      dword ks of lane l expands with 3 shifts + 4 masks into the 16 bytes lane l feeds
//      the MFMA for k-step ks.  B never touches LDS: every wave streams its own n-blocks
//      straight from global memory (they are 16x smaller than the int8 tile they become).
//   The stored code is t+1 in {0,1,2}; the epilogue subtracts sum_k q[m,k] (qsum).
//
// Tiling: a workgroup of WGM x WGN waves computes a (WGM*WM*32) x (WGN*WN*32) tile; each
// wave owns WM x WN accumulators of 32x32 (16 VGPRs each).  A is staged through LDS in
// K-slabs of 128, double buffered, one barrier per slab; global loads for slab kb+1 are in
// flight while slab kb is multiplied.
#include "mmf_common.h"
#include "../../include/mmf.h"

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

struct MfmaArgs {
    const int8_t* a;      // tiled codes
    const uint4* b;       // packed weights
    const float* deq;     // [M]
    const int* qsum;      // [M]
    const float* wdeq;    // per segment
    const void* bias;     // [N] or null
    const void* addend;   // [M, N] (leading dimension ldo) or null: out = T(T(o) + addend)
    void* out;            // [M, N]
    int64_t M, N, Kp, seg_rows, ldo;
    int tiles_m, tiles_n;
    int vec_store;        // outputs can be written as aligned 16-byte vectors
};

template <typename T, int WGM, int WGN, int WM, int WN, int KSL>
__global__ __launch_bounds__(64 * WGM * WGN) void bitlinear_mfma_kernel(MfmaArgs p) {
    constexpr int NT = 64 * WGM * WGN;
    constexpr int BMB = WGM * WM;                 // m-blocks (of 32 rows) per workgroup tile
    constexpr int BNB = WGN * WN;                 // n-blocks per workgroup tile
    constexpr int CH = KSL * 4096;                // bytes of one m-block's slab (KSL k-blocks of 128)
    constexpr int PIECES = BMB * (CH / 16);       // 16-byte pieces of one A slab
    constexpr int NPA = (PIECES + NT - 1) / NT;   // pieces per thread
    extern __shared__ __align__(16) unsigned char smem[];   // 2 x BMB x CH bytes

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int wm = wave / WGN, wn = wave % WGN;

    // XCD-aware tile order: hardware deals consecutive workgroup ids round-robin to the 8
    // XCDs; remap so each XCD walks a contiguous run of tiles (shared A panel stays in its L2).
    int64_t wg = blockIdx.x;
    const int64_t total = (int64_t)p.tiles_m * p.tiles_n;
    if (total % 8 == 0) wg = (wg % 8) * (total / 8) + wg / 8;
    const int64_t tile_m = wg / p.tiles_n, tile_n = wg % p.tiles_n;

    const int64_t MB = (p.M + 31) >> 5, NB = (p.N + 31) >> 5;
    const int64_t KB = p.Kp >> 7, KG = p.Kp >> 4;
    const int64_t mb0 = tile_m * BMB, nb0 = tile_n * BNB + wn * WN;

    v16i acc[WM][WN];
#pragma unroll
    for (int i = 0; i < WM; ++i)
#pragma unroll
        for (int j = 0; j < WN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;

    uint4 areg[NPA];
    uint4 breg[KSL][WN], bnext[KSL][WN];

    auto load_a = [&](int64_t kb) {
#pragma unroll
        for (int i = 0; i < NPA; ++i) {
            const int pc = threadIdx.x + i * NT;
            const int chunk = pc / (CH / 16), within = pc % (CH / 16);
            areg[i] = make_uint4(0, 0, 0, 0);
            if (pc < PIECES && mb0 + chunk < MB && kb * 8 + (within >> 5) < KG)
                areg[i] = *reinterpret_cast<const uint4*>(p.a + ((mb0 + chunk) * KG + kb * 8) * 512 + within * 16);
        }
    };
    auto store_a = [&](int buf) {
#pragma unroll
        for (int i = 0; i < NPA; ++i) {
            const int pc = threadIdx.x + i * NT;
            if (pc < PIECES) *reinterpret_cast<uint4*>(smem + buf * (BMB * CH) + pc * 16) = areg[i];
        }
    };
    auto load_b = [&](int64_t kb, uint4 (&dst)[KSL][WN]) {
#pragma unroll
        for (int q = 0; q < KSL; ++q)
#pragma unroll
            for (int j = 0; j < WN; ++j) {
                dst[q][j] = make_uint4(0x55555555u, 0x55555555u, 0x55555555u, 0x55555555u);   // all codes 1 = ternary 0
                if (nb0 + j < NB && kb + q < KB) dst[q][j] = p.b[((nb0 + j) * KB + kb + q) * 64 + lane];
            }
    };

    load_a(0);
    load_b(0, breg);
    store_a(0);
    __syncthreads();

    for (int64_t kb = 0; kb < KB; kb += KSL) {
        const int buf = (int)((kb / KSL) & 1);
        const bool more = kb + KSL < KB;
        if (more) {
            load_a(kb + KSL);
            load_b(kb + KSL, bnext);
        }
        const unsigned char* abase = smem + buf * (BMB * CH) + (wm * WM) * CH + lane * 16;
        // Software pipeline over the 32-wide k-steps of the slab: the LDS reads of step ks+1
        // are issued before the MFMAs of step ks.
        v4i af[2][WM];
#pragma unroll
        for (int i = 0; i < WM; ++i) af[0][i] = *reinterpret_cast<const v4i*>(abase + i * CH);
#pragma unroll
        for (int ks = 0; ks < 4 * KSL; ++ks) {
            if (ks + 1 < 4 * KSL) {
#pragma unroll
                for (int i = 0; i < WM; ++i)
                    af[(ks + 1) & 1][i] = *reinterpret_cast<const v4i*>(abase + i * CH + (ks + 1) * 1024);
            }
            v4i bf[WN];
#pragma unroll
            for (int j = 0; j < WN; ++j) {
                const uint4 bq = breg[ks >> 2][j];
                const uint32_t w = (ks & 3) == 0 ? bq.x : (ks & 3) == 1 ? bq.y : (ks & 3) == 2 ? bq.z : bq.w;
                bf[j][0] = (int)(w & 0x03030303u);
                bf[j][1] = (int)((w >> 2) & 0x03030303u);
                bf[j][2] = (int)((w >> 4) & 0x03030303u);
                bf[j][3] = (int)((w >> 6) & 0x03030303u);
            }
#pragma unroll
            for (int i = 0; i < WM; ++i)
#pragma unroll
                for (int j = 0; j < WN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[ks & 1][i], bf[j], acc[i][j], 0, 0, 0);
        }
        if (more) {
            store_a(buf ^ 1);
#pragma unroll
            for (int q = 0; q < KSL; ++q)
#pragma unroll
                for (int j = 0; j < WN; ++j) breg[q][j] = bnext[q][j];
        }
        __syncthreads();
    }

    // ---- epilogue.  Accumulator register r of lane l is row 8*(r/4) + 4*(l/32) + r%4,
    // column l%32 of the 32x32 block.  Everything that depends only on the column (weight
    // scale, bias, bounds) or only on the row (deq, qsum) is fetched once, not per element.
    const T* bias = static_cast<const T*>(p.bias);
    const T* addend = static_cast<const T*>(p.addend);
    T* out = static_cast<T*>(p.out);
    float wdq[WN], bs[WN];
    int64_t ncol[WN];
#pragma unroll
    for (int j = 0; j < WN; ++j) {
        ncol[j] = (nb0 + j) * 32 + (lane & 31);
        const bool ok = ncol[j] < p.N;
        wdq[j] = ok ? p.wdeq[(uint32_t)ncol[j] / (uint32_t)p.seg_rows] : 0.0f;
        bs[j] = (ok && bias) ? mmf_to_float(bias[ncol[j]]) : 0.0f;
        if (!ok) ncol[j] = -1;
    }
    constexpr int E = sizeof(T);
    constexpr int RS = WN * 32 * E + 16;          // LDS row stride of a wave's 32 x (WN*32) staging tile
    constexpr int CPR = WN * 32 * E / 16;         // 16-byte chunks per row
    unsigned char* stage = smem + wave * (32 * RS);
#pragma unroll
    for (int i = 0; i < WM; ++i) {
        const int64_t mblk = (mb0 + wm * WM + i) * 32;
        const int64_t mrow0 = mblk + 4 * (lane >> 5);
        float dqv[16];
        int qsv[16];
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int64_t m = mrow0 + 8 * (r >> 2) + (r & 3);
            dqv[r] = m < p.M ? p.deq[m] : 0.0f;
            qsv[r] = m < p.M ? p.qsum[m] : 0;
        }
        if (p.vec_store) {
            // Stage the wave's 32 x (WN*32) outputs through LDS so every lane stores 16 bytes and a
            // store instruction covers whole 128-byte row segments (2-byte scattered stores cost
            // more than the whole K loop).  The region is private to the wave: no block barrier.
#pragma unroll
            for (int j = 0; j < WN; ++j)
#pragma unroll
                for (int r = 0; r < 16; r += 2) {
                    float o0 = __fmul_rn(__fmul_rn((float)(acc[i][j][r] - qsv[r]), dqv[r]), wdq[j]);
                    float o1 = __fmul_rn(__fmul_rn((float)(acc[i][j][r + 1] - qsv[r + 1]), dqv[r + 1]), wdq[j]);
                    if (bias) { o0 = __fadd_rn(o0, bs[j]); o1 = __fadd_rn(o1, bs[j]); }
                    const int row0 = 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                    if constexpr (E == 2) {
                        // lanes 2k / 2k+1 trade one value so each holds two adjacent columns of one row
                        const T t0 = mmf_from_float<T>(o0), t1 = mmf_from_float<T>(o1);
                        const uint32_t b0 = *reinterpret_cast<const uint16_t*>(&t0), b1 = *reinterpret_cast<const uint16_t*>(&t1);
                        const uint32_t recv = __shfl_xor((lane & 1) ? b0 : b1, 1, 64);
                        const uint32_t word = (lane & 1) ? (recv | (b1 << 16)) : (b0 | (recv << 16));
                        const int row = row0 + (lane & 1);
                        *reinterpret_cast<uint32_t*>(stage + row * RS + (j * 32 + (lane & 30)) * 2) = word;
                    } else {
                        *reinterpret_cast<float*>(stage + row0 * RS + (j * 32 + (lane & 31)) * 4) = o0;
                        *reinterpret_cast<float*>(stage + (row0 + 1) * RS + (j * 32 + (lane & 31)) * 4) = o1;
                    }
                }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
            for (int c0 = 0; c0 < 32 * CPR; c0 += 64) {
                const int c = c0 + lane;
                const int row = c / CPR, cc = c % CPR;
                const int64_t m = mblk + row, n = nb0 * 32 + cc * (16 / E);
                if (m < p.M && n < p.N) {
                    uint4 v = *reinterpret_cast<const uint4*>(stage + row * RS + cc * 16);
                    if (addend) {
                        const uint4 av = *reinterpret_cast<const uint4*>(addend + m * p.ldo + n);
                        const T* pe = reinterpret_cast<const T*>(&v);
                        const T* ae = reinterpret_cast<const T*>(&av);
                        uint4 ov;
                        T* oe = reinterpret_cast<T*>(&ov);
#pragma unroll
                        for (int e = 0; e < 16 / E; ++e) oe[e] = mmf_from_float<T>(__fadd_rn(mmf_to_float(pe[e]), mmf_to_float(ae[e])));
                        v = ov;
                    }
                    *reinterpret_cast<uint4*>(out + m * p.ldo + n) = v;
                }
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        } else {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int64_t m = mrow0 + 8 * (r >> 2) + (r & 3);
                if (m >= p.M) continue;
                T* orow = out + m * p.ldo;
#pragma unroll
                for (int j = 0; j < WN; ++j) {
                    if (ncol[j] < 0) continue;
                    float o = __fmul_rn(__fmul_rn((float)(acc[i][j][r] - qsv[r]), dqv[r]), wdq[j]);
                    if (bias) o = __fadd_rn(o, bs[j]);
                    if (addend) o = __fadd_rn(mmf_round_to<T>(o), mmf_to_float(addend[m * p.ldo + ncol[j]]));
                    orow[ncol[j]] = mmf_from_float<T>(o);
                }
            }
        }
    }
}

// ------------------------------------------------------------------------------------------
// Decode-sized M (<= 64): the contraction is a weight stream, not a GEMM, and the enemy is
// latency, so nothing is staged and nothing waits on a barrier until the very end.
// One workgroup of 8 waves owns one 32-row n-block; wave w takes the k-blocks w, w+8, ...
// A fragments (1 KiB each, L2 resident: the whole A is M x K bytes) and the packed B block
// are loaded straight into registers, three k-blocks in flight per wave; the 8 partial
// accumulators meet in LDS and all 512 threads run the epilogue.
template <typename T, int MB>
__global__ __launch_bounds__(512) void bitlinear_mfma_skinny_kernel(MfmaArgs p) {
    constexpr int NWV = 8, PF = 3, MAXK = 8;            // Kp <= 8 * 8 * 128
    __shared__ int red[NWV][MB][16][64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t nb = blockIdx.x;
    const int64_t KB = p.Kp >> 7, KG = p.Kp >> 4;
    const int64_t MBtot = (p.M + 31) >> 5;

    v16i acc[MB];
#pragma unroll
    for (int i = 0; i < MB; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][r] = 0;

    uint4 breg[PF];
    v4i areg[PF][MB][4];
    auto load_stage = [&](int st, int64_t kb) {
        if (kb < KB) {
            breg[st] = p.b[(nb * KB + kb) * 64 + lane];
#pragma unroll
            for (int i = 0; i < MB; ++i)
#pragma unroll
                for (int ks = 0; ks < 4; ++ks) {
                    areg[st][i][ks] = (v4i){0, 0, 0, 0};
                    if (i < MBtot)
                        areg[st][i][ks] = *reinterpret_cast<const v4i*>(p.a + ((int64_t)i * KG + kb * 8 + ks * 2) * 512 + lane * 16);
                }
        }
    };
#pragma unroll
    for (int st = 0; st < PF; ++st) load_stage(st, wave + (int64_t)st * NWV);
#pragma unroll
    for (int it = 0; it < MAXK; ++it) {
        const int st = it % PF;
        const int64_t kb = wave + (int64_t)it * NWV;
        if (kb < KB) {
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) {
                const uint32_t w = ks == 0 ? breg[st].x : ks == 1 ? breg[st].y : ks == 2 ? breg[st].z : breg[st].w;
                v4i bf;
                bf[0] = (int)(w & 0x03030303u);
                bf[1] = (int)((w >> 2) & 0x03030303u);
                bf[2] = (int)((w >> 4) & 0x03030303u);
                bf[3] = (int)((w >> 6) & 0x03030303u);
#pragma unroll
                for (int i = 0; i < MB; ++i)
                    acc[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(areg[st][i][ks], bf, acc[i], 0, 0, 0);
            }
        }
        if (it + PF < MAXK) load_stage(st, wave + (int64_t)(it + PF) * NWV);
    }
#pragma unroll
    for (int i = 0; i < MB; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) red[wave][i][r][lane] = acc[i][r];
    __syncthreads();

    const T* bias = static_cast<const T*>(p.bias);
    const T* addend = static_cast<const T*>(p.addend);
    T* out = static_cast<T*>(p.out);
#pragma unroll
    for (int j = 0; j < MB * 2; ++j) {
        const int e = threadIdx.x + j * 512;             // (mb, r, lane) flattened
        const int l = e & 63, r = (e >> 6) & 15, mb = e >> 10;
        int tot = 0;
#pragma unroll
        for (int w = 0; w < NWV; ++w) tot += red[w][mb][r][l];
        const int64_t m = (int64_t)mb * 32 + 8 * (r >> 2) + 4 * (l >> 5) + (r & 3);
        const int64_t n = nb * 32 + (l & 31);
        if (m < p.M && n < p.N) {
            float o = __fmul_rn(__fmul_rn((float)(tot - p.qsum[m]), p.deq[m]), p.wdeq[(uint32_t)n / (uint32_t)p.seg_rows]);
            if (bias) o = __fadd_rn(o, mmf_to_float(bias[n]));
            if (addend) o = __fadd_rn(mmf_round_to<T>(o), mmf_to_float(addend[m * p.ldo + n]));
            out[m * p.ldo + n] = mmf_from_float<T>(o);
        }
    }
}

template <typename T, int MB>
int launch_skinny(const MfmaArgs& a, hipStream_t s) {
    bitlinear_mfma_skinny_kernel<T, MB><<<dim3((unsigned)mmf_ceil_div(a.N, 32)), dim3(512), 0, s>>>(a);
    MMF_CHECK_LAUNCH();
    return 0;
}

template <typename T, int WGM, int WGN, int WM, int WN, int KSL = 1>
int launch_mfma(MfmaArgs a, hipStream_t s) {
    constexpr int BM = WGM * WM * 32, BN = WGN * WN * 32;
    a.tiles_m = (int)mmf_ceil_div(a.M, BM);
    a.tiles_n = (int)mmf_ceil_div(a.N, BN);
    size_t lds = 2u * (WGM * WM) * 4096u * KSL;
    const size_t lds_epi = (size_t)(WGM * WGN) * 32u * (WN * 32u * sizeof(T) + 16u);   // per-wave output staging
    if (lds_epi > lds) lds = lds_epi;
    const int per_vec = 16 / (int)sizeof(T);
    a.vec_store = (a.N % per_vec == 0) && (a.ldo % per_vec == 0) && ((reinterpret_cast<uintptr_t>(a.out) & 15u) == 0) &&
                  ((reinterpret_cast<uintptr_t>(a.addend) & 15u) == 0);
    auto kern = bitlinear_mfma_kernel<T, WGM, WGN, WM, WN, KSL>;
    if (lds > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                           (int)lds);
        if (e != hipSuccess) return (int)e;
    }
    kern<<<dim3((unsigned)((int64_t)a.tiles_m * a.tiles_n)), dim3(64 * WGM * WGN), lds, s>>>(a);
    MMF_CHECK_LAUNCH();
    return 0;
}

template <typename T>
int dispatch_mfma(const MfmaArgs& a, int config, hipStream_t s) {
    // config < 0: pick by M.  Tiled kernels (BM x BN): 0: 32x256, 1: 64x256, 2: 128x256, 3: 256x256,
    // 4: 256x256 with 2x4 accumulators per wave.  5 / 6: the decode-sized weight-stream kernel
    // for M <= 32 / M <= 64 (needs Kp <= 8192).
    if (config < 0) {
        if (a.M <= 64 && a.Kp <= 8192) config = a.M <= 32 ? 5 : 6;
        else config = a.M <= 32 ? 0 : a.M <= 64 ? 1 : a.M <= 128 ? 2 : 3;
    }
    if ((config == 5 && a.M > 32) || (config == 6 && a.M > 64) || ((config == 5 || config == 6) && a.Kp > 8192))
        return MMF_ERR_ARG;
    switch (config) {
        case 5: return launch_skinny<T, 1>(a, s);
        case 6: return launch_skinny<T, 2>(a, s);
        case 0: return launch_mfma<T, 1, 8, 1, 1>(a, s);
        case 1: return launch_mfma<T, 1, 8, 2, 1>(a, s);
        case 2: return launch_mfma<T, 2, 4, 2, 2>(a, s);
        case 3: return launch_mfma<T, 2, 4, 4, 2>(a, s);
        case 4: return launch_mfma<T, 4, 2, 2, 4>(a, s);
        case 7: return launch_mfma<T, 2, 4, 4, 2, 2>(a, s);
        case 8: return launch_mfma<T, 2, 4, 2, 2, 2>(a, s);
        case 9: return launch_mfma<T, 1, 8, 4, 2, 2>(a, s);
    }
    return MMF_ERR_ARG;
}

}  // namespace

extern "C" {

int mmf_bitlinear_mfma(const int8_t* codes_tiled, const float* deq, const int* qsum, const void* packed,
                       const float* wdeq, int64_t seg_rows, const void* bias, const void* addend, void* out, int64_t ldo,
                       int64_t M,
                       int64_t K, int64_t N, int out_dtype, int config, void* stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (M < 0 || K <= 0 || N <= 0 || seg_rows <= 0 || ldo < N || N > 0x7fffffff) return MMF_ERR_ARG;
    if (M == 0) return 0;
    if (!codes_tiled || !deq || !qsum || !packed || !wdeq || !out) return MMF_ERR_ARG;
    if ((reinterpret_cast<uintptr_t>(codes_tiled) & 15u) || (reinterpret_cast<uintptr_t>(packed) & 15u)) return MMF_ERR_ALIGN;
    MfmaArgs a{};
    a.a = codes_tiled; a.b = static_cast<const uint4*>(packed); a.deq = deq; a.qsum = qsum; a.wdeq = wdeq; a.bias = bias; a.addend = addend;
    a.out = out; a.M = M; a.N = N; a.Kp = mmf_round_up(K, 128); a.seg_rows = seg_rows; a.ldo = ldo;
    switch (out_dtype) {
        case MMF_F32: return dispatch_mfma<float>(a, config, stream);
        case MMF_BF16: return dispatch_mfma<bf16_t>(a, config, stream);
        case MMF_F16: return dispatch_mfma<f16_t>(a, config, stream);
    }
    return MMF_ERR_ARG;
}

}  // extern "C"
