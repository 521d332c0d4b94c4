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
};

template <typename T, int WGM, int WGN, int WM, int WN>
__global__ __launch_bounds__(64 * WGM * WGN) void bitlinear_mfma_kernel(MfmaArgs p) {
    constexpr int NT = 64 * WGM * WGN;
    constexpr int BMB = WGM * WM;                 // m-blocks (of 32 rows) per workgroup tile
    constexpr int BNB = WGN * WN;                 // n-blocks per workgroup tile
    constexpr int PIECES = BMB * 256;             // 16-byte pieces of one A slab (BMB x 4 KiB)
    constexpr int NPA = (PIECES + NT - 1) / NT;   // pieces per thread
    extern __shared__ __align__(16) unsigned char smem[];   // 2 x BMB x 4096 bytes

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
    uint4 breg[WN], bnext[WN];

    auto load_a = [&](int64_t kb) {
#pragma unroll
        for (int i = 0; i < NPA; ++i) {
            const int pc = threadIdx.x + i * NT;
            const int chunk = pc >> 8, within = pc & 255;
            areg[i] = make_uint4(0, 0, 0, 0);
            if (pc < PIECES && mb0 + chunk < MB)
                areg[i] = *reinterpret_cast<const uint4*>(p.a + ((mb0 + chunk) * KG + kb * 8) * 512 + within * 16);
        }
    };
    auto store_a = [&](int buf) {
#pragma unroll
        for (int i = 0; i < NPA; ++i) {
            const int pc = threadIdx.x + i * NT;
            if (pc < PIECES) *reinterpret_cast<uint4*>(smem + buf * (BMB * 4096) + pc * 16) = areg[i];
        }
    };
    auto load_b = [&](int64_t kb, uint4 (&dst)[WN]) {
#pragma unroll
        for (int j = 0; j < WN; ++j) {
            dst[j] = make_uint4(0x55555555u, 0x55555555u, 0x55555555u, 0x55555555u);   // all codes 1 = ternary 0
            if (nb0 + j < NB) dst[j] = p.b[((nb0 + j) * KB + kb) * 64 + lane];
        }
    };

    load_a(0);
    load_b(0, breg);
    store_a(0);
    __syncthreads();

    for (int64_t kb = 0; kb < KB; ++kb) {
        const int buf = (int)(kb & 1);
        const bool more = kb + 1 < KB;
        if (more) {
            load_a(kb + 1);
            load_b(kb + 1, bnext);
        }
        const unsigned char* abase = smem + buf * (BMB * 4096) + (wm * WM) * 4096 + lane * 16;
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            v4i af[WM], bf[WN];
#pragma unroll
            for (int i = 0; i < WM; ++i) af[i] = *reinterpret_cast<const v4i*>(abase + i * 4096 + ks * 1024);
#pragma unroll
            for (int j = 0; j < WN; ++j) {
                const uint32_t w = ks == 0 ? breg[j].x : ks == 1 ? breg[j].y : ks == 2 ? breg[j].z : breg[j].w;
                bf[j][0] = (int)(w & 0x03030303u);
                bf[j][1] = (int)((w >> 2) & 0x03030303u);
                bf[j][2] = (int)((w >> 4) & 0x03030303u);
                bf[j][3] = (int)((w >> 6) & 0x03030303u);
            }
#pragma unroll
            for (int i = 0; i < WM; ++i)
#pragma unroll
                for (int j = 0; j < WN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[i], bf[j], acc[i][j], 0, 0, 0);
        }
        if (more) {
            store_a(buf ^ 1);
#pragma unroll
            for (int j = 0; j < WN; ++j) breg[j] = bnext[j];
        }
        __syncthreads();
    }

    // ---- epilogue.  Accumulator register r of lane l is row 8*(r/4) + 4*(l/32) + r%4,
    // column l%32 of the 32x32 block.
    const T* bias = static_cast<const T*>(p.bias);
    const T* addend = static_cast<const T*>(p.addend);
    T* out = static_cast<T*>(p.out);
#pragma unroll
    for (int i = 0; i < WM; ++i) {
        const int64_t mb = mb0 + wm * WM + i;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int64_t m = mb * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
            if (m >= p.M) continue;
            const float dq = p.deq[m];
            const int qs = p.qsum[m];
#pragma unroll
            for (int j = 0; j < WN; ++j) {
                const int64_t n = (nb0 + j) * 32 + (lane & 31);
                if (n >= p.N) continue;
                float o = __fmul_rn(__fmul_rn((float)(acc[i][j][r] - qs), dq), p.wdeq[n / p.seg_rows]);
                if (bias) o = __fadd_rn(o, mmf_to_float(bias[n]));
                if (addend) o = __fadd_rn(mmf_round_to<T>(o), mmf_to_float(addend[m * p.ldo + n]));
                out[m * p.ldo + n] = mmf_from_float<T>(o);
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
            float o = __fmul_rn(__fmul_rn((float)(tot - p.qsum[m]), p.deq[m]), p.wdeq[n / p.seg_rows]);
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

template <typename T, int WGM, int WGN, int WM, int WN>
int launch_mfma(MfmaArgs a, hipStream_t s) {
    constexpr int BM = WGM * WM * 32, BN = WGN * WN * 32;
    a.tiles_m = (int)mmf_ceil_div(a.M, BM);
    a.tiles_n = (int)mmf_ceil_div(a.N, BN);
    const size_t lds = 2u * (WGM * WM) * 4096u;
    auto kern = bitlinear_mfma_kernel<T, WGM, WGN, WM, WN>;
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
    if (M < 0 || K <= 0 || N <= 0 || seg_rows <= 0 || ldo < N) return MMF_ERR_ARG;
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
