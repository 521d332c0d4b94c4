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
// Three kernels, chosen by a measured cost model (dispatch_mfma):
//   large problems : a workgroup of WGM x WGN waves computes a (WGM*WM*32) x (WGN*WN*32) tile; each
//                    wave owns WM x WN accumulators of 32x32 (16 VGPRs each); A is staged through
//                    LDS by DMA in k-blocks of 128, three buffers, one barrier per k-block
//                    (bitlinear_mfma_dma3_kernel);
//   small problems : one 32x32 output block per workgroup, 8 waves split K, operands straight
//                    into registers (bitlinear_mfma_skinny_kernel);
//   small M with K > 8192 : A staged through registers, double buffered (bitlinear_mfma_kernel).
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
    int rows_per_xcd;     // tile rows an XCD keeps in its L2 while it walks the columns (0: row-major tile order)
    int vec_store;        // outputs can be written as aligned 16-byte vectors
    long long* clocks;    // null, or [clock_cap][2]: shader-clock and 100 MHz ticks a workgroup spent in the kernel
    int64_t clock_cap;
};

// Where the tiled kernel notes its clocks (mmf_bitlinear_mfma_clock_sink); null: nothing is noted.
long long* g_clock_sink = nullptr;
int64_t g_clock_cap = 0;

// Pack rounded outputs: two floats -> one dword of bf16/f16 (round to nearest even).
template <typename T>
__device__ __forceinline__ uint32_t pack2(float a, float b) {
    const T ta = mmf_from_float<T>(a), tb = mmf_from_float<T>(b);
    return (uint32_t)mmf_bits16(ta) | ((uint32_t)mmf_bits16(tb) << 16);
}

// Epilogue of the tiled kernels.  The MFMAs are issued with the weights as the first operand,
// so an accumulator holds the TRANSPOSED 32x32 block: register r of lane l is output column
// n = 8*(r/4) + 4*(l/32) + r%4 and output row m = l%32.  A lane therefore needs one (deq, qsum)
// pair per block and holds four consecutive columns in registers 4g..4g+3, which pack into one
// 8-byte piece with no cross-lane traffic.  The wave stages its 32 x (WN*32) outputs in a
// private LDS region and writes them out as aligned 16-byte vectors (128-byte row segments).
// Per-lane row scales and per-block weight scales of the epilogue, fetched at kernel start so
// their latency hides behind the whole K loop.
template <int WM, int WN>
struct EpiScales { float dq[WM]; int qs[WM]; float wdq[WN]; };

template <int WM, int WN>
__device__ __forceinline__ void mfma_prefetch_scales(const MfmaArgs& p, EpiScales<WM, WN>& sc, int lane, int wm,
                                                     int64_t mb0, int64_t nb0) {
    const int64_t NB = (p.N + 31) >> 5;
#pragma unroll
    for (int i = 0; i < WM; ++i) {
        const int64_t m = (mb0 + wm * WM + i) * 32 + (lane & 31);
        sc.dq[i] = m < p.M ? p.deq[m] : 0.0f;
        sc.qs[i] = m < p.M ? p.qsum[m] : 0;
    }
#pragma unroll
    for (int j = 0; j < WN; ++j)   // seg_rows is a multiple of 32: one weight scale per n-block
        sc.wdq[j] = (nb0 + j < NB) ? p.wdeq[(uint32_t)((nb0 + j) * 32) / (uint32_t)p.seg_rows] : 0.0f;
}

template <typename T, int WM, int WN>
__device__ __forceinline__ void mfma_epilogue(const MfmaArgs& p, v16i (&acc)[WM][WN], const EpiScales<WM, WN>& sc,
                                              unsigned char* smem, int lane, int wave, int wm, int64_t mb0, int64_t nb0) {
    const T* bias = static_cast<const T*>(p.bias);
    const T* addend = static_cast<const T*>(p.addend);
    T* out = static_cast<T*>(p.out);
    const float (&wdq)[WN] = sc.wdq;
    constexpr int E = sizeof(T);
    constexpr int RS = WN * 32 * E + 16;          // LDS row stride of a wave's 32 x (WN*32) staging tile
    constexpr int CPR = WN * 32 * E / 16;         // 16-byte chunks per row
    unsigned char* stage = smem + wave * (32 * RS);
    const int half = lane >> 5, mloc = lane & 31;
#pragma unroll
    for (int i = 0; i < WM; ++i) {
        const int64_t mblk = (mb0 + wm * WM + i) * 32;
        const int64_t m = mblk + mloc;
        const float dq = sc.dq[i];
        const int qs = sc.qs[i];
#pragma unroll
        for (int j = 0; j < WN; ++j)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int ncol = j * 32 + 8 * g + 4 * half;          // first of 4 consecutive columns, tile-relative
                float o[4];
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    o[t] = __fmul_rn(__fmul_rn((float)(acc[i][j][4 * g + t] - qs), dq), wdq[j]);
                    if (bias) {
                        const int64_t n = nb0 * 32 + ncol + t;
                        o[t] = __fadd_rn(o[t], n < p.N ? mmf_to_float(bias[n]) : 0.0f);
                    }
                }
                if (p.vec_store) {
                    if constexpr (E == 2)
                        *reinterpret_cast<uint2*>(stage + mloc * RS + ncol * 2) = make_uint2(pack2<T>(o[0], o[1]), pack2<T>(o[2], o[3]));
                    else
                        *reinterpret_cast<float4*>(stage + mloc * RS + ncol * 4) = make_float4(o[0], o[1], o[2], o[3]);
                } else if (m < p.M) {
#pragma unroll
                    for (int t = 0; t < 4; ++t) {
                        const int64_t n = nb0 * 32 + ncol + t;
                        if (n < p.N) {
                            float v = o[t];
                            if (addend) v = __fadd_rn(mmf_round_to<T>(v), mmf_to_float(addend[m * p.ldo + n]));
                            out[m * p.ldo + n] = mmf_from_float<T>(v);
                        }
                    }
                }
            }
        if (p.vec_store) {
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
            for (int c0 = 0; c0 < 32 * CPR; c0 += 64) {
                const int c = c0 + lane;
                const int row = c / CPR, cc = c % CPR;
                const int64_t mr = mblk + row, n = nb0 * 32 + cc * (16 / E);
                if (mr < p.M && n < p.N) {
                    uint4 v = *reinterpret_cast<const uint4*>(stage + row * RS + cc * 16);
                    if (addend) {
                        const uint4 av = *reinterpret_cast<const uint4*>(addend + mr * p.ldo + n);
                        T pe[16 / E], ae[16 / E], oe[16 / E];
                        __builtin_memcpy(pe, &v, 16);
                        __builtin_memcpy(ae, &av, 16);
#pragma unroll
                        for (int e = 0; e < 16 / E; ++e) oe[e] = mmf_from_float<T>(__fadd_rn(mmf_to_float(pe[e]), mmf_to_float(ae[e])));
                        __builtin_memcpy(&v, oe, 16);
                    }
                    *reinterpret_cast<uint4*>(out + mr * p.ldo + n) = v;
                }
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        }
    }
}

// Lean epilogue of the common case (16-byte stores possible, no bias): the accumulators were
// started at -qsum[m], so a value costs one convert and two multiplies; lane-constant parts of the
// store addresses are computed once; interior tiles skip the bounds tests.
template <typename T, int WM, int WN>
__device__ __forceinline__ void mfma_epilogue_fast(const MfmaArgs& p, v16i (&acc)[WM][WN], const EpiScales<WM, WN>& sc,
                                                   unsigned char* smem, int lane, int wave, int wm, int64_t mb0, int64_t nb0) {
    const T* addend = static_cast<const T*>(p.addend);
    T* out = static_cast<T*>(p.out);
    constexpr int E = sizeof(T);
    constexpr int RS = WN * 32 * E + 16;          // LDS row stride of a wave's 32 x (WN*32) staging tile
    constexpr int CPR = WN * 32 * E / 16;         // 16-byte chunks per row (divides 64)
    constexpr int RPI = 64 / CPR;                 // rows covered by one 64-lane store
    unsigned char* stage = smem + wave * (32 * RS);
    const int half = lane >> 5, mloc = lane & 31;
    const int cc = lane % CPR, rsub = lane / CPR;
    const int64_t m_first = (mb0 + wm * WM) * 32, n_first = nb0 * 32;
    const bool interior = m_first + WM * 32 <= p.M && n_first + WN * 32 <= p.N;
    const int64_t n = n_first + cc * (16 / E);
    const int64_t lane_off = (m_first + rsub) * p.ldo + n;         // element offset of this lane's first chunk
    unsigned char* wr = stage + mloc * RS + 4 * half * E;
    const unsigned char* rd = stage + rsub * RS + cc * 16;
#pragma unroll
    for (int i = 0; i < WM; ++i) {
        const float dq = sc.dq[i];
#pragma unroll
        for (int j = 0; j < WN; ++j)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                float o[4];
#pragma unroll
                for (int t = 0; t < 4; ++t) o[t] = __fmul_rn(__fmul_rn((float)acc[i][j][4 * g + t], dq), sc.wdq[j]);
                unsigned char* w = wr + (j * 32 + 8 * g) * E;
                if constexpr (E == 2) *reinterpret_cast<uint2*>(w) = make_uint2(pack2<T>(o[0], o[1]), pack2<T>(o[2], o[3]));
                else *reinterpret_cast<float4*>(w) = make_float4(o[0], o[1], o[2], o[3]);
            }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
        for (int r0 = 0; r0 < 32; r0 += RPI) {
            const int64_t off = lane_off + (int64_t)(i * 32 + r0) * p.ldo;
            if (interior || (m_first + i * 32 + r0 + rsub < p.M && n < p.N)) {
                uint4 v = *reinterpret_cast<const uint4*>(rd + r0 * RS);
                if (addend) {
                    const uint4 av = *reinterpret_cast<const uint4*>(addend + off);
                    T pe[16 / E], ae[16 / E], oe[16 / E];
                    __builtin_memcpy(pe, &v, 16);
                    __builtin_memcpy(ae, &av, 16);
#pragma unroll
                    for (int e = 0; e < 16 / E; ++e) oe[e] = mmf_from_float<T>(__fadd_rn(mmf_to_float(pe[e]), mmf_to_float(ae[e])));
                    __builtin_memcpy(&v, oe, 16);
                }
                *reinterpret_cast<uint4*>(out + off) = v;
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
}

// Epilogue of the gate/up contraction with the MLP activation folded in (mmfreelm/models/hgrn_bit/modeling_hgrn_bit.py:55-59):
// the wave's two n-blocks are the gate and the up projection of the same 32 channels, so a lane holds both operands of
// out = T((g * u) / (1 + exp(-g))), g = T(gate), u = T(up), and the wave writes 32 columns of the [M, N/2] result.
// Same conditions as the lean epilogue (accumulators started at -qsum, 16-byte stores).
template <typename T, int WM>
__device__ __forceinline__ void mfma_epilogue_swiglu(const MfmaArgs& p, v16i (&acc)[WM][2], const EpiScales<WM, 2>& sc,
                                                     unsigned char* smem, int lane, int wave, int wm, int64_t mb0, int64_t nbg) {
    T* out = static_cast<T*>(p.out);
    constexpr int E = sizeof(T);
    constexpr int RS = 32 * E + 16;               // LDS row stride of a wave's 32 x 32 staging tile
    constexpr int CPR = 32 * E / 16;              // 16-byte chunks per row
    constexpr int RPI = 64 / CPR;                 // rows covered by one 64-lane store
    unsigned char* stage = smem + wave * (32 * RS);
    const int half = lane >> 5, mloc = lane & 31;
    const int cc = lane % CPR, rsub = lane / CPR;
    const int64_t nseg = p.N >> 1;
    const int64_t m_first = (mb0 + wm * WM) * 32, n_first = nbg * 32;
    const bool interior = m_first + WM * 32 <= p.M && n_first + 32 <= nseg;
    const int64_t n = n_first + cc * (16 / E);
    const int64_t lane_off = (m_first + rsub) * p.ldo + n;
    unsigned char* wr = stage + mloc * RS + 4 * half * E;
    const unsigned char* rd = stage + rsub * RS + cc * 16;
#pragma unroll
    for (int i = 0; i < WM; ++i) {
        const float dq = sc.dq[i];
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            float o[4];
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const float gv = mmf_round_to<T>(__fmul_rn(__fmul_rn((float)acc[i][0][4 * g + t], dq), sc.wdq[0]));
                const float uv = mmf_round_to<T>(__fmul_rn(__fmul_rn((float)acc[i][1][4 * g + t], dq), sc.wdq[1]));
                o[t] = __fdiv_rn(__fmul_rn(gv, uv), __fadd_rn(1.0f, mmf_exp(-gv)));
            }
            unsigned char* w = wr + (8 * g) * E;
            if constexpr (E == 2) *reinterpret_cast<uint2*>(w) = make_uint2(pack2<T>(o[0], o[1]), pack2<T>(o[2], o[3]));
            else *reinterpret_cast<float4*>(w) = make_float4(o[0], o[1], o[2], o[3]);
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
        for (int r0 = 0; r0 < 32; r0 += RPI) {
            const int64_t off = lane_off + (int64_t)(i * 32 + r0) * p.ldo;
            if (interior || (m_first + i * 32 + r0 + rsub < p.M && n < nseg))
                *reinterpret_cast<uint4*>(out + off) = *reinterpret_cast<const uint4*>(rd + r0 * RS);
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
}

template <typename T, int WGM, int WGN, int WM, int WN, int KSL>
__global__ __launch_bounds__(64 * WGM * WGN) void bitlinear_mfma_kernel(MfmaArgs p) {
    constexpr int NT = 64 * WGM * WGN;
    constexpr int BMB = WGM * WM;                 // m-blocks (of 32 rows) per workgroup tile
    constexpr int BNB = WGN * WN;                 // n-blocks per workgroup tile
    constexpr int CH = KSL * 4096;                // bytes of one m-block's slab (KSL k-blocks of 128)
    constexpr int PIECES = BMB * (CH / 16);       // 16-byte pieces of one A slab
    constexpr int NPA = (PIECES + NT - 1) / NT;   // pieces per thread
    extern __shared__ __align__(16) unsigned char smem[];   // 2 x BMB x CH bytes

    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);   // wave-uniform: keep it in a scalar register
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
    EpiScales<WM, WN> sc;
    mfma_prefetch_scales<WM, WN>(p, sc, lane, wm, mb0, nb0);

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
                    acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(bf[j], af[ks & 1][i], acc[i][j], 0, 0, 0);
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

    mfma_epilogue<T, WM, WN>(p, acc, sc, smem, lane, wave, wm, mb0, nb0);
}

typedef __attribute__((address_space(3))) void* mmf_lds_ptr;
typedef __attribute__((address_space(1))) const void* mmf_glb_ptr;

// One 1 KiB wave-load global -> LDS (16 bytes per lane; lane l lands at lds + 16 l) from `base` (wave-uniform) + 16 l.
// Written in assembly so that the compiler does not know of an LDS write in flight: it answers the builtin with waits
// for all vector-memory traffic in front of later LDS reads and barriers, at places of its own choosing (the top of the
// k-loop, half a k-block after the request).  The kernel waits for its transfers itself, once per k-block, where the
// data is needed.
__device__ __forceinline__ void mfma_dma_1k(const void* base, uint32_t lane16, const unsigned char* lds) {
    const uint32_t l = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const unsigned char*)lds;
    const uint64_t b = (uint64_t)base;
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(l), "v"(lane16), "s"(b) : "memory");
}
// Workgroup barrier behind an explicit wait: at most `VM` vector-memory operations may stay in flight, LDS traffic done.
// Only VM = 0 says anything about a transfer into LDS: such transfers and ordinary loads complete in no fixed order.
template <int VM>
__device__ __forceinline__ void mfma_barrier_vm() {
    static_assert(VM >= 0 && VM < 64, "vmcnt is a 6-bit count");
    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(VM) : "memory");
}

// ------------------------------------------------------------------------------------------
// The large-M kernel.  Same tiling, but A goes global -> LDS by DMA (global_load_lds_dwordx4:
// lane l's 16 bytes land at the wave-uniform LDS base + 16*l, which is exactly the
// fragment-tiled layout), so no VGPRs stage it and no ds_write sits in the instruction stream.
// Three A buffers of one 128-wide k-block each and ONE barrier per k-block,
// placed after the second of its four k-steps.  At that barrier every wave has left the previous
// k-block, so its buffer is free for the DMA of k-block s+2, and k-block s+1 (issued one k-block
// earlier, waited for by each wave just before the barrier, together with the packed weights
// requested with it) is complete for everybody.  K-block
// boundaries therefore carry no synchronisation: the A fragments of the next k-block's first
// step are read while the current one's last MFMAs run, and the matrix pipe never drains.
// FAST (chosen by the launcher): 16-byte stores possible and no bias -> lean epilogue, accumulators start at -qsum.
// SWI: the weight is the stacked [gate; up] projection (N = 2 * I): a wave's two n-blocks are the gate and the up rows
// of the same 32 channels, a workgroup tile covers WGN such channel blocks, and the epilogue writes swiglu(gate, up).
template <typename T, int WGM, int WGN, int WM, int WN, bool FAST, bool SWI = false>
__global__ __launch_bounds__(64 * WGM * WGN, (WM * WN <= 4 ? 4 : 1))   // small wave tiles: 4 waves per SIMD = two workgroups per CU
void bitlinear_mfma_dma3_kernel(MfmaArgs p) {
    constexpr int NW = WGM * WGN;
    constexpr int BMB = WGM * WM;
    constexpr int BNB = WGN * WN;
    constexpr int CH = 4096;                       // bytes of one m-block's k-block
    constexpr int BUF = BMB * CH;
    constexpr int WPIECES = BMB * CH / 1024;       // 1 KiB wave-loads per k-block
    constexpr int NDMA = (WPIECES + NW - 1) / NW;  // per wave
    static_assert(WPIECES % NW == 0, "every wave issues the same number of DMA pieces");
    extern __shared__ __align__(16) unsigned char smem[];

    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wm = wave / WGN, wn = wave % WGN;
    long long clk0 = 0, wall0 = 0;
    if (p.clocks) { clk0 = __builtin_amdgcn_s_memtime(); wall0 = __builtin_amdgcn_s_memrealtime(); }
    // Workgroup ids are dealt round-robin to the 8 XCDs.  The tile rows are cut into bands of 8 * RB rows; inside a band
    // XCD x owns rows [x * RB, (x + 1) * RB) and walks the columns with the rows running fastest: the RB workgroups that
    // share a weight tile run together, and the RB activation panels (sized by the host to stay in that XCD's L2) are
    // re-read from L2 for every column.  Bands follow one another.
    int64_t wg = blockIdx.x;
    const int64_t total = (int64_t)p.tiles_m * p.tiles_n;
    int64_t tile_m, tile_n;
    if (p.rows_per_xcd > 0) {
        const int RB = p.rows_per_xcd, x = (int)(wg & 7);
        const int64_t l = wg >> 3, per_band = (int64_t)RB * p.tiles_n;
        const int64_t band = l / per_band, l2 = l % per_band;
        tile_m = band * 8 * RB + x * RB + l2 % RB;
        tile_n = l2 / RB;
    } else {
        if (total % 8 == 0) wg = (wg % 8) * (total / 8) + wg / 8;
        tile_m = wg / p.tiles_n;
        tile_n = wg % p.tiles_n;
    }
    const int64_t MB = (p.M + 31) >> 5, NB = (p.N + 31) >> 5;
    const int KB = (int)(p.Kp >> 7);
    const int64_t KG = p.Kp >> 4;
    static_assert(!SWI || (WN == 2 && FAST), "the swiglu epilogue pairs a gate and an up n-block per wave");
    const int64_t NBs = NB >> 1;                                  // SWI: n-blocks per stacked segment
    const int64_t mb0 = tile_m * BMB, nb0 = SWI ? tile_n * WGN + wn : tile_n * BNB + wn * WN;
    // the n-block behind accumulator column j (columns past the end re-read a valid block and are never stored)
    auto nblock = [&](int j) -> int64_t {
        if constexpr (SWI) return (nb0 < NBs ? nb0 : NBs - 1) + j * NBs;
        else return nb0 + j < NB ? nb0 + j : NB - 1;
    };
    EpiScales<WM, WN> sc;
    mfma_prefetch_scales<WM, WN>(p, sc, lane, wm, mb0, nb0);
    if constexpr (SWI) {
#pragma unroll
        for (int j = 0; j < WN; ++j) sc.wdq[j] = p.wdeq[(uint32_t)(nblock(j) * 32) / (uint32_t)p.seg_rows];
    }

    auto dma_block = [&](int kb, int boff) {                      // k-block kb -> buffer at byte offset boff
#pragma unroll
        for (int i = 0; i < NDMA; ++i) {
            const int w = i * NW + wave;
            const int chunk = w >> 2, within = w & 3;             // 4 pieces per m-block
            int64_t mb = mb0 + chunk;
            if (mb >= MB) mb = MB - 1;                            // rows past M are never stored: any valid data will do
            const int kbc = kb < KB ? kb : KB - 1;                // past the end: harmless re-read, never consumed
            const unsigned char* g = reinterpret_cast<const unsigned char*>(p.a) + (mb * KG + kbc * 8 + within * 2) * 512;
            mfma_dma_1k(g, (uint32_t)lane * 16u, smem + boff + w * 1024);
        }
    };
    auto load_b = [&](int kb, uint4 (&dst)[WN]) {                 // unconditional: the barrier's vmcnt counts on WN loads
#pragma unroll
        for (int j = 0; j < WN; ++j) {
            const int64_t nb = nblock(j);
            const int kbc = kb < KB ? kb : KB - 1;                // past the end: never consumed
            // wave-uniform block address + a 32-bit lane offset: the load then takes its base from scalar registers and
            // no 64-bit per-lane address is kept alive
            const unsigned char* blk = reinterpret_cast<const unsigned char*>(p.b + (nb * KB + kbc) * 64);
            dst[j] = *reinterpret_cast<const uint4*>(blk + (uint32_t)(lane * 16));
        }
    };
    auto expand_b = [&](const uint4 (&src)[WN], int ks, v4i (&bf)[WN]) {
#pragma unroll
        for (int j = 0; j < WN; ++j) {
            const uint32_t w = ks == 0 ? src[j].x : ks == 1 ? src[j].y : ks == 2 ? src[j].z : src[j].w;
            bf[j][0] = (int)(w & 0x03030303u);
            bf[j][1] = (int)((w >> 2) & 0x03030303u);
            bf[j][2] = (int)((w >> 4) & 0x03030303u);
            bf[j][3] = (int)((w >> 6) & 0x03030303u);
        }
    };

    // B is requested a k-block and a half before its first use, into a ring of three register sets.  The ring is walked
    // by unrolling the k-loop three times, so a set keeps its registers from its load to its last use (rotating the sets
    // with copies at the loop's back edge makes the compiler wait there for everything in flight: the copy reads the set
    // loaded last).
    uint4 bset0[WN], bset1[WN], bset2[WN];
    dma_block(0, 0);
    dma_block(1, BUF);
    load_b(0, bset0);
    load_b(1, bset1);
    __builtin_amdgcn_s_waitcnt(0x0F70);            // vmcnt(0): this wave's pieces of k-blocks 0 and 1 have landed
    __syncthreads();

    // a lane's 16 accumulator registers of one tile all belong to output row (lane % 32)
    v16i acc[WM][WN];
#pragma unroll
    for (int i = 0; i < WM; ++i) {
        const int init = FAST ? -sc.qs[i] : 0;
#pragma unroll
        for (int j = 0; j < WN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = init;
    }
    const int aoff = (wm * WM) * CH + lane * 16;
    int cur = 0, nxt = BUF, fre = 2 * BUF;         // byte offsets of the buffers of k-blocks s, s+1, s+2
    v4i af[2][WM];
#pragma unroll
    for (int i = 0; i < WM; ++i) af[0][i] = *reinterpret_cast<const v4i*>(smem + cur + aoff + i * CH);

    // one k-block: contracts with the set `bcur`, requests k-block kb + 2 into `bfar`; the expansion of the NEXT step's
    // weights (the first step of `bnxt` at the end) is interleaved with this step's MFMAs
    v4i bf[WN];
    expand_b(bset0, 0, bf);
    auto kblock = [&](int kb, const uint4 (&bcur)[WN], const uint4 (&bnxt)[WN], uint4 (&bfar)[WN]) {
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            if (ks == 2) {
                // Everything requested one k-block ago -- this wave's pieces of A k-block kb+1 and the weights of kb+1 --
                // has to be here now.  The wait is for ALL vector-memory traffic: a transfer into LDS and an ordinary load
                // do not complete in the order they were issued (a count that leaves the younger weight loads in flight let
                // warm weight loads overtake a cold A transfer and gave wrong sums), so the next requests go out right
                // behind the barrier and have a whole k-block to land.
                mfma_barrier_vm<0>();
                dma_block(kb + 2, fre);
                load_b(kb + 2, bfar);
            }
            const unsigned char* nsrc = ks < 3 ? smem + cur + aoff + (ks + 1) * 1024 : smem + nxt + aoff;
#pragma unroll
            for (int i = 0; i < WM; ++i) af[(ks + 1) & 1][i] = *reinterpret_cast<const v4i*>(nsrc + i * CH);
            // weight columns outermost: once the MFMAs of column j are issued, the next step's expansion of column j can
            // reuse its registers and runs in the shadow of the matrix pipe
            v4i bn[WN];
#pragma unroll
            for (int j = 0; j < WN; ++j) {
#pragma unroll
                for (int i = 0; i < WM; ++i)
                    acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(bf[j], af[ks & 1][i], acc[i][j], 0, 0, 0);
                const uint32_t w = ks == 0 ? bcur[j].y : ks == 1 ? bcur[j].z : ks == 2 ? bcur[j].w : bnxt[j].x;
                bn[j][0] = (int)(w & 0x03030303u);
                bn[j][1] = (int)((w >> 2) & 0x03030303u);
                bn[j][2] = (int)((w >> 4) & 0x03030303u);
                bn[j][3] = (int)((w >> 6) & 0x03030303u);
            }
            __builtin_amdgcn_sched_group_barrier(0x100, WM, 0);
#pragma unroll
            for (int j = 0; j < WN; ++j) {
                __builtin_amdgcn_sched_group_barrier(0x008, WM, 0);
                __builtin_amdgcn_sched_group_barrier(0x002, 7, 0);
            }
#pragma unroll
            for (int j = 0; j < WN; ++j) bf[j] = bn[j];
            __builtin_amdgcn_sched_barrier(0);
        }
        const int t = cur; cur = nxt; nxt = fre; fre = t;
    };
    int kb = 0;
    for (; kb + 3 <= KB; kb += 3) {
        kblock(kb, bset0, bset1, bset2);
        kblock(kb + 1, bset1, bset2, bset0);
        kblock(kb + 2, bset2, bset0, bset1);
    }
    if (kb < KB) {
        kblock(kb, bset0, bset1, bset2);
        if (kb + 1 < KB) kblock(kb + 1, bset1, bset2, bset0);
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);            // the trailing DMA must not land in the epilogue's staging area
    __syncthreads();
    if constexpr (SWI) mfma_epilogue_swiglu<T, WM>(p, acc, sc, smem, lane, wave, wm, mb0, nb0);
    else if constexpr (FAST) mfma_epilogue_fast<T, WM, WN>(p, acc, sc, smem, lane, wave, wm, mb0, nb0);
    else mfma_epilogue<T, WM, WN>(p, acc, sc, smem, lane, wave, wm, mb0, nb0);
    if (p.clocks && threadIdx.x == 0 && (int64_t)blockIdx.x < p.clock_cap) {
        p.clocks[2 * blockIdx.x] = __builtin_amdgcn_s_memtime() - clk0;
        p.clocks[2 * blockIdx.x + 1] = __builtin_amdgcn_s_memrealtime() - wall0;
    }
}

// Tile rows per XCD and band (see the kernel): the largest divisor of tiles_m / 8 whose activation panels
// (tile_rows * Kp bytes each) stay within 1.5 MiB of an XCD's 4 MiB L2 (measured at 16384 x 2048 x 11264: 0.389 ms
// against 0.410 ms with all 32 panels of an XCD in one band; smaller budgets are no better); 0 when tiles_m is not a
// multiple of 8.
inline int mfma_rows_per_xcd(int tiles_m, int tile_rows, int64_t Kp) {
    if (tiles_m % 8 != 0) return 0;
    const int R = tiles_m / 8;
    const int64_t budget = 1536 << 10;
    int64_t cap = budget / ((int64_t)tile_rows * Kp);
    if (cap < 1) cap = 1;
    int best = 1;
    for (int d = 1; d <= R && d <= cap; ++d)
        if (R % d == 0) best = d;
    return best;
}

// The 64 x 512 tile on the stacked [gate; up] weight with the swiglu epilogue: a tile is 64 rows x 256 channels.
template <typename T>
int launch_mfma_dma3_swiglu(MfmaArgs a, hipStream_t s) {
    constexpr int WGM = 1, WGN = 8, WM = 2, WN = 2;
    a.clocks = g_clock_sink; a.clock_cap = g_clock_cap;
    a.tiles_m = (int)mmf_ceil_div(a.M, WGM * WM * 32);
    a.tiles_n = (int)mmf_ceil_div(a.N / 2, WGN * 32);
    a.rows_per_xcd = mfma_rows_per_xcd(a.tiles_m, WGM * WM * 32, a.Kp);
    size_t lds = 3u * (WGM * WM) * 4096u;
    const size_t lds_epi = (size_t)(WGM * WGN) * 32u * (32u * sizeof(T) + 16u);
    if (lds_epi > lds) lds = lds_epi;
    a.vec_store = 1;
    auto kern = bitlinear_mfma_dma3_kernel<T, WGM, WGN, WM, WN, true, true>;
    if (lds > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                           (int)lds);
        if (e != hipSuccess) return (int)e;
    }
    kern<<<dim3((unsigned)((int64_t)a.tiles_m * a.tiles_n)), dim3(64 * WGM * WGN), lds, s>>>(a);
    MMF_CHECK_LAUNCH();
    return 0;
}

template <typename T, int WGM, int WGN, int WM, int WN>
int launch_mfma_dma3(MfmaArgs a, hipStream_t s) {
    constexpr int BM = WGM * WM * 32, BN = WGN * WN * 32;
    a.clocks = g_clock_sink; a.clock_cap = g_clock_cap;
    a.tiles_m = (int)mmf_ceil_div(a.M, BM);
    a.tiles_n = (int)mmf_ceil_div(a.N, BN);
    a.rows_per_xcd = mfma_rows_per_xcd(a.tiles_m, BM, a.Kp);
    size_t lds = 3u * (WGM * WM) * 4096u;
    const size_t lds_epi = (size_t)(WGM * WGN) * 32u * (WN * 32u * sizeof(T) + 16u);
    if (lds_epi > lds) lds = lds_epi;
    const int per_vec = 16 / (int)sizeof(T);
    a.vec_store = (a.N % per_vec == 0) && (a.ldo % per_vec == 0) && ((reinterpret_cast<uintptr_t>(a.out) & 15u) == 0) &&
                  ((reinterpret_cast<uintptr_t>(a.addend) & 15u) == 0);
    const bool fast = a.vec_store && !a.bias;
    auto kern = fast ? bitlinear_mfma_dma3_kernel<T, WGM, WGN, WM, WN, true> : bitlinear_mfma_dma3_kernel<T, WGM, WGN, WM, WN, false>;
    if (lds > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                           (int)lds);
        if (e != hipSuccess) return (int)e;
    }
    kern<<<dim3((unsigned)((int64_t)a.tiles_m * a.tiles_n)), dim3(64 * WGM * WGN), lds, s>>>(a);
    MMF_CHECK_LAUNCH();
    return 0;
}

// ------------------------------------------------------------------------------------------
// Small problems (decode batches, short prompts): the contraction is a weight stream, not a
// GEMM, and the enemy is latency, so nothing is staged and nothing waits on a barrier until the
// very end.  One workgroup of 8 waves owns MB 32x32 output blocks of one 32-row n-block (grid.y
// walks M); wave w takes the k-blocks w, w+8, ...
// A fragments (1 KiB each, L2 resident: the whole A is M x K bytes) and the packed B block
// are loaded straight into registers, three k-blocks in flight per wave; the 8 partial
// accumulators meet in LDS and all 512 threads run the epilogue.
template <typename T, int MB>
__global__ __launch_bounds__(512) void bitlinear_mfma_skinny_kernel(MfmaArgs p) {
    constexpr int NWV = 8, PF = 3, MAXK = 8;            // Kp <= 8 * 8 * 128
    __shared__ int red[NWV][MB][16][64];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);   // wave-uniform: keep it in a scalar register
    const int64_t nb = blockIdx.x, mbase = (int64_t)blockIdx.y * MB;   // this workgroup's first m-block
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
                    if (mbase + i < MBtot)
                        areg[st][i][ks] = *reinterpret_cast<const v4i*>(p.a + ((mbase + i) * KG + kb * 8 + ks * 2) * 512 + lane * 16);
                }
        }
    };
#pragma unroll
    for (int st = 0; st < PF; ++st) load_stage(st, wave + (int64_t)st * NWV);

    // the epilogue's operands, requested now so that the end of the kernel waits for nothing
    const T* bias = static_cast<const T*>(p.bias);
    const T* addend = static_cast<const T*>(p.addend);
    T* out = static_cast<T*>(p.out);
    const int64_t n_ep = nb * 32 + (lane & 31);
    const bool n_ok = n_ep < p.N;
    const float ep_wdeq = p.wdeq[(uint32_t)(nb * 32) / (uint32_t)p.seg_rows];   // an n-block never straddles a segment
    const float ep_bias = (bias && n_ok) ? mmf_to_float(bias[n_ep]) : 0.0f;
    int ep_qsum[MB * 2];
    float ep_deq[MB * 2], ep_add[MB * 2];
#pragma unroll
    for (int j = 0; j < MB * 2; ++j) {
        const int e = threadIdx.x + j * 512;             // (mb, r, lane) flattened
        const int r = (e >> 6) & 15, mb = e >> 10;
        const int64_t m = (mbase + mb) * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
        const int64_t mc = m < p.M ? m : 0;
        ep_qsum[j] = p.qsum[mc];
        ep_deq[j] = p.deq[mc];
        ep_add[j] = (addend && n_ok) ? mmf_to_float(addend[mc * p.ldo + n_ep]) : 0.0f;
    }

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

#pragma unroll
    for (int j = 0; j < MB * 2; ++j) {
        const int e = threadIdx.x + j * 512;             // (mb, r, lane) flattened
        const int r = (e >> 6) & 15, mb = e >> 10;
        int tot = 0;
#pragma unroll
        for (int w = 0; w < NWV; ++w) tot += red[w][mb][r][lane];
        const int64_t m = (mbase + mb) * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
        if (m < p.M && n_ok) {
            float o = __fmul_rn(__fmul_rn((float)(tot - ep_qsum[j]), ep_deq[j]), ep_wdeq);
            if (bias) o = __fadd_rn(o, ep_bias);
            if (addend) o = __fadd_rn(mmf_round_to<T>(o), ep_add[j]);
            out[m * p.ldo + n_ep] = mmf_from_float<T>(o);
        }
    }
}

template <typename T, int MB>
int launch_skinny(const MfmaArgs& a, hipStream_t s) {
    bitlinear_mfma_skinny_kernel<T, MB><<<dim3((unsigned)mmf_ceil_div(a.N, 32), (unsigned)mmf_ceil_div(a.M, 32 * MB)), dim3(512), 0, s>>>(a);
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
    // config < 0: pick by shape.
    //   5        weight-stream kernel: one 32x32 output block per workgroup, 8 waves split K (needs Kp <= 8192)
    //   0 / 1    32x256 / 64x256 tiles, A staged through registers (small M with Kp > 8192)
    //   15 / 16 / 17  256x256 / 128x256 / 64x512 tiles, A staged by DMA (17: every wave reads the whole activation
    //            tile from LDS and owns its own weight columns, so no weight block is fetched twice)
    if (config < 0) {
        const int64_t KB = a.Kp >> 7;
        const double wgs = (double)mmf_ceil_div(a.M, 32) * (double)mmf_ceil_div(a.N, 32);
        const double tiles = (double)mmf_ceil_div(a.M, 128) * (double)mmf_ceil_div(a.N, 256);
        // measured on MI355X: the stream kernel costs ~3 us + 0.33 ns per (output block x k-block); a round of
        // tiles of the DMA kernel ~0.9 us per k-block whatever the problem size
        const double t_stream = 3.0 + wgs * (double)KB * 0.00033;
        const double t_tiled = (double)KB * 0.9 * (double)mmf_ceil_div((int64_t)tiles, 256);
        if (a.Kp <= 8192 && (a.M <= 64 || t_stream < t_tiled)) config = 5;
        else if (a.M <= 32) config = 0;
        else if (a.M <= 64) config = 1;
        else config = a.N >= 512 ? 17 : 16;
    }
    if (config == 5 && (a.Kp > 8192 || a.M > 65535 * 32)) return MMF_ERR_ARG;
    switch (config) {
        case 5: return launch_skinny<T, 1>(a, s);
        case 0: return launch_mfma<T, 1, 8, 1, 1>(a, s);
        case 1: return launch_mfma<T, 1, 8, 2, 1>(a, s);
        case 15: return launch_mfma_dma3<T, 2, 4, 4, 2>(a, s);
        case 16: return launch_mfma_dma3<T, 2, 4, 2, 2>(a, s);
        case 17: return launch_mfma_dma3<T, 1, 8, 2, 2>(a, s);
    }
    return MMF_ERR_ARG;
}

// The matrix pipe with nothing else to do: every wave issues the tiled kernel's four independent 32x32x32 int8 MFMAs per
// step on operands that never leave its registers (8 waves per workgroup, 4 waves per SIMD with two workgroups per CU).
// random_operands: int8 codes and ternary weights drawn per lane (the switching activity of real operands) instead of the
// constant 1s, on which the pipe draws far less power.
__global__ __launch_bounds__(512, 4) void mfma_pipe_probe_kernel(int64_t steps, int random_operands, long long* clocks, int* sink) {
    const long long clk0 = __builtin_amdgcn_s_memtime(), wall0 = __builtin_amdgcn_s_memrealtime();
    auto mix = [](uint32_t x) { x ^= x >> 16; x *= 0x7feb352du; x ^= x >> 15; x *= 0x846ca68bu; x ^= x >> 16; return x; };
    v4i a[2], b[2];
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            a[h][i] = random_operands ? (int)mix(threadIdx.x * 16 + h * 4 + i) : 0x01010101 * (int)(threadIdx.x & 1);
            b[h][i] = random_operands ? (int)(mix(threadIdx.x * 16 + 8 + h * 4 + i) & 0x03030303u) : 0x01010101;
        }
    v16i acc[4];
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[t][r] = 0;
    for (int64_t s = 0; s < steps; ++s) {
#pragma unroll
        for (int t = 0; t < 4; ++t) acc[t] = __builtin_amdgcn_mfma_i32_32x32x32_i8(b[t & 1], a[t >> 1], acc[t], 0, 0, 0);
    }
    int x = 0;
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) x ^= acc[t][r];
    if (x == 0x7fffffff) *sink = x;                              // keeps the accumulators live; never true
    if (threadIdx.x == 0) {
        clocks[2 * blockIdx.x] = __builtin_amdgcn_s_memtime() - clk0;
        clocks[2 * blockIdx.x + 1] = __builtin_amdgcn_s_memrealtime() - wall0;
    }
}

}  // namespace

extern "C" {

int mmf_bitlinear_mfma_clock_sink(int64_t* sink, int64_t workgroups) {
    if (workgroups < 0 || (sink && workgroups == 0)) return MMF_ERR_ARG;
    g_clock_sink = reinterpret_cast<long long*>(sink);
    g_clock_cap = sink ? workgroups : 0;
    return 0;
}

int mmf_mfma_pipe_probe(int64_t steps, int64_t workgroups, int random_operands, int64_t* clocks, void* stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (steps < 0 || workgroups <= 0 || workgroups > 65535 || !clocks) return MMF_ERR_ARG;
    // the word after the clocks is the sink of the never-taken store
    mfma_pipe_probe_kernel<<<(unsigned)workgroups, 512, 0, stream>>>(steps, random_operands, reinterpret_cast<long long*>(clocks),
                                                                    reinterpret_cast<int*>(clocks + 2 * workgroups));
    MMF_CHECK_LAUNCH();
    return 0;
}

int mmf_bitlinear_mfma(const int8_t* codes_tiled, const float* deq, const int* qsum, const void* packed,
                       const float* wdeq, int64_t seg_rows, const void* bias, const void* addend, void* out, int64_t ldo,
                       int64_t M,
                       int64_t K, int64_t N, int out_dtype, int config, void* stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (M < 0 || K <= 0 || N <= 0 || seg_rows <= 0 || seg_rows % 32 != 0 || ldo < N || N > 0x7fffffff) return MMF_ERR_ARG;
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

int mmf_bitlinear_mfma_swiglu(const int8_t* codes_tiled, const float* deq, const int* qsum, const void* packed,
                              const float* wdeq, int64_t seg_rows, void* out, int64_t ldo, int64_t M, int64_t K, int64_t N,
                              int out_dtype, void* stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (M < 0 || K <= 0 || N <= 0 || N % 64 != 0 || seg_rows <= 0 || seg_rows % 32 != 0 || ldo < N / 2 || N > 0x7fffffff)
        return MMF_ERR_ARG;
    if (M == 0) return 0;
    if (!codes_tiled || !deq || !qsum || !packed || !wdeq || !out) return MMF_ERR_ARG;
    const int64_t per_vec = out_dtype == MMF_F32 ? 4 : 8;
    if ((reinterpret_cast<uintptr_t>(codes_tiled) & 15u) || (reinterpret_cast<uintptr_t>(packed) & 15u) ||
        (reinterpret_cast<uintptr_t>(out) & 15u) || ldo % per_vec != 0)
        return MMF_ERR_ALIGN;
    MfmaArgs a{};
    a.a = codes_tiled; a.b = static_cast<const uint4*>(packed); a.deq = deq; a.qsum = qsum; a.wdeq = wdeq;
    a.out = out; a.M = M; a.N = N; a.Kp = mmf_round_up(K, 128); a.seg_rows = seg_rows; a.ldo = ldo;
    switch (out_dtype) {
        case MMF_F32: return launch_mfma_dma3_swiglu<float>(a, stream);
        case MMF_BF16: return launch_mfma_dma3_swiglu<bf16_t>(a, stream);
        case MMF_F16: return launch_mfma_dma3_swiglu<f16_t>(a, stream);
    }
    return MMF_ERR_ARG;
}

}  // extern "C"
