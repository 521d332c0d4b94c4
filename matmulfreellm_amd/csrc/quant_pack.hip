// Absmean ternarisation of a latent weight matrix and 2-bit packing.
//
// Replaces the per-forward weight_quant() of mmfreelm/ops/fusedbitnet.py:32-46 (called at
// :456 on every forward) with a one-time pass that stores the codes 2-bit packed.
//
// Packed layout (the contraction kernels' native operand layout): the [N, K] matrix is
// padded with code 0 to Np = ceil32(N), Kp = ceil128(K) and cut into blocks of 32 output
// rows x 128 inputs.  One block is 64 lanes x 4 dwords = 1 KiB, blocks ordered
// [Np/32][Kp/128].  Dword s of lane l (half = l / 32, row = l % 32) holds the 16 inputs
// k = kb*128 + s*32 + half*16 + i, i = 0..15; input i is the 2-bit field (t + 1) at bit
// 8*(i % 4) + 2*(i / 4), so (dword >> 2j) & 0x03030303 is four byte-wide codes for
// i = 4j..4j+3 -- exactly the int8 B-operand bytes one lane feeds v_mfma_i32_32x32x32_i8.
#include "mmf_common.h"
#include "../../include/mmf.h"

namespace {

constexpr int kPartials = 1024;   // fp64 partial sums of |w| (8 KiB of workspace)

template <typename T>
__global__ __launch_bounds__(256) void abs_sum_kernel(const T* __restrict__ w, int64_t numel, double* __restrict__ partial) {
    __shared__ double red[4];
    double s = 0.0;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < numel; i += (int64_t)gridDim.x * 256)
        s += (double)fabsf(mmf_to_float(w[i]));
    s = mmf_block_sum<4>(s, red);
    if (threadIdx.x == 0) partial[blockIdx.x] = s;
}

// scale = T(1 / max(T(mean|w|), T(1e-5))) with every step rounded to the weight dtype.
template <typename T>
__device__ __forceinline__ float weight_scale(const double* __restrict__ partial, int nparts, int64_t numel) {
    double s = 0.0;
    for (int i = 0; i < nparts; ++i) s += partial[i];
    float mean = mmf_round_to<T>((float)(s / (double)numel));
    mean = fmaxf(mean, mmf_round_to<T>(1e-5f));
    return mmf_round_to<T>(__fdiv_rn(1.0f, mean));
}

template <typename T>
__device__ __forceinline__ uint32_t code_of(T w, float scale) {
    float p = mmf_round_to<T>(__fmul_rn(mmf_to_float(w), scale));
    float t = fminf(fmaxf(rintf(p), -1.0f), 1.0f);
    return (uint32_t)((int)t + 1);
}

// One thread builds one lane's 4 dwords (64 codes) of one block.
template <typename T>
__global__ __launch_bounds__(256) void pack_kernel(const T* __restrict__ w, int64_t N, int64_t K, int64_t KB,
                                                   int64_t total_lanes, const double* __restrict__ partial,
                                                   int nparts, uint4* __restrict__ packed, float* __restrict__ wdeq) {
    __shared__ float scale_s;
    if (threadIdx.x == 0) scale_s = weight_scale<T>(partial, nparts, N * K);
    __syncthreads();
    const float scale = scale_s;
    if (blockIdx.x == 0 && threadIdx.x == 0) *wdeq = mmf_round_to<T>(__fdiv_rn(1.0f, scale));

    const int64_t gid = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (gid >= total_lanes) return;
    const int lane = (int)(gid & 63);
    const int64_t blk = gid >> 6;
    const int64_t nb = blk / KB, kb = blk % KB;
    const int64_t n = nb * 32 + (lane & 31);
    const int half = lane >> 5;
    uint32_t d[4];
#pragma unroll
    for (int s = 0; s < 4; ++s) {
        const int64_t k0 = kb * 128 + s * 32 + half * 16;
        uint32_t v = 0;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            uint32_t c = 1u;   // padding = ternary 0
            if (n < N && k0 + i < K) c = code_of<T>(w[n * K + k0 + i], scale);
            v |= c << (8 * (i & 3) + 2 * (i >> 2));
        }
        d[s] = v;
    }
    packed[gid] = make_uint4(d[0], d[1], d[2], d[3]);
}

// packed -> int8 codes [N, K] row-major; one thread per (n, group of 16 inputs).
__global__ __launch_bounds__(256) void unpack_kernel(const uint32_t* __restrict__ packed, int64_t N, int64_t K,
                                                     int64_t KB, int8_t* __restrict__ codes) {
    const int64_t groups = mmf_ceil_div(K, 16);
    const int64_t gid = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (gid >= N * groups) return;
    const int64_t n = gid / groups, kg = gid % groups;
    const int64_t k0 = kg * 16;
    const int64_t nb = n >> 5, kb = k0 >> 7;
    const int s = (int)((k0 >> 5) & 3), half = (int)((k0 >> 4) & 1);
    const int lane = half * 32 + (int)(n & 31);
    const uint32_t v = packed[((nb * KB + kb) * 64 + lane) * 4 + s];
#pragma unroll
    for (int i = 0; i < 16; ++i)
        if (k0 + i < K) codes[n * K + k0 + i] = (int8_t)((int)((v >> (8 * (i & 3) + 2 * (i >> 2))) & 3u) - 1);
}

template <typename T>
int launch_pack(const void* w, int64_t N, int64_t K, void* packed, float* wdeq, void* workspace, hipStream_t s) {
    const int64_t numel = N * K;
    const int64_t KB = mmf_ceil_div(K, 128), NB = mmf_ceil_div(N, 32);
    int nparts = (int)(mmf_ceil_div(numel, 256 * 16) < kPartials ? mmf_ceil_div(numel, 256 * 16) : kPartials);
    if (nparts < 1) nparts = 1;
    double* partial = static_cast<double*>(workspace);
    abs_sum_kernel<T><<<nparts, 256, 0, s>>>(static_cast<const T*>(w), numel, partial);
    MMF_CHECK_LAUNCH();
    const int64_t lanes = NB * KB * 64;
    pack_kernel<T><<<(unsigned)mmf_ceil_div(lanes, 256), 256, 0, s>>>(static_cast<const T*>(w), N, K, KB, lanes, partial,
                                                                    nparts, static_cast<uint4*>(packed), wdeq);
    MMF_CHECK_LAUNCH();
    return 0;
}

// Scratch of mmf_ternarize_pack_noalloc: the partial sums live in the library's own device memory (one copy per GPU,
// held until the process ends) instead of a caller-provided workspace.
static __device__ __align__(256) double scratch[kPartials];

constexpr int kMaxDevices = 64;
double* scratch_ptr[kMaxDevices];          // device address of `scratch` on each GPU, looked up on first use

// The address of this GPU's copy of `scratch` (the array's name is only a host-side handle: kernels must be given
// the address hipGetSymbolAddress returns for the current device).
int scratch_of_current_device(double** out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= kMaxDevices) return MMF_ERR_ARG;
    double* p = __atomic_load_n(&scratch_ptr[dev], __ATOMIC_ACQUIRE);
    if (!p) {
        void* sym = nullptr;
        e = hipGetSymbolAddress(&sym, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return (int)e;
        if (!sym) return MMF_ERR_ARG;
        p = static_cast<double*>(sym);
        __atomic_store_n(&scratch_ptr[dev], p, __ATOMIC_RELEASE);   // every thread would store the same address
    }
    *out = p;
    return 0;
}

}  // namespace

extern "C" {

int64_t mmf_packed_bytes(int64_t N, int64_t K) { return mmf_ceil_div(N, 32) * mmf_ceil_div(K, 128) * 1024; }

int64_t mmf_ternarize_workspace_bytes(void) { return (int64_t)kPartials * sizeof(double); }

int mmf_ternarize_pack(const void* w, int w_dtype, int64_t N, int64_t K, void* packed, float* wdeq, void* workspace,
                       void* stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (N <= 0 || K <= 0 || !w || !packed || !wdeq || !workspace) return MMF_ERR_ARG;
    if ((reinterpret_cast<uintptr_t>(packed) & 15u) || (reinterpret_cast<uintptr_t>(workspace) & 7u)) return MMF_ERR_ALIGN;
    switch (w_dtype) {
        case MMF_F32: return launch_pack<float>(w, N, K, packed, wdeq, workspace, stream);
        case MMF_BF16: return launch_pack<bf16_t>(w, N, K, packed, wdeq, workspace, stream);
        case MMF_F16: return launch_pack<f16_t>(w, N, K, packed, wdeq, workspace, stream);
    }
    return MMF_ERR_ARG;
}

int64_t mmf_ternarize_pack_noalloc_max_elements(void) { return (int64_t)1 << 31; }

int mmf_ternarize_pack_noalloc(const void* w, int w_dtype, int64_t N, int64_t K, void* packed, float* wdeq, void* stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (N <= 0 || K <= 0 || !w || !packed || !wdeq) return MMF_ERR_ARG;
    if (N > mmf_ternarize_pack_noalloc_max_elements() / K) return MMF_ERR_WIDE;   // more than 2^31 weights
    if (reinterpret_cast<uintptr_t>(packed) & 15u) return MMF_ERR_ALIGN;
    double* ws = nullptr;
    if (const int rc = scratch_of_current_device(&ws)) return rc;
    switch (w_dtype) {
        case MMF_F32: return launch_pack<float>(w, N, K, packed, wdeq, ws, stream);
        case MMF_BF16: return launch_pack<bf16_t>(w, N, K, packed, wdeq, ws, stream);
        case MMF_F16: return launch_pack<f16_t>(w, N, K, packed, wdeq, ws, stream);
    }
    return MMF_ERR_ARG;
}

int mmf_unpack_ternary(const void* packed, int64_t N, int64_t K, int8_t* codes, void* stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (N <= 0 || K <= 0 || !packed || !codes) return MMF_ERR_ARG;
    const int64_t KB = mmf_ceil_div(K, 128);
    const int64_t work = N * mmf_ceil_div(K, 16);
    unpack_kernel<<<(unsigned)mmf_ceil_div(work, 256), 256, 0, stream>>>(static_cast<const uint32_t*>(packed), N, K, KB,
                                                                        codes);
    MMF_CHECK_LAUNCH();
    return 0;
}

}  // extern "C"
