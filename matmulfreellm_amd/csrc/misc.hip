// Embedding row gather and greedy argmax: the two ends of a decode step, kept as plain
// kernels so the whole step can be captured into one HIP graph without library calls.
//
// mmf_embedding replaces nn.Embedding.forward at mmfreelm/models/hgrn_bit/modeling_hgrn_bit.py:212;
// mmf_argmax replaces the argmax over the vocabulary that greedy decoding performs on the
// logits of HGRNBitForCausalLM.forward (modeling_hgrn_bit.py:386).  Ties go to the lowest
// index (BitLinear logits are integer accumulators times two scalars, so exact ties happen).
#include "mmf_common.h"

namespace {

template <typename T>
__global__ __launch_bounds__(256) void embedding_kernel(const T* __restrict__ table, const int64_t* __restrict__ ids,
                                                        T* __restrict__ out, int64_t rows, int64_t H, int64_t vocab) {
    const int64_t r = blockIdx.x;
    int64_t id = ids[r];
    if (id < 0 || id >= vocab) id = 0;   // out-of-range ids read row 0 instead of faulting
    const T* src = table + id * H;
    T* dst = out + r * H;
    constexpr int PER = 16 / (int)sizeof(T);
    if (H % PER == 0 && ((reinterpret_cast<uintptr_t>(table) | reinterpret_cast<uintptr_t>(out)) & 15u) == 0) {
        // 16 bytes per thread: a 2048-wide 16-bit row is one load and one store per thread
        const uint4* s4 = reinterpret_cast<const uint4*>(src);
        uint4* d4 = reinterpret_cast<uint4*>(dst);
        for (int64_t c = threadIdx.x; c < H / PER; c += 256) d4[c] = s4[c];
    } else {
        for (int64_t c = threadIdx.x; c < H; c += 256) dst[c] = src[c];
    }
}

// One workgroup of 512 threads per row; 8 elements (16 B for 16-bit types) per thread per pass.  The loads of 8 passes
// (32768 elements, a whole 32000-wide row) are issued raw before the first compare, so the row costs one memory round
// trip instead of one per pass.  Lowest index wins ties; NaNs never win.
template <typename T>
__global__ __launch_bounds__(512) void argmax_kernel(const T* __restrict__ logits, int64_t ld, int64_t V,
                                                     int64_t* __restrict__ out) {
    constexpr int PASSES = 8;
    __shared__ float best_v[8];
    __shared__ int64_t best_i[8];
    const int64_t r = blockIdx.x;
    const T* row = logits + r * ld;
    const bool vec_ok = (V % 8) == 0 && (ld % 8) == 0 && (reinterpret_cast<uintptr_t>(logits) & 15u) == 0;
    float bv = -INFINITY;
    int64_t bi = V;   // larger than any valid index: "nothing yet"
    for (int64_t base = (int64_t)threadIdx.x * 8; base < V; base += (int64_t)PASSES * 512 * 8) {
        Raw8<T> raw[PASSES];
#pragma unroll
        for (int p = 0; p < PASSES; ++p) raw[p] = mmf_load8_raw<T>(row, base + (int64_t)p * 512 * 8, V, vec_ok);
#pragma unroll
        for (int p = 0; p < PASSES; ++p) {
            const int64_t c0 = base + (int64_t)p * 512 * 8;
            float v[8];
            mmf_unpack8<T>(raw[p], v);
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int64_t c = c0 + i;
                if (c < V && (v[i] > bv || (bi == V && v[i] == v[i]))) { bv = v[i]; bi = c; }   // ascending c: first max kept
            }
        }
    }
    for (int o = 32; o > 0; o >>= 1) {
        const float ov = __shfl_xor(bv, o, 64);
        const int64_t oi = __shfl_xor(bi, o, 64);
        if (oi < V && (bi == V || ov > bv || (ov == bv && oi < bi))) { bv = ov; bi = oi; }
    }
    const int w = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) { best_v[w] = bv; best_i[w] = bi; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int i = 1; i < 8; ++i)
            if (best_i[i] < V && (bi == V || best_v[i] > bv || (best_v[i] == bv && best_i[i] < bi))) { bv = best_v[i]; bi = best_i[i]; }
        out[r] = bi < V ? bi : 0;
    }
}


// Every float through the kernels' short forms of exp, the sigmoid, the reciprocal, the square root and 127 / a,
// against the sequences that define them.  counts[0..4]: arguments on which mmf_exp / mmf_sigmoid / mmf_rcp_pos /
// mmf_sqrt_pos / mmf_127_over differ from mmf_exp_definition / mmf_sigmoid_definition / __fdiv_rn(1, x) / sqrtf(x) /
// __fdiv_rn(127, x) (two NaNs count as equal); counts[5]: arguments seen; counts[6]: arguments that pass
// mmf_sigmoid_mid_ok and on which mmf_sigmoid_mid differs from the definition.  A grid-stride walk over all 2^32 bit patterns.
__global__ __launch_bounds__(256) void exact_forms_kernel(unsigned long long* counts) {
    unsigned long long bad[5] = {0, 0, 0, 0, 0}, seen = 0, bad_mid = 0;
    auto same = [](float a, float b) { return (a != a && b != b) || __float_as_uint(a) == __float_as_uint(b); };
    const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < (1ull << 32); i += stride) {
        const float x = __uint_as_float((uint32_t)i);
        ++seen;
        if (!same(mmf_exp(x), mmf_exp_definition(x))) ++bad[0];
        if (!same(mmf_sigmoid(x), mmf_sigmoid_definition(x))) ++bad[1];
        if (!same(mmf_rcp_pos(x), __fdiv_rn(1.0f, x))) ++bad[2];
        if (!same(mmf_sqrt_pos(x), sqrtf(x))) ++bad[3];
        if (!same(mmf_127_over(x), __fdiv_rn(127.0f, x))) ++bad[4];
        if (mmf_sigmoid_mid_ok(x) && !same(mmf_sigmoid_mid(x), mmf_sigmoid_definition(x))) ++bad_mid;
    }
#pragma unroll
    for (int j = 0; j < 5; ++j)
        if (bad[j]) atomicAdd(&counts[j], bad[j]);
    atomicAdd(&counts[5], seen);
    if (bad_mid) atomicAdd(&counts[6], bad_mid);
}

}  // namespace

extern "C" {

int mmf_embedding(const void* table, const int64_t* ids, void* out, int64_t rows, int64_t H, int64_t vocab, int dtype,
                  void* stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (rows < 0 || H <= 0 || vocab <= 0) return MMF_ERR_ARG;
    if (rows == 0) return 0;
    if (!table || !ids || !out) return MMF_ERR_ARG;
    switch (dtype) {
        case MMF_F32: embedding_kernel<float><<<(unsigned)rows, 256, 0, stream>>>(static_cast<const float*>(table), ids, static_cast<float*>(out), rows, H, vocab); break;
        case MMF_BF16: embedding_kernel<bf16_t><<<(unsigned)rows, 256, 0, stream>>>(static_cast<const bf16_t*>(table), ids, static_cast<bf16_t*>(out), rows, H, vocab); break;
        case MMF_F16: embedding_kernel<f16_t><<<(unsigned)rows, 256, 0, stream>>>(static_cast<const f16_t*>(table), ids, static_cast<f16_t*>(out), rows, H, vocab); break;
        default: return MMF_ERR_ARG;
    }
    MMF_CHECK_LAUNCH();
    return 0;
}

int mmf_argmax(const void* logits, int64_t ld, int64_t rows, int64_t V, int64_t* out, int dtype, void* stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (rows < 0 || V <= 0 || ld < V) return MMF_ERR_ARG;
    if (rows == 0) return 0;
    if (!logits || !out) return MMF_ERR_ARG;
    switch (dtype) {
        case MMF_F32: argmax_kernel<float><<<(unsigned)rows, 512, 0, stream>>>(static_cast<const float*>(logits), ld, V, out); break;
        case MMF_BF16: argmax_kernel<bf16_t><<<(unsigned)rows, 512, 0, stream>>>(static_cast<const bf16_t*>(logits), ld, V, out); break;
        case MMF_F16: argmax_kernel<f16_t><<<(unsigned)rows, 512, 0, stream>>>(static_cast<const f16_t*>(logits), ld, V, out); break;
        default: return MMF_ERR_ARG;
    }
    MMF_CHECK_LAUNCH();
    return 0;
}

int mmf_diag_check_exact_forms(unsigned long long* counts, void* stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (!counts) return MMF_ERR_ARG;
    exact_forms_kernel<<<4096, 256, 0, stream>>>(counts);
    MMF_CHECK_LAUNCH();
    return 0;
}

}  // extern "C"
