// Per-row cross entropy of next-token logits (forward only): what HGRNBitForCausalLM.forward computes when it is
// given labels (mmfreelm/models/hgrn_bit/modeling_hgrn_bit.py:388-397: FusedCrossEntropyLoss or nn.CrossEntropyLoss over
// logits.view(-1, V) and the labels shifted by one; the forward of mmfreelm/modules/fused_cross_entropy.py without
// label smoothing or z-loss, which that call site leaves at their zero defaults).
//   loss[r] = log(sum_j exp(l[r,j] - max_j l[r,j])) + (max_j l[r,j] - l[r, label[r]]),   0 where label[r] == ignore_index
// in fp32 whatever the logits' dtype.  The mean over the rows that count is left to the caller (two tiny reductions).
// One workgroup of 512 threads per row walks it in steps of 8192 elements (two raw 16-byte loads per thread in
// flight) with the online max / sum update, so a thread needs few registers and four workgroups share a CU: one
// workgroup's exp arithmetic runs under the others' loads (measured: 5.3 TB/s against 3.1 TB/s with a whole
// 32000-wide row held in registers).
// Floating point with hardware exp / log: compared with the reference formulation to a tolerance, not bit for bit.
#include "mmf_common.h"

namespace {

template <typename T>
__global__ __launch_bounds__(512) void cross_entropy_kernel(const T* __restrict__ logits, int64_t ld, int64_t V,
                                                            const int64_t* __restrict__ labels, int64_t ignore_index,
                                                            float* __restrict__ loss) {
    constexpr int PASSES = 2;
    __shared__ float red_m[8], red_s[8];
    const int64_t r = blockIdx.x;
    const int64_t label = labels[r];
    if (label == ignore_index || label < 0 || label >= V) {       // a label outside the vocabulary counts as ignored
        if (threadIdx.x == 0) loss[r] = 0.0f;
        return;
    }
    const T* row = logits + r * ld;
    const bool vec_ok = (V % 8) == 0 && (ld % 8) == 0 && (reinterpret_cast<uintptr_t>(logits) & 15u) == 0;
    const float picked = mmf_to_float(row[label]);
    float mx = -INFINITY, sum = 0.0f;                              // running max and sum of exp(l - mx)
    for (int64_t base = (int64_t)threadIdx.x * 8; base < V; base += (int64_t)PASSES * 512 * 8) {
        Raw8<T> raw[PASSES];
#pragma unroll
        for (int p = 0; p < PASSES; ++p) raw[p] = mmf_load8_raw<T>(row, base + (int64_t)p * 512 * 8, V, vec_ok);
        float v[PASSES][8];
        float cm = mx;
#pragma unroll
        for (int p = 0; p < PASSES; ++p) {
            const int64_t c0 = base + (int64_t)p * 512 * 8;
            mmf_unpack8<T>(raw[p], v[p]);
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                if (c0 + i >= V) v[p][i] = -INFINITY;
                cm = fmaxf(cm, v[p][i]);
            }
        }
        if (cm > mx) {                                            // rescale what has been summed so far
            sum = mx == -INFINITY ? 0.0f : sum * __expf(mx - cm);
            mx = cm;
        }
        if (mx != -INFINITY) {
#pragma unroll
            for (int p = 0; p < PASSES; ++p)
#pragma unroll
                for (int i = 0; i < 8; ++i) sum += __expf(v[p][i] - mx);   // exp(-inf) = 0 for the padding
        }
    }
    // combine (max, sum) pairs: lanes, then waves
    for (int o = 32; o > 0; o >>= 1) {
        const float om = __shfl_xor(mx, o, 64), os = __shfl_xor(sum, o, 64);
        const float nm = fmaxf(mx, om);
        if (nm != -INFINITY) sum = (mx == -INFINITY ? 0.0f : sum * __expf(mx - nm)) + (om == -INFINITY ? 0.0f : os * __expf(om - nm));
        mx = nm;
    }
    const int w = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) { red_m[w] = mx; red_s[w] = sum; }
    __syncthreads();
    if (threadIdx.x == 0) {
        float m = red_m[0], s = red_s[0];
        for (int i = 1; i < 8; ++i) {
            const float om = red_m[i], os = red_s[i];
            const float nm = fmaxf(m, om);
            if (nm != -INFINITY) s = (m == -INFINITY ? 0.0f : s * __expf(m - nm)) + (om == -INFINITY ? 0.0f : os * __expf(om - nm));
            m = nm;
        }
        loss[r] = __logf(s) + (m - picked);       // m - picked first: both can be huge and nearly equal
    }
}

}  // namespace

extern "C" {

int mmf_cross_entropy_fwd(const void* logits, int64_t ld, const int64_t* labels, int64_t ignore_index, float* loss,
                          int64_t rows, int64_t V, int dtype, void* stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (rows < 0 || V <= 0 || ld < V || rows > 0x7fffffff) return MMF_ERR_ARG;
    if (rows == 0) return 0;
    if (!logits || !labels || !loss) return MMF_ERR_ARG;
    switch (dtype) {
        case MMF_F32: cross_entropy_kernel<float><<<(unsigned)rows, 512, 0, stream>>>(static_cast<const float*>(logits), ld, V, labels, ignore_index, loss); break;
        case MMF_BF16: cross_entropy_kernel<bf16_t><<<(unsigned)rows, 512, 0, stream>>>(static_cast<const bf16_t*>(logits), ld, V, labels, ignore_index, loss); break;
        case MMF_F16: cross_entropy_kernel<f16_t><<<(unsigned)rows, 512, 0, stream>>>(static_cast<const f16_t*>(logits), ld, V, labels, ignore_index, loss); break;
        default: return MMF_ERR_ARG;
    }
    MMF_CHECK_LAUNCH();
    return 0;
}

}  // extern "C"
