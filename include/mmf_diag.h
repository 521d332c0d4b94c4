/* libmmf_hip -- measuring aids (no counterpart in the reference; only bench.py binds them).
 *
 * They are exported by the same library as the product entry points of mmf.h but are not part of the drop-in boundary:
 * nothing on a product path calls them.
 */
#ifndef MMF_DIAG_H_
#define MMF_DIAG_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Tiled matrix-core contraction (bench.py's mfma leg).
 * mmf_bitlinear_mfma_clock_sink: sink = [workgroups][2] int64 on the device, or NULL to switch off.  While set, thread 0
 *   of each of the first `workgroups` workgroups of every later tiled launch (mmf_bitlinear_mfma with M > 64,
 *   mmf_bitlinear_mfma_swiglu) stores the shader-clock ticks (s_memtime) and the 100 MHz ticks (s_memrealtime) it
 *   spent in the kernel: their ratio is the clock the part sustained under that kernel.  Process-wide, not
 *   thread-safe; the buffer must outlive the launches.
 * mmf_mfma_pipe_probe: `workgroups` x 8 waves each issue steps x 4 independent v_mfma_i32_32x32x32_i8 on register
 *   operands (the tiled kernel's inner step with every load, barrier and LDS read taken away) and store the same two
 *   tick counts; clocks = [workgroups][2] int64 plus one spare int64.  random_operands != 0: per-lane random int8 codes
 *   and ternary weights (the switching activity, hence the power draw, of real operands) instead of constant ones. */
int mmf_bitlinear_mfma_clock_sink(int64_t* sink, int64_t workgroups);
int mmf_mfma_pipe_probe(int64_t steps, int64_t workgroups, int random_operands, int64_t* clocks, void* stream);

/* mmf_decode_layers_traced: mmf_decode_layers (see mmf.h) built with its cycle trace, and with the hold-back of a link's
 *   first poll as an argument (`delay`, in units of about 64 cycles, 0..64).
 *   trace: mmf_decode_layers_trace_words() int64 words (zeroed by the caller): thread 0 of every workgroup stores the
 *   shader clock at points of each of the first 128 links, [256 workgroups][link][12]: 0 link entered, 1 input row arrived,
 *   2 block norm applied, 3 second sum of squares reduced, 4 absmax reduced, 5 codes in LDS, 6 dot products done,
 *   7 partial sums met, 8 epilogue stored.  The product launch carries none of this. */
int mmf_decode_layers_trace_words(void);
int mmf_decode_layers_traced(const void* phases, int n_layers, const void* table, const int64_t* tok, int64_t vocab, uint32_t* words,
                             void* h_out, const void* head, void* logits, uint64_t* am_words, int64_t* tok_out, uint32_t* epoch, int* err,
                             int64_t* trace, int H, int D, int I, int spin, int delay, int dtype, void* stream);

/* mmf_diag_check_exact_forms: the kernels evaluate exp with one ldexp instead of two scaling multiplications, and the
 *   reciprocal, the square root and 127 / a (the norm's rstd, the sigmoid's 1 / (1 + e), the quantiser's scale) with the
 *   hardware approximations plus Newton steps instead of the general correctly rounded sequences, which they fall back
 *   to outside a middle range of exponents.  This runs ALL 2^32 floats through both forms on the device: counts = 7
 *   zeroed uint64 on the device; [0..4] arguments where exp / sigmoid / 1 / x / sqrt(x) / 127 / x differ from the
 *   defining sequence, [5] arguments seen (2^32), [6] arguments x >= -69 where the branch-free sigmoid that kernels run
 *   on whole vectors of such arguments differs.  All but [5] must be 0 (tests/test_gpu_ops.py). */
int mmf_diag_check_exact_forms(unsigned long long* counts, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MMF_DIAG_H_ */
