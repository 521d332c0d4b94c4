/* libmmf_hip -- C ABI of the MI355X (gfx950) kernels for the MatMul-free LM hot path.
 *
 * The reference (ridgerchu/matmulfreellm, package `mmfreelm`) has no FFI: the path sits
 * behind Python callables (torch.autograd.Function wrappers around Triton kernels).  Each
 * entry point below names the reference callable it replaces; a Python host binds them
 * with ctypes and passes tensor.data_ptr() values.
 *
 * Conventions
 *   - every function returns 0 on success, a negative MMF_ERR_* code for a rejected
 *     argument, or a positive hipError_t from the launch; nothing throws;
 *   - all pointers are DEVICE pointers owned by the caller; no entry point allocates,
 *     frees, synchronises or keeps a pointer after it returns; work is enqueued on
 *     `stream` (a hipStream_t passed as void*; NULL = the default stream);
 *   - `dtype` arguments: 0 = fp32, 1 = bf16, 2 = fp16 (MMF_F32 / MMF_BF16 / MMF_F16);
 *   - matrices are row-major and contiguous unless a leading dimension is given;
 *   - 16-byte alignment is required of every matrix base pointer whose row length is a
 *     multiple of 8 elements (torch allocations always are), of packed weights and codes.
 *
 * Arithmetic (identical on every call, independent of launch shape): fp32 math with one
 * rounding per operation (no fused multiply-add), sums of squares in fp64, correctly
 * rounded divide/sqrt, round-half-to-even for integer codes, and a fixed polynomial exp.
 */
#ifndef MMF_H_
#define MMF_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MMF_F32 0
#define MMF_BF16 1
#define MMF_F16 2

#ifndef MMF_ERR_ARG
#define MMF_ERR_ARG (-1)   /* bad shape, null pointer, unsupported dtype combination */
#define MMF_ERR_WIDE (-2)  /* row wider than the fused kernels hold in registers / LDS */
#define MMF_ERR_ALIGN (-3) /* pointer not 16-byte aligned where required */
#endif

/* ---- weights: absmean ternarisation + 2-bit packing --------------------------------
 * Replaces weight_quant(), mmfreelm/ops/fusedbitnet.py:32-46, which the reference re-runs
 * on the latent matrix in every forward (fusedbitnet.py:456).
 *
 * w [N, K] latent weights (dtype w_dtype, nn.Linear layout).  Writes
 *   packed : mmf_packed_bytes(N, K) bytes, blocks of 32 rows x 128 inputs, 2 bits per
 *            weight holding t + 1, padded with t = 0 to multiples of 32 / 128;
 *   wdeq   : 1 float, the de-quantisation step  dtype(1 / dtype(1 / mean|w|)).
 * workspace: mmf_ternarize_workspace_bytes() bytes of scratch (8-byte aligned). */
int64_t mmf_packed_bytes(int64_t N, int64_t K);
int64_t mmf_ternarize_workspace_bytes(void);
int mmf_ternarize_pack(const void* w, int w_dtype, int64_t N, int64_t K, void* packed, float* wdeq,
                       void* workspace, void* stream);
/* mmf_ternarize_pack_noalloc: mmf_ternarize_pack without the workspace argument, for callers that cannot allocate
 * device memory (code under HIP graph capture, tight serving loops that re-pack updated weights, harnesses that
 * forbid hipMalloc).  It has no counterpart in the reference.  The 8 KiB of partial sums live in a file-scope device
 * array of the library (one copy per GPU, held until the process ends; its address is looked up on the first call
 * on each GPU, which should therefore happen outside a graph capture).  Same kernels, same results as
 * mmf_ternarize_pack.  Nothing is allocated, freed or synchronised.  N * K above
 * mmf_ternarize_pack_noalloc_max_elements() (2^31): MMF_ERR_WIDE.  Every call on a GPU uses that GPU's one array:
 * calls that overlap on one GPU (different streams or threads) race; calls on one stream are ordered and safe.
 * Nothing in the array needs clearing between calls: a call writes every partial sum it later reads. */
int64_t mmf_ternarize_pack_noalloc_max_elements(void);
int mmf_ternarize_pack_noalloc(const void* w, int w_dtype, int64_t N, int64_t K, void* packed, float* wdeq, void* stream);
/* packed -> int8 codes [N, K] in {-1, 0, 1} (inspection / tests). */
int mmf_unpack_ternary(const void* packed, int64_t N, int64_t K, int8_t* codes, void* stream);

/* ---- RMSNorm -------------------------------------------------------------------------
 * Replaces rms_norm_fn / LayerNormFn.forward with is_rms_norm=True,
 * mmfreelm/modules/layernorm.py:445-482, kernel :104-165 (module RMSNorm :586-623).
 * y = T((x [+ residual]) * rstd * weight); residual_out (optional) receives the fp32 sum
 * rounded to residual_dtype (= x_dtype or fp32).  weight may be NULL; weight_dtype is
 * fp32 or x_dtype. */
int mmf_rmsnorm(const void* x, const void* residual, const void* weight, void* y, void* residual_out,
                int64_t M, int64_t K, float eps, int x_dtype, int residual_dtype, int weight_dtype,
                void* stream);

/* Replaces the gated variant, mmfreelm/modules/fused_norm_gate.py:420-460, kernel :68-131
 * (module FusedRMSNormSwishGate :514-536):  y = T(norm(x) * gate * sigmoid(gate)).
 * x may be a column slice of a wider matrix (row stride ldx elements); gate, y are [M, K]. */
int mmf_rmsnorm_swishgate(const void* x, int64_t ldx, const void* gate, const void* residual, const void* weight,
                          void* y, void* residual_out, int64_t M, int64_t K, float eps, int x_dtype,
                          int residual_dtype, int weight_dtype, void* stream);

/* Replaces swiglu(), mmfreelm/modules/activations.py:115-119,143-153:
 * out[r, c] = T((x[r,c] * y[r,c]) / (1 + exp(-x[r,c]))); x and y may be column slices of a
 * wider matrix (leading dimensions ldx, ldy in elements), out is [rows, cols] contiguous. */
int mmf_swiglu(const void* x, int64_t ldx, const void* y, int64_t ldy, void* out, int64_t rows,
               int64_t cols, int dtype, void* stream);

/* ---- activations: RMSNorm + per-row absmax int8 codes ---------------------------------
 * Replaces _layer_norm_fwd_quant / its kernel, mmfreelm/ops/fusedbitnet.py:63-190, and
 * activation_quant(), fusedbitnet.py:15-29.  Instead of a de-quantised tensor it emits
 *   q    : int8 codes, zero padded to Kp = ceil128(K) columns; tiled = 0: row-major
 *          [M, Kp]; tiled = 1: [ceil32(M)/32][Kp/16][32 rows][16 bytes] (the matrix-core
 *          operand layout); mmf_codes_bytes(M, K, tiled) bytes;
 *   deq  : [M] fp32, 1 / scale with scale = 127 / max(max|y|, 1e-5);
 *   qsum : [M] int32, sum of the row's codes. */
int64_t mmf_codes_bytes(int64_t M, int64_t K, int tiled);
int mmf_rmsnorm_quant(const void* x, const void* residual, const void* weight, int8_t* q, float* deq,
                      int* qsum, void* residual_out, int64_t M, int64_t K, float eps, int x_dtype,
                      int residual_dtype, int weight_dtype, int tiled, void* stream);
/* mmf_layernorm_quant: the IS_RMS_NORM = False branch of the same reference kernel (fusedbitnet.py:102-121, reached
 * through layer_norm_linear_quant_fn(..., is_rms_norm=False), :513-536): mean = fp32(sum x / K), the variance is that of
 * the fp32 differences x - mean, y = (x - mean) * rstd * weight + bias.  bias: [K] in the weight's dtype, or NULL. */
int mmf_layernorm_quant(const void* x, const void* residual, const void* weight, const void* bias, int8_t* q,
                        float* deq, int* qsum, void* residual_out, int64_t M, int64_t K, float eps, int x_dtype,
                        int residual_dtype, int weight_dtype, int tiled, void* stream);

/* mmf_rmsnorm_quant_fused: the same quantiser (tiled codes) with the elementwise op that precedes a
 * BitLinear in the model folded in, for batches that go to the matrix cores:
 *   0 PLAIN      v = x (what mmf_rmsnorm_quant computes, in the many-rows-per-workgroup form; w1 unused)
 *   1 NORM       v = RMSNorm(x; w1, eps1)                                  modeling_hgrn_bit.py:98
 *   2 RESNORM    s = x + aux; res_out = s; v = RMSNorm(s; w1, eps1)        modeling_hgrn_bit.py:107
 *   3 STEP_GATE  x, aux, aux2 = raw i, f, g projections of ONE token per row: gate math and one recurrence
 *                step on state[M, K] (fp32, in place) as mmf_hgrn_step, then
 *                v = RMSNorm(g; w1, eps1) * o * sigmoid(o)                  layers/hgrn_bit.py:113-139
 *   4 SWIGLU     v = (x * aux) / (1 + exp(-x))                             modeling_hgrn_bit.py:58
 *   5 GATEDNORM  v = RMSNorm(x; w1, eps1) * aux * sigmoid(aux)             layers/hgrn_bit.py:138 (any number of tokens)
 * v is rounded to the activation dtype like the tensor it replaces; then q = codes of RMSNorm(v; norm_weight, eps). */
int mmf_rmsnorm_quant_fused(int prologue, const void* x, int64_t ldx, const void* aux, int64_t ldaux, const void* aux2,
                            int64_t ldaux2, void* res_out, const void* w1, float eps1, const void* norm_weight, float eps,
                            const float* lower_bound, float* state, int8_t* q, float* deq, int* qsum, int64_t M, int64_t K,
                            int x_dtype, int weight_dtype, void* stream);

/* ---- BitLinear contraction ------------------------------------------------------------
 * Both replace F.linear(y, weight_quant(W)) at mmfreelm/ops/fusedbitnet.py:456-458 (class
 * FusedBitLinear :584-610, layer_norm_linear_quant_fn :513-536):
 *   out[m, n] = T( fp32(sum_k q[m,k] * t[n,k]) * deq[m] * wdeq[n / seg_rows] (+ bias[n]) ),
 * and, when `addend` ([M, N], same dtype and leading dimension as out) is given,
 *   out = T(out + addend)  -- the block's residual add (modeling_hgrn_bit.py:109) fused in.
 * `packed` may be several matrices with the same K packed one after the other (each a
 * multiple of 32 rows); wdeq then holds one step per seg_rows output rows.
 *
 * mmf_bitlinear_gemv: decode-sized M; norm + quantiser + contraction in one launch, x is
 *   the un-normalised input [M, K] (K <= mmf_bitlinear_gemv_max_k()).
 * mmf_bitlinear_mfma: int8 matrix-core contraction on codes from mmf_rmsnorm_quant
 *   (tiled = 1); out has leading dimension ldo; config < 0 picks the tile shape from M. */
int64_t mmf_bitlinear_gemv_max_k(void);
/* mmf_bitlinear_gemv_fused: the same launch with the elementwise ops the model runs around a
 * BitLinear folded in (a decode step is latency bound: one launch per BitLinear, none between).
 *   prologue (what the BitLinear sees as input, v, rounded to the activation dtype like the
 *   tensor it replaces):
 *     0 PLAIN      v = x
 *     1 NORM       v = RMSNorm(x; w1, eps1)             block norm, modeling_hgrn_bit.py:98
 *     2 RESNORM    s = x + aux; res_out = s; v = RMSNorm(s; w1, eps1)   fused residual norm, :107
 *     3 GATEDNORM  v = RMSNorm(x; w1, eps1) * aux * sigmoid(aux)        g_norm, layers/hgrn_bit.py:139
 *     4 SWIGLU     v = (x * aux) / (1 + exp(-x))        MLP activation, modeling_hgrn_bit.py:58
 *   epilogue (r = the BitLinear output):
 *     0 PLAIN   out[M, N] = r (+ bias), or T(r + addend)
 *     1 STEP    packed = [i; f; g] stacked (N = 3D): gate math of layers/hgrn_bit.py:113-117 and one
 *               recurrence step on state[M, D] (fp32, in place); out = o [M, D], g_out = raw g [M, D]
 *     2 SWIGLU  packed = [gate; up] rows (N = 2I): out[M, I] = swiglu(gate, up)
 * x / aux are [M, K] with row strides ldx / ldaux; all weights (w1, norm_weight) share weight_dtype. */
int mmf_bitlinear_gemv_fused(int prologue, int epilogue, const void* x, int64_t ldx, const void* aux, int64_t ldaux,
                             void* res_out, const void* w1, float eps1, const void* norm_weight, float eps,
                             const void* packed, const float* wdeq, int64_t seg_rows, const void* bias,
                             const void* addend, void* out, void* g_out, const float* lower_bound, float* state,
                             int64_t M, int64_t K, int64_t N, int x_dtype, int weight_dtype, void* stream);
int mmf_bitlinear_gemv(const void* x, const void* norm_weight, const void* packed, const float* wdeq,
                       int64_t seg_rows, const void* bias, const void* addend, void* out, int64_t M, int64_t K,
                       int64_t N, float eps, int x_dtype, int norm_weight_dtype, void* stream);
int mmf_bitlinear_mfma(const int8_t* codes_tiled, const float* deq, const int* qsum, const void* packed,
                       const float* wdeq, int64_t seg_rows, const void* bias, const void* addend, void* out,
                       int64_t ldo, int64_t M, int64_t K, int64_t N, int out_dtype, int config, void* stream);

/* mmf_bitlinear_mfma_swiglu: the tiled matrix-core contraction on the STACKED [gate; up] weight of the MLP
 *   (N = 2 * I rows, I a multiple of 32: rows [0, I) = gate, [I, 2I) = up, as gate_proj stores them) with the activation
 *   of mmfreelm/models/hgrn_bit/modeling_hgrn_bit.py:55-59 (swiglu, mmfreelm/modules/activations.py:143) in its epilogue:
 *     out[m, c] = T((g * u) / (1 + exp(-g))),  g = T(gate projection [m, c]),  u = T(up projection [m, c]),
 *   i.e. exactly what mmf_bitlinear_mfma followed by mmf_swiglu on the two halves gives, without the [M, 2I] round trip.
 *   out: [M, I] with leading dimension ldo (16-byte aligned rows: else MMF_ERR_ALIGN).  Other arguments as above. */
int mmf_bitlinear_mfma_swiglu(const int8_t* codes_tiled, const float* deq, const int* qsum, const void* packed,
                              const float* wdeq, int64_t seg_rows, void* out, int64_t ldo, int64_t M, int64_t K, int64_t N,
                              int out_dtype, void* stream);

/* ---- HGRN recurrence ------------------------------------------------------------------
 * x, g, o: [BH, T, D] contiguous (BH = batch * heads); h0 / ht: [BH, D] fp32 or NULL.
 * mmf_hgrn_recurrent replaces fused_recurrent_hgrn, mmfreelm/ops/hgrn/recurrent_fuse.py:
 *   176-185 (kernel :32-68): h = g*h + x with g the decay itself.
 * mmf_hgrn_chunk replaces chunk_hgrn, mmfreelm/ops/hgrn/chunk.py:287-296 (kernels :49-116):
 *   h = exp(g)*h + x with g the log decay, evaluated as the reference's chunked form: per chunk of `chunk` steps
 *   (1 <= chunk <= 64; the reference fixes 128) a scan from zero (the first chunk from h0) with the running sum gc of
 *   the log gates, then o_t += exp(gc_t) * (last output of the chunk before).  One pass over x and g with the chunk in
 *   registers (no fp32 [B,H,T,D] scratch tensors).  When BH * ceil(D / 64) < 256 the time axis is also cut into
 *   segments that run in parallel (a first launch leaves each segment's (decay product, end state from zero) pair in
 *   `workspace`, mmf_hgrn_chunk_workspace_bytes(BH, T, D, chunk) bytes, 4-byte aligned, may be NULL when that is 0).
 *   exp is the hardware one: results agree with the reference's within rounding, not bit for bit.
 * The final state is fp32 in both (the reference rounds the recurrent one to x's dtype).
 * MMF_ERR_WIDE when 64 rows of D elements reach 2 GiB. */
int mmf_hgrn_recurrent(const void* x, const void* g, const float* h0, void* o, float* ht, int64_t BH,
                       int64_t T, int64_t D, int dtype, void* stream);
int64_t mmf_hgrn_chunk_workspace_bytes(int64_t BH, int64_t T, int64_t D, int chunk);
int mmf_hgrn_chunk(const void* x, const void* g, const float* h0, void* o, float* ht, int64_t BH,
                   int64_t T, int64_t D, int chunk, int dtype, void* workspace, void* stream);

/* Gate math of HGRNBitAttention.forward, mmfreelm/layers/hgrn_bit.py:113-120, fused:
 *   g_out = T(lb + (1 - lb) * sigmoid(f))  (lower_bound NULL: T(sigmoid(f)))
 *   x_out = T((i * (1 - g_out)) / (1 + exp(-i))), 0 where mask[row] == 0.
 * i_in / f_in: [rows, D] with leading dimensions ldi / ldf; lower_bound [D] fp32 or NULL;
 * mask [rows] bytes or NULL.  mmf_hgrn_step fuses the same math with one recurrence step
 * (T = 1 decode): state [rows, D] fp32 is updated in place, o = T(state). */
int mmf_hgrn_gate(const void* i_in, int64_t ldi, const void* f_in, int64_t ldf, const float* lower_bound,
                  const uint8_t* mask, void* x_out, void* g_out, int64_t rows, int64_t D, int dtype,
                  void* stream);
int mmf_hgrn_step(const void* i_in, int64_t ldi, const void* f_in, int64_t ldf, const float* lower_bound,
                  const uint8_t* mask, float* state, void* o, int64_t rows, int64_t D, int dtype,
                  void* stream);

/* ---- the two ends of a decode step ------------------------------------------------------
 * mmf_embedding replaces nn.Embedding.forward at mmfreelm/models/hgrn_bit/modeling_hgrn_bit.py:212:
 *   out[r, :] = table[ids[r], :]  (ids int64; an id outside [0, vocab) reads row 0).
 * mmf_argmax is the greedy choice over the logits of HGRNBitForCausalLM.forward
 *   (modeling_hgrn_bit.py:386): out[r] = lowest index of the row maximum (int64). */
int mmf_embedding(const void* table, const int64_t* ids, void* out, int64_t rows, int64_t H, int64_t vocab,
                  int dtype, void* stream);
int mmf_argmax(const void* logits, int64_t ld, int64_t rows, int64_t V, int64_t* out, int dtype, void* stream);

/* ---- next-token loss (forward only) -----------------------------------------------------------
 * mmf_cross_entropy_fwd replaces the loss that HGRNBitForCausalLM.forward computes from labels
 *   (mmfreelm/models/hgrn_bit/modeling_hgrn_bit.py:388-397: FusedCrossEntropyLoss / nn.CrossEntropyLoss on
 *   logits.view(-1, V); forward of mmfreelm/modules/fused_cross_entropy.py with its default zero smoothing and z-loss):
 *   loss[r] = logsumexp(logits[r, :]) - logits[r, labels[r]] in fp32, 0 where labels[r] == ignore_index (or lies
 *   outside [0, V)).  The caller shifts the labels and takes the mean over the rows that count.  No backward. */
int mmf_cross_entropy_fwd(const void* logits, int64_t ld, const int64_t* labels, int64_t ignore_index, float* loss,
                          int64_t rows, int64_t V, int dtype, void* stream);

/* ---- training side: backward kernels and the fused loss ------------------------------------------
 * Gradients are fp32 arithmetic (hardware exp / log), compared with autograd through the reference formulation to a
 * tolerance.  Sums over rows (norm weight, lower bound) are accumulated per workgroup, written as [groups, K] fp32
 * partials (groups = mmf_backward_groups(rows); the caller provides the buffer) and added in a fixed order.
 *
 * mmf_rmsnorm_bwd replaces the Triton backward kernels of the three norms:
 *   mode 0  RMSNorm                    mmfreelm/modules/layernorm.py:245-330 (LayerNormFn.backward :484-531)
 *   mode 1  RMSNorm * swish gate       mmfreelm/modules/fused_norm_gate.py:210-300 (:462-500); also returns dgate
 *   mode 2  BitLinear's norm           mmfreelm/ops/fusedbitnet.py:209-317 (LayerNormLinearQuantFn.backward :470-510): the
 *           gradient passes through the activation quantiser unchanged (straight-through, :571) and y_quant receives the
 *           de-quantised int8 output recomputed with the forward arithmetic, for the weight gradient dout^T y (:498)
 *   x [M, K] (row stride ldx) is what the norm normalised (the summed residual where the forward added one); rstd is
 *   recomputed from it.  dx = (w dy - xhat mean(xhat w dy)) rstd (+ dresidual, the gradient arriving through a prenorm
 *   residual output); dweight [K] (weight dtype) = sum over rows of dy xhat, needs dw_partial [groups, K] fp32. */
int mmf_backward_groups(int64_t rows);
int mmf_rmsnorm_bwd(int mode, const void* x, int64_t ldx, const void* gate, int64_t ldg, const void* weight, const void* dy,
                    int64_t lddy, const void* dresidual, void* dx, void* dgate, void* y_quant, float* dw_partial, void* dweight,
                    int64_t M, int64_t K, float eps, int x_dtype, int weight_dtype, void* stream);
/* mmf_swiglu_bwd replaces swiglu_bwd, mmfreelm/modules/activations.py:121-126: with s = sigmoid(x),
 *   dx = s (1 + x (1 - s)) g y,  dy = x s g; every operand may be a column slice (leading dimensions in elements). */
int mmf_swiglu_bwd(const void* x, int64_t ldx, const void* y, int64_t ldy, const void* g, int64_t ldg, void* dx, int64_t lddx,
                   void* dy, int64_t lddy, int64_t rows, int64_t cols, int dtype, void* stream);
/* mmf_hgrn_gate_bwd: gradient of the gate math mmf_hgrn_gate fuses (what autograd derives for
 *   mmfreelm/layers/hgrn_bit.py:113-120): from grad_x, grad_g [rows, D] to di, df (leading dimensions lddi, lddf) and, with a
 *   lower bound, dlb [D] fp32 = sum over rows of (grad_g - grad_x i sigmoid(i)) (1 - sigmoid(f)) (dlb_partial: [groups, D]). */
int mmf_hgrn_gate_bwd(const void* i_in, int64_t ldi, const void* f_in, int64_t ldf, const float* lower_bound, const uint8_t* mask,
                      const void* grad_x, const void* grad_g, void* di, int64_t lddi, void* df, int64_t lddf, float* dlb_partial,
                      float* dlb, int64_t rows, int64_t D, int dtype, void* stream);
/* mmf_hgrn_recurrent_bwd replaces fused_recurrent_hgrn_bwd_kernel, mmfreelm/ops/hgrn/recurrent_fuse.py:89-133 (backward
 *   :158-173): time runs backwards, dh += do_t; dx_t = dh; dg_t = dh h_{t-1}; dh *= g_t, with h_{-1} = h0 (or 0).  o is the
 *   forward output.  log_gates = 1: g holds log decays (chunk_hgrn, mmfreelm/ops/hgrn/chunk.py:137-220): the step uses
 *   exp(g_t) and dg_t = dh h_{t-1} exp(g_t).  As in the reference the gradient of the final state is not propagated. */
int mmf_hgrn_recurrent_bwd(const void* g, const void* o, const void* grad_o, const float* h0, void* dx, void* dg, int64_t BH,
                           int64_t T, int64_t D, int log_gates, int dtype, void* stream);
/* mmf_cross_entropy_train_fwd / _bwd replace cross_entropy_fwd_kernel / cross_entropy_bwd_kernel,
 *   mmfreelm/modules/fused_cross_entropy.py:26-98 / :98-160 (CrossEntropyLossFunction :163-310, one device): per row, with
 *   l = logit_scale * logits, lse = logsumexp(l):
 *     loss = lse - smoothing mean(l) - (1 - smoothing) l[label] + lse_square_scale lse^2   (0 where label == ignore_index;
 *            a label outside [0, V) keeps only the smoothing and z terms, as the reference's out-of-range case does);
 *     z_loss (optional) = lse_square_scale lse^2;  lse is kept for the backward;
 *     dlogits = dloss logit_scale ( exp(l - lse) (1 + 2 lse_square_scale lse) - onehot (1 - smoothing) - smoothing / V ).
 *   dlogits may be the logits buffer itself (the reference's inplace_backward). */
int mmf_cross_entropy_train_fwd(const void* logits, int64_t ld, const int64_t* labels, int64_t ignore_index, float smoothing,
                                float logit_scale, float lse_square_scale, float* loss, float* lse, float* z_loss, int64_t rows,
                                int64_t V, int dtype, void* stream);
int mmf_cross_entropy_train_bwd(const void* logits, int64_t ld, const int64_t* labels, int64_t ignore_index, const float* lse,
                                const float* dloss, float smoothing, float logit_scale, float lse_square_scale, void* dlogits,
                                int64_t ldd, int64_t rows, int64_t V, int dtype, void* stream);

/* ---- ShortConvolution (mmfreelm/modules/convolution.py:45-162) -------------------------------
 * The causal depthwise convolution of kernel size W (<= mmf_short_conv_max_kernel_size() = 8, else MMF_ERR_WIDE) with an
 * optional SiLU (activation = 1) that HGRNBitAttention(use_short_conv=True) puts in front of its projections.
 * x, y: [B, T, D] contiguous; weight: [D, W] (nn.Conv1d's [D, 1, W]); bias: [D] or NULL; all in `dtype`.
 *   pre[b, t, d] = T( sum_{w, t-(W-1)+w >= 0} weight[d, w] * x[b, t-(W-1)+w, d]  (+ bias[d]) ),   fp32 sum, oldest input first
 *   y = T( pre / (1 + exp(-pre)) )  or  pre
 * mmf_short_conv_fwd replaces ShortConvolution.forward for whole sequences (:98-131; causal_conv1d_fn or
 *   nn.Conv1d + activation there); cache ([B, D, W], `dtype`) may be NULL, else it receives the last W inputs of every
 *   channel, oldest first, zero filled when T < W (the state a following step continues from).
 * mmf_short_conv_step replaces ShortConvolution.step (:133-158; causal_conv1d_update there): x, y [B, D]; the cache drops
 *   its oldest entry, takes x, and y is the same sum over it.
 * mmf_short_conv_bwd: gradients of the whole-sequence form.  dpre: [B, T, D] fp32 scratch; partial:
 *   [mmf_short_conv_bwd_groups(B * T), (W + 1) * D] fp32 scratch; dweight_bias: [(W + 1) * D] fp32, entry w * D + d =
 *   dweight[d, w], the last D entries = dbias. */
int mmf_short_conv_max_kernel_size(void);
int mmf_short_conv_fwd(const void* x, const void* weight, const void* bias, void* y, void* cache, int64_t B, int64_t T,
                       int64_t D, int W, int activation, int dtype, void* stream);
int mmf_short_conv_step(const void* x, const void* weight, const void* bias, void* cache, void* y, int64_t B, int64_t D,
                        int W, int activation, int dtype, void* stream);
int mmf_short_conv_bwd_groups(int64_t rows);
int mmf_short_conv_bwd(const void* x, const void* weight, const void* bias, const void* dy, void* dx, float* dpre,
                       float* partial, float* dweight_bias, int64_t B, int64_t T, int64_t D, int W, int activation,
                       int dtype, void* stream);

/* ---- top-p (nucleus) sampling of the next token -----------------------------------------------
 * mmf_sample_top_p replaces, per decoded token of the loop that mmfreelm's generate.py:11 runs
 *   (model.generate(do_sample=True, top_p=0.4, temperature=0.6)), what transformers' sampling path does with the
 *   logits of HGRNBitForCausalLM.forward (modeling_hgrn_bit.py:386): temperature scaling, softmax, descending sort,
 *   cumulative sum, nucleus mask, renormalisation and the multinomial draw -- one launch, no sort.
 *   All decisions are made on integer probability masses, so the result does not depend on a summation order:
 *     l_i = logit_i / temperature (NaN counts as -inf);  p_i = 1 if l_i == max l, else exp(l_i - max l) in fp32;
 *     top_k > 0: l_i = -inf unless l_i >= the top_k-th largest l (transformers' TopKLogitsWarper runs before the
 *       top-p one; the reference's call passes no top_k and so gets the default generation parameters' 50;
 *       equal values stay together; top_k = 0 or >= V: no limit) -- applied before p_i, with max l unchanged;
 *     m_i = trunc(p_i * 2^31);
 *     Z = sum m_i;  P = max(1, trunc(double(top_p) * double(Z)))  (top_p clamped to [0, 1]);
 *     token i is kept iff m_i > 0 and the mass of all tokens with m_j > m_i is below P;
 *     S = mass of the kept tokens;  target = trunc(double(u[r]) * double(S));
 *     out[r] = lowest index whose running sum of kept masses, in index order, exceeds target.
 *   u: one uniform number in [0, 1) per row, drawn by the caller (fp32, device memory); out: int64 [rows].
 *   temperature <= 0 or NaN, top_k < 0: MMF_ERR_ARG;  V > mmf_sample_top_p_max_vocab() (65536): MMF_ERR_WIDE. */
int64_t mmf_sample_top_p_max_vocab(void);
int mmf_sample_top_p(const void* logits, int64_t ld, int64_t rows, int64_t V, float temperature, float top_p,
                     int64_t top_k, const float* u, int64_t* out, int dtype, void* stream);

/* ---- one whole batch-1 decode step in one persistent launch ---------------------------------
 * mmf_decode_layers replaces, for one token, the loop over HGRNBitBlock.forward in HGRNBitModel.forward
 *   (mmfreelm/models/hgrn_bit/modeling_hgrn_bit.py:236-262, the block at :97-109, the attention at
 *   mmfreelm/layers/hgrn_bit.py:83-162): embedding row of *tok -> n_layers x [block norm, i/f/g BitLinear, gate math +
 *   recurrence step, gated norm, o_proj BitLinear, residual + norm, gate_proj BitLinear, swiglu, down_proj BitLinear +
 *   residual] -> h_out [H] (the input of the final norm + lm_head).  Same arithmetic, operation for operation, as the
 *   chain of mmf_bitlinear_gemv_fused launches it stands for.
 *   256 workgroups stay resident and hand activations to each other as 32-bit words (16-bit value | 16-bit tag of the
 *   producing link), each row kept in mmf_decode_layers_copies() copies (one per XCD), so the device must have at least
 *   256 CUs free for the launch (fewer CUs: MMF_ERR_ARG).
 *   phases: device array of 4 * n_layers records of mmf_decode_layers_phase_bytes() bytes each, in the order i/f/g, o,
 *     gate, down: { const void* w1; const void* norm_w; const void* packed; const float* wdeq; const float* lower_bound;
 *     float* state; double inv_K; float eps; float eps1; int K; int N; int seg_rows; int pad; } (w1: weight of the norm
 *     in front of the BitLinear, null for down; norm weights in the activation dtype; inv_K = 1.0 / K; seg_rows = N for
 *     one matrix, the rows of a segment for stacked ones).  The table must not change while the launch runs.
 *   words: mmf_decode_layers_words(H, D, I) uint32 scratch words (16-byte aligned), zero-initialised once, owned by the
 *     caller and reused by every call; epoch: one uint32, zero-initialised once, advanced by the kernel; err: one int,
 *     set to 1 if a wait ran out of its `spin` polling rounds (results are then invalid; the launch still terminates).
 *   head: null, or a device record like the ones of `phases` for the final norm + lm_head (w1 = final norm weight,
 *     K = H, N = vocabulary size); the launch then also writes the logits [N] (activation dtype), and the greedy token
 *     (lowest index of the largest logit; NaNs never win) to *tok_out, which may be the buffer `tok` points to.
 *     am_words: 256 uint64 scratch words, zero-initialised once.  With head == null the three pointers are ignored.
 *   Requires D == H, H, I multiples of 128, H <= 4096, I <= 8192 (else MMF_ERR_WIDE), 16-bit activations (dtype 1 or 2),
 *   batch 1, norm weights of magnitude below 2^40.  Calls on one device must not overlap (they share the scratch words). */
int mmf_decode_layers_phase_bytes(void);
int mmf_decode_layers_copies(void);
int64_t mmf_decode_layers_words(int H, int D, int I);
int mmf_decode_layers(const void* phases, int n_layers, const void* table, const int64_t* tok, int64_t vocab, uint32_t* words,
                      void* h_out, const void* head, void* logits, uint64_t* am_words, int64_t* tok_out, uint32_t* epoch, int* err,
                      int H, int D, int I, int spin, int dtype, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MMF_H_ */
