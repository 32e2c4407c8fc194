/* libtmb_hip — C ABI of the MI355X (gfx950) kernels behind torch_mojo_backend's hot ATen ops.
 *
 * Conventions (shared by every entry point):
 *   - plain pointers are DEVICE pointers supplied by the caller; the caller owns every buffer,
 *     outputs included (the reference's "classic" raw-pointer ABI, e.g.
 *     torch_mojo_backend/eager_kernels/aten_fast.py:2763-2776 and :4588-4600);
 *   - `stream` is a hipStream_t passed as void* (NULL = the legacy default stream); launches
 *     are asynchronous and never synchronise, like the reference's enqueue-and-return kernels
 *     (torch_mojo_backend/eager_kernels/__init__.py:9-12);
 *   - dtypes cross as `tmb_dtype` ints;
 *   - the return value is 0 on success, a negative `tmb_status` for argument errors detected
 *     on the host before anything is enqueued, or a positive hipError_t from the launch.
 *   - no entry point allocates or frees device memory; kernels that need scratch take a
 *     caller-provided workspace whose size `tmb_*_workspace_bytes` reports.
 */
#ifndef TMB_HIP_H_
#define TMB_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum tmb_dtype {
  TMB_F32 = 0,
  TMB_F16 = 1,
  TMB_BF16 = 2,
  TMB_I64 = 3,
  TMB_I32 = 4
} tmb_dtype;

typedef enum tmb_status {
  TMB_OK = 0,
  TMB_ERR_INVALID_ARGUMENT = -1, /* null pointer, negative size, unknown enum */
  TMB_ERR_UNSUPPORTED = -2,      /* well-formed request this build has no kernel for */
  TMB_ERR_WORKSPACE = -3,        /* workspace missing or too small */
  TMB_ERR_SCRATCH_LIMIT = -4     /* shape needs more scratch than the library's static array holds */
} tmb_status;

typedef enum tmb_reduce_op { TMB_SUM = 0, TMB_MEAN = 1, TMB_AMAX = 2 } tmb_reduce_op;

typedef enum tmb_epilogue {
  TMB_EPI_NONE = 0,
  TMB_EPI_GELU_TANH = 1, /* 0.5*x*(1+tanh(sqrt(2/pi)*(x+0.044715*x^3))) applied after bias */
  TMB_EPI_GELU_ERF = 2   /* 0.5*x*(1+erf(x/sqrt(2))) applied after bias */
} tmb_epilogue;

/* Flag or-ed into an `epilogue` argument. Without it a fused epilogue stays in fp32 from the
 * accumulator to the one cast: T(gelu(acc + bias)), T(acc + bias + residual) - the reference's
 * rule for what it fuses into a GEMM (matmul_ops.mojo:2651-2657: "forming A@B + bias in fp32 and
 * casting to the output dtype exactly once"). With it every fused step rounds to the storage
 * type where a separate kernel would have stored its result: T(gelu(T(acc + bias))),
 * T(T(acc + bias) + residual), the bits of the unfused sequence of kernels. */
#define TMB_EPI_ROUND_LIKE_UNFUSED 0x100

/* Library/ABI version (major*1000 + minor). */
int tmb_version(void);

/* Human-readable text for a return code of any entry point (static storage). */
const char* tmb_status_string(int code);

/* Row softmax / log-softmax over the last (contiguous) dimension of a [rows, cols] matrix.
 * fp32 arithmetic, one cast on store: m = max_j x; s = sum_j exp(x - m);
 * softmax = exp(x - m)/s, log_softmax = x - m - log(s).
 * `in_dtype` in {F32,F16,BF16}; `out_dtype` equals `in_dtype` or F32 (half_to_float).
 * Replaces nn_ops.mojo:413-493 (`_softmax_rows`, scale=1, causal=0) behind SoftmaxSpec
 * (nn_ops.mojo:2818-2864) and reduction_ops.mojo:778-933 (`_log_softmax_rows`). */
int tmb_softmax_rows(void* out, const void* in, int64_t rows, int64_t cols, int in_dtype,
                     int out_dtype, int log_mode, void* stream);

/* Attention form of the row softmax: y = softmax_j(x[r][j] * scale), and with q_len > 0 only
 * columns j <= r % q_len take part (causal mask of a [.., q_len, cols] score tensor flattened
 * to rows); the masked columns are written as exact zeros and their input is not read.
 * `round_scaled` != 0 rounds x*scale to `dtype` before the max, i.e. reproduces the bits of a
 * separate `mul` kernel followed by masked_fill(-inf) and softmax. `dtype` in {F32,F16,BF16},
 * output of the same type.
 * Replaces nn_ops.mojo:413-493 (`_softmax_rows(scale, causal, q_len)`: m = max(x*scale),
 * denom = sum exp(x*scale - m), causal zeroes j > r % q_len). */
int tmb_softmax_rows_scaled(void* out, const void* in, int64_t rows, int64_t cols, int dtype,
                            float scale, int round_scaled, int64_t q_len, void* stream);

/* Layer norm over the last dimension of [rows, cols]: two-pass fp32 statistics
 * (mean = sum(x)/cols, var = sum((x-mean)^2)/cols biased, rstd = 1/sqrt(var+eps)),
 * out = (x-mean)*rstd*gamma + beta cast once. `dtype` in {F32,F16,BF16} is the type of `out`,
 * `gamma` and `beta`; `in_dtype` is `dtype`, or F32 for fp32 rows normalised into a 16-bit
 * tensor (a residual stream kept in fp32 between the blocks of a 16-bit model). `gamma`/`beta`
 * may be NULL (no affine); `mean`/`rstd` ([rows] fp32) may be NULL when the caller proved them
 * dead.
 * Replaces normalization_forward_ops.mojo `LayerNormForwardF32`
 * (called at aten_fast.py:2763-2776) and nn_ops.mojo:208-346 `LayerNorm` (aten_fast.py:2783-2793). */
int tmb_layer_norm_rows(void* out, float* mean, float* rstd, const void* x, const void* gamma,
                        const void* beta, int64_t rows, int64_t cols, double eps, int in_dtype,
                        int dtype, void* stream);

/* Reduction over the LEADING dimension of a row-major [rows, cols] matrix: out[c] = op_r in[r, c]
 * (SUM, MEAN = sum / rows, AMAX with NaN propagation), floats only, fp32 accumulation, one cast.
 * The bias gradient of a linear layer and every sum(x, dim=0): the input is read once in row
 * order, row slabs are reduced into float32 partial rows in the workspace
 * (tmb_reduce_cols_workspace_bytes) and added slab by slab in a fixed order. rows == 0 returns
 * TMB_ERR_UNSUPPORTED (the identity of an empty reduction is the caller's rule).
 * Replaces the permute + contiguous copy into [kept, reduced] order (op_utils/__init__.mojo:651-720)
 * that precedes SumSpec/MeanSpec/AmaxSpec (reduction_ops.mojo:1094-1184) for such dims. */
size_t tmb_reduce_cols_workspace_bytes(int64_t rows, int64_t cols, int dtype);
int tmb_reduce_cols(void* out, const void* in, int64_t rows, int64_t cols, int op, int dtype,
                    void* workspace, size_t workspace_bytes, void* stream);

/* Bytes of device workspace `tmb_reduce_rows` needs for a shape (may be 0). */
size_t tmb_reduce_workspace_bytes(int64_t rows, int64_t cols, int dtype);
/* The same for `tmb_argmax_rows`, whose rows are cut into smaller pieces (may be 0). */
size_t tmb_argmax_workspace_bytes(int64_t rows, int64_t cols, int dtype);

/* Row reduction of [rows, cols] (cols contiguous) to [rows]; a full reduction is rows == 1.
 * Floats accumulate in fp32 and are cast once (F32/F16/BF16); I64 sums and I64/I32 maxima use
 * their own type. The combine order is a fixed tree that depends only on (rows, cols), so
 * results are bit-reproducible. MEAN is the fp32 sum divided by cols.
 * AMAX propagates NaN. Replaces reduction_ops.mojo:161-263 (`_reduce_rows`), nn_ops.mojo:981-1027
 * (`_mean_rows`) behind SumSpec/MeanSpec/AmaxSpec (reduction_ops.mojo:1094-1184). */
int tmb_reduce_rows(void* out, const void* in, int64_t rows, int64_t cols, int op, int dtype,
                    void* workspace, size_t workspace_bytes, void* stream);

/* tmb_reduce_rows for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc): same kernels, same partition and
 * therefore the same bits, but the partials of a split reduction go to a static array of
 * TMB_REDUCE_STATIC_SCRATCH_BYTES inside the library (one copy per GPU, held until the process
 * ends) instead of a caller's workspace. Allocates and frees nothing. Shapes whose
 * tmb_reduce_workspace_bytes exceeds the array are refused with TMB_ERR_SCRATCH_LIMIT before
 * anything is enqueued. A split reduction has at most rows + 8192 partials of 16 bytes, and only
 * for rows < 4096, unless a row is longer than 2^30 elements: such rows are cut into chunks of
 * 2^30 whatever the row count, and thousands of them exceed the array (4000 rows of 6 * 2^30
 * elements need 4000 * 6 * 16 bytes). The stream must belong to the calling thread's current
 * device (checked: TMB_ERR_INVALID_ARGUMENT otherwise), whose copy of the array is used. The first
 * call on a device looks the array's address up (hipGetSymbolAddress); make that call outside
 * graph capture. A HIP runtime failure of that lookup, of the device queries or of a launch is
 * returned as the positive hipError_t value, as from every other entry point; the library's own
 * codes (tmb_status) are negative.
 * All calls on one GPU share the array: calls that overlap there (two streams, two threads)
 * race; calls on one stream are ordered and safe. Nothing in it needs clearing between calls:
 * the first stage writes every partial the second stage reads.
 * No counterpart in the reference, whose spec ops allocate their scratch inside the call
 * (op_utils/__init__.mojo:389-447). */
#define TMB_REDUCE_STATIC_SCRATCH_BYTES (256 * 1024)
int tmb_reduce_rows_static(void* out, const void* in, int64_t rows, int64_t cols, int op,
                           int dtype, void* stream);

/* First-occurrence argmax of every row of [rows, cols] to int64 [rows]; NaN counts as the
 * maximum (first NaN wins), otherwise greater value wins and equal values keep the lower index
 * at every stage of the tree. `dtype` in {F32,F16,BF16,I64,I32}. Long rows are cut into pieces
 * whose (value, index) partials (16 bytes each, tmb_argmax_workspace_bytes in total) a second
 * launch combines in column order.
 * Replaces nn_ops.mojo:1424-1522 (`_argmax_rows`) behind ArgmaxSpec (nn_ops.mojo:2599-2653). */
int tmb_argmax_rows(int64_t* out, const void* in, int64_t rows, int64_t cols, int dtype,
                    void* workspace, size_t workspace_bytes, void* stream);

/* Batched GEMM  C[b] = epilogue(op(A[b]) . op(B[b]) + bias)  with fp32 accumulation; bias
 * (length n, same dtype, may be NULL) is added in fp32 before the single down-cast
 * (matmul_ops.mojo:2651-2657). Logical shapes: op(A) is [m,k], op(B) is [k,n], C is [m,n]
 * row-major with leading dimension ldc. `trans_a`/`trans_b` = 0: the operand is stored
 * row-major as its logical shape ([m,k] with lda / [k,n] with ldb); = 1: stored as the
 * transpose ([k,m] with lda / [n,k] with ldb — the layout of a torch `weight.t()` view).
 * stride_* are element strides between batch entries (stride 0 broadcasts an operand).
 * `dtype` in {F32,F16,BF16} for A, B, bias and C alike. `epilogue` is a tmb_epilogue, optionally
 * or-ed with TMB_EPI_ROUND_LIKE_UNFUSED.
 * Replaces the raw-pointer GEMM bridges `Bf16GemmBF16` (aten_fast.py:4588-4600),
 * `Bf16BmmBF16` (aten_fast.py:4707-4721) and MatmulSpec/MatmulBiasSpec/BmmSpec
 * (matmul_ops.mojo:3451-3636). */
int tmb_gemm(void* c, const void* a, const void* b, const void* bias, int64_t batch, int64_t m,
             int64_t n, int64_t k, int64_t lda, int64_t ldb, int64_t ldc, int64_t stride_a,
             int64_t stride_b, int64_t stride_c, int trans_a, int trans_b, int dtype,
             int epilogue, void* stream);

/* tmb_gemm with a caller-provided workspace. Products with few output tiles and a long K (the
 * weight gradient dy^T x, narrow projections) then run split along K: fp32 partials
 * [splits][m][n] in the workspace, added in split order by a second kernel that applies bias,
 * epilogue and the one cast (still fp32 accumulation and one rounding; the result depends on the
 * shape only). tmb_gemm_workspace_bytes is 0 when the shape would not be split; with a NULL or
 * too small workspace the call behaves exactly like tmb_gemm.
 * The reference's GPU GEMM takes its split-K scratch from the MAX runtime
 * (eager_kernels/matmul_ops.mojo:1040-1049, `multistage_gemm_kernel`); here the caller owns it,
 * as with every other buffer. */
size_t tmb_gemm_workspace_bytes(int64_t batch, int64_t m, int64_t n, int64_t k, int dtype);
int tmb_gemm_ws(void* c, const void* a, const void* b, const void* bias, int64_t batch, int64_t m,
                int64_t n, int64_t k, int64_t lda, int64_t ldb, int64_t ldc, int64_t stride_a,
                int64_t stride_b, int64_t stride_c, int trans_a, int trans_b, int dtype,
                int epilogue, void* workspace, size_t workspace_bytes, void* stream);

/* tmb_gemm followed by an elementwise add of `residual` [batch][m, n] (row pitch `ldr`, batch
 * stride `stride_r`) in the same launch (the residual connection of a transformer block:
 * demo_scripts/gpt2.py:85-86 `x = x + self.attn(...)`, which reaches the graph as
 * addmm -> view -> add): c = OUT(a b + bias + residual), summed in fp32 and cast once; with
 * TMB_EPI_ROUND_LIKE_UNFUSED c = T(T(epilogue(a b + bias)) + residual), rounded twice exactly as a
 * GEMM kernel followed by an add kernel would.
 * `residual_dtype` and `out_dtype` are `dtype` or TMB_F32: a 16-bit model may keep its residual
 * stream in fp32 (fp32 residual in, fp32 sum out, nothing rounded in between; not together
 * with TMB_EPI_ROUND_LIKE_UNFUSED). 16-bit A and B on the MFMA path only; TMB_ERR_UNSUPPORTED
 * otherwise (fp32 A/B, k == 0, transposed A, unaligned operands, a GELU epilogue unless
 * TMB_EPI_ROUND_LIKE_UNFUSED): the caller then launches tmb_gemm and adds separately.
 * Replaces `AddF32Bf16Spec` / the residual add of aten_fast.py:657-687 together with the GEMM
 * in front of it. */
int tmb_gemm_residual(void* c, const void* a, const void* b, const void* bias,
                      const void* residual, int64_t batch, int64_t m, int64_t n, int64_t k,
                      int64_t lda, int64_t ldb, int64_t ldc, int64_t ldr, int64_t stride_a,
                      int64_t stride_b, int64_t stride_c, int64_t stride_r, int trans_a,
                      int trans_b, int dtype, int residual_dtype, int out_dtype, int epilogue,
                      void* stream);

/* Fused attention forward: out[b,t,h,:] = softmax_j(scale * q[b,h,t,:] . k[b,h,j,:]) v[b,h,j,:],
 * with `causal` != 0 only keys j <= t take part. The [batch, heads, q_len, kv_len] scores never
 * reach memory (online softmax over blocks of 64 keys). `dtype` in {F16,BF16}; head_dim must
 * be 64 and contiguous; every tensor is described by three element strides {batch, head,
 * token}, multiples of 8 (q, k, v; 16-byte aligned bases) or 4 (out; 8-byte aligned), so q, k
 * and v may be slices of one packed [batch, q_len, 3*heads*64] projection and out may be laid
 * out [batch, q_len, heads, 64]. fp32 scores and statistics; probabilities are rounded to
 * `dtype` before they multiply v; `round_like_unfused` != 0 also rounds the scores and the
 * scaled scores to `dtype`, as a separate bmm and mul kernel would have stored them.
 * Returns TMB_ERR_UNSUPPORTED for other head sizes, scale <= 0, kv_len == 0 or unaligned layouts (the
 * caller then runs the unfused chain).
 * Replaces aten_functions.py:443-677 (`aten__scaled_dot_product_*`, built from matmul, softmax
 * and matmul graph ops) and aten_fast.py:5177-5285 (`fast_aten_scaled_dot_product_attention`). */
int tmb_attention_fwd(void* out, void* lse, const void* q, const void* k, const void* v,
                      int64_t batch, int64_t heads, int64_t q_len, int64_t kv_len, int64_t head_dim,
                      const int64_t* q_strides, const int64_t* k_strides,
                      const int64_t* v_strides, const int64_t* out_strides, float scale,
                      int causal, int round_like_unfused, int dtype, void* stream);

/* Fused attention backward: dq, dk, dv of tmb_attention_fwd's `out` given its gradient `dout`,
 * the forward's inputs, `out` itself and the `lse` it wrote. With p[t,j] = exp(scale * q_t . k_j -
 * lse[t]) (0 where the causal rule hides key j) and delta[t] = sum_d dout[t,d] * out[t,d]:
 *   dv[j] = sum_t p[t,j] dout[t],   ds[t,j] = p[t,j] * (dout[t] . v[j] - delta[t]) * scale,
 *   dq[t] = sum_j ds[t,j] k[j],     dk[j] = sum_t ds[t,j] q[t].
 * Nothing of size q_len x kv_len reaches memory; p and ds are rounded to `dtype` before they enter
 * a product, all sums are float32, and no atomics are used (the same call gives the same bits).
 * Tensors are addressed [batch, heads, tokens, 64] through three element strides {batch, head,
 * token} each: multiples of 8 with 16-byte aligned bases for q, k, v, out, dout, multiples of 4
 * with 8-byte aligned bases for dq, dk, dv. `workspace` is device memory of
 * tmb_attention_bwd_workspace_bytes(batch, heads, q_len) bytes, 16-byte aligned, that the call
 * overwrites (delta and lse in base-2 units). `dtype` in {F16, BF16}, head_dim 64, scale > 0.
 * Returns TMB_ERR_UNSUPPORTED for anything else (the caller then differentiates the unfused
 * chain). Replaces `fast_fa4_bf16_d64_causal_backward` (eager_kernels/aten_fast.py:4089-4170),
 * the kernel behind aten::_scaled_dot_product_flash_attention_backward
 * (mojo_device/mojo_device_aten_ops.py:881-882). */
int64_t tmb_attention_bwd_workspace_bytes(int64_t batch, int64_t heads, int64_t q_len);
int tmb_attention_bwd(void* dq, void* dk, void* dv, const void* dout, const void* q, const void* k,
                      const void* v, const void* out, const void* lse, void* workspace,
                      int64_t batch, int64_t heads, int64_t q_len, int64_t kv_len,
                      int64_t head_dim, const int64_t* q_strides, const int64_t* k_strides,
                      const int64_t* v_strides, const int64_t* out_strides,
                      const int64_t* dout_strides, const int64_t* dq_strides,
                      const int64_t* dk_strides, const int64_t* dv_strides, float scale,
                      int causal, int dtype, void* stream);

/* Attention for a few queries per (batch, head) — the decode step of a generation loop — as one
 * memory-bound launch (K and V are read once, nothing goes through MFMA): out = softmax(scale *
 * q k^T [+ mask]) v with an online softmax in fp32. Strides are in elements as in
 * tmb_attention_fwd; head_dim 64 or 128, fp16 / bf16. `mask` is NULL or a boolean (1 byte, nonzero
 * = the key takes part) tensor addressed as mask[b*ms[0] + h*ms[1] + t*ms[2] + s*ms[3]] (stride 0
 * where it broadcasts); `causal` keeps key s for query t if s <= t. A query without any key
 * yields NaN, as in ATen. Returns TMB_ERR_UNSUPPORTED for layouts it does not take (the caller
 * then composes GEMM + softmax + GEMM).
 * Replaces `fast_aten_scaled_dot_product_attention` (aten_fast.py:5177-5285) on decode shapes. */
int tmb_attention_decode(void* out, const void* q, const void* k, const void* v, const void* mask,
                         int64_t batch, int64_t heads, int64_t q_len, int64_t kv_len,
                         int64_t head_dim, const int64_t* q_strides, const int64_t* k_strides,
                         const int64_t* v_strides, const int64_t* out_strides,
                         const int64_t* mask_strides, float scale, int causal, int dtype,
                         void* stream);

/* Embedding lookup: out[i, :] = table[indices[i], :] for a contiguous [num_rows, row_len] table of
 * type `dtype` and `num_indices` contiguous indices of type `index_dtype` (TMB_I64 or TMB_I32).
 * Replaces `Gather0(out, table, indices, idx_dtype, num_indices, row_len, dtype, ctx)`
 * (eager_kernels/nn_ops.mojo:1153-1176, 3098-3099; called from aten_fast.py:5336-5371) and
 * `aten_embedding` (aten_functions.py:1780-1795). An index outside [0, num_rows) reads the
 * nearest valid row instead of memory outside the table (the reference leaves it undefined). */
int tmb_gather_rows(void* out, const void* table, const void* indices, int64_t num_indices,
                    int64_t row_len, int64_t num_rows, int dtype, int index_dtype, void* stream);

/* Elementwise GELU over `numel` contiguous elements, fp32 inside, one cast.
 * `approximate_tanh` != 0 selects the tanh form. Replaces activation_forward_kernels.mojo:22-56
 * (used when the GELU cannot be fused into the producing GEMM's epilogue). */
int tmb_gelu(void* out, const void* in, int64_t numel, int dtype, int approximate_tanh,
             void* stream);

/* GELU backward over `numel` contiguous elements: grad_in = grad_out * gelu'(in), fp32 inside,
 * one cast; all three tensors have type `dtype`. Replaces `GeluBackwardF32` / `GeluBackwardBF16`
 * (eager_kernels/activation_backward_ops.mojo:50-73 for the two derivatives, aten_fast.py:1413-1447
 * for the call) and `custom_mojo_ops.gelu_backward` (aten_functions.py:2070-2102). */
int tmb_gelu_backward(void* grad_in, const void* grad_out, const void* in, int64_t numel,
                      int dtype, int approximate_tanh, void* stream);

/* Backward of a row softmax (log_mode 0: grad_in = out * (grad_out - sum(grad_out * out))) or
 * log-softmax (log_mode 1: grad_in = grad_out - exp(out) * sum(grad_out)) from the saved output;
 * contiguous [rows, cols], one dtype for the three tensors. Replaces the composed
 * sum -> exp -> addcmul of aten_functions.py:788-833 and the fused kernel behind
 * `fast_aten__log_softmax_backward_data` (aten_fast.py:3237-3330). */
int tmb_softmax_backward_rows(void* grad_in, const void* grad_out, const void* out, int64_t rows,
                              int64_t cols, int dtype, int log_mode, void* stream);

/* The gradient a cross-entropy loss sends to the logits, from the saved log-probabilities
 * logp [rows, cols] (row pitch ldi) and the int64 targets [rows]: the dense NLL gradient (-w at a
 * row's target unless that is ignore_index or no class; w = grad_out / total_weight for
 * reduction 1 = mean, grad_out for 2 = sum, grad_out[row] for 0 = none; grad_out and total_weight
 * are device scalars of the tensor type) sent through the log-softmax backward,
 * dx = g - exp(logp) * rowsum(g), without g being stored. dx has a row pitch of its own
 * (ldo >= cols, a whole number of 16-byte vectors, dx 16-byte aligned); columns cols .. ldo-1 are
 * set to zero, so a consumer that needs rows of whole vectors can take dx as it is.
 * Replaces NllLossBackwardF32 (eager_kernels/aten_fast.py:3450-3497, loss_ops.mojo:234-311)
 * followed by `_log_softmax_backward_data` (aten_functions.py:788-833). */
int tmb_nll_log_softmax_backward_rows(void* dx, const void* logp, const int64_t* target,
                                      const void* grad_out, const void* total_weight, int64_t rows,
                                      int64_t cols, int64_t ldi, int64_t ldo, int reduction,
                                      int64_t ignore_index, int dtype, void* stream);

/* Layer-norm backward over contiguous [rows, cols] from the saved fp32 statistics:
 *   grad_in    = rstd * (g dy - mean_row(g dy) - xhat * mean_row(g dy xhat)),  xhat = (x - mean) rstd
 *   grad_gamma = sum over rows of dy * xhat,   grad_beta = sum over rows of dy
 * Any of the three outputs may be NULL (ATen's output_mask); `gamma` may be NULL (no affine).
 * The parameter gradients are summed slab by slab through `workspace`
 * (tmb_layer_norm_backward_workspace_bytes) in an order that depends on the shape only.
 * Replaces `LayerNormBackwardF32(grad_input, grad_weight, grad_bias, grad, x, mean, rstd, gamma,
 * rows, cols, mask_bits, ctx)` (aten_fast.py:2797-2913). */
size_t tmb_layer_norm_backward_workspace_bytes(int64_t rows, int64_t cols, int dtype);
int tmb_layer_norm_backward_rows(void* grad_in, void* grad_gamma, void* grad_beta,
                                 const void* grad_out, const void* in, const float* mean,
                                 const float* rstd, const void* gamma, int64_t rows, int64_t cols,
                                 int dtype, void* workspace, size_t workspace_bytes, void* stream);

/* tmb_layer_norm_backward_rows where the gradient re-joins the residual stream of a decoder
 * block (x <- x + f(norm(x))): what is stored is grad_in = round(dx) + addend, rounded again
 * (addend: the gradient that by-passed the block, same shape and type, may be NULL), and
 * grad_sum [cols] receives the column sums of the stored grad_in (may be NULL): the bias gradient
 * of the projection in front of the norm. At least one of the two is given; grad_in, grad_gamma
 * and grad_beta are all wanted. The result equals the three separate steps it replaces, each
 * storing its result in the tensor type: this layer-norm backward, `aten.add`
 * (aten_functions.py:939, fast_aten_add aten_fast.py:1010-1024) and `aten.sum` over the leading
 * dimension (aten_functions.py:3310-3312); the column sums are added in an order of their own
 * that depends on the shape only. Shapes outside the one-pass kernels (cols not a whole number of
 * 16-byte vectors, more than 8192 columns) report TMB_ERR_UNSUPPORTED and a workspace size of 0:
 * the caller then runs the three steps. */
size_t tmb_layer_norm_backward_add_workspace_bytes(int64_t rows, int64_t cols, int dtype);
int tmb_layer_norm_backward_add_rows(void* grad_in, void* grad_gamma, void* grad_beta,
                                     void* grad_sum, const void* grad_out, const void* in,
                                     const float* mean, const float* rstd, const void* gamma,
                                     const void* addend, int64_t rows, int64_t cols, int dtype,
                                     void* workspace, size_t workspace_bytes, void* stream);

/* Concatenation of two contiguous row blocks: out[r] = a[r] ++ b[r] for `rows` rows of
 * `a_row_bytes` and `b_row_bytes` bytes (any element type; the widest of 16/4/2/1-byte pieces that
 * the lengths and the three addresses allow is moved). With rows = the product of the dims in
 * front of the concatenated one this is aten::cat of two contiguous tensors, in particular the
 * append of one token to a [batch, heads, tokens, head_dim] key/value cache.
 * Replaces `Cat2` (eager_kernels/data_movement_ops.mojo:217-340, called from
 * aten_fast.py:2203-2228). */
int tmb_cat2_rows(void* out, const void* a, const void* b, int64_t rows, int64_t a_row_bytes,
                  int64_t b_row_bytes, void* stream);

/* Row copy with zero padding: out[r, 0:row_len] = in[r, 0:row_len], out[r, row_len:out_pitch] = 0
 * for `rows` rows of 2- or 4-byte elements (`itemsize`); pitches in elements. The source needs
 * element alignment only, the destination 16-byte aligned rows (out_pitch * itemsize % 16 == 0).
 * It turns an operand whose rows are not whole 16-byte vectors (K = 50257 in the backward of a
 * vocabulary projection) into one the matrix-core GEMM kernels read, at copy speed. No counterpart
 * entry in the reference: its GEMM wrappers pass only exact dense layouts in place
 * (`_tf32_dense_2d_layout`, aten_fast.py:4457-4467) and leave the rest to MAX's matmul. */
int tmb_pad_rows(void* out, const void* in, int64_t rows, int64_t row_len, int64_t in_pitch,
                 int64_t out_pitch, int itemsize, void* stream);

/* Plain device copy kernel (16-byte vectors, grid-stride) — the bandwidth yardstick the
 * benchmark and the counter calibration use. No reference counterpart. */
int tmb_copy_bytes(void* out, const void* in, size_t bytes, void* stream);

/* The read-only yardstick beside it: reads `bytes` (whole 16-byte vectors of them) once and
 * writes nothing (`sink`, at least 4 bytes of device memory, is written only if a 16 KiB piece
 * folds to one particular bit pattern). What a reduction over the same bytes is measured
 * against. No reference counterpart. */
int tmb_read_bytes(const void* in, size_t bytes, void* sink, void* stream);

#ifdef __cplusplus
}
#endif

#endif /* TMB_HIP_H_ */
