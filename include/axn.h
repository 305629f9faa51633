/*
 * axn.h - C ABI of libaxn_gfx950.so: the per-GPU training hot path of AxoNN's
 * tensor-parallel Linear layer and mixed-precision optimizer step, as
 * hand-written gfx950 (MI355X, CDNA4) kernels.
 *
 * The reference (axonn-ai/axonn) is pure Python and has no FFI of its own; its seam
 * is the torch.autograd.Function / torch.optim.Optimizer protocol.  Each entry
 * point below replaces the torch call(s) the reference makes at the cited
 * file:line (paths relative to the reference checkout).
 *
 * Conventions
 *   - Every pointer is a DEVICE pointer unless the parameter name starts with
 *     "h_" (host array).  The library never frees or retains caller memory.
 *   - Every call is asynchronous on the hipStream_t passed as `stream`
 *     (void*; NULL = the default stream).  No call synchronises the device.
 *   - Return value: AXN_OK (0) or a negative axn_status.  axn_last_error()
 *     returns a thread-local description of the last failure on this thread.
 *   - Argument validation happens before any HIP call, so bad-argument
 *     behaviour is testable on a host without a GPU.
 *   - Matrices are row-major.  "ld*" are row strides in ELEMENTS.
 *   - bf16 = bfloat16 stored as uint16_t, fp32 accumulate everywhere.
 */
#ifndef AXN_H_
#define AXN_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define AXN_ABI_VERSION 12

#if defined(__GNUC__)
#define AXN_API __attribute__((visibility("default")))
#else
#define AXN_API
#endif

typedef enum axn_status {
  AXN_OK = 0,
  AXN_EINVAL = -1, /* null pointer, negative size, unknown enum value      */
  AXN_EALIGN = -2, /* pointer or leading dimension not aligned as required */
  AXN_ESHAPE = -3, /* shape not supported by the kernels                   */
  AXN_EHIP = -4,   /* a HIP runtime call failed (message has the detail)   */
  AXN_ELIMIT = -5  /* size exceeds a documented limit of the entry point   */
} axn_status;

typedef enum axn_dtype {
  AXN_BF16 = 0,
  AXN_F16 = 1,
  AXN_F32 = 2
} axn_dtype;

/* Epilogue fused into the forward GEMM. */
typedef enum axn_epilogue {
  AXN_EPI_NONE = 0,      /* Y = X W^T                                 */
  AXN_EPI_BIAS = 1,      /* Y = X W^T + b                             */
  AXN_EPI_BIAS_GELU = 2, /* Z = X W^T + b ; Y = gelu(Z) (exact erf)   */
  AXN_EPI_GELU = 3       /* Z = X W^T     ; Y = gelu(Z)               */
} axn_epilogue;

AXN_API int axn_abi_version(void);
AXN_API const char* axn_last_error(void);

/* ------------------------------------------------------------------------
 * Linear layer: the three shard GEMMs.
 * M = tokens, K = local in_features, N = local out_features.
 * Requirements (else AXN_ESHAPE / AXN_EALIGN): M,N,K >= 1; N % 8 == 0 and
 * K % 8 == 0; all pointers 16-byte aligned; every ld a multiple of 8.
 * ------------------------------------------------------------------------ */

/* Forward.  Replaces `input_.matmul(weight.t())`
 * (axonn/intra_layer/fully_connected.py:118) and the separate broadcast
 * `x + bias` (fully_connected.py:348); the GELU the reference's callers place
 * after the layer (docs/user_guide.rst:120) can be fused as well.
 *   X [M,K] bf16, W [N,K] bf16, bias [N] fp32 or NULL,
 *   Y [M,N] bf16, Zsave [M,N] bf16 or NULL (pre-activation, saved for
 *   axn_dgelu_dbias when a GELU epilogue is used; same ld as Y). */
AXN_API int axn_gemm_fwd(const void* X, const void* W, const float* bias, void* Y,
                 void* Zsave, int64_t M, int64_t N, int64_t K, int64_t ldx,
                 int64_t ldw, int64_t ldy, int epilogue, void* stream);

/* Input gradient.  Replaces `grad_output.matmul(weight)`
 * (fully_connected.py:140 and :186).
 *   dY [M,N] bf16, W [N,K] bf16, dX [M,K] bf16. */
AXN_API int axn_gemm_dgrad(const void* dY, const void* W, void* dX, int64_t M,
                   int64_t N, int64_t K, int64_t lddy, int64_t ldw,
                   int64_t lddx, void* stream);

/* Weight gradient.  Replaces
 * `grad_output.reshape(-1,N).t().mm(input_.view(-1,K))`
 * (fully_connected.py:147-151 and :171-175) and, with beta = 1, the
 * accumulation `param.grad.add_(grad)` across micro-batches
 * (axonn/intra_layer/overlap_communication.py:42-45 / autograd AccumulateGrad).
 *   dY [M,N] bf16, X [M,K] bf16, dW [N,K] of dw_dtype (AXN_BF16 or AXN_F32),
 *   dW = beta * dW + dY^T X  with beta in {0, 1}. */
AXN_API int axn_gemm_wgrad(const void* dY, const void* X, void* dW, int64_t M,
                   int64_t N, int64_t K, int64_t lddy, int64_t ldx,
                   int64_t lddw, int beta, int dw_dtype, void* stream);

/* Backward of the fused bias/GELU epilogue, one pass over [M,N]:
 *   dZ = dY * gelu'(Z)   (Z = NULL: dZ is not written, dbias = colsum(dY))
 *   dbias[n] = beta * dbias[n] + sum_m dZ[m,n]        (dbias NULL: skipped)
 * Replaces what autograd derives from `x + bias` (fully_connected.py:348)
 * and from the caller's nn.GELU.  dY, Z, dZ are of `dtype` (AXN_BF16, AXN_F16 or
 * AXN_F32), row stride ld; dbias is fp32.  N % 8 == 0, pointers 16-byte
 * aligned, ld % 8 == 0.  Deterministic: column partial sums go through
 * `workspace` (axn_dgelu_dbias_workspace_bytes, needed only when dbias is
 * given) and are reduced in a fixed order.  dZ may alias dY. */
AXN_API int axn_dgelu_dbias(const void* dY, const void* Z, void* dZ, int dtype,
                    float* dbias, int64_t M, int64_t N, int64_t ld, int beta,
                    void* workspace, size_t workspace_bytes, void* stream);
AXN_API size_t axn_dgelu_dbias_workspace_bytes(int64_t M, int64_t N);

/* The three GEMMs on IEEE half operands (the reference's default mixed
 * precision is fp16 autocast with a loss scaler: axonn/axonn.py:21-67,
 * axonn/inter_layer.py:274-302).  Same arguments, requirements and kernels as
 * axn_gemm_fwd / _dgrad / _wgrad with every bf16 operand and result fp16
 * instead; fp32 accumulate; dw_dtype AXN_F16 or AXN_F32. */
AXN_API int axn_gemm_fwd_f16(const void* X, const void* W, const float* bias, void* Y,
                     void* Zsave, int64_t M, int64_t N, int64_t K, int64_t ldx,
                     int64_t ldw, int64_t ldy, int epilogue, void* stream);
AXN_API int axn_gemm_dgrad_f16(const void* dY, const void* W, void* dX, int64_t M,
                       int64_t N, int64_t K, int64_t lddy, int64_t ldw, int64_t lddx,
                       void* stream);
AXN_API int axn_gemm_wgrad_f16(const void* dY, const void* X, void* dW, int64_t M,
                       int64_t N, int64_t K, int64_t lddy, int64_t ldx, int64_t lddw,
                       int beta, int dw_dtype, void* stream);

/* Input gradient and weight gradient of one layer in one call: what AsyncLinear.backward
 * computes (axonn/intra_layer/fully_connected.py:140 and :147-151, with beta = 1 the
 * accumulation of overlap_communication.py:42-45).  Arguments as axn_gemm_dgrad and
 * axn_gemm_wgrad together (dtype AXN_BF16 or AXN_F16 for dY, W, X, dX; dW of dw_dtype), the
 * results are theirs bit for bit.  Shapes whose two tile counts would each leave CUs idle
 * in a launch of their own (8192 x 5120 x 2560: 320 and 200 tiles of 256 x 256 on 256 CUs)
 * run as ONE launch, the longer tiles first, so that a CU takes a tile of the other product
 * as soon as it is free; any other shape is the two calls one after the other. */
AXN_API int axn_gemm_bwd(const void* dY, const void* W, const void* X, void* dX, void* dW,
                 int dtype, int64_t M, int64_t N, int64_t K, int64_t lddy, int64_t ldw,
                 int64_t ldx, int64_t lddx, int64_t lddw, int beta, int dw_dtype, void* stream);

/* Forward with the result in fp32.  Under autocast the reference's product is 16-bit and
 * its bias an fp32 parameter, so `x + bias` (fully_connected.py:348) is promoted to fp32:
 * this is that sum - Y = X W^T + b (AXN_EPI_BIAS) or gelu of it (AXN_EPI_BIAS_GELU; other
 * epilogues AXN_EINVAL) - added in fp32 to the fp32 accumulators and stored unrounded.
 *   X, W, Zsave of `dtype` (AXN_BF16 or AXN_F16), bias fp32, Y [M,N] fp32 (ld ldy, a
 *   multiple of 8); requirements otherwise as axn_gemm_fwd. */
AXN_API int axn_gemm_fwd_f32out(const void* X, const void* W, const float* bias, float* Y,
                        void* Zsave, int dtype, int64_t M, int64_t N, int64_t K, int64_t ldx,
                        int64_t ldw, int64_t ldy, int epilogue, void* stream);

/* Variants of the three GEMMs that divide the contraction among workgroups, given a
 * workspace.  No reference counterpart: torch picks such kernels inside its GEMM library.
 *   A problem with few output tiles (a short batch, a narrow shard) leaves most CUs
 *   without work: the contraction is cut into 2, 4 or 8 parts whose fp32 partial
 *   products a second pass adds in a fixed order (epilogue NONE only; results are
 *   reproducible bit for bit).
 *   axn_gemm_workspace_bytes(op, M, N, K): bytes the call below would use for dense
 *   operands and epilogue NONE, 0 if it would not split.  op, M, N, K as in the call.
 *   axn_gemm_*_ws: arguments as axn_gemm_fwd / _dgrad / _wgrad, plus dtype (AXN_BF16 or
 *   AXN_F16) of the 16-bit operands and results, and the workspace (16-byte aligned, used
 *   by this call alone until it has finished; contents need not be initialised).
 *   workspace == NULL, an epilogue, or a shape that does not profit: the call is the
 *   plain GEMM. */
typedef enum axn_gemm_op { AXN_GEMM_FWD = 0, AXN_GEMM_DGRAD = 1, AXN_GEMM_WGRAD = 2 } axn_gemm_op;
AXN_API size_t axn_gemm_workspace_bytes(int op, int64_t M, int64_t N, int64_t K);
AXN_API int axn_gemm_fwd_ws(const void* X, const void* W, const float* bias, void* Y, void* Zsave,
                    int dtype, int64_t M, int64_t N, int64_t K, int64_t ldx, int64_t ldw,
                    int64_t ldy, int epilogue, void* workspace, size_t workspace_bytes,
                    void* stream);
AXN_API int axn_gemm_dgrad_ws(const void* dY, const void* W, void* dX, int dtype, int64_t M,
                      int64_t N, int64_t K, int64_t lddy, int64_t ldw, int64_t lddx,
                      void* workspace, size_t workspace_bytes, void* stream);
AXN_API int axn_gemm_wgrad_ws(const void* dY, const void* X, void* dW, int dtype, int64_t M,
                      int64_t N, int64_t K, int64_t lddy, int64_t ldx, int64_t lddw,
                      int beta, int dw_dtype, void* workspace, size_t workspace_bytes,
                      void* stream);

/* Gate and up projection of a gated MLP with the activation in the epilogue:
 *   gate = X Wg^T,  up = X Wu^T,  H = silu(gate) * up     (one launch)
 * for `down_proj(act_fn(gate_proj(x)) * up_proj(x))` of the model the reference patches
 * (axonn/models/transformers/modify_llama.py:76-95 builds gate_proj, up_proj and
 * down_proj from its Linear; each projection is one fully_connected.py:118 product).
 * X [M,K] (ld ldx), Wg and Wu [N,K] (both ld ldw), H [M,N] (ld ldh) of `dtype`
 * (AXN_BF16 or AXN_F16); gate_save / up_save (optional, [M,N], ld ldh) receive the two
 * pre-activations rounded to `dtype`, which is what the backward pass (axn_swiglu_bwd)
 * reads.  H is computed from the rounded pre-activations: the result equals
 * axn_gemm_fwd twice followed by axn_swiglu_fwd bit for bit.
 * Shapes: M % 256 == 0, N % 128 == 0, K % 64 == 0, every operand below 2 GiB
 * (AXN_ESHAPE otherwise: use the three separate calls); pointers 16-byte aligned,
 * leading dimensions multiples of 8. */
AXN_API int axn_gemm_swiglu_fwd(const void* X, const void* Wg, const void* Wu, void* H,
                                void* gate_save, void* up_save, int dtype, int64_t M, int64_t N,
                                int64_t K, int64_t ldx, int64_t ldw, int64_t ldh, void* stream);

/* Input gradient of two layers that read the same input, in one pass:
 *   dX = dY1 W1 + dY2 W2
 * (two fully_connected.py:140 products whose results autograd would add, as for the
 * gate and up projections of the MLP above).  dY1 [M,N1], dY2 [M,N2] (both ld lddy),
 * W1 [N1,K], W2 [N2,K] (both ld ldw), dX [M,K] (ld lddx) of `dtype` (AXN_BF16 or
 * AXN_F16).  The sum runs through one set of fp32 accumulators and is rounded once.
 * Shapes: M % 128 == 0, K % 128 == 0, N1 % 64 == 0 and >= 128, N2 % 64 == 0 and >= 64,
 * operands below 2 GiB (AXN_ESHAPE otherwise: two axn_gemm_dgrad calls and an add). */
AXN_API int axn_gemm_dgrad_pair(const void* dY1, const void* W1, const void* dY2, const void* W2,
                                void* dX, int dtype, int64_t M, int64_t N1, int64_t N2, int64_t K,
                                int64_t lddy, int64_t ldw, int64_t lddx, void* stream);

/* SwiGLU activation of the Llama MLP, one pass over [M,N]:
 *   out = silu(gate) * up,  silu(x) = x / (1 + exp(-x)).
 * The reference's Llama patch (axonn/models/transformers/modify_llama.py:76-95)
 * replaces gate_proj / up_proj / down_proj by its Linear and leaves
 * `act_fn(gate_proj(x)) * up_proj(x)` of the model's forward to two elementwise
 * kernels; this entry point and the next replace those and their autograd.
 * gate, up, out of `dtype` (AXN_BF16, AXN_F16 or AXN_F32), row stride ld; N % 8 == 0,
 * ld % 8 == 0, pointers 16-byte aligned.  Computed in fp32, rounded once.
 * out may alias gate or up. */
AXN_API int axn_swiglu_fwd(const void* gate, const void* up, void* out, int dtype,
                   int64_t M, int64_t N, int64_t ld, void* stream);

/* Backward of the above:
 *   dgate = dout * up * silu'(gate),  dup = dout * silu(gate),
 *   silu'(x) = s (1 + x (1 - s)),  s = 1 / (1 + exp(-x)).
 * dgate may alias gate and dup may alias up (each element is read before the
 * element at the same position is written). */
AXN_API int axn_swiglu_bwd(const void* dout, const void* gate, const void* up,
                   void* dgate, void* dup, int dtype, int64_t M, int64_t N,
                   int64_t ld, void* stream);

/* ------------------------------------------------------------------------
 * Embedding table.  T = tokens, V = rows of the (local) table, H = (local)
 * embedding width.  ids are int64 as torch hands them over.  Rows are moved
 * in 16-byte vectors: H and every ld a multiple of 16 / sizeof(element)
 * (4 for fp32, 8 for bf16), pointers 16-byte aligned.  T may be 0.
 * T < 2^31, V < 2^31 - 1.
 * ------------------------------------------------------------------------ */

/* Forward.  Replaces the gather of `F.embedding(x, weight, ...)`
 * (axonn/intra_layer/embedding.py:164-172): out[t, :] = W[ids[t], :].
 * W [V,H] and out [T,H] of `dtype` (any axn_dtype; rows are copied verbatim).
 * torch raises a device-side assertion for an id outside [0, V); here such a
 * token reads as a row of zeros and, if `status` (device int32, may be NULL) is
 * given, *status is set to 1 - it is never cleared by the call. */
AXN_API int axn_embedding_fwd(const int64_t* ids, const void* W, void* out, int dtype,
                      int64_t T, int64_t V, int64_t H, int64_t ldw, int64_t ldo,
                      int32_t* status, void* stream);

/* Workspace of the two entry points below (token positions sorted by id: four int32 per
 * token, one per table row, and the sort's digit counts - 2 to 8 bytes per token and pass).
 * Like every entry point of this library they launch kernels only (the sort is a radix sort
 * of the library's own) and can be captured in a HIP graph. */
AXN_API size_t axn_embedding_workspace_bytes(int64_t T, int64_t V);

/* Backward.  Replaces the autograd of the same F.embedding call
 * (torch's embedding_dense_backward; sparse gradients are not supported):
 *   dW[v, :] = beta * dW[v, :] + sum_{t : ids[t] == v} s_v * dY[t, :]
 * with s_v = 1, or 1 / #{t : ids[t] == v} when scale_grad_by_freq is set;
 * row `padding_idx` (-1: none) receives no gradient.  beta = 0 writes every
 * row of dW (zeros where no token points), so dW needs no clearing.
 * dY [T,H] of dy_dtype, dW [V,H] of dw_dtype (each AXN_BF16 or AXN_F32).
 * Terms are added in fp32 in ascending token order: the result is
 * deterministic and equals a sequential loop over the tokens.  Ids outside
 * [0, V) are skipped. */
AXN_API int axn_embedding_bwd(const int64_t* ids, const void* dY, void* dW, int dy_dtype,
                      int dw_dtype, int64_t T, int64_t V, int64_t H, int64_t lddy,
                      int64_t lddw, int64_t padding_idx, int scale_grad_by_freq,
                      int beta, void* workspace, size_t workspace_bytes, void* stream);

/* max_norm of F.embedding (torch.embedding_renorm_, applied to the table in
 * place before the lookup): every row named by at least one id whose
 * norm_type-norm exceeds max_norm is scaled by max_norm / (norm + 1e-7).
 * W [V,H] of any axn_dtype; max_norm > 0, norm_type > 0. */
AXN_API int axn_embedding_renorm(const int64_t* ids, void* W, int dtype, int64_t T,
                         int64_t V, int64_t H, int64_t ldw, float max_norm,
                         float norm_type, void* workspace, size_t workspace_bytes,
                         void* stream);

/* fp32 variants of the three GEMMs for full-precision layers (the reference's
 * own tests run the layer in fp32: axonn/tests/test_intra_layer_fc.py:25).
 * Same argument meaning as above with fp32 operands and results; bias fp32.
 * Any M,N,K >= 1, pointers 4-byte aligned. */
AXN_API int axn_gemm_fwd_f32(const float* X, const float* W, const float* bias,
                     float* Y, float* Zsave, int64_t M, int64_t N, int64_t K,
                     int epilogue, void* stream);
AXN_API int axn_gemm_dgrad_f32(const float* dY, const float* W, float* dX, int64_t M,
                       int64_t N, int64_t K, void* stream);
AXN_API int axn_gemm_wgrad_f32(const float* dY, const float* X, float* dW, int64_t M,
                       int64_t N, int64_t K, int beta, void* stream);

/* ------------------------------------------------------------------------
 * Mixed-precision optimizer step over a list of tensors (multi-tensor).
 * The tensor list is given as host arrays of device pointers and element
 * counts; tensors may be views into one flat buffer at arbitrary element
 * offsets (axonn/utils.py:11-30), so only natural alignment is required.
 * ------------------------------------------------------------------------ */

/* Device-resident result of the gradient scan, consumed by axn_mt_adam and
 * axn_mt_scale without a host round trip.  32 bytes. */
typedef struct axn_scan_result {
  double sumsq;       /* sum over all tensors of |g * inv_scale|^p (p = 2 unless
                         axn_mt_scan_norm names another order)                */
  float total_norm;   /* sumsq^(1/p)                                          */
  float clip_coef;    /* min(1, max_norm / (total_norm + 1e-6)); 1 if no clip */
  int32_t found_inf;  /* 1 if the overflow check fired, else 0                */
  int32_t reserved[3];
} axn_scan_result;

/* Scratch bytes axn_mt_scan needs for `n` tensors of `total` elements. */
AXN_API size_t axn_mt_scan_workspace_bytes(int64_t n, int64_t total);

/* One read pass over the gradients.  Replaces, fused:
 *   - the overflow test `s = tensor.sum(); isinf(s) + isnan(s) > 0` applied
 *     per tensor to the scaled low-precision gradients
 *     (axonn/inter_layer.py:435-445 called from :455, and optim.py:161):
 *     found_inf = OR over tensors of [the tensor's sum, rounded to g_dtype,
 *     is non-finite]; any inf/nan element makes its tensor's sum non-finite;
 *   - the global gradient 2-norm of the unscaled gradients and the clip
 *     coefficient (axonn/intra_layer/gradient_normalization.py:18-34, :86-87).
 *   h_g[n]: device pointers to gradients of g_dtype (BF16, F16 or F32);
 *   h_sizes[n]: element counts; inv_scale = 1 / loss_scale;
 *   max_norm <= 0 disables clipping (clip_coef = 1).
 *   result: device axn_scan_result; overwritten when accumulate = 0; with
 *   accumulate = 1 the new sum of squares and flag are combined with what
 *   `result` already holds (a gradient list of several dtypes takes one call
 *   per dtype on the same stream) and norm and coefficient are recomputed. */
AXN_API int axn_mt_scan(const void* const* h_g, const int64_t* h_sizes, int64_t n,
                int g_dtype, float inv_scale, float max_norm, int accumulate,
                axn_scan_result* result, void* workspace,
                size_t workspace_bytes, void* stream);

/* The same scan with the norm's order as an argument: total_norm = (sum |g * inv_scale|^p)^(1/p)
 * for p = norm_type, which is what the reference's get_total_norm accepts
 * (axonn/intra_layer/gradient_normalization.py:18-34 takes torch.norm(g, norm_type) per
 * gradient and the norm_type-norm of those; :74-87 the coefficient).  p = 0 follows
 * torch.norm's meaning there: the number of gradients that have a non-zero element;
 * p = +inf / -inf give the largest / smallest |g * inv_scale| (`sumsq` then holds that
 * value, a NaN element makes it NaN as in torch).  A NaN order: AXN_EINVAL.
 * axn_mt_scan is this call with norm_type = 2.  Calls that accumulate into one result
 * must name the same order. */
AXN_API int axn_mt_scan_norm(const void* const* h_g, const int64_t* h_sizes, int64_t n,
                     int g_dtype, float inv_scale, float max_norm, float norm_type,
                     int accumulate, axn_scan_result* result, void* workspace,
                     size_t workspace_bytes, void* stream);

/* axn_mt_scan for callers that cannot allocate device memory and have no workspace to
 * hand over (code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc).  No counterpart in the reference.  Arguments and results as axn_mt_scan
 * without the workspace: the per-chunk partial results go to an array of
 * AXN_MT_SCAN_SCRATCH_BYTES that is part of the library's device image (each GPU the
 * library runs on holds its own copy until the process ends).  The call allocates and
 * frees nothing, on the device or through a library.
 * Limit: axn_mt_scan_workspace_bytes(n, total) <= AXN_MT_SCAN_SCRATCH_BYTES, i.e. about
 * 4.29e9 gradient elements in up to a few thousand tensors; beyond it the call returns
 * AXN_ELIMIT before it touches the device.
 * All calls on one GPU share that GPU's array: calls that may overlap in time on one GPU
 * (different streams, different host threads) race and must be serialised by the caller.
 * Nothing in the array needs to start at zero (every partial result a call reads it has
 * written itself), so the array is never cleared. */
#define AXN_MT_SCAN_SCRATCH_BYTES 1048576
AXN_API int axn_mt_scan_noalloc(const void* const* h_g, const int64_t* h_sizes, int64_t n,
                        int g_dtype, float inv_scale, float max_norm, int accumulate,
                        axn_scan_result* result, void* stream);

/* Scalar hyper-parameters of one Adam step.  The bias corrections are
 * computed by the caller in double precision, as torch does
 * (torch/optim/adam.py::_single_tensor_adam, reached from
 * axonn/optim.py:168-182). */
typedef struct axn_adam_hparams {
  float lr_over_bc1;     /* lr / (1 - beta1^t)            */
  float inv_sqrt_bc2;    /* 1 / sqrt(1 - beta2^t)         */
  float beta1;
  float one_minus_beta1;
  float beta2;
  float one_minus_beta2;
  float eps;
  float weight_decay;    /* L2 form: g += weight_decay * p */
} axn_adam_hparams;

/* One streaming pass: for every element
 *   g  = float(g_lowp) * inv_scale * clip_coef          (optim.py:157-160,
 *                                      gradient_normalization.py:88-93)
 *   g += weight_decay * p
 *   m += (g - m) * (1 - beta1);  v = v * beta2 + (1 - beta2) * g * g
 *   p -= lr_over_bc1 * m / (sqrt(v) * inv_sqrt_bc2 + eps)       (optim.py:168-182)
 *   p_lowp = round_to_nearest_even(p)                            (optim.py:183-185)
 * `scan` may be NULL (no overflow gate, clip_coef = 1); otherwise, when
 * scan->found_inf != 0 NOTHING is written (the whole step is skipped on the
 * device, axonn/inter_layer.py:428-430), and scan->clip_coef is applied.
 *   h_g/h_p/h_m/h_v/h_plow[n]: device pointers; h_plow may be NULL (no
 *   low-precision copy) ; p, m, v are fp32. */
AXN_API int axn_mt_adam(const void* const* h_g, void* const* h_p, void* const* h_m,
                void* const* h_v, void* const* h_plow, const int64_t* h_sizes,
                int64_t n, int g_dtype, int plow_dtype, float inv_scale,
                const axn_scan_result* scan, const axn_adam_hparams* hp,
                void* stream);

/* In-place g = g * inv_scale * (use_clip ? scan->clip_coef : 1) on every
 * tensor, in g_dtype.  Replaces `p.grad.div_(loss_scale)`
 * (axonn/inter_layer.py:458) and the clipping `g.mul_(clip_coef_clamped)`
 * (gradient_normalization.py:88-93).  `scan` may be NULL when use_clip = 0. */
AXN_API int axn_mt_scale(void* const* h_g, const int64_t* h_sizes, int64_t n,
                 int g_dtype, float inv_scale, const axn_scan_result* scan,
                 int use_clip, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* AXN_H_ */
