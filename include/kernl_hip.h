/*
 * kernl_hip.h — C ABI of libkernl_hip.so: hand-written gfx950 (CDNA4) kernels for the three fused
 * transformer ops that kernl's graph rewriting swaps into a model.
 *
 * The reference (ELS-RD/kernl) has no FFI: its operator boundary is three Python callables that launch
 * Triton kernels.  Each entry point below replaces the *launch* inside one of those callables; the Python
 * host layer (kernl_amd/implementations/) keeps the reference's signatures, asserts and allocation
 * rules and forwards raw pointers, sizes, strides and the current HIP stream to these functions.
 *
 * Common rules for every entry point
 *   - plain pointers and integers only; all pointers are device pointers unless stated otherwise;
 *   - asynchronous: work is enqueued on `stream` (a hipStream_t passed as void*; NULL = default stream)
 *     and the call returns immediately — safe under hipGraph stream capture;
 *   - no allocation, no host synchronisation, no retained pointers; re-entrant;
 *   - returns KERNL_OK (0) or a negative kernl_status; kernl_last_error_string() gives the reason
 *     (thread-local);
 *   - strides are in ELEMENTS, not bytes.
 */
#ifndef KERNL_HIP_H
#define KERNL_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum {
    KERNL_OK = 0,
    KERNL_ERR_INVALID_ARG = -1, /* NULL pointer, non-positive size, inconsistent broadcast sizes ... */
    KERNL_ERR_UNSUPPORTED = -2, /* dtype / shape outside what the kernels implement                   */
    KERNL_ERR_LAUNCH = -3       /* hipLaunchKernel reported an error                                   */
} kernl_status;

typedef enum { KERNL_F16 = 0, KERNL_BF16 = 1, KERNL_F32 = 2 } kernl_dtype;

/* Epilogues of the fused linear layer.  Reference: src/kernl/implementations/activation_func.py:28-49
 * ("tanh", "relu", "fast_gelu" = tanh approximation, "gelu" = erf form).  SILU is new (SwiGLU gate). */
typedef enum {
    KERNL_ACT_NONE = 0,
    KERNL_ACT_RELU = 1,
    KERNL_ACT_TANH = 2,
    KERNL_ACT_GELU_ERF = 3,
    KERNL_ACT_GELU_TANH = 4,
    KERNL_ACT_SILU = 5
} kernl_activation;

/* Library version, MAJOR*10000 + MINOR*100 + PATCH. */
int kernl_version(void);

/* Reason for the last non-zero status returned on the calling thread ("" if none). */
const char *kernl_last_error_string(void);

/*
 * Flash-attention forward:  out = softmax(q·kᵀ·sm_scale + causal + mask) · v, never materialising q·kᵀ.
 * Replaces the `_fwd_kernel[grid](...)` launch of src/kernl/implementations/attention.py:499-528
 * (kernel body :122-435).
 *
 *   q   [B,H,M,D]   k,v [B,H,N,D]   out [B,H,M,D]   — any strides (q_strides etc. = {batch, head, row, col});
 *                    the MFMA path needs col stride 1 and 16-byte aligned rows, other layouts take a slower
 *                    scalar kernel with identical semantics.
 *   dtype           KERNL_F16 or KERNL_BF16 for q,k,v,out (reference asserts the same, attention.py:471-474).
 *   mask            NULL, or an ADDITIVE mask of mask_dtype with sizes mask_sizes = {B|1, H|1, M|1, N}
 *                   (size-1 batch/head dims broadcast; third size 1 = one value per key, else a full matrix;
 *                   attention.py:311-323,349-385).  -inf entries are replaced by mask_min_clamp before the add
 *                   (attention.py:380; the host passes finfo(mask dtype).min as the reference does, :516).
 *   is_causal       non-zero: key n contributes to query m only if n <= m (top-left aligned, attention.py:346-347).
 *   Softmax statistics and both accumulators are fp32; P is rounded to `dtype` before P·V (attention.py:424).
 */
int kernl_attention_fwd(const void *q, const void *k, const void *v, void *out, const void *mask,
                        int64_t B, int64_t H, int64_t M, int64_t N, int64_t D,
                        const int64_t q_strides[4], const int64_t k_strides[4],
                        const int64_t v_strides[4], const int64_t o_strides[4],
                        const int64_t mask_sizes[4], const int64_t mask_strides[4], int mask_dtype,
                        float sm_scale, int is_causal, float mask_min_clamp, int dtype, void *stream);

/*
 * Causal attention of M new query rows at positions start_position .. start_position + M - 1 over the N keys of a
 * key/value cache: key n contributes to query row m only if n <= m + start_position (start_position = 0 is
 * kernl_attention_fwd with is_causal; N is usually start_position + M, later keys are never visible) — the mask
 * the reference model builds, `triu(full(-inf), diagonal=start_pos + 1)` (experimental/llama-v2/llama/model.py:338-343).
 * Replaces the `_fwd_kernel[grid](...)` launch of experimental/llama-v2/kernel/fused_kernel_attention.py:127-144
 * (kernel body :21-117, `start_position` at :59-76; that kernel's own comparison agrees with the model's mask at
 * start_position 0, the only value its self-test runs).  All other arguments as kernl_attention_fwd.
 */
int kernl_attention_cached_fwd(const void *q, const void *k, const void *v, void *out, const void *mask,
                               int64_t B, int64_t H, int64_t M, int64_t N, int64_t D,
                               const int64_t q_strides[4], const int64_t k_strides[4],
                               const int64_t v_strides[4], const int64_t o_strides[4],
                               const int64_t mask_sizes[4], const int64_t mask_strides[4], int mask_dtype,
                               float sm_scale, int64_t start_position, float mask_min_clamp, int dtype,
                               void *stream);

/*
 * kernl_attention_fwd / kernl_attention_cached_fwd over keys and values stored as one byte per element, fp8 e5m2 — the
 * upper byte of the fp16 encoding (reference: `get_model_fp8` turns `cache_k` / `cache_v` into int8 tensors holding
 * float8e5, experimental/llama-v2/kernel/fused_kernel_fp8.py:68-74, and the attention kernel widens them on load,
 * fused_kernel_attention.py:66-70, :90-94).  k8, v8: bytes, strides in elements (= bytes); q, out, dtype: KERNL_F16
 * only; head size 64 or 128, unit feature strides, the other strides multiples of 8, 16-byte aligned bases; no mask or
 * a per-key mask ([B|1, H|1, 1, N]); with is_causal, query row m sees keys 0 .. m + start_position (ignored
 * otherwise).  Anything else returns KERNL_ERR_UNSUPPORTED.  Scores, softmax and accumulation as kernl_attention_fwd on
 * the decoded values.
 */
int kernl_attention_kv8_fwd(const void *q, const void *k8, const void *v8, void *out, const void *mask,
                            int64_t B, int64_t H, int64_t M, int64_t N, int64_t D,
                            const int64_t q_strides[4], const int64_t k_strides[4],
                            const int64_t v_strides[4], const int64_t o_strides[4],
                            const int64_t mask_sizes[4], const int64_t mask_strides[4], int mask_dtype,
                            float sm_scale, int is_causal, int64_t start_position, float mask_min_clamp,
                            int dtype, void *stream);

/*
 * Split-K attention for very few query rows (decoding: q_len = 1 against a long key sequence).  Same arguments and
 * semantics as kernl_attention_fwd plus a workspace; the keys of every (batch, head, query row) are split into
 * ranges that run in parallel and are merged by a second kernel.  Replaces the `_fwd_part_1[grid]` /
 * `_fwd_part_2[grid_part2]` launches of src/kernl/implementations/attention_skinny.py:458-535 (the reference
 * allocates its partial maxima / sums / products there, :416-441; here the caller passes them as one workspace).
 * Unlike the reference's dispatch (src/kernl/optimizer/attention.py:45-49, which falls back to eager PyTorch for
 * masked or causal single-query attention) masks and is_causal are handled.
 *
 *   workspace        device memory of at least kernl_attention_skinny_workspace_bytes(B,H,M,N,D) bytes (fp32
 *                    partial results); may be NULL / smaller, which only reduces the number of key ranges.
 *   D                a power of two in 8..256; q, k, v need unit feature stride and 16-byte aligned rows.
 *   B*H*M            at most 65535.
 */
int64_t kernl_attention_skinny_workspace_bytes(int64_t B, int64_t H, int64_t M, int64_t N, int64_t D);
int kernl_attention_skinny_fwd(const void *q, const void *k, const void *v, void *out, const void *mask,
                               void *workspace, int64_t workspace_bytes, int64_t B, int64_t H, int64_t M, int64_t N,
                               int64_t D, const int64_t q_strides[4], const int64_t k_strides[4],
                               const int64_t v_strides[4], const int64_t o_strides[4], const int64_t mask_sizes[4],
                               const int64_t mask_strides[4], int mask_dtype, float sm_scale, int is_causal,
                               float mask_min_clamp, int dtype, void *stream);

/*
 * kernl_attention_skinny_fwd with the keys and values stored as one byte per element: fp8 e5m2, i.e. the upper byte
 * of the fp16 encoding (what the reference keeps in its int8 key/value caches, experimental/llama-v2/kernel/
 * fused_kernel_fp8.py:40-56,68-72, and widens inside its kernel, fused_kernel_attention.py:69-71,90-92).  k and v
 * strides count bytes; rows must be 8-byte aligned.  q, out and `dtype` are 16-bit as before; half the bytes of the
 * key/value stream, the same arithmetic (fp32) on the decoded values.
 */
int kernl_attention_skinny_kv8_fwd(const void *q, const void *k, const void *v, void *out, const void *mask,
                                   void *workspace, int64_t workspace_bytes, int64_t B, int64_t H, int64_t M, int64_t N,
                                   int64_t D, const int64_t q_strides[4], const int64_t k_strides[4],
                                   const int64_t v_strides[4], const int64_t o_strides[4], const int64_t mask_sizes[4],
                                   const int64_t mask_strides[4], int mask_dtype, float sm_scale, int is_causal,
                                   float mask_min_clamp, int dtype, void *stream);

/*
 * kernl_attention_skinny_fwd for callers that cannot allocate device memory (code under hipGraph capture, tight
 * serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference, whose operator allocates its
 * partial maxima / sums / products with torch on every call (src/kernl/implementations/attention_skinny.py:416-441).
 * The partial results of the key ranges live in a device array of kernl_attention_skinny_static_max_bytes() bytes
 * (512 KiB) that is part of the library image: every GPU the library runs on holds it until the process ends.  The call
 * itself performs no hipMalloc / hipFree; the first call on a device looks the array's address up once
 * (hipGetSymbolAddress, which may load the code object): that first call must happen OUTSIDE any stream capture.
 * kernl_attention_skinny_static_init() performs just that lookup for the current device and launches nothing — call
 * it (or make one eager call) per device before capturing a graph that holds kernl_attention_skinny_static_fwd.
 *
 *   - 16-bit keys and values only; arguments as kernl_attention_skinny_fwd without the workspace pair.
 *   - Problems with kernl_attention_skinny_workspace_bytes(B,H,M,N,D) above the array's size (the largest workspace
 *     any problem asks for is about 1 MiB: 256..511 rows of head size 256) are refused with KERNL_ERR_UNSUPPORTED
 *     (nothing is launched); results are bit-identical to kernl_attention_skinny_fwd given a
 *     workspace of the reported size.
 *   - Nothing in the array has to start at zero: every slot the merge kernel reads was written by the same call.
 *   - All calls on one GPU share the array: calls that may overlap in time on one GPU (different streams, different
 *     threads) race.  Calls on one stream are ordered and safe.
 */
int64_t kernl_attention_skinny_static_max_bytes(void);
int kernl_attention_skinny_static_init(void);
int kernl_attention_skinny_static_fwd(const void *q, const void *k, const void *v, void *out, const void *mask,
                                      int64_t B, int64_t H, int64_t M, int64_t N, int64_t D,
                                      const int64_t q_strides[4], const int64_t k_strides[4],
                                      const int64_t v_strides[4], const int64_t o_strides[4],
                                      const int64_t mask_sizes[4], const int64_t mask_strides[4], int mask_dtype,
                                      float sm_scale, int is_causal, float mask_min_clamp, int dtype, void *stream);

/*
 * Rotary position embedding, half-split convention:  out = x·cos + rotate_half(x)·sin, with
 * rotate_half(x)[d] = -x[d + D/2] (d < D/2), x[d - D/2] (d >= D/2); fp32 arithmetic, one rounding.
 * The reference applies the same rotation (in Meta's interleaved-pair convention) inside its fused query/key
 * projection: experimental/llama-v2/kernel/fused_kernel_proj_qkv.py:69-100 (`rbe_triton`), eager form
 * experimental/llama-v2/llama/model.py:78-88.  Here it is one kernel per tensor, replacing the eight element-wise
 * kernels a traced Hugging Face decoder runs for it.
 *
 *   x, out           [B,H,S,D], f16, bf16 or f32 (dtype), any strides (16-byte vector path for the 16-bit types when
 *                    the feature stride is 1 and rows are 16-byte aligned); D even.
 *   cos, sin         tables of table_dtype (f16 / bf16 / f32) with sizes table_sizes = {B|1, H|1, S, D}.
 */
int kernl_rope_fwd(const void *x, const void *cos, const void *sin, void *out, int64_t B, int64_t H, int64_t S,
                   int64_t D, const int64_t x_strides[4], const int64_t out_strides[4], const int64_t table_sizes[4],
                   const int64_t cos_strides[4], const int64_t sin_strides[4], int table_dtype, int dtype,
                   void *stream);

/*
 * Fused linear layer:  out[M,N] = act(x[M,K] · w[N,K]ᵀ + bias[N]).
 * Replaces the `kernel_fma[grid](...)` launch of src/kernl/implementations/linear_layer.py:254-278
 * (kernel body :92-210).
 *
 *   x        [M,K] with strides x_strides = {row, col}; w [N,K] contiguous and bias [N] contiguous
 *            (the reference asserts both, linear_layer.py:242-244); out [M,N] with out_strides.
 *   act_in   NULL, or an [M,N] buffer with strides act_in_strides that receives x·wᵀ + bias BEFORE the
 *            activation (linear_layer.py:193-195).
 *   dtype    KERNL_F16 / KERNL_BF16 (MFMA path when x col stride is 1, K % 8 == 0 and rows are 16-byte
 *            aligned) or KERNL_F32 (FMA path).  Accumulation is fp32; the activation is applied to the
 *            fp32 accumulator (linear_layer.py:198-205).  On the 16-bit path KERNL_ACT_GELU_ERF is evaluated as
 *            x * sigmoid(x * p(x^2)) with a fitted three-term p: absolute error <= 2.6e-5 before the rounding to the
 *            16-bit output; the f32 path uses an erf approximation with error <= 1.5e-7.
 */
int kernl_linear_fwd(const void *x, const void *w, const void *bias, void *out, void *act_in,
                     int64_t M, int64_t N, int64_t K,
                     const int64_t x_strides[2], const int64_t out_strides[2],
                     const int64_t act_in_strides[2], int activation, int dtype, void *stream);

/*
 * kernl_linear_fwd for a weight stored as one byte per element, fp8 e5m2 — the upper byte of the fp16 encoding
 * (reference: `get_model_fp8` turns the weights of the projections into int8 tensors holding float8e5,
 * experimental/llama-v2/kernel/fused_kernel_fp8.py:75-84, and its kernels widen them on load,
 * fused_kernel_ff.py:43-47).  w8 [N, K] contiguous bytes, K % 8 == 0, dtype KERNL_F16 (x, bias, out, act_in);
 * anything else returns KERNL_ERR_UNSUPPORTED.  Up to 64 rows of x (with K % 64 == 0) the weight is streamed once by
 * every CU; larger inputs take a tiled MFMA kernel that fetches the bytes and widens them on their way into LDS.
 * Half the bytes of the weight either way, fp32 accumulation of the decoded values.
 */
int kernl_linear_w8_fwd(const void *x, const void *w8, const void *bias, void *out, void *act_in,
                        int64_t M, int64_t N, int64_t K, const int64_t x_strides[2],
                        const int64_t out_strides[2], const int64_t act_in_strides[2], int activation,
                        int dtype, void *stream);

/*
 * RMSNorm fused into the linear layer that consumes it:
 *     out = activation( rsqrt(mean(x^2) + eps) * ((x * rms_weight) @ w^T) + bias )        (gated = 0)
 *     out = activation(gate) * value, both computed like that from the interleaved weight    (gated != 0)
 * Replaces the `rms_matmul_rbe[grid](...)` launch without its rotary epilogue (experimental/llama-v2/kernel/
 * fused_kernel_proj_qkv.py:116-183, 186-213) and the RMSNorm prologue of `ff_llama` (fused_kernel_ff.py:10-79): as
 * there, x * rms_weight is rounded to the 16-bit type before the product and the inverse root mean square, one
 * scalar per row, multiplies the finished sums.  This is the decoding-step kernel: M <= 64, K % 64 == 0, f16 / bf16;
 * anything else returns KERNL_ERR_UNSUPPORTED and the caller normalises and multiplies in two calls.  w [N, K], or
 * [2N, K] interleaved as for kernl_linear_glu_fwd; bias likewise or NULL.
 */
int kernl_linear_rms_fwd(const void *x, const void *rms_weight, float eps, const void *w, const void *bias, void *out,
                         int64_t M, int64_t N, int64_t K, const int64_t x_strides[2], const int64_t out_strides[2],
                         int activation, int gated, int dtype, void *stream);

/*
 * The linear layer behind an RMSNorm for MANY rows (a prompt), with the norm folded away:
 *     rmsnorm(x) @ w^T  =  rstd[m] * (x @ (w * norm_weight)^T),   rstd[m] = 1 / sqrt(mean(x[m]^2) + eps)
 * so the caller multiplies the norm's weight into the columns of w once, obtains rstd from whoever produced x
 * (kernl_add_rms_stats_fwd below) and this entry point computes
 *     out = (x @ w^T) * row_scale[:, None] + bias                                    plain:  activation KERNL_ACT_NONE
 *     out = silu(y_gate * row_scale + b_gate) * (y_value * row_scale + b_value)      gated != 0, activation KERNL_ACT_SILU:
 *                                                                                     w [2N, K], bias [2N] interleaved as
 *                                                                                     for kernl_linear_glu_fwd
 * in the epilogue of the wide tile kernels: the normalised tensor is never written or read.  Replaces, for prompts, what
 * the reference's `rms_matmul_rbe` (experimental/llama-v2/kernel/fused_kernel_proj_qkv.py:116-183) and `ff_llama`
 * (fused_kernel_ff.py:10-79) do for decoding steps — normalise inside the product — where those kernels re-compute the
 * row statistics in every program.  row_scale: fp32 [M], 16-byte aligned.  f16 / bf16, K % 8 == 0, x with unit feature
 * stride and 16-byte aligned rows; other activations return KERNL_ERR_UNSUPPORTED.
 */
int kernl_linear_scaled_fwd(const void *x, const void *w, const void *bias, const float *row_scale, void *out, int64_t M,
                            int64_t N, int64_t K, const int64_t x_strides[2], const int64_t out_strides[2],
                            int activation, int gated, int dtype, void *stream);

/*
 * The linear layer of MANY rows with the residual addition that follows it in a transformer layer:
 *     out = round(x @ w^T + bias) + residual
 * (the projection is rounded to the 16-bit type first and the sum once more: bit for bit what kernl_linear_fwd followed
 * by an addition of the two 16-bit tensors gives).  The reference's fused linear kernel (src/kernl/implementations/
 * linear_layer.py:92-210) has no residual operand: its models add in eager PyTorch (`hidden_states + input_tensor` in
 * front of every LayerNorm of the graph in docs/how-to-guides/support-new-model.md:481-520; experimental/llama-v2/llama/
 * model.py:262-264).  Here the wide tile kernels fetch the residual one 16-row block ahead of the epilogue that adds it,
 * so the addition costs no pass over memory.  residual: [M, N] of the same dtype with its strides; it must not overlap
 * out.  No activation.  f16 / bf16, K % 8 == 0, x with unit feature stride and 16-byte aligned rows.
 */
int kernl_linear_residual_fwd(const void *x, const void *w, const void *bias, const void *residual, void *out, int64_t M,
                              int64_t N, int64_t K, const int64_t x_strides[2], const int64_t out_strides[2],
                              const int64_t residual_strides[2], int dtype, void *stream);

/*
 * Whether kernl_linear_fwd runs M x N x K (16-bit, plain epilogue, x with unit feature stride) on one of its
 * small-problem kernels, and which: 0 = no; otherwise the kernl_linear_force_tile value of the kernel (10 .. 15).  A
 * caller that would otherwise route such a shape to the stream-K or split-K entry points (kernl_linear_fewrow_fwd,
 * kernl_linear_splitk_fwd) should call kernl_linear_fwd instead: a few hundred rows against a weight of a few million
 * elements run faster as one launch of small tiles.  No counterpart in the reference, which has one kernel and an
 * autotuner (src/kernl/implementations/linear_layer.py:47-91).
 */
int kernl_linear_small_kind(int64_t M, int64_t N, int64_t K);

/*
 * Whether kernl_linear_fwd runs M x N x K (16-bit, plain epilogue) on one of its wide tile kernels, and which: 0 = no,
 * otherwise the kernl_linear_force_tile value of the kernel (5 .. 8).  kernl_linear_residual_fwd and
 * kernl_linear_scaled_fwd exist on those kernels only and run them whatever the shape: a caller asks here first and
 * keeps the separate addition (or normalisation) where another kernel is the faster one.  No counterpart in the
 * reference (one kernel and an autotuner, src/kernl/implementations/linear_layer.py:47-91).
 */
int kernl_linear_wide_kind(int64_t M, int64_t N, int64_t K);

/*
 * kernl_linear_fwd for row counts between the two regimes (129 to a few hundred rows against a few thousand columns),
 * where the 128-row tiles of the tiled kernels are too few to occupy the chip: every output tile is computed by up to
 * four workgroups over disjoint ranges of K, and a second small launch adds their fp32 partial tiles in range order and
 * runs the epilogue (same semantics and arguments as kernl_linear_fwd, reference src/kernl/implementations/
 * linear_layer.py:92-210; the split over K is the `SPLIT_K` axis of the reference's configurations, which it leaves
 * at 1, linear_layer.py:47-67).
 *   kernl_linear_splitk_workspace_bytes(M, N, K) returns 0 when splitting does not pay (enough tiles, or a short K):
 *   call kernl_linear_fwd then.  Otherwise pass a 16-byte aligned workspace of at least that many bytes (contents
 *   irrelevant before and after the call; calls that overlap in time need workspaces of their own).
 *   f16 / bf16, K % 64 == 0, x with unit feature stride and 16-byte aligned rows; anything else returns
 *   KERNL_ERR_UNSUPPORTED.
 */
int64_t kernl_linear_splitk_workspace_bytes(int64_t M, int64_t N, int64_t K);
int kernl_linear_splitk_fwd(const void *x, const void *w, const void *bias, void *out, void *act_in, void *workspace,
                            int64_t workspace_bytes, int64_t M, int64_t N, int64_t K, const int64_t x_strides[2],
                            const int64_t out_strides[2], const int64_t act_in_strides[2], int activation, int dtype,
                            void *stream);

/*
 * The linear layer for a FEW rows of x with many columns and a long K (batched decoding steps: 17 to 128 rows, where
 * kernl_linear_fwd's weight-streaming kernel re-reads x once per 16 to 64 output columns and its tile kernels leave
 * most of their rows empty), with everything a decoder layer puts around its projections:
 *     y   = (rms_weight ? rsqrt(mean(x^2) + eps) * ((x * rms_weight) @ w^T) : x @ w^T) + bias
 *     y   = activation(y)                                  plain form, w [N, K]
 *     y   = activation(y_gate) * y_value                   gated != 0: w [2N, K], bias [2N], interleaved as for
 *                                                          kernl_linear_glu_fwd
 *     y   = rotate(y) on the columns below rope_cols       cos / sin given (no activation, not gated)
 *     out = y + residual                                   residual given
 * Semantics of kernl_linear_fwd (reference: src/kernl/implementations/linear_layer.py:92-210), kernl_linear_glu_fwd,
 * kernl_linear_rms_fwd and kernl_linear_decode_fwd, whose comments name the reference kernels of the fused forms; the
 * decomposition is the reference's stream-K experiment (experimental/streamk/kernel_streamk.py): the (128-row tile of
 * the weight, 64-wide k chunk) units are dealt in equal contiguous runs to at most 256 workgroups, tiles cut by a run
 * boundary are completed from fp32 partial tiles by a second small launch that adds them in a fixed order (results do
 * not depend on timing) and runs the epilogue.
 *   M <= 128, K % 64 == 0, K >= 256, f16 / bf16, x with unit feature stride and 16-byte aligned rows, w contiguous.
 *   workspace  device memory of at least kernl_linear_fewrow_workspace_bytes(M, N, K, gated, rotated) bytes, 16-byte
 *              aligned, contents irrelevant before and after the call (NULL when that function returns 0); calls that
 *              overlap in time need workspaces of their own.
 *   residual   [M, N] of the same dtype with its strides, or NULL.
 *   rotation   arguments as for kernl_linear_decode_fwd; head_dim 32, 64 or 128.
 * Anything else returns KERNL_ERR_UNSUPPORTED; a workspace that is too small KERNL_ERR_INVALID_ARG.
 */
int64_t kernl_linear_fewrow_workspace_bytes(int64_t M, int64_t N, int64_t K, int gated, int rotated);
int kernl_linear_fewrow_fwd(const void *x, const void *rms_weight, float eps, const void *w, const void *bias,
                            const void *residual, void *out, void *workspace, int64_t workspace_bytes, int64_t M,
                            int64_t N, int64_t K, const int64_t x_strides[2], const int64_t out_strides[2],
                            const int64_t residual_strides[2], const void *cos, const void *sin, int64_t head_dim,
                            int64_t rope_cols, int64_t rows_per_batch, const int64_t table_strides[3], int table_dtype,
                            int activation, int gated, int dtype, void *stream);
/* The same with the weight stored as fp8 e5m2 bytes (w8 [N, K] or [2N, K] of one byte per element, decoded to fp16 on
 * its way into the MFMA as in kernl_linear_w8_fwd; reference experimental/llama-v2/kernel/fused_kernel_fp8.py:75-84,
 * fused_kernel_ff.py:43-47); f16 activations only. */
int kernl_linear_fewrow_w8_fwd(const void *x, const void *rms_weight, float eps, const void *w8, const void *bias,
                               const void *residual, void *out, void *workspace, int64_t workspace_bytes, int64_t M,
                               int64_t N, int64_t K, const int64_t x_strides[2], const int64_t out_strides[2],
                               const int64_t residual_strides[2], const void *cos, const void *sin, int64_t head_dim,
                               int64_t rope_cols, int64_t rows_per_batch, const int64_t table_strides[3],
                               int table_dtype, int activation, int gated, int dtype, void *stream);

/*
 * A decoding step's projection with everything around it in ONE launch (at most 64 rows of x, K % 64 == 0, f16 / bf16,
 * plain 16-bit weight w [N, K]):
 *     y   = (rms_weight ? rsqrt(mean(x^2) + eps) * ((x * rms_weight) @ w^T) : x @ w^T) + bias
 *     y   = rotate(y)           on the columns below rope_cols, when cos / sin are given
 *     out = y + residual        when residual is given
 * Replaces the `rms_matmul_rbe_qkv[grid](...)` launch WITH its rotary epilogue (experimental/llama-v2/kernel/
 * fused_kernel_proj_qkv.py:250-347: RMSNorm prologue, the three projections as one product, rotation of the query and
 * key columns, :69-100).  Differences: the rotation uses the half-split convention of Hugging Face decoders (inside a
 * head of head_dim columns, column d pairs with d + head_dim / 2) and reads the cos / sin tables the model computed —
 * element (b, s, d) at b * table_strides[0] + s * table_strides[1] + d, where row m of x is position m % rows_per_batch
 * of batch entry m / rows_per_batch — instead of computing angles from a base; and the residual add, which the
 * reference model leaves to eager PyTorch (experimental/llama-v2/llama/model.py:262-264), has no counterpart there.
 * cos / sin NULL: no rotation (then rms_weight may be NULL too); with rotation rms_weight is required, head_dim a
 * multiple of 32 dividing N and rope_cols.  Anything else returns KERNL_ERR_UNSUPPORTED.
 */
int kernl_linear_decode_fwd(const void *x, const void *rms_weight, float eps, const void *w, const void *bias,
                            const void *residual, void *out, int64_t M, int64_t N, int64_t K,
                            const int64_t x_strides[2], const int64_t out_strides[2],
                            const int64_t residual_strides[2], const void *cos, const void *sin,
                            int64_t head_dim, int64_t rope_cols, int64_t rows_per_batch,
                            const int64_t table_strides[3], int table_dtype, int dtype, void *stream);

/*
 * Gated linear unit:  out[M,N] = act(x·w_gateᵀ + b_gate) * (x·w_valueᵀ + b_value)  as ONE GEMM.
 * Replaces the `ff_llama` launch of experimental/llama-v2/kernel/fused_kernel_ff.py:10-79 (SwiGLU: act = SiLU; that
 * kernel's RMSNorm prologue is not part of this entry point) — and the three kernels (two GEMMs, one multiply) a
 * traced decoder runs for `act_fn(gate_proj(x)) * up_proj(x)`.
 *
 *   w     [2N,K] contiguous, the two weights interleaved in blocks of 32 rows: rows [64b, 64b+32) are rows
 *         [32b, 32b+32) of w_gate, rows [64b+32, 64b+64) the same rows of w_value.  N must be a multiple of 32.
 *   bias  NULL or [2N], interleaved like w.
 *   x     [M,K] with unit feature stride, 16-byte aligned rows, K a multiple of 8; f16 or bf16 only.
 *   activation  KERNL_ACT_* applied to the gate half (SILU for SwiGLU, GELU_TANH / GELU_ERF for GeGLU).
 */
int kernl_linear_glu_fwd(const void *x, const void *w, const void *bias, void *out, int64_t M, int64_t N, int64_t K,
                         const int64_t x_strides[2], const int64_t out_strides[2], int activation, int dtype,
                         void *stream);

/*
 * LayerNorm / RMSNorm forward over the last dimension of a 2-D view x[M,N].
 * Replaces the `implementation[(M,)](...)` launch of src/kernl/implementations/layer_norm.py:314-331
 * (kernel body :115-205).
 *
 *   LayerNorm: out = (x - mean) * rstd * w (+ bias),  rstd = 1/sqrt(biased_var + eps)
 *   RMSNorm  (is_rms != 0): out = x * rstd * w (+ bias), rstd = 1/sqrt(mean(x²) + eps); mean is written as 0.
 *   mean, rstd  NULL or fp32 [M] side outputs (layer_norm.py:186-187).
 *   eps is used as given: the fp16 clamp max(eps, 1.6e-5) of layer_norm.py:295-296 is host-side policy.
 *   Statistics are fp32; x is read from HBM once when a row fits the register-resident path
 *   (col strides 1, N a multiple of 16 bytes / element size, N <= 8192 elements).
 */
int kernl_layernorm_fwd(const void *x, const void *w, const void *bias, void *out, float *mean,
                        float *rstd, int64_t M, int64_t N, int64_t x_row_stride, int64_t x_col_stride,
                        int64_t out_row_stride, int64_t out_col_stride, float eps, int is_rms, int dtype,
                        void *stream);

/*
 * LayerNorm / RMSNorm of (x + residual), same arguments as kernl_layernorm_fwd plus `residual` [M,N]
 * (strides res_row_stride/res_col_stride).  The sum is formed in fp32 and is not written back.
 * No counterpart kernel in the reference, which leaves `x + residual` as a separate eager op in front of
 * every LayerNorm (e.g. the graph in docs/how-to-guides/support-new-model.md:481-520).
 */
int kernl_add_layernorm_fwd(const void *x, const void *residual, const void *w, const void *bias,
                            void *out, float *mean, float *rstd, int64_t M, int64_t N,
                            int64_t x_row_stride, int64_t x_col_stride, int64_t res_row_stride,
                            int64_t res_col_stride, int64_t out_row_stride, int64_t out_col_stride,
                            float eps, int is_rms, int dtype, void *stream);

/*
 * sum = a + b, rounded to the tensors' dtype, and rstd[m] = 1 / sqrt(mean(sum[m]^2) + eps) of the ROUNDED sum — the
 * residual addition of a decoder layer together with the row statistics of the RMSNorm that follows it
 * (kernl_linear_scaled_fwd takes them).  b == NULL (then sum is not written): the statistics of `a` alone.  a, b, sum
 * [M, N] with unit feature stride, 16-byte aligned rows, N % 8 == 0, f16 / bf16; rstd fp32 [M].  No counterpart in the
 * reference, whose model adds in eager PyTorch (experimental/llama-v2/llama/model.py:262-264) and normalises inside its
 * projection kernels.
 */
int kernl_add_rms_stats_fwd(const void *a, const void *b, void *sum, float *rstd, int64_t M, int64_t N,
                            int64_t a_row_stride, int64_t b_row_stride, int64_t sum_row_stride, float eps, int dtype,
                            void *stream);

/*
 * The embedding stage of an encoder in one launch: up to three lookups summed in the tensors' dtype, one addition after
 * the other, and the LayerNorm behind them,
 *     out[b, s, :] = LayerNorm(round(round(table0[ids0[b, s]] + table1[ids1[b, s]]) + table2[ids2[b, s]])) * w + bias
 * (BERT: word, token-type and position embeddings).  The reference leaves this stage to PyTorch — three gathers, two
 * additions and its LayerNorm kernel (src/kernl/implementations/layer_norm.py:115-205, whose statistics and eps handling
 * this kernel keeps); at batch 1 those launches are a tenth of a BERT-base forward.  tables [rows_i, N] contiguous
 * (table1 / table2 may be NULL, in that order), ids int64 with entry (b, s) at b * batch_stride + s * seq_stride
 * (a stride of 0 broadcasts: position ids shared by all sequences); an id outside its table is clamped into it.
 * f16 / bf16, N % 8 == 0, N <= 2048, 16-byte aligned tables, w, bias (or NULL) and out [batch * seq, N] contiguous.
 */
int kernl_embedding_layernorm_fwd(const void *table0, const int64_t *ids0, int64_t ids0_batch_stride, int64_t ids0_seq_stride,
                                  int64_t rows0, const void *table1, const int64_t *ids1, int64_t ids1_batch_stride,
                                  int64_t ids1_seq_stride, int64_t rows1, const void *table2, const int64_t *ids2,
                                  int64_t ids2_batch_stride, int64_t ids2_seq_stride, int64_t rows2, const void *w,
                                  const void *bias, void *out, int64_t batch, int64_t seq, int64_t N, float eps, int dtype,
                                  void *stream);

/* The process-wide test and tuning hooks are not part of this interface: they are declared in kernl_hip_test.h. */

#ifdef __cplusplus
}
#endif
#endif /* KERNL_HIP_H */
