/*
 * tprime_hip.h — C ABI of libtprime_hip.so: gfx950 (MI355X) HIP kernels for the decoder-attention
 * hot path of AI-Hypercomputer/torchprime: causal GQA attention forward/backward with segment-id
 * document masking, RMSNorm forward/backward, rotary position embedding (table + apply).
 *
 * Conventions
 *   - Every pointer is a DEVICE pointer owned by the caller (workspaces included); the library keeps
 *     no persistent allocation and never synchronises the host.
 *   - All launches are asynchronous on `stream` (a hipStream_t passed as void*; NULL = default stream).
 *   - Strides are in ELEMENTS.  Tensors are addressed as (batch, head, seq, dim); the innermost (dim)
 *     stride must be 1, the others are free, so both (B,H,S,D)-contiguous memory and the
 *     (B,S,H,D)-memory-viewed-as-(B,H,S,D) layout the reference's attention modules produce
 *     (torchprime/torch_xla_models/model/llama/model.py:219-227) are accepted without a copy.
 *   - Every entry point returns TP_OK (0) or a negative TP_ERR_* code; tp_last_error() gives the
 *     message for the calling thread.  Nothing throws or aborts.
 *   - dtype codes: TP_BF16 / TP_F16 / TP_F32.
 */
#ifndef TPRIME_HIP_H
#define TPRIME_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TP_OK 0
#define TP_ERR_BAD_ARG (-1)     /* null pointer, non-positive size, misaligned pointer or stride */
#define TP_ERR_UNSUPPORTED (-2) /* shape / dtype combination no kernel is built for */
#define TP_ERR_LAUNCH (-3)      /* hipLaunch reported an error */

#define TP_BF16 0
#define TP_F16 1
#define TP_F32 2

/* Library version (major*10000 + minor*100 + patch). */
int tp_version(void);
/* Message of the last error on this thread ("" if none). The pointer stays valid until the next
 * failing call on the same thread. */
const char* tp_last_error(void);

/* ------------------------------------------------------------------------------------------------
 * RMSNorm.  Replaces LlamaRMSNorm.forward (torchprime/torch_xla_models/model/llama/model.py:38-52),
 * MixtralRMSNorm.forward (model/mixtral/model.py:44-59) and DeepseekV3RMSNorm.forward
 * (model/deepseek_v3/model.py:32-44), which share one body:
 *     y = weight * (x.float() * rsqrt(mean(x.float()^2, -1) + eps)).to(x.dtype)
 * The normalised value is rounded to x's dtype before the weight multiply, as there.
 *   x      (rows, hidden), row stride x_row_stride, dtype x_dtype
 *   w      (hidden), dtype w_dtype: either x_dtype or TP_F32
 *   y      (rows, hidden), row stride y_row_stride, dtype = x_dtype if w_dtype == x_dtype else TP_F32
 *   rstd   (rows) fp32 out: rsqrt(mean(x^2) + eps), kept for the backward
 * ---------------------------------------------------------------------------------------------- */
int tp_rmsnorm_fwd(const void* x, const void* w, void* y, float* rstd, int64_t rows, int hidden,
                   int64_t x_row_stride, int64_t y_row_stride, float eps, int x_dtype, int w_dtype,
                   void* stream);

/* Bytes of fp32 workspace tp_rmsnorm_bwd needs for (rows, hidden). */
size_t tp_rmsnorm_bwd_workspace_bytes(int64_t rows, int hidden);

/* Backward of the expression above (what autograd derives from model/llama/model.py:47-52):
 *     n  = x * rstd;  g = dy * w
 *     dx = rstd * (g - n * mean(g * n, -1))          (dtype x_dtype)
 *     dw = sum_rows dy * n.to(x_dtype)               (dtype w_dtype)
 *   dy     (rows, hidden), row stride dy_row_stride, dtype of y
 *   ws     fp32 workspace of tp_rmsnorm_bwd_workspace_bytes(rows, hidden) bytes
 * dw is reduced in a fixed order (no atomics): results are bitwise reproducible. */
int tp_rmsnorm_bwd(const void* dy, const void* x, const void* w, const float* rstd, void* dx,
                   void* dw, float* ws, int64_t rows, int hidden, int64_t dy_row_stride,
                   int64_t x_row_stride, int64_t dx_row_stride, int x_dtype, int w_dtype,
                   void* stream);

/* tp_rmsnorm_bwd without a workspace argument and without any allocation.  No counterpart in the
 * reference: it is for callers that cannot allocate (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc).  The partial-dw rows go to an array built into the library, 16 MiB of
 * device memory per GPU the library runs on, held until the process ends; shapes whose workspace
 * (tp_rmsnorm_bwd_workspace_bytes) exceeds it, i.e. hidden > 8192 at 512 partial rows, return
 * TP_ERR_UNSUPPORTED.  Calls on one GPU share the array: calls that overlap in time on one GPU race.
 * The first call on a device looks the array's address up (no allocation, but make it outside a graph
 * capture).  Same results as tp_rmsnorm_bwd, bit for bit. */
int tp_rmsnorm_bwd_noalloc(const void* dy, const void* x, const void* w, const float* rstd, void* dx,
                           void* dw, int64_t rows, int hidden, int64_t dy_row_stride,
                           int64_t x_row_stride, int64_t dx_row_stride, int x_dtype, int w_dtype,
                           void* stream);

/* ------------------------------------------------------------------------------------------------
 * Rotary tables.  Replaces LlamaRotaryEmbedding.forward (model/llama/model.py:68-88) and
 * DeepseekV3RotaryEmbedding.forward (model/deepseek_v3/model.py:57-75):
 *     ang[b,s,i] = fp32(position_ids[b,s]) * inv_freq[i]          (fp32 product, as the K=1 matmul)
 *     cos[b,s,:] = (cat(cos(ang), cos(ang)) * attention_scaling).to(dtype), sin likewise
 *   inv_freq      (half) fp32;  position_ids (Bp, S) fp32 contiguous (the models pass float ids)
 *   cos, sin      (Bp, S, 2*half) contiguous, dtype `dtype`
 * ---------------------------------------------------------------------------------------------- */
int tp_rope_table(const float* inv_freq, const float* position_ids, void* cos, void* sin, int Bp,
                  int S, int half, float attention_scaling, int dtype, void* stream);

/* ------------------------------------------------------------------------------------------------
 * Rotary apply on q and k in one launch.  Replaces apply_rotary_pos_emb
 * (model/llama/model.py:98-122), the position_ids-gather variant (model/mixtral/model.py:115-140)
 * and apply_rotary_pos_emb_interleave (model/deepseek_v3/model.py:84-103):
 *     x' = (x * cos) + (rotate_half(x) * sin),   rotate_half(x) = cat(-x[D/2:], x[:D/2])
 * with each product and the sum rounded to the tensor dtype, as the eager expression does.
 *   q (B,Hq,S,D), k (B,Hkv,S,D)  strided (dim stride 1); q_out/k_out same shapes, own strides
 *   cos, sin  (Bc or T, S or T, D): row (b, s) is at  cs_b_stride*b + cs_s_stride*s  unless `pos`
 *             is given, then at  cs_s_stride * pos[b*pos_b_stride + s]  (table gather, Mixtral);
 *             `table_rows` is then the number of table rows: positions are clamped to it in the
 *             kernel (callers reject out-of-range ids first, as the reference's indexing does)
 *   interleaved == 1: x is first permuted [x0,x1,x2,...] -> [evens | odds] (DeepSeek); outputs stay
 *             in the permuted order, as in the reference
 *   interleaved == 2: adjacent pairs (x[2i], x[2i+1]) are rotated by angle i, taken from the first half
 *             of the cos/sin row, and stay in place (Llama-4 apply_rotary_emb, model/llama4/model.py:364-409)
 *   backward != 0: q,k are gradients w.r.t. the outputs and q_out,k_out receive gradients w.r.t.
 *             the inputs (transpose of the rotation, then the inverse permutation if interleaved)
 *   k may be NULL (Hkv = 0) to rotate a single tensor.
 * All base pointers and the b/h/s strides must keep rows 16-byte aligned; D % 16 == 0.
 * ---------------------------------------------------------------------------------------------- */
int tp_rope_apply(const void* q, const void* k, const void* cos, const void* sin,
                  const int64_t* pos, void* q_out, void* k_out, int B, int Hq, int Hkv, int S, int D,
                  const int64_t q_strides[3], const int64_t k_strides[3],
                  const int64_t qo_strides[3], const int64_t ko_strides[3], int64_t cs_b_stride,
                  int64_t cs_s_stride, int64_t pos_b_stride, int64_t table_rows, int interleaved,
                  int backward, int dtype, void* stream);

/* ------------------------------------------------------------------------------------------------
 * Attention forward.  Replaces the three branches of AttentionModule.forward
 * (torchprime/torch_xla_models/attention.py:70-123 splash, :124-150 flash, :151-170 eager) and the
 * segment-id path of tpu_splash_attention_jax_call_wrapper (torchprime/utils/kernel_utils.py:28-131,
 * 215-220, 259-263):
 *     allowed[b,i,j] = (!causal || j <= i) && (seg == NULL || seg[b,i] == seg[b,j])
 *     out[b,h,i,:]   = softmax_j(sm_scale * q[b,h,i,:].k[b,h/n_rep,j,:] | allowed) . v[b,h/n_rep,j,:]
 *     lse[b,h,i]     = log sum_j exp(sm_scale * q.k) over allowed j   (natural log; -inf if none)
 * GQA is by indexing (n_rep = Hq / Hkv), K/V are never expanded (attention.py:18-29, 46-51).
 * A row with no allowed key gives out = 0 and lse = -inf.
 *   q (B,Hq,Sq,Dqk)  k (B,Hkv,Skv,Dqk)  v (B,Hkv,Skv,Dv)  out (B,Hq,Sq,Dv)   strided, dim stride 1
 *   seg   (B, Skv) int32 contiguous or NULL (requires Sq == Skv);  lse (B,Hq,Sq) fp32 contiguous
 *   (Dqk, Dv) in {(64,64), (128,128), (192,128)};  dtype TP_BF16 or TP_F16
 * ---------------------------------------------------------------------------------------------- */
int tp_attn_fwd(const void* q, const void* k, const void* v, const int32_t* seg, void* out,
                float* lse, int B, int Hq, int Hkv, int Sq, int Skv, int Dqk, int Dv,
                const int64_t q_strides[3], const int64_t k_strides[3], const int64_t v_strides[3],
                const int64_t o_strides[3], float sm_scale, int causal, int dtype, void* stream);

/* Bytes of fp32 workspace tp_attn_bwd needs (two floats per query row: rowsum(dO o O) and the LSE in
 * log2 units). */
size_t tp_attn_bwd_workspace_bytes(int B, int Hq, int Sq);

/* Attention backward (the reference gets it from autograd through attention.py:151-170, or from
 * the Pallas backward kernels behind :121-123 / :144-150).  P is recomputed from lse:
 *     P = exp(sm_scale*q.k - lse);  dV = P^T dO;  dS = P o (dO V^T - rowsum(dO o O));
 *     dQ = sm_scale * dS K;  dK = sm_scale * dS^T Q   (dK, dV summed over the n_rep query heads)
 * No atomics: results are bitwise reproducible.
 *   dout, out (B,Hq,Sq,Dv), each with its own stride array (do_strides, o_strides)
 *   dq/dk/dv  strided like q/k/v but with their own stride arrays
 *   ws        fp32 workspace of tp_attn_bwd_workspace_bytes(B,Hq,Sq) bytes
 *   dtype     TP_BF16 / TP_F16 (head dims (64,64), (128,128), (192,128)) or TP_F32 (head dims 64 and 128)
 * ---------------------------------------------------------------------------------------------- */
int tp_attn_bwd(const void* dout, const void* q, const void* k, const void* v, const void* out,
                const float* lse, const int32_t* seg, void* dq, void* dk, void* dv, float* ws, int B,
                int Hq, int Hkv, int Sq, int Skv, int Dqk, int Dv, const int64_t do_strides[3],
                const int64_t q_strides[3], const int64_t k_strides[3], const int64_t v_strides[3],
                const int64_t o_strides[3], const int64_t dq_strides[3], const int64_t dk_strides[3],
                const int64_t dv_strides[3], float sm_scale, int causal, int dtype, void* stream);

/* tp_attn_bwd with timing marks.  No counterpart in the reference; for benchmarks and profilers that
 * want per-kernel times without an external tracer.  `events` is NULL or an array of four
 * hipEvent_t (as void*; individual entries may be NULL) recorded on `stream`: [0] before the first
 * kernel, [1] after the delta kernel, [2] after the dK/dV kernel, [3] after the dQ kernel.  The kernels
 * run in the order delta, dK/dV, dQ - or, where the dQ kernel computes delta itself
 * (tp_attn_bwd_dq_first(...) != 0: no delta kernel, [1] follows [0] at once), dQ then dK/dV, so that
 * [3] is recorded before [2].  Nothing is synchronised. */
int tp_attn_bwd_ex(const void* dout, const void* q, const void* k, const void* v, const void* out,
                   const float* lse, const int32_t* seg, void* dq, void* dk, void* dv, float* ws, int B,
                   int Hq, int Hkv, int Sq, int Skv, int Dqk, int Dv, const int64_t do_strides[3],
                   const int64_t q_strides[3], const int64_t k_strides[3], const int64_t v_strides[3],
                   const int64_t o_strides[3], const int64_t dq_strides[3], const int64_t dk_strides[3],
                   const int64_t dv_strides[3], float sm_scale, int causal, int dtype, void* stream,
                   void* const* events);

/* 1 when tp_attn_bwd / tp_attn_bwd_ex run the dQ kernel first for such a problem (it then computes
 * rowsum(dO o O) itself and there is no separate pass over dO and O), else 0.  `masked`: the call uses
 * q_positions, a soft cap or an additive mask (tp_attn_bwd_masked / tp_attn_bwd_biased; a window or a causal
 * offset alone does not count: those run through the same kernels as plain causality).  No counterpart in
 * the reference (see tp_attn_bwd_ex). */
int tp_attn_bwd_dq_first(int Skv, int Dqk, int Dv, int causal, int has_seg, int masked, int dtype);

/* ------------------------------------------------------------------------------------------------
 * Mask extensions of the functional API (torchprime/utils/kernel_utils.py:259-294,
 * torchprime/utils/parallelism_utils.py:87-152, call site torchprime/torch_xla_models/attention.py:75-119).
 * tp_attn_fwd / tp_attn_bwd with, on top of `causal` and `seg`:
 *   q_positions     NULL or (Sq) int32: query row i stands for position q_positions[i] of the key order
 *                   (LoadBalancedCausalMask.q_sequence); NULL: position i
 *   causal_offset   with causal != 0, key j is allowed iff j <= position + causal_offset (the mask's `offset`)
 *   window_left / window_right   >= 0: key j is allowed only if position - window_left <= j <= position +
 *                   window_right (LocalMask, kernel_utils.py:266-275); < 0: unbounded on that side
 *   logits_soft_cap > 0: scores become cap * tanh(sm_scale * q.k / cap) before masking and softmax
 *                   (attn_logits_soft_cap, kernel_utils.py:292); <= 0: none
 * Tiles outside every row's band are skipped.  A window and / or a causal offset without q_positions and soft
 * cap runs through the causal kernels of tp_attn_fwd / tp_attn_bwd (their causal bound generalised to the
 * band), the other combinations through a general instantiation that evaluates them element by element where a
 * tile is not wholly inside the band.  Rows left without any allowed key give out = 0, lse = -inf and
 * zero gradients.  Dtypes and head dims as tp_attn_fwd.  With none of the extensions in use the calls are
 * tp_attn_fwd / tp_attn_bwd.
 * ---------------------------------------------------------------------------------------------- */
int tp_attn_fwd_masked(const void* q, const void* k, const void* v, const int32_t* seg,
                       const int32_t* q_positions, void* out, float* lse, int B, int Hq, int Hkv, int Sq,
                       int Skv, int Dqk, int Dv, const int64_t q_strides[3], const int64_t k_strides[3],
                       const int64_t v_strides[3], const int64_t o_strides[3], float sm_scale, int causal,
                       int causal_offset, int window_left, int window_right, float logits_soft_cap,
                       int dtype, void* stream);
int tp_attn_bwd_masked(const void* dout, const void* q, const void* k, const void* v, const void* out,
                       const float* lse, const int32_t* seg, const int32_t* q_positions, void* dq,
                       void* dk, void* dv, float* ws, int B, int Hq, int Hkv, int Sq, int Skv, int Dqk,
                       int Dv, const int64_t do_strides[3], const int64_t q_strides[3],
                       const int64_t k_strides[3], const int64_t v_strides[3], const int64_t o_strides[3],
                       const int64_t dq_strides[3], const int64_t dk_strides[3],
                       const int64_t dv_strides[3], float sm_scale, int causal, int causal_offset,
                       int window_left, int window_right, float logits_soft_cap, int dtype, void* stream);

/* ------------------------------------------------------------------------------------------------
 * Additive attention mask: the eager branch of the reference's attention module adds a mask tensor to the
 * scaled scores before the softmax (torchprime/torch_xla_models/attention.py:137-158:
 *     attn_weights = matmul(q, k^T) * scaling; attn_weights = attn_weights + causal_mask).
 * tp_attn_fwd_masked / tp_attn_bwd_masked with, on top of their arguments:
 *   bias            fp32, element (b, h, i, j) at bias[b*bias_strides[0] + h*bias_strides[1] + i*bias_strides[2] + j]
 *                   (key axis contiguous; a broadcast batch or head axis has stride 0); it is added to the
 *                   scaled (and soft-capped) score of query row i of query head h and key j; -inf forbids
 *                   the pair, large negative finite values behave as in the reference (they underflow to a
 *                   zero weight unless every key of the row carries one)
 * The mask gets no gradient (the reference's is a constant).  Every tile is evaluated element by element:
 * use causal / seg / the band arguments for what they can express, they skip tiles.  Rows whose every key is
 * forbidden give out = 0, lse = -inf and zero gradients (the reference's softmax would give NaN there).
 * ---------------------------------------------------------------------------------------------- */
int tp_attn_fwd_biased(const void* q, const void* k, const void* v, const int32_t* seg,
                       const int32_t* q_positions, const float* bias, const int64_t bias_strides[3],
                       void* out, float* lse, int B, int Hq, int Hkv, int Sq, int Skv, int Dqk, int Dv,
                       const int64_t q_strides[3], const int64_t k_strides[3], const int64_t v_strides[3],
                       const int64_t o_strides[3], float sm_scale, int causal, int causal_offset,
                       int window_left, int window_right, float logits_soft_cap, int dtype, void* stream);
int tp_attn_bwd_biased(const void* dout, const void* q, const void* k, const void* v, const void* out,
                       const float* lse, const int32_t* seg, const int32_t* q_positions, const float* bias,
                       const int64_t bias_strides[3], void* dq, void* dk, void* dv, float* ws, int B, int Hq,
                       int Hkv, int Sq, int Skv, int Dqk, int Dv, const int64_t do_strides[3],
                       const int64_t q_strides[3], const int64_t k_strides[3], const int64_t v_strides[3],
                       const int64_t o_strides[3], const int64_t dq_strides[3], const int64_t dk_strides[3],
                       const int64_t dv_strides[3], float sm_scale, int causal, int causal_offset,
                       int window_left, int window_right, float logits_soft_cap, int dtype, void* stream);

/* ------------------------------------------------------------------------------------------------
 * The steps either side of the attention path (HBM-bound, one pass over each tensor).
 * ---------------------------------------------------------------------------------------------- */

/* Residual add fused with the RMSNorm that follows it in a decoder layer
 * (torchprime/torch_xla_models/model/llama/model.py:288-291:
 *     hidden_states = residual + hidden_states; residual = hidden_states;
 *     hidden_states = self.post_attention_layernorm(hidden_states)):
 *     h = (residual + x) rounded to x_dtype;  y = weight * (h.float() * rsqrt(mean(h^2) + eps)).to(x_dtype)
 *   x, residual, h (rows, hidden) of x_dtype with their own row strides; y, rstd, dtypes as tp_rmsnorm_fwd */
int tp_add_rmsnorm_fwd(const void* x, const void* residual, const void* w, void* h, void* y,
                       float* rstd, int64_t rows, int hidden, int64_t x_row_stride,
                       int64_t res_row_stride, int64_t h_row_stride, int64_t y_row_stride, float eps,
                       int x_dtype, int w_dtype, void* stream);

/* Its backward: dx = d(residual) = (RMSNorm backward of dy at h) rounded to x_dtype + dh, where dh is the
 * gradient that reaches h through the residual path; dw as tp_rmsnorm_bwd.  ws: tp_rmsnorm_bwd_workspace_bytes. */
int tp_add_rmsnorm_bwd(const void* dy, const void* dh, const void* h, const void* w, const float* rstd,
                       void* dx, void* dw, float* ws, int64_t rows, int hidden, int64_t dy_row_stride,
                       int64_t dh_row_stride, int64_t h_row_stride, int64_t dx_row_stride, int x_dtype,
                       int w_dtype, void* stream);

/* Llama4TextL2Norm.forward (model/llama4/model.py:104-116): y = (x.float() * rsqrt(mean(x^2, -1) + eps)).type_as(x)
 * over rows of `dim` elements (a head dim: 16 bytes times a power of two up to 64 lanes); rstd (rows) fp32 out. */
int tp_l2norm_fwd(const void* x, void* y, float* rstd, int64_t rows, int dim, int64_t x_row_stride,
                  int64_t y_row_stride, float eps, int dtype, void* stream);
/* dx = rstd * (dy - n * mean(dy * n, -1)),  n = x * rstd */
int tp_l2norm_bwd(const void* dy, const void* x, const float* rstd, void* dx, int64_t rows, int dim,
                  int64_t dy_row_stride, int64_t x_row_stride, int64_t dx_row_stride, int dtype,
                  void* stream);

/* Temperature scale of the Llama-4 NoPE layers (model/llama4/model.py:513-525):
 * y[r, :] = (x[r, :] * scale[(r / heads) % seq]).to(dtype) for rows numbered (batch, position, head);
 * `scale` (seq) fp32.  The backward is the same call on the gradient. */
int tp_scale_rows(const void* x, const float* scale, void* y, int64_t rows, int dim, int64_t x_row_stride,
                  int64_t y_row_stride, int heads, int seq, int dtype, void* stream);

/* act_fn(gate) * up of LlamaMLP.forward (model/llama/model.py:137-139) for act_fn = SiLU:
 * out = (silu(gate).to(dtype) * up).to(dtype), (rows, cols) tensors with their own row strides. */
int tp_swiglu_fwd(const void* gate, const void* up, void* out, int64_t rows, int cols,
                  int64_t gate_row_stride, int64_t up_row_stride, int64_t out_row_stride, int dtype,
                  void* stream);
/* dup = dout * silu(gate).to(dtype);  dgate = (dout * up).to(dtype) * silu'(gate) */
int tp_swiglu_bwd(const void* dout, const void* gate, const void* up, void* dgate, void* dup, int64_t rows,
                  int cols, int64_t dout_row_stride, int64_t gate_row_stride, int64_t up_row_stride,
                  int64_t dgate_row_stride, int64_t dup_row_stride, int dtype, void* stream);

/* cross_entropy_loss (torchprime/torch_xla_models/loss.py:5-20): logits (B,S,V), labels (B,S) int64; position s
 * of a sequence is scored against labels[b, s+1], the last position has no target, labels equal to ignore_index
 * are skipped, the loss is the mean over the scored positions.  The shift is done by indexing (no copies).
 *   lse, row_loss  (B*S) fp32 out: logsumexp of every row, and its loss (0 where there is no target)
 *   loss_and_count (2) fp32 out: the mean loss, and the number of scored positions
 *   dtype          TP_F32 or TP_BF16 logits (the models cast to fp32 first, model/llama/model.py:393) */
int tp_cross_entropy_fwd(const void* logits, const int64_t* labels, float* lse, float* row_loss,
                         float* loss_and_count, int B, int S, int V, int64_t logits_b_stride,
                         int64_t logits_s_stride, int64_t labels_b_stride, int ignore_index, int dtype,
                         void* stream);
/* dlogits = dloss / count * (softmax(logits) - onehot(label)) on scored rows, 0 elsewhere; dloss (1) fp32 */
int tp_cross_entropy_bwd(const void* logits, const int64_t* labels, const float* lse,
                         const float* loss_and_count, const float* dloss, void* dlogits, int B, int S,
                         int V, int64_t logits_b_stride, int64_t logits_s_stride,
                         int64_t labels_b_stride, int64_t dlogits_b_stride, int64_t dlogits_s_stride,
                         int ignore_index, int dtype, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* TPRIME_HIP_H */
