"""CPU ORACLE — TEST INFRASTRUCTURE ONLY.

A plain-PyTorch (CPU, fp32/fp64) restatement of the arithmetic of torchprime's decoder-attention hot
path.  Only tests, ``__graft_entry__.smoke()`` and ``bench.py``'s ``cpu_baseline`` leg may import
this module; nothing under ``torchprime_amd/`` does.  Every function cites the reference lines it
follows (paths relative to the reference checkout).

Pinning status (what each function is checked against in tests/test_oracle.py, without importing the
reference, which needs torch_xla / jax / omegaconf):

  rms_norm                  F.rms_norm, fp64 numpy brute force, invariants          pinned
  rms_norm_grads_eager_order  torch autograd through rms_norm itself (bf16 and fp32), explicit
                            sum_rows dy * round(x_hat) loop                          pinned
  default/llama3 inv_freq   closed form; llm.c loop restated from torchprime/tests/test_rope.py:83-108;
                            transformers ROPE_INIT_FUNCTIONS["llama3"] when installed   pinned
  yarn inv_freq             transformers ROPE_INIT_FUNCTIONS["yarn"] when installed; closed-form
                            special cases (factor 1 -> plain RoPE)                  pinned
  rotary_cos_sin            closed form cos(p * f_i)                                pinned
  apply_rotary_pos_emb      complex rotation, norm preservation, relative-position invariant  pinned
  ..._interleave            permutation o rotate-half, QK^T invariance              pinned
  eager_attention           F.scaled_dot_product_attention, brute-force loops       pinned
  attention_ref             eager_attention (causal), block-diagonal decomposition for segments,
                            brute force incl. fully-masked rows                     pinned
  llama_attention           the pieces above composed; HF LlamaAttention when installed    pinned
  mixtral_attention         equals llama_attention with tables taken at position_ids; shifted ids  pinned
  deepseek_v3_attention     brute-force per-head loops with the rotary part as a complex rotation of
                            adjacent pairs (independent of the [evens|odds] layout); attention_ref with
                            k_rot expanded by hand; gradient of k_rot = sum over heads       pinned
  add_rms_norm, l2_norm     F.rms_norm without a weight, explicit fp64 loops                pinned
  apply_rotary_emb_llama4   complex rotation of adjacent pairs (torch.polar), norm preservation      pinned
  llama_decoder_layer       HuggingFace LlamaDecoderLayer (eager) where importable; composed of pinned parts  pinned
  llama_for_causal_lm       HuggingFace LlamaForCausalLM (eager; the reference's two test fixtures, with and without
                            Llama 3.1 rope scaling, at its three input sizes): logits, loss, every gradient      pinned
  llama4_attention          explicit loops (pair rotation, unit-RMS q/k, per-position scale, softmax);
                            = llama_attention with de-interleaved projection rows on rotary layers     pinned
  attn temperature          closed form log(floor((p+1)/f)+1) a + 1 at hand-computed positions       pinned
  swiglu                    x * sigmoid(x) * u in fp64 loops                                          pinned
  cross_entropy_loss        explicit per-token -log softmax loops incl. ignored labels; F.cross_entropy   pinned
  allowed_mask extensions   window = band matrix (torch.tril/triu); permuted causal = causal on the un-permuted
                            order (reorder o attention o reorder^-1); soft cap = explicit loops         pinned
                            (exact inclusivity of jax's LocalMask bounds: restated from its published source,
                            jax is not installed and pinned to no version by the reference: PARITY UNPINNED)
  segment masking vs the reference's TPU splash kernel numerics                     PARITY UNPINNED:
                            no reference test exercises decoder_segment_ids and the Pallas kernel is
                            not in the tree; semantics are the closed form
                            allowed = (j <= i) & (seg_i == seg_j) from kernel_utils.py:215-220, 259-263.
"""

from __future__ import annotations

import math

import torch
import torch.nn.functional as F

NEG_INF = float("-inf")


# ------------------------------------------------------------------------------------------------
# RMSNorm — torchprime/torch_xla_models/model/llama/model.py:46-52 (same body at
# model/mixtral/model.py:53-59, model/deepseek_v3/model.py:38-44)
# ------------------------------------------------------------------------------------------------
def rms_norm(hidden_states: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
  input_dtype = hidden_states.dtype
  h = hidden_states.to(torch.float32)
  variance = h.pow(2).mean(-1, keepdim=True)
  h = h * torch.rsqrt(variance + eps)
  return weight * h.to(input_dtype)


def rms_norm_grads_eager_order(x: torch.Tensor, weight: torch.Tensor, dy: torch.Tensor, eps: float):
  """(dx, dw) autograd returns for ``rms_norm`` above, evaluated in fp64: the normalised value is rounded to
  the input dtype before the weight multiply (model/llama/model.py:51-52) and the cast passes gradients
  straight through, so ``dw = sum_rows dy * round(x_hat)`` while ``dx`` flows through the unrounded x_hat."""
  x64 = x.double().requires_grad_(True)
  w64 = weight.double().requires_grad_(True)
  h = x64 * torch.rsqrt(x64.pow(2).mean(-1, keepdim=True) + eps)
  h_rounded = h + (h.detach().to(x.dtype).double() - h.detach())  # value of the cast, gradient of the identity
  (w64 * h_rounded).backward(dy.double())
  return x64.grad, w64.grad


def rms_norm_exact(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
  """The same function without intermediate rounding, in fp64 (what tolerances are measured against)."""
  x = x.double()
  return weight.double() * (x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps))


# ------------------------------------------------------------------------------------------------
# inverse-frequency tables — torchprime/rope/rope.py
# ------------------------------------------------------------------------------------------------
def default_rope_frequencies(head_dim: int, theta: float = 10000.0) -> torch.Tensor:
  """rope/rope.py:25-39."""
  return 1.0 / (theta ** (torch.arange(0, head_dim, 2, dtype=torch.int64).float() / head_dim))


def llama3_rope_frequencies(head_dim, theta=10000.0, factor=None, low_freq_factor=1.0, high_freq_factor=4.0,
                            original_context_len=8192) -> torch.Tensor:
  """rope/rope.py:42-75; ``factor=None`` means no scaling."""
  freqs = default_rope_frequencies(head_dim, theta)
  if factor is None:
    return freqs
  low_wl = original_context_len / low_freq_factor
  high_wl = original_context_len / high_freq_factor
  assert low_wl >= high_wl
  wavelen = 2 * math.pi / freqs
  freqs = torch.where(wavelen > low_wl, freqs / factor, freqs)
  smooth = (original_context_len / wavelen - low_freq_factor) / (high_freq_factor - low_freq_factor)
  smoothed = (1 - smooth) * freqs / factor + smooth * freqs
  medium = ~(wavelen < high_wl) * ~(wavelen > low_wl)
  return torch.where(medium, smoothed, freqs)


def yarn_rope_frequencies(dim, base, factor, original_max, max_position_embeddings=None, beta_fast=32, beta_slow=1,
                          mscale=None, mscale_all_dim=None, attention_factor=None, has_original=True):
  """rope/rope.py:78-177 with the config fields spelled out as arguments."""
  if has_original:
    factor = max_position_embeddings / original_max
  def get_mscale(scale, m=1):
    return 1.0 if scale <= 1 else 0.1 * m * math.log(scale) + 1.0
  if attention_factor is None:
    if mscale and mscale_all_dim:
      attention_factor = float(get_mscale(factor, mscale) / get_mscale(factor, mscale_all_dim))
    else:
      attention_factor = get_mscale(factor)
  def corr(num_rot):
    return (dim * math.log(original_max / (num_rot * 2 * math.pi))) / (2 * math.log(base))
  low, high = max(math.floor(corr(beta_fast)), 0), min(math.ceil(corr(beta_slow)), dim - 1)
  if low == high:
    high += 0.001
  pos_freqs = base ** (torch.arange(0, dim, 2).to(dtype=torch.float) / dim)
  extra, inter = 1.0 / pos_freqs, 1.0 / (factor * pos_freqs)
  ramp = torch.clamp((torch.arange(dim // 2, dtype=torch.float32) - low) / (high - low), 0, 1)
  ef = 1 - ramp
  return inter * (1 - ef) + extra * ef, attention_factor


# ------------------------------------------------------------------------------------------------
# cos/sin tables — model/llama/model.py:68-88; model/deepseek_v3/model.py:57-75 (attention_scaling)
# ------------------------------------------------------------------------------------------------
def rotary_cos_sin(inv_freq: torch.Tensor, position_ids: torch.Tensor, dtype: torch.dtype, attention_scaling=1.0):
  inv = inv_freq[None, :, None].float().expand(position_ids.shape[0], -1, 1)
  pos = position_ids[:, None, :].float()
  freqs = (inv.float() @ pos.float()).transpose(1, 2)
  emb = torch.cat((freqs, freqs), dim=-1)
  cos, sin = emb.cos() * attention_scaling, emb.sin() * attention_scaling
  return cos.to(dtype), sin.to(dtype)


# ------------------------------------------------------------------------------------------------
# rotary apply — model/llama/model.py:91-122; model/mixtral/model.py:136-140;
# model/deepseek_v3/model.py:84-103
# ------------------------------------------------------------------------------------------------
def rotate_half(x):
  x1 = x[..., : x.shape[-1] // 2]
  x2 = x[..., x.shape[-1] // 2 :]
  return torch.cat((-x2, x1), dim=-1)


def apply_rotary_pos_emb(q, k, cos, sin, position_ids=None, unsqueeze_dim=1, gather=False):
  if gather:  # Mixtral: tables (T, D) gathered by integer positions
    cos, sin = cos[position_ids.long()], sin[position_ids.long()]
  cos, sin = cos.unsqueeze(unsqueeze_dim), sin.unsqueeze(unsqueeze_dim)
  return (q * cos) + (rotate_half(q) * sin), (k * cos) + (rotate_half(k) * sin)


def apply_rotary_pos_emb_interleave(q, k, cos, sin, unsqueeze_dim=1):
  cos, sin = cos.unsqueeze(unsqueeze_dim), sin.unsqueeze(unsqueeze_dim)
  b, h, s, d = q.shape
  q = q.reshape(b, h, s, d // 2, 2).transpose(4, 3).reshape(b, h, s, d)
  b, h, s, d = k.shape
  k = k.reshape(b, h, s, d // 2, 2).transpose(4, 3).reshape(b, h, s, d)
  return (q * cos) + (rotate_half(q) * sin), (k * cos) + (rotate_half(k) * sin)


# ------------------------------------------------------------------------------------------------
# attention — torchprime/torch_xla_models/attention.py
# ------------------------------------------------------------------------------------------------
def repeat_kv(hidden_states: torch.Tensor, n_rep: int) -> torch.Tensor:
  """attention.py:18-29."""
  batch, kvh, slen, hd = hidden_states.shape
  if n_rep == 1:
    return hidden_states
  return hidden_states[:, :, None, :, :].expand(batch, kvh, n_rep, slen, hd).reshape(batch, kvh * n_rep, slen, hd)


def causal_additive_mask(seq_length: int, dtype=torch.float32) -> torch.Tensor:
  """model/llama/model.py:347-352: -inf strictly above the diagonal, (1,1,S,S)."""
  return torch.triu(torch.full((seq_length, seq_length), NEG_INF, dtype=dtype), diagonal=1)[None, None]


def eager_attention(q, k, v, attention_mask=None):
  """The eager branch of AttentionModule.forward, op for op (attention.py:46-60, 151-170), with
  dropout p=0.  q (B,Hq,S,D), k/v (B,Hkv,S,D*); GQA by repeat_kv; scale 1/sqrt(v.shape[-1])."""
  n_rep = q.shape[1] // k.shape[1]
  k, v = repeat_kv(k, n_rep), repeat_kv(v, n_rep)
  head_dim = v.shape[-1]
  w = torch.matmul(q, k.transpose(2, 3)) / math.sqrt(head_dim)
  if attention_mask is not None:
    w = w + attention_mask[:, :, :, : k.shape[-2]]
  w = F.softmax(w, dim=-1, dtype=torch.float32).to(q.dtype)
  return torch.matmul(w, v)


def allowed_mask(segment_ids, q_len: int, kv_len: int, causal: bool, window=None, q_positions=None,
                 causal_offset: int = 0) -> torch.Tensor:
  """Boolean (B or 1, q_len, kv_len): (j <= i if causal) AND same segment.  Closed form of
  CausalMask/FullMask (kernel_utils.py:259-263) combined with SegmentIds(q=ids, kv=ids) (:215-220).

  Extensions: ``window=(left, right)`` ANDs in jax's LocalMask as kernel_utils.py:271-275 builds it (offset 0;
  its mask function is ``q - left <= kv`` and ``kv <= q + right``, either side optional);
  ``q_positions`` replaces the row index i by the position the row stands for and ``causal_offset`` shifts the
  causal bound, ``q_positions[i] + offset >= j``: LoadBalancedCausalMask (parallelism_utils.py:109-132)."""
  i = torch.arange(q_len) if q_positions is None else torch.as_tensor(q_positions).to(torch.int64).cpu()
  i = i[:, None]
  j = torch.arange(kv_len)[None, :]
  m = (j <= i + causal_offset) if causal else torch.ones((q_len, kv_len), dtype=torch.bool)
  if window is not None:
    left, right = window
    if left is not None:
      m = m & (i - left <= j)
    if right is not None:
      m = m & (j <= i + right)
  m = m[None]
  if segment_ids is not None:
    seg = segment_ids.to("cpu")
    m = m & (seg[:, :, None] == seg[:, None, :])
  return m


def attention_ref(q, k, v, segment_ids=None, causal=True, sm_scale=None, dtype=torch.float32, window=None, soft_cap=None,
                  q_positions=None, causal_offset=0):
  """softmax(sm_scale * q k^T | allowed) v in ``dtype`` with no intermediate rounding; returns
  (out, lse).  Rows with no allowed key give out = 0, lse = -inf (the eager formula gives NaN there;
  tests assert that divergence explicitly).  ``soft_cap``: logits <- cap * tanh(logits / cap) before masking, the
  published definition of the splash kernel's ``attn_logits_soft_cap`` (kernel_utils.py:292)."""
  q, k, v = q.to(dtype), k.to(dtype), v.to(dtype)
  n_rep = q.shape[1] // k.shape[1]
  k, v = repeat_kv(k, n_rep), repeat_kv(v, n_rep)
  if sm_scale is None:
    sm_scale = 1.0 / math.sqrt(v.shape[-1])
  s = torch.matmul(q, k.transpose(2, 3)) * sm_scale
  if soft_cap is not None:
    s = soft_cap * torch.tanh(s / soft_cap)
  m = allowed_mask(segment_ids, q.shape[2], k.shape[2], causal, window, q_positions, causal_offset)[:, None]
  s = s.masked_fill(~m, NEG_INF)
  lse = torch.logsumexp(s, dim=-1)
  any_allowed = m.any(-1)
  p = torch.exp(s - torch.where(any_allowed, lse, torch.zeros_like(lse))[..., None])
  p = torch.where(m, p, torch.zeros_like(p))
  out = torch.matmul(p, v)
  return out, lse


def attention_ref_chunked(q, k, v, segment_ids=None, causal=True, sm_scale=None, dtype=torch.float32, heads_per_chunk=4):
  """attention_ref evaluated a few heads at a time so S=8192 fits in host memory; same arithmetic."""
  outs, lses = [], []
  n_rep = q.shape[1] // k.shape[1]
  step = n_rep * max(1, heads_per_chunk // n_rep)  # whole GQA groups per chunk
  for h0 in range(0, q.shape[1], step):
    h1 = min(h0 + step, q.shape[1])
    ks, vs = k[:, h0 // n_rep : h1 // n_rep], v[:, h0 // n_rep : h1 // n_rep]
    o, l = attention_ref(q[:, h0:h1], ks, vs, segment_ids, causal, sm_scale, dtype)
    outs.append(o)
    lses.append(l)
  return torch.cat(outs, 1), torch.cat(lses, 1)


def attention_grads_ref(q, k, v, dout, segment_ids=None, causal=True, sm_scale=None, dtype=torch.float32, **mask_kw):
  """(out, dq, dk, dv) by autograd through attention_ref."""
  q = q.detach().to(dtype).requires_grad_(True)
  k = k.detach().to(dtype).requires_grad_(True)
  v = v.detach().to(dtype).requires_grad_(True)
  out, _ = attention_ref(q, k, v, segment_ids, causal, sm_scale, dtype, **mask_kw)
  dq, dk, dv = torch.autograd.grad(out, (q, k, v), dout.to(dtype))
  return out.detach(), dq, dk, dv


# ------------------------------------------------------------------------------------------------
# whole attention blocks — the callers (model/llama/model.py:206-238, 276-279)
# ------------------------------------------------------------------------------------------------
def llama_attention_block(x, w_norm, wq, wk, wv, wo, n_heads, n_kv_heads, eps, theta, attention_mask="causal"):
  """input RMSNorm -> q/k/v projections -> RoPE -> eager attention -> output projection for one
  Llama decoder layer's attention half (model/llama/model.py:276-279, 206-238, 331-360)."""
  B, S, hidden = x.shape
  hd = hidden // n_heads
  h = rms_norm(x, w_norm, eps)
  q = (h @ wq.T).view(B, S, n_heads, hd).transpose(1, 2)
  k = (h @ wk.T).view(B, S, n_kv_heads, hd).transpose(1, 2)
  v = (h @ wv.T).view(B, S, n_kv_heads, hd).transpose(1, 2)
  pos = torch.arange(S)[None].float()
  cos, sin = rotary_cos_sin(llama3_rope_frequencies(hd, theta), pos, x.dtype)
  q, k = apply_rotary_pos_emb(q, k, cos, sin)
  mask = causal_additive_mask(S, x.dtype) if isinstance(attention_mask, str) else attention_mask
  o = eager_attention(q, k, v, mask)
  o = o.transpose(1, 2).contiguous().reshape(B, S, hidden)
  return o @ wo.T


def llama_attention(x, wq, wk, wv, wo, n_heads, n_kv_heads, cos, sin, attention_mask="causal"):
  """``LlamaAttention.forward`` (model/llama/model.py:206-238): q/k/v projections, head split, RoPE with the
  given (batch, seq, dim) tables, eager attention, head merge, output projection."""
  B, S, hidden = x.shape
  hd = hidden // n_heads
  q = (x @ wq.T).view(B, S, n_heads, hd).transpose(1, 2)
  k = (x @ wk.T).view(B, S, n_kv_heads, hd).transpose(1, 2)
  v = (x @ wv.T).view(B, S, n_kv_heads, hd).transpose(1, 2)
  q, k = apply_rotary_pos_emb(q, k, cos, sin)
  mask = causal_additive_mask(S, x.dtype) if isinstance(attention_mask, str) else attention_mask
  o = eager_attention(q, k, v, mask)
  return o.transpose(1, 2).contiguous().reshape(B, S, hidden) @ wo.T


def llama_decoder_layer(x, w, n_heads, n_kv_heads, eps, cos, sin, attention_mask="causal"):
  """``LlamaDecoderLayer.forward`` (model/llama/model.py:276-296): norm, attention, residual add, norm, SwiGLU MLP
  (``down(silu(gate(h)) * up(h))``, :137-139), residual add.  ``w``: weights under the reference's state-dict names."""
  h = rms_norm(x, w["input_layernorm.weight"], eps)
  h = llama_attention(h, w["self_attn.q_proj.weight"], w["self_attn.k_proj.weight"], w["self_attn.v_proj.weight"],
                      w["self_attn.o_proj.weight"], n_heads, n_kv_heads, cos, sin, attention_mask)
  h = x + h
  m = rms_norm(h, w["post_attention_layernorm.weight"], eps)
  m = swiglu(m @ w["mlp.gate_proj.weight"].T, m @ w["mlp.up_proj.weight"].T) @ w["mlp.down_proj.weight"].T
  return h + m


def llama_for_causal_lm(input_ids, labels, w, n_heads, n_kv_heads, eps, rope_theta, rope_scaling=None, attention_mask=None):
  """``LlamaForCausalLM.forward`` (model/llama/model.py:386-400) over ``LlamaModel.forward`` (:333-367): embedding
  lookup, position ids ``arange(S)`` as floats, one rotary table for all layers, the additive causal mask (times the
  padding mask when one is given, :354-355), the decoder layers, the final norm, ``lm_head``, logits in fp32 (or the
  weights' higher precision) and the shifted cross entropy.  ``w``: weights under the reference's state-dict names;
  ``rope_scaling``: the four Llama 3.1 numbers (factor, low_freq_factor, high_freq_factor, original_context_len) or None.
  Returns (logits, loss)."""
  emb = w["model.embed_tokens.weight"]
  x = emb[input_ids]
  B, S, hidden = x.shape
  hd = hidden // n_heads
  inv_freq = default_rope_frequencies(hd, rope_theta) if rope_scaling is None else llama3_rope_frequencies(hd, rope_theta, *rope_scaling)
  cos, sin = rotary_cos_sin(inv_freq, torch.arange(S)[None].float(), torch.float32)
  cos, sin = cos.to(x.dtype), sin.to(x.dtype)
  mask = causal_additive_mask(S, x.dtype)
  if attention_mask is not None:
    mask = mask * attention_mask[:, None, None, :].to(x.dtype)
  n_layers = 1 + max(int(k.split(".")[2]) for k in w if k.startswith("model.layers."))
  for i in range(n_layers):
    pre = f"model.layers.{i}."
    x = llama_decoder_layer(x, {k[len(pre):]: v for k, v in w.items() if k.startswith(pre)}, n_heads, n_kv_heads, eps, cos, sin, mask)
  x = rms_norm(x, w["model.norm.weight"], eps)
  logits = x @ w["lm_head.weight"].T
  if logits.dtype in (torch.bfloat16, torch.float16):
    logits = logits.float()
  if labels is None:
    return logits, None
  return logits, cross_entropy_loss(logits, labels, logits.shape[-1])


def mixtral_attention(x, wq, wk, wv, wo, n_heads, n_kv_heads, rope_theta, max_position_embeddings, position_ids,
                      attention_mask="causal", table_dtype=None, act_dtype=None):
  """``MixtralAttention.forward`` (model/mixtral/model.py:208-243) with its rotary module
  (model/mixtral/model.py:62-103): cos/sin tables of ``max_position_embeddings`` rows cached in the default
  dtype at construction (``table_dtype``), sliced to the sequence, cast to the activations' dtype (``act_dtype``;
  ``x.dtype`` unless the block is being evaluated in higher precision than the model runs in) and gathered by
  ``position_ids`` (model/mixtral/model.py:136-137)."""
  B, S, hidden = x.shape
  hd = hidden // n_heads
  q = (x @ wq.T).view(B, S, n_heads, hd).transpose(1, 2)
  k = (x @ wk.T).view(B, S, n_kv_heads, hd).transpose(1, 2)
  v = (x @ wv.T).view(B, S, n_kv_heads, hd).transpose(1, 2)
  inv_freq = 1.0 / (rope_theta ** (torch.arange(0, hd, 2, dtype=torch.int64).float() / hd))
  t = torch.arange(max(max_position_embeddings, S), dtype=torch.int64).type_as(inv_freq)
  emb = torch.cat((torch.outer(t, inv_freq),) * 2, dim=-1)
  table_dtype = x.dtype if table_dtype is None else table_dtype
  act_dtype = x.dtype if act_dtype is None else act_dtype
  cos = emb.cos().to(table_dtype)[:S].to(act_dtype).to(x.dtype)
  sin = emb.sin().to(table_dtype)[:S].to(act_dtype).to(x.dtype)
  q, k = apply_rotary_pos_emb(q, k, cos, sin, position_ids, gather=True)
  mask = causal_additive_mask(S, x.dtype) if isinstance(attention_mask, str) else attention_mask
  o = eager_attention(q, k, v, mask)
  return o.transpose(1, 2).contiguous().reshape(B, S, hidden) @ wo.T


def deepseek_v3_attention(x, w, n_heads, qk_nope_head_dim, qk_rope_head_dim, v_head_dim, kv_lora_rank, cos, sin,
                          rope_interleave=True, eps=1e-6, attention_mask="causal"):
  """``DeepseekV3Attention.forward`` (model/deepseek_v3/model.py:403-455), multi-headed latent attention.
  ``w`` holds ``q_a_proj, q_a_layernorm, q_b_proj`` (or ``q_proj`` when there is no q latent),
  ``kv_a_proj_with_mqa, kv_a_layernorm, kv_b_proj, o_proj``.  The latent norms use the class default eps 1e-6
  (model/deepseek_v3/model.py:373, 383); the single rotated k head is expanded to every head (:444); the
  softmax scale is 1/sqrt(v_head_dim) because AttentionModule takes it from v (attention.py:54-58)."""
  B, S, _ = x.shape
  qk_head_dim = qk_nope_head_dim + qk_rope_head_dim
  if "q_proj" in w:
    q = x @ w["q_proj"].T
  else:
    q = rms_norm(x @ w["q_a_proj"].T, w["q_a_layernorm"], eps) @ w["q_b_proj"].T
  q = q.view(B, S, -1, qk_head_dim).transpose(1, 2)
  q_pass, q_rot = torch.split(q, [qk_nope_head_dim, qk_rope_head_dim], dim=-1)
  ckv = x @ w["kv_a_proj_with_mqa"].T
  k_pass, k_rot = torch.split(ckv, [kv_lora_rank, qk_rope_head_dim], dim=-1)
  k_pass = (rms_norm(k_pass, w["kv_a_layernorm"], eps) @ w["kv_b_proj"].T).view(B, S, -1, qk_nope_head_dim + v_head_dim).transpose(1, 2)
  k_pass, v = torch.split(k_pass, [qk_nope_head_dim, v_head_dim], dim=-1)
  k_rot = k_rot.view(B, 1, S, qk_rope_head_dim)
  if rope_interleave:
    q_rot, k_rot = apply_rotary_pos_emb_interleave(q_rot, k_rot, cos, sin)
  else:
    q_rot, k_rot = apply_rotary_pos_emb(q_rot, k_rot, cos, sin)
  k_rot = k_rot.expand(*k_pass.shape[:-1], -1)
  q = torch.cat((q_pass, q_rot), dim=-1)
  k = torch.cat((k_pass, k_rot), dim=-1)
  mask = causal_additive_mask(S, x.dtype) if isinstance(attention_mask, str) else attention_mask
  o = eager_attention(q, k, v, mask)
  return o.transpose(1, 2).contiguous().reshape(B, S, -1) @ w["o_proj"].T


# ------------------------------------------------------------------------------------------------
# the steps either side of the attention path
# ------------------------------------------------------------------------------------------------
def add_rms_norm(x, residual, weight, eps):
  """model/llama/model.py:288-291: ``h = residual + x`` (in the activation dtype), then ``rms_norm(h)``;
  returns ``(y, h)``."""
  h = residual + x
  return rms_norm(h, weight, eps), h


def l2_norm(x, eps):
  """Llama4TextL2Norm.forward, model/llama4/model.py:104-116."""
  xf = x.float() if x.dtype != torch.float64 else x
  return (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)).type_as(x)


def apply_rotary_emb_llama4(q, k, cos_full, sin_full, unsqueeze_dim=2):
  """apply_rotary_emb, model/llama4/model.py:364-409: q, k (B, S, N, D); pairs (x[2i], x[2i+1]) rotated by the
  angle whose cos/sin are entry i of the (B, S, D) tables; results interleaved back."""
  hd = q.size(-1)
  c = cos_full.unsqueeze(unsqueeze_dim)[..., : hd // 2]
  s = sin_full.unsqueeze(unsqueeze_dim)[..., : hd // 2]

  def rot(t):
    x, y = t[..., ::2], t[..., 1::2]
    xo, yo = x * c - y * s, y * c + x * s
    return torch.stack([xo, yo], dim=-1).reshape(t.shape).type_as(t)

  return rot(q), rot(k)


def attn_temperature_scales(seq_len, floor_scale, attn_scale):
  """model/llama4/model.py:515-521."""
  pos = torch.arange(seq_len).float()
  return torch.log(torch.floor((pos + 1.0) / floor_scale) + 1.0) * attn_scale + 1.0


def apply_attn_temperature(q, floor_scale, attn_scale):
  """model/llama4/model.py:522-525: q (B, S, N, D) times the per-position scale, cast back to q's dtype."""
  sc = attn_temperature_scales(q.shape[1], floor_scale, attn_scale).view(1, -1, 1, 1)
  return (q * (sc.double() if q.dtype == torch.float64 else sc)).to(q.dtype)


def llama4_attention(x, wq, wk, wv, wo, n_heads, n_kv_heads, cos, sin, use_rope, use_qk_norm, eps,
                     attn_temperature_tuning, floor_scale, attn_scale, attention_mask="causal"):
  """``Llama4TextAttention.forward`` (model/llama4/model.py:489-533): projections viewed (B, S, N, D); on rotary layers
  the adjacent-pair rotation and, with ``use_qk_norm``, the weightless L2 norm of q and k; on the others the attention
  temperature on q; then eager attention, head merge, output projection."""
  B, S, hidden = x.shape
  hd = hidden // n_heads
  q = (x @ wq.T).view(B, S, n_heads, hd)
  k = (x @ wk.T).view(B, S, n_kv_heads, hd)
  v = (x @ wv.T).view(B, S, n_kv_heads, hd).transpose(1, 2)
  if use_rope:
    q, k = apply_rotary_emb_llama4(q, k, cos, sin)
    if use_qk_norm:
      q, k = l2_norm(q, eps), l2_norm(k, eps)
  if attn_temperature_tuning and not use_rope:
    q = apply_attn_temperature(q, floor_scale, attn_scale)
  mask = causal_additive_mask(S, x.dtype) if isinstance(attention_mask, str) else attention_mask
  o = eager_attention(q.transpose(1, 2), k.transpose(1, 2), v, mask)
  return o.transpose(1, 2).contiguous().reshape(B, S, hidden) @ wo.T


def swiglu(gate, up):
  """``act_fn(gate_proj(x)) * up_proj(x)`` of LlamaMLP.forward (model/llama/model.py:137-139), act_fn = SiLU."""
  return F.silu(gate) * up


def cross_entropy_loss(logits, labels, vocab_size):
  """loss.py:5-20."""
  shift_logits = logits[..., :-1, :].contiguous().view(-1, vocab_size)
  shift_labels = labels[..., 1:].contiguous().view(-1)
  return torch.nn.CrossEntropyLoss()(shift_logits, shift_labels)
