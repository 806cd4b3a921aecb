"""Rotary-embedding modules and apply functions with the reference's names and signatures.

* LlamaRotaryEmbedding        torchprime/torch_xla_models/model/llama/model.py:55-88
* MixtralRotaryEmbedding      model/mixtral/model.py:62-103
* DeepseekV3RotaryEmbedding   model/deepseek_v3/model.py:47-75
* rotate_half                 model/llama/model.py:91-95
* apply_rotary_pos_emb        model/llama/model.py:98-122 (position_ids unused) and
                              model/mixtral/model.py:115-140 (cos/sin tables gathered by position_ids)
* apply_rotary_pos_emb_interleave   model/deepseek_v3/model.py:84-103

The per-step work is two HIP kernels: ``tprime::rope_table`` (cos/sin) and ``tprime::rope_apply``
(q and k rotated in one launch, differentiable).
"""

from __future__ import annotations

import torch
from torch import nn

from . import _lib, ops
from .rope import RopeScaling, deepseek_v3_rope_init_fn, llama3_rope_frequencies


class _Fp32Frequencies(nn.Module):
  """``inv_freq`` stays fp32 whatever the module is cast to.  The reference builds its models under a default dtype
  and never casts them, so its fp32 buffer (rope/rope.py:25-39 ends in ``.float()``) is never rounded; a
  ``model.to(torch.bfloat16)`` would round the frequencies to 8 bits and turn the angles at a few hundred positions
  wrong by several percent.  Device moves apply as usual."""

  def _apply(self, fn, recurse=True):
    kept = self.inv_freq
    super()._apply(fn, recurse)
    if self.inv_freq.dtype != kept.dtype:
      self.inv_freq = kept.to(self.inv_freq.device)
    return self


class LlamaRotaryEmbedding(_Fp32Frequencies):
  inv_freq: torch.Tensor

  def __init__(self, head_dim, rope_theta, scaling: RopeScaling | None = None):
    super().__init__()
    inv_freq = llama3_rope_frequencies(head_dim, theta=rope_theta, scaling=scaling)
    self.register_buffer("inv_freq", inv_freq, persistent=False)

  @torch.no_grad()
  def forward(self, x, position_ids):
    # x: [bs, num_attention_heads, seq_len, head_size]; position_ids: (bs or 1, seq_len), float in the models
    _lib.require_gpu(x, position_ids)
    return ops.rope_table(self.inv_freq, position_ids, 1.0, x.dtype)


class DeepseekV3RotaryEmbedding(_Fp32Frequencies):
  inv_freq: torch.Tensor

  def __init__(self, config):
    super().__init__()
    self.config = config
    inv_freq, self.attention_scaling = deepseek_v3_rope_init_fn(self.config)
    self.register_buffer("inv_freq", inv_freq.to(torch.float32), persistent=False)
    self.original_inv_freq = self.inv_freq

  @torch.no_grad()
  def forward(self, x: torch.Tensor, position_ids: torch.Tensor):
    _lib.require_gpu(x, position_ids)
    return ops.rope_table(self.inv_freq, position_ids, float(self.attention_scaling), x.dtype)


class MixtralRotaryEmbedding(nn.Module):
  """cos/sin cached up to ``max_position_embeddings`` in the default dtype at construction and
  sliced per call (model/mixtral/model.py:62-103)."""

  def __init__(self, dim, max_position_embeddings=2048, base=10000, device=None):
    super().__init__()
    self.dim = dim
    self.max_position_embeddings = max_position_embeddings
    self.base = base
    inv_freq = 1.0 / (self.base ** (torch.arange(0, self.dim, 2, dtype=torch.int64).float().to(device) / self.dim))
    self.register_buffer("inv_freq", inv_freq, persistent=False)
    # The reference fills the cache here, from the fp32 frequencies, before any ``module.to(dtype)`` can round the
    # ``inv_freq`` buffer.  This build fills it on the first GPU call, so it keeps the fp32 values out of reach of
    # ``.to()`` (a plain attribute, not a buffer).
    self._inv_freq_fp32 = inv_freq.detach().clone().float()
    self._cache_dtype = torch.get_default_dtype()
    self.max_seq_len_cached = 0
    self.register_buffer("cos_cached", torch.empty(0), persistent=False)
    self.register_buffer("sin_cached", torch.empty(0), persistent=False)

  def _set_cos_sin_cache(self, seq_len, device, dtype):
    self.max_seq_len_cached = seq_len
    t = torch.arange(seq_len, device=device, dtype=torch.int64).float()[None]
    cos, sin = ops.rope_table(self._inv_freq_fp32.to(device), t, 1.0, dtype)
    self.cos_cached, self.sin_cached = cos[0], sin[0]

  def forward(self, x, seq_len=None):
    # x: [bs, num_attention_heads, seq_len, head_size]
    _lib.require_gpu(x)
    if self.max_seq_len_cached == 0 or self.cos_cached.device != x.device:
      # the reference fills the cache in __init__ on the construction device; the table kernel is
      # GPU-only, so the first call on the GPU fills it (same values, same dtype)
      self._set_cos_sin_cache(max(self.max_position_embeddings, seq_len or 0), x.device, self._cache_dtype)
    if seq_len > self.max_seq_len_cached:
      self._set_cos_sin_cache(seq_len=seq_len, device=x.device, dtype=x.dtype)
    return self.cos_cached[:seq_len].to(dtype=x.dtype), self.sin_cached[:seq_len].to(dtype=x.dtype)


def rotate_half(x):
  """Rotates half the hidden dims of the input (pure data movement; kept for API parity)."""
  half = x.shape[-1] // 2
  return torch.cat((-x[..., half:], x[..., :half]), dim=-1)


def _heads_first(t, unsqueeze_dim):
  if unsqueeze_dim == 1:
    return t
  if unsqueeze_dim == 2:  # (B,S,H,D) tensors: present them as (B,H,S,D) views
    return t.transpose(1, 2)
  raise ValueError(f"unsqueeze_dim must be 1 or 2, got {unsqueeze_dim}")


def apply_rotary_pos_emb(q, k, cos, sin, position_ids=None, unsqueeze_dim=1):
  """``q*cos + rotate_half(q)*sin`` and the same for k.

  With 3-D ``cos``/``sin`` (batch, seq, dim) this is the Llama form and ``position_ids`` is unused
  (model/llama/model.py:98-122).  With 2-D tables (max_pos, dim) it is the Mixtral form and the rows
  are gathered by ``position_ids.long()`` first (model/mixtral/model.py:136-137).
  """
  qh, kh = _heads_first(q, unsqueeze_dim), _heads_first(k, unsqueeze_dim)
  if cos.dim() == 2:
    if position_ids is None:
      raise ValueError("2-D cos/sin tables need position_ids to gather rows")
    qo, ko = ops.rope_apply(qh, kh, cos, sin, position_ids.long(), False)
  else:
    qo, ko = ops.rope_apply(qh, kh, cos, sin, None, False)
  return _heads_first(qo, unsqueeze_dim), _heads_first(ko, unsqueeze_dim)


def apply_rotary_pos_emb_interleave(q, k, cos, sin, position_ids=None, unsqueeze_dim=1):
  """DeepSeek form: de-interleave ``[x0,x1,x2,..] -> [evens | odds]`` then rotate-half; the outputs
  stay in the de-interleaved order, as in the reference (model/deepseek_v3/model.py:84-103)."""
  qh, kh = _heads_first(q, unsqueeze_dim), _heads_first(k, unsqueeze_dim)
  qo, ko = ops.rope_apply(qh, kh, cos, sin, None, True)
  return _heads_first(qo, unsqueeze_dim), _heads_first(ko, unsqueeze_dim)
