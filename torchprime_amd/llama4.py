"""Llama-4 variants of the attention path's element-wise steps, with the reference's names and signatures
(torchprime/torch_xla_models/model/llama4/model.py):

* Llama4TextL2Norm            :104-116   weightless RMSNorm on q / k ("qk_norm"), one HIP kernel
* Llama4TextRotaryEmbedding   :324-351   cos/sin tables, same kernel as the Llama module's
* apply_rotary_emb            :364-409   adjacent-pair rotation on (B, S, N, D) tensors, output in place order
* attn_temperature_scales / apply_attn_temperature   :513-525   per-position query scale of the NoPE layers
"""

from __future__ import annotations

import torch
from torch import nn

from . import _lib, ops
from .rope import RopeScaling, llama3_rope_frequencies


class Llama4TextL2Norm(nn.Module):
  def __init__(self, eps: float = 1e-6):
    super().__init__()
    self.eps = eps

  def forward(self, x):
    return ops.l2norm(x, self.eps)

  def extra_repr(self):
    return f"eps={self.eps}"


class Llama4TextRotaryEmbedding(nn.Module):
  inv_freq: torch.Tensor

  def __init__(self, head_dim, rope_theta, scaling: RopeScaling | None = None):
    super().__init__()
    inv_freq = llama3_rope_frequencies(head_dim, theta=rope_theta, scaling=scaling)
    self.register_buffer("inv_freq", inv_freq, persistent=False)

  @torch.no_grad()
  def forward(self, x, position_ids):
    _lib.require_gpu(x, position_ids)
    return ops.rope_table(self.inv_freq, position_ids, 1.0, x.dtype)


def apply_rotary_emb(q, k, freqs_cos_sin, unsqueeze_dim: int = 2):
  """``q``/``k`` (B, S, N, D), cos/sin (B, S, D) whose first D/2 entries are the angles' cos/sin: pair
  ``(x[2i], x[2i+1])`` becomes ``(x cos_i - y sin_i, y cos_i + x sin_i)``, each product and the sum rounded to the
  tensor dtype as the eager expression does, results written back interleaved."""
  cos, sin = freqs_cos_sin
  if unsqueeze_dim == 2:
    qh, kh = q.transpose(1, 2), k.transpose(1, 2)  # (B, N, S, D) views of (B, S, N, D) memory
  elif unsqueeze_dim == 1:
    qh, kh = q, k
  else:
    raise ValueError(f"unsqueeze_dim must be 1 or 2, got {unsqueeze_dim}")
  qo, ko = ops.rope_apply(qh, kh, cos, sin, None, 2)
  if unsqueeze_dim == 2:
    qo, ko = qo.transpose(1, 2), ko.transpose(1, 2)
  return qo.type_as(q), ko.type_as(k)


def attn_temperature_scales(seq_len: int, floor_scale: float, attn_scale: float, device=None) -> torch.Tensor:
  """``log(floor((pos + 1) / floor_scale) + 1) * attn_scale + 1`` for pos = 0..seq_len-1, fp32 (tiny: host-side torch)."""
  pos = torch.arange(seq_len, device=device).float()
  return torch.log(torch.floor((pos + 1.0) / floor_scale) + 1.0) * attn_scale + 1.0


def apply_attn_temperature(query_states: torch.Tensor, floor_scale: float, attn_scale: float) -> torch.Tensor:
  """``(query_states * attn_scales).to(query_states.dtype)`` for (B, S, N, D) queries, one pass."""
  scales = attn_temperature_scales(query_states.shape[1], floor_scale, attn_scale, query_states.device)
  return ops.scale_rows(query_states, scales)
