"""RMSNorm modules with the reference's constructor, parameter and attribute names.

Drop-in for LlamaRMSNorm (torchprime/torch_xla_models/model/llama/model.py:38-52), MixtralRMSNorm
(model/mixtral/model.py:44-59) and DeepseekV3RMSNorm (model/deepseek_v3/model.py:32-44); the three
bodies are identical there, so they share one implementation here.  ``forward`` is one HIP kernel
(``tprime::rmsnorm_fwd``) instead of five eager ops; the backward is ``tprime::rmsnorm_bwd``.
"""

from __future__ import annotations

import torch
from torch import nn

from . import ops


class _RMSNorm(nn.Module):
  def __init__(self, hidden_size, eps=1e-6):
    super().__init__()
    self.weight = nn.Parameter(torch.ones(hidden_size))
    self.variance_epsilon = eps

  def forward(self, hidden_states: torch.Tensor) -> torch.Tensor:
    return ops.rmsnorm(hidden_states, self.weight, self.variance_epsilon)

  def extra_repr(self) -> str:
    return f"{tuple(self.weight.shape)}, eps={self.variance_epsilon}"


def add_rms_norm(hidden_states: torch.Tensor, residual: torch.Tensor, norm: "_RMSNorm"):
  """The residual add and the norm after it of a decoder layer (model/llama/model.py:288-291) in one pass:
  returns ``(norm(residual + hidden_states), residual + hidden_states)``; the second value is the next residual."""
  return ops.add_rmsnorm(hidden_states, residual, norm.weight, norm.variance_epsilon)


class LlamaRMSNorm(_RMSNorm):
  """LlamaRMSNorm is equivalent to T5LayerNorm (model/llama/model.py:38-52)."""


class MixtralRMSNorm(_RMSNorm):
  """model/mixtral/model.py:44-59."""


class DeepseekV3RMSNorm(_RMSNorm):
  """model/deepseek_v3/model.py:32-44."""
