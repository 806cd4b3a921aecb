"""LlamaMLP (torchprime/torch_xla_models/model/llama/model.py:125-139) with the activation and the gate product in
one HIP kernel (``tprime::swiglu_fwd``); the three projections stay stock ``nn.Linear`` GEMMs."""

from __future__ import annotations

from torch import nn

from . import ops


class LlamaMLP(nn.Module):
  def __init__(self, config):
    super().__init__()
    self.config = config
    self.hidden_size = config.hidden_size
    self.intermediate_size = config.intermediate_size
    self.gate_proj = nn.Linear(self.hidden_size, self.intermediate_size, bias=False)
    self.up_proj = nn.Linear(self.hidden_size, self.intermediate_size, bias=False)
    self.down_proj = nn.Linear(self.intermediate_size, self.hidden_size, bias=False)
    act = getattr(config, "hidden_act", "silu")
    if act not in ("silu", "swish"):
      raise NotImplementedError(f"hidden_act={act!r}: the fused kernel implements SiLU (every shipped Llama config uses it)")

  def forward(self, x):
    return self.down_proj(ops.swiglu(self.gate_proj(x), self.up_proj(x)))
