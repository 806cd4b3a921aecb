"""Drop-in for ``torchprime.torch_xla_models.attention`` on one MI355X.

``AttentionModule`` keeps the reference's constructor, attributes, forward signature, shape checks
and softmax scale (torchprime/torch_xla_models/attention.py:32-177).  Where the reference dispatches
to a TPU Pallas kernel (splash :70-123, flash :124-150) or materialises the (B,H,S,S) logits
(eager :151-170), this module calls one HIP kernel pair (``tprime::attn_fwd`` / ``tprime::attn_bwd``)
with native GQA, so K/V are never expanded by ``repeat_kv``.  Mesh and partition specs do not exist
on a single GPU: they are accepted and ignored.
"""

from __future__ import annotations

import math
import weakref
from typing import Any

import torch
from torch import nn

from . import kernel_utils, ops, parallelism_utils
from .config import has_key


def repeat_kv(hidden_states: torch.Tensor, n_rep: int) -> torch.Tensor:
  """(batch, kv_heads, seq, dim) -> (batch, kv_heads * n_rep, seq, dim), each head repeated n_rep
  times in place (``torch.repeat_interleave(x, n_rep, dim=1)``); attention.py:18-29.  The kernels
  index kv head ``h // n_rep`` instead and never call this; it is exported for API parity."""
  if n_rep == 1:
    return hidden_states
  b, h, s, d = hidden_states.shape
  return hidden_states.unsqueeze(2).expand(b, h, n_rep, s, d).reshape(b, h * n_rep, s, d)


def _is_causal_additive_mask(mask: torch.Tensor, q_len: int, kv_len: int) -> bool:
  """True when ``mask[..., :kv_len]`` is 0 on and below the diagonal and -inf above it, the mask the
  models build at model/llama/model.py:347-355."""
  if mask.dim() != 4 or mask.shape[1] != 1 or mask.shape[2] != q_len or mask.shape[3] < kv_len:
    return False
  m = mask[:, :, :, :kv_len]
  keep = torch.ones((q_len, kv_len), dtype=torch.bool, device=mask.device).tril()
  ok = ((m == 0) == keep) & ((m == float("-inf")) == ~keep)
  return bool(ok.all())


# Verdicts of the check above, kept per mask tensor object (a weak reference and the tensor's version counter).  A
# model builds its mask once per forward and hands the same tensor to every layer, so the (S x S) compare and its
# host sync run once per mask rather than once per layer.  The key is the object, never its address: a mask built
# for the next forward is a new tensor that the caching allocator may well place where the last one was.
# ``kernel_config={"assume_causal_mask": True}`` skips the check altogether.
_MASK_VERDICTS: dict = {}


def _causal_mask_verdict(mask: torch.Tensor, q_len: int, kv_len: int) -> bool:
  ident = id(mask)
  key = (mask._version, tuple(mask.shape), q_len, kv_len)
  entry = _MASK_VERDICTS.get(ident)
  if entry is not None and entry[0]() is mask and entry[1] == key:
    return entry[2]
  verdict = _is_causal_additive_mask(mask, q_len, kv_len)
  # the entry leaves with the tensor (its id may be reused afterwards, hence also the identity check above)
  ref = weakref.ref(mask, lambda _r, ident=ident: _MASK_VERDICTS.pop(ident, None))
  _MASK_VERDICTS[ident] = (ref, key, verdict)
  return verdict


class AttentionModule(nn.Module):
  def __init__(self, config, kernel_config: dict[str, Any] | None = None):
    super().__init__()
    self.config = config
    self.kernel_config = kernel_config
    self.partition_spec = None

  def forward(
    self,
    query_states: torch.Tensor,  # (batch_size, num_heads, q_len, head_dim)
    key_states: torch.Tensor,  # (batch_size, num_kv_heads, kv_len, head_dim)
    value_states: torch.Tensor,  # (batch_size, num_kv_heads, kv_len, head_dim)
    attention_mask: torch.Tensor | None = None,
  ):
    kernel = self.config.attention_kernel
    bsz, num_heads, q_len, _ = query_states.size()
    # the reference scales by, and checks the output against, v's head dim (attention.py:54-58)
    head_dim = value_states.shape[-1]
    kv_seq_len = key_states.shape[-2]
    self.partition_spec = None  # no mesh on one GPU (attention.py:61-67)

    if kernel == "splash_attention" and has_key(self.config, "load_balance_cp") and self.config.load_balance_cp:
      # Load-balanced context parallelism (attention.py:75-119), the part one GPU sees: the sequence arrives in the
      # striped order, K / V are put back into the original order, and a causal mask whose query rows are in the
      # striped order (LoadBalancedCausalMask) relates the two.  The kernel evaluates that mask from q_sequence.
      cp_size = self.config.context
      key_states = parallelism_utils.reorder_sequence(tensor=key_states, cp_size=cp_size, seq_dim=2, to_contiguous=True)
      value_states = parallelism_utils.reorder_sequence(tensor=value_states, cp_size=cp_size, seq_dim=2, to_contiguous=True)
      custom_mask = parallelism_utils.LoadBalancedCausalMask(shape=(q_len, q_len), cp_size=cp_size)
      attn_output = kernel_utils.tpu_splash_attention_jax_call_wrapper(
        mask=custom_mask, query=query_states, key=key_states, value=value_states, config=None, decoder_segment_ids=None,
        causal=False, q_seq_shards=cp_size, sm_scale=1.0 / math.sqrt(head_dim),
      )[0]  # fmt: skip
      if attn_output.size() != (bsz, num_heads, q_len, head_dim):
        raise ValueError(
          f"`attn_output` should be of size {(bsz, num_heads, q_len, head_dim)}, but is {attn_output.size()}"
        )
      return attn_output

    if kernel in ("splash_attention", "flash_attention"):
      # both kernel branches are causal and never see attention_mask (attention.py:121-123, 144-150)
      causal = True
    else:
      # eager branch: softmax(QK^T/sqrt(d) + mask); no mask means full attention (attention.py:151-170)
      p = getattr(self.config, "attention_dropout", 0.0)
      if p and self.training:
        raise NotImplementedError("attention_dropout > 0 is not supported (every shipped config uses 0)")
      bias = None
      if attention_mask is None:
        causal = False
      else:
        assume = bool(self.kernel_config and self.kernel_config.get("assume_causal_mask"))
        causal = assume or _causal_mask_verdict(attention_mask, q_len, kv_seq_len)
        if not causal:
          # any other mask is added to the scaled logits as it is (attention.py:153-158); the causal one, which
          # the models build, takes the kernels that skip the tiles above the diagonal instead
          if attention_mask.dim() != 4 or attention_mask.shape[-1] < kv_seq_len:
            raise ValueError(
              f"attention_mask must be 4-D with at least {kv_seq_len} keys, got {tuple(attention_mask.shape)}"
            )
          bias = attention_mask[:, :, :, :kv_seq_len]
      if bias is not None:
        attn_output = ops.attention(
          query_states, key_states, value_states, None, 1.0 / math.sqrt(head_dim), False, bias=bias
        )
        if attn_output.size() != (bsz, num_heads, q_len, head_dim):
          raise ValueError(
            f"`attn_output` should be of size {(bsz, num_heads, q_len, head_dim)}, but is {attn_output.size()}"
          )
        return attn_output

    attn_output = ops.attention(
      query_states, key_states, value_states, None, 1.0 / math.sqrt(head_dim), causal
    )

    if attn_output.size() != (bsz, num_heads, q_len, head_dim):
      raise ValueError(
        f"`attn_output` should be of size {(bsz, num_heads, q_len, head_dim)}, but is {attn_output.size()}"
      )
    return attn_output
