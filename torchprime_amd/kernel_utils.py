"""Drop-in for ``torchprime.utils.kernel_utils``: the functional splash-attention entry point with
``decoder_segment_ids`` (torchprime/utils/kernel_utils.py:28-131, 134-329), served by the HIP
attention kernels.  Unlike the reference's wrapper, which is forward-only (:124-131), the result is
differentiable.
"""

from __future__ import annotations

import json
from dataclasses import asdict, dataclass, field

import torch

from . import ops
from .parallelism_utils import LoadBalancedCausalMask

# q_sequence arrays as device tensors, one per (mask, device): the mask object is rebuilt every layer call
# (attention.py:92-96) but equal masks hash equal
_QSEQ_CACHE: dict = {}


def _q_positions(mask: LoadBalancedCausalMask, device) -> torch.Tensor:
  key = (mask, str(device))
  t = _QSEQ_CACHE.get(key)
  if t is None:
    if len(_QSEQ_CACHE) > 16:
      _QSEQ_CACHE.clear()
    t = _QSEQ_CACHE[key] = torch.from_numpy(mask.q_sequence.astype("int32")).to(device)
  return t


@dataclass
class SplashAttentionConfig:
  """Fields the reference reads from ``torch_xla.experimental.splash_attention.SplashAttentionConfig``
  (kernel_utils.py:224-235, 266-270; attention.py:98-106).  Block sizes, layouts, mesh and partition
  specs steer the TPU kernel and the SPMD partitioner; here they are carried and ignored."""

  mesh: str | None = None
  qkv_partition_spec: tuple = (("data", "fsdp"), "tensor", None, None)
  segment_ids_partition_spec: tuple = (("data", "fsdp"), None)
  sa_block_q: int = 2048
  sa_block_kv: int = 512
  sa_block_kv_compute: int = 512
  sa_block_q_dkv: int = 2048
  sa_block_kv_dkv: int = 512
  sa_block_kv_dkv_compute: int = 512
  sa_block_q_dq: int = 2048
  sa_block_kv_dq: int = 512
  sa_use_fused_bwd_kernel: bool = True
  sa_q_layout: str = "HEAD_DIM_MINOR"
  sa_k_layout: str = "HEAD_DIM_MINOR"
  sa_v_layout: str = "HEAD_DIM_MINOR"
  attentiontype_local_sliding: bool = False
  slide_window_size: int | None = None
  extra: dict = field(default_factory=dict)

  def to_json(self) -> str:
    return json.dumps(asdict(self))

  @classmethod
  def from_json(cls, s: str) -> "SplashAttentionConfig":
    d = json.loads(s) if s else {}
    known = {k: d.pop(k) for k in list(d) if k in cls.__dataclass_fields__ and k != "extra"}
    return cls(**known, extra=d)


def splash_attention_jax_wrapper(
  mask, query, key, value, decoder_segment_ids, causal: bool, config, attn_logits_soft_cap, q_seq_shards, sm_scale=None
):
  """Mask composition of kernel_utils.py:215-220, 238-241, 259-278: (causal | full) AND same-segment.
  ``query`` is expected pre-scaled like the reference's callers do (attention.py:107), so
  ``sm_scale=None`` means 1.0."""
  q_positions, causal_offset = None, 0
  if mask is not None:
    # the one custom mask the reference builds (attention.py:92-96); it replaces the causal / full choice
    # (kernel_utils.py:259-263 only builds one when mask is None)
    if not isinstance(mask, LoadBalancedCausalMask):
      raise NotImplementedError(f"mask objects of type {type(mask).__name__} are not supported (LoadBalancedCausalMask is)")
    if tuple(mask.shape) != (query.shape[2], key.shape[2]):
      raise ValueError(f"mask shape {tuple(mask.shape)} does not match (q_len, kv_len) = {(query.shape[2], key.shape[2])}")
    q_positions, causal_offset, causal = _q_positions(mask, query.device), int(mask.offset), True
  if isinstance(config, str):
    config = SplashAttentionConfig.from_json(config)
  window = None
  if config is not None and getattr(config, "attentiontype_local_sliding", False):
    if getattr(config, "slide_window_size", None) is None:
      raise ValueError("Sliding_window_size must be set if Local Sliding attention type")
    # LocalMask(window_size=(w, w), offset=0) ANDed into the mask (kernel_utils.py:266-275)
    window = (int(config.slide_window_size), int(config.slide_window_size))
  if decoder_segment_ids is not None and not tuple(decoder_segment_ids.shape):
    decoder_segment_ids = None
  if decoder_segment_ids is not None:
    assert query.shape[2] == decoder_segment_ids.shape[1], (
      "Sharding along sequence dimension not allowed in tpu kernel attention"
    )
  return ops.attention(
    query, key, value, decoder_segment_ids, 1.0 if sm_scale is None else float(sm_scale), bool(causal),
    window=window, soft_cap=attn_logits_soft_cap, q_positions=q_positions, causal_offset=causal_offset,
  )


def tpu_splash_attention_jax_call_wrapper(
  mask,
  query: torch.Tensor,
  key: torch.Tensor,
  value: torch.Tensor,
  config: str,
  decoder_segment_ids: torch.Tensor | None,
  causal: bool,
  attn_logits_soft_cap: float | None = None,
  is_forward: bool = True,
  q_seq_shards: int = 1,
  grad_output: torch.Tensor | None = None,
  sm_scale: float | None = None,
) -> tuple[torch.Tensor, torch.Tensor | None, torch.Tensor | None]:
  """Same arguments and 3-tuple result as kernel_utils.py:29-41; ``config`` (JSON), ``q_seq_shards``
  and ``grad_output`` are accepted and ignored.  ``sm_scale`` is this build's addition."""
  if not is_forward:
    return None  # the reference returns nothing for is_forward=False (kernel_utils.py:129-131)
  out = splash_attention_jax_wrapper(
    mask, query, key, value, decoder_segment_ids, causal, config, attn_logits_soft_cap, q_seq_shards, sm_scale
  )
  return (out, None, None)
