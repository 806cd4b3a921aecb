"""RoPE inverse-frequency tables; mirrors ``torchprime.rope.rope`` (torchprime/rope/rope.py).

These run once at module construction on the host, exactly as in the reference; the per-step work
(cos/sin tables, rotation of q and k) is in :mod:`torchprime_amd.rotary` on the GPU.

``deepseek_v3_rope_init_fn`` accepts any config object with attribute access whose
``rope_scaling`` is a mapping (OmegaConf ``DictConfig``, ``dict`` or :class:`Config`); the reference
asserts ``isinstance(config.rope_scaling, DictConfig)`` (rope/rope.py:94), which this build relaxes to
"is a mapping" because omegaconf is not a dependency here.
"""

from __future__ import annotations

import math
from collections.abc import Mapping
from dataclasses import dataclass

import torch


@dataclass(kw_only=True)
class RopeScaling:
  """RoPE scaling parameters; the defaults are the Llama 3.1 values (rope/rope.py:13-22)."""

  factor: float = 8.0
  low_freq_factor: float = 1.0
  high_freq_factor: float = 4.0
  original_context_len: int = 8192


def default_rope_frequencies(head_dim: int, theta: float = 10000.0) -> torch.Tensor:
  """Original RoPE frequencies ``theta ** -(2i / head_dim)`` (rope/rope.py:25-39)."""
  exponent = torch.arange(0, head_dim, 2, dtype=torch.int64).float() / head_dim
  return 1.0 / (theta**exponent)


def llama3_rope_frequencies(head_dim: int, theta: float = 10000.0, scaling: RopeScaling | None = None) -> torch.Tensor:
  """Llama 3 / 3.1 frequencies: long wavelengths are divided by ``factor``, short ones kept, the
  band in between blended smoothly (rope/rope.py:42-75)."""
  freqs = default_rope_frequencies(head_dim=head_dim, theta=theta)
  if scaling is None:
    return freqs
  ctx = scaling.original_context_len
  low_freq_wavelen = ctx / scaling.low_freq_factor
  high_freq_wavelen = ctx / scaling.high_freq_factor
  assert low_freq_wavelen >= high_freq_wavelen, (
    f"low_freq_wavelen {low_freq_wavelen} must be greater or equal to high_freq_wavelen {high_freq_wavelen}"
  )
  wavelen = 2 * math.pi / freqs
  long_wave = wavelen > low_freq_wavelen
  short_wave = wavelen < high_freq_wavelen
  scaled = torch.where(long_wave, freqs / scaling.factor, freqs)
  smooth = (ctx / wavelen - scaling.low_freq_factor) / (scaling.high_freq_factor - scaling.low_freq_factor)
  blended = (1 - smooth) * scaled / scaling.factor + smooth * scaled
  return torch.where(~short_wave & ~long_wave, blended, scaled)


def _get(mapping, key, default=None):
  return mapping.get(key, default) if hasattr(mapping, "get") else getattr(mapping, key, default)


def deepseek_v3_rope_init_fn(config) -> tuple[torch.Tensor, float]:
  """YaRN inverse frequencies and the cos/sin post-scale ("attention factor") (rope/rope.py:78-177)."""
  rs = getattr(config, "rope_scaling", None)
  assert rs is not None and (isinstance(rs, Mapping) or hasattr(rs, "get")), "config.rope_scaling must be a mapping"
  assert _get(rs, "rope_type", _get(rs, "type")) == "yarn"
  base = config.rope_theta
  partial_rotary_factor = config.partial_rotary_factor if hasattr(config, "partial_rotary_factor") else 1.0
  head_dim = getattr(config, "head_dim", None)
  if head_dim is None:
    head_dim = config.hidden_size // config.num_attention_heads
  dim = int(head_dim * partial_rotary_factor)
  factor = rs["factor"]
  attention_factor = _get(rs, "attention_factor")
  mscale = _get(rs, "mscale")
  mscale_all_dim = _get(rs, "mscale_all_dim")

  # DeepSeek-V3 keeps the pretrained length in `original_max_position_embeddings` and derives the
  # scaling factor from the ratio of the two lengths instead of `factor`.
  if "original_max_position_embeddings" in rs:
    original_max = rs["original_max_position_embeddings"]
    factor = config.max_position_embeddings / original_max
  else:
    original_max = config.max_position_embeddings

  def get_mscale(scale, m=1):
    return 1.0 if scale <= 1 else 0.1 * m * math.log(scale) + 1.0

  if attention_factor is None:
    if mscale and mscale_all_dim:
      attention_factor = float(get_mscale(factor, mscale) / get_mscale(factor, mscale_all_dim))
    else:
      attention_factor = get_mscale(factor)

  beta_fast = _get(rs, "beta_fast") or 32
  beta_slow = _get(rs, "beta_slow") or 1

  def correction_dim(num_rotations):
    # dimension whose wavelength makes `num_rotations` turns over the original context
    return (dim * math.log(original_max / (num_rotations * 2 * math.pi))) / (2 * math.log(base))

  low = max(math.floor(correction_dim(beta_fast)), 0)
  high = min(math.ceil(correction_dim(beta_slow)), dim - 1)
  if low == high:
    high += 0.001  # avoid a zero-width ramp

  pos_freqs = base ** (torch.arange(0, dim, 2).to(dtype=torch.float) / dim)
  extrapolation = 1.0 / pos_freqs
  interpolation = 1.0 / (factor * pos_freqs)
  ramp = torch.clamp((torch.arange(dim // 2, dtype=torch.float32) - low) / (high - low), 0, 1)
  keep = 1 - ramp  # 1 where the original (extrapolated) frequency is kept
  inv_freq = interpolation * (1 - keep) + extrapolation * keep
  return inv_freq, attention_factor
