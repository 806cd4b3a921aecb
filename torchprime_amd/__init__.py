"""torchprime_amd — the decoder-attention hot path of AI-Hypercomputer/torchprime on MI355X (gfx950).

Public names match the reference's so its attention modules can import from here instead:

=====================================  =============================================================
reference                              here
=====================================  =============================================================
torchprime.torch_xla_models.attention  :mod:`torchprime_amd.attention` (AttentionModule, repeat_kv)
torchprime.utils.kernel_utils          :mod:`torchprime_amd.kernel_utils`
torchprime.rope.rope                   :mod:`torchprime_amd.rope`
RMSNorm / rotary classes and apply     :mod:`torchprime_amd.norm`, :mod:`torchprime_amd.rotary`
functions in model/{llama,mixtral,
deepseek_v3}/model.py
=====================================  =============================================================

Compute runs only in ``libtprime_hip.so`` (hand-written HIP kernels reached through ``torch.library``
ops in :mod:`torchprime_amd.ops`); there is no CPU or torch-math fallback.
"""

from . import kernel_utils, ops, parallelism_utils, rope  # noqa: F401
from .attention import AttentionModule, repeat_kv
from .blocks import (DeepseekV3Attention, Llama4TextAttention, LlamaAttention, LlamaDecoderLayer, LlamaForCausalLM, LlamaModel,
                     MixtralAttention)
from .config import Config
from .kernel_utils import SplashAttentionConfig, splash_attention_jax_wrapper, tpu_splash_attention_jax_call_wrapper
from .llama4 import (
  Llama4TextL2Norm,
  Llama4TextRotaryEmbedding,
  apply_attn_temperature,
  apply_rotary_emb,
  attn_temperature_scales,
)
from .loss import cross_entropy_loss
from .mlp import LlamaMLP
from .norm import DeepseekV3RMSNorm, LlamaRMSNorm, MixtralRMSNorm, add_rms_norm
from .rope import RopeScaling, default_rope_frequencies, deepseek_v3_rope_init_fn, llama3_rope_frequencies
from .rotary import (
  DeepseekV3RotaryEmbedding,
  LlamaRotaryEmbedding,
  MixtralRotaryEmbedding,
  apply_rotary_pos_emb,
  apply_rotary_pos_emb_interleave,
  rotate_half,
)

__all__ = [
  "AttentionModule", "repeat_kv", "tpu_splash_attention_jax_call_wrapper", "splash_attention_jax_wrapper",
  "SplashAttentionConfig", "LlamaRMSNorm", "MixtralRMSNorm", "DeepseekV3RMSNorm", "RopeScaling",
  "default_rope_frequencies", "llama3_rope_frequencies", "deepseek_v3_rope_init_fn", "LlamaRotaryEmbedding",
  "MixtralRotaryEmbedding", "DeepseekV3RotaryEmbedding", "rotate_half", "apply_rotary_pos_emb",
  "apply_rotary_pos_emb_interleave", "LlamaAttention", "MixtralAttention", "DeepseekV3Attention", "Llama4TextAttention", "LlamaDecoderLayer", "LlamaModel", "LlamaForCausalLM", "Config",
  "Llama4TextL2Norm", "Llama4TextRotaryEmbedding", "apply_rotary_emb", "attn_temperature_scales", "apply_attn_temperature",
  "cross_entropy_loss", "LlamaMLP", "add_rms_norm",
]  # fmt: skip
