"""Attention blocks that call the hot path the way the reference's models do.  They exist so tests
and the benchmark can drive RMSNorm -> projections -> RoPE -> attention -> output projection with the
reference's tensor layouts; the projections are stock ``nn.Linear`` (GEMMs are outside the path).

* LlamaAttention        torchprime/torch_xla_models/model/llama/model.py:156-238
* MixtralAttention      model/mixtral/model.py:159-243
* DeepseekV3Attention   model/deepseek_v3/model.py:341-455
* LlamaDecoderLayer, LlamaModel, LlamaForCausalLM   model/llama/model.py:241-400 (the callers of the path, one and
  two levels up: embedding, the layers, final norm, ``lm_head`` and the shifted cross entropy)
"""

from __future__ import annotations

import torch
from torch import nn

from .attention import AttentionModule
from .norm import DeepseekV3RMSNorm
from .rotary import MixtralRotaryEmbedding, apply_rotary_pos_emb, apply_rotary_pos_emb_interleave


class LlamaAttention(nn.Module):
  def __init__(self, config, layer_idx: int | None = None):
    super().__init__()
    self.config = config
    self.attention_block = AttentionModule(config)
    self.layer_idx = layer_idx
    self.hidden_size = config.hidden_size
    self.num_heads = config.num_attention_heads
    self.head_dim = self.hidden_size // self.num_heads
    self.num_key_value_heads = config.num_key_value_heads
    self.num_key_value_groups = self.num_heads // self.num_key_value_heads
    if (self.head_dim * self.num_heads) != self.hidden_size:
      raise ValueError(
        f"hidden_size must be divisible by num_heads (got `hidden_size`: {self.hidden_size}"
        f" and `num_heads`: {self.num_heads})."
      )
    bias = bool(getattr(config, "attention_bias", False))
    self.q_proj = nn.Linear(self.hidden_size, self.num_heads * self.head_dim, bias=bias)
    self.k_proj = nn.Linear(self.hidden_size, self.num_key_value_heads * self.head_dim, bias=bias)
    self.v_proj = nn.Linear(self.hidden_size, self.num_key_value_heads * self.head_dim, bias=bias)
    self.o_proj = nn.Linear(self.hidden_size, self.hidden_size, bias=bias)

  def forward(self, hidden_states, position_embeddings, attention_mask=None, position_ids=None):
    bsz, q_len, _ = hidden_states.size()
    q = self.q_proj(hidden_states).view(bsz, q_len, self.num_heads, self.head_dim).transpose(1, 2)
    k = self.k_proj(hidden_states).view(bsz, q_len, self.num_key_value_heads, self.head_dim).transpose(1, 2)
    v = self.v_proj(hidden_states).view(bsz, q_len, self.num_key_value_heads, self.head_dim).transpose(1, 2)
    cos, sin = position_embeddings
    q, k = apply_rotary_pos_emb(q, k, cos, sin)
    out = self.attention_block(q, k, v, attention_mask)
    out = out.transpose(1, 2).contiguous().reshape(bsz, q_len, self.hidden_size)
    return self.o_proj(out)


class MixtralAttention(nn.Module):
  def __init__(self, config, layer_idx: int | None = None):
    super().__init__()
    self.config = config
    self.attention_block = AttentionModule(config)
    self.layer_idx = layer_idx
    self.hidden_size = config.hidden_size
    self.num_heads = config.num_attention_heads
    self.head_dim = self.hidden_size // self.num_heads
    self.num_key_value_heads = config.num_key_value_heads
    self.num_key_value_groups = self.num_heads // self.num_key_value_heads
    self.max_position_embeddings = config.max_position_embeddings
    self.rope_theta = config.rope_theta
    if (self.head_dim * self.num_heads) != self.hidden_size:
      raise ValueError(
        f"hidden_size must be divisible by num_heads (got `hidden_size`: {self.hidden_size}"
        f" and `num_heads`: {self.num_heads})."
      )
    self.q_proj = nn.Linear(self.hidden_size, self.num_heads * self.head_dim, bias=False)
    self.k_proj = nn.Linear(self.hidden_size, self.num_key_value_heads * self.head_dim, bias=False)
    self.v_proj = nn.Linear(self.hidden_size, self.num_key_value_heads * self.head_dim, bias=False)
    self.o_proj = nn.Linear(self.num_heads * self.head_dim, self.hidden_size, bias=False)
    self.rotary_emb = MixtralRotaryEmbedding(
      self.head_dim, max_position_embeddings=self.max_position_embeddings, base=self.rope_theta
    )

  def forward(self, hidden_states, attention_mask=None, position_ids=None):
    bsz, q_len, _ = hidden_states.size()
    q = self.q_proj(hidden_states).view(bsz, q_len, self.num_heads, self.head_dim).transpose(1, 2)
    k = self.k_proj(hidden_states).view(bsz, q_len, self.num_key_value_heads, self.head_dim).transpose(1, 2)
    v = self.v_proj(hidden_states).view(bsz, q_len, self.num_key_value_heads, self.head_dim).transpose(1, 2)
    cos, sin = self.rotary_emb(v, seq_len=k.shape[-2])
    q, k = apply_rotary_pos_emb(q, k, cos, sin, position_ids)
    out = self.attention_block(q, k, v, attention_mask)
    out = out.transpose(1, 2).contiguous().reshape(bsz, q_len, self.hidden_size)
    return self.o_proj(out)


class DeepseekV3Attention(nn.Module):
  """Multi-headed latent attention: low-rank q and kv projections with RMSNorm on the latents,
  128 un-rotated + 64 rotated q/k dims, one shared rotated k head, v head dim 128."""

  def __init__(self, config, layer_idx: int | None = None):
    super().__init__()
    self.config = config
    self.attention_block = AttentionModule(config)
    self.layer_idx = layer_idx
    self.num_heads = config.num_attention_heads
    self.qk_head_dim = config.qk_head_dim
    bias = bool(getattr(config, "attention_bias", False))
    if config.q_lora_rank is None:
      self.q_proj = nn.Linear(config.hidden_size, self.num_heads * self.qk_head_dim, bias=False)
    else:
      self.q_a_proj = nn.Linear(config.hidden_size, config.q_lora_rank, bias=bias)
      self.q_a_layernorm = DeepseekV3RMSNorm(config.q_lora_rank)
      self.q_b_proj = nn.Linear(config.q_lora_rank, self.num_heads * self.qk_head_dim, bias=False)
    self.kv_a_proj_with_mqa = nn.Linear(config.hidden_size, config.kv_lora_rank + config.qk_rope_head_dim, bias=bias)
    self.kv_a_layernorm = DeepseekV3RMSNorm(config.kv_lora_rank)
    self.kv_b_proj = nn.Linear(
      config.kv_lora_rank, self.num_heads * (config.qk_nope_head_dim + config.v_head_dim), bias=False
    )
    self.o_proj = nn.Linear(self.num_heads * config.v_head_dim, config.hidden_size, bias=bias)

  def forward(self, hidden_states, position_embeddings, attention_mask=None, position_ids=None):
    cfg = self.config
    bsz, q_len = hidden_states.shape[:2]
    if cfg.q_lora_rank is None:
      q = self.q_proj(hidden_states)
    else:
      q = self.q_b_proj(self.q_a_layernorm(self.q_a_proj(hidden_states)))
    q = q.view(bsz, q_len, -1, self.qk_head_dim).transpose(1, 2)
    q_pass, q_rot = torch.split(q, [cfg.qk_nope_head_dim, cfg.qk_rope_head_dim], dim=-1)

    compressed_kv = self.kv_a_proj_with_mqa(hidden_states)
    k_pass, k_rot = torch.split(compressed_kv, [cfg.kv_lora_rank, cfg.qk_rope_head_dim], dim=-1)
    k_pass = self.kv_b_proj(self.kv_a_layernorm(k_pass))
    k_pass = k_pass.view(bsz, q_len, -1, cfg.qk_nope_head_dim + cfg.v_head_dim).transpose(1, 2)
    k_pass, v = torch.split(k_pass, [cfg.qk_nope_head_dim, cfg.v_head_dim], dim=-1)

    k_rot = k_rot.view(bsz, 1, q_len, cfg.qk_rope_head_dim)
    cos, sin = position_embeddings
    if cfg.rope_interleave:
      q_rot, k_rot = apply_rotary_pos_emb_interleave(q_rot, k_rot, cos, sin)
    else:
      q_rot, k_rot = apply_rotary_pos_emb(q_rot, k_rot, cos, sin)
    k_rot = k_rot.expand(*k_pass.shape[:-1], -1)

    q = torch.cat((q_pass, q_rot), dim=-1)
    k = torch.cat((k_pass, k_rot), dim=-1)
    out = self.attention_block(q, k, v, attention_mask)
    out = out.transpose(1, 2).contiguous().reshape(bsz, q_len, -1)
    return self.o_proj(out)


class Llama4TextAttention(nn.Module):
  """model/llama4/model.py:427-533: rotary layers apply the adjacent-pair rotation and (``use_qk_norm``) the weightless
  L2 norm to q and k; layers without rotary ("NoPE") scale the queries by the position-dependent attention temperature
  instead.  Which kind a layer is comes from ``config.no_rope_layers[layer_idx]`` as in the reference."""

  def __init__(self, config, layer_idx: int | None = None):
    super().__init__()
    from .llama4 import Llama4TextL2Norm

    self.config = config
    self.attention_block = AttentionModule(config)
    self.layer_idx = layer_idx
    self.num_attention_heads = config.num_attention_heads
    self.num_key_value_heads = config.num_key_value_heads
    self.num_key_value_groups = self.num_attention_heads // self.num_key_value_heads
    self.attn_scale = config.attn_scale
    self.floor_scale = config.floor_scale
    self.attn_temperature_tuning = config.attn_temperature_tuning
    no_rope = getattr(config, "no_rope_layers", None)
    self.use_rope = bool(no_rope and layer_idx is not None and layer_idx < len(no_rope) and no_rope[layer_idx])
    if (config.head_dim * config.num_attention_heads) != config.hidden_size:
      raise ValueError(
        f"hidden_size must be divisible by num_attention_heads (got `hidden_size`: {config.hidden_size}"
        f" and `num_attention_heads`: {config.num_attention_heads})."
      )
    self.hidden_size = config.hidden_size
    self.head_dim = self.hidden_size // self.num_attention_heads
    bias = bool(getattr(config, "attention_bias", False))
    self.q_proj = nn.Linear(self.hidden_size, self.num_attention_heads * self.head_dim, bias=bias)
    self.k_proj = nn.Linear(self.hidden_size, self.num_key_value_heads * self.head_dim, bias=bias)
    self.v_proj = nn.Linear(self.hidden_size, self.num_key_value_heads * self.head_dim, bias=bias)
    self.o_proj = nn.Linear(self.hidden_size, self.hidden_size, bias=bias)
    if getattr(config, "use_qk_norm", False) and self.use_rope:
      self.qk_norm = Llama4TextL2Norm(config.rms_norm_eps)

  def forward(self, hidden_states, position_embeddings, attention_mask=None, position_ids=None):
    from .llama4 import apply_attn_temperature, apply_rotary_emb

    bsz, q_len, _ = hidden_states.size()
    q = self.q_proj(hidden_states).view(bsz, q_len, -1, self.head_dim)
    k = self.k_proj(hidden_states).view(bsz, q_len, -1, self.head_dim)
    v = self.v_proj(hidden_states).view(bsz, q_len, -1, self.head_dim).transpose(1, 2)
    if self.use_rope:
      q, k = apply_rotary_emb(q, k, position_embeddings)
    if hasattr(self, "qk_norm"):
      q, k = self.qk_norm(q), self.qk_norm(k)
    if self.attn_temperature_tuning and not self.use_rope:
      q = apply_attn_temperature(q, self.floor_scale, self.attn_scale)
    out = self.attention_block(q.transpose(1, 2), k.transpose(1, 2), v, attention_mask)
    out = out.transpose(1, 2).contiguous().reshape(bsz, q_len, self.hidden_size)
    return self.o_proj(out)


class LlamaDecoderLayer(nn.Module):
  """model/llama/model.py:241-296 with the package's modules: the residual add after the attention and the norm that
  follows it are one kernel (``add_rms_norm``), the MLP's gate product another; the four adds / norms / products of
  the reference's layer are evaluated in the same order and with the same roundings."""

  def __init__(self, config, layer_idx: int):
    super().__init__()
    from .mlp import LlamaMLP
    from .norm import LlamaRMSNorm

    self.hidden_size = config.hidden_size
    self.self_attn = LlamaAttention(config=config, layer_idx=layer_idx)
    self.mlp = LlamaMLP(config)
    self.input_layernorm = LlamaRMSNorm(config.hidden_size, eps=config.rms_norm_eps)
    self.post_attention_layernorm = LlamaRMSNorm(config.hidden_size, eps=config.rms_norm_eps)

  def forward(self, hidden_states, attention_mask=None, position_ids=None, position_embeddings=None):
    from .norm import add_rms_norm

    residual = hidden_states
    hidden_states = self.input_layernorm(hidden_states)
    hidden_states = self.self_attn(hidden_states, position_embeddings, attention_mask, position_ids)
    # residual + hidden_states, then post_attention_layernorm of the sum, in one pass
    hidden_states, residual = add_rms_norm(hidden_states, residual, self.post_attention_layernorm)
    hidden_states = self.mlp(hidden_states)
    return residual + hidden_states



  def forward_deferred(self, x, residual, attention_mask=None, position_ids=None, position_embeddings=None):
    """The same layer with the residual adds at its two ends left to the neighbours.  The layer's input is
    ``x + residual`` (``residual`` None: ``x`` itself), added inside the first norm's kernel; the return value is
    ``(mlp_out, h)`` whose sum is the layer's output, for the next layer (or the model's final norm) to add the same
    way.  Same values as ``forward``, bit for bit, with one pass over the hidden states less per layer."""
    from .norm import add_rms_norm

    if residual is None:
      residual, hidden_states = x, self.input_layernorm(x)
    else:
      hidden_states, residual = add_rms_norm(x, residual, self.input_layernorm)
    hidden_states = self.self_attn(hidden_states, position_embeddings, attention_mask, position_ids)
    hidden_states, residual = add_rms_norm(hidden_states, residual, self.post_attention_layernorm)
    return self.mlp(hidden_states), residual


class LlamaModel(nn.Module):
  """model/llama/model.py:300-367: embedding, the decoder layers, the final norm; position ids ``arange(S)`` as
  floats, one rotary table for all layers.  Parameter names are the reference's (and HuggingFace's), so
  ``load_state_dict(hf_model.state_dict())`` works as in the reference's tests.

  The (S, S) additive causal mask of :347-355 is only consumed by the eager branch of ``AttentionModule`` (the kernel
  branches are causal by themselves), so it is built only for ``attention_kernel=None``, and kept per sequence length
  while no padding mask multiplies it."""

  def __init__(self, config):
    super().__init__()
    from .norm import LlamaRMSNorm
    from .rope import RopeScaling
    from .rotary import LlamaRotaryEmbedding

    self.config = config
    self.vocab_size = config.vocab_size
    self.embed_tokens = nn.Embedding(config.vocab_size, config.hidden_size)
    self.layers = nn.ModuleList(LlamaDecoderLayer(config, i) for i in range(config.num_hidden_layers))
    self.norm = LlamaRMSNorm(config.hidden_size, eps=config.rms_norm_eps)
    rope_scaling = config.get("rope_scaling", None)
    if rope_scaling is not None:
      rope_scaling = RopeScaling(**dict(rope_scaling))
    self.rope_theta = config.rope_theta
    self.rotary_emb = LlamaRotaryEmbedding(
      head_dim=config.hidden_size // config.num_attention_heads, rope_theta=config.rope_theta, scaling=rope_scaling
    )
    self._causal_masks: dict = {}

  def _mask(self, seq_length, attention_mask, device):
    if self.config.attention_kernel in ("splash_attention", "flash_attention"):
      return None  # never read on those branches (attention.py:121-123, 144-150)
    key = (seq_length, str(device))
    causal = self._causal_masks.get(key)
    if causal is None:
      if len(self._causal_masks) > 4:
        self._causal_masks.clear()
      causal = torch.triu(torch.full((seq_length, seq_length), float("-inf"), device=device), diagonal=1)[None, None]
      self._causal_masks[key] = causal
    if attention_mask is not None:
      causal = causal * attention_mask[:, None, None, :]
    return causal

  def forward(self, input_ids, attention_mask=None):
    from .norm import add_rms_norm

    inputs_embeds = self.embed_tokens(input_ids)
    seq_length = inputs_embeds.size(1)
    position_ids = torch.arange(seq_length, device=inputs_embeds.device).unsqueeze(0).float()
    causal_mask = self._mask(seq_length, attention_mask, inputs_embeds.device)
    position_embeddings = self.rotary_emb(inputs_embeds, position_ids)
    x, residual = inputs_embeds, None
    for layer in self.layers:
      x, residual = layer.forward_deferred(x, residual, attention_mask=causal_mask, position_ids=position_ids,
                                           position_embeddings=position_embeddings)
    if residual is None:
      return self.norm(x)
    return add_rms_norm(x, residual, self.norm)[0]


class LlamaForCausalLM(nn.Module):
  """model/llama/model.py:370-400: the model, ``lm_head``, logits in fp32 and the shifted cross entropy; returns
  ``(logits, loss)`` (loss None without labels).  Linear and embedding weights start from a normal distribution of
  standard deviation ``config.initializer_range``, biases from zero (model/base_causal_lm.py:38-54)."""

  def __init__(self, config):
    super().__init__()
    self.config = config
    self.model = LlamaModel(config)
    self.vocab_size = config.vocab_size
    self.lm_head = nn.Linear(config.hidden_size, config.vocab_size, bias=False)
    self.apply(self._init_weights)

  def _init_weights(self, module):
    std = self.config.initializer_range
    if isinstance(module, (nn.Linear, nn.Embedding)):
      module.weight.data.normal_(mean=0.0, std=std)
      if getattr(module, "bias", None) is not None:
        module.bias.data.zero_()

  def forward(self, input_ids, labels=None, attention_mask=None):
    from .loss import cross_entropy_loss

    hidden_states = self.model(input_ids=input_ids, attention_mask=attention_mask)
    logits = self.lm_head(hidden_states).float()
    if labels is None:
      return logits, None
    return logits, cross_entropy_loss(logits, labels=labels, vocab_size=self.config.vocab_size)
