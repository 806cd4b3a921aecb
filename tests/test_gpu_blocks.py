"""GPU parity of the callers: ``LlamaAttention``, ``MixtralAttention`` and ``DeepseekV3Attention`` built from the
package (projections are stock ``nn.Linear``; RMSNorm, RoPE and attention are the HIP kernels), same weights as the
CPU oracle's restatement of the reference's modules, forward and the gradients of the input and of every weight.

bf16 modules against the oracle in fp64 on the same bf16-rounded inputs and weights.  Activations (block output,
input gradient) meet the kernels' own bounds, relative-L2 1e-2 and 2e-2 + 2^-7 |ref| per element, through the
three to five bf16 GEMMs a block chains around them.  Weight gradients come out of stock bf16 GEMMs that sum
batch x seq products of already rounded operands: relative-L2 1e-2, and every element within two bf16 ulps of the
tensor's largest value (2^-6 |ref|_inf)."""

import pytest
import torch

import torchprime_amd as tpa
from oracle import tprime_oracle as orc
from tests.util import assert_close, randn

pytestmark = pytest.mark.gpu
DEV = "cuda"
DT = torch.bfloat16


def _load(module, weights):
  """weights: name -> bf16 CPU tensor; copies into the module's parameters (state-dict names of the reference)."""
  sd = module.state_dict()
  assert set(sd.keys()) == set(weights.keys()), (sorted(sd.keys()), sorted(weights.keys()))
  module.load_state_dict({k: v.to(DEV) for k, v in weights.items()})


def _compare(y, y_ref, x, x_ref, params, refs, do, rel_l2=1e-2):
  y.backward(do.to(DEV))
  y_ref.backward(do.double())
  assert_close(y, y_ref, "out", scale_abs=True, rel_l2=rel_l2)
  assert_close(x.grad, x_ref.grad, "dx", scale_abs=True, rel_l2=rel_l2)
  for name, p in params.items():
    assert p.grad is not None, name
    ref = refs[name].grad
    assert_close(p.grad, ref, f"d{name}", max_abs=max(2e-2, 2.0**-6 * ref.abs().max().item()), rel_l2=rel_l2)


def _cfg(**kw):
  base = dict(attention_dropout=False, attention_bias=False)
  base.update(kw)
  return tpa.Config(base)


@pytest.mark.parametrize("kernel,Hkv", [("flash_attention", 8), ("splash_attention", 2), (None, 8)])
def test_llama_attention_module(kernel, Hkv):
  # benchmark configuration 1's block shape (B=2, S=128, hidden 512, 8 heads of 64), plus a GQA variant
  B, S, hidden, H, hd = 2, 128, 512, 8, 64
  cfg = _cfg(attention_kernel=kernel, hidden_size=hidden, num_attention_heads=H, num_key_value_heads=Hkv)
  m = tpa.LlamaAttention(cfg).to(DEV).to(DT)
  w = {
    "q_proj.weight": randn((hidden, hidden), 1, DT, 0.02), "k_proj.weight": randn((Hkv * hd, hidden), 2, DT, 0.02),
    "v_proj.weight": randn((Hkv * hd, hidden), 3, DT, 0.02), "o_proj.weight": randn((hidden, hidden), 4, DT, 0.02),
  }
  _load(m, w)
  x = randn((B, S, hidden), 5, DT)
  do = randn((B, S, hidden), 6, DT)
  pos = torch.arange(S)[None].float()
  rot = tpa.LlamaRotaryEmbedding(hd, 500000.0).to(DEV)
  xg = x.to(DEV).requires_grad_(True)
  cos, sin = rot(xg, pos.to(DEV))
  mask = orc.causal_additive_mask(S).to(DEV) if kernel is None else None
  y = m(xg, (cos, sin), mask)
  assert y.shape == (B, S, hidden) and y.dtype == DT

  c_ref, s_ref = orc.rotary_cos_sin(orc.llama3_rope_frequencies(hd, 500000.0), pos, DT)
  assert torch.equal(cos.cpu(), c_ref) or (cos.cpu().float() - c_ref.float()).abs().max() <= 8e-3
  x64 = x.double().requires_grad_(True)
  r = {k: v.double().requires_grad_(True) for k, v in w.items()}
  y_ref = orc.llama_attention(x64, r["q_proj.weight"], r["k_proj.weight"], r["v_proj.weight"], r["o_proj.weight"], H, Hkv,
                              cos.cpu().double(), sin.cpu().double())
  _compare(y, y_ref, xg, x64, dict(m.named_parameters()), r, do)


@pytest.mark.parametrize("table_default", [torch.float32, torch.bfloat16])
def test_mixtral_attention_module(table_default):
  B, S, hidden, H, Hkv, hd = 2, 160, 512, 8, 2, 64
  cfg = _cfg(attention_kernel="splash_attention", hidden_size=hidden, num_attention_heads=H, num_key_value_heads=Hkv,
             max_position_embeddings=256, rope_theta=1e6)
  old = torch.get_default_dtype()
  torch.set_default_dtype(table_default)  # the rotary cache takes the default dtype at construction (train.py:66 sets bf16)
  try:
    m = tpa.MixtralAttention(cfg)
  finally:
    torch.set_default_dtype(old)
  m = m.to(DEV).to(DT)
  w = {
    "q_proj.weight": randn((hidden, hidden), 11, DT, 0.02), "k_proj.weight": randn((Hkv * hd, hidden), 12, DT, 0.02),
    "v_proj.weight": randn((Hkv * hd, hidden), 13, DT, 0.02), "o_proj.weight": randn((hidden, hidden), 14, DT, 0.02),
  }
  _load(m, w)
  x, do = randn((B, S, hidden), 15, DT), randn((B, S, hidden), 16, DT)
  pos = torch.stack([torch.arange(S), torch.arange(S).flip(0)])  # per-batch ids, the second row reversed
  xg = x.to(DEV).requires_grad_(True)
  y = m(xg, None, pos.to(DEV))
  x64 = x.double().requires_grad_(True)
  r = {k: v.double().requires_grad_(True) for k, v in w.items()}
  y_ref = orc.mixtral_attention(x64, r["q_proj.weight"], r["k_proj.weight"], r["v_proj.weight"], r["o_proj.weight"], H, Hkv,
                                1e6, 256, pos, table_dtype=table_default, act_dtype=DT)
  # (the oracle rotates in fp64 with the table values the model sees: cached in table_default, cast to bf16)
  _compare(y, y_ref, xg, x64, dict(m.named_parameters()), r, do)


@pytest.mark.parametrize("q_lora,interleave", [(1536, True), (None, True), (1536, False)])
def test_deepseek_v3_attention_module(q_lora, interleave):
  # head and latent dims of configs/model/deepseek-v3.yaml (128 + 64 rotated q/k dims, v 128, latents 1536 / 512);
  # 8 heads and hidden 1024 keep the fp64 oracle quick
  B, S, hidden, H, nope, rope, vd, kvl = 1, 256, 1024, 8, 128, 64, 128, 512
  cfg = _cfg(attention_kernel="splash_attention", hidden_size=hidden, num_attention_heads=H, num_key_value_heads=H,
             q_lora_rank=q_lora, kv_lora_rank=kvl, qk_rope_head_dim=rope, qk_nope_head_dim=nope, v_head_dim=vd,
             qk_head_dim=nope + rope, head_dim=rope, rope_interleave=interleave, rope_theta=10000.0,
             max_position_embeddings=4096, rms_norm_eps=1e-6,
             rope_scaling=dict(beta_fast=32, beta_slow=1, factor=40, mscale=1.0, mscale_all_dim=1.0,
                               original_max_position_embeddings=4096, rope_type="yarn", type="yarn"))
  m = tpa.DeepseekV3Attention(cfg).to(DEV).to(DT)
  w = {
    "kv_a_proj_with_mqa.weight": randn((kvl + rope, hidden), 21, DT, 0.02), "kv_a_layernorm.weight": (1 + randn((kvl,), 22, torch.float32, 0.1)).to(DT),
    "kv_b_proj.weight": randn((H * (nope + vd), kvl), 23, DT, 0.02), "o_proj.weight": randn((hidden, H * vd), 24, DT, 0.02),
  }
  if q_lora:
    w.update({"q_a_proj.weight": randn((q_lora, hidden), 25, DT, 0.02), "q_a_layernorm.weight": (1 + randn((q_lora,), 26, torch.float32, 0.1)).to(DT),
              "q_b_proj.weight": randn((H * (nope + rope), q_lora), 27, DT, 0.02)})
  else:
    w["q_proj.weight"] = randn((H * (nope + rope), hidden), 28, DT, 0.02)
  _load(m, w)
  x, do = randn((B, S, hidden), 29, DT), randn((B, S, hidden), 30, DT)
  pos = torch.arange(S)[None].float()
  rot = tpa.DeepseekV3RotaryEmbedding(cfg).to(DEV)
  xg = x.to(DEV).requires_grad_(True)
  cos, sin = rot(xg, pos.to(DEV))
  y = m(xg, (cos, sin))
  assert y.shape == (B, S, hidden)

  x64 = x.double().requires_grad_(True)
  r = {k: v.double().requires_grad_(True) for k, v in w.items()}
  y_ref = orc.deepseek_v3_attention(x64, {k.replace(".weight", ""): v for k, v in r.items()}, H, nope, rope, vd, kvl,
                                    cos.cpu().double(), sin.cpu().double(), rope_interleave=interleave)
  _compare(y, y_ref, xg, x64, dict(m.named_parameters()), r, do)


@pytest.mark.parametrize("layer,qk_norm,temperature", [(0, True, True), (0, False, True), (1, True, True), (1, True, False)])
def test_llama4_attention_module(layer, qk_norm, temperature):
  """``Llama4TextAttention``: layer 0 is a rotary layer (adjacent-pair rotation, optional L2 norm of q and k), layer 1
  a NoPE layer (attention temperature on q), GQA 8:2, head dim 128 as in the Llama-4 configurations."""
  B, S, H, Hkv, hd = 2, 192, 8, 2, 128
  hidden = H * hd
  cfg = _cfg(attention_kernel="splash_attention", hidden_size=hidden, num_attention_heads=H, num_key_value_heads=Hkv,
             head_dim=hd, no_rope_layers=[1, 0], use_qk_norm=qk_norm, rms_norm_eps=1e-5, attn_temperature_tuning=temperature,
             floor_scale=64.0, attn_scale=0.1, max_position_embeddings=4096)
  m = tpa.Llama4TextAttention(cfg, layer_idx=layer).to(DEV).to(DT)
  assert m.use_rope == (layer == 0) and hasattr(m, "qk_norm") == (qk_norm and layer == 0)
  w = {
    "q_proj.weight": randn((hidden, hidden), 41, DT, 0.02), "k_proj.weight": randn((Hkv * hd, hidden), 42, DT, 0.02),
    "v_proj.weight": randn((Hkv * hd, hidden), 43, DT, 0.02), "o_proj.weight": randn((hidden, hidden), 44, DT, 0.02),
  }
  _load(m, w)
  x, do = randn((B, S, hidden), 45, DT), randn((B, S, hidden), 46, DT)
  pos = torch.arange(S)[None].float()
  rot = tpa.Llama4TextRotaryEmbedding(hd, 500000.0).to(DEV)
  xg = x.to(DEV).requires_grad_(True)
  cos, sin = rot(xg, pos.to(DEV))
  y = m(xg, (cos, sin))
  assert y.shape == (B, S, hidden) and y.dtype == DT
  x64 = x.double().requires_grad_(True)
  r = {k: v.double().requires_grad_(True) for k, v in w.items()}
  y_ref = orc.llama4_attention(x64, r["q_proj.weight"], r["k_proj.weight"], r["v_proj.weight"], r["o_proj.weight"], H, Hkv,
                               cos.cpu().double(), sin.cpu().double(), layer == 0, qk_norm, 1e-5, temperature, 64.0, 0.1)
  _compare(y, y_ref, xg, x64, dict(m.named_parameters()), r, do)


@pytest.mark.parametrize("kernel", ["splash_attention", None])
def test_llama_decoder_layer(kernel):
  """A whole decoder layer from the package's modules (norms, attention, residual add fused into the second norm,
  SwiGLU MLP) against the oracle's restatement of LlamaDecoderLayer: output, input gradient and every weight gradient."""
  B, S, hidden, H, Hkv, hd, inter = 2, 160, 512, 8, 2, 64, 1024
  cfg = _cfg(attention_kernel=kernel, hidden_size=hidden, num_attention_heads=H, num_key_value_heads=Hkv,
             intermediate_size=inter, rms_norm_eps=1e-5, hidden_act="silu")
  m = tpa.LlamaDecoderLayer(cfg, 0).to(DEV).to(DT)
  w = {
    "self_attn.q_proj.weight": randn((hidden, hidden), 51, DT, 0.02), "self_attn.k_proj.weight": randn((Hkv * hd, hidden), 52, DT, 0.02),
    "self_attn.v_proj.weight": randn((Hkv * hd, hidden), 53, DT, 0.02), "self_attn.o_proj.weight": randn((hidden, hidden), 54, DT, 0.02),
    "mlp.gate_proj.weight": randn((inter, hidden), 55, DT, 0.02), "mlp.up_proj.weight": randn((inter, hidden), 56, DT, 0.02),
    "mlp.down_proj.weight": randn((hidden, inter), 57, DT, 0.02),
    "input_layernorm.weight": (1 + randn((hidden,), 58, std=0.1)).to(DT), "post_attention_layernorm.weight": (1 + randn((hidden,), 59, std=0.1)).to(DT),
  }
  _load(m, w)
  x, do = randn((B, S, hidden), 60, DT), randn((B, S, hidden), 61, DT)
  pos = torch.arange(S)[None].float()
  rot = tpa.LlamaRotaryEmbedding(hd, 500000.0).to(DEV)
  xg = x.to(DEV).requires_grad_(True)
  cos, sin = rot(xg, pos.to(DEV))
  mask = orc.causal_additive_mask(S).to(DEV) if kernel is None else None
  y = m(xg, attention_mask=mask, position_embeddings=(cos, sin))
  assert y.shape == (B, S, hidden) and y.dtype == DT
  x64 = x.double().requires_grad_(True)
  r = {k: v.double().requires_grad_(True) for k, v in w.items()}
  y_ref = orc.llama_decoder_layer(x64, r, H, Hkv, 1e-5, cos.cpu().double(), sin.cpu().double())
  _compare(y, y_ref, xg, x64, dict(m.named_parameters()), r, do)


def test_llama_attention_module_fp32_forward_and_backward():
  """benchmark configuration 1's block in fp32 end to end on the GPU (fp32 RMSNorm-free attention block: projections,
  RoPE, fp32 attention forward and backward, output projection): output, input gradient and weight gradients against
  the fp64 oracle at the fp32 class of tolerance (relative-L2 2e-5, 2e-5 of the tensor's largest value per element)."""
  B, S, hidden, H, hd = 2, 128, 512, 8, 64
  cfg = _cfg(attention_kernel=None, hidden_size=hidden, num_attention_heads=H, num_key_value_heads=H)
  m = tpa.LlamaAttention(cfg).to(DEV)
  w = {
    "q_proj.weight": randn((hidden, hidden), 71, std=0.02), "k_proj.weight": randn((hidden, hidden), 72, std=0.02),
    "v_proj.weight": randn((hidden, hidden), 73, std=0.02), "o_proj.weight": randn((hidden, hidden), 74, std=0.02),
  }
  _load(m, w)
  x, do = randn((B, S, hidden), 75), randn((B, S, hidden), 76)
  pos = torch.arange(S)[None].float()
  rot = tpa.LlamaRotaryEmbedding(hd, 500000.0).to(DEV)
  xg = x.to(DEV).requires_grad_(True)
  cos, sin = rot(xg, pos.to(DEV))
  old = torch.backends.cuda.matmul.allow_tf32
  torch.backends.cuda.matmul.allow_tf32 = False
  try:
    y = m(xg, (cos, sin), orc.causal_additive_mask(S).to(DEV))
    assert y.dtype == torch.float32
    y.backward(do.to(DEV))
  finally:
    torch.backends.cuda.matmul.allow_tf32 = old
  x64 = x.double().requires_grad_(True)
  r = {k: v.double().requires_grad_(True) for k, v in w.items()}
  y_ref = orc.llama_attention(x64, r["q_proj.weight"], r["k_proj.weight"], r["v_proj.weight"], r["o_proj.weight"], H, H,
                              cos.cpu().double(), sin.cpu().double())
  y_ref.backward(do.double())
  def tight(got, ref, name):
    assert_close(got, ref, name, max_abs=2e-5 * max(1.0, ref.abs().max().item()), rel_l2=2e-5)
  tight(y, y_ref, "out")
  tight(xg.grad, x64.grad, "dx")
  for name, p in m.named_parameters():
    tight(p.grad, r[name].grad, f"d{name}")
