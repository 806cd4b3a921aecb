"""GPU parity of the path's callers two levels up: ``LlamaForCausalLM`` built from the package's modules (embedding,
decoder layers with the residual adds fused into the norms, final norm, ``lm_head``, shifted cross entropy; every
RMSNorm, rotary, attention, SwiGLU and loss step a HIP kernel, the GEMMs stock ``nn.Linear``), laid out like the
reference's own test of the same class (torch_xla_models/tests/test_llama.py:136-188): its two fixtures (Llama 3.0
8B and Llama 3.1 405B cut down to hidden 512, 8 heads of 64, one / two layers), its input sizes 8 / 128 / 256, labels
= input ids, an attention mask of ones; logits, loss and the gradient of every parameter are compared.

The checker is the CPU oracle's ``llama_for_causal_lm`` (pinned on HuggingFace's LlamaForCausalLM in
tests/test_oracle.py), evaluated in fp64.  fp32 tolerances: the reference asks 1e-6 / 1e-4 / 1e-5 (logits / loss /
gradients) of two models on ONE backend and 1e-2 / 1e-4 / 1e-5 of the same model on two backends
(test_llama.py:191-240).  This is the second kind of comparison; logits are held to 2e-5 (fp32 GEMMs and the fp32
attention kernels accumulate in another order than the CPU), loss and gradients to the reference's own numbers."""

import pytest
import torch

import torchprime_amd as tpa
from oracle import tprime_oracle as orc

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _fixture(which, kernel):
  base = dict(hidden_size=512, intermediate_size=64, num_attention_heads=8, num_key_value_heads=8, hidden_act="silu",
              initializer_range=0.02, rms_norm_eps=1e-5, attention_dropout=False, attention_bias=False,
              attention_kernel=kernel, rope_theta=500000.0)
  if which == "llama3_8b":
    cfg, scaling = tpa.Config(vocab_size=128, num_hidden_layers=1, max_position_embeddings=8192, **base), None
  else:
    cfg = tpa.Config(vocab_size=256, num_hidden_layers=2, max_position_embeddings=131072,
                     rope_scaling={"factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0, "original_context_len": 8192}, **base)
    scaling = (8.0, 1.0, 4.0, 8192)
  torch.manual_seed(42)
  return tpa.LlamaForCausalLM(cfg), cfg, scaling


def _no_tf32():
  class Ctx:
    def __enter__(self):
      self.old = torch.backends.cuda.matmul.allow_tf32
      torch.backends.cuda.matmul.allow_tf32 = False
    def __exit__(self, *a):
      torch.backends.cuda.matmul.allow_tf32 = self.old
  return Ctx()


@pytest.mark.parametrize("which", ["llama3_8b", "llama3_1_405b"])
@pytest.mark.parametrize("kernel", [None, "splash_attention"])
@pytest.mark.parametrize("input_size", [8, 128, 256])
def test_forward_and_backward_our_model_against_oracle_fp32(which, kernel, input_size):
  model, cfg, scaling = _fixture(which, kernel)
  weights = {k: v.detach().clone() for k, v in model.state_dict().items()}
  ids = torch.randint(cfg.vocab_size, (2, input_size // 2), generator=torch.Generator().manual_seed(input_size))
  ones = torch.ones_like(ids)
  model = model.to(DEV)
  model.zero_grad()
  with _no_tf32():
    logits, loss = model(input_ids=ids.to(DEV), labels=ids.to(DEV), attention_mask=ones.to(DEV))
    loss.backward()
  assert logits.dtype == torch.float32 and logits.shape == (2, input_size // 2, cfg.vocab_size)
  w64 = {k: v.double().requires_grad_(True) for k, v in weights.items()}
  ref_logits, ref_loss = orc.llama_for_causal_lm(ids, ids, w64, 8, 8, 1e-5, 500000.0, scaling, attention_mask=ones)
  ref_loss.backward()
  torch.testing.assert_close(logits.cpu().double(), ref_logits, atol=2e-5, rtol=1e-9, msg=lambda m: f"logits: {m}")
  torch.testing.assert_close(loss.cpu().double(), ref_loss, atol=1e-4, rtol=1e-7, msg=lambda m: f"loss: {m}")
  names = [n for n, _ in model.named_parameters()]
  assert names == list(w64.keys()), "parameter names and order are the reference's state-dict names"
  for name, p in model.named_parameters():
    assert p.grad is not None, f"no gradient for {name}"
    torch.testing.assert_close(p.grad.cpu().double(), w64[name].grad, atol=1e-5, rtol=1e-9, msg=lambda m, name=name: f"gradient of {name}: {m}")


def test_state_dict_loads_from_huggingface_and_matches_it():
  """``model.load_state_dict(hf_model.state_dict())`` as in the reference's fixtures (test_llama.py:62-66), then the
  two models against each other directly."""
  try:
    from transformers import LlamaConfig
    from transformers import LlamaForCausalLM as HfLlamaForCausalLM
    hcfg = LlamaConfig(vocab_size=256, num_hidden_layers=2, max_position_embeddings=131072, hidden_size=512, num_attention_heads=8,
                       num_key_value_heads=8, head_dim=64, intermediate_size=64, rms_norm_eps=1e-5, rope_theta=500000.0,
                       attention_bias=False, mlp_bias=False, hidden_act="silu", tie_word_embeddings=False, use_cache=False,
                       rope_scaling={"factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                                     "original_max_position_embeddings": 8192, "rope_type": "llama3"})
    hcfg._attn_implementation = "eager"
    torch.manual_seed(42)
    hf = HfLlamaForCausalLM(hcfg)
    ids = torch.randint(256, (2, 64), generator=torch.Generator().manual_seed(3))
    hf.zero_grad()
    out = hf(input_ids=ids, labels=ids, attention_mask=torch.ones_like(ids))
    out.loss.backward()
  except Exception as e:
    pytest.skip(f"transformers LlamaForCausalLM not usable here: {e}")
  model, cfg, _ = _fixture("llama3_1_405b", None)
  model.load_state_dict(hf.state_dict())
  torch.testing.assert_close(model.model.rotary_emb.inv_freq, hf.model.rotary_emb.inv_freq)
  assert model.model.rotary_emb.inv_freq.shape == (32,)
  model = model.to(DEV)
  with _no_tf32():
    logits, loss = model(input_ids=ids.to(DEV), labels=ids.to(DEV), attention_mask=torch.ones_like(ids).to(DEV))
    loss.backward()
  torch.testing.assert_close(logits.cpu(), out.logits, atol=2e-5, rtol=1e-6)
  torch.testing.assert_close(loss.cpu(), out.loss, atol=1e-4, rtol=1e-7)
  for (name_hf, p_hf), (name, p) in zip(hf.named_parameters(), model.named_parameters(), strict=True):
    assert name_hf == name
    torch.testing.assert_close(p.grad.cpu(), p_hf.grad, atol=1e-5, rtol=1e-6, msg=lambda m, name=name: f"gradient of {name}: {m}")


def test_deferred_residual_adds_equal_the_layer_by_layer_model():
  """The model hands each layer's closing residual add to the next norm's kernel; layer by layer through
  ``LlamaDecoderLayer.forward`` the result is the same, bit for bit (bf16, where the order of roundings would show)."""
  model, cfg, _ = _fixture("llama3_1_405b", "flash_attention")
  model = model.to(DEV).to(torch.bfloat16)
  ids = torch.randint(cfg.vocab_size, (2, 96), generator=torch.Generator().manual_seed(5)).to(DEV)
  with torch.no_grad():
    fused = model.model(ids)
    m = model.model
    x = m.embed_tokens(ids)
    pos = torch.arange(96, device=DEV)[None].float()
    pe = m.rotary_emb(x, pos)
    for layer in m.layers:
      x = layer(x, attention_mask=None, position_ids=pos, position_embeddings=pe)
    plain = m.norm(x)
  assert torch.equal(fused, plain)


def test_bf16_model_with_gqa_against_oracle():
  """A bf16 model at head dim 128 with grouped kv heads (the shape class of the headline benchmark, cut down) through
  the bf16 attention kernels.  Two layers of bf16 modules round every activation, so the yardstick is the reference's
  own arithmetic: the oracle evaluated in bf16 on the CPU (eager, op by op) against the oracle in fp64 on the same
  bf16-rounded weights.  Logits, loss and every gradient of the GPU model must be within 1.25 times that error of the
  fp64 values (relative-L2; plus 1e-3 for tensors whose eager error happens to be tiny).  Measured: 0.7-1.4e-2 for
  both, the GPU model within 3 % of the eager evaluation on every tensor.  The model is cast with ``.to(bfloat16)``
  on purpose: the rotary frequencies must survive that in fp32 (rounded to bf16 they cost 6 % on the rotated q)."""
  cfg = tpa.Config(vocab_size=512, hidden_size=1024, intermediate_size=2048, num_hidden_layers=2, num_attention_heads=8,
                   num_key_value_heads=2, hidden_act="silu", max_position_embeddings=8192, initializer_range=0.02, rms_norm_eps=1e-5,
                   attention_dropout=False, attention_bias=False, attention_kernel="splash_attention", rope_theta=500000.0)
  torch.manual_seed(7)
  model = tpa.LlamaForCausalLM(cfg).to(torch.bfloat16)
  weights = {k: v.detach().clone() for k, v in model.state_dict().items()}
  ids = torch.randint(512, (2, 320), generator=torch.Generator().manual_seed(9))
  model = model.to(DEV)
  logits, loss = model(input_ids=ids.to(DEV), labels=ids.to(DEV))
  loss.backward()

  def oracle(dtype):
    w = {k: v.to(dtype).requires_grad_(True) for k, v in weights.items()}
    lg, ls = orc.llama_for_causal_lm(ids, ids, w, 8, 2, 1e-5, 500000.0)
    ls.backward()
    return lg.detach().double(), ls.item(), {k: v.grad.double() for k, v in w.items()}

  ref_logits, ref_loss, ref_grads = oracle(torch.float64)
  cpu_logits, cpu_loss, cpu_grads = oracle(torch.bfloat16)

  def rel(a, b):
    return ((a.double().cpu() - b).norm() / b.norm()).item()

  bad, seen = [], []

  def check(name, got, eager, ref):
    e_gpu, e_cpu = rel(got, ref), rel(eager, ref)
    assert torch.isfinite(got.float()).all(), name
    seen.append(f"{name}: {e_gpu:.3e} vs {e_cpu:.3e}")
    if e_gpu > 1.25 * e_cpu + 1e-3:
      bad.append(f"{name}: relative-L2 {e_gpu:.3e} on the GPU, {e_cpu:.3e} for the eager bf16 evaluation")

  check("logits", logits.detach(), cpu_logits, ref_logits)
  assert abs(loss.item() - ref_loss) <= 1.25 * abs(cpu_loss - ref_loss) + 2e-3, (loss.item(), cpu_loss, ref_loss)
  for name, p in model.named_parameters():
    check(f"gradient of {name}", p.grad, cpu_grads[name], ref_grads[name])
  assert not bad, "\n".join(bad)
