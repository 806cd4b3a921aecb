"""Golden fixtures (tests/golden/*.npz, written by tests/golden/make_golden.py from the oracle):
CPU: the oracle still reproduces them.  GPU: the HIP path matches them."""

import os

import numpy as np
import pytest
import torch

from oracle import tprime_oracle as orc
from tests.golden.make_golden import attn_inputs, c1_inputs
from tests.util import assert_close

G = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _load(name):
  return {k: torch.from_numpy(np.asarray(v)) for k, v in np.load(os.path.join(G, name), allow_pickle=False).items()}


def test_oracle_reproduces_golden():
  x, w_norm, w = c1_inputs()
  y = orc.llama_attention_block(x, w_norm, w["wq"], w["wk"], w["wv"], w["wo"], 8, 8, 1e-5, 500000.0)
  torch.testing.assert_close(y[:, ::8], _load("c1_llama_block.npz")["out_rows"], rtol=1e-4, atol=2e-5)  # fp32 matmul chains: reduction order differs with the thread count
  q, k, v, do, seg = attn_inputs()
  g = _load("attn_segments_small.npz")
  out, dq, dk, dv = orc.attention_grads_ref(q, k, v, do, seg, True, None, torch.float64)
  for name, t in (("out", out), ("dq", dq), ("dk", dk), ("dv", dv)):
    torch.testing.assert_close(t.float(), g[name], rtol=1e-5, atol=1e-6)
  f = _load("rope_frequencies.npz")
  torch.testing.assert_close(orc.llama3_rope_frequencies(128, 500000.0, factor=8.0), f["llama3_d128"])
  torch.testing.assert_close(orc.default_rope_frequencies(128, 500000.0), f["default_d128"])


def test_product_rope_tables_match_golden():
  import torchprime_amd as tpa

  f = _load("rope_frequencies.npz")
  torch.testing.assert_close(tpa.llama3_rope_frequencies(128, 500000.0, tpa.RopeScaling()), f["llama3_d128"])
  torch.testing.assert_close(tpa.default_rope_frequencies(128, 500000.0), f["default_d128"])
  cfg = tpa.Config(rope_theta=10000.0, head_dim=64, hidden_size=512, num_attention_heads=8, max_position_embeddings=16384,
                   rope_scaling={"rope_type": "yarn", "factor": 4.0, "original_max_position_embeddings": 4096})
  inv, att = tpa.deepseek_v3_rope_init_fn(cfg)
  torch.testing.assert_close(inv, f["yarn_d64_f4"])
  assert att == pytest.approx(float(f["yarn_attention_factor"]))


@pytest.mark.gpu
def test_hip_attention_matches_golden():
  q, k, v, do, seg = attn_inputs()
  g = _load("attn_segments_small.npz")
  dev = "cuda"
  qd, kd, vd = (t.bfloat16().to(dev).requires_grad_(True) for t in (q, k, v))
  out, lse = torch.ops.tprime.attn_fwd(qd, kd, vd, seg.to(dev), 64**-0.5, True)
  out.backward(do.bfloat16().to(dev))
  # inputs are rounded to bf16 for the kernel while the fixture is from fp32 inputs: bf16 tolerance
  assert_close(out, g["out"], "out")
  assert_close(lse, g["lse"], "lse", max_abs=2e-2)
  assert_close(qd.grad, g["dq"], "dq", scale_abs=True)
  assert_close(kd.grad, g["dk"], "dk", scale_abs=True)
  assert_close(vd.grad, g["dv"], "dv", scale_abs=True)


@pytest.mark.gpu
def test_hip_llama_block_matches_golden_c1():
  """benchmark configuration 1 on the GPU in fp32 end to end: RMSNorm -> projections -> RoPE -> fp32 attention ->
  o_proj, at the fp32 tolerance class of the reference's own test of this shape
  (torchprime/torch_xla_models/tests/test_llama.py:143-188)."""
  import torchprime_amd as tpa

  dev = "cuda"
  x, w_norm, w = c1_inputs()
  x, w_norm = x.to(dev), w_norm.to(dev)
  w = {k_: v_.to(dev) for k_, v_ in w.items()}
  h = tpa.ops.rmsnorm(x, w_norm, 1e-5)
  B, S, hid, H, D = 2, 128, 512, 8, 64
  q = (h @ w["wq"].T).view(B, S, H, D).transpose(1, 2)
  k = (h @ w["wk"].T).view(B, S, H, D).transpose(1, 2)
  v = (h @ w["wv"].T).view(B, S, H, D).transpose(1, 2)
  rot = tpa.LlamaRotaryEmbedding(D, 500000.0).to(dev)
  cos, sin = rot(q, torch.arange(S, device=dev)[None].float())
  q, k = tpa.apply_rotary_pos_emb(q, k, cos, sin)
  cfg = tpa.Config(attention_kernel=None, num_attention_heads=H, num_key_value_heads=H, attention_dropout=False)
  mask = orc.causal_additive_mask(S).to(dev)
  old = torch.backends.cuda.matmul.allow_tf32
  torch.backends.cuda.matmul.allow_tf32 = False
  try:
    o = tpa.AttentionModule(cfg)(q, k, v, mask)
    assert o.dtype == torch.float32
    y = o.transpose(1, 2).contiguous().reshape(B, S, hid) @ w["wo"].T
  finally:
    torch.backends.cuda.matmul.allow_tf32 = old
  ref = _load("c1_llama_block.npz")["out_rows"]
  assert_close(y[:, ::8], ref, "C1 block", max_abs=2e-5, rel_l2=2e-5)
  # and with 16-bit attention, as the production configurations run it
  o16 = tpa.AttentionModule(cfg)(q.bfloat16(), k.bfloat16(), v.bfloat16(), mask).float()
  y16 = o16.transpose(1, 2).contiguous().reshape(B, S, hid) @ w["wo"].T
  assert_close(y16[:, ::8], ref, "C1 block, bf16 attention", max_abs=2e-2, rel_l2=1e-2)
