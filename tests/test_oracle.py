"""Pins the CPU oracle (oracle/tprime_oracle.py) without importing the reference: against library
routines it must reduce to, closed forms, invariants and brute force, chosen so that a dropped term,
a wrong sign or index, or a transposed operand fails at least one check."""

import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import tprime_oracle as orc
from tests.util import packed_segment_ids, randn


# ---- RMSNorm ----------------------------------------------------------------------------------------
def test_rms_norm_reduces_to_library_routine_and_brute_force():
  x, w = randn((3, 5, 64), 1), 1 + randn((64,), 2, std=0.1)
  y = orc.rms_norm(x, w, 1e-5)
  torch.testing.assert_close(y, F.rms_norm(x, (64,), w, 1e-5), rtol=1e-5, atol=1e-6)
  xn = x.double().numpy()
  ref = np.empty_like(xn)
  for i in range(3):
    for j in range(5):
      ms = sum(float(v) ** 2 for v in xn[i, j]) / 64
      ref[i, j] = w.double().numpy() * xn[i, j] / math.sqrt(ms + 1e-5)
  np.testing.assert_allclose(y.double().numpy(), ref, rtol=2e-6, atol=1e-6)
  np.testing.assert_allclose(orc.rms_norm_exact(x, w, 1e-5).numpy(), ref, rtol=1e-12, atol=1e-12)


def test_rms_norm_invariants_and_rounding_order():
  x = randn((4, 128), 3)
  ones = torch.ones(128)
  y = orc.rms_norm(x, ones, 0.0)
  torch.testing.assert_close(y.pow(2).mean(-1), torch.ones(4), rtol=1e-5, atol=1e-5)  # unit RMS
  torch.testing.assert_close(orc.rms_norm(7.5 * x, ones, 0.0), y, rtol=1e-5, atol=1e-6)  # scale invariance
  assert orc.rms_norm(torch.zeros(2, 16), torch.ones(16), 1e-6).abs().max() == 0
  # the normalised value is rounded to the input dtype BEFORE the weight multiply (model.py:51-52)
  xb, wb = x.bfloat16(), (1 + randn((128,), 4, std=0.3)).bfloat16()
  n = (xb.float() * torch.rsqrt(xb.float().pow(2).mean(-1, keepdim=True) + 1e-5)).bfloat16()
  assert torch.equal(orc.rms_norm(xb, wb, 1e-5), wb * n)
  assert orc.rms_norm(xb, wb.float(), 1e-5).dtype == torch.float32  # fp32 weight promotes the result


# ---- inverse frequencies -------------------------------------------------------------------------------
@pytest.mark.parametrize("head_dim,theta", [(128, 500000.0), (128, 10000.0), (512, 500000.0), (64, 10000.0)])
def test_default_frequencies_closed_form(head_dim, theta):
  f = orc.default_rope_frequencies(head_dim, theta)
  ref = torch.tensor([theta ** (-2.0 * i / head_dim) for i in range(head_dim // 2)], dtype=torch.float64)
  assert f.dtype == torch.float32 and f.shape == (head_dim // 2,)
  torch.testing.assert_close(f.double(), ref, rtol=2e-6, atol=0)
  assert f[0] == 1.0


def _llmc_apply_scaling(freqs):
  """The llm.c loop the reference's own test restates (torchprime/tests/test_rope.py:83-108)."""
  scale_factor, low_ff, high_ff, old_ctx = 8, 1, 4, 8192
  low_wl, high_wl = old_ctx / low_ff, old_ctx / high_ff
  out = []
  for freq in freqs:
    wavelen = 2 * math.pi / freq
    if wavelen < high_wl:
      out.append(freq)
    elif wavelen > low_wl:
      out.append(freq / scale_factor)
    else:
      smooth = (old_ctx / wavelen - low_ff) / (high_ff - low_ff)
      out.append((1 - smooth) * freq / scale_factor + smooth * freq)
  return torch.tensor(out, dtype=freqs.dtype)


@pytest.mark.parametrize("hidden,heads", [(4096, 32), (16384, 128), (65536, 128)])  # test_rope.py:18-21
def test_llama3_frequencies_against_llmc_loop_and_hf(hidden, heads):
  hd = hidden // heads
  ours = orc.llama3_rope_frequencies(hd, 500000.0, factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0)
  torch.testing.assert_close(ours, _llmc_apply_scaling(orc.default_rope_frequencies(hd, 500000.0)))
  # three bands are all populated, so every branch is exercised
  base = orc.default_rope_frequencies(hd, 500000.0)
  assert (ours == base).any() and torch.isclose(ours, base / 8).any() and ((ours != base) & ~torch.isclose(ours, base / 8)).any()
  try:
    from transformers import LlamaConfig
    from transformers.modeling_rope_utils import ROPE_INIT_FUNCTIONS
    cfg = LlamaConfig(hidden_size=hidden, num_attention_heads=heads, max_position_embeddings=131072, rope_parameters={
      "rope_type": "llama3", "rope_theta": 500000.0, "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
      "original_max_position_embeddings": 8192})
    hf, scale = ROPE_INIT_FUNCTIONS["llama3"](cfg, device="cpu")
  except Exception as e:  # library absent or its config API differs: the llm.c pin above stands
    pytest.skip(f"transformers llama3 rope init not usable here: {e}")
  assert scale == 1
  torch.testing.assert_close(ours, hf)


def test_yarn_frequencies_special_cases_and_hf():
  # factor 1 (the DeepSeek-V3 yaml: max_position_embeddings == original, configs/model/deepseek-v3.yaml:15,43)
  inv, att = orc.yarn_rope_frequencies(64, 10000.0, 40, 4096, max_position_embeddings=4096, mscale=1.0, mscale_all_dim=1.0)
  torch.testing.assert_close(inv, orc.default_rope_frequencies(64, 10000.0))
  assert att == 1.0
  # factor 4: low dims keep the original frequency, high dims are interpolated (divided by 4)
  inv, att = orc.yarn_rope_frequencies(64, 10000.0, 4, 4096, max_position_embeddings=16384)
  base = orc.default_rope_frequencies(64, 10000.0)
  torch.testing.assert_close(inv[:4], base[:4])
  torch.testing.assert_close(inv[-4:], base[-4:] / 4)
  assert (inv <= base + 1e-12).all() and (inv >= base / 4 - 1e-12).all()
  assert att == pytest.approx(0.1 * math.log(4) + 1.0)
  try:
    from transformers import LlamaConfig
    from transformers.modeling_rope_utils import ROPE_INIT_FUNCTIONS
    cfg = LlamaConfig(hidden_size=512, num_attention_heads=8, head_dim=64, max_position_embeddings=16384, rope_parameters={
      "rope_type": "yarn", "rope_theta": 10000.0, "factor": 4.0, "original_max_position_embeddings": 4096,
      "beta_fast": 32, "beta_slow": 1})
    hf, hf_att = ROPE_INIT_FUNCTIONS["yarn"](cfg, device="cpu")
  except Exception as e:
    pytest.skip(f"transformers yarn rope init not usable here: {e}")
  torch.testing.assert_close(inv, hf)
  assert att == pytest.approx(hf_att)


def test_cos_sin_closed_form_and_dtype():
  inv = orc.default_rope_frequencies(16, 10000.0)
  pos = torch.tensor([[0.0, 1.0, 5.0, 8191.0]])
  cos, sin = orc.rotary_cos_sin(inv, pos, torch.float32)
  assert cos.shape == (1, 4, 16)
  for s, p in enumerate([0.0, 1.0, 5.0, 8191.0]):
    for i in range(8):
      ang = np.float32(p) * inv[i].numpy()  # fp32 product, as the K=1 matmul
      assert cos[0, s, i].item() == pytest.approx(math.cos(float(ang)), abs=1e-6)
      assert sin[0, s, i + 8].item() == pytest.approx(math.sin(float(ang)), abs=1e-6)
  c16, _ = orc.rotary_cos_sin(inv, pos, torch.bfloat16, attention_scaling=0.5)
  assert c16.dtype == torch.bfloat16 and torch.equal(c16, (cos * 0.5).bfloat16())


# ---- rotary apply ---------------------------------------------------------------------------------------
def _rope_case(B=2, Hq=4, Hkv=2, S=9, D=16, theta=10000.0, dtype=torch.float64):
  q, k = randn((B, Hq, S, D), 5).to(dtype), randn((B, Hkv, S, D), 6).to(dtype)
  pos = torch.arange(S)[None].float() * 3
  inv = orc.default_rope_frequencies(D, theta)
  cos, sin = orc.rotary_cos_sin(inv, pos, torch.float32)
  return q, k, cos.to(dtype), sin.to(dtype), pos, inv


def test_rotary_is_complex_rotation():
  q, k, cos, sin, pos, inv = _rope_case()
  qo, ko = orc.apply_rotary_pos_emb(q, k, cos, sin)
  half = q.shape[-1] // 2
  ang = pos[0, :, None].double() * inv.double()[None]  # (S, half)
  rot = torch.polar(torch.ones_like(ang), ang)
  for x, xo in ((q, qo), (k, ko)):
    z = torch.complex(x[..., :half], x[..., half:]) * rot  # pairs (i, i + D/2)
    torch.testing.assert_close(xo[..., :half], z.real, rtol=1e-6, atol=1e-6)
    torch.testing.assert_close(xo[..., half:], z.imag, rtol=1e-6, atol=1e-6)
    torch.testing.assert_close(xo.norm(dim=-1), x.norm(dim=-1), rtol=1e-6, atol=1e-6)  # norm preserved
  torch.testing.assert_close(qo[:, :, 0], q[:, :, 0])  # position 0 is the identity


def test_rotary_scores_depend_on_relative_position_only():
  D, inv = 16, orc.default_rope_frequencies(16, 10000.0)
  q, k = randn((1, 1, 1, D), 7).double(), randn((1, 1, 1, D), 8).double()
  def score(m, n):
    cm, sm = orc.rotary_cos_sin(inv, torch.tensor([[float(m)]]), torch.float64)
    cn, sn = orc.rotary_cos_sin(inv, torch.tensor([[float(n)]]), torch.float64)
    qm, _ = orc.apply_rotary_pos_emb(q, q, cm, sm)
    kn, _ = orc.apply_rotary_pos_emb(k, k, cn, sn)
    return (qm * kn).sum().item()
  assert score(5, 2) == pytest.approx(score(13, 10), abs=1e-5)
  assert score(5, 2) != pytest.approx(score(5, 3), abs=1e-3)


def test_rotary_interleave_is_permutation_then_rotate_half_and_gather_variant():
  q, k, cos, sin, pos, inv = _rope_case()
  D = q.shape[-1]
  perm = list(range(0, D, 2)) + list(range(1, D, 2))
  qi, ki = orc.apply_rotary_pos_emb_interleave(q, k, cos, sin)
  qp, kp = orc.apply_rotary_pos_emb(q[..., perm], k[..., perm], cos, sin)
  torch.testing.assert_close(qi, qp)
  torch.testing.assert_close(ki, kp)
  # same permutation on q and k: q.k unchanged relative to rotating the HF (non-interleaved pairs) way
  z = lambda x: torch.complex(x[..., 0::2], x[..., 1::2])
  ang = pos[0, :, None].double() * inv.double()[None]
  rot = torch.polar(torch.ones_like(ang), ang)
  s_ref = torch.einsum("bhsd,bgtd->bhgst", torch.view_as_real(z(q) * rot).flatten(-2), torch.view_as_real(z(k) * rot).flatten(-2))
  s_got = torch.einsum("bhsd,bgtd->bhgst", qi, ki)
  torch.testing.assert_close(s_got, s_ref, rtol=1e-6, atol=1e-6)
  # Mixtral: tables gathered by integer positions
  table_pos = torch.arange(40)[None].float()
  ct, st = orc.rotary_cos_sin(inv, table_pos, torch.float64)
  ids = (pos[0].long())[None]
  qg, kg = orc.apply_rotary_pos_emb(q, k, ct[0], st[0], ids, gather=True)
  torch.testing.assert_close(qg, orc.apply_rotary_pos_emb(q, k, cos, sin)[0], rtol=1e-6, atol=1e-6)


# ---- attention -------------------------------------------------------------------------------------------
def test_repeat_kv_is_repeat_interleave():
  x = randn((2, 3, 5, 4), 9)
  assert torch.equal(orc.repeat_kv(x, 4), torch.repeat_interleave(x, 4, dim=1))
  assert orc.repeat_kv(x, 1) is x


def test_eager_attention_reduces_to_sdpa_and_brute_force():
  B, Hq, Hkv, S, D = 2, 4, 2, 12, 8
  q, k, v = randn((B, Hq, S, D), 10).double(), randn((B, Hkv, S, D), 11).double(), randn((B, Hkv, S, D), 12).double()
  mask = orc.causal_additive_mask(S, torch.float64)
  out = orc.eager_attention(q, k, v, mask)
  sdpa = F.scaled_dot_product_attention(q, k, v, is_causal=True, scale=1 / math.sqrt(D), enable_gqa=True)
  torch.testing.assert_close(out, sdpa, rtol=1e-6, atol=1e-6)  # softmax runs in fp32 in the eager branch
  full = F.scaled_dot_product_attention(q, k, v, scale=1 / math.sqrt(D), enable_gqa=True)
  torch.testing.assert_close(orc.eager_attention(q, k, v, None), full, rtol=1e-6, atol=1e-6)
  # brute force: explicit loops, kv head = h // n_rep, scale by sqrt of V's head dim
  ref = torch.zeros(B, Hq, S, D, dtype=torch.float64)
  for b in range(B):
    for h in range(Hq):
      g = h // (Hq // Hkv)
      for i in range(S):
        sc = [sum(q[b, h, i, d].item() * k[b, g, j, d].item() for d in range(D)) / math.sqrt(D) for j in range(i + 1)]
        mx = max(sc)
        e = [math.exp(s - mx) for s in sc]
        z = sum(e)
        for j in range(i + 1):
          ref[b, h, i] += (e[j] / z) * v[b, g, j]
  torch.testing.assert_close(out, ref, rtol=1e-6, atol=1e-6)
  torch.testing.assert_close(out[:, :, 0], orc.repeat_kv(v, 2)[:, :, 0], rtol=1e-6, atol=1e-6)  # row 0 sees only key 0


def test_eager_scale_uses_v_head_dim():
  # attention.py:54-58: head_dim := value_states.shape[-1], so qk dim 24 / v dim 16 scales by 1/sqrt(16)
  q, k, v = randn((1, 2, 6, 24), 13).double(), randn((1, 2, 6, 24), 14).double(), randn((1, 2, 6, 16), 15).double()
  out = orc.eager_attention(q, k, v, None)
  w = torch.softmax(q @ k.transpose(2, 3) / 4.0, -1)
  torch.testing.assert_close(out, w @ v, rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("causal", [True, False])
def test_attention_ref_matches_eager_and_segments_decompose(causal):
  B, Hq, Hkv, S, D = 2, 4, 2, 40, 8
  q, k, v = randn((B, Hq, S, D), 16).double(), randn((B, Hkv, S, D), 17).double(), randn((B, Hkv, S, D), 18).double()
  out, lse = orc.attention_ref(q, k, v, None, causal, None, torch.float64)
  mask = orc.causal_additive_mask(S, torch.float64) if causal else None
  torch.testing.assert_close(out, orc.eager_attention(q, k, v, mask), rtol=1e-6, atol=1e-6)
  s = q @ orc.repeat_kv(k, 2).transpose(2, 3) / math.sqrt(D)
  if causal:
    s = s + mask
  torch.testing.assert_close(lse, torch.logsumexp(s, -1))
  # segments: equal to running each document alone (block-diagonal decomposition)
  seg, lengths = packed_segment_ids(B, S, 3, 15, seed=2)
  out_s, lse_s = orc.attention_ref(q, k, v, seg, causal, None, torch.float64)
  for b in range(B):
    pos = 0
    for L in lengths[b]:
      sl = slice(pos, pos + L)
      o, l = orc.attention_ref(q[b : b + 1, :, sl], k[b : b + 1, :, sl], v[b : b + 1, :, sl], None, causal, None, torch.float64)
      torch.testing.assert_close(out_s[b : b + 1, :, sl], o)
      torch.testing.assert_close(lse_s[b : b + 1, :, sl], l)
      pos += L
  am = orc.allowed_mask(seg, S, S, causal)
  i, j = 7, 3
  assert am[0, i, j].item() == ((j <= i or not causal) and seg[0, i] == seg[0, j])
  assert am.any(-1).all()  # a token always sees itself: no fully-masked row can arise from this mask


def test_attention_ref_fully_masked_row_convention():
  # forced through the internals: a -inf row gives out = 0 and lse = -inf (the eager formula gives NaN)
  q = randn((1, 1, 3, 4), 19).double()
  s = torch.full((1, 1, 3, 3), float("-inf"))
  assert torch.isnan(torch.softmax(s, -1)).all()
  import unittest.mock as um
  with um.patch.object(orc, "allowed_mask", lambda seg, ql, kl, c: torch.tensor([[[True, False, False], [False, False, False], [True, True, True]]])):
    out, lse = orc.attention_ref(q, q, q, None, True, None, torch.float64)
  assert out[0, 0, 1].abs().max() == 0 and lse[0, 0, 1] == float("-inf")
  assert torch.isfinite(out).all() and torch.isfinite(lse[0, 0, [0, 2]]).all()


def test_attention_grads_gradcheck_and_gqa_group_sum():
  B, Hq, Hkv, S, D = 1, 4, 2, 6, 4
  q, k, v = (randn(sh, sd).double().requires_grad_(True) for sh, sd in (((B, Hq, S, D), 20), ((B, Hkv, S, D), 21), ((B, Hkv, S, D), 22)))
  seg = torch.tensor([[0, 0, 0, 1, 1, 1]], dtype=torch.int32)
  f = lambda a, b, c: orc.attention_ref(a, b, c, seg, True, 0.37, torch.float64)[0]
  assert torch.autograd.gradcheck(f, (q, k, v), eps=1e-6, atol=1e-5)
  do = randn((B, Hq, S, D), 23).double()
  _, dq, dk, dv = orc.attention_grads_ref(q, k, v, do, seg, True, 0.37, torch.float64)
  # MHA on expanded K/V: dK/dV of GQA are the sums over each group
  ke, ve = orc.repeat_kv(k.detach(), 2).requires_grad_(True), orc.repeat_kv(v.detach(), 2).requires_grad_(True)
  _, dq2, dke, dve = orc.attention_grads_ref(q, ke, ve, do, seg, True, 0.37, torch.float64)
  torch.testing.assert_close(dq, dq2)
  torch.testing.assert_close(dk, dke.view(B, Hkv, 2, S, D).sum(2))
  torch.testing.assert_close(dv, dve.view(B, Hkv, 2, S, D).sum(2))


def test_attention_ref_chunked_equals_whole():
  q, k, v = randn((1, 8, 33, 8), 24), randn((1, 2, 33, 8), 25), randn((1, 2, 33, 8), 26)
  a, la = orc.attention_ref(q, k, v)
  b, lb = orc.attention_ref_chunked(q, k, v, heads_per_chunk=4)
  torch.testing.assert_close(a, b)
  torch.testing.assert_close(la, lb)


def test_llama_block_matches_hf_llama_when_available():
  """C1 shape (the reference's own test fixture, torch_xla_models/tests/test_llama.py:26-64): the oracle's
  attention block against HuggingFace's Llama attention + input norm, as the reference's tests do."""
  try:
    from transformers import LlamaConfig
    from transformers.models.llama.modeling_llama import LlamaAttention, LlamaRMSNorm, LlamaRotaryEmbedding
    cfg = LlamaConfig(hidden_size=512, num_attention_heads=8, num_key_value_heads=8, head_dim=64, intermediate_size=64,
                      num_hidden_layers=1, vocab_size=128, rms_norm_eps=1e-5, rope_theta=500000.0, attention_bias=False,
                      max_position_embeddings=8192)
    cfg._attn_implementation = "eager"
    torch.manual_seed(0)
    attn, norm, rot = LlamaAttention(cfg, 0).eval(), LlamaRMSNorm(512, 1e-5), LlamaRotaryEmbedding(cfg)
    x = randn((2, 128, 512), 27)
    with torch.no_grad():
      norm.weight.copy_(1 + randn((512,), 28, std=0.02))
      pos = torch.arange(128)[None]
      mask = orc.causal_additive_mask(128)
      ref = attn(norm(x), position_embeddings=rot(x, pos), attention_mask=mask)[0]
  except Exception as e:
    pytest.skip(f"transformers Llama modules not usable here: {e}")
  got = orc.llama_attention_block(x, norm.weight.detach(), attn.q_proj.weight.detach(), attn.k_proj.weight.detach(),
                                  attn.v_proj.weight.detach(), attn.o_proj.weight.detach(), 8, 8, 1e-5, 500000.0)
  torch.testing.assert_close(got, ref, rtol=1e-4, atol=1e-5)
