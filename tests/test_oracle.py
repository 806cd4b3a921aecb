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

def test_rms_norm_eager_order_grads_match_autograd_and_explicit_sum():
  """The gradient the reference's autograd produces: dw sums dy * (normalised value ROUNDED to the input dtype)."""
  g = torch.Generator().manual_seed(3)
  for dtype in (torch.bfloat16, torch.float32):
    x = torch.randn((6, 40, 64), generator=g).to(dtype)
    w = (1 + 0.1 * torch.randn((64,), generator=g)).to(dtype)
    dy = torch.randn((6, 40, 64), generator=g).to(dtype)
    dx, dw = orc.rms_norm_grads_eager_order(x, w, dy, 1e-5)
    # explicit form of dw
    h = x.double() * torch.rsqrt(x.double().pow(2).mean(-1, keepdim=True) + 1e-5)
    dw_explicit = (dy.double() * h.to(dtype).double()).sum((0, 1))
    torch.testing.assert_close(dw, dw_explicit, rtol=1e-12, atol=1e-12)
    # torch's own autograd through the eager expression in the input dtype (its sums round, hence the tolerance)
    xa, wa = x.clone().requires_grad_(True), w.clone().requires_grad_(True)
    orc.rms_norm(xa, wa, 1e-5).backward(dy)
    tol = dict(rtol=2e-2, atol=0.3) if dtype == torch.bfloat16 else dict(rtol=1e-4, atol=1e-4)
    torch.testing.assert_close(wa.grad.double(), dw, **tol)
    torch.testing.assert_close(xa.grad.double(), dx, **(dict(rtol=2e-2, atol=3e-2) if dtype == torch.bfloat16 else tol))
    if dtype == torch.float32:
      # fp32 input: the cast only rounds fp64 to fp32, so dw agrees with the exact-math gradient to fp32 precision
      # and dx, which does not see the rounded value, exactly
      x64, w64 = x.double().requires_grad_(True), w.double().requires_grad_(True)
      orc.rms_norm_exact(x64, w64, 1e-5).backward(dy.double())
      torch.testing.assert_close(dw, w64.grad, rtol=1e-5, atol=1e-5)
      torch.testing.assert_close(dx, x64.grad, rtol=1e-12, atol=1e-12)

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
  with um.patch.object(orc, "allowed_mask", lambda seg, ql, kl, c, *rest: torch.tensor([[[True, False, False], [False, False, False], [True, True, True]]])):
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


def test_llama_decoder_layer_matches_hf_when_available():
  """The whole layer (norms, attention, SwiGLU MLP, both residual adds) against HuggingFace's LlamaDecoderLayer."""
  try:
    from transformers import LlamaConfig
    from transformers.models.llama.modeling_llama import LlamaDecoderLayer, LlamaRotaryEmbedding
    cfg = LlamaConfig(hidden_size=256, num_attention_heads=4, num_key_value_heads=2, head_dim=64, intermediate_size=384,
                      num_hidden_layers=1, vocab_size=128, rms_norm_eps=1e-5, rope_theta=500000.0, attention_bias=False,
                      mlp_bias=False, hidden_act="silu", max_position_embeddings=8192)
    cfg._attn_implementation = "eager"
    torch.manual_seed(1)
    layer, rot = LlamaDecoderLayer(cfg, 0).eval(), LlamaRotaryEmbedding(cfg)
    x = randn((2, 48, 256), 29)
    with torch.no_grad():
      layer.input_layernorm.weight.copy_(1 + randn((256,), 30, std=0.05))
      layer.post_attention_layernorm.weight.copy_(1 + randn((256,), 31, std=0.05))
      pos = torch.arange(48)[None]
      cos, sin = rot(x, pos)
      ref = layer(x, attention_mask=orc.causal_additive_mask(48), position_ids=pos, position_embeddings=(cos, sin))
      ref = ref[0] if isinstance(ref, tuple) else ref
  except Exception as e:
    pytest.skip(f"transformers Llama modules not usable here: {e}")
  w = {k: v.detach() for k, v in layer.state_dict().items()}
  got = orc.llama_decoder_layer(x, w, 4, 2, 1e-5, cos, sin)
  torch.testing.assert_close(got, ref, rtol=1e-4, atol=1e-5)


def _hf_llama_fixture(which):
  """The two models of the reference's own test (torch_xla_models/tests/test_llama.py:26-125): its HuggingFace configs
  (tests/hf_model_config/meta-llama-3-8b and meta-llama-3.1-405b: rope_theta 5e5, eps 1e-5, no biases, the 405B one
  with the Llama 3.1 rope scaling) cut down to hidden 512, 8 heads of 64, intermediate 64, one / two layers,
  vocabulary 128 / 256, seed 42."""
  from transformers import LlamaConfig
  from transformers import LlamaForCausalLM as HfLlamaForCausalLM
  common = dict(hidden_size=512, num_attention_heads=8, num_key_value_heads=8, head_dim=64, intermediate_size=64, rms_norm_eps=1e-5,
                rope_theta=500000.0, attention_bias=False, attention_dropout=0.0, hidden_act="silu", initializer_range=0.02,
                tie_word_embeddings=False, use_cache=False)
  if which == "llama3_8b":
    cfg = LlamaConfig(vocab_size=128, num_hidden_layers=1, max_position_embeddings=8192, **common)
    scaling = None
  else:
    cfg = LlamaConfig(vocab_size=256, num_hidden_layers=2, max_position_embeddings=131072, mlp_bias=False,
                      rope_scaling={"factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                                    "original_max_position_embeddings": 8192, "rope_type": "llama3"}, **common)
    scaling = (8.0, 1.0, 4.0, 8192)
  cfg._attn_implementation = "eager"
  torch.manual_seed(42)
  return HfLlamaForCausalLM(cfg), cfg.vocab_size, scaling


@pytest.mark.parametrize("which", ["llama3_8b", "llama3_1_405b"])
@pytest.mark.parametrize("input_size", [8, 128, 256])
def test_llama_for_causal_lm_matches_hf_when_available(which, input_size):
  """The reference's test_forward_and_backward_our_model_against_hf_model with the oracle in the model's place: same
  fixtures, input sizes, inputs (labels = input ids, a mask of ones) and the reference's tolerances for loss and
  gradients (1e-4, 1e-5); logits to 2e-6 where the reference (on XLA) asks 1e-6: the softmax scale is a division in
  the reference and the oracle, a product in HuggingFace."""
  try:
    hf, vocab, scaling = _hf_llama_fixture(which)
    ids = torch.randint(vocab, (2, input_size // 2), generator=torch.Generator().manual_seed(input_size))
    hf.zero_grad()
    out = hf(input_ids=ids, labels=ids, attention_mask=torch.ones_like(ids))
    out.loss.backward()
  except Exception as e:
    pytest.skip(f"transformers LlamaForCausalLM not usable here: {e}")
  w = {k: v.detach().clone().requires_grad_(True) for k, v in hf.state_dict().items()}
  logits, loss = orc.llama_for_causal_lm(ids, ids, w, 8, 8, 1e-5, 500000.0, scaling, attention_mask=torch.ones_like(ids))
  loss.backward()
  torch.testing.assert_close(logits, out.logits, atol=2e-6, rtol=1e-9)
  torch.testing.assert_close(loss, out.loss, atol=1e-4, rtol=1e-7)
  for name, p in hf.named_parameters():
    assert w[name].grad is not None, name
    torch.testing.assert_close(w[name].grad, p.grad, atol=1e-5, rtol=1e-9, msg=lambda m, name=name: f"{name}: {m}")


# ---- the callers ------------------------------------------------------------------------------------------
def test_mixtral_attention_is_llama_attention_with_gathered_tables():
  B, S, H, Hkv, hd = 2, 12, 4, 2, 16
  hidden = H * hd
  x = randn((B, S, hidden), 31).double()
  wq, wk, wv, wo = (randn(s, 32 + i, std=0.1).double() for i, s in enumerate(((hidden, hidden), (Hkv * hd, hidden), (Hkv * hd, hidden), (hidden, hidden))))
  theta, max_pos = 1e6, 64
  pos = torch.arange(S)[None].expand(B, S)
  y = orc.mixtral_attention(x, wq, wk, wv, wo, H, Hkv, theta, max_pos, pos)
  cos, sin = orc.rotary_cos_sin(orc.default_rope_frequencies(hd, theta), torch.arange(S)[None].float(), torch.float32)
  y_llama = orc.llama_attention(x, wq, wk, wv, wo, H, Hkv, cos.double(), sin.double())
  torch.testing.assert_close(y, y_llama, rtol=1e-6, atol=1e-6)
  # other per-batch position ids: the tables are read at those rows (model/mixtral/model.py:136-137).  The rotary
  # module hands over the first S rows only (model/mixtral/model.py:100-103), so ids stay below S.
  pos2 = torch.stack([torch.arange(S).flip(0), (torch.arange(S) * 5) % S])
  y2 = orc.mixtral_attention(x, wq, wk, wv, wo, H, Hkv, theta, max_pos, pos2)
  c2, s2 = orc.rotary_cos_sin(orc.default_rope_frequencies(hd, theta), pos2.float(), torch.float32)
  torch.testing.assert_close(y2, orc.llama_attention(x, wq, wk, wv, wo, H, Hkv, c2.double(), s2.double()), rtol=1e-6, atol=1e-6)
  assert (y2 - y).abs().max() > 1e-3
  with pytest.raises(IndexError):  # an id beyond the rows handed over fails like the reference's cos[position_ids]
    orc.mixtral_attention(x, wq, wk, wv, wo, H, Hkv, theta, max_pos, pos + 1)
  # a table cached in bf16 is what reaches the rotation (trap: the default dtype at construction)
  y_bf = orc.mixtral_attention(x, wq, wk, wv, wo, H, Hkv, theta, max_pos, pos, table_dtype=torch.bfloat16)
  y_bf_ref = orc.llama_attention(x, wq, wk, wv, wo, H, Hkv, cos.bfloat16().double(), sin.bfloat16().double())
  torch.testing.assert_close(y_bf, y_bf_ref, rtol=1e-6, atol=1e-6)


def _mla_case(q_lora=True, seed=41):
  B, S, H, nope, rope, vd, kvl, ql, hidden = 2, 10, 3, 8, 6, 8, 12, 10, 20
  w = {
    "kv_a_proj_with_mqa": randn((kvl + rope, hidden), seed + 1, std=0.3), "kv_a_layernorm": 1 + randn((kvl,), seed + 2, std=0.1),
    "kv_b_proj": randn((H * (nope + vd), kvl), seed + 3, std=0.3), "o_proj": randn((hidden, H * vd), seed + 4, std=0.3),
  }
  if q_lora:
    w.update({"q_a_proj": randn((ql, hidden), seed + 5, std=0.3), "q_a_layernorm": 1 + randn((ql,), seed + 6, std=0.1),
              "q_b_proj": randn((H * (nope + rope), ql), seed + 7, std=0.3)})
  else:
    w["q_proj"] = randn((H * (nope + rope), hidden), seed + 8, std=0.3)
  w = {k: v.double() for k, v in w.items()}
  x = randn((B, S, hidden), seed).double()
  inv = orc.default_rope_frequencies(rope, 10000.0)
  pos = torch.arange(S)[None].float()
  cos, sin = orc.rotary_cos_sin(inv, pos, torch.float64)
  return x, w, (B, S, H, nope, rope, vd, kvl), cos, sin, inv


@pytest.mark.parametrize("q_lora", [True, False])
def test_deepseek_attention_against_brute_force_mla(q_lora):
  """Explicit per-(batch, head, query) loops; the rotary part of the scores is computed as a complex rotation of
  ADJACENT pairs (x_2i + i x_2i+1) e^{i p f_i}, which never builds the [evens | odds] layout."""
  x, w, (B, S, H, nope, rope, vd, kvl), cos, sin, inv = _mla_case(q_lora)
  y = orc.deepseek_v3_attention(x, w, H, nope, rope, vd, kvl, cos, sin, rope_interleave=True)

  def rms(t, g):
    return g * t / torch.sqrt(t.pow(2).mean(-1, keepdim=True) + 1e-6)

  q = (x @ w["q_proj"].T) if not q_lora else rms(x @ w["q_a_proj"].T, w["q_a_layernorm"]) @ w["q_b_proj"].T
  q = q.view(B, S, H, nope + rope)
  ckv = x @ w["kv_a_proj_with_mqa"].T
  kvb = (rms(ckv[..., :kvl], w["kv_a_layernorm"]) @ w["kv_b_proj"].T).view(B, S, H, nope + vd)
  k_rot = ckv[..., kvl:]  # (B, S, rope), one head
  ang = torch.arange(S)[:, None].double() * inv.double()[None]  # (S, rope/2)
  e = torch.polar(torch.ones_like(ang), ang)
  zq = torch.complex(q[..., nope::2], q[..., nope + 1 :: 2]) * e[None, :, None]  # (B,S,H,rope/2)
  zk = torch.complex(k_rot[..., 0::2], k_rot[..., 1::2]) * e[None]                # (B,S,rope/2)
  out = torch.zeros(B, S, H * vd, dtype=torch.float64)
  for b in range(B):
    for h in range(H):
      for i in range(S):
        sc = torch.empty(i + 1, dtype=torch.float64)
        for j in range(i + 1):
          sc[j] = (q[b, i, h, :nope] * kvb[b, j, h, :nope]).sum() + (zq[b, i, h] * zk[b, j].conj()).real.sum()
        p = torch.softmax(sc / math.sqrt(vd), 0)  # scale from v's head dim (attention.py:54-58)
        out[b, i, h * vd : (h + 1) * vd] = (p[:, None] * kvb[b, : i + 1, h, nope:]).sum(0)
  # (the oracle's tables are fp32 values, the loops above use fp64 angles: agreement to fp32 precision)
  torch.testing.assert_close(y, out @ w["o_proj"].T, rtol=1e-5, atol=5e-6)


def test_deepseek_attention_equals_attention_ref_with_expanded_k_rot_and_k_rot_grad_sums_heads():
  x, w, (B, S, H, nope, rope, vd, kvl), cos, sin, inv = _mla_case(True, seed=51)
  for il in (True, False):
    xr = x.clone().requires_grad_(True)
    wr = {k: v.clone().requires_grad_(True) for k, v in w.items()}
    y = orc.deepseek_v3_attention(xr, wr, H, nope, rope, vd, kvl, cos, sin, rope_interleave=il)
    # the same pipeline by hand: k_rot copied per head (separate leaves), attention_ref instead of the eager branch
    q = (orc.rms_norm(x @ w["q_a_proj"].T, w["q_a_layernorm"], 1e-6) @ w["q_b_proj"].T).view(B, S, H, nope + rope).transpose(1, 2)
    ckv = x @ w["kv_a_proj_with_mqa"].T
    kvb = (orc.rms_norm(ckv[..., :kvl], w["kv_a_layernorm"], 1e-6) @ w["kv_b_proj"].T).view(B, S, H, nope + vd).transpose(1, 2)
    k_rot_heads = ckv[..., kvl:].view(B, 1, S, rope).repeat(1, H, 1, 1).detach().requires_grad_(True)
    fn = orc.apply_rotary_pos_emb_interleave if il else orc.apply_rotary_pos_emb
    q_rot, k_rot = fn(q[..., nope:], k_rot_heads, cos, sin)
    qq, kk = torch.cat((q[..., :nope], q_rot), -1), torch.cat((kvb[..., :nope], k_rot), -1)
    o, _ = orc.attention_ref(qq, kk, kvb[..., nope:], None, True, 1 / math.sqrt(vd), torch.float64)
    y2 = o.transpose(1, 2).reshape(B, S, -1) @ w["o_proj"].T
    # (the eager branch takes its softmax in fp32, attention.py:163-165: agreement to fp32 precision)
    torch.testing.assert_close(y, y2, rtol=1e-5, atol=2e-6)
    # gradient reaching the single rotated k head = sum over heads of the per-head gradients
    do = randn(tuple(y.shape), 77).double()
    y.backward(do)
    (g_heads,) = torch.autograd.grad(y2, k_rot_heads, do)
    g_shared = g_heads.sum(1)  # (B,S,rope): d/d(ckv[..., kvl:]) through the rotated part only
    # route it into kv_a_proj_with_mqa's rows of the rotated dims and compare with autograd of the block
    gw = torch.einsum("bsr,bsh->rh", g_shared, x)
    torch.testing.assert_close(wr["kv_a_proj_with_mqa"].grad[kvl:], gw, rtol=1e-4, atol=1e-5)


# ---- the steps either side of the path ----------------------------------------------------------------------
def test_l2_norm_and_add_rms_norm_reduce_to_library_routines():
  x = randn((3, 5, 4, 32), 61)
  torch.testing.assert_close(orc.l2_norm(x, 1e-6), F.rms_norm(x, (32,), None, 1e-6), rtol=1e-6, atol=1e-6)
  xb = x.bfloat16()
  ref = torch.empty_like(x)
  for idx in np.ndindex(3, 5, 4):
    row = xb[idx].double()
    ref[idx] = (row / math.sqrt((row * row).mean().item() + 1e-6)).float()
  assert torch.equal(orc.l2_norm(xb, 1e-6), ref.bfloat16())  # fp32 math, one rounding at the end
  h, r, w = randn((4, 7, 64), 62).bfloat16(), randn((4, 7, 64), 63).bfloat16(), (1 + randn((64,), 64, std=0.1)).bfloat16()
  y, s = orc.add_rms_norm(h, r, w, 1e-5)
  assert torch.equal(s, (r.float() + h.float()).bfloat16()) and torch.equal(y, orc.rms_norm(s, w, 1e-5))


def test_llama4_rotary_is_adjacent_pair_complex_rotation():
  B, S, N, D = 2, 9, 3, 16
  q, k = randn((B, S, N, D), 65).double(), randn((B, S, 2, D), 66).double()
  inv = orc.default_rope_frequencies(D, 500000.0)
  pos = torch.arange(S)[None].float() * 5
  cos, sin = orc.rotary_cos_sin(inv, pos, torch.float32)
  qo, ko = orc.apply_rotary_emb_llama4(q, k, cos.double(), sin.double())
  ang = pos[0, :, None].double() * inv.double()[None]
  e = torch.polar(torch.ones_like(ang), ang)[None, :, None]  # (1, S, 1, D/2)
  for x, xo in ((q, qo), (k, ko)):
    z = torch.complex(x[..., 0::2], x[..., 1::2]) * e
    torch.testing.assert_close(xo[..., 0::2], z.real, rtol=1e-6, atol=1e-6)
    torch.testing.assert_close(xo[..., 1::2], z.imag, rtol=1e-6, atol=1e-6)
    torch.testing.assert_close(xo.norm(dim=-1), x.norm(dim=-1), rtol=1e-6, atol=1e-6)


def test_attn_temperature_closed_form():
  sc = orc.attn_temperature_scales(20000, 8192.0, 0.1)
  assert sc[0].item() == 1.0 and sc[8190].item() == 1.0  # floor((p+1)/8192) = 0 below position 8191
  assert sc[8191].item() == pytest.approx(math.log(2.0) * 0.1 + 1.0, rel=1e-6)
  assert sc[16383].item() == pytest.approx(math.log(3.0) * 0.1 + 1.0, rel=1e-6)
  q = randn((2, 6, 2, 8), 67).bfloat16()
  out = orc.apply_attn_temperature(q, 2.0, 0.5)
  s6 = orc.attn_temperature_scales(6, 2.0, 0.5)
  assert torch.equal(out, (q.float() * s6.view(1, 6, 1, 1)).bfloat16())


@pytest.mark.parametrize("use_rope,qk_norm,temperature", [(True, True, False), (True, False, False), (False, False, True), (False, False, False)])
def test_llama4_attention_against_explicit_loops(use_rope, qk_norm, temperature):
  B, S, H, Hkv, hd = 1, 7, 4, 2, 8
  hidden = H * hd
  x = randn((B, S, hidden), 90).double()
  wq, wk, wv, wo = (randn(shape, 91 + i, std=0.2).double() for i, shape in
                    enumerate(((hidden, hidden), (Hkv * hd, hidden), (Hkv * hd, hidden), (hidden, hidden))))
  inv = orc.default_rope_frequencies(hd, 10000.0).double()
  pos = torch.arange(S).double() * 3
  ang = pos[:, None] * inv[None]  # (S, hd/2)
  cos = torch.cat([ang.cos(), ang.cos()], -1)[None]
  sin = torch.cat([ang.sin(), ang.sin()], -1)[None]
  eps, floor_scale, attn_scale = 1e-6, 2.0, 0.3
  out = orc.llama4_attention(x, wq, wk, wv, wo, H, Hkv, cos, sin, use_rope, qk_norm, eps, temperature, floor_scale, attn_scale)
  # explicit form
  q = (x[0] @ wq.T).view(S, H, hd)
  k = (x[0] @ wk.T).view(S, Hkv, hd)
  v = (x[0] @ wv.T).view(S, Hkv, hd)
  def prep(t, i, n):
    vec = t[i, n].clone()
    if use_rope:
      z = torch.complex(vec[0::2], vec[1::2]) * torch.polar(torch.ones(hd // 2, dtype=torch.float64), ang[i])
      vec = torch.stack([z.real, z.imag], -1).reshape(hd)
      if qk_norm:
        vec = vec / math.sqrt((vec * vec).mean().item() + eps)
    return vec
  merged = torch.zeros(S, hidden, dtype=torch.float64)
  for h in range(H):
    for i in range(S):
      qi = prep(q, i, h)
      if temperature and not use_rope:
        qi = qi * (math.log(math.floor((i + 1.0) / floor_scale) + 1.0) * attn_scale + 1.0)
      sc = torch.tensor([float(qi @ prep(k, j, h // (H // Hkv))) / math.sqrt(hd) for j in range(i + 1)], dtype=torch.float64)
      p_ = torch.softmax(sc, 0)
      merged[i, h * hd : (h + 1) * hd] = sum(p_[j] * v[j, h // (H // Hkv)] for j in range(i + 1))
  # (the eager softmax is evaluated in fp32, attention.py:163-165: 1e-7-sized differences from the fp64 loops)
  torch.testing.assert_close(out[0], merged @ wo.T, rtol=2e-5, atol=2e-6)
  if use_rope and not qk_norm:
    # the adjacent-pair rotation is the rotate-half rotation on de-interleaved head dims, and q.k does not care
    perm = torch.cat([torch.arange(0, hd, 2), torch.arange(1, hd, 2)])
    pq = torch.cat([h * hd + perm for h in range(H)])
    pk = torch.cat([h * hd + perm for h in range(Hkv)])
    ref = orc.llama_attention(x, wq[pq], wk[pk], wv, wo, H, Hkv, cos, sin)
    torch.testing.assert_close(out, ref, rtol=2e-5, atol=2e-6)


def test_swiglu_and_cross_entropy_explicit_forms():
  g, u = randn((5, 24), 68).double(), randn((5, 24), 69).double()
  ref = torch.empty_like(g)
  for i, j in np.ndindex(5, 24):
    x = g[i, j].item()
    ref[i, j] = x / (1.0 + math.exp(-x)) * u[i, j].item()
  torch.testing.assert_close(orc.swiglu(g, u), ref, rtol=1e-12, atol=1e-12)
  B, S, V = 2, 7, 11
  logits = randn((B, S, V), 70).double()
  labels = torch.randint(0, V, (B, S), generator=torch.Generator().manual_seed(71))
  labels[0, 3] = -100
  labels[1, 0] = -100  # position 0's label is never a target: no effect
  total, n = 0.0, 0
  for b in range(B):
    for s in range(S - 1):
      lab = labels[b, s + 1].item()
      if lab == -100:
        continue
      row = logits[b, s]
      total += math.log(sum(math.exp(v) for v in row.tolist())) - row[lab].item()
      n += 1
  assert n == B * (S - 1) - 1
  assert orc.cross_entropy_loss(logits, labels, V).item() == pytest.approx(total / n, rel=1e-12)


# ---- mask extensions ---------------------------------------------------------------------------------------
def test_window_is_a_band_matrix_and_soft_cap_explicit():
  S = 23
  ones = torch.ones(S, S, dtype=torch.bool)
  for left, right in ((4, 0), (3, 5), (None, 2), (6, None), (0, 0)):
    band = ones.clone()
    if left is not None:
      band &= torch.triu(ones, diagonal=-left)
    if right is not None:
      band &= torch.tril(ones, diagonal=right)
    assert torch.equal(orc.allowed_mask(None, S, S, False, window=(left, right))[0], band)
    assert torch.equal(orc.allowed_mask(None, S, S, True, window=(left, right))[0], band & torch.tril(ones))
  q, k, v = randn((1, 2, 5, 8), 81).double(), randn((1, 2, 5, 8), 82).double(), randn((1, 2, 5, 8), 83).double()
  out, _ = orc.attention_ref(q, k, v, None, True, 0.4, torch.float64, soft_cap=1.5)
  for h in range(2):
    for i in range(5):
      sc = [1.5 * math.tanh(0.4 * float((q[0, h, i] * k[0, h, j]).sum()) / 1.5) for j in range(i + 1)]
      p = torch.softmax(torch.tensor(sc, dtype=torch.float64), 0)
      torch.testing.assert_close(out[0, h, i], (p[:, None] * v[0, h, : i + 1]).sum(0), rtol=1e-10, atol=1e-12)


@pytest.mark.parametrize("cp_size", [2, 4])
def test_load_balanced_causal_mask_is_causal_attention_in_the_original_order(cp_size):
  """Queries in the striped order against keys in the original order under LoadBalancedCausalMask == plain causal
  attention on the original order, re-striped: reorder o attention o reorder^-1."""
  from torchprime_amd import parallelism_utils as pu

  B, H, S, D = 1, 2, 32, 8
  q, k, v = randn((B, H, S, D), 91).double(), randn((B, H, S, D), 92).double(), randn((B, H, S, D), 93).double()
  plain, _ = orc.attention_ref(q, k, v, None, True, None, torch.float64)
  mask = pu.LoadBalancedCausalMask(shape=(S, S), cp_size=cp_size)
  q_striped = pu.reorder_sequence(q, cp_size, seq_dim=2)
  out, _ = orc.attention_ref(q_striped, k, v, None, True, None, torch.float64, q_positions=mask.q_sequence)
  torch.testing.assert_close(out, pu.reorder_sequence(plain, cp_size, seq_dim=2), rtol=1e-12, atol=1e-12)
  assert torch.equal(orc.allowed_mask(None, S, S, True, q_positions=mask.q_sequence)[0], torch.from_numpy(mask.dense()))
  off = pu.LoadBalancedCausalMask(shape=(S, S), cp_size=cp_size, offset=-3)
  assert torch.equal(orc.allowed_mask(None, S, S, True, q_positions=off.q_sequence, causal_offset=-3)[0], torch.from_numpy(off.dense()))
