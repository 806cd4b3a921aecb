"""GPU parity of the mask extensions (sliding window, logits soft cap, load-balanced causal mask with query rows in
the striped order) through the ops, the functional wrapper and AttentionModule, against the CPU oracle: forward,
gradients and the exact support of P."""

import math

import pytest
import torch

import torchprime_amd as tpa
from oracle import tprime_oracle as orc
from tests.util import assert_close, heads_view, packed_segment_ids
from torchprime_amd import parallelism_utils as pu

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _check(B, Hq, Hkv, S, D, dtype=torch.bfloat16, causal=True, seg=None, window=None, soft_cap=None, q_positions=None,
           causal_offset=0, Skv=None, seed=0, Dv=None):
  Skv = S if Skv is None else Skv
  Dv = D if Dv is None else Dv
  q, k, v, do = (heads_view(B, h, s_, d, seed + i, dtype)
                 for i, (h, s_, d) in enumerate(((Hq, S, D), (Hkv, Skv, D), (Hkv, Skv, Dv), (Hq, S, Dv))))
  sm = 1.0 / math.sqrt(Dv)
  qd, kd, vd = (t.to(DEV).requires_grad_(True) for t in (q, k, v))
  qp = None if q_positions is None else torch.as_tensor(q_positions).to(DEV)
  out = tpa.ops.attention(qd, kd, vd, None if seg is None else seg.to(DEV), sm, causal, window=window, soft_cap=soft_cap,
                          q_positions=qp, causal_offset=causal_offset)
  out.backward(do.to(DEV))
  kw = dict(window=window, soft_cap=soft_cap, q_positions=q_positions, causal_offset=causal_offset)
  o_ref, dq_ref, dk_ref, dv_ref = orc.attention_grads_ref(q, k, v, do, seg, causal, sm, torch.float64, **kw)
  assert_close(out, o_ref, "out")
  assert_close(qd.grad, dq_ref, "dq", scale_abs=True)
  assert_close(kd.grad, dk_ref, "dk", scale_abs=True)
  assert_close(vd.grad, dv_ref, "dv", scale_abs=True)


@pytest.mark.parametrize("D", [128, 64])
@pytest.mark.parametrize("causal,window", [(True, (100, 100)), (True, (17, None)), (False, (64, 64)), (False, (0, 200)), (False, (300, None)),
                                            (True, (1000, 1000))])
def test_sliding_window_fwd_bwd(D, causal, window):
  _check(2, 4, 2, 520, D, causal=causal, window=window)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_sliding_window_with_segments_and_ragged_kv(dtype):
  seg, _ = packed_segment_ids(2, 333, 10, 150, seed=2)
  _check(2, 4, 2, 333, 128, dtype=dtype, causal=True, seg=seg, window=(40, 40))
  _check(1, 2, 1, 130, 64, dtype=dtype, causal=False, window=(50, 20), Skv=300)


@pytest.mark.parametrize("D,causal", [(128, True), (64, True), (128, False)])
def test_soft_cap_fwd_bwd(D, causal):
  _check(1, 4, 2, 300, D, causal=causal, soft_cap=2.0)       # caps visibly: |logit| reaches ~3 with N(0,1) inputs
  _check(1, 2, 2, 200, D, causal=causal, soft_cap=30.0, window=(64, 64) if not causal else None)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_mask_extensions_with_wide_heads(dtype):
  """qk head dim 192, v head dim 128 (the single-buffer dK/dV path and the four-wave dQ kernel): window, window with
  segment ids and a ragged kv length, soft cap, and the load-balanced causal order."""
  _check(1, 4, 4, 330, 192, dtype=dtype, causal=True, window=(70, 70), Dv=128, seed=3)
  _check(1, 4, 2, 200, 192, dtype=dtype, causal=False, window=(50, 20), Dv=128, Skv=300, seed=4)
  seg, _ = packed_segment_ids(2, 260, 10, 120, seed=5)
  _check(2, 4, 4, 260, 192, dtype=dtype, causal=True, seg=seg, window=(40, 40), Dv=128, seed=6)
  _check(1, 4, 2, 300, 192, dtype=dtype, causal=True, soft_cap=2.0, Dv=128, seed=7)
  _check(1, 2, 2, 200, 192, dtype=dtype, causal=False, soft_cap=5.0, window=(64, 64), Dv=128, seed=8)
  mask = pu.LoadBalancedCausalMask(shape=(256, 256), cp_size=4)
  _check(1, 4, 4, 256, 192, dtype=dtype, causal=True, q_positions=mask.q_sequence, Dv=128, seed=9)


@pytest.mark.parametrize("D", [64, 128])
def test_mask_extensions_fp32(D):
  """fp32 tensors through the fp32 kernels: window, window with segment ids and a ragged kv length, soft cap, the
  load-balanced causal order; fp32 class of tolerance against the fp64 oracle."""
  def check32(B, Hq, Hkv, S, seed, Skv=None, **kw):
    Skv_ = S if Skv is None else Skv
    q, k, v, do = (heads_view(B, h, s_, D, seed + i, torch.float32) for i, (h, s_) in enumerate(((Hq, S), (Hkv, Skv_), (Hkv, Skv_), (Hq, S))))
    sm = 1.0 / math.sqrt(D)
    qd, kd, vd = (t.to(DEV).requires_grad_(True) for t in (q, k, v))
    seg = kw.pop("seg", None)
    causal = kw.pop("causal", True)
    qp = kw.get("q_positions")
    out = tpa.ops.attention(qd, kd, vd, None if seg is None else seg.to(DEV), sm, causal, window=kw.get("window"), soft_cap=kw.get("soft_cap"),
                            q_positions=None if qp is None else torch.as_tensor(qp).to(DEV), causal_offset=kw.get("causal_offset", 0))
    assert out.dtype == torch.float32
    out.backward(do.to(DEV))
    o_ref, dq_ref, dk_ref, dv_ref = orc.attention_grads_ref(q, k, v, do, seg, causal, sm, torch.float64, **kw)
    for got, ref, name in ((out, o_ref, "out"), (qd.grad, dq_ref, "dq"), (kd.grad, dk_ref, "dk"), (vd.grad, dv_ref, "dv")):
      assert_close(got, ref, name, max_abs=2e-5 * max(1.0, ref.abs().max().item()), rel_l2=2e-5)

  check32(2, 4, 2, 200, 1, window=(50, 50))
  check32(1, 2, 1, 130, 2, causal=False, window=(50, 20), Skv=260)
  seg, _ = packed_segment_ids(2, 160, 10, 80, seed=3)
  check32(2, 4, 4, 160, 3, seg=seg, window=(30, 30))
  check32(1, 4, 2, 150, 4, soft_cap=2.0)
  check32(1, 2, 2, 140, 5, causal=False, soft_cap=5.0, window=(40, 40))
  mask = pu.LoadBalancedCausalMask(shape=(128, 128), cp_size=4)
  check32(1, 4, 2, 128, 6, q_positions=mask.q_sequence)
  check32(1, 2, 2, 128, 7, q_positions=mask.q_sequence, causal_offset=5)


@pytest.mark.parametrize("cp_size,D", [(2, 128), (4, 128), (4, 64)])
def test_load_balanced_causal_mask_fwd_bwd(cp_size, D):
  S = 512
  mask = pu.LoadBalancedCausalMask(shape=(S, S), cp_size=cp_size)
  _check(2, 4, 2, S, D, causal=True, q_positions=mask.q_sequence)
  _check(1, 2, 2, S, D, causal=True, q_positions=mask.q_sequence, causal_offset=5)


def test_rows_without_any_allowed_key_give_zero_output_and_gradients():
  """A negative causal offset leaves the first rows with no key at all: the kernels' convention for such rows,
  out = 0, lse = -inf, no gradient through them (where the eager formula would give NaN), executed on the device."""
  B, H, S, D, off = 1, 2, 200, 128, -7
  q, k, v, do = (heads_view(B, H, S, D, i, torch.bfloat16) for i in range(4))
  qd, kd, vd = (t.to(DEV).requires_grad_(True) for t in (q, k, v))
  out, lse = torch.ops.tprime.attn_fwd_masked(qd, kd, vd, None, None, D**-0.5, True, off, -1, -1, 0.0)
  out.backward(do.to(DEV))
  assert out[:, :, : -off].abs().max().item() == 0 and (lse[:, :, : -off] == float("-inf")).all()
  assert torch.isfinite(out.float()).all() and torch.isfinite(lse[:, :, -off:]).all()
  assert qd.grad[:, :, : -off].abs().max().item() == 0
  o_ref, dq_ref, dk_ref, dv_ref = orc.attention_grads_ref(q, k, v, do, None, True, D**-0.5, torch.float64, causal_offset=off)
  assert_close(out, o_ref, "out")
  assert_close(qd.grad, dq_ref, "dq", scale_abs=True)
  assert_close(kd.grad, dk_ref, "dk", scale_abs=True)
  assert_close(vd.grad, dv_ref, "dv", scale_abs=True)


@pytest.mark.parametrize("kind", ["window_causal", "window_full", "load_balanced", "window_segments"])
def test_mask_pattern_exact_extensions(kind):
  """The support of P, recovered through the public op with one-hot V blocks, equals the closed-form mask."""
  B, H, S, D = 1, 2, 192, 64
  kw, seg, causal = {}, None, True
  if kind == "window_causal":
    kw = dict(window=(37, 37))
  elif kind == "window_full":
    kw, causal = dict(window=(20, 45)), False
  elif kind == "load_balanced":
    kw = dict(q_positions=pu.LoadBalancedCausalMask(shape=(S, S), cp_size=4).q_sequence)
  else:
    kw, seg = dict(window=(50, 50)), packed_segment_ids(B, S, 5, 70, seed=4)[0]
  q = heads_view(B, H, S, D, 1, torch.bfloat16, 0.3).to(DEV)
  k = heads_view(B, H, S, D, 2, torch.bfloat16, 0.3).to(DEV)
  allowed = orc.allowed_mask(seg, S, S, causal, **kw)[0]
  dkw = {n: (torch.as_tensor(x).to(DEV) if n == "q_positions" else x) for n, x in kw.items()}
  P = torch.zeros((H, S, S))
  for j0 in range(0, S, D):
    v = torch.zeros((B, H, S, D), dtype=torch.bfloat16)
    for j in range(j0, min(j0 + D, S)):
      v[:, :, j, j - j0] = 1
    o = tpa.ops.attention(q, k, v.to(DEV), None if seg is None else seg.to(DEV), None, causal, **dkw)
    P[:, :, j0 : j0 + D] = o[0, :, :, : min(D, S - j0)].float().cpu()
  assert torch.equal(P > 0, allowed[None].expand_as(P)), "support of P differs from the mask"
  assert_close(P.sum(-1), torch.ones(H, S), "rows sum to 1", max_abs=2e-2)


def test_wrapper_and_module_paths():
  B, Hq, Hkv, S, D, cp = 2, 4, 2, 256, 128, 4
  q, k, v = (heads_view(B, h, S, D, s, torch.bfloat16) for h, s in ((Hq, 1), (Hkv, 2), (Hkv, 3)))
  qs = (q.float() / math.sqrt(D)).to(torch.bfloat16)  # callers pre-scale q (attention.py:107)
  # sliding window through the config JSON, soft cap through the argument (kernel_utils.py:266-275, 292)
  cfg = tpa.SplashAttentionConfig(attentiontype_local_sliding=True, slide_window_size=48).to_json()
  res = tpa.tpu_splash_attention_jax_call_wrapper(None, qs.to(DEV), k.to(DEV), v.to(DEV), cfg, None, True, attn_logits_soft_cap=20.0)
  ref, _ = orc.attention_ref(qs, k, v, None, True, 1.0, torch.float64, window=(48, 48), soft_cap=20.0)
  assert_close(res[0], ref, "window + soft cap via wrapper")
  # load-balanced causal mask object, causal=False as the reference passes it (attention.py:110-119)
  mask = pu.LoadBalancedCausalMask(shape=(S, S), cp_size=cp)
  res = tpa.tpu_splash_attention_jax_call_wrapper(mask, qs.to(DEV), k.to(DEV), v.to(DEV), None, None, False, q_seq_shards=cp)
  ref, _ = orc.attention_ref(qs, k, v, None, True, 1.0, torch.float64, q_positions=mask.q_sequence)
  assert_close(res[0], ref, "LoadBalancedCausalMask via wrapper")
  # AttentionModule with load_balance_cp: inputs in the striped order; equals plain causal attention on the original
  # order, re-striped
  cfgm = tpa.Config(attention_kernel="splash_attention", num_attention_heads=Hq, num_key_value_heads=Hkv, attention_dropout=False,
                    load_balance_cp=True, context=cp)
  striped = [pu.reorder_sequence(t, cp, seq_dim=2) for t in (q, k, v)]
  out = tpa.AttentionModule(cfgm)(*(t.to(DEV) for t in striped))
  plain, _ = orc.attention_ref(q, k, v, None, True, 1 / math.sqrt(D), torch.float64)
  assert_close(out, pu.reorder_sequence(plain, cp, seq_dim=2), "AttentionModule, load_balance_cp")
  plain_dev = tpa.AttentionModule(tpa.Config(attention_kernel="splash_attention"))(q.to(DEV), k.to(DEV), v.to(DEV))
  assert_close(out, pu.reorder_sequence(plain_dev.float().cpu(), cp, seq_dim=2), "vs the plain causal kernel")


@pytest.mark.parametrize("cp,offset", [(2, 0), (4, 0), (4, 3), (16, 0)])
def test_load_balanced_mask_fwd_bwd(cp, offset):
  """A load-balanced causal mask through the wrapper, forward and backward, against the oracle on the positions
  themselves (cp 2 .. 16: three to 31 runs of consecutive positions, down to 16 rows each)."""
  B, Hq, Hkv, S, D = 1, 4, 2, 512, 128
  q, k, v, do = (heads_view(B, h, S, D, 70 + i, torch.bfloat16) for i, h in enumerate((Hq, Hkv, Hkv, Hq)))
  mask = pu.LoadBalancedCausalMask(shape=(S, S), offset=offset, cp_size=cp)
  scale = 1 / math.sqrt(D)
  qd, kd, vd = (t.to(DEV).requires_grad_(True) for t in (q, k, v))
  out = tpa.tpu_splash_attention_jax_call_wrapper(mask, qd, kd, vd, None, None, False, q_seq_shards=cp, sm_scale=scale)[0]
  out.backward(do.to(DEV))
  o_ref, dq_ref, dk_ref, dv_ref = orc.attention_grads_ref(q, k, v, do, None, True, scale, torch.float32,
                                                          q_positions=mask.q_sequence, causal_offset=offset)
  assert_close(out, o_ref, "out")
  assert_close(qd.grad, dq_ref, "dq", scale_abs=True)
  assert_close(kd.grad, dk_ref, "dk", scale_abs=True)
  assert_close(vd.grad, dv_ref, "dv", scale_abs=True)


def test_full_size_sliding_window_slice():
  """Llama-3-8B layer shape with a 1024-token causal window: one (batch, kv group) slice against the oracle."""
  B, Hq, Hkv, S, D, W = 2, 32, 8, 8192, 128, 1024
  q, k, v, do = (heads_view(B, h, S, D, 40 + i, torch.bfloat16) for i, h in enumerate((Hq, Hkv, Hkv, Hq)))
  qd, kd, vd = (t.to(DEV).requires_grad_(True) for t in (q, k, v))
  out = tpa.ops.attention(qd, kd, vd, None, None, True, window=(W, W))
  out.backward(do.to(DEV))
  b, g = 1, 3
  hs = slice(g * 4, g * 4 + 4)
  o_ref, dq_ref, dk_ref, dv_ref = orc.attention_grads_ref(q[b : b + 1, hs], k[b : b + 1, g : g + 1], v[b : b + 1, g : g + 1], do[b : b + 1, hs],
                                                          None, True, None, torch.float32, window=(W, W))
  assert_close(out[b : b + 1, hs], o_ref, "out")
  assert_close(qd.grad[b : b + 1, hs], dq_ref, "dq", scale_abs=True)
  assert_close(kd.grad[b : b + 1, g : g + 1], dk_ref, "dk", scale_abs=True)
  assert_close(vd.grad[b : b + 1, g : g + 1], dv_ref, "dv", scale_abs=True)


def _random_band_case(seed):
  """A random window / causal offset problem: sizes around the tile edges (32, 64, 128 rows), every head-dim pair, GQA
  group sizes 1..4, ragged key lengths, segment ids now and then, windows from zero to beyond the sequence."""
  g = torch.Generator().manual_seed(9000 + seed)
  r = lambda lo, hi: int(torch.randint(lo, hi + 1, (1,), generator=g))  # noqa: E731
  D, Dv = ((64, 64), (128, 128), (192, 128))[r(0, 2)]
  Hkv = r(1, 2)
  Hq = Hkv * r(1, 4)
  S = (r(1, 70), r(100, 200), r(250, 420))[r(0, 2)]
  use_seg = r(0, 3) == 0
  # (a handful of keys under hundreds of queries would put a thousand rounded dS terms into every dK element: that is
  # a question for the tolerance, not for the band arithmetic this test is about)
  Skv = S if use_seg or r(0, 2) else max(r(1, 450), S // 6)
  causal = bool(r(0, 2))
  left = None if r(0, 3) == 0 else r(0, (5, 40, 150, 500)[r(0, 3)])
  right = None if (causal and r(0, 1)) or r(0, 3) == 0 else r(0, (3, 30, 200)[r(0, 2)])
  if left is None and right is None and not causal:
    left = r(0, 60)
  offset = r(-6, 50) if causal and r(0, 1) else 0
  seg = packed_segment_ids(1 + r(0, 1), S, 1, max(2, S // 2), seed)[0] if use_seg else None
  B = seg.shape[0] if use_seg else r(1, 2)
  dtype = (torch.bfloat16, torch.float16)[r(0, 1)]
  return dict(B=B, Hq=Hq, Hkv=Hkv, S=S, D=D, Dv=Dv, Skv=Skv, causal=causal, window=(left, right), causal_offset=offset,
              seg=seg, dtype=dtype)


@pytest.mark.parametrize("seed", range(48))
def test_randomised_windows_and_offsets(seed):
  """The causal kernels evaluate a window and / or a causal offset as a band around the row's own index (first and
  last tile of a workgroup's loop, per-wave skips, which tiles need masks, the bit range of a masked tile): 48 random
  problems against the oracle, forward and gradients, rows without any allowed key included."""
  c = _random_band_case(seed)
  _check(c["B"], c["Hq"], c["Hkv"], c["S"], c["D"], dtype=c["dtype"], causal=c["causal"], seg=c["seg"], window=c["window"],
         causal_offset=c["causal_offset"], Skv=c["Skv"], seed=seed, Dv=c["Dv"])


# ---- additive masks: the eager branch's ``attn_weights + causal_mask`` (attention.py:151-158) for any mask ----------
def _eager_grads(q, k, v, do, mask):
  """(out, dq, dk, dv) of the oracle's eager attention in float64, by autograd."""
  q64, k64, v64 = (t.double().requires_grad_(True) for t in (q, k, v))
  out = orc.eager_attention(q64, k64, v64, None if mask is None else mask.double())
  dq, dk, dv = torch.autograd.grad(out, (q64, k64, v64), do.double())
  return out.detach(), dq, dk, dv


def _padding_mask(B, S, Skv, lengths, causal, dtype=torch.float32, fill=float("-inf")):
  """(B,1,S,Skv): keys at or past ``lengths[b]`` are forbidden for batch row b; optionally causal on top."""
  j = torch.arange(Skv)[None, None, None, :]
  bad = j >= torch.as_tensor(lengths)[:, None, None, None]
  if causal:
    bad = bad | (j > torch.arange(S)[None, None, :, None])
  return torch.zeros((B, 1, S, Skv), dtype=dtype).masked_fill(bad, fill)


def _check_bias(B, Hq, Hkv, S, D, mask, dtype=torch.bfloat16, Skv=None, Dv=None, seed=0, causal=False, ref_mask=None):
  Skv = S if Skv is None else Skv
  Dv = D if Dv is None else Dv
  q, k, v, do = (heads_view(B, h, s_, d, seed + i, dtype)
                 for i, (h, s_, d) in enumerate(((Hq, S, D), (Hkv, Skv, D), (Hkv, Skv, Dv), (Hq, S, Dv))))
  qd, kd, vd = (t.to(DEV).requires_grad_(True) for t in (q, k, v))
  out = tpa.ops.attention(qd, kd, vd, None, None, causal, bias=mask.to(DEV))
  out.backward(do.to(DEV))
  o_ref, dq_ref, dk_ref, dv_ref = _eager_grads(q, k, v, do, mask if ref_mask is None else ref_mask)
  assert torch.isfinite(o_ref).all()
  assert_close(out, o_ref, "out")
  assert_close(qd.grad, dq_ref, "dq", scale_abs=True)
  assert_close(kd.grad, dk_ref, "dk", scale_abs=True)
  assert_close(vd.grad, dv_ref, "dv", scale_abs=True)


@pytest.mark.parametrize("D,Dv", [(128, 128), (64, 64), (192, 128)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_additive_padding_mask_fwd_bwd(D, Dv, dtype):
  B, S = 3, 200
  _check_bias(B, 4, 2, S, D, _padding_mask(B, S, S, [200, 131, 64], causal=True), dtype=dtype, Dv=Dv)
  _check_bias(B, 4, 2, S, D, _padding_mask(B, S, 333, [333, 7, 190], causal=False), dtype=dtype, Dv=Dv, Skv=333, seed=3)


@pytest.mark.parametrize("D", [128, 64])
def test_additive_mask_fp32_operands(D):
  B, S = 2, 150
  _check_bias(B, 4, 2, S, D, _padding_mask(B, S, S, [150, 77], causal=True), dtype=torch.float32)
  bias = 2.0 * torch.randn((1, 4, S, S), generator=torch.Generator().manual_seed(5))
  _check_bias(B, 4, 2, S, D, bias, dtype=torch.float32, seed=2)


def test_additive_mask_with_finite_values_per_head_and_the_causal_flag():
  """A per-head finite bias (ALiBi-like slopes plus noise), broadcast over the batch; once with causality inside the
  mask and once through the kernel's own causal flag: both are the eager formula with the summed mask."""
  B, Hq, Hkv, S, D = 2, 8, 2, 260, 128
  i, j = torch.arange(S)[:, None], torch.arange(S)[None, :]
  slopes = 2.0 ** -torch.arange(1, Hq + 1).float()
  bias = -(i - j).abs().float()[None, None] * slopes[None, :, None, None]
  bias = bias + 0.5 * torch.randn((1, Hq, S, S), generator=torch.Generator().manual_seed(1))
  causal = orc.causal_additive_mask(S)
  _check_bias(B, Hq, Hkv, S, D, bias + causal)
  _check_bias(B, Hq, Hkv, S, D, bias, causal=True, ref_mask=bias + causal, seed=4)
  _check_bias(B, Hq, Hkv, S, D, bias)  # no forbidden pair at all


def test_additive_mask_with_the_dtype_minimum_instead_of_minus_infinity():
  """Masks built as ``finfo(dtype).min`` (the other common convention): the weights underflow to zero exactly as in
  the eager formula, also where the mask is a 16-bit tensor and where it is longer than the keys."""
  B, S = 2, 180
  for mdtype in (torch.float32, torch.bfloat16, torch.float16):
    m = _padding_mask(B, S, S + 20, [S, 99], causal=True, dtype=mdtype, fill=torch.finfo(mdtype).min)
    q, k, v = (heads_view(B, h, S, 128, s, torch.bfloat16) for h, s in ((4, 1), (2, 2), (2, 3)))
    mod = tpa.AttentionModule(tpa.Config(attention_kernel=None, num_attention_heads=4, num_key_value_heads=2))
    out = mod(q.to(DEV), k.to(DEV), v.to(DEV), m.to(DEV))
    assert_close(out, orc.eager_attention(q.float(), k.float(), v.float(), m.float()), f"mask dtype {mdtype}")


def test_rows_with_every_key_forbidden_give_zeros_and_zero_gradients():
  """The eager softmax gives NaN on such rows (padding queries); the kernels define them as out = 0 with no gradient,
  as for segment masks, and every other row is unaffected."""
  B, Hq, Hkv, S, D = 1, 4, 2, 140, 128
  mask = _padding_mask(B, S, S, [S], causal=True)
  mask[:, :, 40:75, :] = float("-inf")
  q, k, v, do = (heads_view(B, h, S, D, s, torch.bfloat16) for h, s in ((Hq, 1), (Hkv, 2), (Hkv, 3), (Hq, 4)))
  qd, kd, vd = (t.to(DEV).requires_grad_(True) for t in (q, k, v))
  out = tpa.ops.attention(qd, kd, vd, None, None, False, bias=mask.to(DEV))
  out.backward(do.to(DEV))
  assert torch.isfinite(out).all() and torch.isfinite(qd.grad).all() and torch.isfinite(kd.grad).all()
  assert (out[:, :, 40:75] == 0).all() and (qd.grad[:, :, 40:75] == 0).all()
  live = torch.ones(S, dtype=torch.bool)
  live[40:75] = False
  do_live = do.clone()
  do_live[:, :, ~live] = 0
  ref_mask = mask.clone()
  ref_mask[:, :, 40:75, 0] = 0.0  # any allowed key: with dO = 0 these rows contribute nothing
  o_ref, dq_ref, dk_ref, dv_ref = _eager_grads(q, k, v, do_live, ref_mask)
  assert_close(out[:, :, live], o_ref[:, :, live], "out, live rows")
  assert_close(qd.grad[:, :, live], dq_ref[:, :, live], "dq, live rows", scale_abs=True)
  assert_close(kd.grad, dk_ref, "dk", scale_abs=True)
  assert_close(vd.grad, dv_ref, "dv", scale_abs=True)


def test_additive_mask_shape_errors():
  q = torch.zeros((2, 4, 32, 128), dtype=torch.bfloat16, device=DEV)
  with pytest.raises(ValueError, match="mask must have shape"):
    tpa.ops.attention(q, q, q, None, None, False, bias=torch.zeros((3, 1, 32, 32), device=DEV))
  with pytest.raises(ValueError, match="mask must have shape"):
    tpa.ops.attention(q, q, q, None, None, False, bias=torch.zeros((32, 32), device=DEV))
  with pytest.raises(RuntimeError, match="no CPU path"):
    tpa.ops.attention(q, q, q, None, None, False, bias=torch.zeros((1, 1, 32, 32)))
