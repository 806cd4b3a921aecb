"""GPU parity: attention forward/backward (through the torch.library ops, i.e. through the C ABI)
against the fp32/fp64 CPU oracle on the same seeded inputs.  Tolerance for 16-bit outputs and
gradients: max-abs <= 2e-2 and relative-L2 <= 1e-2 (tests/util.py)."""

import math
import random

import pytest
import torch

import torchprime_amd as tpa
from oracle import tprime_oracle as orc
from tests.util import assert_close, heads_view, packed_segment_ids, randn

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _run(q, k, v, do, seg, causal, sm_scale):
  qd, kd, vd = (t.to(DEV).requires_grad_(True) for t in (q, k, v))
  segd = None if seg is None else seg.to(DEV)
  out, lse = torch.ops.tprime.attn_fwd(qd, kd, vd, segd, sm_scale, causal)
  out.backward(do.to(DEV))
  return out.detach(), lse, qd.grad, kd.grad, vd.grad


def _check(B, Hq, Hkv, S, Dqk, Dv, dtype, causal, seg=None, layout="bshd", seed=0, Skv=None, sm_scale=None, std=1.0, v_std=None,
           grad_abs=2e-2):
  Skv = S if Skv is None else Skv
  mk = heads_view if layout == "bshd" else (lambda B_, H, S_, D, sd, dt, std=1.0: randn((B_, H, S_, D), sd, dt, std))
  q = mk(B, Hq, S, Dqk, seed + 1, dtype, std)
  k = mk(B, Hkv, Skv, Dqk, seed + 2, dtype, std)
  v = mk(B, Hkv, Skv, Dv, seed + 3, dtype, std if v_std is None else v_std)
  do = mk(B, Hq, S, Dv, seed + 4, dtype, 1.0)
  sm_scale = 1.0 / math.sqrt(Dv) if sm_scale is None else sm_scale
  out, lse, dq, dk, dv = _run(q, k, v, do, seg, causal, sm_scale)
  o_ref, dq_ref, dk_ref, dv_ref = orc.attention_grads_ref(q, k, v, do, seg, causal, sm_scale, torch.float64)
  _, lse_ref = orc.attention_ref(q, k, v, seg, causal, sm_scale, torch.float64)
  assert out.shape == (B, Hq, S, Dv) and out.dtype == dtype
  assert_close(out, o_ref, "out")
  assert_close(lse, lse_ref, "lse", max_abs=5e-3, rel_l2=1e-3)  # row sums add the 16-bit-rounded p the PV product uses
  # gradients reach |x| > 4 with N(0,1) inputs, where one bf16 rounding alone is up to 1.6e-2: every element
  # gets the stated bound plus one bf16 ulp of its own magnitude, |err| <= 2e-2 + 2^-7 |ref| (tests/util.py)
  assert_close(dq, dq_ref, "dq", max_abs=grad_abs, scale_abs=True)
  assert_close(dk, dk_ref, "dk", max_abs=grad_abs, scale_abs=True)
  assert_close(dv, dv_ref, "dv", max_abs=grad_abs, scale_abs=True)
  return out


def _check_against_eager_16_bit(B, Hq, Hkv, S, Dqk, Dv, dtype, causal, seg=None, seed=0, std=1.0, v_std=None):
  """For inputs outside what the stated bound is meant for (scores far larger than N(0,1) inputs give, or a softmax
  so sharp that a single rounding of dS decides an element): the yardstick is the same formula evaluated eagerly in
  the tensors' 16-bit dtype on the CPU, the reference's own arithmetic.  Every gradient must be within 1.25 times that
  evaluation's error against fp64, in max-abs and in relative-L2 (which also stays under 1e-2); the forward output is
  held to the usual bound."""
  q = heads_view(B, Hq, S, Dqk, seed + 1, dtype, std)
  k = heads_view(B, Hkv, S, Dqk, seed + 2, dtype, std)
  v = heads_view(B, Hkv, S, Dv, seed + 3, dtype, std if v_std is None else v_std)
  do = heads_view(B, Hq, S, Dv, seed + 4, dtype, 1.0)
  sm_scale = 1.0 / math.sqrt(Dv)
  out, _, dq, dk, dv = _run(q, k, v, do, seg, causal, sm_scale)
  ref = orc.attention_grads_ref(q, k, v, do, seg, causal, sm_scale, torch.float64)
  eager = orc.attention_grads_ref(q, k, v, do, seg, causal, sm_scale, dtype)
  assert_close(out, ref[0], "out")
  for name, got, e16, r64 in zip(("dq", "dk", "dv"), (dq, dk, dv), eager[1:], ref[1:]):
    err_gpu, err_16 = (got.double().cpu() - r64).abs(), (e16.double() - r64).abs()
    assert torch.isfinite(got.float()).all(), name
    assert err_gpu.max().item() <= 1.25 * err_16.max().item(), (name, err_gpu.max().item(), err_16.max().item())
    rl_gpu, rl_16 = (err_gpu.norm() / r64.norm()).item(), (err_16.norm() / r64.norm()).item()
    assert rl_gpu <= 1e-2 and rl_gpu <= 1.25 * rl_16 + 1e-3, (name, rl_gpu, rl_16)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize(
  "B,Hq,Hkv,S,Dqk,Dv",
  [
    (2, 8, 8, 128, 64, 64),      # C1 attention shape
    (1, 4, 1, 256, 128, 128),    # GQA 4:1, tile-aligned
    (2, 8, 2, 200, 128, 128),    # ragged length
    (1, 2, 2, 77, 64, 64),       # shorter than one tile
    (1, 4, 4, 321, 192, 128),    # DeepSeek-style asymmetric heads
    (1, 16, 2, 640, 128, 128),   # GQA 8:1 (Llama-3-70B grouping)
    (1, 1, 1, 1, 128, 128),      # single token
  ],
)
def test_causal_fwd_bwd(dtype, B, Hq, Hkv, S, Dqk, Dv):
  _check(B, Hq, Hkv, S, Dqk, Dv, dtype, True)


def _random_draw(seed):
  """One seeded draw over what the kernels branch on (see test_randomised_shapes_and_segment_layouts)."""
  rng = random.Random(1000 + seed)
  Dqk, Dv = rng.choice([(64, 64), (128, 128), (128, 128), (192, 128)])
  Hkv = rng.choice([1, 2])
  Hq = Hkv * rng.choice([1, 2, 4])
  S = rng.choice([31, 32, 33, 63, 64, 65, 127, 128, 129, 191, 255, 256, 257, 300, 383, 448, 513])
  causal = rng.random() < 0.6
  dtype = rng.choice([torch.bfloat16, torch.bfloat16, torch.float16])
  B = rng.choice([1, 2])
  kind = rng.choice(["none", "packed", "tiny", "unsorted"])
  if kind == "none":
    seg = None
  elif kind == "packed":
    seg = packed_segment_ids(B, S, 1, max(2, S // 2), seed=seed)[0]
  elif kind == "tiny":
    seg = packed_segment_ids(B, S, 1, 9, seed=seed)[0]
  else:
    g = torch.Generator().manual_seed(seed)
    seg = torch.randint(-3, 4, (B, S), generator=g, dtype=torch.int32)
  return dict(B=B, Hq=Hq, Hkv=Hkv, S=S, Dqk=Dqk, Dv=Dv, dtype=dtype, causal=causal, seg=seg, seed=10 * seed)


@pytest.mark.parametrize("seed", range(64))
def test_randomised_shapes_and_segment_layouts(seed):
  """Seeded random draws over what the kernels branch on: length (around tile edges too), GQA ratio, head dims, dtype,
  causality, and the id layout (none, packed documents, short documents of a few rows, unsorted ids with repeats):
  masked tiles are resolved through per-tile bit masks and per-workgroup tile lists, whose corner cases are lengths
  and document boundaries that fall on or next to tile and wave boundaries."""
  d = _random_draw(seed)
  _check(d["B"], d["Hq"], d["Hkv"], d["S"], d["Dqk"], d["Dv"], d["dtype"], d["causal"], seg=d["seg"], seed=d["seed"])


def test_sharp_softmax_draw_against_the_eager_16_bit_evaluation():
  """The one draw of 248 further seeds of the sweep above that leaves the per-element bound (seed 144: 192/128 heads,
  65 rows, seven interleaved ids, bf16; one element of dq 7e-4 over ``2e-2 + 2^-7 |ref|``).  With a handful of allowed
  keys per row the softmax is sharp, dS is large, and its one rounding to 16 bits is what that element carries: no
  16-bit evaluation does better there.  So this case is held to the yardstick that is independent of the bound's
  constants: the same formula evaluated eagerly in bf16 on the CPU (the reference's own arithmetic).  Every gradient
  must be within 1.25 times that evaluation's error against fp64, in max-abs and in relative-L2; the forward output
  and the relative-L2 limit of 1e-2 hold as everywhere."""
  d = _random_draw(144)
  assert (d["Dqk"], d["Dv"], d["S"], d["dtype"]) == (192, 128, 65, torch.bfloat16) and d["seg"] is not None
  _check_against_eager_16_bit(d["B"], d["Hq"], d["Hkv"], d["S"], d["Dqk"], d["Dv"], d["dtype"], d["causal"], seg=d["seg"], seed=d["seed"])


@pytest.mark.parametrize("B,Hq,Hkv,S,Skv,Dqk,Dv", [(1, 4, 2, 130, 130, 128, 128), (2, 2, 2, 64, 300, 64, 64), (1, 2, 1, 257, 100, 128, 128)])
def test_full_attention_fwd_bwd(B, Hq, Hkv, S, Skv, Dqk, Dv):
  # the eager branch without a mask (attention.py:151-170 with attention_mask=None)
  _check(B, Hq, Hkv, S, Dqk, Dv, torch.bfloat16, False, Skv=Skv)


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_running_max_moves_often(seed):
  # large score spread: the row maximum keeps growing by more than the lazy-rescale threshold, in either
  # half of a KV tile, so the rescale paths (including the one deferred past the first half's P V) run
  # (q and k are 2.5x / 3x the N(0,1) scale the tolerance is stated for, so the gradients are held to the eager 16-bit
  # evaluation of the same inputs instead of a bound scaled to fit)
  _check_against_eager_16_bit(1, 4, 2, 512, 128, 128, torch.bfloat16, True, seed=10 * seed, std=2.5, v_std=1.0)
  _check_against_eager_16_bit(1, 2, 2, 300, 64, 64, torch.bfloat16, False, seed=10 * seed + 5, std=3.0, v_std=1.0)


def test_contiguous_bhsd_layout_and_scale():
  _check(2, 4, 2, 150, 128, 128, torch.bfloat16, True, layout="bhsd", sm_scale=0.2)


@pytest.mark.parametrize("S,lo,hi,causal", [(512, 16, 200, True), (700, 1, 90, True), (384, 64, 384, True), (300, 10, 120, False)])
def test_segment_ids_fwd_bwd(S, lo, hi, causal):
  seg, _ = packed_segment_ids(2, S, lo, hi, seed=S)
  _check(2, 4, 2, S, 128, 128, torch.bfloat16, causal, seg=seg)


@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("Dqk,Dv,dtype", [(128, 128, torch.float16), (64, 64, torch.float16), (192, 128, torch.bfloat16), (192, 128, torch.float16)])
def test_segment_ids_other_dtypes_and_head_dims(causal, Dqk, Dv, dtype):
  # fp16 with segment ids, and the asymmetric 192/128 heads (single-buffer dK/dV path) with segment ids / non-causal
  seg, _ = packed_segment_ids(1, 330, 8, 120, seed=Dqk + causal)
  _check(1, 4, 2 if Dqk != 192 else 4, 330, Dqk, Dv, dtype, causal, seg=seg)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_full_attention_wide_and_small_heads(dtype):
  _check(1, 4, 4, 200, 192, 128, dtype, False, Skv=260)   # 192/128 non-causal, Skv != Sq
  _check(2, 4, 2, 100, 64, 64, dtype, False, Skv=333)     # 64/64 non-causal backward, Skv != Sq


def test_segment_ids_unsorted_and_negative_ids():
  # ids need not be sorted or non-negative: equality is all that matters
  g = torch.Generator().manual_seed(3)
  seg = torch.randint(-2, 3, (2, 260), generator=g, dtype=torch.int32)
  _check(2, 2, 1, 260, 64, 64, torch.bfloat16, True, seg=seg)
  _check(2, 2, 1, 260, 64, 64, torch.bfloat16, False, seg=seg)


@pytest.mark.parametrize("D", [128, 64])
def test_segment_ids_alternating_blocks(D):
  # ids alternate every 64 rows (0,1,0,1,... and 0,0,1,1,...): inside one 256-row workgroup some waves need a
  # kv tile that the others skip, tile after tile, so the backward's carried second kv block is finished both
  # ways (inside the next tile's body and on its own after a skipped tile)
  S = 1024
  r = torch.arange(S)
  seg = torch.stack([(r // 64) % 2, (r // 128) % 2]).to(torch.int32)
  _check(2, 4, 2, S, D, D, torch.bfloat16, True, seg=seg)


def test_segment_equals_block_diagonal_decomposition():
  """Document masking == running each document through causal attention on its own."""
  B, Hq, Hkv, S, D = 1, 4, 2, 448, 128
  seg, lengths = packed_segment_ids(B, S, 32, 200, seed=9)
  q, k, v = (heads_view(B, h, S, D, s, torch.bfloat16) for h, s in ((Hq, 1), (Hkv, 2), (Hkv, 3)))
  full = tpa.ops.attention(q.to(DEV), k.to(DEV), v.to(DEV), seg.to(DEV), None, True)
  pos = 0
  for L in lengths[0]:
    sl = slice(pos, pos + L)
    part = tpa.ops.attention(q[:, :, sl].to(DEV), k[:, :, sl].to(DEV), v[:, :, sl].to(DEV), None, None, True)
    assert_close(full[:, :, sl], part.float().cpu(), f"doc@{pos}")  # two bf16 results: within one output ulp
    pos += L


@pytest.mark.parametrize("causal,use_seg", [(True, False), (True, True), (False, True)])
def test_mask_pattern_exact(causal, use_seg):
  """Recover P through the public op with one-hot V blocks and compare its support with the closed-form
  mask: entries that must be masked are exactly 0, allowed entries are > 0."""
  B, H, S, D = 1, 2, 192, 64
  seg = None
  if use_seg:
    seg, _ = packed_segment_ids(B, S, 5, 70, seed=4)
  q = heads_view(B, H, S, D, 1, torch.bfloat16, 0.3).to(DEV)
  k = heads_view(B, H, S, D, 2, torch.bfloat16, 0.3).to(DEV)
  allowed = orc.allowed_mask(seg, S, S, causal)[0]
  P = torch.zeros((H, S, S))
  for j0 in range(0, S, D):
    v = torch.zeros((B, H, S, D), dtype=torch.bfloat16)
    for j in range(j0, min(j0 + D, S)):
      v[:, :, j, j - j0] = 1
    o = tpa.ops.attention(q, k, v.to(DEV), None if seg is None else seg.to(DEV), None, causal)
    P[:, :, j0 : j0 + D] = o[0, :, :, : min(D, S - j0)].float().cpu()
  assert torch.equal(P > 0, allowed[None].expand_as(P)), "support of P differs from the mask"
  assert_close(P.sum(-1), torch.ones(H, S), "rows sum to 1", max_abs=2e-2)


def test_eager_formula_is_nan_on_fully_masked_rows_but_kernel_convention_is_zero():
  """The eager expression gives NaN for a row whose mask is all -inf; the documented convention of
  the oracle (and the kernels) for such a row is out = 0, lse = -inf.  Through the public mask
  definition (causal and/or same-segment with Sq == Skv) every row keeps at least its own key, so
  the convention is only reachable with Sq > Skv... which the API does not mask; asserted on the oracle."""
  q = randn((1, 1, 4, 8), 1)
  mask = torch.full((1, 1, 4, 4), float("-inf"))
  assert torch.isnan(orc.eager_attention(q, q, q, mask)).all()


def test_deterministic_backward():
  B, Hq, Hkv, S, D = 1, 8, 2, 384, 128
  q, k, v, do = (heads_view(B, h, S, D, s, torch.bfloat16) for h, s in ((Hq, 1), (Hkv, 2), (Hkv, 3), (Hq, 4)))
  r1 = _run(q, k, v, do, None, True, D**-0.5)
  r2 = _run(q, k, v, do, None, True, D**-0.5)
  for a, b in zip(r1, r2):
    assert torch.equal(a, b)


# ---- module / functional API ----------------------------------------------------------------------
def _cfg(kernel, hq, hkv):
  return tpa.Config(attention_kernel=kernel, num_attention_heads=hq, num_key_value_heads=hkv, attention_dropout=False)


@pytest.mark.parametrize("kernel", ["splash_attention", "flash_attention", None, "pytorch"])
def test_attention_module_matches_eager_branch(kernel):
  B, Hq, Hkv, S, D = 2, 8, 2, 160, 128
  q, k, v = (heads_view(B, h, S, D, s, torch.bfloat16) for h, s in ((Hq, 1), (Hkv, 2), (Hkv, 3)))
  mask = orc.causal_additive_mask(S)
  m = tpa.AttentionModule(_cfg(kernel, Hq, Hkv))
  out = m(q.to(DEV), k.to(DEV), v.to(DEV), mask.to(DEV))
  ref = orc.eager_attention(q.float(), k.float(), v.float(), mask)
  assert_close(out, ref, f"kernel={kernel}")
  assert m.partition_spec is None and out.transpose(1, 2).is_contiguous()


def test_mask_verdict_is_not_reused_for_a_new_mask_at_the_same_address():
  """A model rebuilds its additive mask every forward (model/llama/model.py:347-355).  The allocator hands the freed
  mask's memory to the next one, so a verdict remembered by address would let a padded mask of the same shape pass as
  the causal one (and take the causal kernels, which never read the mask); the verdict belongs to the tensor object."""
  from torchprime_amd import attention as att

  B, H, S, D = 1, 2, 96, 64
  q, k, v = (heads_view(B, H, S, D, s, torch.bfloat16) for s in (1, 2, 3))
  qd, kd, vd = q.to(DEV), k.to(DEV), v.to(DEV)
  m = tpa.AttentionModule(_cfg(None, H, H))
  causal = orc.causal_additive_mask(S).to(DEV)
  out_causal = m(qd, kd, vd, causal)  # accepted as causal, verdict remembered
  m(qd, kd, vd, causal)  # same tensor again: no second check needed
  ptr, n_entries = causal.data_ptr(), len(att._MASK_VERDICTS)
  assert n_entries >= 1
  del causal
  assert len(att._MASK_VERDICTS) == n_entries - 1  # the entry left with the tensor
  padded_cpu = orc.causal_additive_mask(S).clone()
  padded_cpu[..., 3 * S // 4 :] = float("-inf")  # a padded batch: the last keys masked for every query
  ref = orc.eager_attention(q.float(), k.float(), v.float(), padded_cpu)
  hit = False
  for _ in range(8):  # (the allocator normally reuses the block at once; a few tries in case it does not)
    padded = padded_cpu.to(DEV)
    hit = hit or padded.data_ptr() == ptr
    out = m(qd, kd, vd, padded)
    assert_close(out, ref, "padded mask")
    assert (out.float() - out_causal.float()).abs().max() > 5e-2  # not the causal result
    del padded
  assert hit, "the allocator never reused the freed mask's address: the test did not exercise the aliasing"


def test_attention_module_scale_uses_v_head_dim():
  # DeepSeek: qk dim 192, v dim 128 -> 1/sqrt(128) (attention.py:54-58)
  B, H, S = 1, 4, 96
  q, k = heads_view(B, H, S, 192, 1, torch.bfloat16, 0.5), heads_view(B, H, S, 192, 2, torch.bfloat16, 0.5)
  v = heads_view(B, H, S, 128, 3, torch.bfloat16)
  out = tpa.AttentionModule(_cfg("splash_attention", H, H))(q.to(DEV), k.to(DEV), v.to(DEV))
  ref, _ = orc.attention_ref(q, k, v, None, True, 1 / math.sqrt(128), torch.float64)
  wrong, _ = orc.attention_ref(q, k, v, None, True, 1 / math.sqrt(192), torch.float64)
  assert_close(out, ref, "scale 1/sqrt(v_dim)")
  assert (out.float().cpu() - wrong.float()).abs().max() > 5e-2


def test_attention_module_eager_without_mask_is_full_attention_and_other_masks_are_added():
  B, H, S, D = 1, 2, 80, 64
  q, k, v = (heads_view(B, H, S, D, s, torch.bfloat16) for s in (1, 2, 3))
  m = tpa.AttentionModule(_cfg(None, H, H))
  out = m(q.to(DEV), k.to(DEV), v.to(DEV), None)
  full = orc.eager_attention(q.float(), k.float(), v.float(), None)
  assert_close(out, full, "no mask")
  # an all-zero mask is full attention too; a random one is added to the logits (attention.py:153-158)
  assert_close(m(q.to(DEV), k.to(DEV), v.to(DEV), torch.zeros((1, 1, S, S), device=DEV)), full, "zero mask")
  noise = torch.randn((1, 1, S, S), generator=torch.Generator().manual_seed(0))
  assert_close(m(q.to(DEV), k.to(DEV), v.to(DEV), noise.to(DEV)), orc.eager_attention(q.float(), k.float(), v.float(), noise), "noise")
  with pytest.raises(ValueError, match="attention_mask must be 4-D"):
    m(q.to(DEV), k.to(DEV), v.to(DEV), torch.zeros((S, S), device=DEV))


def test_splash_wrapper_signature_and_segments():
  B, Hq, Hkv, S, D = 2, 4, 2, 256, 128
  seg, _ = packed_segment_ids(B, S, 20, 100, seed=5)
  q, k, v = (heads_view(B, h, S, D, s, torch.bfloat16) for h, s in ((Hq, 1), (Hkv, 2), (Hkv, 3)))
  qs = (q.float() / math.sqrt(D)).to(torch.bfloat16)  # callers pre-scale q (attention.py:107)
  cfg = tpa.SplashAttentionConfig(mesh="ignored").to_json()
  res = tpa.tpu_splash_attention_jax_call_wrapper(
    mask=None, query=qs.to(DEV), key=k.to(DEV), value=v.to(DEV), config=cfg,
    decoder_segment_ids=seg.to(DEV), causal=True, q_seq_shards=1,
  )
  assert isinstance(res, tuple) and len(res) == 3 and res[1] is None and res[2] is None
  ref, _ = orc.attention_ref(qs, k, v, seg, True, 1.0, torch.float64)
  assert_close(res[0], ref, "segments via wrapper")
  assert tpa.tpu_splash_attention_jax_call_wrapper(None, qs.to(DEV), k.to(DEV), v.to(DEV), cfg, None, True, is_forward=False) is None
  with pytest.raises(AssertionError):
    tpa.tpu_splash_attention_jax_call_wrapper(None, qs.to(DEV), k.to(DEV), v.to(DEV), cfg, seg[:, :100].to(DEV), True)
  slide = tpa.SplashAttentionConfig(attentiontype_local_sliding=True).to_json()
  with pytest.raises(ValueError):
    tpa.tpu_splash_attention_jax_call_wrapper(None, qs.to(DEV), k.to(DEV), v.to(DEV), slide, None, True)


@pytest.mark.parametrize("B,Hq,Hkv,S,Skv,D,causal,use_seg", [
  (2, 8, 8, 128, 128, 64, True, False),    # benchmark configuration 1's attention
  (1, 4, 2, 200, 200, 128, True, False),   # GQA, ragged
  (2, 4, 1, 77, 300, 64, False, False),    # full attention, Skv != Sq
  (2, 4, 2, 260, 260, 128, True, True),    # segment ids
  (1, 2, 2, 1, 1, 64, True, False),
])
def test_fp32_attention_forward(B, Hq, Hkv, S, Skv, D, causal, use_seg):
  """fp32 operands (v_mfma_f32_32x32x2_f32): the fp32 tolerance class of the reference's CPU tests, atol 1e-5."""
  q, k, v = heads_view(B, Hq, S, D, 1, torch.float32), heads_view(B, Hkv, Skv, D, 2, torch.float32), heads_view(B, Hkv, Skv, D, 3, torch.float32)
  seg = packed_segment_ids(B, S, 5, 90, seed=8)[0] if use_seg else None
  out, lse = torch.ops.tprime.attn_fwd(q.to(DEV), k.to(DEV), v.to(DEV), None if seg is None else seg.to(DEV), D**-0.5, causal)
  o_ref, lse_ref = orc.attention_ref(q, k, v, seg, causal, D**-0.5, torch.float64)
  assert out.dtype == torch.float32
  assert_close(out, o_ref, "out", max_abs=1e-5, rel_l2=1e-5)
  assert_close(lse, lse_ref, "lse", max_abs=1e-5, rel_l2=1e-6)
  if use_seg is False and causal:
    m = tpa.AttentionModule(_cfg(None, Hq, Hkv))
    o2 = m(q.to(DEV), k.to(DEV), v.to(DEV), orc.causal_additive_mask(S).to(DEV)) if S == Skv else None
    if o2 is not None:
      assert_close(o2, orc.eager_attention(q, k, v, orc.causal_additive_mask(S)), "module, fp32 eager branch", max_abs=1e-5, rel_l2=1e-5)


@pytest.mark.parametrize("B,Hq,Hkv,S,Skv,D,causal,use_seg", [
  (2, 8, 8, 128, 128, 64, True, False),    # benchmark configuration 1's attention shape
  (1, 4, 2, 200, 200, 128, True, False),   # GQA 2:1, ragged length
  (1, 4, 1, 97, 161, 64, False, False),    # full attention, Sq != Skv, GQA 4:1
  (2, 4, 2, 260, 260, 128, True, True),    # segment ids
  (1, 2, 2, 150, 150, 64, False, True),    # segment ids without causality
  (1, 2, 2, 1, 1, 64, True, False),
])
def test_fp32_attention_backward(B, Hq, Hkv, S, Skv, D, causal, use_seg):
  """fp32 operands, gradients through the registered autograd: relative-L2 1e-5 and 2e-5 of the tensor's largest value
  per element against the fp64 oracle (fp32 accumulation over up to 260 keys)."""
  q, k, v = heads_view(B, Hq, S, D, 1, torch.float32), heads_view(B, Hkv, Skv, D, 2, torch.float32), heads_view(B, Hkv, Skv, D, 3, torch.float32)
  do = heads_view(B, Hq, S, D, 4, torch.float32)
  seg = packed_segment_ids(B, S, 5, 90, seed=8)[0] if use_seg else None
  qd, kd, vd = (t.to(DEV).requires_grad_(True) for t in (q, k, v))
  out = tpa.ops.attention(qd, kd, vd, None if seg is None else seg.to(DEV), D**-0.5, causal)
  out.backward(do.to(DEV))
  o_ref, dq_ref, dk_ref, dv_ref = orc.attention_grads_ref(q, k, v, do, seg, causal, D**-0.5, torch.float64)
  assert_close(out, o_ref, "out", max_abs=1e-5, rel_l2=1e-5)
  for name, got, ref in (("dq", qd.grad, dq_ref), ("dk", kd.grad, dk_ref), ("dv", vd.grad, dv_ref)):
    assert got.dtype == torch.float32 and got.shape == ref.shape
    assert_close(got, ref, name, max_abs=2e-5 * max(1.0, ref.abs().max().item()), rel_l2=1e-5)


def test_long_packed_sequence_65536_rows():
  """S = 65536 with 96 packed documents, one head of 128: 1024 query tiles per workgroup list (the longest the dK/dV
  kernel's LDS holds at this head dim).  A packed row is a set of independent causal problems, so three documents
  are checked against the oracle run on each of them alone; everything else must be finite."""
  B, H, S, D = 1, 1, 65536, 128
  seg, lengths = packed_segment_ids(B, S, 300, 1000, seed=11)
  q, k, v, do = (heads_view(B, H, S, D, 20 + i, torch.bfloat16) for i in range(4))
  out, lse, dq, dk, dv = _run(q, k, v, do, seg, True, D**-0.5)
  for t in (out, dq, dk, dv):
    assert torch.isfinite(t.float()).all()
  starts = [0]
  for L in lengths[0]:
    starts.append(starts[-1] + L)
  for d in (0, len(lengths[0]) // 2, len(lengths[0]) - 1):
    a, b_ = starts[d], starts[d + 1]
    sl = (slice(None), slice(None), slice(a, b_))
    o_ref, dq_ref, dk_ref, dv_ref = orc.attention_grads_ref(q[sl], k[sl], v[sl], do[sl], None, True, D**-0.5, torch.float32)
    assert_close(out[sl], o_ref, f"out, document {d}")
    assert_close(dq[sl], dq_ref, f"dq, document {d}", scale_abs=True)
    assert_close(dk[sl], dk_ref, f"dk, document {d}", scale_abs=True)
    assert_close(dv[sl], dv_ref, f"dv, document {d}", scale_abs=True)


def test_long_packed_sequence_with_wide_heads():
  """S = 32768 with packed documents at head dims (192, 128), two query heads on one kv head: the tile lists of the
  three-buffer dK/dV pipeline (120 KB of tiles) and of the lean dQ kernel at their longest tested; checked document by
  document like the case above."""
  B, Hq, Hkv, S, D, Dv = 1, 2, 1, 32768, 192, 128
  seg, lengths = packed_segment_ids(B, S, 200, 3000, seed=12)
  q, k, v, do = (heads_view(B, h, S, d, 30 + i, torch.bfloat16)
                 for i, (h, d) in enumerate(((Hq, D), (Hkv, D), (Hkv, Dv), (Hq, Dv))))
  out, lse, dq, dk, dv = _run(q, k, v, do, seg, True, Dv**-0.5)
  for t in (out, dq, dk, dv):
    assert torch.isfinite(t.float()).all()
  starts = [0]
  for L in lengths[0]:
    starts.append(starts[-1] + L)
  for d in (0, len(lengths[0]) // 2, len(lengths[0]) - 1):
    a, b_ = starts[d], starts[d + 1]
    sl = (slice(None), slice(None), slice(a, b_))
    o_ref, dq_ref, dk_ref, dv_ref = orc.attention_grads_ref(q[sl], k[sl], v[sl], do[sl], None, True, Dv**-0.5, torch.float32)
    assert_close(out[sl], o_ref, f"out, document {d}")
    assert_close(dq[sl], dq_ref, f"dq, document {d}", scale_abs=True)
    assert_close(dk[sl], dk_ref, f"dk, document {d}", scale_abs=True)
    assert_close(dv[sl], dv_ref, f"dv, document {d}", scale_abs=True)


def test_unsupported_inputs_raise():
  q = torch.zeros((1, 2, 16, 96), dtype=torch.bfloat16, device=DEV)
  with pytest.raises(NotImplementedError):
    tpa.ops.attention(q, q, q)
  q64 = torch.zeros((1, 2, 16, 64), dtype=torch.float64, device=DEV)
  with pytest.raises(TypeError):
    tpa.ops.attention(q64, q64, q64)
  q32 = torch.zeros((1, 2, 16, 192), dtype=torch.float32, device=DEV)
  with pytest.raises(NotImplementedError):  # fp32 tensors: head dims 64 and 128
    tpa.ops.attention(q32, q32, q32[..., :128])
  with pytest.raises(RuntimeError):
    tpa.ops.attention(q.cpu(), q.cpu(), q.cpu())


# ---- full-size cases ----------------------------------------------------------------------------
def _slice_check(B, Hq, Hkv, S, Dqk, Dv, seg, seed, b_sel, g_sel, sm_scale=None):
  """Run the kernels on the full problem, check one (batch, kv-head group) slice against the oracle
  (attention is independent per batch and kv head, so the slice is an exact sub-problem)."""
  n_rep = Hq // Hkv
  dt = torch.bfloat16
  q, k, v, do = (heads_view(B, h, S, d, seed + i, dt) for i, (h, d) in enumerate(((Hq, Dqk), (Hkv, Dqk), (Hkv, Dv), (Hq, Dv))))
  sm_scale = 1.0 / math.sqrt(Dv) if sm_scale is None else sm_scale
  out, lse, dq, dk, dv = _run(q, k, v, do, seg, True, sm_scale)
  hs = slice(g_sel * n_rep, (g_sel + 1) * n_rep)
  qs, ks, vs, dos = q[b_sel : b_sel + 1, hs], k[b_sel : b_sel + 1, g_sel : g_sel + 1], v[b_sel : b_sel + 1, g_sel : g_sel + 1], do[b_sel : b_sel + 1, hs]
  segs = None if seg is None else seg[b_sel : b_sel + 1]
  o_ref, dq_ref, dk_ref, dv_ref = orc.attention_grads_ref(qs, ks, vs, dos, segs, True, sm_scale, torch.float32)
  assert_close(out[b_sel : b_sel + 1, hs], o_ref, "out")
  assert_close(dq[b_sel : b_sel + 1, hs], dq_ref, "dq", scale_abs=True)
  assert_close(dk[b_sel : b_sel + 1, g_sel : g_sel + 1], dk_ref, "dk", scale_abs=True)
  assert_close(dv[b_sel : b_sel + 1, g_sel : g_sel + 1], dv_ref, "dv", scale_abs=True)
  # every row is a convex combination of V rows: bounded by max |v|
  assert out.abs().max().item() <= v.abs().max().item() * (1 + 2.0**-7) + 1e-2  # P is rounded to bf16 for PV
  assert torch.isfinite(lse).all() and torch.isfinite(dq.float()).all()


def test_llama3_8b_shape_slice():  # benchmark configuration 2: B=4, S=8192, 32q/8kv, d=128
  _slice_check(4, 32, 8, 8192, 128, 128, None, 1234 + 1, b_sel=3, g_sel=5)


def test_llama3_8b_packed_segments_slice():  # benchmark configuration 3: documents of 64..4096 packed to 8192
  seg, _ = packed_segment_ids(4, 8192, 64, 4096, seed=1234 + 2)
  _slice_check(4, 32, 8, 8192, 128, 128, seg, 1234 + 2, b_sel=1, g_sel=2)


def test_llama3_70b_shape_slice():  # benchmark configuration 3: B=1, S=8192, 64q/8kv
  _slice_check(1, 64, 8, 8192, 128, 128, None, 1234 + 3, b_sel=0, g_sel=7)


def test_deepseek_v3_shape_slice():  # benchmark configuration 4: B=1, S=4096, 128 heads, qk 192 / v 128, scale 1/sqrt(128)
  _slice_check(1, 128, 128, 4096, 192, 128, None, 1234 + 4, b_sel=0, g_sel=77)


def test_deepseek_v3_shape_slice_qk_scale():
  # the same configuration with the scale a 192-wide q.k product would usually take (the reference uses the v head dim)
  _slice_check(1, 128, 128, 4096, 192, 128, None, 1234 + 4, b_sel=0, g_sel=3, sm_scale=192 ** -0.5)


def _closed_form_check(B, Hq, Hkv, S, Dqk, Dv, seg, seed):
  """What the mathematics fixes on the WHOLE full-size problem, every (batch, head), no oracle needed.  With V constant
  along the sequence (one value per (batch, kv head, column)) every output row is that value whatever the scores are,
  dP = dO V^T is constant along a row, so dS = P o (dP - rowsum(P o dP)) = 0 and with it dQ = dK = 0; and because the
  rows of P sum to one, the sum of dV over the keys equals the sum of dO over the queries of the group's heads.  A wrong
  LSE, a wrong delta, a mask that empties a row or a tile visited twice or not at all breaks one of the three."""
  n_rep = Hq // Hkv
  dt = torch.bfloat16
  g = torch.Generator().manual_seed(seed)
  q, k, do = (heads_view(B, h, S, d, seed + i, dt) for i, (h, d) in enumerate(((Hq, Dqk), (Hkv, Dqk), (Hq, Dv))))
  vals = torch.randn((B, Hkv, 1, Dv), generator=g).to(dt)
  v = vals.expand(B, Hkv, S, Dv).transpose(1, 2).contiguous().transpose(1, 2)  # (B,H,S,D) view of a (B,S,H,D) buffer
  out, lse, dq, dk, dv = _run(q, k, v, do, seg, True, 1.0 / math.sqrt(Dv))
  expect = vals.to(DEV).float().repeat_interleave(n_rep, dim=1)  # (B, Hq, 1, Dv)
  assert (out.float() - expect).abs().max().item() <= 2.0**-7 * vals.abs().max().item() + 1e-3  # P is rounded to 16 bit for PV
  # dQ and dK against the size of one of their terms, |dO| |V| |K|: with a random V of the same size the same kernels
  # give |dQ|, |dK| of 0.03-0.08 on average and 4-7 at most, so a delta or LSE off by one percent would show up as
  # 0.04-0.07 here; what the cancellation leaves in 16-bit arithmetic is 3e-5 (plain) to 7e-3 (packed documents)
  scale = do.float().abs().mean().item() * vals.float().abs().mean().item() * k.float().abs().mean().item()
  assert dq.float().abs().max().item() <= 0.05 * scale, (dq.float().abs().max().item(), scale)
  assert dk.float().abs().max().item() <= 0.05 * scale, (dk.float().abs().max().item(), scale)
  dv_sum = dv.double().sum(dim=2)  # (B, Hkv, Dv)
  do_sum = do.to(DEV).double().sum(dim=2).view(B, Hkv, n_rep, Dv).sum(dim=2)
  rel = (dv_sum - do_sum).abs().max().item() / do_sum.abs().max().item()
  assert rel <= 2e-3, rel
  assert torch.isfinite(lse).all()


def test_llama3_8b_shape_closed_forms():
  _closed_form_check(4, 32, 8, 8192, 128, 128, None, 4321)


def test_llama3_8b_packed_segments_closed_forms():
  seg, _ = packed_segment_ids(4, 8192, 64, 4096, seed=1234 + 2)
  _closed_form_check(4, 32, 8, 8192, 128, 128, seg, 4322)


def test_deepseek_v3_shape_closed_forms():
  _closed_form_check(1, 128, 128, 4096, 192, 128, None, 4323)
