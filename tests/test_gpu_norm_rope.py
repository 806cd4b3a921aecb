"""GPU parity: RMSNorm and rotary kernels (through the torch.library ops, i.e. through the C ABI)
against the CPU oracle on the same seeded inputs."""

import pytest
import torch

import torchprime_amd as tpa
from oracle import tprime_oracle as orc
from tests.util import assert_close, randn

pytestmark = pytest.mark.gpu
DEV = "cuda"


@pytest.mark.parametrize(
  "shape,dtype,wdtype,eps",
  [
    ((2, 128, 512), torch.float32, torch.float32, 1e-5),      # C1
    ((2, 256, 4096), torch.bfloat16, torch.bfloat16, 1e-5),   # Llama-3-8B hidden
    ((1, 64, 8192), torch.bfloat16, torch.bfloat16, 1e-5),    # Llama-3-70B hidden
    ((1, 512, 1536), torch.bfloat16, torch.bfloat16, 1e-6),   # DeepSeek q latent
    ((1, 512, 512), torch.bfloat16, torch.bfloat16, 1e-6),    # DeepSeek kv latent
    ((3, 7, 4096), torch.bfloat16, torch.float32, 1e-5),      # fp32 weight: result promotes to fp32
    ((1, 40, 16384), torch.bfloat16, torch.bfloat16, 1e-5),   # Llama-3.1-405B hidden: 16 waves per row in the backward
    ((2, 9, 16384), torch.bfloat16, torch.float32, 1e-5),     # the same with fp32 weight and dy
    ((1, 70, 7168), torch.bfloat16, torch.bfloat16, 1e-6),    # DeepSeek-V3 hidden
    ((3, 900, 5120), torch.float16, torch.float16, 1e-5),     # Llama-4 hidden; more rows than partial dw rows
    ((1, 5000, 1024), torch.bfloat16, torch.bfloat16, 1e-5),  # single-wave rows, more rows than partial dw rows
    ((5, 333), torch.float16, torch.float16, 1e-6),           # ragged hidden: scalar path
    ((4, 3, 100), torch.float32, torch.float32, 1e-6),
    ((0, 512), torch.bfloat16, torch.bfloat16, 1e-6),         # empty
  ],
)
def test_rmsnorm_fwd_bwd(shape, dtype, wdtype, eps):
  hidden = shape[-1]
  x = randn(shape, 11, dtype)
  w = (1.0 + randn((hidden,), 12, torch.float32, 0.1)).to(wdtype)
  dy = randn(shape, 13, torch.result_type(w, x))

  xg = x.to(DEV).requires_grad_(True)
  wg = w.to(DEV).requires_grad_(True)
  y = tpa.ops.rmsnorm(xg, wg, eps)
  assert y.dtype == torch.result_type(w, x) and y.shape == x.shape
  y.backward(dy.to(DEV))

  # same rounding order as the eager reference: bit-level agreement expected up to reduction order
  y_ref = orc.rms_norm(x, w, eps)
  if x.numel():
    # same roundings as the eager expression: identical bits except where the row sum's last ulp
    # (reduction order) flips a rounding
    if dtype != torch.float32:
      mism = (y.detach().cpu() != y_ref).float().mean().item()
      assert mism < 2e-3, f"{mism:.2e} of the elements differ from the eager-order oracle"
    assert_close(y, y_ref, "y vs eager-order oracle", max_abs=1e-5 if dtype == torch.float32 else 2e-2,
                 rel_l2=1e-6 if dtype == torch.float32 else 1e-3, scale_abs=True)
    assert_close(y, orc.rms_norm_exact(x, w, eps), "y vs fp64", scale_abs=True)
  # gradients: dx against autograd through the fp64 formula; dw against the gradient the reference's own autograd
  # defines, sum_rows dy * (normalised value rounded to the input dtype), evaluated in fp64.  (Against the
  # unrounded formula the rounding of each of the `rows` terms adds up to ~2^-9 sqrt(rows): relative-L2 only.)
  x64 = x.double().requires_grad_(True)
  w64 = w.double().requires_grad_(True)
  orc.rms_norm_exact(x64, w64, eps).backward(dy.double())
  if x.numel():
    assert_close(xg.grad, x64.grad, "dx", scale_abs=True)
    _, dw_eager = orc.rms_norm_grads_eager_order(x, w, dy, eps)
    assert_close(wg.grad, dw_eager, "dw", scale_abs=True)
    assert_close(wg.grad, w64.grad, "dw vs unrounded formula", max_abs=float("inf"), rel_l2=1e-2)
  else:
    assert wg.grad.abs().max().item() == 0


def test_rmsnorm_module_names_and_state_dict():
  for cls in (tpa.LlamaRMSNorm, tpa.MixtralRMSNorm, tpa.DeepseekV3RMSNorm):
    m = cls(256, eps=1e-5).to(DEV)
    assert list(m.state_dict().keys()) == ["weight"] and m.variance_epsilon == 1e-5
    x = randn((2, 9, 256), 5, torch.bfloat16)
    m = m.to(torch.bfloat16)
    assert_close(m(x.to(DEV)), orc.rms_norm_exact(x, m.weight.detach().cpu(), 1e-5), cls.__name__, scale_abs=True)


def test_rmsnorm_rejects_cpu_tensors():
  with pytest.raises(RuntimeError):
    tpa.ops.rmsnorm(torch.ones(2, 8), torch.ones(8), 1e-6)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("Bp,S,half,scaling", [(1, 128, 32, 1.0), (2, 1000, 64, 1.0), (1, 8192, 64, 1.0), (1, 512, 32, 0.7)])
def test_rope_table(dtype, Bp, S, half, scaling):
  inv = orc.default_rope_frequencies(2 * half, 500000.0)
  pos = torch.arange(S)[None].float().repeat(Bp, 1) + (torch.arange(Bp)[:, None] * 3).float()
  cos, sin = tpa.ops.rope_table(inv.to(DEV), pos.to(DEV), scaling, dtype)
  cr, sr = orc.rotary_cos_sin(inv, pos, dtype, scaling)
  assert cos.shape == (Bp, S, 2 * half) and cos.dtype == dtype
  # device sinf/cosf vs host: a few fp32 ulp on |angle| up to 8191 rad, at most one 16-bit ulp after rounding
  tol = 1e-5 if dtype == torch.float32 else 8e-3
  assert (cos.cpu().float() - cr.float()).abs().max().item() <= tol
  assert (sin.cpu().float() - sr.float()).abs().max().item() <= tol


def _rope_inputs(B, Hq, Hkv, S, D, dtype, theta=500000.0):
  q = randn((B, S, Hq, D), 21, dtype).transpose(1, 2)
  k = randn((B, S, Hkv, D), 22, dtype).transpose(1, 2)
  pos = torch.arange(S)[None].float()
  cos, sin = orc.rotary_cos_sin(orc.default_rope_frequencies(D, theta), pos, dtype)
  return q, k, cos, sin


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
@pytest.mark.parametrize("B,Hq,Hkv,S,D", [(2, 8, 8, 128, 64), (2, 32, 8, 512, 128), (1, 3, 1, 77, 32)])
def test_rope_apply_matches_eager_bitwise(dtype, B, Hq, Hkv, S, D):
  q, k, cos, sin = _rope_inputs(B, Hq, Hkv, S, D, dtype)
  qo, ko = tpa.apply_rotary_pos_emb(q.to(DEV), k.to(DEV), cos.to(DEV), sin.to(DEV))
  qr, kr = orc.apply_rotary_pos_emb(q, k, cos, sin)
  # same products, same roundings, same order: identical bits
  assert torch.equal(qo.cpu(), qr) and torch.equal(ko.cpu(), kr)
  assert qo.shape == q.shape and qo.transpose(1, 2).is_contiguous()


def test_rope_apply_backward():
  q, k, cos, sin = _rope_inputs(2, 8, 2, 96, 64, torch.bfloat16)
  gq, gk = randn(q.shape, 31, torch.bfloat16), randn(k.shape, 32, torch.bfloat16)
  qd, kd = q.to(DEV).requires_grad_(True), k.to(DEV).requires_grad_(True)
  qo, ko = tpa.apply_rotary_pos_emb(qd, kd, cos.to(DEV), sin.to(DEV))
  torch.autograd.backward((qo, ko), (gq.to(DEV), gk.to(DEV)))
  q64, k64 = q.double().requires_grad_(True), k.double().requires_grad_(True)
  qr, kr = orc.apply_rotary_pos_emb(q64, k64, cos.double(), sin.double())
  torch.autograd.backward((qr, kr), (gq.double(), gk.double()))
  assert_close(qd.grad, q64.grad, "dq", scale_abs=True)
  assert_close(kd.grad, k64.grad, "dk", scale_abs=True)


def test_rope_interleave_deepseek_layout():
  # q_rot (B,128,S,64) is the tail of a 192-wide head; k_rot (B,1,S,64) the tail of the 576-wide latent
  B, S = 1, 200
  qfull = randn((B, S, 16, 192), 41, torch.bfloat16)
  kvfull = randn((B, S, 576), 42, torch.bfloat16)
  pos = torch.arange(S)[None].float()
  cos, sin = orc.rotary_cos_sin(orc.default_rope_frequencies(64, 10000.0), pos, torch.bfloat16)

  def split(qf, kvf):
    q_rot = qf.transpose(1, 2)[..., 128:]
    k_rot = kvf[..., 512:].view(B, 1, S, 64)
    return q_rot, k_rot

  q_rot, k_rot = split(qfull, kvfull)
  qr, kr = orc.apply_rotary_pos_emb_interleave(q_rot, k_rot, cos, sin)
  qd, kd = qfull.to(DEV).requires_grad_(True), kvfull.to(DEV).requires_grad_(True)
  q_rot_d, k_rot_d = split(qd, kd)
  qo, ko = tpa.apply_rotary_pos_emb_interleave(q_rot_d, k_rot_d, cos.to(DEV), sin.to(DEV))
  assert torch.equal(qo.cpu(), qr) and torch.equal(ko.cpu(), kr)
  gq, gk = randn(qr.shape, 43, torch.bfloat16), randn(kr.shape, 44, torch.bfloat16)
  torch.autograd.backward((qo, ko), (gq.to(DEV), gk.to(DEV)))
  q64, k64 = qfull.double().requires_grad_(True), kvfull.double().requires_grad_(True)
  a, b_ = split(q64, k64)
  qr64, kr64 = orc.apply_rotary_pos_emb_interleave(a, b_, cos.double(), sin.double())
  torch.autograd.backward((qr64, kr64), (gq.double(), gk.double()))
  assert_close(qd.grad, q64.grad, "dq", scale_abs=True)
  assert_close(kd.grad, k64.grad, "dkv", scale_abs=True)


def test_rope_mixtral_gather():
  B, Hq, Hkv, S, D = 2, 4, 2, 50, 64
  q = randn((B, S, Hq, D), 51, torch.bfloat16).transpose(1, 2)
  k = randn((B, S, Hkv, D), 52, torch.bfloat16).transpose(1, 2)
  old = torch.get_default_dtype()
  emb = tpa.MixtralRotaryEmbedding(D, max_position_embeddings=256, base=1e6)
  torch.set_default_dtype(old)
  cos, sin = emb(q.to(DEV), seq_len=S)
  assert cos.shape == (S, D)
  pos = torch.stack([torch.arange(S), torch.arange(S).flip(0)]).float()  # the models pass float ids
  qo, ko = tpa.apply_rotary_pos_emb(q.to(DEV), k.to(DEV), cos, sin, pos.to(DEV))
  t = torch.arange(256)[None].float()
  cr, sr = orc.rotary_cos_sin(orc.default_rope_frequencies(D, 1e6), t, torch.float32)
  cr, sr = cr[0][:S].to(torch.bfloat16), sr[0][:S].to(torch.bfloat16)
  qr, kr = orc.apply_rotary_pos_emb(q, k, cr, sr, pos, gather=True)
  assert_close(qo, qr.float(), "q", scale_abs=True)
  assert_close(ko, kr.float(), "k", scale_abs=True)


def test_rotary_embedding_modules():
  x = torch.zeros((1, 1, 1, 1), dtype=torch.bfloat16, device=DEV)
  pos = torch.arange(300, device=DEV)[None].float()
  m = tpa.LlamaRotaryEmbedding(128, 500000.0, tpa.RopeScaling()).to(DEV)
  cos, sin = m(x, pos)
  inv = orc.llama3_rope_frequencies(128, 500000.0, factor=8.0)
  cr, sr = orc.rotary_cos_sin(inv, pos.cpu(), torch.bfloat16)
  assert (cos.cpu().float() - cr.float()).abs().max() <= 8e-3 and (sin.cpu().float() - sr.float()).abs().max() <= 8e-3
  assert "inv_freq" not in m.state_dict()
  cfg = tpa.Config(
    rope_theta=10000, head_dim=64, hidden_size=7168, num_attention_heads=128, max_position_embeddings=4096,
    rope_scaling=dict(beta_fast=32, beta_slow=1, factor=40, mscale=1.0, mscale_all_dim=1.0,
                      original_max_position_embeddings=4096, rope_type="yarn", type="yarn"),
  )
  d = tpa.DeepseekV3RotaryEmbedding(cfg).to(DEV)
  assert d.attention_scaling == 1.0
  cos, sin = d(x, pos)
  cr, sr = orc.rotary_cos_sin(orc.default_rope_frequencies(64, 10000.0), pos.cpu(), torch.bfloat16)
  assert (cos.cpu().float() - cr.float()).abs().max() <= 8e-3


def test_rope_gather_rejects_positions_outside_the_table():
  # the reference's cos[position_ids] raises IndexError (model/mixtral/model.py:136-137)
  B, H, S, D = 1, 2, 16, 64
  q = randn((B, S, H, D), 61, torch.bfloat16).transpose(1, 2).to(DEV)
  inv = tpa.default_rope_frequencies(D, 1e6).to(DEV)
  cos, sin = tpa.ops.rope_table(inv, torch.arange(S, device=DEV)[None].float(), 1.0, torch.bfloat16)
  cos, sin = cos[0], sin[0]
  ok = torch.arange(S, device=DEV)[None]
  tpa.apply_rotary_pos_emb(q, q, cos, sin, ok)
  with pytest.raises(IndexError):
    tpa.apply_rotary_pos_emb(q, q, cos, sin, ok + 1)


# ---- full-size cases (the benchmark's layer shape) ---------------------------------------------------------
def test_rmsnorm_full_size_llama3_8b():
  """x (4, 8192, 4096) bf16: 32768 rows walk the grid-stride backward with 512 partial-dw rows.  y and dx are
  checked on a sample of rows against the oracle, dw (a sum over every row) in full."""
  B, S, H, eps = 4, 8192, 4096, 1e-5
  g = torch.Generator(device="cpu").manual_seed(1234 + 1)
  x = torch.randn((B, S, H), generator=g).to(torch.bfloat16)
  dy = torch.randn((B, S, H), generator=g).to(torch.bfloat16)
  w = (1 + 0.1 * torch.randn((H,), generator=g)).to(torch.bfloat16)
  xg, wg = x.to(DEV).requires_grad_(True), w.to(DEV).requires_grad_(True)
  y = tpa.ops.rmsnorm(xg, wg, eps)
  y.backward(dy.to(DEV))
  rows = torch.arange(0, B * S, 97)
  xs, dys = x.view(-1, H)[rows], dy.view(-1, H)[rows]
  y_ref = orc.rms_norm(xs, w, eps)
  ys = y.detach().view(-1, H)[rows.to(DEV)].cpu()
  assert (ys != y_ref).float().mean().item() < 2e-3  # same roundings as the eager expression
  assert_close(ys, y_ref, "y rows", rel_l2=1e-3, scale_abs=True)
  x64 = xs.double().requires_grad_(True)
  orc.rms_norm_exact(x64, w.double(), eps).backward(dys.double())
  assert_close(xg.grad.view(-1, H)[rows.to(DEV)], x64.grad, "dx rows", scale_abs=True)
  # dw over all rows, eager order (normalised value rounded to bf16), accumulated in fp64 chunk by chunk
  dw = torch.zeros(H, dtype=torch.float64)
  for r0 in range(0, B * S, 4096):
    xc = x.view(-1, H)[r0 : r0 + 4096].float()
    h = (xc * torch.rsqrt(xc.pow(2).mean(-1, keepdim=True) + eps)).to(torch.bfloat16)
    dw += (dy.view(-1, H)[r0 : r0 + 4096].double() * h.double()).sum(0)
  assert_close(wg.grad, dw, "dw", scale_abs=True)
  assert torch.isfinite(y.float()).all() and torch.isfinite(xg.grad.float()).all()


def test_rope_full_size_llama3_8b_bitwise():
  """q (4, 32, 8192, 128) and k (4, 8, 8192, 128) bf16, (B,S,H,D) memory: identical bits to the eager expression
  (evaluated with the oracle's function on the same device tensors, and on the host for one batch element)."""
  B, Hq, Hkv, S, D = 4, 32, 8, 8192, 128
  g = torch.Generator(device="cpu").manual_seed(1234 + 1)
  q = torch.randn((B, S, Hq, D), generator=g).to(torch.bfloat16).transpose(1, 2)
  k = torch.randn((B, S, Hkv, D), generator=g).to(torch.bfloat16).transpose(1, 2)
  pos = torch.arange(S)[None].float()
  cos, sin = orc.rotary_cos_sin(orc.default_rope_frequencies(D, 500000.0), pos, torch.bfloat16)
  qd, kd, cd, sd = q.to(DEV), k.to(DEV), cos.to(DEV), sin.to(DEV)
  qo, ko = tpa.apply_rotary_pos_emb(qd, kd, cd, sd)
  qr, kr = orc.apply_rotary_pos_emb(qd, kd, cd, sd)
  assert torch.equal(qo, qr) and torch.equal(ko, kr)
  qh, kh = orc.apply_rotary_pos_emb(q[2:3], k[2:3], cos, sin)
  assert torch.equal(qo[2:3].cpu(), qh) and torch.equal(ko[2:3].cpu(), kh)
  # backward = the transposed rotation: also bit-identical to the eager expression with -sin
  gq, gk = torch.ops.tprime.rope_apply(qd, kd, cd, sd, None, 0, True)
  gqr, gkr = orc.apply_rotary_pos_emb(qd, kd, cd, -sd)
  assert torch.equal(gq, gqr) and torch.equal(gk, gkr)


@pytest.mark.parametrize("hidden", [1536, 512])
def test_rmsnorm_full_size_deepseek_latents(hidden):
  """The DeepSeek-V3 configuration's norms: x (1, 4096, hidden) bf16 with hidden = the q / kv latent widths, eps 1e-6
  (narrow rows: one wave per row for 512).  y bit-compared with the eager-order oracle, dx and dw against fp64."""
  S, eps = 4096, 1e-6
  g = torch.Generator(device="cpu").manual_seed(1234 + 4)
  x = torch.randn((1, S, hidden), generator=g).to(torch.bfloat16)
  dy = torch.randn((1, S, hidden), generator=g).to(torch.bfloat16)
  w = (1 + 0.1 * torch.randn((hidden,), generator=g)).to(torch.bfloat16)
  xg, wg = x.to(DEV).requires_grad_(True), w.to(DEV).requires_grad_(True)
  y = tpa.ops.rmsnorm(xg, wg, eps)
  y.backward(dy.to(DEV))
  y_ref = orc.rms_norm(x, w, eps)
  assert (y.detach().cpu() != y_ref).float().mean().item() < 2e-3
  assert_close(y, y_ref, "y", rel_l2=1e-3, scale_abs=True)
  x64 = x.double().requires_grad_(True)
  orc.rms_norm_exact(x64, w.double(), eps).backward(dy.double())
  assert_close(xg.grad, x64.grad, "dx", scale_abs=True)
  _, dw = orc.rms_norm_grads_eager_order(x, w, dy, eps)
  assert_close(wg.grad, dw, "dw", scale_abs=True)


def test_rope_full_size_deepseek_interleaved_bitwise():
  """The DeepSeek-V3 configuration's rotary step: the 64 rotated dims of q (1, 128, 4096, 64) and of the shared key
  (1, 1, 4096, 64), interleaved pairs, theta 1e4: identical bits to the eager expression, forward and backward."""
  Hq, S, D = 128, 4096, 64
  g = torch.Generator(device="cpu").manual_seed(1234 + 4)
  q = torch.randn((1, S, Hq, D), generator=g).to(torch.bfloat16).transpose(1, 2)
  k = torch.randn((1, S, 1, D), generator=g).to(torch.bfloat16).transpose(1, 2)
  pos = torch.arange(S)[None].float()
  cos, sin = orc.rotary_cos_sin(orc.default_rope_frequencies(D, 10000.0), pos, torch.bfloat16)
  qd, kd, cd, sd = q.to(DEV), k.to(DEV), cos.to(DEV), sin.to(DEV)
  qo, ko = tpa.apply_rotary_pos_emb_interleave(qd, kd, cd, sd)
  qr, kr = orc.apply_rotary_pos_emb_interleave(q, k, cos, sin)
  assert torch.equal(qo.cpu(), qr) and torch.equal(ko.cpu(), kr)
  # gradient of sum(out * w) with respect to the inputs, against autograd through the eager expression in fp64
  wq = torch.randn((1, S, Hq, D), generator=g).to(torch.bfloat16).transpose(1, 2)
  qg = qd.clone().requires_grad_(True)
  kg = kd.clone().requires_grad_(True)
  qo2, ko2 = tpa.apply_rotary_pos_emb_interleave(qg, kg, cd, sd)
  (qo2.float() * wq.to(DEV).float()).sum().backward()
  q64 = q.double().requires_grad_(True)
  qr64, _ = orc.apply_rotary_pos_emb_interleave(q64, k.double(), cos.double(), sin.double())
  (qr64 * wq.double()).sum().backward()
  assert_close(qg.grad, q64.grad, "dq rot", scale_abs=True)
  assert kg.grad is None or float(kg.grad.abs().max()) == 0.0


def test_rope_offsets_beyond_32_bits():
  """A q view whose rows lie 2^18 elements apart: offsets inside one batch element pass 2^31 elements, which
  takes the kernel instantiation with 64-bit per-lane offsets."""
  B, H, S, D = 1, 2, 8192 + 8, 128
  stride_s = 1 << 18
  base = torch.empty(((S - 1) * stride_s + H * D,), dtype=torch.bfloat16, device=DEV)
  q = base.as_strided((B, H, S, D), (0, D, stride_s, 1))
  g = torch.Generator(device="cpu").manual_seed(5)
  vals = torch.randn((B, H, S, D), generator=g).to(torch.bfloat16)
  q.copy_(vals.to(DEV))
  assert (S - 1) * stride_s >= 2**31
  pos = torch.arange(S)[None].float()
  cos, sin = orc.rotary_cos_sin(orc.default_rope_frequencies(D, 500000.0), pos, torch.bfloat16)
  qo, ko = tpa.apply_rotary_pos_emb(q, q, cos.to(DEV), sin.to(DEV))
  qr, _ = orc.apply_rotary_pos_emb(vals, vals, cos, sin)
  assert torch.equal(qo.cpu(), qr) and torch.equal(ko.cpu(), qr)
