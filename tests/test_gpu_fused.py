"""GPU parity of the steps either side of the attention path: residual add + RMSNorm, Llama-4 L2 norm / adjacent-pair
rotary / temperature scale, SwiGLU and the shifted cross entropy (through the torch.library ops, i.e. the C ABI),
against the CPU oracle on the same seeded inputs.  Element-wise kernels reproduce the eager roundings, so 16-bit
results are compared bit for bit where the arithmetic allows it."""

import pytest
import torch

import torchprime_amd as tpa
from oracle import tprime_oracle as orc
from tests.util import assert_close, randn

pytestmark = pytest.mark.gpu
DEV = "cuda"


# ---- residual add + RMSNorm -----------------------------------------------------------------------------------
@pytest.mark.parametrize("shape,dtype,wdtype", [((2, 128, 512), torch.float32, torch.float32), ((2, 256, 4096), torch.bfloat16, torch.bfloat16),
                                                ((3, 50, 8192), torch.bfloat16, torch.bfloat16), ((5, 333), torch.float16, torch.float16),
                                                ((1, 33, 16384), torch.bfloat16, torch.bfloat16), ((2, 17, 16384), torch.bfloat16, torch.float32), ((2, 700, 7168), torch.bfloat16, torch.bfloat16),
                                                ((4, 7, 1536), torch.bfloat16, torch.float32)])
def test_add_rmsnorm_fwd_bwd(shape, dtype, wdtype):
  hidden, eps = shape[-1], 1e-5
  x, res = randn(shape, 1, dtype), randn(shape, 2, dtype)
  w = (1 + randn((hidden,), 3, torch.float32, 0.1)).to(wdtype)
  odt = torch.result_type(w, x)
  dy, dh = randn(shape, 4, odt), randn(shape, 5, dtype)
  xg, rg, wg = (t.to(DEV).requires_grad_(True) for t in (x, res, w))
  y, h = tpa.ops.add_rmsnorm(xg, rg, wg, eps)
  torch.autograd.backward((y, h), (dy.to(DEV), dh.to(DEV)))
  y_ref, h_ref = orc.add_rms_norm(x, res, w, eps)
  assert torch.equal(h.detach().cpu(), h_ref), "h = residual + x must match the eager add bit for bit"
  if dtype != torch.float32:
    assert (y.detach().cpu() != y_ref).float().mean().item() < 2e-3
  assert_close(y, y_ref, "y", max_abs=1e-5 if dtype == torch.float32 else 2e-2, rel_l2=1e-6 if dtype == torch.float32 else 1e-3, scale_abs=True)
  # gradients: autograd through the eager-order expression in fp64 (rounding of the normalised value as in the reference)
  h64 = h_ref.double().requires_grad_(True)
  w64 = w.double().requires_grad_(True)
  hn = h64 * torch.rsqrt(h64.pow(2).mean(-1, keepdim=True) + eps)
  hr = hn + (hn.detach().to(dtype).double() - hn.detach())
  torch.autograd.backward((w64 * hr, h64), (dy.double(), dh.double()))
  assert_close(xg.grad, h64.grad, "dx", scale_abs=True)
  assert torch.equal(xg.grad, rg.grad)
  assert_close(wg.grad, w64.grad, "dw", scale_abs=True)


def test_add_rms_norm_helper_matches_separate_ops_and_decoder_wiring():
  B, S, H = 2, 64, 1024
  norm = tpa.LlamaRMSNorm(H, eps=1e-5).to(DEV).to(torch.bfloat16)
  attn_out, residual = randn((B, S, H), 7, torch.bfloat16).to(DEV), randn((B, S, H), 8, torch.bfloat16).to(DEV)
  y, h = tpa.add_rms_norm(attn_out, residual, norm)
  h2 = residual + attn_out           # model/llama/model.py:288-291, op by op
  y2 = norm(h2)
  assert torch.equal(h, h2) and torch.equal(y, y2)


# ---- Llama-4 ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("shape", [(2, 33, 8, 128), (1, 200, 5, 64), (3, 7, 2, 256), (4, 256)])  # head dims: a row is at most one wavefront of 16-byte vectors
def test_l2norm_fwd_bwd(dtype, shape):
  x, dy = randn(shape, 11, dtype), randn(shape, 12, dtype)
  xg = x.to(DEV).requires_grad_(True)
  m = tpa.Llama4TextL2Norm(1e-6)
  y = m(xg)
  y.backward(dy.to(DEV))
  y_ref = orc.l2_norm(x, 1e-6)
  if dtype == torch.float32:
    assert_close(y, y_ref, "y", max_abs=1e-5, rel_l2=1e-6)
  else:
    assert (y.detach().cpu() != y_ref).float().mean().item() < 2e-3  # one rounding; the row sum's order may flip an ulp
    assert_close(y, y_ref, "y", rel_l2=1e-3, scale_abs=True)
  x64 = x.double().requires_grad_(True)
  orc.l2_norm(x64, 1e-6).backward(dy.double())
  assert_close(xg.grad, x64.grad, "dx", max_abs=1e-5 if dtype == torch.float32 else 2e-2, scale_abs=True)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
def test_llama4_rotary_bitwise_and_backward(dtype):
  B, S, N, Nk, D = 2, 130, 8, 2, 128
  q, k = randn((B, S, N, D), 21, dtype), randn((B, S, Nk, D), 22, dtype)
  pos = torch.arange(S)[None].float().repeat(B, 1)
  rot = tpa.Llama4TextRotaryEmbedding(D, 500000.0).to(DEV)
  cos, sin = rot(q.to(DEV), pos.to(DEV))
  qd, kd = q.to(DEV).requires_grad_(True), k.to(DEV).requires_grad_(True)
  qo, ko = tpa.apply_rotary_emb(qd, kd, (cos, sin))
  qr, kr = orc.apply_rotary_emb_llama4(q, k, cos.cpu(), sin.cpu())
  assert qo.shape == q.shape and torch.equal(qo.detach().cpu(), qr) and torch.equal(ko.detach().cpu(), kr)
  gq, gk = randn(q.shape, 23, dtype), randn(k.shape, 24, dtype)
  torch.autograd.backward((qo, ko), (gq.to(DEV), gk.to(DEV)))
  q64, k64 = q.double().requires_grad_(True), k.double().requires_grad_(True)
  a, b = orc.apply_rotary_emb_llama4(q64, k64, cos.cpu().double(), sin.cpu().double())
  torch.autograd.backward((a, b), (gq.double(), gk.double()))
  tol = dict(max_abs=1e-5, rel_l2=1e-6) if dtype == torch.float32 else dict(scale_abs=True)
  assert_close(qd.grad, q64.grad, "dq", **tol)
  assert_close(kd.grad, k64.grad, "dk", **tol)


def test_llama4_temperature_scale_bitwise():
  B, S, N, D = 2, 300, 4, 128
  q = randn((B, S, N, D), 31, torch.bfloat16)
  qd = q.to(DEV).requires_grad_(True)
  out = tpa.apply_attn_temperature(qd, 64.0, 0.1)
  ref = orc.apply_attn_temperature(q, 64.0, 0.1)
  assert torch.equal(out.detach().cpu(), ref)
  torch.testing.assert_close(tpa.attn_temperature_scales(S, 64.0, 0.1), orc.attn_temperature_scales(S, 64.0, 0.1))
  g = randn(q.shape, 32, torch.bfloat16)
  out.backward(g.to(DEV))
  assert torch.equal(qd.grad.cpu(), orc.apply_attn_temperature(g, 64.0, 0.1))


# ---- SwiGLU -------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("shape", [(2, 64, 1024), (3, 14336), (1, 5, 8, 256)])
def test_swiglu_fwd_bwd(dtype, shape):
  g, u, do = randn(shape, 41, dtype, 2.0), randn(shape, 42, dtype), randn(shape, 43, dtype)
  gd, ud = g.to(DEV).requires_grad_(True), u.to(DEV).requires_grad_(True)
  out = tpa.ops.swiglu(gd, ud)
  out.backward(do.to(DEV))
  ref = orc.swiglu(g, u)
  if dtype == torch.float32:
    assert_close(out, ref, "out", max_abs=2e-6, rel_l2=1e-6)
  else:
    # silu rounded, then the product rounded, as the two eager ops do; the device exponential may flip a last bit
    assert (out.detach().cpu() != ref).float().mean().item() < 2e-3
    assert_close(out, ref, "out", rel_l2=1e-3, scale_abs=True)
  g64, u64 = g.double().requires_grad_(True), u.double().requires_grad_(True)
  orc.swiglu(g64, u64).backward(do.double())
  tol = dict(max_abs=1e-5, rel_l2=1e-6) if dtype == torch.float32 else dict(scale_abs=True)
  assert_close(gd.grad, g64.grad, "dgate", **tol)
  assert_close(ud.grad, u64.grad, "dup", **tol)


def test_llama_mlp_module():
  cfg = tpa.Config(hidden_size=512, intermediate_size=1408, hidden_act="silu")
  m = tpa.LlamaMLP(cfg).to(DEV).to(torch.bfloat16)
  w = {"gate_proj.weight": randn((1408, 512), 51, torch.bfloat16, 0.02), "up_proj.weight": randn((1408, 512), 52, torch.bfloat16, 0.02),
       "down_proj.weight": randn((512, 1408), 53, torch.bfloat16, 0.02)}
  m.load_state_dict({k: v.to(DEV) for k, v in w.items()})
  x = randn((2, 96, 512), 54, torch.bfloat16)
  y = m(x.to(DEV))
  xd = x.double()
  ref = orc.swiglu(xd @ w["gate_proj.weight"].double().T, xd @ w["up_proj.weight"].double().T) @ w["down_proj.weight"].double().T
  assert_close(y, ref, "mlp", scale_abs=True)


# ---- cross entropy ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("B,S,V,dtype", [(2, 17, 1000, torch.float32), (1, 64, 32003, torch.float32), (3, 9, 128, torch.float32),
                                         (2, 33, 4096, torch.bfloat16)])
def test_cross_entropy_fwd_bwd(B, S, V, dtype):
  logits = randn((B, S, V), 61, dtype, 3.0)
  labels = torch.randint(0, V, (B, S), generator=torch.Generator().manual_seed(62))
  labels[0, 3] = -100
  labels[-1, -1] = -100
  ld = logits.to(DEV).requires_grad_(True)
  loss = tpa.cross_entropy_loss(ld, labels.to(DEV), V)
  (loss * 1.7).backward()
  l64 = logits.double().requires_grad_(True)
  ref = orc.cross_entropy_loss(l64, labels, V)
  (ref * 1.7).backward()
  assert loss.dtype == torch.float32 and loss.dim() == 0
  assert abs(loss.item() - ref.item()) <= 2e-6 * max(1.0, abs(ref.item()))
  if dtype == torch.float32:
    assert_close(ld.grad, l64.grad, "dlogits", max_abs=1e-7, rel_l2=1e-5)
  else:
    assert_close(ld.grad, l64.grad, "dlogits", max_abs=1e-4, rel_l2=5e-3)  # gradients are rounded to bf16
  assert ld.grad[:, -1].abs().max().item() == 0  # the last position has no target


def test_cross_entropy_all_ignored_is_nan_like_torch_and_vocab_128k_row():
  V = 128256
  logits = randn((1, 3, V), 63, torch.float32, 2.0)
  labels = torch.tensor([[5, 100000, 128255]])
  loss = tpa.cross_entropy_loss(logits.to(DEV), labels.to(DEV), V)
  assert loss.item() == pytest.approx(orc.cross_entropy_loss(logits.double(), labels, V).item(), rel=2e-6)
  ign = torch.full((1, 3), -100)
  assert torch.isnan(tpa.cross_entropy_loss(logits.to(DEV), ign.to(DEV), V))
  assert torch.isnan(orc.cross_entropy_loss(logits, ign, V))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_cross_entropy_with_a_masked_vocabulary_range(dtype):
  """-inf logits (a masked range of the vocabulary, here the low column indices, which every thread of the kernel
  meets first, and a block in the middle) add nothing to the row's sum: the loss and the gradient stay finite and
  match the oracle, and the masked columns get gradient 0."""
  B, S, V = 2, 9, 5000
  logits = randn((B, S, V), 71, dtype, 2.0)
  logits[:, :, :2100] = float("-inf")
  logits[:, :, 3000:3300] = float("-inf")
  labels = torch.randint(2100, 3000, (B, S), generator=torch.Generator().manual_seed(72))
  ld = logits.to(DEV).requires_grad_(True)
  loss = tpa.cross_entropy_loss(ld, labels.to(DEV), V)
  loss.backward()
  l64 = logits.double().requires_grad_(True)
  ref = orc.cross_entropy_loss(l64, labels, V)
  ref.backward()
  assert torch.isfinite(loss).item()
  assert abs(loss.item() - ref.item()) <= 2e-6 * max(1.0, abs(ref.item()))
  assert torch.isfinite(ld.grad).all().item()
  assert ld.grad[:, :, :2100].abs().max().item() == 0 and ld.grad[:, :, 3000:3300].abs().max().item() == 0
  assert_close(ld.grad, l64.grad, "dlogits", max_abs=1e-7 if dtype == torch.float32 else 1e-4, rel_l2=1e-5 if dtype == torch.float32 else 5e-3)

