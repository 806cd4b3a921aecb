"""The ops under HIP graph capture.  The library's entry points launch on the stream they are given and neither
allocate, clear memory with a memset node, nor wait for the device, so a caller may record them into a graph
(torch.cuda.graph makes the capture stream the current one, which is the stream the ops hand down).  Each graph is
replayed several times with new contents in its static inputs, with the program's own eager work and
synchronisations between the replays, and every replay must equal the eager result bit for bit: the kernels are
deterministic (no atomics), so anything else is a capture problem."""

import pytest
import torch

import torchprime_amd as tpa
from tests.util import randn

pytestmark = pytest.mark.gpu
DEV = "cuda"
REPLAYS = 4


def _capture(fn, warmup=2):
  """Warm up on a side stream (first calls look up kernel attributes and fill host-side caches), then capture."""
  side = torch.cuda.Stream()
  side.wait_stream(torch.cuda.current_stream())
  with torch.cuda.stream(side):
    for _ in range(warmup):
      fn()
  torch.cuda.current_stream().wait_stream(side)
  torch.cuda.synchronize()
  g = torch.cuda.CUDAGraph()
  with torch.cuda.graph(g):
    out = fn()
  return g, out


def _same(got, want, what):
  for i, (a, b) in enumerate(zip(got, want)):
    assert torch.equal(a, b), f"{what}: output {i} of the replay differs from the eager result"


@pytest.mark.parametrize("dtype,dims,with_ids", [(torch.bfloat16, (128, 128), False), (torch.bfloat16, (128, 128), True),
                                                 (torch.float16, (64, 64), True), (torch.bfloat16, (192, 128), False),
                                                 (torch.float32, (64, 64), False)])
def test_attention_forward_backward_replays(dtype, dims, with_ids):
  B, Hq, Hkv, S = 2, 8, 2, 640
  dqk, dv = dims
  q = torch.empty((B, Hq, S, dqk), dtype=dtype, device=DEV)
  k = torch.empty((B, Hkv, S, dqk), dtype=dtype, device=DEV)
  v = torch.empty((B, Hkv, S, dv), dtype=dtype, device=DEV)
  do = torch.empty((B, Hq, S, dv), dtype=dtype, device=DEV)
  seg = torch.zeros((B, S), dtype=torch.int32, device=DEV) if with_ids else None
  scale = dqk**-0.5

  def step():
    out, lse = tpa.ops.attn_fwd(q, k, v, seg, scale, True)
    dq, dk, dv_ = tpa.ops.attn_bwd(do, q, k, v, out, lse, seg, scale, True)
    return out, lse, dq, dk, dv_

  def fill(seed):
    q.copy_(randn(q.shape, seed, dtype)); k.copy_(randn(k.shape, seed + 1, dtype))
    v.copy_(randn(v.shape, seed + 2, dtype)); do.copy_(randn(do.shape, seed + 3, dtype))
    if with_ids:
      # a different document layout each time: the tile lists are rebuilt on the device by every replay
      cuts = torch.sort(torch.randint(1, S, (B, 3 + seed % 3), generator=torch.Generator().manual_seed(seed)), dim=1).values
      ids = (torch.arange(S)[None, :, None] >= cuts[:, None, :]).sum(-1).to(torch.int32)
      seg.copy_(ids)

  fill(100)
  g, outs = _capture(step)
  for r in range(REPLAYS):
    fill(200 + 7 * r)
    want = [t.clone() for t in step()]            # eager, on the ordinary stream
    torch.cuda.synchronize()
    for t in outs:
      t.fill_(float("nan")) if t.is_floating_point() else t.zero_()
    g.replay()
    torch.cuda.synchronize()
    _same(outs, want, f"attention replay {r}")


def test_layer_elementwise_chain_replays():
  """RMSNorm (+ residual), rotary, SwiGLU and the cross entropy, forward and backward, as one graph."""
  B, S, H, Hq, D, V = 2, 256, 1024, 8, 128, 4096
  dt = torch.bfloat16
  x = torch.empty((B, S, H), dtype=dt, device=DEV)
  res = torch.empty_like(x)
  w = (1 + randn((H,), 1, torch.float32, 0.1)).to(dt).to(DEV)
  dy = torch.empty_like(x)
  cos = randn((1, S, D), 2, dt).to(DEV)
  sin = randn((1, S, D), 3, dt).to(DEV)
  logits = torch.empty((B, S, V), dtype=torch.float32, device=DEV)
  labels = torch.randint(0, V, (B, S), generator=torch.Generator().manual_seed(4)).to(DEV)
  labels[0, :5] = -100
  one = torch.ones((), dtype=torch.float32, device=DEV)

  def step():
    y, h, rstd = tpa.ops.add_rmsnorm_fwd(x, res, w, 1e-5)
    dx, dw = tpa.ops.add_rmsnorm_bwd(dy, dy, h, w, rstd)
    y2, rstd2 = tpa.ops.rmsnorm_fwd(h, w, 1e-5)
    dx2, dw2 = tpa.ops.rmsnorm_bwd(dy, h, w, rstd2)
    qh = y.view(B, S, Hq, D).transpose(1, 2)
    q_rot, k_rot = tpa.ops.rope_apply_op(qh, qh, cos, sin, None, 0, False)
    act = tpa.ops.swiglu_fwd(y, y2)
    dgate, dup = tpa.ops.swiglu_bwd(dy, y, y2)
    loss, lse, lc = tpa.ops.cross_entropy_fwd(logits, labels, -100)
    dlogits = tpa.ops.cross_entropy_bwd(one, logits, labels, lse, lc, -100)
    return y, h, dx, dw, dx2, dw2, q_rot, k_rot, act, dgate, dup, loss, dlogits

  def fill(seed):
    x.copy_(randn(x.shape, seed, dt)); res.copy_(randn(x.shape, seed + 1, dt)); dy.copy_(randn(x.shape, seed + 2, dt))
    logits.copy_(randn(logits.shape, seed + 3, torch.float32, 3.0))

  fill(10)
  g, outs = _capture(step)
  for r in range(REPLAYS):
    fill(20 + 5 * r)
    want = [t.clone() for t in step()]
    torch.cuda.synchronize()
    for t in outs:
      t.fill_(float("nan"))
    g.replay()
    torch.cuda.synchronize()
    _same(outs, want, f"element-wise chain replay {r}")


def test_no_alloc_rmsnorm_backward_replays():
  """The allocation-free entry point is the one meant for capture: called through the C ABI with no torch allocation
  inside the captured region at all."""
  from torchprime_amd import _lib
  rows, hidden = 1024, 2048
  dt = torch.bfloat16
  x = torch.empty((rows, hidden), dtype=dt, device=DEV)
  dy = torch.empty_like(x)
  w = (1 + randn((hidden,), 1, torch.float32, 0.1)).to(dt).to(DEV)
  rstd = torch.empty((rows,), dtype=torch.float32, device=DEV)
  dx, dw = torch.empty_like(x), torch.empty_like(w)

  def step():
    _lib.call("tp_rmsnorm_bwd_noalloc", dy.data_ptr(), x.data_ptr(), w.data_ptr(), rstd.data_ptr(), dx.data_ptr(), dw.data_ptr(),
              rows, hidden, hidden, hidden, hidden, _lib.dtype_code(dt), _lib.dtype_code(dt), _lib.stream_ptr(x.device))
    return dx, dw

  def fill(seed):
    x.copy_(randn(x.shape, seed, dt)); dy.copy_(randn(x.shape, seed + 1, dt))
    rstd.copy_(torch.rsqrt(x.float().pow(2).mean(-1) + 1e-5))

  fill(1)
  g, outs = _capture(step)
  for r in range(REPLAYS):
    fill(30 + r)
    want = tpa.ops.rmsnorm_bwd(dy, x, w, rstd)
    torch.cuda.synchronize()
    for t in outs:
      t.fill_(float("nan"))
    g.replay()
    torch.cuda.synchronize()
    _same(outs, want, f"allocation-free RMSNorm backward replay {r}")
