"""Benchmark of the attention hot path on one MI355X.

One step = one forward + backward pass of causal GQA attention at the Llama-3-8B layer shape
(benchmark configuration 2: B=4, S=8192, 32 q heads / 8 kv heads, d=128, bf16) with q, k, v and dO already
resident in HBM.  Prints ONE JSON line:

  value        algorithmic TFLOP/s of the whole step, 6*B*Hq*S^2*d FLOP per step (the reference's own
               MFU convention, torchprime/metrics/train_flops.py:208-228: causal forward 2*B*Hq*S^2*d,
               backward twice that; recomputation is not counted)
  roofline     the dominant kernel (dK/dV backward) against the 2.5 PFLOP/s dense bf16 MFMA peak;
               its launch time comes from HIP events recorded on the launch stream inside the timed
               region (tp_attn_bwd_ex), `kernels` lists the same for every kernel of the step
  cpu_baseline the oracle's eager attention (fwd+bwd by autograd) timed on this host's cores on a
               bounded sample of the same workload (one batch element, one kv-head group)
  extra        RMSNorm and RoPE at the same layer shape: GB/s against the 8 TB/s HBM3E peak

Usage: python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--no-extra]
"""

from __future__ import annotations

import argparse
import ctypes
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
  sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0
PEAK_HBM_GBPS = 8000.0


class HipEvents:
  """hipEvent_t handles through the HIP runtime torch already loaded (timing on an explicit stream)."""

  def __init__(self):
    import torch  # noqa: F401

    self.hip = None
    for name in ("libamdhip64.so.7", "libamdhip64.so", "libamdhip64.so.6"):
      try:
        self.hip = ctypes.CDLL(name)
        break
      except OSError:
        continue
    if self.hip is None:
      raise RuntimeError("HIP runtime not found")
    self.hip.hipEventCreate.argtypes = [ctypes.POINTER(ctypes.c_void_p)]
    self.hip.hipEventRecord.argtypes = [ctypes.c_void_p, ctypes.c_void_p]
    self.hip.hipEventSynchronize.argtypes = [ctypes.c_void_p]
    self.hip.hipEventElapsedTime.argtypes = [ctypes.POINTER(ctypes.c_float), ctypes.c_void_p, ctypes.c_void_p]
    self.hip.hipEventDestroy.argtypes = [ctypes.c_void_p]

  def create(self, n):
    out = []
    for _ in range(n):
      e = ctypes.c_void_p()
      rc = self.hip.hipEventCreate(ctypes.byref(e))
      if rc != 0:
        raise RuntimeError(f"hipEventCreate failed: {rc}")
      out.append(e)
    return out

  def record(self, e, stream):
    rc = self.hip.hipEventRecord(e, ctypes.c_void_p(stream))
    if rc != 0:
      raise RuntimeError(f"hipEventRecord failed: {rc}")

  def elapsed_ms(self, a, b):
    self.hip.hipEventSynchronize(b)
    ms = ctypes.c_float()
    rc = self.hip.hipEventElapsedTime(ctypes.byref(ms), a, b)
    if rc != 0:
      raise RuntimeError(f"hipEventElapsedTime failed: {rc}")
    return ms.value


def make_inputs(B, Hq, Hkv, S, D, dev, seed=1235):
  import torch

  g = torch.Generator(device="cpu").manual_seed(seed)

  def mk(h):
    # (B,S,H,D) memory viewed as (B,H,S,D): what the attention modules hand over
    return torch.randn((B, S, h, D), generator=g, dtype=torch.float32).to(torch.bfloat16).to(dev).transpose(1, 2)

  return mk(Hq), mk(Hkv), mk(Hkv), mk(Hq)


def attention_step_fn(q, k, v, do, sm_scale, hipev=None, ev=None):
  """Returns step(i): one fwd + bwd through the C ABI with caller-owned buffers, events optional."""
  import torch

  from torchprime_amd import _lib

  lib = _lib.load()
  B, Hq, S, D = q.shape
  Hkv = k.shape[1]
  dev = q.device
  out = torch.empty((B, S, Hq, D), dtype=q.dtype, device=dev).transpose(1, 2)
  lse = torch.empty((B, Hq, S), dtype=torch.float32, device=dev)
  dq, dk, dv = (torch.empty_like(t.transpose(1, 2)).transpose(1, 2) for t in (q, k, v))
  ws = torch.empty((lib.tp_attn_bwd_workspace_bytes(B, Hq, S) // 4,), dtype=torch.float32, device=dev)
  st = _lib.stream_ptr(dev)
  s3 = _lib.strides3
  code = _lib.dtype_code(q.dtype)
  EvArr = ctypes.c_void_p * 4

  def step(i):
    if ev is not None:
      hipev.record(ev[i][0], st)
    _lib.call("tp_attn_fwd", q.data_ptr(), k.data_ptr(), v.data_ptr(), None, out.data_ptr(), lse.data_ptr(),
              B, Hq, Hkv, S, S, D, D, s3(q), s3(k), s3(v), s3(out), sm_scale, 1, code, st)  # fmt: skip
    arr = EvArr(*[e.value for e in ev[i][1:5]]) if ev is not None else None
    _lib.call("tp_attn_bwd_ex", do.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), lse.data_ptr(),
              None, dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), ws.data_ptr(), B, Hq, Hkv, S, S, D, D,
              s3(do), s3(q), s3(k), s3(v), s3(out), s3(dq), s3(dk), s3(dv), sm_scale, 1, code, st, arr)  # fmt: skip

  return step, (out, lse, dq, dk, dv)


def bench_attention(args, dev):
  import torch

  B, Hq, Hkv, S, D = 4, 32, 8, 8192, 128
  sm_scale = 1.0 / math.sqrt(D)
  q, k, v, do = make_inputs(B, Hq, Hkv, S, D, dev)
  hipev = HipEvents()
  ev = [hipev.create(5) for _ in range(args.steps)]
  warm, _ = attention_step_fn(q, k, v, do, sm_scale)
  step, _bufs = attention_step_fn(q, k, v, do, sm_scale, hipev, ev)
  for _ in range(args.warmup):
    warm(0)
  torch.cuda.synchronize()
  t0 = time.perf_counter()
  for i in range(args.steps):
    step(i)
  torch.cuda.synchronize()
  t1 = time.perf_counter()
  ms_per_step = (t1 - t0) * 1e3 / args.steps

  unit = B * Hq * S * S * D  # one causal matmul over the attention matrix: 2 * (S^2/2) * d per (b, h)
  flops_step = 6.0 * unit
  # events per step: [0] before fwd, [1] after fwd, [2] after the delta kernel, [3] after dK/dV, [4] after dQ.  Where
  # the dQ kernel computes delta itself there is no delta kernel and dQ runs before dK/dV ([4] is recorded before [3]).
  from torchprime_amd import _lib

  dq_first = bool(_lib.load().tp_attn_bwd_dq_first(S, D, D, 1, 0, 0, _lib.dtype_code(q.dtype)))
  names = ["attn_fwd", "attn_delta", "attn_bwd_dkdv", "attn_bwd_dq"]
  spans = {"attn_fwd": (0, 1), "attn_delta": (1, 2), "attn_bwd_dkdv": (4, 3) if dq_first else (2, 3),
           "attn_bwd_dq": (2, 4) if dq_first else (3, 4)}  # fmt: skip
  algo = {"attn_fwd": 2.0 * unit, "attn_delta": 0.0, "attn_bwd_dkdv": 3.0 * unit, "attn_bwd_dq": 1.0 * unit}
  avg = {}
  for n in names:
    j0, j1 = spans[n]
    avg[n] = sum(hipev.elapsed_ms(ev[i][j0], ev[i][j1]) for i in range(args.steps)) / args.steps
  kernels = {
    n: {"ms": round(avg[n], 4), "algorithmic_TFLOPs": round(algo[n] / (avg[n] * 1e-3) / 1e12, 2) if avg[n] > 0 else None}
    for n in names
  }
  # HBM bytes per launch: counters cannot be read from inside this process, so the figures of the last counter
  # runs of this script (FETCH_SIZE + WRITE_SIZE, two rocprofv3 --pmc runs, each scaled by what the counter reads
  # for the 256 MiB copy of --calib-copy) are kept in a data file next to the summary that documents them,
  # profiles/attn_fwd_bwd_llama3_8b_S8192_hbm_traffic.{md,json}; null when the file is absent.
  measured_traffic = {}
  try:
    with open(os.path.join(ROOT, "profiles", "attn_fwd_bwd_llama3_8b_S8192_hbm_traffic.json")) as f:
      measured_traffic = json.load(f)["hbm_bytes_per_launch"]
  except (OSError, KeyError, ValueError):
    pass
  dom = max(("attn_fwd", "attn_bwd_dkdv", "attn_bwd_dq"), key=lambda n: avg[n])
  achieved = algo[dom] / (avg[dom] * 1e-3) / 1e12
  roofline = {
    "bound": "mfma", "kernel": dom, "achieved": round(achieved, 2), "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
    "frac": round(achieved / PEAK_BF16_TFLOPS, 4), "traffic": measured_traffic.get(dom), "launch_ms": round(avg[dom], 4),
    "step_frac_of_peak": round(flops_step / (ms_per_step * 1e-3) / 1e12 / PEAK_BF16_TFLOPS, 4),
  }  # fmt: skip
  return ms_per_step, flops_step, roofline, kernels, dict(B=B, Hq=Hq, Hkv=Hkv, S=S, D=D)


def bench_norm_rope(dev, iters=20):
  """RMSNorm fwd/bwd on x (4,8192,4096) and RoPE on q (4,32,8192,128) + k (4,8,8192,128), bf16."""
  import torch

  import torchprime_amd as tpa

  res = {}
  g = torch.Generator(device="cpu").manual_seed(7)
  B, S, H = 4, 8192, 4096
  x = torch.randn((B, S, H), generator=g).to(torch.bfloat16).to(dev)
  w = torch.ones((H,), dtype=torch.bfloat16, device=dev)
  dy = torch.randn((B, S, H), generator=g).to(torch.bfloat16).to(dev)
  flush = torch.empty((256 << 20,), dtype=torch.int8, device=dev)  # evict L2 / MALL between iterations

  def timed(fn):
    fn()
    torch.cuda.synchronize()
    ts = []
    for _ in range(iters):
      flush.zero_()
      a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
      a.record()
      fn()
      b.record()
      torch.cuda.synchronize()
      ts.append(a.elapsed_time(b))
    ts.sort()
    return ts[len(ts) // 2]

  # straight through the C ABI with outputs allocated up front: the window between the two events then
  # holds the kernels and nothing of the host-side op dispatch
  from torchprime_amd import _lib

  st = _lib.stream_ptr(dev)
  bf = _lib.dtype_code(torch.bfloat16)
  n, rows = B * S * H, B * S
  y = torch.empty_like(x)
  dx = torch.empty_like(x)
  dw = torch.empty_like(w)
  rstd = torch.empty((rows,), dtype=torch.float32, device=dev)
  ws = torch.empty((_lib.load().tp_rmsnorm_bwd_workspace_bytes(rows, H),), dtype=torch.uint8, device=dev)
  ms = timed(lambda: _lib.call("tp_rmsnorm_fwd", x.data_ptr(), w.data_ptr(), y.data_ptr(), rstd.data_ptr(), rows, H,
                               H, H, 1e-5, bf, bf, st))  # fmt: skip
  res["rmsnorm_fwd"] = {"ms": round(ms, 4), "GBps": round(2 * n * 2 / ms / 1e6, 1)}
  ms = timed(lambda: _lib.call("tp_rmsnorm_bwd", dy.data_ptr(), x.data_ptr(), w.data_ptr(), rstd.data_ptr(),
                               dx.data_ptr(), dw.data_ptr(), ws.data_ptr(), rows, H, H, H, H, bf, bf, st))  # fmt: skip
  res["rmsnorm_bwd"] = {"ms": round(ms, 4), "GBps": round(3 * n * 2 / ms / 1e6, 1)}
  del y, dy, dx, ws

  # The DeepSeek-V3 configuration's own norms: RMSNorm on the q / kv latents (hidden 1536 / 512,
  # model/deepseek_v3/model.py:373,383).  At that configuration's B=1, S=4096 a tensor is 12.6 / 4.2 MB and a launch
  # lasts a few microseconds ("c5" entries: what a layer sees, bound by launch latency); the same kernels over
  # 128 Mi elements ("128Mi" entries) show what they stream.
  for hid in (1536, 512):
    for tag, r5 in (("c5", 4096), ("128Mi", (128 << 20) // hid)):
      x5 = torch.randn((r5, hid), generator=None, device=dev, dtype=torch.bfloat16)
      g5 = torch.randn((r5, hid), generator=None, device=dev, dtype=torch.bfloat16)
      w5 = torch.ones((hid,), dtype=torch.bfloat16, device=dev)
      y5, dx5, dw5 = torch.empty_like(x5), torch.empty_like(x5), torch.empty_like(w5)
      rs5 = torch.empty((r5,), dtype=torch.float32, device=dev)
      ws5 = torch.empty((_lib.load().tp_rmsnorm_bwd_workspace_bytes(r5, hid),), dtype=torch.uint8, device=dev)
      ms = timed(lambda: _lib.call("tp_rmsnorm_fwd", x5.data_ptr(), w5.data_ptr(), y5.data_ptr(), rs5.data_ptr(), r5, hid,
                                   hid, hid, 1e-6, bf, bf, st))  # fmt: skip
      res[f"rmsnorm_fwd_h{hid}_{tag}"] = {"ms": round(ms, 4), "GBps": round(2 * r5 * hid * 2 / ms / 1e6, 1)}
      ms = timed(lambda: _lib.call("tp_rmsnorm_bwd", g5.data_ptr(), x5.data_ptr(), w5.data_ptr(), rs5.data_ptr(),
                                   dx5.data_ptr(), dw5.data_ptr(), ws5.data_ptr(), r5, hid, hid, hid, hid, bf, bf, st))  # fmt: skip
      res[f"rmsnorm_bwd_h{hid}_{tag}"] = {"ms": round(ms, 4), "GBps": round(3 * r5 * hid * 2 / ms / 1e6, 1)}
      del x5, g5, y5, dx5, ws5

  Hq, Hkv, D = 32, 8, 128
  q = torch.randn((B, S, Hq, D), generator=g).to(torch.bfloat16).to(dev).transpose(1, 2)
  k = torch.randn((B, S, Hkv, D), generator=g).to(torch.bfloat16).to(dev).transpose(1, 2)
  qo, ko = torch.empty_like(q), torch.empty_like(k)  # keeps the (B,S,H,D) memory order of q / k
  inv = tpa.default_rope_frequencies(D, 500000.0).to(dev)
  pos = torch.arange(S, device=dev)[None].float()
  cos, sin = tpa.ops.rope_table(inv, pos, 1.0, torch.bfloat16)
  cos, sin = cos.reshape(S, D), sin.reshape(S, D)
  nb = 2 * (q.numel() + k.numel()) * 2
  for name, backward in (("rope_fwd", 0), ("rope_bwd", 1)):
    ms = timed(lambda: _lib.call("tp_rope_apply", q.data_ptr(), k.data_ptr(), cos.data_ptr(), sin.data_ptr(), None,
                                 qo.data_ptr(), ko.data_ptr(), B, Hq, Hkv, S, D, _lib.strides3(q), _lib.strides3(k),
                                 _lib.strides3(qo), _lib.strides3(ko), 0, D, 0, 0, 0, backward, bf, st))  # fmt: skip
    res[name] = {"ms": round(ms, 4), "GBps": round(nb / ms / 1e6, 1)}
  # Llama-4 adjacent-pair rotary on the same tensors presented as (B, S, N, D)
  ms = timed(lambda: _lib.call("tp_rope_apply", q.data_ptr(), k.data_ptr(), cos.data_ptr(), sin.data_ptr(), None,
                               qo.data_ptr(), ko.data_ptr(), B, Hq, Hkv, S, D, _lib.strides3(q), _lib.strides3(k),
                               _lib.strides3(qo), _lib.strides3(ko), 0, D, 0, 0, 2, 0, bf, st))  # fmt: skip
  res["rope_llama4_pairs_fwd"] = {"ms": round(ms, 4), "GBps": round(nb / ms / 1e6, 1)}
  # The DeepSeek-V3 configuration's rotary: interleaved pairs on the 64 rotated dims of q (1, 128, 4096, 64) and of
  # the shared key (1, 1, 4096, 64); model/deepseek_v3/model.py:84-103
  H5, S5, D5 = 128, 4096, 64
  q5 = torch.randn((1, S5, H5, D5), generator=None, device=dev, dtype=torch.bfloat16).transpose(1, 2)
  k5 = torch.randn((1, S5, 1, D5), generator=None, device=dev, dtype=torch.bfloat16).transpose(1, 2)
  qo5, ko5 = torch.empty_like(q5), torch.empty_like(k5)
  inv5 = tpa.default_rope_frequencies(D5, 10000.0).to(dev)
  cos5, sin5 = tpa.ops.rope_table(inv5, torch.arange(S5, device=dev)[None].float(), 1.0, torch.bfloat16)
  cos5, sin5 = cos5.reshape(S5, D5), sin5.reshape(S5, D5)
  nb5 = 2 * (q5.numel() + k5.numel()) * 2
  for name, backward in (("rope_interleaved_c5_fwd", 0), ("rope_interleaved_c5_bwd", 1)):
    ms = timed(lambda: _lib.call("tp_rope_apply", q5.data_ptr(), k5.data_ptr(), cos5.data_ptr(), sin5.data_ptr(), None,
                                 qo5.data_ptr(), ko5.data_ptr(), 1, H5, 1, S5, D5, _lib.strides3(q5), _lib.strides3(k5),
                                 _lib.strides3(qo5), _lib.strides3(ko5), 0, D5, 0, 0, 1, backward, bf, st))  # fmt: skip
    res[name] = {"ms": round(ms, 4), "GBps": round(nb5 / ms / 1e6, 1)}
  del q5, k5, qo5, ko5
  # Llama-4 qk L2 norm over the head dim of q: rows = B * S * Hq of 128
  qrows = B * S * Hq
  rstd_q = torch.empty((qrows,), dtype=torch.float32, device=dev)
  ms = timed(lambda: _lib.call("tp_l2norm_fwd", q.data_ptr(), qo.data_ptr(), rstd_q.data_ptr(), qrows, D, D, D, 1e-6, bf, st))
  res["l2norm_fwd"] = {"ms": round(ms, 4), "GBps": round(2 * q.numel() * 2 / ms / 1e6, 1)}
  ms = timed(lambda: _lib.call("tp_l2norm_bwd", qo.data_ptr(), q.data_ptr(), rstd_q.data_ptr(), qo.data_ptr(), qrows, D, D, D, D, bf, st))
  res["l2norm_bwd"] = {"ms": round(ms, 4), "GBps": round(3 * q.numel() * 2 / ms / 1e6, 1)}
  del q, k, qo, ko, rstd_q

  # residual add + RMSNorm in one pass: reads x and the residual, writes their sum and the normalised row
  x2 = torch.randn((B, S, H), generator=g).to(torch.bfloat16).to(dev)
  r2 = torch.randn((B, S, H), generator=g).to(torch.bfloat16).to(dev)
  h2, y2, dx2 = torch.empty_like(x), torch.empty_like(x), torch.empty_like(x)
  ws2 = torch.empty((_lib.load().tp_rmsnorm_bwd_workspace_bytes(rows, H),), dtype=torch.uint8, device=dev)
  ms = timed(lambda: _lib.call("tp_add_rmsnorm_fwd", x2.data_ptr(), r2.data_ptr(), w.data_ptr(), h2.data_ptr(), y2.data_ptr(),
                               rstd.data_ptr(), rows, H, H, H, H, H, 1e-5, bf, bf, st))  # fmt: skip
  res["add_rmsnorm_fwd"] = {"ms": round(ms, 4), "GBps": round(4 * n * 2 / ms / 1e6, 1)}
  ms = timed(lambda: _lib.call("tp_add_rmsnorm_bwd", x2.data_ptr(), r2.data_ptr(), h2.data_ptr(), w.data_ptr(), rstd.data_ptr(),
                               dx2.data_ptr(), dw.data_ptr(), ws2.data_ptr(), rows, H, H, H, H, H, bf, bf, st))  # fmt: skip
  res["add_rmsnorm_bwd"] = {"ms": round(ms, 4), "GBps": round(4 * n * 2 / ms / 1e6, 1)}
  del x2, r2, h2, y2, dx2, ws2

  # SwiGLU at the Llama-3-8B MLP width (32768 tokens x 14336): fwd reads gate, up, writes out; bwd reads three, writes two
  I = 14336
  gt, up, ot = (torch.randn((rows, I), generator=None, device=dev, dtype=torch.bfloat16) for _ in range(3))
  dgt, dup = torch.empty_like(gt), torch.empty_like(gt)
  ms = timed(lambda: _lib.call("tp_swiglu_fwd", gt.data_ptr(), up.data_ptr(), ot.data_ptr(), rows, I, I, I, I, bf, st))
  res["swiglu_fwd"] = {"ms": round(ms, 4), "GBps": round(3 * rows * I * 2 / ms / 1e6, 1)}
  ms = timed(lambda: _lib.call("tp_swiglu_bwd", ot.data_ptr(), gt.data_ptr(), up.data_ptr(), dgt.data_ptr(), dup.data_ptr(),
                               rows, I, I, I, I, I, I, bf, st))  # fmt: skip
  res["swiglu_bwd"] = {"ms": round(ms, 4), "GBps": round(5 * rows * I * 2 / ms / 1e6, 1)}
  del gt, up, ot, dgt, dup

  # shifted cross entropy over a 128256-entry vocabulary, fp32 logits of one 8192-token sequence: fwd reads the logits
  # once, bwd reads them and writes their gradient
  V, Sx = 128256, 8192
  logits = torch.randn((1, Sx, V), device=dev, dtype=torch.float32)
  labels = torch.randint(0, V, (1, Sx), device=dev)
  lse, rl, lc = (torch.empty((n_,), dtype=torch.float32, device=dev) for n_ in (Sx, Sx, 2))
  dl = torch.ones((1,), dtype=torch.float32, device=dev)
  dlog = torch.empty_like(logits)
  f32 = _lib.dtype_code(torch.float32)
  ms = timed(lambda: _lib.call("tp_cross_entropy_fwd", logits.data_ptr(), labels.data_ptr(), lse.data_ptr(), rl.data_ptr(),
                               lc.data_ptr(), 1, Sx, V, Sx * V, V, Sx, -100, f32, st))  # fmt: skip
  res["cross_entropy_fwd"] = {"ms": round(ms, 4), "GBps": round(Sx * V * 4 / ms / 1e6, 1)}
  ms = timed(lambda: _lib.call("tp_cross_entropy_bwd", logits.data_ptr(), labels.data_ptr(), lse.data_ptr(), lc.data_ptr(),
                               dl.data_ptr(), dlog.data_ptr(), 1, Sx, V, Sx * V, V, Sx, Sx * V, V, -100, f32, st))  # fmt: skip
  res["cross_entropy_bwd"] = {"ms": round(ms, 4), "GBps": round(2 * Sx * V * 4 / ms / 1e6, 1)}
  del logits, dlog
  for v in res.values():
    v["frac_of_hbm_peak"] = round(v["GBps"] / PEAK_HBM_GBPS, 4)
  return res


def packed_segment_ids(B, S, lo, hi, seed):
  """Rows packed with documents of uniform-random lengths lo..hi summing to S (a last piece shorter than lo joins
  its predecessor); ids 0,1,2,... per row.  Returns the ids and the realised lengths."""
  import torch

  g = torch.Generator(device="cpu").manual_seed(seed)
  seg = torch.empty((B, S), dtype=torch.int32)
  lengths = []
  for b in range(B):
    rem, i, pos, ls = S, 0, 0, []
    while rem > 0:
      L = int(torch.randint(lo, hi + 1, (1,), generator=g))
      if rem - L < lo:
        L = rem
      seg[b, pos : pos + L] = i
      pos, rem, i = pos + L, rem - L, i + 1
      ls.append(L)
    lengths.append(ls)
  return seg, lengths


def bench_other_configs(dev, iters=10, only=None):
  """The other benchmark configurations, forward + backward through the C ABI, inputs resident: packed documents
  (configuration 3), the Llama-3-70B layer (4) and the DeepSeek-V3 head dims (5).  FLOPs are counted like the
  headline: 3 x 2 * Hq * (dqk + dv) * (allowed query/key pairs)."""
  import torch

  from torchprime_amd import _lib

  lib = _lib.load()
  res = {}
  cases = [
    ("llama3_8b_packed_segments", 4, 32, 8, 8192, 128, 128, True),
    ("llama3_70b_layer", 1, 64, 8, 8192, 128, 128, False),
    ("deepseek_v3_heads", 1, 128, 128, 4096, 192, 128, False),
  ]
  if only is not None:
    unknown = [n for n in only if n not in [c[0] for c in cases]]
    if unknown:
      sys.exit(f"bench.py: unknown configuration(s) {unknown}")
  for name, B, Hq, Hkv, S, Dqk, Dv, packed in cases:
    if only is not None and name not in only:
      continue
    g = torch.Generator(device="cpu").manual_seed(1236)

    def mk(h, d):
      return torch.randn((B, S, h, d), generator=g, dtype=torch.float32).to(torch.bfloat16).to(dev).transpose(1, 2)

    q, k, v, do = mk(Hq, Dqk), mk(Hkv, Dqk), mk(Hkv, Dv), mk(Hq, Dv)
    seg, pairs = None, B * S * (S + 1) // 2
    if packed:
      seg_cpu, lengths = packed_segment_ids(B, S, 64, 4096, 1236)
      seg = seg_cpu.to(dev)
      pairs = sum(L * (L + 1) // 2 for row in lengths for L in row)
    out = torch.empty((B, S, Hq, Dv), dtype=q.dtype, device=dev).transpose(1, 2)
    lse = torch.empty((B, Hq, S), dtype=torch.float32, device=dev)
    dq, dk, dv = (torch.empty_like(t.transpose(1, 2)).transpose(1, 2) for t in (q, k, v))
    ws = torch.empty((lib.tp_attn_bwd_workspace_bytes(B, Hq, S) // 4,), dtype=torch.float32, device=dev)
    st, s3, code, sm = _lib.stream_ptr(dev), _lib.strides3, _lib.dtype_code(q.dtype), 1.0 / math.sqrt(Dv)

    def fwd():
      _lib.call("tp_attn_fwd", q.data_ptr(), k.data_ptr(), v.data_ptr(), _lib.ptr(seg), out.data_ptr(), lse.data_ptr(),
                B, Hq, Hkv, S, S, Dqk, Dv, s3(q), s3(k), s3(v), s3(out), sm, 1, code, st)  # fmt: skip

    def bwd():
      _lib.call("tp_attn_bwd", do.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), lse.data_ptr(),
                _lib.ptr(seg), dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), ws.data_ptr(), B, Hq, Hkv, S, S, Dqk, Dv,
                s3(do), s3(q), s3(k), s3(v), s3(out), s3(dq), s3(dk), s3(dv), sm, 1, code, st)  # fmt: skip

    for _ in range(3):  # warm-up steps, as for the headline workload
      fwd()
      bwd()

    def timed(fn):
      fn()
      torch.cuda.synchronize()
      a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
      a.record()
      for _ in range(iters):
        fn()
      b.record()
      torch.cuda.synchronize()
      return a.elapsed_time(b) / iters

    tf, tb = timed(fwd), timed(bwd)
    flops = 3.0 * 2.0 * Hq * (Dqk + Dv) * pairs
    tfl = flops / ((tf + tb) * 1e-3) / 1e12
    res[name] = {"fwd_ms": round(tf, 4), "bwd_ms": round(tb, 4), "TFLOPs": round(tfl, 1),
                 "frac_of_bf16_mfma_peak": round(tfl / PEAK_BF16_TFLOPS, 4), "allowed_pairs": pairs,
                 "shape": dict(B=B, Hq=Hq, Hkv=Hkv, S=S, Dqk=Dqk, Dv=Dv)}  # fmt: skip
    del q, k, v, do, out, lse, dq, dk, dv, ws
  return res


def bench_tiny_config_graph(dev, iters=200):
  """Configuration 1 (B2, S128, hidden 512, 8 heads of 64, fp32: the reference's own CPU-runnable case) is bound by
  launches, not by the kernels: the hot path's launches of one layer (RMSNorm, rotary, attention, and their backward)
  timed launched one by one and replayed as one HIP graph.  Microseconds per pass, inputs resident."""
  import torch

  from torchprime_amd import _lib

  lib = _lib.load()
  B, S, H, D = 2, 128, 8, 64
  hidden, dt = H * D, torch.float32
  g = torch.Generator(device="cpu").manual_seed(7)
  rnd = lambda *shape: torch.randn(shape, generator=g, dtype=dt).to(dev)  # noqa: E731
  x, dy, w = rnd(B * S, hidden), rnd(B * S, hidden), rnd(hidden)
  y, dx, dw = torch.empty_like(x), torch.empty_like(x), torch.empty_like(w)
  rstd = torch.empty((B * S,), dtype=torch.float32, device=dev)
  ws_n = torch.empty((lib.tp_rmsnorm_bwd_workspace_bytes(B * S, hidden) // 4,), dtype=torch.float32, device=dev)
  q, k, v, do = (rnd(B, S, H, D).transpose(1, 2) for _ in range(4))
  cos, sin = rnd(1, S, D), rnd(1, S, D)
  qr, kr, dqr, dkr = (torch.empty_like(q.transpose(1, 2)).transpose(1, 2) for _ in range(4))
  out, dq, dk, dv = (torch.empty_like(q.transpose(1, 2)).transpose(1, 2) for _ in range(4))
  lse = torch.empty((B, H, S), dtype=torch.float32, device=dev)
  ws_a = torch.empty((lib.tp_attn_bwd_workspace_bytes(B, H, S) // 4,), dtype=torch.float32, device=dev)
  s3, code, sm = _lib.strides3, _lib.dtype_code(dt), 1.0 / math.sqrt(D)

  def rope(a, b, ao, bo, backward):
    _lib.call("tp_rope_apply", a.data_ptr(), b.data_ptr(), cos.data_ptr(), sin.data_ptr(), None, ao.data_ptr(), bo.data_ptr(),
              B, H, H, S, D, s3(a), s3(b), s3(ao), s3(bo), 0, cos.stride(1), 0, 0, 0, int(backward), code, _lib.stream_ptr(dev))  # fmt: skip

  def one_pass():
    st = _lib.stream_ptr(dev)
    _lib.call("tp_rmsnorm_fwd", x.data_ptr(), w.data_ptr(), y.data_ptr(), rstd.data_ptr(), B * S, hidden, hidden, hidden, 1e-5, code, code, st)
    rope(q, k, qr, kr, False)
    _lib.call("tp_attn_fwd", qr.data_ptr(), kr.data_ptr(), v.data_ptr(), None, out.data_ptr(), lse.data_ptr(),
              B, H, H, S, S, D, D, s3(qr), s3(kr), s3(v), s3(out), sm, 1, code, st)  # fmt: skip
    _lib.call("tp_attn_bwd", do.data_ptr(), qr.data_ptr(), kr.data_ptr(), v.data_ptr(), out.data_ptr(), lse.data_ptr(), None,
              dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), ws_a.data_ptr(), B, H, H, S, S, D, D,
              s3(do), s3(qr), s3(kr), s3(v), s3(out), s3(dq), s3(dk), s3(dv), sm, 1, code, st)  # fmt: skip
    rope(dq, dk, dqr, dkr, True)
    _lib.call("tp_rmsnorm_bwd", dy.data_ptr(), x.data_ptr(), w.data_ptr(), rstd.data_ptr(), dx.data_ptr(), dw.data_ptr(),
              ws_n.data_ptr(), B * S, hidden, hidden, hidden, hidden, code, code, st)  # fmt: skip

  def timed(fn):
    fn()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(iters):
      fn()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / iters * 1e3

  side = torch.cuda.Stream()
  side.wait_stream(torch.cuda.current_stream())
  with torch.cuda.stream(side):
    one_pass()
  torch.cuda.current_stream().wait_stream(side)
  torch.cuda.synchronize()
  eager_us = timed(one_pass)
  ref = [t.clone() for t in (y, out, dqr, dkr, dv, dx, dw)]
  graph = torch.cuda.CUDAGraph()
  with torch.cuda.graph(graph):
    one_pass()
  graph_us = timed(graph.replay)
  same = all(torch.equal(a, b) for a, b in zip(ref, (y, out, dqr, dkr, dv, dx, dw)))
  return {"shape": dict(B=B, S=S, heads=H, head_dim=D, hidden=hidden, dtype="f32"), "launched_one_by_one_us": round(eager_us, 1),
          "hip_graph_replay_us": round(graph_us, 1), "replay_equals_eager": same}  # fmt: skip


def bench_decoder_layer(dev, iters=5):
  """One Llama-3-8B decoder layer (hidden 4096, 32 q / 8 kv heads of 128, MLP 14336; B4, S8192, bf16), forward and
  backward through autograd: the package's modules around stock ``nn.Linear`` GEMMs.  Context for the headline
  number: what share of a layer's step the hot path is.  Milliseconds per forward + backward, inputs resident."""
  import torch

  import torchprime_amd as tpa

  B, S, hidden, H, Hkv, inter = 4, 8192, 4096, 32, 8, 14336
  cfg = tpa.Config(attention_kernel="splash_attention", hidden_size=hidden, num_attention_heads=H, num_key_value_heads=Hkv,
                   intermediate_size=inter, rms_norm_eps=1e-5, hidden_act="silu", attention_dropout=False, attention_bias=False)
  torch.manual_seed(0)
  layer = tpa.LlamaDecoderLayer(cfg, 0).to(dev).to(torch.bfloat16)
  for p in layer.parameters():
    if p.dim() == 2:
      torch.nn.init.normal_(p, std=0.02)
  g = torch.Generator(device="cpu").manual_seed(3)
  x = torch.randn((B, S, hidden), generator=g).to(torch.bfloat16).to(dev).requires_grad_(True)
  do = torch.randn((B, S, hidden), generator=g).to(torch.bfloat16).to(dev)
  rot = tpa.LlamaRotaryEmbedding(hidden // H, 500000.0).to(dev)
  pe = rot(x, torch.arange(S, device=dev)[None].float())

  def step():
    layer.zero_grad(set_to_none=True)
    x.grad = None
    y = layer(x, position_embeddings=pe)
    y.backward(do)

  step()
  torch.cuda.synchronize()
  a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
  a.record()
  for _ in range(iters):
    step()
  b.record()
  torch.cuda.synchronize()
  ms = a.elapsed_time(b) / iters
  params = sum(p.numel() for p in layer.parameters() if p.dim() == 2)
  gemm_flops = 6.0 * B * S * params
  attn_flops = 6.0 * B * H * S * S * (hidden // H)
  return {"shape": dict(B=B, S=S, hidden=hidden, q_heads=H, kv_heads=Hkv, head_dim=hidden // H, intermediate=inter, dtype="bf16"),
          "fwd_bwd_ms": round(ms, 3), "gemm_TFLOP": round(gemm_flops / 1e12, 2), "attention_TFLOP_counted": round(attn_flops / 1e12, 2),
          "layer_TFLOPs": round((gemm_flops + attn_flops) / (ms * 1e-3) / 1e12, 1)}  # fmt: skip


class ClockSampler:
  """Reads the shader clock every 50 ms on a thread while a region runs: the starred line of the first
  /sys/class/drm/card*/device/pp_dpm_sclk that has one (no child process, so it is safe under a profiler); where that
  file is missing or unreadable, `rocm-smi --showclocks` as a child process."""

  def __init__(self):
    import glob

    self.path = None
    for p in sorted(glob.glob("/sys/class/drm/card*/device/pp_dpm_sclk")):
      if self._sysfs(p) is not None:
        self.path = p
        break
    self.samples = []
    self._stop = False
    self._thread = None

  @staticmethod
  def _sysfs(path):
    import re

    try:
      with open(path) as f:
        for line in f:
          if "*" in line:
            m = re.search(r"(\d+)\s*Mhz", line, re.IGNORECASE)
            return int(m.group(1)) if m else None
    except OSError:
      pass
    return None

  @staticmethod
  def _smi():
    import re
    import subprocess

    try:
      out = subprocess.run(["rocm-smi", "--showclocks"], capture_output=True, text=True, timeout=10).stdout
    except (OSError, subprocess.SubprocessError):
      return None
    m = re.search(r"sclk clock level: \S+ \((\d+)Mhz\)", out)
    return int(m.group(1)) if m else None

  def _run(self):
    while not self._stop:
      v = self._sysfs(self.path) if self.path else self._smi()
      if v is not None:
        self.samples.append((time.time(), v))
      time.sleep(0.05)

  def start(self):
    import threading

    self._thread = threading.Thread(target=self._run, daemon=True)
    self._thread.start()

  def stop(self):
    self._stop = True
    if self._thread is not None:
      self._thread.join(timeout=15)

  def mean_mhz(self, t0, t1):
    xs = [v for (t, v) in self.samples if t0 <= t <= t1]
    return round(sum(xs) / len(xs)) if xs else None


def bench_clock_probe(dev, seconds=2.5):
  """What the part sustains under load, and how much of that is the data: the headline attention step and one
  hipBLASLt GEMM (torch.matmul, 8192^3 bf16), each run back to back for `seconds` on normal-distributed inputs (the
  benchmark's data) and on zeros, with the shader clock sampled meanwhile.  The quoted MFMA peak assumes 2.4 GHz; with
  operands that toggle the matrix pipes' inputs the part lowers its clock to hold its power limit, with zeros it does
  not.  A diagnostic: the zero-input rates are no benchmark figures."""
  import torch

  B, Hq, Hkv, S, D = 4, 32, 8, 8192, 128
  sampler = ClockSampler()
  sampler.start()
  res = {"clock_source": sampler.path or "rocm-smi --showclocks"}

  def sustained(fn):
    for _ in range(3):
      fn(0)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    n = 0
    t0 = time.time()
    e0.record()
    while time.time() - t0 < seconds:
      for _ in range(5):
        fn(0)
      n += 5
      torch.cuda.synchronize()
    e1.record()
    torch.cuda.synchronize()
    t1 = time.time()
    return e0.elapsed_time(e1) / n, sampler.mean_mhz(t0 + 0.5, t1)

  try:
    for kind in ("normal", "zeros"):
      n = 8192
      a = torch.randn((n, n), dtype=torch.bfloat16, device=dev) if kind == "normal" else torch.zeros((n, n), dtype=torch.bfloat16, device=dev)
      b = a.clone()
      c = torch.empty_like(a)
      ms, mhz = sustained(lambda i: torch.matmul(a, b, out=c))
      res[f"gemm_8192_{kind}"] = {"ms": round(ms, 4), "TFLOPs": round(2.0 * n**3 / (ms * 1e-3) / 1e12, 1), "sclk_mhz": mhz}
      del a, b, c
      q, k, v, do = make_inputs(B, Hq, Hkv, S, D, dev)
      if kind == "zeros":
        q, k, v, do = (torch.zeros_like(t.transpose(1, 2)).transpose(1, 2) for t in (q, k, v, do))
      step, _bufs = attention_step_fn(q, k, v, do, 1.0 / math.sqrt(D))
      ms, mhz = sustained(step)
      res[f"attn_step_{kind}"] = {
        "ms": round(ms, 4), "algorithmic_TFLOPs": round(6.0 * B * Hq * S * S * D / (ms * 1e-3) / 1e12, 1),
        "executed_TFLOPs": round(9.0 * B * Hq * S * S * D / (ms * 1e-3) / 1e12, 1), "sclk_mhz": mhz,
      }  # fmt: skip
      del q, k, v, do, step, _bufs
      torch.cuda.empty_cache()
  finally:
    sampler.stop()
  return res


def cpu_baseline(max_seconds=24.0):
  """The oracle's eager attention (attention.py:151-170 restated), fwd + bwd by autograd, bf16 inputs, on
  this host's cores: one batch element and one kv-head group (4 q heads) of the benchmark workload."""
  import torch

  from oracle import tprime_oracle as orc

  S, D, n_rep = 8192, 128, 4
  g = torch.Generator(device="cpu").manual_seed(1235)
  q = torch.randn((1, n_rep, S, D), generator=g).to(torch.bfloat16).requires_grad_(True)
  k = torch.randn((1, 1, S, D), generator=g).to(torch.bfloat16).requires_grad_(True)
  v = torch.randn((1, 1, S, D), generator=g).to(torch.bfloat16).requires_grad_(True)
  do = torch.randn((1, n_rep, S, D), generator=g).to(torch.bfloat16)
  mask = orc.causal_additive_mask(S, torch.bfloat16)
  cores = torch.get_num_threads()
  t0 = time.perf_counter()
  reps = 0
  while True:
    out = orc.eager_attention(q, k, v, mask)
    out.backward(do)
    q.grad = k.grad = v.grad = None
    reps += 1
    if time.perf_counter() - t0 > max_seconds / 2:
      break
  sec = (time.perf_counter() - t0) / reps
  flops = 6.0 * 1 * n_rep * S * S * D
  # the two HBM-bound parts of the path on the same cores: eager RMSNorm fwd+bwd on 2048 rows of 4096 and eager
  # rotate-half on q (1, 32, 2048, 128) + k (1, 8, 2048, 128), bf16 (1/16 of the layer's tensors each)
  rows, H = 2048, 4096
  x = torch.randn((rows, H), generator=g).to(torch.bfloat16).requires_grad_(True)
  w = torch.ones((H,), dtype=torch.bfloat16, requires_grad=True)
  dy = torch.randn((rows, H), generator=g).to(torch.bfloat16)
  t0 = time.perf_counter()
  n = 0
  while time.perf_counter() - t0 < 2.0:
    orc.rms_norm(x, w, 1e-5).backward(dy)
    x.grad = w.grad = None
    n += 1
  norm_gbps = 5 * rows * H * 2 / ((time.perf_counter() - t0) / n) / 1e9  # fwd 2 N + bwd 3 N elements of 2 bytes
  qr = torch.randn((1, 2048, 32, D), generator=g).to(torch.bfloat16).transpose(1, 2)
  kr = torch.randn((1, 2048, 8, D), generator=g).to(torch.bfloat16).transpose(1, 2)
  cos, sin = orc.rotary_cos_sin(orc.default_rope_frequencies(D, 500000.0), torch.arange(2048)[None].float(), torch.bfloat16)
  t0 = time.perf_counter()
  n = 0
  while time.perf_counter() - t0 < 2.0:
    orc.apply_rotary_pos_emb(qr, kr, cos, sin)
    n += 1
  rope_gbps = 2 * (qr.numel() + kr.numel()) * 2 / ((time.perf_counter() - t0) / n) / 1e9
  return {
    "value": round(flops / sec / 1e12, 5), "unit": "TFLOP/s", "cores": cores, "kind": "port",
    "sample": f"oracle eager attention fwd+bwd (autograd), bf16, B=1, {n_rep} q heads / 1 kv head, S={S}, d={D}: "
              f"1/32 of one step; {reps} rep(s), {sec:.2f} s each",
    "rmsnorm_fwd_bwd_GBps": round(norm_gbps, 2), "rope_fwd_GBps": round(rope_gbps, 2),
  }  # fmt: skip


# ---- summaries of rocprofv3 runs of this script -----------------------------------------------------------------
_PRE = "from the repository root, after `cd /tmp && export TMPDIR=/tmp && cd -`"
_PROFILE_COMMANDS = {
  "kt_c2": "rocprofv3 --kernel-trace --stats --output-format csv -d {d}/kt_c2 -o kt -- python3 bench.py --steps 10 --warmup 3 --no-cpu --no-extra > {d}/kt_c2.log",
  "pmc_fetch": "rocprofv3 --pmc FETCH_SIZE --output-format csv -d {d}/pmc_fetch -o p -- python3 bench.py --steps 2 --warmup 1 --no-cpu --no-extra --calib-copy",
  "pmc_write": "rocprofv3 --pmc WRITE_SIZE --output-format csv -d {d}/pmc_write -o p -- python3 bench.py --steps 2 --warmup 1 --no-cpu --no-extra --calib-copy",
  "pmc_a": "rocprofv3 --pmc SQ_BUSY_CU_CYCLES SQ_VALU_MFMA_BUSY_CYCLES SQ_ACTIVE_INST_VALU SQ_VALU_MFMA_COEXEC_CYCLES SQ_INSTS_VALU SQ_WAIT_INST_ANY SQ_ACTIVE_INST_ANY SQ_WAVE_CYCLES --output-format csv -d {d}/pmc_a -o p -- python3 bench.py --steps 2 --warmup 1 --no-cpu --no-extra > {d}/pmc_a.log",
  "pmc_b": "rocprofv3 --pmc SQ_INSTS_MFMA SQ_INSTS_LDS SQ_LDS_ADDR_CONFLICT SQ_LDS_BANK_CONFLICT SQ_LDS_IDX_ACTIVE SQ_ACTIVE_INST_LDS SQ_WAIT_INST_LDS SQ_BUSY_CU_CYCLES --output-format csv -d {d}/pmc_b -o p -- python3 bench.py --steps 2 --warmup 1 --no-cpu --no-extra",
  "kt_oc": "rocprofv3 --kernel-trace --stats --output-format csv -d {d}/kt_oc -o kt -- python3 bench.py --other-configs all --steps 10 > {d}/kt_oc.log",
  "kt_extra": "rocprofv3 --kernel-trace --stats --output-format csv -d {d}/kt_extra -o kt -- python3 bench.py --steps 10 --warmup 3 --no-cpu --no-clock-probe > {d}/kt_extra.log",
}  # fmt: skip


def _short_kernel_name(n):
  """tp::name<dtype, integer / boolean template arguments in declaration order> from a mangled or demangled name."""
  import re

  m = re.match(r"_ZN2tp\d+([a-z_0-9]+?)I(.*)", n)
  if not m:
    return re.sub(r"^void ", "", n).split("(")[0][:70]
  rest = m.group(2)
  ty = "f16" if rest.startswith("DF16_") else "bf16" if rest.startswith("DF16b") else "f32" if rest.startswith("f") else "?"
  ints = ",".join(re.findall(r"L[ib](\d+)E", rest))
  return f"tp::{m.group(1)}<{ty},{ints}>"


def _attn_kernel_of(name):
  for key, short in (("dkdv", "attn_bwd_dkdv"), ("bwd_dq", "attn_bwd_dq"), ("attn_fwd", "attn_fwd"), ("delta", "attn_delta")):
    if key in name:
      return short
  return None


def summarize_profiles(d, commit):
  """Turn the rocprofv3 output of the commands in _PROFILE_COMMANDS (run with -d ``d``/<name>, this script's stdout
  in ``d``/<name>.log) into the text summaries and the traffic data file under profiles/.  Parts whose input is
  absent are left as they are."""
  import collections
  import csv

  prof = os.path.join(ROOT, "profiles")
  have = lambda *rel: all(os.path.exists(os.path.join(d, r)) for r in rel)  # noqa: E731
  bench_line = lambda rel: [json.loads(l) for l in open(os.path.join(d, rel)) if l.startswith("{")][-1]  # noqa: E731
  cmd = lambda name: "    " + _PROFILE_COMMANDS[name].format(d=d)  # noqa: E731
  head = f"Library and script at commit {commit}.  "

  def stats_table(rel, keep, min_pct=0.0):
    rows = list(csv.DictReader(open(os.path.join(d, rel))))
    out = ["| kernel | calls | avg us | min us | max us | % of GPU time |", "|---|---:|---:|---:|---:|---:|"]
    for r in rows:
      if keep(r["Name"]) and float(r["Percentage"]) >= min_pct:
        out.append(f"| {_short_kernel_name(r['Name'])} | {r['Calls']} | {float(r['AverageNs']) / 1e3:.1f} | "
                   f"{float(r['MinNs']) / 1e3:.1f} | {float(r['MaxNs']) / 1e3:.1f} | {float(r['Percentage']):.2f} |")
    return out

  ours = lambda n: n.startswith("_ZN2tp") or "tp::" in n  # noqa: E731

  # 1. the headline workload alone: per-kernel averages with and without the warm-up launches
  if have("kt_c2/kt_kernel_stats.csv", "kt_c2/kt_kernel_trace.csv", "kt_c2.log"):
    b = bench_line("kt_c2.log")
    per = collections.defaultdict(list)
    for r in csv.DictReader(open(os.path.join(d, "kt_c2/kt_kernel_trace.csv"))):
      k = _attn_kernel_of(r["Kernel_Name"])
      if k and "f32" not in r["Kernel_Name"]:
        per[k].append((int(r["Start_Timestamp"]), int(r["End_Timestamp"]) - int(r["Start_Timestamp"])))
    warm, steps = b["warmup"], b["steps"]
    o = ["# Kernel trace: attention fwd+bwd at the Llama-3-8B shape (S=8192), the headline workload alone\n",
         head + "Workload: q (4,32,8192,128), k/v (4,8,8192,128) bf16, causal, no segment ids, inputs resident in HBM.",
         f"One MI355X, {warm + steps} steps ({warm} warm-up + {steps} timed); nothing else runs in the process.\n",
         f"Command ({_PRE}):\n", cmd("kt_c2"), "",
         "`kt_kernel_stats.csv` (times in microseconds; template arguments are the integer and boolean ones in declaration order):\n"]
    o += stats_table("kt_c2/kt_kernel_stats.csv", ours) + [""]
    o += ["From `kt_kernel_trace.csv`, the same launches split into warm-up and timed ones, beside the averages this script",
          "measures itself with HIP events on the launch stream (profiler attached):\n",
          "| kernel | launches | avg us, all | avg us, warm-up launches | avg us, timed launches | bench.py events, us |",
          "|---|---:|---:|---:|---:|---:|"]
    timed_avg = {}
    for k in ("attn_fwd", "attn_delta", "attn_bwd_dkdv", "attn_bwd_dq"):
      v = [x[1] for x in sorted(per[k])]
      if not v:
        continue  # (no delta kernel where the dQ kernel computes delta itself)
      if len(v) != warm + steps:
        o.append(f"| {k} | {len(v)} | (expected {warm + steps} launches) | | | |")
        continue
      timed_avg[k] = sum(v[warm:]) / steps
      o.append(f"| {k} | {len(v)} | {sum(v) / len(v) / 1e3:.1f} | {sum(v[:warm]) / warm / 1e3:.1f} | {timed_avg[k] / 1e3:.1f} | "
               f"{b['kernels'][k]['ms'] * 1e3:.1f} |")
    dom = b["roofline"]["kernel"]
    unit = b["config"]["algorithmic_flop_per_step"] / 6.0
    share = {"attn_fwd": 2.0, "attn_bwd_dkdv": 3.0, "attn_bwd_dq": 1.0}[dom]
    if dom in timed_avg:
      t = timed_avg[dom] * 1e-9
      o += ["", f"The same run's bench line: ms_per_step {b['ms_per_step']}, value {b['value']} TFLOP/s = {b['pct_of_bf16_mfma_peak']} % of the "
            "2.5 PFLOP/s bf16 MFMA peak.\n",
            f"Roofline arithmetic for the longest kernel ({dom}): algorithmic FLOPs per launch = {share:.0f} x B*Hq*S^2*d = {share:.0f} x {unit:.4e}",
            f"= {share * unit:.4e} (of the 6 x B*Hq*S^2*d that fwd+bwd count, attributed fwd 2 / dK,dV 3 / dQ 1; recomputed products",
            f"are not counted).  At the traced average of the timed launches, {t * 1e3:.3f} ms, that is {share * unit / t / 1e12:.0f} TFLOP/s = "
            f"{100 * share * unit / t / 2.5e15:.1f} % of the peak;",
            f"the bench line's roofline object says {b['roofline']['achieved']} TFLOP/s = {100 * b['roofline']['frac']:.1f} % from its own "
            f"{b['roofline']['launch_ms']} ms.  The whole step reaches {100 * b['roofline']['step_frac_of_peak']:.1f} %."]
    open(os.path.join(prof, "attn_fwd_bwd_llama3_8b_S8192_kernel_trace.md"), "w").write("\n".join(o) + "\n")

  # 2. HBM traffic per launch, scaled by the 256 MiB copy
  if have("pmc_fetch/p_counter_collection.csv", "pmc_write/p_counter_collection.csv"):
    def counter(rel, name):
      agg, n, copy = collections.defaultdict(float), collections.defaultdict(set), None
      for r in csv.DictReader(open(os.path.join(d, rel))):
        if r["Counter_Name"] != name:
          continue
        if "copyBuffer" in r["Kernel_Name"] and int(r["Grid_Size"]) >= 131072 and copy is None:
          copy = float(r["Counter_Value"])
        k = _attn_kernel_of(r["Kernel_Name"])
        if k and "f32" not in r["Kernel_Name"]:
          agg[k] += float(r["Counter_Value"])
          n[k].add(r["Dispatch_Id"])
      return {k: agg[k] / len(n[k]) for k in agg}, {k: len(n[k]) for k in agg}, copy
    fetch, nf, cf = counter("pmc_fetch/p_counter_collection.csv", "FETCH_SIZE")
    write, _, cw = counter("pmc_write/p_counter_collection.csv", "WRITE_SIZE")
    if cf and cw:
      sf, sw = 262144.0 / cf, 262144.0 / cw
      o = ["# HBM traffic per launch: attention kernels at the Llama-3-8B shape (S=8192, bf16, causal)\n",
           head + f"Two counter runs, one counter each ({_PRE}):\n", cmd("pmc_fetch"), cmd("pmc_write"), "",
           "`--calib-copy` runs one device-to-device copy of 256 MiB (262144 KiB read, 262144 KiB written) before the timed work;",
           f"the counters read {cf:.1f} (FETCH_SIZE) and {cw:.1f} (WRITE_SIZE) for it, so the scale factors are",
           f"{sf:.3f} and {sw:.3f} KiB per count.\n",
           "| kernel | dispatches | FETCH_SIZE avg | WRITE_SIZE avg | HBM read MiB | HBM write MiB |", "|---|---:|---:|---:|---:|---:|"]
      traffic = {}
      for k in ("attn_fwd", "attn_delta", "attn_bwd_dkdv", "attn_bwd_dq"):
        if k not in fetch or k not in write:
          continue
        rd, wr = fetch[k] * sf / 1024, write[k] * sw / 1024
        traffic[k] = float(f"{(rd + wr) * (1 << 20):.3g}")
        o.append(f"| {k}_kernel | {nf[k]} | {fetch[k]:.0f} | {write[k]:.0f} | {rd:.0f} | {wr:.0f} |")
      o += ["", "Algorithmic bytes for comparison (each operand once): forward 640 MiB (q, k, v in; out, lse out), dK/dV kernel",
            "about 770 MiB (q, dO, k, v, row vectors in; dk, dv out), dQ kernel about 1160 MiB (q, dO, out, k, v, lse in; dq and",
            "the two row vectors for dK/dV out: it computes rowsum(dO o O) itself, there is no delta kernel).  The dK/dV kernel's workgroups",
            "(one per 128 kv rows) each stream the Q and dO rows at or below their diagonal, 32 passes over Q and dO on",
            "average; what the table shows beyond the algorithmic bytes is the part of those passes that the L2 shared by a",
            "(batch, kv head) group's workgroups did not serve.  The kernels are MFMA-issue bound, not HBM-bound: at their",
            "launch times the read rates are a quarter of the 8 TB/s peak or less."]
      open(os.path.join(prof, "attn_fwd_bwd_llama3_8b_S8192_hbm_traffic.md"), "w").write("\n".join(o) + "\n")
      with open(os.path.join(prof, "attn_fwd_bwd_llama3_8b_S8192_hbm_traffic.json"), "w") as f:
        json.dump({"source": "profiles/attn_fwd_bwd_llama3_8b_S8192_hbm_traffic.md", "written_by": "bench.py --summarize",
                   "commit": commit, "hbm_bytes_per_launch": traffic}, f, indent=2)
        f.write("\n")

  # 3. MFMA pipe utilisation and LDS counters
  if have("pmc_a/p_counter_collection.csv", "pmc_b/p_counter_collection.csv", "pmc_a.log"):
    def agg(rel):
      a, disp = collections.defaultdict(lambda: collections.defaultdict(float)), collections.defaultdict(dict)
      for r in csv.DictReader(open(os.path.join(d, rel))):
        k = _attn_kernel_of(r["Kernel_Name"])
        if k and "f32" not in r["Kernel_Name"]:
          a[k][r["Counter_Name"]] += float(r["Counter_Value"])
          disp[k][r["Dispatch_Id"]] = int(r["End_Timestamp"]) - int(r["Start_Timestamp"])
      res = {k: {c: x / len(disp[k]) for c, x in v.items()} for k, v in a.items()}
      for k in res:
        res[k]["duration_ns"] = sum(disp[k].values()) / len(disp[k])
      return res
    A, Bc = agg("pmc_a/p_counter_collection.csv"), agg("pmc_b/p_counter_collection.csv")
    b = bench_line("pmc_a.log")
    o = ["# MFMA pipe utilisation, issue and LDS counters: attention kernels at the Llama-3-8B shape (S=8192, bf16, causal)\n",
         head + f"Two counter runs of eight SQ counters each ({_PRE}):\n", cmd("pmc_a"), cmd("pmc_b"), "",
         "Values are averages per launch over the three launches of each run, summed over the chip.  SQ_BUSY_CU_CYCLES counts per compute",
         "unit (256 of them), SQ_VALU_MFMA_BUSY_CYCLES per SIMD (4 per CU), so the MFMA pipes' busy fraction is MFMA_BUSY / (4 x BUSY_CU).",
         "The clock column is BUSY_CU_CYCLES / 256 / the duration of the same dispatches (their timestamps in the counter file; a compute",
         "unit that idles at either end of a launch does not count, so this reads a little under the shader clock).\n",
         "| kernel | BUSY_CU_CYCLES | VALU_MFMA_BUSY_CYCLES | MFMA pipe busy | VALU_MFMA_COEXEC / (4 x BUSY_CU) | ACTIVE_INST_VALU x 4 / (4 x BUSY_CU) | WAIT_INST_ANY / WAVE_CYCLES | INSTS_MFMA | INSTS_LDS | LDS_BANK_CONFLICT / LDS_IDX_ACTIVE | clock GHz |",
         "|---|---:|---:|---:|---:|---:|---:|---:|---:|---:|---:|"]
    tb = tm = 0.0
    clocks = []
    for k in ("attn_fwd", "attn_delta", "attn_bwd_dkdv", "attn_bwd_dq"):
      if k not in A or k not in Bc:
        continue
      a, bb = A[k], Bc[k]
      simd = 4 * a["SQ_BUSY_CU_CYCLES"]
      tb += simd
      tm += a["SQ_VALU_MFMA_BUSY_CYCLES"]
      conf = bb["SQ_LDS_BANK_CONFLICT"] / bb["SQ_LDS_IDX_ACTIVE"] if bb.get("SQ_LDS_IDX_ACTIVE") else 0.0
      ghz = a["SQ_BUSY_CU_CYCLES"] / 256 / a["duration_ns"]
      if k != "attn_delta":
        clocks.append(ghz)
      o.append(f"| {k} | {a['SQ_BUSY_CU_CYCLES']:.3g} | {a['SQ_VALU_MFMA_BUSY_CYCLES']:.3g} | {100 * a['SQ_VALU_MFMA_BUSY_CYCLES'] / simd:.1f} % | "
               f"{100 * a['SQ_VALU_MFMA_COEXEC_CYCLES'] / simd:.1f} % | {100 * 4 * a['SQ_ACTIVE_INST_VALU'] / simd:.1f} % | "
               f"{100 * a['SQ_WAIT_INST_ANY'] / a['SQ_WAVE_CYCLES']:.1f} % | {bb['SQ_INSTS_MFMA']:.3g} | {bb['SQ_INSTS_LDS']:.3g} | {100 * conf:.1f} % | {ghz:.2f} |")
    clk = sum(clocks) / len(clocks)
    o += ["", f"All kernels of a step together: MFMA pipes busy {100 * tm / tb:.1f} % of the SIMD cycles.\n",
          "Cross-check.  The dK/dV kernel executes four S x S x d products per head (S, dP, dV, dK) on the causal half plus the",
          "diagonal tiles: 4 x 1.0995e12 / 32768 FLOP per v_mfma_f32_32x32x16_bf16 = 1.34e8 instructions (SQ_INSTS_MFMA counts per wave) x 32",
          f"cycles = 4.3e9 busy cycles; the counter reads {A['attn_bwd_dkdv']['SQ_VALU_MFMA_BUSY_CYCLES']:.3g}.\n",
          "What the numbers say about the headline fraction.  bench.py counts 6 product-units per step (forward 2, backward 4: the",
          "reference's MFU convention); the kernels execute 9 (forward 2, dK/dV 4, dQ 3: S and dP are recomputed in both backward",
          f"kernels; the dQ kernel's -delta k-steps add 4 % to its MFMA count).  Algorithmic fraction of the 2.5 PFLOP/s peak = MFMA-busy fraction x 6/9 x (sustained clock / 2.4 GHz) = {tm / tb:.3f} x 0.667 x",
          f"{clk / 2.4:.3f} = {100 * tm / tb * 0.6667 * clk / 2.4:.1f} %, against {b['pct_of_bf16_mfma_peak']} % on this run's bench line (the causal diagonal tiles are",
          f"computed whole and counted half).  With this split of the backward and this clock, MFMA pipes that never idled would give",
          f"{100 * 0.6667 * clk / 2.4:.0f} %; 40 % asks for {100 * 0.40 / 0.6667 / (clk / 2.4):.0f} % busy."]
    open(os.path.join(prof, "attn_fwd_bwd_llama3_8b_S8192_mfma_busy.md"), "w").write("\n".join(o) + "\n")

  # 4. the other configurations
  if have("kt_oc/kt_kernel_stats.csv", "kt_oc.log"):
    oc = bench_line("kt_oc.log")["other_configs"]
    o = ["# Kernel trace: attention fwd+bwd at the other benchmark configurations\n",
         head + "Configurations (bf16, causal, inputs resident in HBM; 3 warm-up steps, then 1 + 10 launches of forward and of backward, the 10 timed):\n",
         "- packed documents: q (4,32,8192,128), k/v (4,8,8192,128), segment ids of documents of 64..4096 tokens packed into every row  -> kernels `<...,1,1>` (causal, segments)",
         "- Llama-3-70B layer: q (1,64,8192,128), k/v (1,8,8192,128)  -> the plain causal kernels, as the headline",
         "- DeepSeek-V3 head dims: q/k (1,128,4096,192), v (1,128,4096,128)  -> kernels `<bf16,192,128,...>`\n",
         f"Command ({_PRE}):\n", cmd("kt_oc"), "", "`kt_kernel_stats.csv` (times in microseconds):\n"]
    o += stats_table("kt_oc/kt_kernel_stats.csv", ours) + ["", "The same run's line (torch events around 10 launches; FLOPs = 3 x 2 x Hq x (dqk + dv) x allowed pairs):\n"]
    for n, v in oc.items():
      o.append(f"    {n}: fwd {v['fwd_ms']} ms, bwd {v['bwd_ms']} ms, {v['TFLOPs']} TFLOP/s = {100 * v['frac_of_bf16_mfma_peak']:.1f} % "
               f"of the bf16 MFMA peak ({v['allowed_pairs']} pairs per head)")
    open(os.path.join(prof, "attn_fwd_bwd_other_configs_kernel_trace.md"), "w").write("\n".join(o) + "\n")

  # 5. the bandwidth-bound kernels either side of attention
  if have("kt_extra/kt_kernel_stats.csv", "kt_extra.log"):
    b = bench_line("kt_extra.log")
    o = ["# Kernel trace: the bandwidth-bound kernels either side of attention\n",
         head + "RMSNorm (+ residual add), RoPE (rotate-half, adjacent pairs, interleaved), L2 norm, SwiGLU, shifted cross entropy, at the",
         "sizes bench.py's `extra` leg uses (Llama-3-8B layer: hidden 4096, 32768 rows; the DeepSeek-V3 norm widths 1536 / 512 at their",
         "own row count and at 128 Mi elements; vocabulary 128256 x 8192 rows for the loss).\n",
         f"Command ({_PRE}):\n", cmd("kt_extra"), "",
         "`kt_kernel_stats.csv`, this library's non-attention kernels above 0.02 % of GPU time (times in microseconds; one kernel",
         "template serves several sizes, so a row averages them; the last template argument of rmsnorm_bwd_vec tells the residual-add form",
         "(1) from the plain one (0); the `float` rows with hundreds of calls are the tiny fp32 configuration's launch-by-launch / graph leg):\n"]
    o += stats_table("kt_extra/kt_kernel_stats.csv", lambda n: ours(n) and "attn" not in n, 0.02)
    o += ["", "The same run's `extra` leg (torch events around 20 launches each, a 256 MiB fill between launches to empty the caches):\n"]
    for n, v in b["extra"].items():
      if isinstance(v, dict) and "ms" in v and "GBps" in v:
        o.append(f"    {n}: {v['ms']} ms, {v['GBps']} GB/s = {100 * v['frac_of_hbm_peak']:.1f} % of 8 TB/s")
    open(os.path.join(prof, "norm_rope_mlp_loss_kernel_trace.md"), "w").write("\n".join(o) + "\n")


def main():
  ap = argparse.ArgumentParser()
  ap.add_argument("--gpus", type=int, default=1)
  ap.add_argument("--steps", type=int, default=10)
  ap.add_argument("--warmup", type=int, default=3)
  ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
  ap.add_argument("--no-extra", action="store_true", help="skip the RMSNorm / RoPE bandwidth leg")
  ap.add_argument("--calib-copy", action="store_true",
                  help="also run one 256 MiB device copy (the known-size kernel the HBM counters are scaled by)")
  ap.add_argument("--other-configs", default=None, metavar="NAME[,NAME]",
                  help="run only the named other configurations (llama3_8b_packed_segments, llama3_70b_layer, "
                       "deepseek_v3_heads, or 'all') and print their line: the command the per-configuration kernel traces use")
  ap.add_argument("--decoder-layer", action="store_true",
                  help="run only one Llama-3-8B decoder layer forward + backward (GEMMs included) and print its line")
  ap.add_argument("--tiny-config", action="store_true",
                  help="run only the tiny fp32 configuration's launch-by-launch / HIP graph comparison and print its line")
  ap.add_argument("--no-clock-probe", action="store_true", help="leave the sustained-clock diagnostic out of the default run's extra")
  ap.add_argument("--clock-probe", action="store_true",
                  help="run only the sustained-clock diagnostic (attention step and a hipBLASLt GEMM on normal and on zero inputs, "
                       "shader clock sampled meanwhile) and print its line")
  ap.add_argument("--summarize", default=None, metavar="DIR",
                  help="no GPU work: turn the rocprofv3 output under DIR (see _PROFILE_COMMANDS) into the summaries under profiles/")
  ap.add_argument("--commit", default=None, help="with --summarize: the commit the profiled tree was at (default: git rev-parse)")
  args = ap.parse_args()
  if args.summarize:
    commit = args.commit
    if commit is None:
      import subprocess

      commit = subprocess.run(["git", "-C", ROOT, "rev-parse", "--short", "HEAD"], capture_output=True, text=True).stdout.strip() or "unknown"
    summarize_profiles(args.summarize, commit)
    return
  if args.gpus != 1:
    sys.exit("bench.py measures the one-GPU hot path only: run with --gpus 1 (no multi-GPU path is part of this build)")

  import torch

  import torchprime_amd  # noqa: F401

  if not torch.cuda.is_available():
    sys.exit("bench.py needs a GPU")
  dev = torch.device("cuda", 0)
  if args.calib_copy:
    src = torch.zeros((64 << 20,), dtype=torch.float32, device=dev)
    dst = torch.empty_like(src)
    dst.copy_(src)  # reads 256 MiB, writes 256 MiB
    torch.cuda.synchronize()
    del src, dst
  if args.other_configs:
    names = None if args.other_configs == "all" else args.other_configs.split(",")
    print(json.dumps({"other_configs": bench_other_configs(dev, iters=args.steps, only=names)}))
    return
  if args.decoder_layer:
    print(json.dumps({"llama3_8b_decoder_layer": bench_decoder_layer(dev, iters=args.steps)}))
    return
  if args.tiny_config:
    print(json.dumps({"tiny_fp32_config_hip_graph": bench_tiny_config_graph(dev, iters=args.steps)}))
    return
  if args.clock_probe:
    print(json.dumps({"clock_probe": bench_clock_probe(dev)}))
    return
  ms_per_step, flops_step, roofline, kernels, shape = bench_attention(args, dev)
  extra = None if args.no_extra else bench_norm_rope(dev)
  if extra is not None:
    extra["other_configs"] = bench_other_configs(dev)
    extra["tiny_fp32_config_hip_graph"] = bench_tiny_config_graph(dev)
    extra["llama3_8b_decoder_layer"] = bench_decoder_layer(dev, iters=3)
    if not args.no_clock_probe:
      extra["clock_probe"] = bench_clock_probe(dev, seconds=2.0)
    torch.cuda.empty_cache()
  torch.cuda.empty_cache()
  cpu = None if args.no_cpu else cpu_baseline()
  value = flops_step / (ms_per_step * 1e-3) / 1e12
  line = {
    "metric": "attn fwd+bwd TFLOP/s & % bf16 MFMA peak, Llama-3-8B shape S=8192",
    "value": round(value, 2),
    "unit": "TFLOP/s",
    "n_gpus": 1,
    "steps": args.steps,
    "warmup": args.warmup,
    "ms_per_step": round(ms_per_step, 4),
    "higher_is_better": True,
    "scaling": "weak",
    "vs_baseline": None,
    "dtype": "bf16",
    "data": "synthetic",
    "config": {
      "workload": "Llama-3-8B attention layer fwd+bwd, causal GQA, inputs resident in HBM",
      "B": shape["B"], "S": shape["S"], "q_heads": shape["Hq"], "kv_heads": shape["Hkv"], "head_dim": shape["D"],
      "algorithmic_flop_per_step": flops_step,
    },
    "pct_of_bf16_mfma_peak": round(100.0 * value / PEAK_BF16_TFLOPS, 2),
    "roofline": roofline,
    "kernels": kernels,
    "cpu_baseline": cpu,
    "extra": extra,
  }  # fmt: skip
  print(json.dumps(line))


if __name__ == "__main__":
  main()
