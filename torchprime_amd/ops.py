"""``torch.library`` custom ops (namespace ``tprime``) over the HIP kernels in ``libtprime_hip.so``.

Pattern follows the reference's own custom-op precedent, ``xla::offload_name`` in
torchprime/torch_xla_models/offloading.py:14-38 (custom_op + register_fake + register_autograd), so
the ops stay traceable by functorch/AOT autograd as torchprime's remat tooling expects
(torchprime/torch_xla_models/tests/test_remat_all.py:143-202).

Every op is GPU-only: CPU tensors raise, nothing falls back to torch math.
"""

from __future__ import annotations

import math

import torch
from torch import Tensor

from . import _lib

__all__ = [
  "rmsnorm",
  "rope_table",
  "rope_apply",
  "attention",
]


# ------------------------------------------------------------------------------------------------
# helpers
# ------------------------------------------------------------------------------------------------
def _empty_like_heads(x: Tensor, last: int | None = None) -> Tensor:
  """New (B,H,S,D') tensor.  Head-minor inputs (the (B,S,H,D)-memory views the attention modules
  build with ``.view(B,S,H,D).transpose(1,2)``) get the same head-minor memory order so the caller's
  ``transpose(1,2).contiguous()`` afterwards is free; anything else gets plain contiguous memory."""
  B, H, S, D = x.shape
  D = D if last is None else last
  if x.stride(1) < x.stride(2):
    return torch.empty((B, S, H, D), dtype=x.dtype, device=x.device).transpose(1, 2)
  return torch.empty((B, H, S, D), dtype=x.dtype, device=x.device)


def _rows(x: Tensor) -> Tensor:
  """(..., hidden) -> (rows, hidden) with unit inner stride (view when possible)."""
  h = x.shape[-1]
  x2 = x.reshape(-1, h)
  if x2.stride(-1) != 1 or (x2.shape[0] > 1 and x2.stride(0) < h):
    x2 = x2.contiguous()
  return x2


# ------------------------------------------------------------------------------------------------
# RMSNorm
# ------------------------------------------------------------------------------------------------
@torch.library.custom_op("tprime::rmsnorm_fwd", mutates_args=(), device_types="cuda")
def rmsnorm_fwd(x: Tensor, weight: Tensor, eps: float) -> tuple[Tensor, Tensor]:
  _lib.require_gpu(x, weight)
  hidden = x.shape[-1]
  if weight.shape != (hidden,):
    raise ValueError(f"weight shape {tuple(weight.shape)} does not match hidden size {hidden}")
  x2 = _rows(x)
  w = weight.contiguous()
  out_dtype = torch.result_type(weight, x)
  rows = x2.shape[0]
  y = torch.empty((rows, hidden), dtype=out_dtype, device=x.device)
  rstd = torch.empty((rows,), dtype=torch.float32, device=x.device)
  if rows:
    _lib.call(
      "tp_rmsnorm_fwd", x2.data_ptr(), w.data_ptr(), y.data_ptr(), rstd.data_ptr(), rows, hidden,
      x2.stride(0) if rows > 1 else hidden, hidden, float(eps), _lib.dtype_code(x.dtype),
      _lib.dtype_code(w.dtype), _lib.stream_ptr(x.device),
    )  # fmt: skip
  return y.view(*x.shape[:-1], hidden), rstd


@rmsnorm_fwd.register_fake
def _(x, weight, eps):
  out_dtype = torch.result_type(weight, x)
  rows = x.numel() // max(x.shape[-1], 1)
  return x.new_empty(x.shape, dtype=out_dtype), x.new_empty((rows,), dtype=torch.float32)


@torch.library.custom_op("tprime::rmsnorm_bwd", mutates_args=(), device_types="cuda")
def rmsnorm_bwd(dy: Tensor, x: Tensor, weight: Tensor, rstd: Tensor) -> tuple[Tensor, Tensor]:
  _lib.require_gpu(dy, x, weight, rstd)
  hidden = x.shape[-1]
  x2, g2, w = _rows(x), _rows(dy), weight.contiguous()
  rows = x2.shape[0]
  dx = torch.empty((rows, hidden), dtype=x.dtype, device=x.device)
  dw = torch.empty((hidden,), dtype=w.dtype, device=x.device)
  if rows == 0:
    return dx.view(x.shape), dw.zero_()
  lib = _lib.load()
  ws = torch.empty((lib.tp_rmsnorm_bwd_workspace_bytes(rows, hidden) // 4,), dtype=torch.float32, device=x.device)
  _lib.call(
    "tp_rmsnorm_bwd", g2.data_ptr(), x2.data_ptr(), w.data_ptr(), rstd.data_ptr(), dx.data_ptr(), dw.data_ptr(),
    ws.data_ptr(), rows, hidden, g2.stride(0) if rows > 1 else hidden, x2.stride(0) if rows > 1 else hidden, hidden,
    _lib.dtype_code(x.dtype), _lib.dtype_code(w.dtype), _lib.stream_ptr(x.device),
  )  # fmt: skip
  return dx.view(x.shape), dw


@rmsnorm_bwd.register_fake
def _(dy, x, weight, rstd):
  return torch.empty_like(x, memory_format=torch.contiguous_format), torch.empty_like(weight)


def _rmsnorm_setup(ctx, inputs, output):
  x, weight, _eps = inputs
  _y, rstd = output
  ctx.save_for_backward(x, weight, rstd)


def _rmsnorm_backward(ctx, dy, _drstd):
  x, weight, rstd = ctx.saved_tensors
  dx, dw = rmsnorm_bwd(dy.to(torch.result_type(weight, x)), x, weight, rstd)
  return dx, dw, None


rmsnorm_fwd.register_autograd(_rmsnorm_backward, setup_context=_rmsnorm_setup)


def rmsnorm(x: Tensor, weight: Tensor, eps: float) -> Tensor:
  """``weight * (x.float() * rsqrt(mean(x.float()**2, -1) + eps)).to(x.dtype)`` in one pass."""
  _lib.require_gpu(x, weight)
  return rmsnorm_fwd(x, weight, eps)[0]


# ------------------------------------------------------------------------------------------------
# rotary tables and apply
# ------------------------------------------------------------------------------------------------
@torch.library.custom_op("tprime::rope_table", mutates_args=(), device_types="cuda")
def rope_table(inv_freq: Tensor, position_ids: Tensor, attention_scaling: float, dtype: torch.dtype) -> tuple[Tensor, Tensor]:
  """cos/sin tables ``(Bp, S, 2*half)`` from ``inv_freq (half)`` and float ``position_ids (Bp, S)``."""
  _lib.require_gpu(inv_freq, position_ids)
  f = inv_freq.to(torch.float32).contiguous()
  p = position_ids.to(torch.float32).contiguous()
  if p.dim() != 2 or f.dim() != 1:
    raise ValueError("expected inv_freq (half,) and position_ids (batch, seq)")
  Bp, S = p.shape
  half = f.shape[0]
  cos = torch.empty((Bp, S, 2 * half), dtype=dtype, device=f.device)
  sin = torch.empty_like(cos)
  _lib.call(
    "tp_rope_table", f.data_ptr(), p.data_ptr(), cos.data_ptr(), sin.data_ptr(), Bp, S, half,
    float(attention_scaling), _lib.dtype_code(dtype), _lib.stream_ptr(f.device),
  )  # fmt: skip
  return cos, sin


@rope_table.register_fake
def _(inv_freq, position_ids, attention_scaling, dtype):
  Bp, S = position_ids.shape
  c = inv_freq.new_empty((Bp, S, 2 * inv_freq.shape[0]), dtype=dtype)
  return c, torch.empty_like(c)


# verdicts of the position range check, keyed on the tensor's storage, shape and version: a model hands the same
# position_ids tensor to every layer (and to the backward of each), so the device reduction and its host sync run
# once per tensor, not once per call
_POS_OK: dict = {}


def _check_positions(pos: Tensor, rows: int) -> None:
  """``cos[position_ids]`` raises IndexError for ids outside the table (model/mixtral/model.py:136-137); so does this."""
  key = (pos.data_ptr(), tuple(pos.shape), pos._version, rows)
  if key in _POS_OK:
    return
  lo, hi = (int(v) for v in torch.stack((pos.min(), pos.max())).tolist()) if pos.numel() else (0, 0)
  if lo < -rows or hi >= rows:
    raise IndexError(f"position id {hi if hi >= rows else lo} is out of bounds for a rotary table of {rows} rows")
  if lo < 0:
    raise NotImplementedError("negative position ids (indexing the table from its end) are not supported")
  if len(_POS_OK) > 64:
    _POS_OK.clear()
  _POS_OK[key] = True


def _rope_launch(q, k, cos, sin, pos, interleaved: bool, backward: bool):
  dev = _lib.require_gpu(q, k, cos, sin, pos)
  if q.dim() != 4 or (k is not None and k.dim() != 4):
    raise ValueError("rotary apply expects (batch, heads, seq, dim) tensors")
  B, Hq, S, D = q.shape
  if k is not None and (k.shape[0] != B or k.shape[2] != S or k.shape[3] != D or k.dtype != q.dtype):
    raise ValueError(f"q {tuple(q.shape)} and k {tuple(k.shape)} disagree on batch/seq/dim or dtype")
  if cos.dtype != q.dtype or sin.dtype != q.dtype:
    cos, sin = cos.to(q.dtype), sin.to(q.dtype)
  esz = q.element_size()

  def _prep(t):
    if t is None:
      return None
    ok = t.stride(-1) == 1 and t.data_ptr() % 16 == 0 and all((s * esz) % 16 == 0 for s in t.stride()[:3])
    return t if ok else t.contiguous()

  q, k = _prep(q), _prep(k)
  if pos is not None:
    # table gather (Mixtral): cos/sin are (T, D), pos is (B or 1, S) integer
    if cos.dim() != 2:
      raise ValueError("with position_ids the cos/sin tables must be (max_pos, dim)")
    cos, sin = cos.contiguous(), sin.contiguous()
    pos = pos.to(torch.int64).contiguous()
    if pos.dim() == 1:
      pos = pos[None]
    if pos.shape[-1] != S or pos.shape[0] not in (1, B):
      raise ValueError(f"position_ids shape {tuple(pos.shape)} does not match (batch, seq) = ({B}, {S})")
    _check_positions(pos, cos.shape[0])
    cs_b, cs_s, pos_b, table_rows = 0, cos.stride(0), (pos.stride(0) if pos.shape[0] == B and B > 1 else 0), cos.shape[0]
  else:
    if cos.dim() == 2:
      cos, sin = cos[None], sin[None]
    if cos.dim() != 3 or cos.shape[1] != S or cos.shape[2] != D or cos.shape[0] not in (1, B):
      raise ValueError(f"cos/sin shape {tuple(cos.shape)} does not broadcast to (batch, seq, dim) = ({B}, {S}, {D})")
    if cos.stride(-1) != 1 or sin.stride() != cos.stride():
      cos, sin = cos.contiguous(), sin.contiguous()
    cs_b, cs_s, pos_b, table_rows = (cos.stride(0) if cos.shape[0] == B and B > 1 else 0), cos.stride(1), 0, 0
  qo = _empty_like_heads(q)
  ko = _empty_like_heads(k) if k is not None else None
  z3 = _lib._I64x3(0, 0, 0)
  _lib.call(
    "tp_rope_apply", q.data_ptr(), _lib.ptr(k), cos.data_ptr(), sin.data_ptr(), _lib.ptr(pos), qo.data_ptr(),
    _lib.ptr(ko), B, Hq, 0 if k is None else k.shape[1], S, D, _lib.strides3(q),
    z3 if k is None else _lib.strides3(k), _lib.strides3(qo), z3 if k is None else _lib.strides3(ko),
    cs_b, cs_s, pos_b, table_rows, int(interleaved), int(backward), _lib.dtype_code(q.dtype), _lib.stream_ptr(dev),
  )  # fmt: skip
  return qo, ko


@torch.library.custom_op("tprime::rope_apply", mutates_args=(), device_types="cuda")
def rope_apply_op(
  q: Tensor, k: Tensor, cos: Tensor, sin: Tensor, pos: Tensor | None, interleaved: bool, backward: bool
) -> tuple[Tensor, Tensor]:
  return _rope_launch(q, k, cos, sin, pos, interleaved, backward)


@rope_apply_op.register_fake
def _(q, k, cos, sin, pos, interleaved, backward):
  return _empty_like_heads(q), _empty_like_heads(k)


def _rope_setup(ctx, inputs, output):
  _q, _k, cos, sin, pos, interleaved, backward = inputs
  ctx.save_for_backward(cos, sin, pos) if pos is not None else ctx.save_for_backward(cos, sin)
  ctx.has_pos = pos is not None
  ctx.interleaved = interleaved
  ctx.backward_mode = backward


def _rope_backward(ctx, dq, dk):
  if ctx.has_pos:
    cos, sin, pos = ctx.saved_tensors
  else:
    (cos, sin), pos = ctx.saved_tensors, None
  # the transpose of the transposed rotation is the rotation itself
  gq, gk = rope_apply_op(dq, dk, cos, sin, pos, ctx.interleaved, not ctx.backward_mode)
  return gq, gk, None, None, None, None, None


rope_apply_op.register_autograd(_rope_backward, setup_context=_rope_setup)


def rope_apply(q: Tensor, k: Tensor, cos: Tensor, sin: Tensor, pos: Tensor | None = None, interleaved: bool = False):
  """``(q*cos + rotate_half(q)*sin, k*cos + rotate_half(k)*sin)`` for (B,H,S,D) q and k in one launch."""
  _lib.require_gpu(q, k, cos, sin, pos)
  return rope_apply_op(q, k, cos, sin, pos, interleaved, False)


# ------------------------------------------------------------------------------------------------
# attention
# ------------------------------------------------------------------------------------------------
_SUPPORTED_HEAD_DIMS = ((64, 64), (128, 128), (192, 128))


def _check_attn(q, k, v, seg):
  if q.dim() != 4 or k.dim() != 4 or v.dim() != 4:
    raise ValueError("attention expects (batch, heads, seq, dim) tensors")
  B, Hq, Sq, Dqk = q.shape
  Bk, Hkv, Skv, Dk = k.shape
  if (Bk, Dk) != (B, Dqk) or v.shape[:3] != k.shape[:3]:
    raise ValueError(f"q {tuple(q.shape)}, k {tuple(k.shape)}, v {tuple(v.shape)} are inconsistent")
  if Hkv == 0 or Hq % Hkv != 0:
    raise ValueError(f"num query heads {Hq} must be a multiple of num kv heads {Hkv}")
  if q.dtype not in (torch.bfloat16, torch.float16) or k.dtype != q.dtype or v.dtype != q.dtype:
    raise TypeError(f"attention kernels take bfloat16 or float16 q/k/v of one dtype, got {q.dtype}/{k.dtype}/{v.dtype}")
  Dv = v.shape[-1]
  if (Dqk, Dv) not in _SUPPORTED_HEAD_DIMS:
    raise NotImplementedError(f"head dims (qk={Dqk}, v={Dv}) not built; supported: {_SUPPORTED_HEAD_DIMS}")
  if seg is not None:
    # kernel_utils.py:238-241: segment ids must cover the whole (unsharded) sequence
    assert seg.shape == (B, Skv) and Sq == Skv, "Sharding along sequence dimension not allowed in tpu kernel attention"
  return B, Hq, Hkv, Sq, Skv, Dqk, Dv


def _prep_heads(t: Tensor) -> Tensor:
  ok = t.stride(-1) == 1 and t.data_ptr() % 16 == 0 and all((s * 2) % 16 == 0 for s in t.stride()[:3])
  return t if ok else t.contiguous()


@torch.library.custom_op("tprime::attn_fwd", mutates_args=(), device_types="cuda")
def attn_fwd(q: Tensor, k: Tensor, v: Tensor, seg: Tensor | None, sm_scale: float, causal: bool) -> tuple[Tensor, Tensor]:
  dev = _lib.require_gpu(q, k, v, seg)
  B, Hq, Hkv, Sq, Skv, Dqk, Dv = _check_attn(q, k, v, seg)
  q, k, v = _prep_heads(q), _prep_heads(k), _prep_heads(v)
  if seg is not None:
    seg = seg.to(torch.int32).contiguous()
  out = _empty_like_heads(q, Dv)
  lse = torch.empty((B, Hq, Sq), dtype=torch.float32, device=dev)
  if out.numel():
    _lib.call(
      "tp_attn_fwd", q.data_ptr(), k.data_ptr(), v.data_ptr(), _lib.ptr(seg), out.data_ptr(), lse.data_ptr(),
      B, Hq, Hkv, Sq, Skv, Dqk, Dv, _lib.strides3(q), _lib.strides3(k), _lib.strides3(v), _lib.strides3(out),
      float(sm_scale), int(causal), _lib.dtype_code(q.dtype), _lib.stream_ptr(dev),
    )  # fmt: skip
  return out, lse


@attn_fwd.register_fake
def _(q, k, v, seg, sm_scale, causal):
  B, Hq, Sq, _ = q.shape
  return _empty_like_heads(q, v.shape[-1]), q.new_empty((B, Hq, Sq), dtype=torch.float32)


@torch.library.custom_op("tprime::attn_bwd", mutates_args=(), device_types="cuda")
def attn_bwd(
  dout: Tensor, q: Tensor, k: Tensor, v: Tensor, out: Tensor, lse: Tensor, seg: Tensor | None, sm_scale: float, causal: bool
) -> tuple[Tensor, Tensor, Tensor]:
  dev = _lib.require_gpu(dout, q, k, v, out, lse, seg)
  B, Hq, Hkv, Sq, Skv, Dqk, Dv = _check_attn(q, k, v, seg)
  q, k, v, out, dout = _prep_heads(q), _prep_heads(k), _prep_heads(v), _prep_heads(out), _prep_heads(dout)
  lse = lse.contiguous()
  if seg is not None:
    seg = seg.to(torch.int32).contiguous()
  dq, dk, dv = _empty_like_heads(q), _empty_like_heads(k), _empty_like_heads(v)
  if dq.numel() == 0 or dk.numel() == 0:
    return dq.zero_(), dk.zero_(), dv.zero_()
  lib = _lib.load()
  ws = torch.empty((lib.tp_attn_bwd_workspace_bytes(B, Hq, Sq) // 4,), dtype=torch.float32, device=dev)
  _lib.call(
    "tp_attn_bwd", dout.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), lse.data_ptr(),
    _lib.ptr(seg), dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), ws.data_ptr(), B, Hq, Hkv, Sq, Skv, Dqk, Dv,
    _lib.strides3(dout), _lib.strides3(q), _lib.strides3(k), _lib.strides3(v), _lib.strides3(out),
    _lib.strides3(dq), _lib.strides3(dk), _lib.strides3(dv), float(sm_scale), int(causal),
    _lib.dtype_code(q.dtype), _lib.stream_ptr(dev),
  )  # fmt: skip
  return dq, dk, dv


@attn_bwd.register_fake
def _(dout, q, k, v, out, lse, seg, sm_scale, causal):
  return _empty_like_heads(q), _empty_like_heads(k), _empty_like_heads(v)


def _attn_setup(ctx, inputs, output):
  q, k, v, seg, sm_scale, causal = inputs
  out, lse = output
  if seg is not None:
    ctx.save_for_backward(q, k, v, out, lse, seg)
  else:
    ctx.save_for_backward(q, k, v, out, lse)
  ctx.has_seg = seg is not None
  ctx.sm_scale = sm_scale
  ctx.causal = causal


def _attn_backward(ctx, dout, _dlse):
  if ctx.has_seg:
    q, k, v, out, lse, seg = ctx.saved_tensors
  else:
    (q, k, v, out, lse), seg = ctx.saved_tensors, None
  dq, dk, dv = attn_bwd(dout, q, k, v, out, lse, seg, ctx.sm_scale, ctx.causal)
  return dq, dk, dv, None, None, None


attn_fwd.register_autograd(_attn_backward, setup_context=_attn_setup)


def attention(
  q: Tensor, k: Tensor, v: Tensor, segment_ids: Tensor | None = None, sm_scale: float | None = None, causal: bool = True
) -> Tensor:
  """Causal / segment-masked GQA attention: q (B,Hq,S,Dqk), k (B,Hkv,S,Dqk), v (B,Hkv,S,Dv) -> (B,Hq,S,Dv).

  ``sm_scale=None`` means ``1/sqrt(v.shape[-1])``, the scale AttentionModule uses
  (torchprime/torch_xla_models/attention.py:54-58, 107, 143, 154)."""
  _lib.require_gpu(q, k, v, segment_ids)
  if sm_scale is None:
    sm_scale = 1.0 / math.sqrt(v.shape[-1])
  return attn_fwd(q, k, v, segment_ids, sm_scale, causal)[0]
