"""``torch.library`` custom ops (namespace ``tprime``) over the HIP kernels in ``libtprime_hip.so``.

Pattern follows the reference's own custom-op precedent, ``xla::offload_name`` in
torchprime/torch_xla_models/offloading.py:14-38 (custom_op + register_fake + register_autograd), so
the ops stay traceable by functorch/AOT autograd as torchprime's remat tooling expects
(torchprime/torch_xla_models/tests/test_remat_all.py:143-202).

Every op is GPU-only: CPU tensors raise, nothing falls back to torch math.
"""

from __future__ import annotations

import math
import weakref

import torch
from torch import Tensor

from . import _lib

__all__ = [
  "rmsnorm",
  "rope_table",
  "rope_apply",
  "attention",
  "add_rmsnorm",
  "l2norm",
  "scale_rows",
  "swiglu",
  "cross_entropy_fwd",
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


# verdicts of the position range check, kept per tensor object (weak reference + version counter, never the address:
# the allocator reuses addresses): a model hands the same position_ids tensor to every layer (and to the backward of
# each), so the device reduction and its host sync run once per tensor, not once per call
_POS_OK: dict = {}


def _check_positions(pos: Tensor, rows: int) -> None:
  """``cos[position_ids]`` raises IndexError for ids outside the table (model/mixtral/model.py:136-137); so does this."""
  ident = id(pos)
  key = (pos._version, tuple(pos.shape), rows)
  entry = _POS_OK.get(ident)
  if entry is not None and entry[0]() is pos and entry[1] == key:
    return
  lo, hi = (int(v) for v in torch.stack((pos.min(), pos.max())).tolist()) if pos.numel() else (0, 0)
  if lo < -rows or hi >= rows:
    raise IndexError(f"position id {hi if hi >= rows else lo} is out of bounds for a rotary table of {rows} rows")
  if lo < 0:
    raise NotImplementedError("negative position ids (indexing the table from its end) are not supported")
  _POS_OK[ident] = (weakref.ref(pos, lambda _r, ident=ident: _POS_OK.pop(ident, None)), key)


def _rope_launch(q, k, cos, sin, pos, interleaved: int, backward: bool):
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
  q: Tensor, k: Tensor, cos: Tensor, sin: Tensor, pos: Tensor | None, interleaved: int, backward: bool
) -> tuple[Tensor, Tensor]:
  """``interleaved``: 0 rotate-half, 1 DeepSeek ([evens | odds] output), 2 adjacent pairs in place (Llama-4)."""
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


def rope_apply(q: Tensor, k: Tensor, cos: Tensor, sin: Tensor, pos: Tensor | None = None, interleaved: int = 0):
  """``(q*cos + rotate_half(q)*sin, k*cos + rotate_half(k)*sin)`` for (B,H,S,D) q and k in one launch."""
  _lib.require_gpu(q, k, cos, sin, pos)
  return rope_apply_op(q, k, cos, sin, pos, int(interleaved), False)


# ------------------------------------------------------------------------------------------------
# attention
# ------------------------------------------------------------------------------------------------
_SUPPORTED_HEAD_DIMS = ((64, 64), (128, 128), (192, 128))
_SUPPORTED_HEAD_DIMS_F32 = ((64, 64), (128, 128))  # fp32 operands (the small fp32 configurations)


def _check_attn(q, k, v, seg):
  if q.dim() != 4 or k.dim() != 4 or v.dim() != 4:
    raise ValueError("attention expects (batch, heads, seq, dim) tensors")
  B, Hq, Sq, Dqk = q.shape
  Bk, Hkv, Skv, Dk = k.shape
  if (Bk, Dk) != (B, Dqk) or v.shape[:3] != k.shape[:3]:
    raise ValueError(f"q {tuple(q.shape)}, k {tuple(k.shape)}, v {tuple(v.shape)} are inconsistent")
  if Hkv == 0 or Hq % Hkv != 0:
    raise ValueError(f"num query heads {Hq} must be a multiple of num kv heads {Hkv}")
  if q.dtype not in (torch.bfloat16, torch.float16, torch.float32) or k.dtype != q.dtype or v.dtype != q.dtype:
    raise TypeError(f"attention kernels take bfloat16, float16 or float32 q/k/v of one dtype, got {q.dtype}/{k.dtype}/{v.dtype}")
  Dv = v.shape[-1]
  dims = _SUPPORTED_HEAD_DIMS_F32 if q.dtype == torch.float32 else _SUPPORTED_HEAD_DIMS
  if (Dqk, Dv) not in dims:
    raise NotImplementedError(f"head dims (qk={Dqk}, v={Dv}) not built for {q.dtype}; supported: {dims}")
  if seg is not None:
    # kernel_utils.py:238-241: segment ids must cover the whole (unsharded) sequence
    assert seg.shape == (B, Skv) and Sq == Skv, "Sharding along sequence dimension not allowed in tpu kernel attention"
  return B, Hq, Hkv, Sq, Skv, Dqk, Dv


def _prep_heads(t: Tensor) -> Tensor:
  esz = t.element_size()
  ok = t.stride(-1) == 1 and t.data_ptr() % 16 == 0 and all((s * esz) % 16 == 0 for s in t.stride()[:3])
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


# ---- mask extensions: sliding window, soft cap, query rows in another order than the keys -------------------
def _prep_qpos(qpos: Tensor | None, Sq: int) -> Tensor | None:
  if qpos is None:
    return None
  if qpos.shape != (Sq,):
    raise ValueError(f"q_positions must have shape ({Sq},), got {tuple(qpos.shape)}")
  return qpos.to(torch.int32).contiguous()


def _prep_bias(bias: Tensor | None, B: int, Hq: int, Sq: int, Skv: int):
  """(fp32 tensor with a contiguous key axis, its (batch, head, query) strides with 0 on broadcast axes)."""
  if bias is None:
    return None, None
  if bias.dim() != 4 or bias.shape[0] not in (1, B) or bias.shape[1] not in (1, Hq) or bias.shape[2:] != (Sq, Skv):
    raise ValueError(f"mask must have shape (1|{B}, 1|{Hq}, {Sq}, {Skv}), got {tuple(bias.shape)}")
  bias = bias.float()
  if bias.stride(-1) != 1:
    bias = bias.contiguous()
  strides = _lib._I64x3(
    0 if bias.shape[0] == 1 else bias.stride(0), 0 if bias.shape[1] == 1 else bias.stride(1), bias.stride(2)
  )
  return bias, strides


@torch.library.custom_op("tprime::attn_fwd_masked", mutates_args=(), device_types="cuda")
def attn_fwd_masked(
  q: Tensor, k: Tensor, v: Tensor, seg: Tensor | None, qpos: Tensor | None, sm_scale: float, causal: bool,
  causal_offset: int, window_left: int, window_right: int, soft_cap: float, bias: Tensor | None = None,
) -> tuple[Tensor, Tensor]:  # fmt: skip
  dev = _lib.require_gpu(q, k, v, seg, qpos, bias)
  B, Hq, Hkv, Sq, Skv, Dqk, Dv = _check_attn(q, k, v, seg)
  q, k, v = _prep_heads(q), _prep_heads(k), _prep_heads(v)
  if seg is not None:
    seg = seg.to(torch.int32).contiguous()
  qpos = _prep_qpos(qpos, Sq)
  out = _empty_like_heads(q, Dv)
  lse = torch.empty((B, Hq, Sq), dtype=torch.float32, device=dev)
  bias, bias_strides = _prep_bias(bias, B, Hq, Sq, Skv)
  if out.numel():
    tail = (
      B, Hq, Hkv, Sq, Skv, Dqk, Dv, _lib.strides3(q), _lib.strides3(k), _lib.strides3(v), _lib.strides3(out),
      float(sm_scale), int(causal), int(causal_offset), int(window_left), int(window_right), float(soft_cap),
      _lib.dtype_code(q.dtype), _lib.stream_ptr(dev),
    )  # fmt: skip
    head = (q.data_ptr(), k.data_ptr(), v.data_ptr(), _lib.ptr(seg), _lib.ptr(qpos))
    if bias is None:
      _lib.call("tp_attn_fwd_masked", *head, out.data_ptr(), lse.data_ptr(), *tail)
    else:
      _lib.call("tp_attn_fwd_biased", *head, bias.data_ptr(), bias_strides, out.data_ptr(), lse.data_ptr(), *tail)
  return out, lse


@attn_fwd_masked.register_fake
def _(q, k, v, seg, qpos, sm_scale, causal, causal_offset, window_left, window_right, soft_cap, bias=None):
  B, Hq, Sq, _ = q.shape
  return _empty_like_heads(q, v.shape[-1]), q.new_empty((B, Hq, Sq), dtype=torch.float32)


@torch.library.custom_op("tprime::attn_bwd_masked", mutates_args=(), device_types="cuda")
def attn_bwd_masked(
  dout: Tensor, q: Tensor, k: Tensor, v: Tensor, out: Tensor, lse: Tensor, seg: Tensor | None, qpos: Tensor | None,
  sm_scale: float, causal: bool, causal_offset: int, window_left: int, window_right: int, soft_cap: float,
  bias: Tensor | None = None,
) -> tuple[Tensor, Tensor, Tensor]:  # fmt: skip
  dev = _lib.require_gpu(dout, q, k, v, out, lse, seg, qpos, bias)
  B, Hq, Hkv, Sq, Skv, Dqk, Dv = _check_attn(q, k, v, seg)
  q, k, v, out, dout = _prep_heads(q), _prep_heads(k), _prep_heads(v), _prep_heads(out), _prep_heads(dout)
  lse = lse.contiguous()
  if seg is not None:
    seg = seg.to(torch.int32).contiguous()
  qpos = _prep_qpos(qpos, Sq)
  dq, dk, dv = _empty_like_heads(q), _empty_like_heads(k), _empty_like_heads(v)
  if dq.numel() == 0 or dk.numel() == 0:
    return dq.zero_(), dk.zero_(), dv.zero_()
  lib = _lib.load()
  ws = torch.empty((lib.tp_attn_bwd_workspace_bytes(B, Hq, Sq) // 4,), dtype=torch.float32, device=dev)
  bias, bias_strides = _prep_bias(bias, B, Hq, Sq, Skv)
  head = (
    dout.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), lse.data_ptr(), _lib.ptr(seg), _lib.ptr(qpos),
  )  # fmt: skip
  tail = (
    dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), ws.data_ptr(), B, Hq, Hkv, Sq, Skv,
    Dqk, Dv, _lib.strides3(dout), _lib.strides3(q), _lib.strides3(k), _lib.strides3(v), _lib.strides3(out),
    _lib.strides3(dq), _lib.strides3(dk), _lib.strides3(dv), float(sm_scale), int(causal), int(causal_offset),
    int(window_left), int(window_right), float(soft_cap), _lib.dtype_code(q.dtype), _lib.stream_ptr(dev),
  )  # fmt: skip
  if bias is None:
    _lib.call("tp_attn_bwd_masked", *head, *tail)
  else:
    _lib.call("tp_attn_bwd_biased", *head, bias.data_ptr(), bias_strides, *tail)
  return dq, dk, dv


@attn_bwd_masked.register_fake
def _(dout, q, k, v, out, lse, seg, qpos, sm_scale, causal, causal_offset, window_left, window_right, soft_cap, bias=None):
  return _empty_like_heads(q), _empty_like_heads(k), _empty_like_heads(v)


def _attn_masked_setup(ctx, inputs, output):
  q, k, v, seg, qpos, sm_scale, causal, causal_offset, window_left, window_right, soft_cap, bias = inputs
  out, lse = output
  ctx.save_for_backward(*(t for t in (q, k, v, out, lse, seg, qpos, bias) if t is not None))
  ctx.has_seg, ctx.has_qpos, ctx.has_bias = seg is not None, qpos is not None, bias is not None
  ctx.scalars = (sm_scale, causal, causal_offset, window_left, window_right, soft_cap)


def _attn_masked_backward(ctx, dout, _dlse):
  saved = list(ctx.saved_tensors)
  q, k, v, out, lse = saved[:5]
  rest = saved[5:]
  seg = rest.pop(0) if ctx.has_seg else None
  qpos = rest.pop(0) if ctx.has_qpos else None
  bias = rest.pop(0) if ctx.has_bias else None
  dq, dk, dv = attn_bwd_masked(dout, q, k, v, out, lse, seg, qpos, *ctx.scalars, bias)
  return (dq, dk, dv) + (None,) * 9


attn_fwd_masked.register_autograd(_attn_masked_backward, setup_context=_attn_masked_setup)


def attention(
  q: Tensor, k: Tensor, v: Tensor, segment_ids: Tensor | None = None, sm_scale: float | None = None, causal: bool = True,
  *, window: tuple[int | None, int | None] | None = None, soft_cap: float | None = None,
  q_positions: Tensor | None = None, causal_offset: int = 0, bias: Tensor | None = None,
) -> Tensor:  # fmt: skip
  """Causal / segment-masked GQA attention: q (B,Hq,S,Dqk), k (B,Hkv,S,Dqk), v (B,Hkv,S,Dv) -> (B,Hq,S,Dv).

  ``sm_scale=None`` means ``1/sqrt(v.shape[-1])``, the scale AttentionModule uses
  (torchprime/torch_xla_models/attention.py:54-58, 107, 143, 154).

  ``window=(left, right)``: key j only if ``pos - left <= j <= pos + right`` (None: unbounded; LocalMask,
  kernel_utils.py:266-275).  ``soft_cap``: logits become ``cap * tanh(logits / cap)`` (kernel_utils.py:292).
  ``q_positions`` (Sq) int: query row i stands for position ``q_positions[i]`` of the key order
  (LoadBalancedCausalMask.q_sequence, parallelism_utils.py:109-132); ``causal_offset``: that mask's ``offset``.
  ``bias`` (1|B, 1|Hq, Sq, Skv): added to the scaled logits before the softmax, the eager branch's additive mask
  (torchprime/torch_xla_models/attention.py:151-158); it is a constant (no gradient), -inf forbids a pair, and a
  query row whose every key is forbidden gives zeros where the reference's softmax gives NaN."""
  if soft_cap is not None and soft_cap <= 0:
    raise ValueError(f"soft_cap must be positive, got {soft_cap}")
  _lib.require_gpu(q, k, v, segment_ids, q_positions, bias)
  if sm_scale is None:
    sm_scale = 1.0 / math.sqrt(v.shape[-1])
  wl, wr = (-1, -1) if window is None else tuple(-1 if w is None else int(w) for w in window)
  if bias is None and q_positions is None and wl < 0 and wr < 0 and soft_cap is None and (causal_offset == 0 or not causal):
    return attn_fwd(q, k, v, segment_ids, sm_scale, causal)[0]
  if bias is not None:
    bias = bias.detach()
  return attn_fwd_masked(
    q, k, v, segment_ids, q_positions, sm_scale, causal, causal_offset, wl, wr, float(soft_cap or 0.0), bias
  )[0]


# ------------------------------------------------------------------------------------------------
# the steps either side of the attention path: residual add + RMSNorm, L2 norm, temperature scale,
# SwiGLU, cross entropy
# ------------------------------------------------------------------------------------------------
@torch.library.custom_op("tprime::add_rmsnorm_fwd", mutates_args=(), device_types="cuda")
def add_rmsnorm_fwd(x: Tensor, residual: Tensor, weight: Tensor, eps: float) -> tuple[Tensor, Tensor, Tensor]:
  """(y, h, rstd): h = residual + x, y = RMSNorm(h) * weight, in one pass."""
  _lib.require_gpu(x, residual, weight)
  hidden = x.shape[-1]
  if residual.shape != x.shape or residual.dtype != x.dtype:
    raise ValueError(f"residual {tuple(residual.shape)}/{residual.dtype} must match x {tuple(x.shape)}/{x.dtype}")
  if weight.shape != (hidden,):
    raise ValueError(f"weight shape {tuple(weight.shape)} does not match hidden size {hidden}")
  x2, r2, w = _rows(x), _rows(residual), weight.contiguous()
  rows = x2.shape[0]
  out_dtype = torch.result_type(weight, x)
  y = torch.empty((rows, hidden), dtype=out_dtype, device=x.device)
  h = torch.empty((rows, hidden), dtype=x.dtype, device=x.device)
  rstd = torch.empty((rows,), dtype=torch.float32, device=x.device)
  if rows:
    _lib.call(
      "tp_add_rmsnorm_fwd", x2.data_ptr(), r2.data_ptr(), w.data_ptr(), h.data_ptr(), y.data_ptr(), rstd.data_ptr(),
      rows, hidden, x2.stride(0) if rows > 1 else hidden, r2.stride(0) if rows > 1 else hidden, hidden, hidden,
      float(eps), _lib.dtype_code(x.dtype), _lib.dtype_code(w.dtype), _lib.stream_ptr(x.device),
    )  # fmt: skip
  return y.view(*x.shape[:-1], hidden), h.view(x.shape), rstd


@add_rmsnorm_fwd.register_fake
def _(x, residual, weight, eps):
  rows = x.numel() // max(x.shape[-1], 1)
  return (x.new_empty(x.shape, dtype=torch.result_type(weight, x)), torch.empty_like(x, memory_format=torch.contiguous_format),
          x.new_empty((rows,), dtype=torch.float32))


@torch.library.custom_op("tprime::add_rmsnorm_bwd", mutates_args=(), device_types="cuda")
def add_rmsnorm_bwd(dy: Tensor, dh: Tensor, h: Tensor, weight: Tensor, rstd: Tensor) -> tuple[Tensor, Tensor]:
  _lib.require_gpu(dy, dh, h, weight, rstd)
  hidden = h.shape[-1]
  h2, g2, d2, w = _rows(h), _rows(dy), _rows(dh), weight.contiguous()
  rows = h2.shape[0]
  dx = torch.empty((rows, hidden), dtype=h.dtype, device=h.device)
  dw = torch.empty((hidden,), dtype=w.dtype, device=h.device)
  if rows == 0:
    return dx.view(h.shape), dw.zero_()
  lib = _lib.load()
  ws = torch.empty((lib.tp_rmsnorm_bwd_workspace_bytes(rows, hidden) // 4,), dtype=torch.float32, device=h.device)
  st = lambda t: t.stride(0) if rows > 1 else hidden  # noqa: E731
  _lib.call(
    "tp_add_rmsnorm_bwd", g2.data_ptr(), d2.data_ptr(), h2.data_ptr(), w.data_ptr(), rstd.data_ptr(), dx.data_ptr(),
    dw.data_ptr(), ws.data_ptr(), rows, hidden, st(g2), st(d2), st(h2), hidden, _lib.dtype_code(h.dtype),
    _lib.dtype_code(w.dtype), _lib.stream_ptr(h.device),
  )  # fmt: skip
  return dx.view(h.shape), dw


@add_rmsnorm_bwd.register_fake
def _(dy, dh, h, weight, rstd):
  return torch.empty_like(h, memory_format=torch.contiguous_format), torch.empty_like(weight)


def _add_rmsnorm_setup(ctx, inputs, output):
  _x, _res, weight, _eps = inputs
  _y, h, rstd = output
  ctx.save_for_backward(h, weight, rstd)


def _add_rmsnorm_backward(ctx, dy, dh, _drstd):
  h, weight, rstd = ctx.saved_tensors
  out_dtype = torch.result_type(weight, h)
  if dy is None:
    dy = torch.zeros_like(h, dtype=out_dtype)
  if dh is None:
    dx, dw = rmsnorm_bwd(dy.to(out_dtype), h, weight, rstd)
  else:
    dx, dw = add_rmsnorm_bwd(dy.to(out_dtype), dh.to(h.dtype), h, weight, rstd)
  return dx, dx, dw, None


add_rmsnorm_fwd.register_autograd(_add_rmsnorm_backward, setup_context=_add_rmsnorm_setup)


def add_rmsnorm(x: Tensor, residual: Tensor, weight: Tensor, eps: float) -> tuple[Tensor, Tensor]:
  """``h = residual + x; y = rms_norm(h, weight, eps)`` in one pass; returns ``(y, h)``."""
  y, h, _ = add_rmsnorm_fwd(x, residual, weight, eps)
  return y, h


def _head_rows(x: Tensor) -> Tensor:
  d = x.shape[-1]
  x2 = x.reshape(-1, d)
  if x2.stride(-1) != 1 or (x2.stride(0) * x2.element_size()) % 16 or x2.data_ptr() % 16:
    x2 = x2.contiguous()
  return x2


@torch.library.custom_op("tprime::l2norm_fwd", mutates_args=(), device_types="cuda")
def l2norm_fwd(x: Tensor, eps: float) -> tuple[Tensor, Tensor]:
  _lib.require_gpu(x)
  x2 = _head_rows(x)
  rows, dim = x2.shape
  y = torch.empty((rows, dim), dtype=x.dtype, device=x.device)
  rstd = torch.empty((rows,), dtype=torch.float32, device=x.device)
  if rows:
    _lib.call("tp_l2norm_fwd", x2.data_ptr(), y.data_ptr(), rstd.data_ptr(), rows, dim, x2.stride(0) if rows > 1 else dim, dim,
              float(eps), _lib.dtype_code(x.dtype), _lib.stream_ptr(x.device))  # fmt: skip
  return y.view(x.shape), rstd


@l2norm_fwd.register_fake
def _(x, eps):
  return torch.empty_like(x, memory_format=torch.contiguous_format), x.new_empty((x.numel() // max(x.shape[-1], 1),), dtype=torch.float32)


@torch.library.custom_op("tprime::l2norm_bwd", mutates_args=(), device_types="cuda")
def l2norm_bwd(dy: Tensor, x: Tensor, rstd: Tensor) -> Tensor:
  _lib.require_gpu(dy, x, rstd)
  x2, g2 = _head_rows(x), _head_rows(dy)
  rows, dim = x2.shape
  dx = torch.empty((rows, dim), dtype=x.dtype, device=x.device)
  if rows:
    st = lambda t: t.stride(0) if rows > 1 else dim  # noqa: E731
    _lib.call("tp_l2norm_bwd", g2.data_ptr(), x2.data_ptr(), rstd.data_ptr(), dx.data_ptr(), rows, dim, st(g2), st(x2), dim,
              _lib.dtype_code(x.dtype), _lib.stream_ptr(x.device))  # fmt: skip
  return dx.view(x.shape)


@l2norm_bwd.register_fake
def _(dy, x, rstd):
  return torch.empty_like(x, memory_format=torch.contiguous_format)


def _l2norm_setup(ctx, inputs, output):
  ctx.save_for_backward(inputs[0], output[1])


def _l2norm_backward(ctx, dy, _drstd):
  x, rstd = ctx.saved_tensors
  return l2norm_bwd(dy.to(x.dtype), x, rstd), None


l2norm_fwd.register_autograd(_l2norm_backward, setup_context=_l2norm_setup)


def l2norm(x: Tensor, eps: float) -> Tensor:
  """``(x.float() * rsqrt(mean(x.float()**2, -1) + eps)).type_as(x)`` over the last dim."""
  return l2norm_fwd(x, eps)[0]


@torch.library.custom_op("tprime::scale_rows", mutates_args=(), device_types="cuda")
def scale_rows(x: Tensor, scale: Tensor) -> Tensor:
  """x (B, S, N, D) times scale (S) fp32 per position, rounded to x's dtype."""
  _lib.require_gpu(x, scale)
  if x.dim() != 4 or scale.shape != (x.shape[1],):
    raise ValueError(f"expected x (batch, seq, heads, dim) and scale (seq,), got {tuple(x.shape)} and {tuple(scale.shape)}")
  B, S, N, D = x.shape
  x2 = _head_rows(x)
  y = torch.empty((B * S * N, D), dtype=x.dtype, device=x.device)
  if y.numel():
    _lib.call("tp_scale_rows", x2.data_ptr(), scale.to(torch.float32).contiguous().data_ptr(), y.data_ptr(), B * S * N, D,
              x2.stride(0) if B * S * N > 1 else D, D, N, S, _lib.dtype_code(x.dtype), _lib.stream_ptr(x.device))  # fmt: skip
  return y.view(x.shape)


@scale_rows.register_fake
def _(x, scale):
  return torch.empty_like(x, memory_format=torch.contiguous_format)


def _scale_rows_setup(ctx, inputs, output):
  ctx.save_for_backward(inputs[1])


def _scale_rows_backward(ctx, dy):
  (scale,) = ctx.saved_tensors
  return scale_rows(dy, scale), None


scale_rows.register_autograd(_scale_rows_backward, setup_context=_scale_rows_setup)


@torch.library.custom_op("tprime::swiglu_fwd", mutates_args=(), device_types="cuda")
def swiglu_fwd(gate: Tensor, up: Tensor) -> Tensor:
  _lib.require_gpu(gate, up)
  if gate.shape != up.shape or gate.dtype != up.dtype:
    raise ValueError(f"gate {tuple(gate.shape)}/{gate.dtype} and up {tuple(up.shape)}/{up.dtype} must match")
  g2, u2 = _head_rows(gate), _head_rows(up)
  rows, cols = g2.shape
  out = torch.empty((rows, cols), dtype=gate.dtype, device=gate.device)
  if out.numel():
    st = lambda t: t.stride(0) if rows > 1 else cols  # noqa: E731
    _lib.call("tp_swiglu_fwd", g2.data_ptr(), u2.data_ptr(), out.data_ptr(), rows, cols, st(g2), st(u2), cols,
              _lib.dtype_code(gate.dtype), _lib.stream_ptr(gate.device))  # fmt: skip
  return out.view(gate.shape)


@swiglu_fwd.register_fake
def _(gate, up):
  return torch.empty_like(gate, memory_format=torch.contiguous_format)


@torch.library.custom_op("tprime::swiglu_bwd", mutates_args=(), device_types="cuda")
def swiglu_bwd(dout: Tensor, gate: Tensor, up: Tensor) -> tuple[Tensor, Tensor]:
  _lib.require_gpu(dout, gate, up)
  d2, g2, u2 = _head_rows(dout), _head_rows(gate), _head_rows(up)
  rows, cols = g2.shape
  dg = torch.empty((rows, cols), dtype=gate.dtype, device=gate.device)
  du = torch.empty_like(dg)
  if dg.numel():
    st = lambda t: t.stride(0) if rows > 1 else cols  # noqa: E731
    _lib.call("tp_swiglu_bwd", d2.data_ptr(), g2.data_ptr(), u2.data_ptr(), dg.data_ptr(), du.data_ptr(), rows, cols, st(d2),
              st(g2), st(u2), cols, cols, _lib.dtype_code(gate.dtype), _lib.stream_ptr(gate.device))  # fmt: skip
  return dg.view(gate.shape), du.view(gate.shape)


@swiglu_bwd.register_fake
def _(dout, gate, up):
  return torch.empty_like(gate, memory_format=torch.contiguous_format), torch.empty_like(up, memory_format=torch.contiguous_format)


def _swiglu_setup(ctx, inputs, output):
  ctx.save_for_backward(*inputs)


def _swiglu_backward(ctx, dout):
  gate, up = ctx.saved_tensors
  return swiglu_bwd(dout.to(gate.dtype), gate, up)


swiglu_fwd.register_autograd(_swiglu_backward, setup_context=_swiglu_setup)


def swiglu(gate: Tensor, up: Tensor) -> Tensor:
  """``silu(gate) * up`` with the eager roundings, one pass."""
  return swiglu_fwd(gate, up)


@torch.library.custom_op("tprime::cross_entropy_fwd", mutates_args=(), device_types="cuda")
def cross_entropy_fwd(logits: Tensor, labels: Tensor, ignore_index: int) -> tuple[Tensor, Tensor, Tensor]:
  """(loss (scalar fp32), lse (B*S), loss_and_count (2)) of the shifted next-token cross entropy."""
  _lib.require_gpu(logits, labels)
  if logits.dim() != 3 or labels.shape != logits.shape[:2]:
    raise ValueError(f"expected logits (batch, seq, vocab) and labels (batch, seq), got {tuple(logits.shape)} and {tuple(labels.shape)}")
  if logits.dtype not in (torch.float32, torch.bfloat16):
    raise TypeError(f"cross entropy takes float32 or bfloat16 logits, got {logits.dtype}")
  B, S, V = logits.shape
  if logits.stride(2) != 1:
    logits = logits.contiguous()
  labels = labels.to(torch.int64)
  if labels.stride(1) != 1:
    labels = labels.contiguous()
  lse = torch.empty((B * S,), dtype=torch.float32, device=logits.device)
  row_loss = torch.empty_like(lse)
  lc = torch.empty((2,), dtype=torch.float32, device=logits.device)
  _lib.call("tp_cross_entropy_fwd", logits.data_ptr(), labels.data_ptr(), lse.data_ptr(), row_loss.data_ptr(), lc.data_ptr(),
            B, S, V, logits.stride(0), logits.stride(1), labels.stride(0), int(ignore_index), _lib.dtype_code(logits.dtype),
            _lib.stream_ptr(logits.device))  # fmt: skip
  return lc[0].clone(), lse, lc


@cross_entropy_fwd.register_fake
def _(logits, labels, ignore_index):
  B, S, _ = logits.shape
  return logits.new_empty((), dtype=torch.float32), logits.new_empty((B * S,), dtype=torch.float32), logits.new_empty((2,), dtype=torch.float32)


@torch.library.custom_op("tprime::cross_entropy_bwd", mutates_args=(), device_types="cuda")
def cross_entropy_bwd(dloss: Tensor, logits: Tensor, labels: Tensor, lse: Tensor, loss_and_count: Tensor, ignore_index: int) -> Tensor:
  _lib.require_gpu(dloss, logits, labels, lse, loss_and_count)
  B, S, V = logits.shape
  if logits.stride(2) != 1:
    logits = logits.contiguous()
  labels = labels.to(torch.int64)
  if labels.stride(1) != 1:
    labels = labels.contiguous()
  dlogits = torch.empty((B, S, V), dtype=logits.dtype, device=logits.device)
  _lib.call("tp_cross_entropy_bwd", logits.data_ptr(), labels.data_ptr(), lse.data_ptr(), loss_and_count.data_ptr(),
            dloss.to(torch.float32).reshape(1).contiguous().data_ptr(), dlogits.data_ptr(), B, S, V, logits.stride(0),
            logits.stride(1), labels.stride(0), dlogits.stride(0), dlogits.stride(1), int(ignore_index),
            _lib.dtype_code(logits.dtype), _lib.stream_ptr(logits.device))  # fmt: skip
  return dlogits


@cross_entropy_bwd.register_fake
def _(dloss, logits, labels, lse, loss_and_count, ignore_index):
  return torch.empty_like(logits, memory_format=torch.contiguous_format)


def _xent_setup(ctx, inputs, output):
  logits, labels, ignore_index = inputs
  _loss, lse, lc = output
  ctx.save_for_backward(logits, labels, lse, lc)
  ctx.ignore_index = ignore_index


def _xent_backward(ctx, dloss, _dlse, _dlc):
  logits, labels, lse, lc = ctx.saved_tensors
  return cross_entropy_bwd(dloss, logits, labels, lse, lc, ctx.ignore_index), None, None


cross_entropy_fwd.register_autograd(_xent_backward, setup_context=_xent_setup)
