"""ctypes binding of ``libtprime_hip.so`` (the C ABI declared in ``include/tprime_hip.h``).

The library is the only compute path: if it is missing or an entry point reports an error the call
raises; nothing falls back to torch ops.
"""

from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_float, c_int, c_int64, c_size_t, c_void_p

import torch  # noqa: F401  (loads the HIP runtime the library links against)

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libtprime_hip.so")

TP_BF16, TP_F16, TP_F32 = 0, 1, 2
_DTYPE_CODE = {torch.bfloat16: TP_BF16, torch.float16: TP_F16, torch.float32: TP_F32}

_I64x3 = c_int64 * 3

# name -> (restype, argtypes); every symbol the header declares
SIGNATURES = {
  "tp_version": (c_int, []),
  "tp_last_error": (c_char_p, []),
  "tp_rmsnorm_fwd": (
    c_int,
    [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int, c_int64, c_int64, c_float, c_int, c_int, c_void_p],
  ),
  "tp_rmsnorm_bwd_workspace_bytes": (c_size_t, [c_int64, c_int]),
  "tp_rmsnorm_bwd": (
    c_int,
    [c_void_p] * 7 + [c_int64, c_int, c_int64, c_int64, c_int64, c_int, c_int, c_void_p],
  ),
  "tp_rmsnorm_bwd_noalloc": (
    c_int,
    [c_void_p] * 6 + [c_int64, c_int, c_int64, c_int64, c_int64, c_int, c_int, c_void_p],
  ),
  "tp_add_rmsnorm_fwd": (
    c_int,
    [c_void_p] * 6 + [c_int64, c_int, c_int64, c_int64, c_int64, c_int64, c_float, c_int, c_int, c_void_p],
  ),
  "tp_add_rmsnorm_bwd": (
    c_int,
    [c_void_p] * 8 + [c_int64, c_int, c_int64, c_int64, c_int64, c_int64, c_int, c_int, c_void_p],
  ),
  "tp_l2norm_fwd": (c_int, [c_void_p] * 3 + [c_int64, c_int, c_int64, c_int64, c_float, c_int, c_void_p]),
  "tp_l2norm_bwd": (c_int, [c_void_p] * 4 + [c_int64, c_int, c_int64, c_int64, c_int64, c_int, c_void_p]),
  "tp_scale_rows": (c_int, [c_void_p] * 3 + [c_int64, c_int, c_int64, c_int64, c_int, c_int, c_int, c_void_p]),
  "tp_swiglu_fwd": (c_int, [c_void_p] * 3 + [c_int64, c_int, c_int64, c_int64, c_int64, c_int, c_void_p]),
  "tp_swiglu_bwd": (c_int, [c_void_p] * 5 + [c_int64, c_int] + [c_int64] * 5 + [c_int, c_void_p]),
  "tp_cross_entropy_fwd": (c_int, [c_void_p] * 5 + [c_int] * 3 + [c_int64] * 3 + [c_int, c_int, c_void_p]),
  "tp_cross_entropy_bwd": (c_int, [c_void_p] * 6 + [c_int] * 3 + [c_int64] * 5 + [c_int, c_int, c_void_p]),
  "tp_rope_table": (c_int, [c_void_p] * 4 + [c_int, c_int, c_int, c_float, c_int, c_void_p]),
  "tp_rope_apply": (
    c_int,
    [c_void_p] * 7
    + [c_int] * 5
    + [_I64x3] * 4
    + [c_int64, c_int64, c_int64, c_int64, c_int, c_int, c_int, c_void_p],
  ),
  "tp_attn_fwd": (
    c_int,
    [c_void_p] * 6 + [c_int] * 7 + [_I64x3] * 4 + [c_float, c_int, c_int, c_void_p],
  ),
  "tp_attn_fwd_masked": (
    c_int,
    [c_void_p] * 7 + [c_int] * 7 + [_I64x3] * 4 + [c_float, c_int, c_int, c_int, c_int, c_float, c_int, c_void_p],
  ),
  "tp_attn_bwd_masked": (
    c_int,
    [c_void_p] * 12 + [c_int] * 7 + [_I64x3] * 8 + [c_float, c_int, c_int, c_int, c_int, c_float, c_int, c_void_p],
  ),
  "tp_attn_fwd_biased": (
    c_int,
    [c_void_p] * 6 + [_I64x3] + [c_void_p] * 2 + [c_int] * 7 + [_I64x3] * 4
    + [c_float, c_int, c_int, c_int, c_int, c_float, c_int, c_void_p],
  ),
  "tp_attn_bwd_biased": (
    c_int,
    [c_void_p] * 9 + [_I64x3] + [c_void_p] * 4 + [c_int] * 7 + [_I64x3] * 8
    + [c_float, c_int, c_int, c_int, c_int, c_float, c_int, c_void_p],
  ),
  "tp_attn_bwd_workspace_bytes": (c_size_t, [c_int, c_int, c_int]),
  "tp_attn_bwd_dq_first": (c_int, [c_int] * 7),
  "tp_attn_bwd": (
    c_int,
    [c_void_p] * 11 + [c_int] * 7 + [_I64x3] * 8 + [c_float, c_int, c_int, c_void_p],
  ),
  "tp_attn_bwd_ex": (
    c_int,
    [c_void_p] * 11 + [c_int] * 7 + [_I64x3] * 8 + [c_float, c_int, c_int, c_void_p, c_void_p],
  ),
}

_lib = None


class TPrimeError(RuntimeError):
  """An entry point of libtprime_hip.so returned a non-zero status."""


def load() -> ctypes.CDLL:
  """Load the shared library once and set the ctypes prototypes."""
  global _lib
  if _lib is not None:
    return _lib
  if not os.path.exists(LIB_PATH):
    raise ImportError(
      f"{LIB_PATH} is not built. Run `python -c 'import __graft_entry__ as g; g.build()'` "
      "(or `make -C torchprime_amd/csrc`) first; there is no fallback path."
    )
  lib = ctypes.CDLL(LIB_PATH)
  for name, (res, args) in SIGNATURES.items():
    fn = getattr(lib, name)
    fn.restype = res
    fn.argtypes = args
  _lib = lib
  return lib


def dtype_code(dt: torch.dtype) -> int:
  try:
    return _DTYPE_CODE[dt]
  except KeyError:
    raise TypeError(f"unsupported dtype {dt}; supported: bfloat16, float16, float32") from None


def strides3(t: torch.Tensor):
  """(batch, head, seq) element strides of a (B,H,S,D) tensor whose last stride is 1."""
  if t.stride(-1) != 1:
    raise ValueError("innermost stride must be 1")
  return _I64x3(t.stride(0), t.stride(1), t.stride(2))


def ptr(t: torch.Tensor | None):
  return None if t is None else t.data_ptr()


def stream_ptr(device) -> int:
  return torch.cuda.current_stream(device).cuda_stream


def require_gpu(*tensors: torch.Tensor | None) -> torch.device:
  """All tensors must live on one GPU; the kernels have no CPU implementation."""
  dev = None
  for t in tensors:
    if t is None:
      continue
    if not t.is_cuda:
      raise RuntimeError(
        "torchprime_amd ops run on MI355X only: got a tensor on "
        f"'{t.device}'. Move the inputs to the GPU (there is no CPU path)."
      )
    if dev is None:
      dev = t.device
    elif t.device != dev:
      raise RuntimeError(f"tensors on different devices: {dev} and {t.device}")
  return dev


def call(name: str, *args) -> None:
  lib = load()
  rc = getattr(lib, name)(*args)
  if rc != 0:
    msg = lib.tp_last_error().decode("utf-8", "replace")
    exc = {-1: ValueError, -2: NotImplementedError}.get(rc, TPrimeError)
    raise exc(f"{name} failed (status {rc}): {msg}")
