"""The allocation-free RMSNorm backward entry point (tp_rmsnorm_bwd_noalloc: partial-dw rows in an array built
into the library) against tp_rmsnorm_bwd with a caller-provided workspace, through the C ABI: identical bits, on
two calls in a row, the second on a smaller input (the array keeps the first call's contents)."""

import pytest
import torch

from tests.util import randn
from torchprime_amd import _lib

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _inputs(rows, hidden, dtype, seed):
  x = randn((rows, hidden), seed, dtype).to(DEV)
  dy = randn((rows, hidden), seed + 1, dtype).to(DEV)
  w = (1 + randn((hidden,), seed + 2, torch.float32, 0.1)).to(dtype).to(DEV)
  rstd = torch.rsqrt(x.float().pow(2).mean(-1) + 1e-5).contiguous()
  return x, dy, w, rstd


def _both(rows, hidden, dtype, seed):
  lib = _lib.load()
  x, dy, w, rstd = _inputs(rows, hidden, dtype, seed)
  code, st = _lib.dtype_code(dtype), _lib.stream_ptr(torch.device(DEV))
  dx_a, dw_a = torch.empty_like(x), torch.empty_like(w)
  ws = torch.empty((lib.tp_rmsnorm_bwd_workspace_bytes(rows, hidden) // 4,), dtype=torch.float32, device=DEV)
  _lib.call("tp_rmsnorm_bwd", dy.data_ptr(), x.data_ptr(), w.data_ptr(), rstd.data_ptr(), dx_a.data_ptr(), dw_a.data_ptr(),
            ws.data_ptr(), rows, hidden, hidden, hidden, hidden, code, code, st)  # fmt: skip
  dx_b, dw_b = torch.full_like(x, float("nan")), torch.full_like(w, float("nan"))
  torch.cuda.synchronize()
  before = torch.cuda.memory_allocated()
  _lib.call("tp_rmsnorm_bwd_noalloc", dy.data_ptr(), x.data_ptr(), w.data_ptr(), rstd.data_ptr(), dx_b.data_ptr(),
            dw_b.data_ptr(), rows, hidden, hidden, hidden, hidden, code, code, st)  # fmt: skip
  torch.cuda.synchronize()
  assert torch.cuda.memory_allocated() == before
  assert torch.equal(dx_a, dx_b), "dx differs from tp_rmsnorm_bwd"
  assert torch.equal(dw_a, dw_b), "dw differs from tp_rmsnorm_bwd"
  assert torch.isfinite(dw_b.float()).all()


def test_noalloc_matches_workspace_entry_point_twice_second_call_smaller():
  _both(4096, 4096, torch.bfloat16, 1)   # 512 partial rows of 4096 floats
  _both(300, 1536, torch.bfloat16, 5)    # fewer rows, narrower: stale partial rows beyond its own must not leak in
  _both(7, 333, torch.float16, 9)        # ragged hidden: the scalar kernels use the array too
  _both(3000, 8192, torch.float32, 11)   # the widest shape the array holds


def test_noalloc_rejects_shapes_beyond_the_array():
  x, dy, w, rstd = _inputs(2048, 8200, torch.bfloat16, 3)
  dx, dw = torch.empty_like(x), torch.empty_like(w)
  code, st = _lib.dtype_code(torch.bfloat16), _lib.stream_ptr(torch.device(DEV))
  with pytest.raises(NotImplementedError, match="built-in array"):
    _lib.call("tp_rmsnorm_bwd_noalloc", dy.data_ptr(), x.data_ptr(), w.data_ptr(), rstd.data_ptr(), dx.data_ptr(),
              dw.data_ptr(), 2048, 8200, 8200, 8200, 8200, code, code, st)  # fmt: skip
