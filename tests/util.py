"""Shared helpers for the parity tests."""

import json
import os

import torch

# tolerance for 16-bit outputs and gradients against the fp32 oracle
MAX_ABS = 2e-2
REL_L2 = 1e-2


def errors(got: torch.Tensor, ref: torch.Tensor):
  got, ref = got.detach().double().cpu(), ref.detach().double().cpu()
  diff = got - ref
  max_abs = diff.abs().max().item() if diff.numel() else 0.0
  # an all-zero reference (e.g. dq of a one-token softmax) has no relative error; the abs bound covers it
  rel_l2 = (diff.norm() / ref.norm()).item() if diff.numel() and ref.norm().item() > 1e-12 else 0.0
  return max_abs, rel_l2


# one bf16 ulp is 2^-8 of the value's binade, i.e. up to 2^-7 of the value itself
ULP_SLACK = 2.0**-7


def _log(name, ma, rl, ref_inf, worst):
  """Measured errors go to the JSON-lines file named by TP_PARITY_LOG (one record per comparison)."""
  path = os.environ.get("TP_PARITY_LOG")
  if not path:
    return
  test = os.environ.get("PYTEST_CURRENT_TEST", "").split(" ")[0]
  with open(path, "a") as f:
    f.write(json.dumps({"test": test, "name": name, "max_abs": ma, "rel_l2": rl, "ref_inf": ref_inf, "worst_excess": worst}) + "\n")


def assert_close(got, ref, name="", max_abs=MAX_ABS, rel_l2=REL_L2, scale_abs=False):
  """Relative-L2 over the tensor plus a max-abs bound on every element.

  ``scale_abs=False``: ``|got - ref| <= max_abs`` everywhere.
  ``scale_abs=True`` (tensors whose values leave the range where a 16-bit result can be 2e-2 accurate: one
  bf16 rounding of a value in [4, 8) is already up to 1.6e-2 off): element-wise
  ``|got - ref| <= max_abs + 2^-7 |ref|``, i.e. the stated bound where the value is small and one bf16 ulp of
  slack where it is large.  The slack follows each element's own magnitude, not the tensor's largest value."""
  assert got.shape == ref.shape, f"{name}: shape {tuple(got.shape)} vs {tuple(ref.shape)}"
  assert torch.isfinite(got.float()).all(), f"{name}: non-finite values in the result"
  ma, rl = errors(got, ref)
  g, r = got.detach().double().cpu(), ref.detach().double().cpu()
  bound = torch.full_like(r, max_abs) + (ULP_SLACK * r.abs() if scale_abs else 0.0)
  excess = ((g - r).abs() - bound)
  worst = excess.max().item() if excess.numel() else -max_abs
  _log(name, ma, rl, r.abs().max().item() if r.numel() else 0.0, worst)
  assert worst <= 0.0 and rl <= rel_l2, (
    f"{name}: max-abs {ma:.3e}, worst element exceeds its bound ({max_abs}{' + 2^-7|ref|' if scale_abs else ''}) by "
    f"{worst:.3e}; rel-L2 {rl:.3e} (limit {rel_l2})"
  )
  return ma, rl


def randn(shape, seed, dtype=torch.float32, std=1.0):
  g = torch.Generator(device="cpu").manual_seed(seed)
  return (torch.randn(shape, generator=g, dtype=torch.float32) * std).to(dtype)


def heads_view(B, H, S, D, seed, dtype, std=1.0):
  """(B,H,S,D) view of (B,S,H,D) memory, the layout the attention modules produce."""
  return randn((B, S, H, D), seed, dtype, std).transpose(1, 2)


def packed_segment_ids(B, S, lo, hi, seed):
  """Rows packed with documents of uniform-random lengths lo..hi summing to S; ids 0,1,2,... per row."""
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
