"""Shared helpers for the parity tests."""

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


def assert_close(got, ref, name="", max_abs=MAX_ABS, rel_l2=REL_L2, scale_abs=False):
  """``scale_abs``: apply the max-abs bound relative to the tensor's scale, max_abs * max(1, |ref|_inf).
  Needed where values exceed ~2.5 in magnitude: a single bf16 rounding of a value in [4, 8) is already
  up to 1.6e-2 off, so an absolute 2e-2 cannot hold for any bf16 result there, the reference's included."""
  assert got.shape == ref.shape, f"{name}: shape {tuple(got.shape)} vs {tuple(ref.shape)}"
  assert torch.isfinite(got.float()).all(), f"{name}: non-finite values in the result"
  ma, rl = errors(got, ref)
  if scale_abs and ref.numel():
    max_abs = max_abs * max(1.0, ref.detach().abs().max().item())
  assert ma <= max_abs and rl <= rel_l2, f"{name}: max-abs {ma:.3e} (limit {max_abs}), rel-L2 {rl:.3e} (limit {rel_l2})"
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
