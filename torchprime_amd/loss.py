"""Drop-in for ``torchprime.torch_xla_models.loss`` (loss.py:5-20): next-token cross entropy in one pass over the
logits (``tprime::cross_entropy_fwd`` / ``_bwd``), the shift done by indexing instead of two contiguous copies."""

from __future__ import annotations

import torch

from . import ops

IGNORE_INDEX = -100  # torch.nn.CrossEntropyLoss's default, which the reference relies on


def cross_entropy_loss(logits: torch.Tensor, labels: torch.Tensor, vocab_size: int) -> torch.Tensor:
  """Mean over the positions whose next-token label is not -100 of ``logsumexp(logits[b, s]) - logits[b, s, labels[b, s+1]]``."""
  if logits.shape[-1] != vocab_size:
    raise ValueError(f"logits' last dim {logits.shape[-1]} does not match vocab_size {vocab_size}")
  lead = logits.shape[:-2]
  if len(lead) != 1:  # (..., S, V): fold the leading dims into one batch dim
    logits = logits.reshape(-1, *logits.shape[-2:])
    labels = labels.reshape(-1, labels.shape[-1])
  labels = labels.to(logits.device)
  return ops.cross_entropy_fwd(logits, labels, IGNORE_INDEX)[0]
