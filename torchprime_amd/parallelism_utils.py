"""Drop-in for the single-GPU half of ``torchprime.utils.parallelism_utils``: the striped ("load-balanced")
sequence layout of context parallelism and the causal mask that goes with it.

* reorder_sequence        parallelism_utils.py:8-84    (torch tensors, any device)
* reorder_mask            parallelism_utils.py:87-...   (numpy arrays; same permutation as the forward reorder)
* LoadBalancedCausalMask  parallelism_utils.py:87-152  a causal mask whose query rows are in the striped order:
                          row i stands for original position ``q_sequence[i]`` and may attend to key j (keys in the
                          original order) iff ``q_sequence[i] + offset >= j``.  The attention kernels evaluate it from
                          ``q_sequence`` directly; no (S, S) array is ever built.
* cp_enabled / lb_cp_enabled   parallelism_utils.py:155-172

A sequence is cut into ``2 * cp_size`` chunks; rank r of a context-parallel group gets chunks r and
``2 * cp_size - 1 - r``, which pairs the cheapest and the most expensive rows of a causal mask.
"""

from __future__ import annotations

import numpy as np
import torch


def _check(shape, seq_len: int, cp_size: int):
  if cp_size % 2 != 0:
    raise ValueError(f"{cp_size=} must be a multiple of 2.")
  # Need to ensure we have 2 pairs to swap for balancing between cp ranks
  if seq_len % (cp_size * 2) != 0:
    raise ValueError(f"tensor.shape={tuple(shape)} is not a multiple of {cp_size*2=}")


def _forward_indices(cp_size: int) -> list[int]:
  # chunk order [0, 2c-1, 1, 2c-2, ...]
  out = []
  for r in range(cp_size):
    out += [r, 2 * cp_size - 1 - r]
  return out


def _to_contiguous_indices(cp_size: int) -> list[int]:
  # positions, in the striped order, of chunks 0, 1, 2, ...: chunk r sits at 2r, chunk 2c-1-r at 2r+1
  half = cp_size // 2
  first_pair = [4 * r for r in range(half)]
  second_pair = [4 * r + 2 for r in range(half)]
  third_pair = [2 * cp_size - 1 - 4 * r for r in range(half)]
  fourth_pair = [i - 2 for i in third_pair]
  first_block = first_pair + third_pair
  second_block = second_pair + fourth_pair
  out = []
  for a, b in zip(first_block, second_block):
    out += [a, b]
  return out


def reorder_sequence(tensor, cp_size: int, seq_dim: int = 1, to_contiguous: bool = False):
  """Reorders the sequence dim of ``tensor`` into the striped layout (``to_contiguous=False``:
  ``[0..7] -> [0, 1, 6, 7, 2, 3, 4, 5]`` for ``cp_size=2``) or back (``to_contiguous=True``)."""
  if tensor is None:
    return tensor
  seq_len = tensor.shape[seq_dim]
  _check(tensor.shape, seq_len, cp_size)
  group_size = seq_len // (2 * cp_size)
  shape = tensor.shape
  reshaped = tensor.reshape(*shape[:seq_dim], 2 * cp_size, group_size, *shape[seq_dim + 1 :])
  idx = _to_contiguous_indices(cp_size) if to_contiguous else _forward_indices(cp_size)
  src = torch.tensor(idx, device=tensor.device)
  return torch.index_select(reshaped, seq_dim, src).reshape(shape)


def reorder_mask(tensor, cp_size: int, seq_dim: int):
  seq_len = tensor.shape[seq_dim]
  _check(tensor.shape, seq_len, cp_size)
  group_size = seq_len // (2 * cp_size)
  shape = tensor.shape
  reshaped = tensor.reshape(*shape[:seq_dim], 2 * cp_size, group_size, *shape[seq_dim + 1 :])
  return np.take(reshaped, np.array(_forward_indices(cp_size)), axis=seq_dim).reshape(shape)


class LoadBalancedCausalMask:
  """Lazy causal mask for query rows in the striped order.

  Attributes:
    offset: offset of q start wrt kv.  A positive offset shifts the bottom triangle upward, a negative one shifts
      it downward (rows left without any allowed key come out as zeros here; the reference calls them undefined).
    shape, cp_size, q_sequence: ``q_sequence[i]`` is the original position of striped row ``i``.
  """

  def __init__(self, shape: tuple[int, int], offset: int = 0, shard_count: int = 1, cp_size: int = 4):
    self.shape = tuple(shape)
    self.offset = offset
    self.shard_count = shard_count
    self.cp_size = cp_size
    arr = np.arange(shape[0])
    out = reorder_mask(tensor=arr[np.newaxis, :, np.newaxis, np.newaxis], cp_size=cp_size, seq_dim=1)
    self.q_sequence = out[0, :, 0, 0]

  def mask_function(self, q_ids, kv_ids):
    return q_ids >= kv_ids if self.offset == 0 else q_ids + self.offset >= kv_ids

  def dense(self) -> np.ndarray:
    """The (q, kv) boolean array, for tests and small shapes."""
    return self.mask_function(self.q_sequence[:, None], np.arange(self.shape[1])[None, :])

  def __eq__(self, other: object):
    if not isinstance(other, type(self)):
      return NotImplemented
    return self.shape == other.shape and self.offset == other.offset and np.array_equal(self.q_sequence, other.q_sequence)

  def __hash__(self):
    return hash((type(self), self.shape, self.offset, self.q_sequence.tobytes() if self.q_sequence is not None else None))


def cp_enabled(config) -> bool:
  """Context parallelism is a multi-GPU layout; a config that asks for it still parses here."""
  return "context" in config.ici_mesh and config.ici_mesh.context > 1


def lb_cp_enabled(config) -> bool:
  return cp_enabled(config) and "load_balance_cp" in config.model and config.model.load_balance_cp
