"""The striped sequence layout and its causal mask against the reference's own known-answer vectors
(tests/golden/parallelism_kats.json, the data of torchprime/tests/test_parallelism_utils.py:16-71): bit-exact
integer results, on the host."""

import json
import os

import numpy as np
import pytest
import torch

from torchprime_amd import parallelism_utils as p_utils

with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "parallelism_kats.json")) as f:
  KAT = json.load(f)


@pytest.mark.parametrize("name,to_contiguous", [("reorder_sequence_forward", False), ("reorder_sequence_backward", True),
                                                ("reorder_sequence_forward_2d", False)])
def test_reorder_sequence_kats(name, to_contiguous):
  k = KAT[name]
  res = p_utils.reorder_sequence(tensor=torch.tensor(k["input"]), cp_size=k["cp_size"], seq_dim=k["seq_dim"], to_contiguous=to_contiguous)
  assert torch.equal(res, torch.tensor(k["expected"]))


def test_load_balanced_causal_mask_kat_and_semantics():
  k = KAT["load_balanced_causal_mask"]
  m = p_utils.LoadBalancedCausalMask(shape=tuple(k["shape"]), cp_size=k["cp_size"])
  assert (m.q_sequence == np.array(k["q_sequence"])).all()
  # row i is the causal row of original position q_sequence[i]
  dense = m.dense()
  for i, p in enumerate(k["q_sequence"]):
    assert dense[i].tolist() == [j <= p for j in range(8)]
  assert m == p_utils.LoadBalancedCausalMask(shape=(8, 8), cp_size=4) and hash(m) == hash(p_utils.LoadBalancedCausalMask(shape=(8, 8), cp_size=4))
  assert m != p_utils.LoadBalancedCausalMask(shape=(8, 8), cp_size=2)
  assert p_utils.LoadBalancedCausalMask(shape=(8, 8), cp_size=4, offset=1).dense()[0].tolist() == [True, True] + [False] * 6


@pytest.mark.parametrize("name", ["reorder_mask_1d", "reorder_mask_2d"])
def test_reorder_mask_kats(name):
  k = KAT[name]
  res = p_utils.reorder_mask(tensor=np.array(k["input"]), cp_size=k["cp_size"], seq_dim=k["seq_dim"])
  assert (res == np.array(k["expected"])).all()


@pytest.mark.parametrize("cp_size", [2, 4, 8, 16])
def test_round_trip_and_agreement_of_the_two_reorders(cp_size):
  k = KAT["large_tensor_roundtrip"]
  x = torch.randint(k["high"], tuple(k["shape"]), generator=torch.Generator().manual_seed(0))
  y = p_utils.reorder_sequence(x, cp_size=cp_size, seq_dim=1, to_contiguous=False)
  assert torch.equal(p_utils.reorder_sequence(y, cp_size=cp_size, seq_dim=1, to_contiguous=True), x)
  assert (p_utils.reorder_mask(x.numpy(), cp_size=cp_size, seq_dim=1) == y.numpy()).all()
  # 4-D activations, sequence at dim 2, as AttentionModule reorders K / V (attention.py:78-89)
  t = torch.arange(2 * 3 * 64 * 4).reshape(2, 3, 64, 4)
  z = p_utils.reorder_sequence(t, cp_size=cp_size, seq_dim=2)
  q_seq = p_utils.LoadBalancedCausalMask(shape=(64, 64), cp_size=cp_size).q_sequence
  assert torch.equal(z, t[:, :, torch.from_numpy(q_seq)])


def test_errors():
  with pytest.raises(ValueError):
    p_utils.reorder_sequence(torch.arange(8), cp_size=3, seq_dim=0)
  with pytest.raises(ValueError):
    p_utils.reorder_sequence(torch.arange(10), cp_size=2, seq_dim=0)
  assert p_utils.reorder_sequence(None, cp_size=2) is None
