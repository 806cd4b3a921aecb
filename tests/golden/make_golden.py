"""Writes the golden fixtures in this directory from the CPU oracle.

The reference cannot be imported here (its hot-path modules import torch_xla, jax and omegaconf at
module top), and its own tests hold no numeric vectors for this path, so these fixtures are the
oracle's outputs on seeded inputs, frozen: they guard the oracle against drift and give the GPU tests
fixed targets.  Inputs are regenerated from the seeds (torch's CPU generator is reproducible), only
the expected outputs are stored.

Run from the repository root:  python tests/golden/make_golden.py
"""

import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import tprime_oracle as orc  # noqa: E402
from tests.util import packed_segment_ids, randn  # noqa: E402


def c1_inputs():
  """benchmark configuration 1: tiny Llama attention block, fp32 (the reference's test fixture shape)."""
  x = randn((2, 128, 512), 1234)
  w = {n: randn((512, 512), 1234 + i + 1, std=0.02) for i, n in enumerate(("wq", "wk", "wv", "wo"))}
  w_norm = 1 + randn((512,), 1239, std=0.02)
  return x, w_norm, w


def attn_inputs():
  B, Hq, Hkv, S, D = 1, 4, 2, 80, 64
  q, k, v, do = (randn((B, h, S, D), 4321 + i) for i, h in enumerate((Hq, Hkv, Hkv, Hq)))
  seg, _ = packed_segment_ids(B, S, 8, 30, seed=4321)
  return q, k, v, do, seg


def main():
  x, w_norm, w = c1_inputs()
  y = orc.llama_attention_block(x, w_norm, w["wq"], w["wk"], w["wv"], w["wo"], 8, 8, 1e-5, 500000.0)
  np.savez_compressed(os.path.join(HERE, "c1_llama_block.npz"), out_rows=y[:, ::8].numpy())

  q, k, v, do, seg = attn_inputs()
  out, dq, dk, dv = orc.attention_grads_ref(q, k, v, do, seg, True, None, torch.float64)
  _, lse = orc.attention_ref(q, k, v, seg, True, None, torch.float64)
  np.savez_compressed(
    os.path.join(HERE, "attn_segments_small.npz"),
    out=out.float().numpy(), lse=lse.float().numpy(), dq=dq.float().numpy(), dk=dk.float().numpy(), dv=dv.float().numpy(),
  )  # fmt: skip

  yarn, att = orc.yarn_rope_frequencies(64, 10000.0, 4, 4096, max_position_embeddings=16384)
  np.savez_compressed(
    os.path.join(HERE, "rope_frequencies.npz"),
    llama3_d128=orc.llama3_rope_frequencies(128, 500000.0, factor=8.0).numpy(),
    default_d128=orc.default_rope_frequencies(128, 500000.0).numpy(),
    yarn_d64_f4=yarn.numpy(), yarn_attention_factor=np.float64(att),
  )  # fmt: skip
  print("golden fixtures written to", HERE)


if __name__ == "__main__":
  main()
