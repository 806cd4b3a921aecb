"""Host-side logic that needs no GPU: the C-ABI library loads and exports what the header declares,
argument validation returns error codes before any launch, the drop-in Python surface has the
reference's names/signatures, and the custom ops trace with fake tensors."""

import ctypes
import inspect
import os
import re

import pytest
import torch

import torchprime_amd as tpa
from oracle import tprime_oracle as orc
from torchprime_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _header_symbols():
  text = open(os.path.join(ROOT, "include", "tprime_hip.h")).read()
  text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
  return sorted(set(re.findall(r"\b(tp_[a-z_0-9]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
  lib = _lib.load()
  syms = _header_symbols()
  assert len(syms) >= 11
  for name in syms:
    assert hasattr(lib, name), f"{name} declared in include/tprime_hip.h but not exported"
  assert sorted(_lib.SIGNATURES) == syms, "ctypes prototypes and header disagree"
  assert lib.tp_version() >= 100
  assert lib.tp_last_error() == b"" or isinstance(lib.tp_last_error(), bytes)


def test_c_abi_validates_arguments_before_launching():
  lib = _lib.load()
  z3 = _lib._I64x3(0, 0, 0)
  assert lib.tp_rmsnorm_fwd(None, None, None, None, 4, 8, 8, 8, 1e-6, 0, 0, None) == -1
  assert b"null pointer" in lib.tp_last_error()
  buf = ctypes.create_string_buffer(4096)
  p = ctypes.addressof(buf)
  p += (-p) % 16
  assert lib.tp_rmsnorm_fwd(p, p, p, p, 4, 8, 4, 8, 1e-6, 0, 0, None) == -1  # stride < hidden
  assert lib.tp_rmsnorm_fwd(p, p, p, p, 4, 8, 8, 8, 1e-6, 2, 0, None) == -2  # fp32 x with bf16 weight
  assert lib.tp_attn_fwd(p, p, p, None, p, p, 1, 3, 2, 8, 8, 128, 128, z3, z3, z3, z3, 0.1, 1, 0, None) == -1  # Hq % Hkv
  s96 = _lib._I64x3(8 * 2 * 96, 96, 2 * 96)
  assert lib.tp_attn_fwd(p, p, p, None, p, p, 1, 2, 2, 8, 8, 96, 96, s96, s96, s96, s96, 0.1, 1, 0, None) == -2  # head dim
  assert b"not built" in lib.tp_last_error()
  assert lib.tp_attn_fwd(p, p, p, None, p, p, 1, 2, 2, 8, 8, 128, 128, z3, z3, z3, z3, 0.1, 1, 7, None) == -2  # unknown dtype
  s192, s128 = _lib._I64x3(8 * 2 * 192, 192, 2 * 192), _lib._I64x3(8 * 2 * 128, 128, 2 * 128)
  assert lib.tp_attn_fwd(p, p, p, None, p, p, 1, 2, 2, 8, 8, 192, 128, s192, s192, s128, s128, 0.1, 1, 2, None) == -2  # fp32: dims 64 / 128 only
  assert lib.tp_attn_fwd(p, p, p, None, p, p, 1, 2, 2, 8, 8, 128, 128, z3, z3, z3, z3, -1.0, 1, 0, None) == -1  # scale
  assert lib.tp_attn_fwd(p, p, p, p, p, p, 1, 2, 2, 8, 16, 128, 128, z3, z3, z3, z3, 0.1, 1, 0, None) == -1  # seg, Sq != Skv
  assert lib.tp_rope_apply(p, None, p, p, None, p, None, 1, 2, 0, 8, 24, z3, z3, z3, z3, 0, 24, 0, 0, 0, 0, 0, None) == -2  # D % 16
  assert lib.tp_rope_apply(p + 2, None, p, p, None, p, None, 1, 2, 0, 8, 32, z3, z3, z3, z3, 0, 32, 0, 0, 0, 0, 0, None) == -1  # alignment
  assert lib.tp_rmsnorm_bwd_workspace_bytes(32768, 4096) == 512 * 4096 * 4
  assert lib.tp_rmsnorm_bwd_workspace_bytes(10, 64) == 12 * 64 * 4
  assert lib.tp_rmsnorm_bwd_workspace_bytes(32768, 512) == 4096 * 512 * 4   # short rows: more partial rows
  assert lib.tp_rmsnorm_bwd_workspace_bytes(32768, 1536) == 2048 * 1536 * 4
  assert lib.tp_rmsnorm_bwd_workspace_bytes(32768, 2048) == 1024 * 2048 * 4
  assert lib.tp_rmsnorm_bwd_workspace_bytes(32768, 16384) == 512 * 16384 * 4
  assert lib.tp_attn_bwd_workspace_bytes(4, 32, 8192) == 2 * 4 * 32 * 8192 * 4


def test_ops_reject_cpu_tensors_and_bad_shapes():
  x = torch.ones(2, 8)
  with pytest.raises(RuntimeError, match="no CPU path"):
    _lib.require_gpu(x)
  with pytest.raises(TypeError):
    _lib.dtype_code(torch.int8)
  q = torch.zeros(1, 4, 8, 64, dtype=torch.bfloat16)
  with pytest.raises(ValueError):
    tpa.ops._check_attn(q, q[:, :3], q[:, :3], None)  # 4 heads over 3 kv heads
  with pytest.raises(NotImplementedError):
    tpa.ops._check_attn(q[..., :32], q[..., :32], q[..., :32], None)
  with pytest.raises(AssertionError, match="Sharding along sequence dimension"):
    tpa.ops._check_attn(q, q, q, torch.zeros(1, 4, dtype=torch.int32))


def test_reference_surface_names_and_signatures():
  sig = inspect.signature(tpa.AttentionModule.forward)
  assert list(sig.parameters) == ["self", "query_states", "key_states", "value_states", "attention_mask"]
  assert list(inspect.signature(tpa.AttentionModule.__init__).parameters) == ["self", "config", "kernel_config"]
  m = tpa.AttentionModule(tpa.Config(attention_kernel="flash_attention"), {"block_q": 1024})
  assert m.kernel_config == {"block_q": 1024} and m.config.attention_kernel == "flash_attention"
  w = inspect.signature(tpa.tpu_splash_attention_jax_call_wrapper)
  assert list(w.parameters)[:11] == ["mask", "query", "key", "value", "config", "decoder_segment_ids", "causal",
                                     "attn_logits_soft_cap", "is_forward", "q_seq_shards", "grad_output"]
  assert list(inspect.signature(tpa.apply_rotary_pos_emb).parameters) == ["q", "k", "cos", "sin", "position_ids", "unsqueeze_dim"]
  assert list(inspect.signature(tpa.apply_rotary_pos_emb_interleave).parameters) == ["q", "k", "cos", "sin", "position_ids", "unsqueeze_dim"]
  for cls in (tpa.LlamaRMSNorm, tpa.MixtralRMSNorm, tpa.DeepseekV3RMSNorm):
    n = cls(32)
    assert n.variance_epsilon == 1e-6 and n.weight.shape == (32,) and torch.equal(n.weight.data, torch.ones(32))
    assert list(n.state_dict()) == ["weight"]
  r = tpa.RopeScaling()
  assert (r.factor, r.low_freq_factor, r.high_freq_factor, r.original_context_len) == (8.0, 1.0, 4.0, 8192)
  with pytest.raises(TypeError):
    tpa.RopeScaling(8.0)  # keyword-only, as in the reference
  emb = tpa.LlamaRotaryEmbedding(128, 500000.0)
  assert "inv_freq" not in emb.state_dict() and emb.inv_freq.shape == (64,)


def test_repeat_kv_and_rotate_half():
  x = torch.randn(2, 3, 5, 8)
  assert torch.equal(tpa.repeat_kv(x, 4), torch.repeat_interleave(x, 4, dim=1))
  assert tpa.repeat_kv(x, 1) is x
  assert torch.equal(tpa.rotate_half(x), torch.cat((-x[..., 4:], x[..., :4]), -1))
  assert torch.equal(tpa.rotate_half(x), orc.rotate_half(x))


def test_rope_frequency_functions_match_oracle_and_assert():
  for hd, theta in ((128, 500000.0), (64, 10000.0), (512, 500000.0)):
    torch.testing.assert_close(tpa.default_rope_frequencies(hd, theta), orc.default_rope_frequencies(hd, theta), rtol=0, atol=0)
    torch.testing.assert_close(tpa.llama3_rope_frequencies(hd, theta), orc.default_rope_frequencies(hd, theta), rtol=0, atol=0)
    for sc in (tpa.RopeScaling(), tpa.RopeScaling(factor=32.0, low_freq_factor=2.0, high_freq_factor=8.0, original_context_len=4096)):
      got = tpa.llama3_rope_frequencies(hd, theta, sc)
      ref = orc.llama3_rope_frequencies(hd, theta, sc.factor, sc.low_freq_factor, sc.high_freq_factor, sc.original_context_len)
      torch.testing.assert_close(got, ref, rtol=0, atol=0)
  with pytest.raises(AssertionError, match="must be greater or equal"):
    tpa.llama3_rope_frequencies(128, 1e4, tpa.RopeScaling(low_freq_factor=8.0, high_freq_factor=1.0))
  # DeepSeek-V3 yaml values (configs/model/deepseek-v3.yaml:14-52): factor collapses to 1
  cfg = tpa.Config(rope_theta=10000, head_dim=64, hidden_size=7168, num_attention_heads=128, max_position_embeddings=4096,
                   rope_scaling=dict(beta_fast=32, beta_slow=1, factor=40, mscale=1.0, mscale_all_dim=1.0,
                                     original_max_position_embeddings=4096, rope_type="yarn", type="yarn"))
  inv, att = tpa.deepseek_v3_rope_init_fn(cfg)
  torch.testing.assert_close(inv, orc.default_rope_frequencies(64, 10000.0))
  assert att == 1.0
  for kw in (dict(factor=4, original_max=4096, max_position_embeddings=16384),
             dict(factor=16, original_max=2048, max_position_embeddings=32768, mscale=0.707, mscale_all_dim=1.0)):
    rs = {"rope_type": "yarn", "factor": kw["factor"], "original_max_position_embeddings": kw["original_max"]}
    rs.update({k: kw[k] for k in ("mscale", "mscale_all_dim") if k in kw})
    c = tpa.Config(rope_theta=10000.0, head_dim=64, hidden_size=512, num_attention_heads=8,
                   max_position_embeddings=kw["max_position_embeddings"], rope_scaling=rs)
    inv, att = tpa.deepseek_v3_rope_init_fn(c)
    ref, ratt = orc.yarn_rope_frequencies(64, 10000.0, kw["factor"], kw["original_max"], kw["max_position_embeddings"],
                                          mscale=kw.get("mscale"), mscale_all_dim=kw.get("mscale_all_dim"))
    torch.testing.assert_close(inv, ref, rtol=0, atol=0)
    assert att == pytest.approx(ratt)
  with pytest.raises(AssertionError):
    tpa.deepseek_v3_rope_init_fn(tpa.Config(rope_theta=1e4, rope_scaling={"rope_type": "linear", "factor": 2}))


def test_config_and_splash_config():
  c = tpa.Config(attention_kernel=None, nested={"a": 1})
  assert "attention_kernel" in c and "load_balance_cp" not in c and c.nested.a == 1 and c["nested"]["a"] == 1
  assert c.get("missing", 3) == 3 and dict(c)["attention_kernel"] is None
  from types import SimpleNamespace
  from torchprime_amd.config import has_key
  assert has_key(SimpleNamespace(x=1), "x") and not has_key(SimpleNamespace(x=1), "y") and has_key({"x": 1}, "x")
  s = tpa.SplashAttentionConfig(mesh="m", sa_block_q=1024)
  r = tpa.SplashAttentionConfig.from_json(s.to_json())
  assert r.sa_block_q == 1024 and r.mesh == "m" and not r.attentiontype_local_sliding
  assert tpa.SplashAttentionConfig.from_json('{"unknown_key": 5}').extra == {"unknown_key": 5}


def test_attention_module_cpu_side_errors():
  q = torch.zeros(1, 2, 8, 64, dtype=torch.bfloat16)
  # load-balanced context parallelism reorders K / V on the host side and then needs the GPU kernels like any other call
  m = tpa.AttentionModule(tpa.Config(attention_kernel="splash_attention", load_balance_cp=True, context=2))
  with pytest.raises(RuntimeError, match="no CPU path"):
    m(q, q, q)
  with pytest.raises(ValueError, match="not a multiple"):
    m(q[:, :, :6], q[:, :, :6], q[:, :, :6])  # 6 rows do not split into 2 * cp_size chunks
  m = tpa.AttentionModule(tpa.Config(attention_kernel="flash_attention", num_attention_heads=2, num_key_value_heads=2))
  with pytest.raises(RuntimeError, match="no CPU path"):
    m(q, q, q)
  with pytest.raises(NotImplementedError, match="mask objects of type"):
    tpa.tpu_splash_attention_jax_call_wrapper(object(), q, q, q, "{}", None, True)
  with pytest.raises(ValueError, match="mask shape"):
    tpa.tpu_splash_attention_jax_call_wrapper(tpa.parallelism_utils.LoadBalancedCausalMask((16, 16), cp_size=2), q, q, q, "{}", None, False)
  with pytest.raises(ValueError, match="soft_cap must be positive"):
    tpa.tpu_splash_attention_jax_call_wrapper(None, q, q, q, "{}", None, True, attn_logits_soft_cap=-1.0)


def test_ops_trace_with_fake_tensors():
  """register_fake shapes/dtypes/layouts: what AOT tracing (torchprime's remat tooling) relies on."""
  from torch._subclasses.fake_tensor import FakeTensorMode

  with FakeTensorMode():
    B, Hq, Hkv, S, D = 2, 8, 2, 64, 128
    q = torch.empty((B, S, Hq, D), dtype=torch.bfloat16, device="cuda").transpose(1, 2)
    k = torch.empty((B, S, Hkv, D), dtype=torch.bfloat16, device="cuda").transpose(1, 2)
    out, lse = torch.ops.tprime.attn_fwd(q, k, k, None, 0.1, True)
    assert out.shape == (B, Hq, S, D) and out.transpose(1, 2).is_contiguous() and lse.shape == (B, Hq, S)
    dq, dk, dv = torch.ops.tprime.attn_bwd(out, q, k, k, out, lse, None, 0.1, True)
    assert dq.shape == q.shape and dk.shape == k.shape and dv.shape == k.shape
    x = torch.empty((B, S, 512), dtype=torch.bfloat16, device="cuda")
    w = torch.empty((512,), dtype=torch.float32, device="cuda")
    y, rstd = torch.ops.tprime.rmsnorm_fwd(x, w, 1e-5)
    assert y.dtype == torch.float32 and y.shape == x.shape and rstd.shape == (B * S,)
    cos = torch.empty((1, S, D), dtype=torch.bfloat16, device="cuda")
    qo, ko = torch.ops.tprime.rope_apply(q, k, cos, cos, None, False, False)
    assert qo.shape == q.shape and ko.shape == k.shape
    c, s = torch.ops.tprime.rope_table(torch.empty(64, device="cuda"), torch.empty((1, S), device="cuda"), 1.0, torch.bfloat16)
    assert c.shape == (1, S, 128) and c.dtype == torch.bfloat16


def test_product_code_does_not_import_the_oracle():
  pkg = os.path.join(ROOT, "torchprime_amd")
  for fn in os.listdir(pkg):
    if fn.endswith(".py"):
      src = open(os.path.join(pkg, fn)).read()
      assert "oracle" not in src, f"{fn} mentions the oracle"


def test_rotary_frequencies_stay_fp32_under_a_dtype_cast():
  """``model.to(torch.bfloat16)`` must not round ``inv_freq`` (8 bits of frequency put the angle at position 300 off
  by more than a radian for the fast dimensions); device moves still apply."""
  import torchprime_amd as tpa
  rot = tpa.LlamaRotaryEmbedding(128, 500000.0)
  before = rot.inv_freq.clone()
  holder = torch.nn.Sequential(rot).to(torch.bfloat16)
  assert holder[0].inv_freq.dtype == torch.float32 and torch.equal(holder[0].inv_freq, before)
  assert "inv_freq" not in rot.state_dict()


def test_bench_refuses_more_than_one_gpu_and_needs_a_gpu():
  """bench.py measures the one-GPU hot path: --gpus above 1 exits with a message that says so, and without a GPU the
  default run stops before any work (no CPU fallback is ever timed in the product's place)."""
  import subprocess
  import sys
  root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
  r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
  assert r.returncode != 0 and "one-GPU" in r.stderr
  if not torch.cuda.is_available():
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py")], capture_output=True, text=True, timeout=300)
    assert r.returncode != 0 and "needs a GPU" in r.stderr and "metric" not in r.stdout

