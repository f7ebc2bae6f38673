"""oracle.packed.PackedModel (quantized matrices left in their blocks, the C restatement multiplies them, only selected experts touched) against
oracle.llm.Model (everything dequantized, float64 products) on small dense and MoE models made of random GGUF blocks: the two restate the same forward
pass of tinygrad/llm/model.py and may differ only by the order of a float32 sum."""
import numpy as np
from oracle import llm as ollm, packed
from tinygrad_amd import synth

def _dense_tensors(rng, c, linear_type, head_type):
  t = {}
  mk = lambda name, rows, cols, typ: t.__setitem__(name, (synth.random_blocks(rng, typ, rows, cols, sigma=0.02), typ, (rows, cols)))
  one = lambda name, n: t.__setitem__(name, (rng.uniform(0.5, 1.5, n).astype(np.float32).view(np.uint8), 0, (1, n)))
  mk("token_embd.weight", c["vocab_size"], c["dim"], linear_type)
  for i in range(c["num_blocks"]):
    p = f"blk.{i}."
    one(p + "attn_norm.weight", c["dim"]); one(p + "ffn_norm.weight", c["dim"])
    mk(p + "attn_q.weight", c["n_heads"] * c["head_dim"], c["dim"], linear_type)
    mk(p + "attn_k.weight", c["n_kv_heads"] * c["head_dim"], c["dim"], linear_type)
    mk(p + "attn_v.weight", c["n_kv_heads"] * c["head_dim"], c["dim"], linear_type)
    mk(p + "attn_output.weight", c["dim"], c["n_heads"] * c["head_dim"], linear_type)
    mk(p + "ffn_gate.weight", c["hidden_dim"], c["dim"], linear_type); mk(p + "ffn_up.weight", c["hidden_dim"], c["dim"], linear_type)
    mk(p + "ffn_down.weight", c["dim"], c["hidden_dim"], linear_type)
  one("output_norm.weight", c["dim"])
  mk("output.weight", c["vocab_size"], c["dim"], head_type)
  return t

def _moe_tensors(rng, c):
  t = {}
  f16 = lambda name, shape, amp: t.__setitem__(name, ((rng.standard_normal(shape) * amp).astype(np.float16).view(np.uint8).reshape(-1), 1, shape))
  one = lambda name, n: t.__setitem__(name, (rng.uniform(0.5, 1.5, n).astype(np.float32).view(np.uint8), 0, (1, n)))
  E, H, D = c["num_experts"], c["hidden_dim"], c["dim"]
  nq, nkv = c["n_heads"] * c["head_dim"], c["n_kv_heads"] * c["head_dim"]
  f16("token_embd.weight", (c["vocab_size"], D), 1.0)
  for i in range(c["num_blocks"]):
    p = f"blk.{i}."
    one(p + "attn_norm.weight", D); one(p + "ffn_norm.weight", D); one(p + "attn_q_norm.weight", nq); one(p + "attn_k_norm.weight", nkv)
    f16(p + "attn_q.weight", (nq, D), D ** -0.5); f16(p + "attn_k.weight", (nkv, D), D ** -0.5); f16(p + "attn_v.weight", (nkv, D), D ** -0.5)
    f16(p + "attn_output.weight", (D, nq), nq ** -0.5); f16(p + "ffn_gate_inp.weight", (E, D), D ** -0.5)
    for nm, shp in (("ffn_gate_exps", (E, H, D)), ("ffn_up_exps", (E, H, D)), ("ffn_down_exps", (E, D, H))):
      t[p + nm + ".weight"] = (synth.random_blocks(rng, 39, shp[0] * shp[1], shp[2], mx_exp=(121, 125)), 39, shp)
  one("output_norm.weight", D)
  f16("output.weight", (c["vocab_size"], D), D ** -0.5)
  return t

def _compare(cfg, tensors, ctx=12, steps=6):
  a, b = ollm.Model(cfg, tensors, ctx, act_round_f16=False), packed.PackedModel(cfg, tensors, ctx, threads=2)
  rng = np.random.default_rng(3)
  worst = 0.0
  for pos in range(steps):
    tok = int(rng.integers(0, cfg["vocab_size"]))
    la, lb = a.forward(tok, pos), b.forward(tok, pos)
    worst = max(worst, float(np.abs(la - lb).max() / np.abs(la).max()))
    assert int(np.argmax(la)) == int(np.argmax(lb))
  return worst, a, b

def test_packed_dense_model_equals_the_dequantized_one():
  cfg = dict(num_blocks=2, dim=128, hidden_dim=256, n_heads=4, n_kv_heads=2, norm_eps=1e-5, vocab_size=96, head_dim=32, rope_theta=10000.0)
  for lt, ht in ((2, 14), (8, 8), (12, 14)):                              # Q4_0 + Q6_K head, Q8_0, Q4_K + Q6_K (K = 256 for the superblock types)
    c = dict(cfg, dim=256, head_dim=64) if lt == 12 else dict(cfg, dim=256) if ht == 14 else cfg    # (superblock types: every K a multiple of 256)
    worst, _, _ = _compare(c, _dense_tensors(np.random.default_rng(lt), c, lt, ht))
    assert worst <= 2e-5, (lt, ht, worst)

def test_packed_moe_model_equals_the_dequantized_one():
  cfg = dict(num_blocks=2, dim=64, hidden_dim=32, n_heads=2, n_kv_heads=2, norm_eps=1e-5, vocab_size=80, head_dim=32, rope_theta=10000.0,
             qk_norm=64, num_experts=6, num_experts_per_tok=2, norm_topk_prob=False, expert_gating_func=1)
  worst, a, b = _compare(cfg, _moe_tensors(np.random.default_rng(9), cfg))
  assert worst <= 2e-5, worst
  assert abs(a.min_route_gap - b.min_route_gap) <= 1e-5 and list(a.last_sel) == list(b.last_sel)
