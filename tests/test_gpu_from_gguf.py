"""End to end through a GGUF file: write a small llama-architecture model (Q4_0 linears, Q8_0 embedding, Q6_K lm-head, F32 norms),
load it with Transformer.from_gguf (byte-level q/k row permutation, tied-embedding rule) and compare greedy tokens with the numpy
restatement of the reference's from_gguf + forward."""
import numpy as np, pytest
from oracle import ggml as og, gguf as ogguf, llm as ollm, linear as ol

pytestmark = pytest.mark.gpu

def _make_file(tmp_path, tied: bool, kquant: bool = False, legacy: bool = False, expand: bool = False, codebook: bool = False, split_ffn: bool = False):
  """kquant: the tensor-type mix of a Q4_K_M file (Q4_K linears and embedding, Q6_K for attn_v / ffn_down / output, one Q5_K matrix).
  legacy: the same mix with Q4_1 / Q5_0 / Q5_1 in place of Q4_K / Q5_K / Q6_K.
  expand: IQ4_XS / Q1_0 / Q6_K.
  codebook: IQ3_S / IQ2_S / IQ3_XXS.  Every one of these types stays in its blocks and is read in place.
  split_ffn: ffn_up of another block type than ffn_gate (Q6_K beside Q4_K)."""
  rng = np.random.default_rng(11)
  c = dict(dim=256, hidden=512, H=4, KV=2, hd=64, L=2, vocab=512)
  def lin(rows, cols): return (rng.uniform(-1, 1, (rows, cols)) * cols ** -0.5).astype(np.float32)
  if kquant or legacy or expand or codebook:
    K4, K5, K6 = (12, og.quantize_q4_k), (13, og.quantize_q5_k), (14, og.quantize_q6_k)
    if expand: K4, K5 = (23, og.quantize_iq4_xs), (41, og.quantize_q1_0)
    if codebook: K4, K5, K6 = (21, og.quantize_iq3_s), (22, og.quantize_iq2_s), (18, og.quantize_iq3_xxs)
    if legacy: K4, K5, K6 = (3, og.quantize_q4_1), (6, og.quantize_q5_0), (7, og.quantize_q5_1)
    tensors = [("token_embd.weight", (c["vocab"], c["dim"]), K4[0], K4[1](lin(c["vocab"], c["dim"]) * 16))]
    for i in range(c["L"]):
      p = f"blk.{i}."
      mk = lambda name, rows, cols, tq: (p + name, (rows, cols), tq[0], tq[1](lin(rows, cols)))
      tensors += [(p + "attn_norm.weight", (c["dim"],), 0, (1 + 0.1 * rng.standard_normal(c["dim"])).astype(np.float32)),
                  mk("attn_q.weight", c["H"] * c["hd"], c["dim"], K4), mk("attn_k.weight", c["KV"] * c["hd"], c["dim"], K4),
                  mk("attn_v.weight", c["KV"] * c["hd"], c["dim"], K6), mk("attn_output.weight", c["dim"], c["H"] * c["hd"], K5 if i else K4),
                  (p + "ffn_norm.weight", (c["dim"],), 0, (1 + 0.1 * rng.standard_normal(c["dim"])).astype(np.float32)),
                  mk("ffn_gate.weight", c["hidden"], c["dim"], K4), mk("ffn_up.weight", c["hidden"], c["dim"], K6 if split_ffn else K4), mk("ffn_down.weight", c["dim"], c["hidden"], K6)]
    tensors.append(("output_norm.weight", (c["dim"],), 0, np.ones(c["dim"], np.float32)))
    tensors.append(("output.weight", (c["vocab"], c["dim"]), K6[0], K6[1](lin(c["vocab"], c["dim"]))))
    kvs = [("general.architecture", "qwen2"), ("qwen2.context_length", 96), ("qwen2.attention.head_count", c["H"]), ("qwen2.attention.head_count_kv", c["KV"]),
           ("qwen2.block_count", c["L"]), ("qwen2.embedding_length", c["dim"]), ("qwen2.feed_forward_length", c["hidden"]),
           ("qwen2.attention.layer_norm_rms_epsilon", 1e-6), ("qwen2.rope.freq_base", 1000000.0), ("tokenizer.ggml.tokens", [f"t{i}" for i in range(c["vocab"])])]
    from tinygrad_amd.gguf import gguf_write
    path = tmp_path / ("legacy.gguf" if legacy else "expand.gguf" if expand else "codebook.gguf" if codebook else "split_ffn.gguf" if split_ffn else "q4_k_m.gguf")
    return path, gguf_write(path, kvs, tensors)
  tensors = [("token_embd.weight", (c["vocab"], c["dim"]), 8, og.quantize_q8_0(lin(c["vocab"], c["dim"]) * 16))]
  for i in range(c["L"]):
    p = f"blk.{i}."
    tensors += [(p + "attn_norm.weight", (c["dim"],), 0, (1 + 0.1 * rng.standard_normal(c["dim"])).astype(np.float32)),
                (p + "attn_q.weight", (c["H"] * c["hd"], c["dim"]), 2, og.quantize_q4_0(lin(c["H"] * c["hd"], c["dim"]))),
                (p + "attn_k.weight", (c["KV"] * c["hd"], c["dim"]), 2, og.quantize_q4_0(lin(c["KV"] * c["hd"], c["dim"]))),
                (p + "attn_v.weight", (c["KV"] * c["hd"], c["dim"]), 2, og.quantize_q4_0(lin(c["KV"] * c["hd"], c["dim"]))),
                (p + "attn_output.weight", (c["dim"], c["H"] * c["hd"]), 2, og.quantize_q4_0(lin(c["dim"], c["H"] * c["hd"]))),
                (p + "ffn_norm.weight", (c["dim"],), 0, (1 + 0.1 * rng.standard_normal(c["dim"])).astype(np.float32)),
                (p + "ffn_gate.weight", (c["hidden"], c["dim"]), 2, og.quantize_q4_0(lin(c["hidden"], c["dim"]))),
                (p + "ffn_up.weight", (c["hidden"], c["dim"]), 2, og.quantize_q4_0(lin(c["hidden"], c["dim"]))),
                (p + "ffn_down.weight", (c["dim"], c["hidden"]), 2, og.quantize_q4_0(lin(c["dim"], c["hidden"])))]
  tensors.append(("output_norm.weight", (c["dim"],), 0, np.ones(c["dim"], np.float32)))
  if not tied: tensors.append(("output.weight", (c["vocab"], c["dim"]), 14, og.quantize_q6_k(lin(c["vocab"], c["dim"]))))
  kvs = [("general.architecture", "llama"), ("llama.context_length", 96), ("llama.attention.head_count", c["H"]), ("llama.attention.head_count_kv", c["KV"]),
         ("llama.block_count", c["L"]), ("llama.embedding_length", c["dim"]), ("llama.feed_forward_length", c["hidden"]),
         ("llama.attention.layer_norm_rms_epsilon", 1e-5), ("llama.rope.freq_base", 10000.0), ("tokenizer.ggml.tokens", [f"t{i}" for i in range(c["vocab"])])]
  from tinygrad_amd.gguf import gguf_write
  path = tmp_path / ("tied.gguf" if tied else "model.gguf")
  return path, gguf_write(path, kvs, tensors)

@pytest.mark.parametrize("tied", [False, True])
def test_from_gguf_greedy_decode(gpu, tmp_path, tied):
  from tinygrad_amd.llm import Transformer
  path, raw = _make_file(tmp_path, tied)
  model, kv = Transformer.from_gguf(path, max_context=64, max_new=32)
  assert model.config.max_context == 64 and model.config.vocab_size == 512 and kv["general.architecture"] == "llama"
  cfg, weights, _ = ogguf.from_gguf_weights(raw)
  prompt = [1, 77, 300, 9, 410, 3]
  got = list(model.generate(prompt, 12))
  o = ollm.Model(cfg, weights, 64, w_round_f16=False, act_round_f16=False)         # weights already prepared (fp16-rounded, permuted)
  ref, margins = o.generate(prompt, 12)
  print(f"min top-2 margin {min(margins):.4f}")
  assert got == ref
  o2 = ollm.Model(cfg, weights, 64, w_round_f16=False, act_round_f16=False); pos = 0
  for t in prompt[:-1]: o2.forward(t, pos); pos += 1
  cur = prompt[-1]
  for _ in range(12): lg = o2.forward(cur, pos); pos += 1; cur = int(np.argmax(lg))
  assert ol.rel_err(model.logits(), lg) <= 1e-3

@pytest.mark.parametrize("legacy", [0, 1, 2, 3, 4], ids=["q4_k_m", "q4_1-q5_0-q5_1", "iq4_xs-q1_0", "iq3_s-iq2_s-iq3_xxs", "ffn_gate-q4_k-ffn_up-q6_k"])
def test_from_gguf_q4_k_m_type_mix(gpu, tmp_path, legacy):
  """A file with the tensor types of a Q4_K_M model (Q4_K / Q5_K / Q6_K matrices, Q4_K embedding; q/k/v of mixed types, so the
  block runs one launch per projection), and the same mix with the older Q4_1 / Q5_0 / Q5_1 blocks: greedy tokens and logits against
  the numpy restatement.  Third case: IQ4_XS matrices (embedding, attention, gate / up) beside a Q1_0 matrix; fourth: IQ3_S / IQ2_S / IQ3_XXS (codebooks and sign patterns in LDS).  All read in place: the
  model streams the file's 1.1 .. 4.25 bits per weight per token, not an fp16 expansion.  Fifth: ffn_gate and ffn_up of different block types (two launches and an elementwise
  silu(gate) * up, model.py:137)."""
  from tinygrad_amd.llm import Transformer
  path, raw = _make_file(tmp_path, False, kquant=legacy in (0, 4), legacy=legacy == 1, expand=legacy == 2, codebook=legacy == 3, split_ffn=legacy == 4)
  model, kv = Transformer.from_gguf(path, max_context=64, max_new=32)
  if legacy == 2: assert model.blk[0].attn_q.ggml_type == 23 and model.embd_type == 23 and model.blk[1].attn_output.ggml_type == 41
  if legacy == 3: assert model.blk[0].attn_q.ggml_type == 21 and model.blk[1].attn_output.ggml_type == 22 and model.blk[0].attn_v.ggml_type == 18 and model.embd_type == 21
  if legacy in (2, 3):
    # what a decode step streams is the file's packed bytes: per block type, weights * bytes per block / weights per block (an fp16 expansion would stream 2 bytes per weight)
    from tinygrad_amd.runtime import GGML_QUANT
    lins = [l for b in model.blk for l in (b.attn_q, b.attn_k, b.attn_v, b.attn_output, b.ffn_gate, b.ffn_up, b.ffn_down)] + [model.output]
    packed = sum(l.out_features * l.in_features // GGML_QUANT[l.ggml_type][0] * GGML_QUANT[l.ggml_type][1] for l in lins)
    nweights = sum(l.out_features * l.in_features for l in lins)
    assert model.weight_bytes_per_token() == packed
    print(f"weight bytes per token {packed} = {8 * packed / nweights:.2f} bits per weight (fp16 expansion: {2 * nweights})")
  cfg, weights, _ = ogguf.from_gguf_weights(raw)
  prompt = [3, 200, 17, 450, 8]
  got = list(model.generate(prompt, 12))
  o = ollm.Model(cfg, weights, 64, w_round_f16=False, act_round_f16=False)
  ref, margins = o.generate(prompt, 12)
  print(f"min top-2 margin {min(margins):.4f}")
  assert got == ref
  o2 = ollm.Model(cfg, weights, 64, w_round_f16=False, act_round_f16=False); pos = 0
  for t in prompt[:-1]: o2.forward(t, pos); pos += 1
  cur = prompt[-1]
  for _ in range(12): lg = o2.forward(cur, pos); pos += 1; cur = int(np.argmax(lg))
  assert ol.rel_err(model.logits(), lg) <= 1e-3

def test_from_gguf_qwen3_shape_per_head_qk_norm(gpu, tmp_path):
  """A Qwen3-shaped file: n_heads * head_dim != embedding_length (key_length given), per-head attn_q_norm / attn_k_norm of head_dim
  weights (model.py:180), Q8_0 matrices, tied embeddings."""
  from tinygrad_amd.llm import Transformer
  from tinygrad_amd.gguf import gguf_write
  rng = np.random.default_rng(21)
  dim, hidden, H, KV, hd, L, vocab = 256, 512, 4, 2, 128, 2, 512
  def lin(rows, cols): return (rng.uniform(-1, 1, (rows, cols)) * cols ** -0.5).astype(np.float32)
  q8 = lambda name, rows, cols, amp=1.0: (name, (rows, cols), 8, og.quantize_q8_0(lin(rows, cols) * amp))
  f32 = lambda name, n: (name, (n,), 0, (1 + 0.2 * rng.standard_normal(n)).astype(np.float32))
  tensors = [q8("token_embd.weight", vocab, dim, 16.0)]
  for i in range(L):
    p = f"blk.{i}."
    tensors += [f32(p + "attn_norm.weight", dim), q8(p + "attn_q.weight", H * hd, dim), q8(p + "attn_k.weight", KV * hd, dim), q8(p + "attn_v.weight", KV * hd, dim),
                f32(p + "attn_q_norm.weight", hd), f32(p + "attn_k_norm.weight", hd), q8(p + "attn_output.weight", dim, H * hd),
                f32(p + "ffn_norm.weight", dim), q8(p + "ffn_gate.weight", hidden, dim), q8(p + "ffn_up.weight", hidden, dim), q8(p + "ffn_down.weight", dim, hidden)]
  tensors.append(f32("output_norm.weight", dim))
  kvs = [("general.architecture", "qwen3"), ("qwen3.context_length", 96), ("qwen3.attention.head_count", H), ("qwen3.attention.head_count_kv", KV),
         ("qwen3.attention.key_length", hd), ("qwen3.block_count", L), ("qwen3.embedding_length", dim), ("qwen3.feed_forward_length", hidden),
         ("qwen3.attention.layer_norm_rms_epsilon", 1e-6), ("qwen3.rope.freq_base", 1000000.0), ("tokenizer.ggml.tokens", [f"t{i}" for i in range(vocab)])]
  path = tmp_path / "qwen3.gguf"
  raw = gguf_write(path, kvs, tensors)
  model, kv = Transformer.from_gguf(path, max_context=64, max_new=32)
  assert model.config.qk_norm == hd == model.config.head_dim
  cfg, weights, _ = ogguf.from_gguf_weights(raw)
  prompt = [9, 100, 321, 5]
  got = list(model.generate(prompt, 12))
  o = ollm.Model(cfg, weights, 64, w_round_f16=False, act_round_f16=False)
  ref, margins = o.generate(prompt, 12)
  print(f"min top-2 margin {min(margins):.4f}")
  assert got == ref
  o2 = ollm.Model(cfg, weights, 64, w_round_f16=False, act_round_f16=False); pos = 0
  for t in prompt[:-1]: o2.forward(t, pos); pos += 1
  cur = prompt[-1]
  for _ in range(12): lg = o2.forward(cur, pos); pos += 1; cur = int(np.argmax(lg))
  assert ol.rel_err(model.logits(), lg) <= 1e-3


def _qwen2_file(tmp_path, extra=()):
  """A Qwen2-shaped file: q / k / v projections with bias vectors (Linear(bias=qkv_bias), model.py:161-163, 443), Q8_0 matrices, F32 biases."""
  from tinygrad_amd.gguf import gguf_write
  rng = np.random.default_rng(33)
  dim, hidden, H, KV, hd, L, vocab = 256, 512, 4, 2, 64, 2, 512
  def lin(rows, cols): return (rng.uniform(-1, 1, (rows, cols)) * cols ** -0.5).astype(np.float32)
  q8 = lambda name, rows, cols, amp=1.0: (name, (rows, cols), 8, og.quantize_q8_0(lin(rows, cols) * amp))
  f32 = lambda name, n, mean=1.0, sd=0.2: (name, (n,), 0, (mean + sd * rng.standard_normal(n)).astype(np.float32))
  tensors = [q8("token_embd.weight", vocab, dim, 16.0)]
  for i in range(L):
    p = f"blk.{i}."
    tensors += [f32(p + "attn_norm.weight", dim), q8(p + "attn_q.weight", H * hd, dim), f32(p + "attn_q.bias", H * hd, 0.0, 0.5),
                q8(p + "attn_k.weight", KV * hd, dim), f32(p + "attn_k.bias", KV * hd, 0.0, 0.5), q8(p + "attn_v.weight", KV * hd, dim), f32(p + "attn_v.bias", KV * hd, 0.0, 0.5),
                q8(p + "attn_output.weight", dim, H * hd), f32(p + "ffn_norm.weight", dim), q8(p + "ffn_gate.weight", hidden, dim), q8(p + "ffn_up.weight", hidden, dim),
                q8(p + "ffn_down.weight", dim, hidden)]
  tensors += [f32("output_norm.weight", dim), q8("output.weight", vocab, dim)]
  tensors += list(extra)
  kvs = [("general.architecture", "qwen2"), ("qwen2.context_length", 96), ("qwen2.attention.head_count", H), ("qwen2.attention.head_count_kv", KV),
         ("qwen2.block_count", L), ("qwen2.embedding_length", dim), ("qwen2.feed_forward_length", hidden),
         ("qwen2.attention.layer_norm_rms_epsilon", 1e-6), ("qwen2.rope.freq_base", 1000000.0), ("tokenizer.ggml.tokens", [f"t{i}" for i in range(vocab)])]
  path = tmp_path / "qwen2.gguf"
  return path, gguf_write(path, kvs, tensors)

def test_from_gguf_qwen2_shape_qkv_bias(gpu, tmp_path):
  from tinygrad_amd.llm import Transformer
  path, raw = _qwen2_file(tmp_path)
  model, kv = Transformer.from_gguf(path, max_context=64, max_new=32)
  assert model.blk[0].qkv_bias is not None
  cfg, weights, _ = ogguf.from_gguf_weights(raw)
  prompt = [9, 100, 321, 5]
  got = list(model.generate(prompt, 12))
  o = ollm.Model(cfg, weights, 64, w_round_f16=False, act_round_f16=False)
  ref, margins = o.generate(prompt, 12)
  print(f"min top-2 margin {min(margins):.4f}")
  assert got == ref
  o2 = ollm.Model(cfg, weights, 64, w_round_f16=False, act_round_f16=False); pos = 0
  for t in prompt[:-1]: o2.forward(t, pos); pos += 1
  cur = prompt[-1]
  for _ in range(12): lg = o2.forward(cur, pos); pos += 1; cur = int(np.argmax(lg))
  assert ol.rel_err(model.logits(), lg) <= 1e-3
  # the biases matter: without them the oracle's logits for the same token stream are far away
  o3 = ollm.Model(cfg, {k: v for k, v in weights.items() if not k.endswith(".bias")}, 64, w_round_f16=False, act_round_f16=False)
  for pos, t in enumerate(prompt + ref[:-1]): lg3 = o3.forward(t, pos)
  assert ol.rel_err(lg3, lg) > 0.05

def test_from_gguf_rejects_tensors_it_would_drop(gpu, tmp_path):
  """A tensor the built path has no use for (here a shared expert's gate) is an error, not a silently different model."""
  from tinygrad_amd.llm import Transformer
  path, _ = _qwen2_file(tmp_path, extra=[("blk.0.ffn_gate_shexp.weight", (64, 256), 8, og.quantize_q8_0(np.zeros((64, 256), np.float32)))])
  with pytest.raises(NotImplementedError, match="ffn_gate_shexp"): Transformer.from_gguf(path, max_context=64, max_new=8)

def test_from_gguf_qwen3moe_shape_expert_stacks(gpu, tmp_path):
  """A Qwen3-MoE-shaped file with the tensor types of a Q4_K_M file: Q4_K expert gate / up stacks and Q6_K down stacks stored as three-dimensional
  tensors (E, out, in), an F32 router, per-head q/k norms, top-k weights normalised by the architecture's default (model.py:432)."""
  from tinygrad_amd.llm import Transformer
  from tinygrad_amd.gguf import gguf_write
  rng = np.random.default_rng(55)
  dim, hidden, H, KV, hd, L, vocab, E, k = 256, 256, 4, 2, 64, 2, 512, 8, 2
  def lin(*shape): return (rng.uniform(-1, 1, shape) * shape[-1] ** -0.5).astype(np.float32)
  q4 = lambda name, *shape, amp=1.0: (name, shape, 12, og.quantize_q4_k(lin(*shape) * amp))
  q6 = lambda name, *shape: (name, shape, 14, og.quantize_q6_k(lin(*shape)))
  f32 = lambda name, n: (name, (n,), 0, (1 + 0.2 * rng.standard_normal(n)).astype(np.float32))
  tensors = [q4("token_embd.weight", vocab, dim, amp=16.0)]
  for i in range(L):
    p = f"blk.{i}."
    tensors += [f32(p + "attn_norm.weight", dim), q4(p + "attn_q.weight", H * hd, dim), q4(p + "attn_k.weight", KV * hd, dim), q6(p + "attn_v.weight", KV * hd, dim),
                f32(p + "attn_q_norm.weight", hd), f32(p + "attn_k_norm.weight", hd), q4(p + "attn_output.weight", dim, H * hd), f32(p + "ffn_norm.weight", dim),
                (p + "ffn_gate_inp.weight", (E, dim), 0, lin(E, dim) * 4), q4(p + "ffn_gate_exps.weight", E, hidden, dim), q4(p + "ffn_up_exps.weight", E, hidden, dim),
                q6(p + "ffn_down_exps.weight", E, dim, hidden)]
  tensors += [f32("output_norm.weight", dim), q6("output.weight", vocab, dim)]
  kvs = [("general.architecture", "qwen3moe"), ("qwen3moe.context_length", 96), ("qwen3moe.attention.head_count", H), ("qwen3moe.attention.head_count_kv", KV),
         ("qwen3moe.attention.key_length", hd), ("qwen3moe.block_count", L), ("qwen3moe.embedding_length", dim), ("qwen3moe.feed_forward_length", 4 * hidden),
         ("qwen3moe.expert_feed_forward_length", hidden), ("qwen3moe.expert_count", E), ("qwen3moe.expert_used_count", k),
         ("qwen3moe.attention.layer_norm_rms_epsilon", 1e-6), ("qwen3moe.rope.freq_base", 1000000.0), ("tokenizer.ggml.tokens", [f"t{i}" for i in range(vocab)])]
  path = tmp_path / "qwen3moe.gguf"
  raw = gguf_write(path, kvs, tensors)
  model, kv = Transformer.from_gguf(path, max_context=64, max_new=32)
  c = model.config
  assert c.num_experts == E and c.num_experts_per_tok == k and c.hidden_dim == hidden and c.norm_topk_prob and c.qk_norm == hd
  cfg, weights, _ = ogguf.from_gguf_weights(raw)
  assert cfg["norm_topk_prob"] and weights["blk.0.ffn_gate_exps.weight"].shape == (E, hidden, dim)
  prompt = [9, 100, 321, 5, 77]
  got = list(model.generate(prompt, 12))
  o = ollm.Model(cfg, weights, 64, w_round_f16=False, act_round_f16=False)
  ref, margins = o.generate(prompt, 12)
  print(f"min top-2 margin {min(margins):.4f}")
  assert got == ref
  o2 = ollm.Model(cfg, weights, 64, w_round_f16=False, act_round_f16=False); pos = 0
  for t in prompt[:-1]: o2.forward(t, pos); pos += 1
  cur = prompt[-1]
  for _ in range(12): lg = o2.forward(cur, pos); pos += 1; cur = int(np.argmax(lg))
  assert ol.rel_err(model.logits(), lg) <= 1e-3

def test_from_gguf_partial_rotary(gpu, tmp_path):
  """rope.dimension_count < head_dim (model.py:180-181, 406): only the first 24 of a head's 64 values rotate.  The file also carries q / k biases and
  per-head q / k norm weights, which follow the same per-head reordering as the q / k rows at load."""
  from tinygrad_amd.llm import Transformer
  from tinygrad_amd.gguf import gguf_write
  rng = np.random.default_rng(77)
  dim, hidden, H, KV, hd, rd, L, vocab = 256, 512, 4, 2, 64, 24, 2, 512
  def lin(rows, cols): return (rng.uniform(-1, 1, (rows, cols)) * cols ** -0.5).astype(np.float32)
  q8 = lambda name, rows, cols, amp=1.0: (name, (rows, cols), 8, og.quantize_q8_0(lin(rows, cols) * amp))
  f32 = lambda name, n, mean=1.0, sd=0.2: (name, (n,), 0, (mean + sd * rng.standard_normal(n)).astype(np.float32))
  tensors = [q8("token_embd.weight", vocab, dim, 16.0)]
  for i in range(L):
    p = f"blk.{i}."
    tensors += [f32(p + "attn_norm.weight", dim), q8(p + "attn_q.weight", H * hd, dim, 3.0), f32(p + "attn_q.bias", H * hd, 0.0, 0.5),
                q8(p + "attn_k.weight", KV * hd, dim, 3.0), f32(p + "attn_k.bias", KV * hd, 0.0, 0.5), q8(p + "attn_v.weight", KV * hd, dim), f32(p + "attn_v.bias", KV * hd, 0.0, 0.5),
                f32(p + "attn_q_norm.weight", hd, 1.0, 0.5), f32(p + "attn_k_norm.weight", hd, 1.0, 0.5),
                q8(p + "attn_output.weight", dim, H * hd), f32(p + "ffn_norm.weight", dim), q8(p + "ffn_gate.weight", hidden, dim), q8(p + "ffn_up.weight", hidden, dim),
                q8(p + "ffn_down.weight", dim, hidden)]
  tensors += [f32("output_norm.weight", dim), q8("output.weight", vocab, dim)]
  kvs = [("general.architecture", "qwen3"), ("qwen3.context_length", 96), ("qwen3.attention.head_count", H), ("qwen3.attention.head_count_kv", KV),
         ("qwen3.attention.key_length", hd), ("qwen3.rope.dimension_count", rd), ("qwen3.block_count", L), ("qwen3.embedding_length", dim), ("qwen3.feed_forward_length", hidden),
         ("qwen3.attention.layer_norm_rms_epsilon", 1e-6), ("qwen3.rope.freq_base", 10000.0), ("tokenizer.ggml.tokens", [f"t{i}" for i in range(vocab)])]
  path = tmp_path / "partial_rope.gguf"
  raw = gguf_write(path, kvs, tensors)
  model, kv = Transformer.from_gguf(path, max_context=64, max_new=32)
  assert model.config.rope_dim == rd and model.config.qk_norm == hd
  cfg, weights, _ = ogguf.from_gguf_weights(raw)
  assert cfg["rope_dim"] == rd
  prompt = [9, 100, 321, 5, 44, 12, 400]
  got = list(model.generate(prompt, 12))
  o = ollm.Model(cfg, weights, 64, w_round_f16=False, act_round_f16=False)
  ref, margins = o.generate(prompt, 12)
  print(f"min top-2 margin {min(margins):.4f}")
  assert got == ref
  o2 = ollm.Model(cfg, weights, 64, w_round_f16=False, act_round_f16=False); pos = 0
  for t in prompt[:-1]: o2.forward(t, pos); pos += 1
  cur = prompt[-1]
  for _ in range(12): lg = o2.forward(cur, pos); pos += 1; cur = int(np.argmax(lg))
  assert ol.rel_err(model.logits(), lg) <= 1e-3
  # the rotation width matters: the oracle with full-width rotation gives other logits for the same token stream
  o3 = ollm.Model(dict(cfg, rope_dim=hd), weights, 64, w_round_f16=False, act_round_f16=False)
  for pos, t in enumerate(prompt + ref[:-1]): lg3 = o3.forward(t, pos)
  assert ol.rel_err(lg3, lg) > 0.01

def test_from_gguf_glm4moe_shape(gpu, tmp_path):
  """A GLM-4.5-shaped file (model.py:403-404, 424, 434-443): `post_attention_norm` tensor names, one leading dense block with its own FFN width, sigmoid
  gating with `exp_probs_b` selection biases, normalised and scaled top-k weights, one shared expert (`expert_shared_count` x the expert width), q / k / v
  biases, partial rotary, and a trailing next-token-prediction layer that the decoder must not load."""
  from tinygrad_amd.llm import Transformer
  from tinygrad_amd.gguf import gguf_write
  rng = np.random.default_rng(91)
  dim, hidden, dense_hidden, H, KV, hd, rd, L, vocab, E, k = 256, 128, 512, 4, 2, 64, 32, 3, 512, 8, 2
  def lin(*shape): return (rng.uniform(-1, 1, shape) * shape[-1] ** -0.5).astype(np.float32)
  q8 = lambda name, *shape, amp=1.0: (name, shape, 8, og.quantize_q8_0(lin(*shape) * amp))
  f32 = lambda name, n, mean=1.0, sd=0.2: (name, (n,), 0, (mean + sd * rng.standard_normal(n)).astype(np.float32))
  tensors = [q8("token_embd.weight", vocab, dim, amp=16.0)]
  for i in range(L + 1):                                                # block L is the next-token-prediction layer
    p = f"blk.{i}."
    tensors += [f32(p + "attn_norm.weight", dim), q8(p + "attn_q.weight", H * hd, dim), f32(p + "attn_q.bias", H * hd, 0.0, 0.3), q8(p + "attn_k.weight", KV * hd, dim),
                f32(p + "attn_k.bias", KV * hd, 0.0, 0.3), q8(p + "attn_v.weight", KV * hd, dim), f32(p + "attn_v.bias", KV * hd, 0.0, 0.3),
                q8(p + "attn_output.weight", dim, H * hd), f32(p + "post_attention_norm.weight", dim)]
    if i == 0:
      tensors += [q8(p + "ffn_gate.weight", dense_hidden, dim), q8(p + "ffn_up.weight", dense_hidden, dim), q8(p + "ffn_down.weight", dim, dense_hidden)]
    else:
      tensors += [(p + "ffn_gate_inp.weight", (E, dim), 0, lin(E, dim) * 4), f32(p + "exp_probs_b.bias", E, 0.0, 0.3),
                  q8(p + "ffn_gate_exps.weight", E, hidden, dim), q8(p + "ffn_up_exps.weight", E, hidden, dim), q8(p + "ffn_down_exps.weight", E, dim, hidden),
                  q8(p + "ffn_gate_shexp.weight", hidden, dim), q8(p + "ffn_up_shexp.weight", hidden, dim), q8(p + "ffn_down_shexp.weight", dim, hidden)]
    if i == L: tensors += [f32(p + "nextn.enorm.weight", dim), q8(p + "nextn.eh_proj.weight", dim, 2 * dim)]
  tensors += [f32("output_norm.weight", dim), q8("output.weight", vocab, dim)]
  a = "glm4moe"
  kvs = [("general.architecture", a), (f"{a}.context_length", 96), (f"{a}.attention.head_count", H), (f"{a}.attention.head_count_kv", KV),
         (f"{a}.attention.key_length", hd), (f"{a}.rope.dimension_count", rd), (f"{a}.block_count", L + 1), (f"{a}.nextn_predict_layers", 1),
         (f"{a}.embedding_length", dim), (f"{a}.feed_forward_length", dense_hidden), (f"{a}.expert_feed_forward_length", hidden),
         (f"{a}.expert_count", E), (f"{a}.expert_used_count", k), (f"{a}.expert_shared_count", 1), (f"{a}.leading_dense_block_count", 1),
         (f"{a}.expert_gating_func", 2), (f"{a}.expert_weights_norm", True), (f"{a}.expert_weights_scale", 1.5),
         (f"{a}.attention.layer_norm_rms_epsilon", 1e-5), (f"{a}.rope.freq_base", 10000.0), ("tokenizer.ggml.tokens", [f"t{i}" for i in range(vocab)])]
  path = tmp_path / "glm4moe.gguf"
  raw = gguf_write(path, kvs, tensors)
  model, kv = Transformer.from_gguf(path, max_context=64, max_new=32)
  c = model.config
  assert (c.num_blocks, c.leading_dense_blocks, c.dense_hidden_dim, c.shared_expert_dim, c.shared_expert_gate, c.expert_bias) == (L, 1, dense_hidden, hidden, False, True)
  assert c.expert_gating_func == 2 and c.norm_topk_prob and c.routed_scaling_factor == 1.5 and c.rope_dim == rd
  assert [b.moe for b in model.blk] == [False, True, True]
  cfg, weights, _ = ogguf.from_gguf_weights(raw)
  assert cfg["num_blocks"] == L and cfg["leading_dense_blocks"] == 1 and "blk.1.ffn_norm.weight" in weights
  prompt = [9, 100, 321, 5, 77, 410]
  got = list(model.generate(prompt, 16))
  o = ollm.Model(cfg, weights, 64, w_round_f16=False, act_round_f16=False)
  ref, margins = o.generate(prompt, 16)
  print(f"min top-2 margin {min(margins):.4f}, min biased-score gap {o.min_route_gap:.2e}")
  assert got == ref
  o2 = ollm.Model(cfg, weights, 64, w_round_f16=False, act_round_f16=False); pos = 0
  for t in prompt[:-1]: o2.forward(t, pos); pos += 1
  cur = prompt[-1]
  for _ in range(16): lg = o2.forward(cur, pos); pos += 1; cur = int(np.argmax(lg))
  assert ol.rel_err(model.logits(), lg) <= 1e-3
