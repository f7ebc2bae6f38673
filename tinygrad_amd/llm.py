"""Batch-1 decode of a llama-architecture Transformer whose linears stay in GGUF blocks (mirror of tinygrad/llm/model.py).

Transformer mirrors the reference's class for the dense (non-MoE) path: token_embd -> blocks -> output_norm -> output ->
greedy argmax (model.py:358-364).  Every Linear call site of the reference (model.py:168,198,137,362) is a fused dequant-GEMV
over the raw GGUF bytes; per block the launches are
  rmsnorm -> q/k/v (one launch) -> RoPE + KV append + attention -> attn_output (+ residual) -> rmsnorm -> gate/up + SwiGLU -> down (+ residual)
and one token step is captured once and replayed (the reference's TinyJit replay), with position/token kept in device memory.
Numerics that differ from the reference's defaults, stated once: activations entering a linear are rounded to fp16
(reference: fp32 activations x fp16 weights), the KV cache is fp16 (config 3; reference default is fp32)."""
from __future__ import annotations
import os
import ctypes
from dataclasses import dataclass
import numpy as np
from tinygrad_amd import runtime as rt
from tinygrad_amd.runtime import Buffer, GGML_QUANT
from tinygrad_amd.nn import QuantLinear, ExpertWeights, qlinear_multi, qlinear_mixed, moe_gate, moe_combine, moe_router, expert_jobs, experts_grouped

@dataclass(frozen=True)
class TransformerConfig:
  """Subset of the reference's TransformerConfig (tinygrad/llm/model.py:52-82) the dense path reads."""
  num_blocks: int
  dim: int
  hidden_dim: int
  n_heads: int
  n_kv_heads: int
  norm_eps: float
  vocab_size: int
  head_dim: int
  rope_theta: float
  max_context: int
  qk_norm: int = 0                 # width of attn_q_norm / attn_k_norm (OLMoE: the full projection width, model.py:169; Qwen3: head_dim, :180)
  num_experts: int = 0
  num_experts_per_tok: int = 0
  norm_topk_prob: bool = False
  expert_gating_func: int = 1      # ExpertGating.SOFTMAX (model.py:9-13)
  routed_scaling_factor: float = 1.0
  rope_dim: int = 0                # rotated leading values of a head (model.py:63, 180-181); 0 = head_dim
  leading_dense_blocks: int = 0    # the first blocks of an MoE model that keep a dense FFN of width dense_hidden_dim (model.py:84, 441)
  dense_hidden_dim: int = 0
  shared_expert_dim: int = 0       # width of the always-on shared expert FFN added to the routed sum (model.py:99-103, 131-134); 0 = none
  shared_expert_gate: bool = False # the shared expert's output is scaled by sigmoid(x . ffn_gate_inp_shexp) (model.py:133)
  expert_bias: bool = False        # exp_probs_b: experts are ranked by score + bias, weighted by the score (model.py:113, 123)

  @property
  def n_summands(self) -> int:     # rows of the weighted sum a MoE block leaves: the routed experts and the shared expert
    return self.num_experts_per_tok + (1 if self.shared_expert_dim else 0)

LLAMA3_8B = dict(num_blocks=32, dim=4096, hidden_dim=14336, n_heads=32, n_kv_heads=8, norm_eps=1e-5, vocab_size=128256,
                 head_dim=128, rope_theta=500000.0)

# OLMoE architecture of benchmark configuration 4 (hidden_dim is the expert FFN width, as expert_feed_forward_length maps in model.py:422)
OLMOE = dict(num_blocks=16, dim=2048, hidden_dim=1024, n_heads=16, n_kv_heads=16, norm_eps=1e-5, vocab_size=50304, head_dim=128,
             rope_theta=10000.0, qk_norm=2048, num_experts=64, num_experts_per_tok=8, norm_topk_prob=False, expert_gating_func=1)

def precompute_freqs_cis(dim: int, end: int, theta: float) -> np.ndarray:
  """tinygrad/llm/model.py:16-19 in float32: cat(cos(pos * f), sin(pos * f)), f = 1 / theta^(2i/dim)."""
  freqs = (np.float32(1.0) / (np.float32(theta) ** (np.arange(0, dim, 2, dtype=np.float32)[:dim // 2] / np.float32(dim)))).astype(np.float32)
  ang = (np.arange(end, dtype=np.float32)[:, None] * freqs[None, :]).astype(np.float32)
  return np.concatenate([np.cos(ang), np.sin(ang)], axis=-1).astype(np.float32)

def partial_rope_order(head_dim: int, rope_dim: int) -> np.ndarray:
  """Order of a head's values that turns the reference's partial rotation (pairs (i, i + rope_dim/2) of the first rope_dim values, the rest untouched,
  model.py:180-181) into a rotation over pairs (i, i + head_dim/2) whose trailing pairs are identities: rotated first halves, first half of the
  untouched values, rotated second halves, second half of the untouched values.  q and k (rows, biases, norm weights) take the same order, so
  every q . k is unchanged."""
  rh, rest = rope_dim // 2, (head_dim - rope_dim) // 2
  return np.concatenate([np.arange(rh), rope_dim + np.arange(rest), rh + np.arange(rh), rope_dim + rest + np.arange(rest)])

def rope_table(head_dim: int, rope_dim: int, end: int, theta: float) -> np.ndarray:
  """[end][head_dim] rotation rows (cos half | sin half); with rope_dim < head_dim the frequencies are those of rope_dim (model.py:204) and the
  trailing pairs of partial_rope_order get cos 1, sin 0."""
  fc = precompute_freqs_cis(rope_dim, end, theta)
  if rope_dim == head_dim: return fc
  rh, rest = rope_dim // 2, (head_dim - rope_dim) // 2
  return np.concatenate([fc[:, :rh], np.ones((end, rest), np.float32), fc[:, rh:], np.zeros((end, rest), np.float32)], axis=-1)

def fast_k(ggml_type: int, k: int) -> bool:
  """Rows of k values of this type are inside the range of the single-row kernel that keeps the activations in registers: whole blocks, whole units of 64,
  at most 65536 values (32768 for the types whose lookup tables share the LDS with the row)."""
  nel = GGML_QUANT.get(ggml_type, (64, 128))[0]
  return k % 64 == 0 and k % nel == 0 and k <= (32768 if ggml_type in (rt.IQ3_XXS, rt.IQ3_S, rt.IQ2_S, rt.Q1_0) else 65536)

def quant_nbytes(ggml_type: int, n: int) -> int:
  if ggml_type == rt.F32: return 4 * n
  if ggml_type == rt.F16: return 2 * n
  nel, nby = GGML_QUANT[ggml_type]
  return n // nel * nby

def synth_state_moe(config: TransformerConfig, seed: int = 1004, dense_type: int = rt.F16, expert_type: int = rt.MXFP4, stream=None) -> dict:
  """OLMoE-architecture random model: fp16 attention / router / embedding / lm-head, MXFP4 expert stacks (E, out, in), norms 1.  The config's
  leading dense blocks, shared expert (with or without its sigmoid gate) and expert selection bias are written when it asks for them."""
  c, sd, tid = config, {}, [0]
  def mk(name, shape, t, amp):
    n = int(np.prod(shape))
    buf = Buffer((quant_nbytes(t, n),), np.uint8)
    tid[0] += 1
    rt.check(rt.lib().tga_synth_weights(t, buf.ptr, n, (seed * 7919 + tid[0]) & 0xFFFFFFFF, amp, stream))
    sd[name] = (buf, t, tuple(shape))
  E, H, D = c.num_experts, c.hidden_dim, c.dim
  mk("token_embd.weight", (c.vocab_size, D), dense_type, 1.0)
  for i in range(c.num_blocks):
    p = f"blk.{i}."
    mk(p + "attn_norm.weight", (1, D), rt.F32, 1.0)
    for nm, rows in (("attn_q", c.n_heads * c.head_dim), ("attn_k", c.n_kv_heads * c.head_dim), ("attn_v", c.n_kv_heads * c.head_dim)):
      mk(p + nm + ".weight", (rows, D), dense_type, D ** -0.5)
    mk(p + "attn_output.weight", (D, c.n_heads * c.head_dim), dense_type, (c.n_heads * c.head_dim) ** -0.5)
    if c.qk_norm:
      mk(p + "attn_q_norm.weight", (1, c.n_heads * c.head_dim), rt.F32, 1.0)
      mk(p + "attn_k_norm.weight", (1, c.n_kv_heads * c.head_dim), rt.F32, 1.0)
    mk(p + "ffn_norm.weight", (1, D), rt.F32, 1.0)
    if i < c.leading_dense_blocks:
      Hd = c.dense_hidden_dim
      mk(p + "ffn_gate.weight", (Hd, D), dense_type, D ** -0.5); mk(p + "ffn_up.weight", (Hd, D), dense_type, D ** -0.5); mk(p + "ffn_down.weight", (D, Hd), dense_type, Hd ** -0.5)
      continue
    mk(p + "ffn_gate_inp.weight", (E, D), dense_type, D ** -0.5)
    mk(p + "ffn_gate_exps.weight", (E, H, D), expert_type, D ** -0.5)
    mk(p + "ffn_up_exps.weight", (E, H, D), expert_type, D ** -0.5)
    mk(p + "ffn_down_exps.weight", (E, D, H), expert_type, H ** -0.5)
    if c.shared_expert_dim:
      Hs = c.shared_expert_dim
      mk(p + "ffn_gate_shexp.weight", (Hs, D), dense_type, D ** -0.5); mk(p + "ffn_up_shexp.weight", (Hs, D), dense_type, D ** -0.5); mk(p + "ffn_down_shexp.weight", (D, Hs), dense_type, Hs ** -0.5)
      if c.shared_expert_gate: mk(p + "ffn_gate_inp_shexp.weight", (1, D), dense_type, D ** -0.5)
    if c.expert_bias:                                                    # float32 holding fp16 values, like every tensor the reference loads (model.py:376)
      bias = np.random.default_rng(seed * 31 + i).uniform(-0.3, 0.3, E).astype(np.float16).astype(np.float32)
      sd[p + "exp_probs_b.bias"] = (Buffer.from_numpy(bias), rt.F32, (1, E))
  mk("output_norm.weight", (1, D), rt.F32, 1.0)
  mk("output.weight", (c.vocab_size, D), dense_type, D ** -0.5)
  return sd

def synth_state(config: TransformerConfig, seed: int = 1003, linear_type: int = rt.Q4_0, head_type: int = rt.Q6_K, stream=None,
                q4_k_m: bool = False) -> dict:
  """Random-init model written straight into HBM as GGUF blocks: {gguf tensor name: (Buffer, ggml_type, (rows, cols))}.
  Linear and embedding weights ~ U(-1/sqrt(in), 1/sqrt(in)) quantized to linear_type, lm-head to head_type, norm weights 1.
  q4_k_m: the tensor-type mix of a Q4_K_M file - Q4_K everywhere except attn_v / ffn_down, which are Q6_K in the first and last eighth
  of the blocks and in every third block between (llama.cpp's use_more_bits rule), else Q4_K."""
  c, sd, tid = config, {}, [0]
  if q4_k_m: linear_type = rt.Q4_K
  def more_bits(i): n = c.num_blocks; return i < n // 8 or i >= 7 * n // 8 or (i - n // 8) % 3 == 2
  def mk(name, rows, cols, t, amp):
    buf = Buffer((quant_nbytes(t, rows * cols),), np.uint8)
    tid[0] += 1
    rt.check(rt.lib().tga_synth_weights(t, buf.ptr, rows * cols, (seed * 7919 + tid[0]) & 0xFFFFFFFF, amp, stream))
    sd[name] = (buf, t, (rows, cols))
  mk("token_embd.weight", c.vocab_size, c.dim, linear_type, 1.0)
  for i in range(c.num_blocks):
    p = f"blk.{i}."
    mk(p + "attn_norm.weight", 1, c.dim, rt.F32, 1.0)
    mk(p + "attn_q.weight", c.n_heads * c.head_dim, c.dim, linear_type, c.dim ** -0.5)
    mk(p + "attn_k.weight", c.n_kv_heads * c.head_dim, c.dim, linear_type, c.dim ** -0.5)
    vd_type = rt.Q6_K if (q4_k_m and more_bits(i)) else linear_type
    mk(p + "attn_v.weight", c.n_kv_heads * c.head_dim, c.dim, vd_type, c.dim ** -0.5)
    mk(p + "attn_output.weight", c.dim, c.n_heads * c.head_dim, linear_type, (c.n_heads * c.head_dim) ** -0.5)
    mk(p + "ffn_norm.weight", 1, c.dim, rt.F32, 1.0)
    mk(p + "ffn_gate.weight", c.hidden_dim, c.dim, linear_type, c.dim ** -0.5)
    mk(p + "ffn_up.weight", c.hidden_dim, c.dim, linear_type, c.dim ** -0.5)
    mk(p + "ffn_down.weight", c.dim, c.hidden_dim, vd_type, c.hidden_dim ** -0.5)
  mk("output_norm.weight", 1, c.dim, rt.F32, 1.0)
  mk("output.weight", c.vocab_size, c.dim, head_type, c.dim ** -0.5)
  return sd

def _to_f32(data: np.ndarray, typ: int) -> np.ndarray:
  raw = np.ascontiguousarray(data).view(np.uint8)
  if typ == rt.F32: return raw.view(np.float32)
  if typ == rt.F16: return raw.view(np.float16).astype(np.float32)
  if typ == 30: return (raw.view(np.uint16).astype(np.uint32) << 16).view(np.float32)      # bfloat16
  raise NotImplementedError(f"ggml type {typ} for a norm / dense tensor")

class _Consumed(dict):
  """A state dict that remembers which tensors the model took."""
  def __init__(self, *a):
    super().__init__(*a); self.used = set()
  def __getitem__(self, k):
    self.used.add(k); return super().__getitem__(k)
  def get(self, k, default=None):
    if k in self: self.used.add(k)
    return super().get(k, default)

class TransformerBlock:
  """One decode step of the reference's TransformerBlock/FFNBlock (tinygrad/llm/model.py:144-204) for batch 1."""
  def __init__(self, config: TransformerConfig, sd: dict, i: int, shared):
    c, p = config, f"blk.{i}."
    lin = lambda name: QuantLinear(sd[p + name][0], sd[p + name][1], *sd[p + name][2])
    self.attn_norm, self.ffn_norm = sd[p + "attn_norm.weight"][0], sd[p + "ffn_norm.weight"][0]
    self.attn_q, self.attn_k, self.attn_v, self.attn_output = lin("attn_q.weight"), lin("attn_k.weight"), lin("attn_v.weight"), lin("attn_output.weight")
    self.moe = c.num_experts > 0 and i >= c.leading_dense_blocks       # leading blocks of an MoE model are dense (model.py:84)
    if self.moe:
      ex = lambda name: ExpertWeights(sd[p + name][0], sd[p + name][1], *sd[p + name][2])
      self.ffn_gate_inp = lin("ffn_gate_inp.weight")                      # router
      self.ffn_gate_exps, self.ffn_up_exps, self.ffn_down_exps = ex("ffn_gate_exps.weight"), ex("ffn_up_exps.weight"), ex("ffn_down_exps.weight")
      self.sel_bias = sd[p + "exp_probs_b.bias"][0] if c.expert_bias else None       # float32 (n_experts,)
      self.shared = c.shared_expert_dim > 0
      if self.shared:
        self.sh_gate, self.sh_up, self.sh_down = lin("ffn_gate_shexp.weight"), lin("ffn_up_shexp.weight"), lin("ffn_down_shexp.weight")
        self.sh_gate_inp = lin("ffn_gate_inp_shexp.weight") if c.shared_expert_gate else None     # (1, dim)
        if self.sh_gate.ggml_type != self.sh_up.ggml_type: raise NotImplementedError("ffn_gate_shexp and ffn_up_shexp of different ggml types are not built")
    else:
      self.ffn_gate, self.ffn_up, self.ffn_down = lin("ffn_gate.weight"), lin("ffn_up.weight"), lin("ffn_down.weight")
    # Linear(bias=config.qkv_bias) of model.py:161-163: the float32 bias rows enter the q / k / v launch as its additive row
    self.qkv_bias = [sd[p + f"attn_{n}.bias"][0] for n in "qkv"] if p + "attn_q.bias" in sd else None
    self.q_norm = sd[p + "attn_q_norm.weight"][0] if c.qk_norm else None
    self.k_norm = sd[p + "attn_k_norm.weight"][0] if c.qk_norm else None
    # KV cache: fp16 [n_kv_heads][max_context][head_dim] each (reference: one [2,B,KvH,ctx,Hd] tensor, model.py:202)
    self.cache_k = Buffer((c.n_kv_heads, c.max_context, c.head_dim), np.float16).zero_()
    self.cache_v = Buffer((c.n_kv_heads, c.max_context, c.head_dim), np.float16).zero_()
    self.config, self.s = c, shared
    # the M = 1 GEMV's register-resident fast path: K % 64 (superblock types: % 256), 4-byte aligned weights
    fast = lambda l: fast_k(l.ggml_type, l.in_features) and l.blocks.ptr % 4 == 0
    # RMSNorm folded into the consuming linear
    self.fuse_norm = all(fast(l) for l in (self.attn_q, self.attn_k, self.attn_v)) and (self.moe or all(fast(l) for l in (self.ffn_gate, self.ffn_up)))
    # a producer with a single consumer writes its fp16 output in the order that consumer's GEMV reads it (no LDS staging there):
    # attention -> attn_output, SwiGLU -> ffn_down, and the unfused ffn_norm -> ffn_gate / ffn_up
    self.stage_attn = fast(self.attn_output)
    self.stage_act = (not self.moe) and fast(self.ffn_down)
    self.stage_xn = (not self.moe) and fast(self.ffn_gate) and self.ffn_gate.ggml_type == self.ffn_up.ggml_type
    self.stage_sh = self.moe and self.shared and fast(self.sh_down)
    # the expert gate/up launch can gate for itself: one fp16 row of at most 4096 values on one wave per row team
    self.route_in_experts = self.moe and self.sel_bias is None and c.dim <= 4096 and c.dim % 64 == 0 and c.num_experts <= 1024 and c.num_experts_per_tok <= 64 \
                            and (c.dim // (32 if self.ffn_gate_exps.ggml_type == rt.MXFP4 else 64)) <= 64
    # the previous block's weighted expert sum can be completed inside this block's q/k/v launch (one 8-value piece per thread: dim <= 2048)
    self.can_fold_combine = self.fuse_norm and self.attn_q.ggml_type == self.attn_k.ggml_type == self.attn_v.ggml_type and c.dim <= 2048 \
                            and 0 < c.n_summands <= 8 and self.qkv_bias is None
    # ffn_gate and ffn_up of different block types: two launches and an elementwise silu(gate) * up instead of one launch with the SwiGLU epilogue
    self.split_gate_up = not self.moe and self.ffn_gate.ggml_type != self.ffn_up.ggml_type
    if self.split_gate_up:
      self.stage_act = False
      if not hasattr(shared, "gate32"): shared.gate32, shared.up32 = (Buffer((1, max(c.hidden_dim, c.dense_hidden_dim)), np.float32) for _ in range(2))
    # The attention as one launch whose split partials attn_output merges (cache of at most six splits, attn_output rows of at most 64 units; the q / k norm inside the launch)
    ns = ctypes.c_int(0)
    rt.check(rt.lib().tga_attention_split_plan(c.max_context, ctypes.byref(ns)))
    ao = self.attn_output
    self.fused_attn = ns.value if (os.environ.get("TGA_ATTN", "fused") == "fused" and fast(ao) and ao.ggml_type != rt.MXFP4
                                   and 512 <= ao.in_features <= 4096 and ao.in_features == c.n_heads * c.head_dim) else 0
    self.kv_touch = os.environ.get("TGA_KV_TOUCH", "1") == "1" and c.n_kv_heads % 8 == 0      # the q / k / v launch touches the cache rows for the attention launch

  def __call__(self, x: Buffer, stream, pending: int = 0, defer: bool = False) -> tuple[Buffer, int]:
    """One block on the residual row x.  pending > 0: the previous (MoE) block left its weighted sum over that many rows + residual to this block
    (expert outputs in s.y_e, weights in s.probs).  defer: leave this block's own weighted sum to the next launch.  Returns the buffer
    that holds the residual row afterwards and whether a weighted sum is still pending."""
    c, s, L = self.config, self.s, rt.lib()
    # h = x + attention(attn_norm(x))                                                     model.py:149
    qkv, qkv_out = [self.attn_q, self.attn_k, self.attn_v], [s.q, s.k, s.v]
    if pending and not self.can_fold_combine:
      moe_combine(s.y_e, s.probs, x, 1, pending, c.dim, x, stream=stream); pending = 0
    if pending:                                                          # x + sum_j probs_j y_j completed inside the q/k/v launch, written to the other row buffer
      x_new = s.x2 if x.ptr == s.x.ptr else s.x
      qlinear_multi(qkv, x, qkv_out, stream=stream, norm=(self.attn_norm, c.norm_eps), combine=(s.y_e, s.probs, pending, x_new))
      x = x_new
    else:
      # one launch per run of equal block types (e.g. Q4_K q / k with a Q6_K v: two launches); each normalises the row while staging it
      # when the fast path allows, else one RMSNorm launch feeds them
      if not self.fuse_norm: rt.check(L.tga_rmsnorm(x.ptr, self.attn_norm.ptr, c.dim, c.norm_eps, s.xn.ptr, None, 0, stream))
      i = 0
      if self.fuse_norm and self.qkv_bias is None and len({l.ggml_type for l in qkv}) > 1:      # (the call shares one launch between two runs where it can)
        qlinear_mixed(qkv, x, qkv_out, norm=(self.attn_norm, c.norm_eps), stream=stream); i = 3
      while i < 3:
        j = i + 1
        while j < 3 and qkv[j].ggml_type == qkv[i].ggml_type: j += 1
        bias = dict(epilogue=1, resid=self.qkv_bias[i:j]) if self.qkv_bias is not None else {}
        touch = (s.state, self.cache_k, self.cache_v, s.rope, c.n_kv_heads, c.head_dim, c.max_context) if (self.kv_touch and j == 3) else None
        if self.fuse_norm: qlinear_multi(qkv[i:j], x, qkv_out[i:j], stream=stream, norm=(self.attn_norm, c.norm_eps), touch=touch, **bias)
        else: qlinear_multi(qkv[i:j], s.xn, qkv_out[i:j], stream=stream, **bias)
        i = j
    # q/k RMSNorm inside the attention launch: full-width before the head split (model.py:169) or per head after it (model.py:180)
    if self.fused_attn:
      # one launch leaves split partials, attn_output merges them while it stages its row (no merge launch)
      rt.check(L.tga_attention_decode_split_normed(s.q.ptr, s.k.ptr, s.v.ptr, self.q_norm.ptr if c.qk_norm else None, self.k_norm.ptr if c.qk_norm else None, c.norm_eps,
                                                   int(c.qk_norm == c.head_dim), self.cache_k.ptr, self.cache_v.ptr, s.attn_part.ptr, s.state.ptr, c.n_heads, c.n_kv_heads, c.head_dim,
                                                   c.max_context, s.rope.ptr, stream))
      ao = self.attn_output
      rt.check(L.tga_attn_merge_qlinear(ao.ggml_type, ao.blocks.ptr, x.ptr, ao.out_features, ao.in_features, x.ptr, s.attn_part.ptr, self.fused_attn, c.head_dim, stream))
    else:
      rt.check(L.tga_attention_decode_normed(s.q.ptr, s.k.ptr, s.v.ptr, self.q_norm.ptr if c.qk_norm else None, self.k_norm.ptr if c.qk_norm else None, c.norm_eps,
                                             int(c.qk_norm == c.head_dim), self.cache_k.ptr, self.cache_v.ptr, s.attn_part.ptr, s.state.ptr, c.n_heads, c.n_kv_heads, c.head_dim, c.max_context,
                                             s.rope.ptr, s.attn.ptr, None, self.attn_output.ggml_type if self.stage_attn else 0, stream))
      qlinear_multi([self.attn_output], s.attn, [x], epilogue=1, resid=[x], stream=stream, x_staged=self.stage_attn)
    # x = h + ffn_down(silu(ffn_gate(n)) * ffn_up(n)), n = ffn_norm(h)                     model.py:137,150
    if not self.moe:
      if self.split_gate_up:
        rt.check(L.tga_rmsnorm(x.ptr, self.ffn_norm.ptr, c.dim, c.norm_eps, s.xn.ptr, None, 0, stream))
        h = self.ffn_gate.out_features
        g32, u32 = s.gate32.view(0, (1, h), np.float32), s.up32.view(0, (1, h), np.float32)
        self.ffn_gate(s.xn, out=g32, stream=stream); self.ffn_up(s.xn, out=u32, stream=stream)
        rt.check(L.tga_silu_mul(g32.ptr, u32.ptr, h, s.act.ptr, stream))
      elif self.fuse_norm:
        qlinear_multi([self.ffn_gate, self.ffn_up], x, [s.act], epilogue=2, stream=stream, norm=(self.ffn_norm, c.norm_eps), stage_out_for=self.ffn_down if self.stage_act else None)
      else:
        rt.check(L.tga_rmsnorm(x.ptr, self.ffn_norm.ptr, c.dim, c.norm_eps, s.xn.ptr, None, self.ffn_gate.ggml_type if self.stage_xn else 0, stream))
        qlinear_multi([self.ffn_gate, self.ffn_up], s.xn, [s.act], epilogue=2, stream=stream, x_staged=self.stage_xn, stage_out_for=self.ffn_down if self.stage_act else None)
      qlinear_multi([self.ffn_down], s.act, [x], epilogue=1, resid=[x], stream=stream, x_staged=self.stage_act)
      return x, 0
    # MoE feed-forward (model.py:110-135): router -> gating + pairwise top-k -> selected experts' SwiGLU -> weighted sum (+ residual)
    k = c.num_experts_per_tok
    one_launch_router = self.ffn_gate_inp.ggml_type == rt.F16 and c.dim % 8 == 0 and c.dim <= 16384 and c.num_experts <= 1024
    if one_launch_router and self.route_in_experts:
      # router logits only; the expert gate/up launch gates for itself (scores, top-k, weights) and writes sel / probs for the launches after it
      moe_router(x, self.ffn_norm, c.norm_eps, self.ffn_gate_inp, 0, None, None, s.router, xn_out=s.xn, stream=stream)
      self.ffn_gate_exps(s.sel, s.xn, s.act_e, jobs_per_x_row=k, up=self.ffn_up_exps, stream=stream,
                         route=(s.router, c.expert_gating_func, c.norm_topk_prob, c.routed_scaling_factor, s.probs))
    else:
      if one_launch_router and self.sel_bias is not None:                # logits in one launch, then the gating with the selection bias
        moe_router(x, self.ffn_norm, c.norm_eps, self.ffn_gate_inp, 0, None, None, s.router, xn_out=s.xn, stream=stream)
        moe_gate(s.router.view(0, (1, c.num_experts), np.float32), 1, c.num_experts, k, s.sel, s.probs, c.expert_gating_func, c.norm_topk_prob,
                 c.routed_scaling_factor, stream=stream, bias=self.sel_bias)
      elif one_launch_router:
        moe_router(x, self.ffn_norm, c.norm_eps, self.ffn_gate_inp, k, s.sel, s.probs, s.router, xn_out=s.xn, gating=c.expert_gating_func,
                   norm_topk_prob=c.norm_topk_prob, scale=c.routed_scaling_factor, stream=stream)
      else:
        rt.check(L.tga_rmsnorm(x.ptr, self.ffn_norm.ptr, c.dim, c.norm_eps, s.xn.ptr, None, 0, stream))
        lg = s.router.view(0, (1, c.num_experts), np.float32)
        self.ffn_gate_inp(s.xn, out=lg, stream=stream)
        moe_gate(lg, 1, c.num_experts, k, s.sel, s.probs, c.expert_gating_func, c.norm_topk_prob, c.routed_scaling_factor, stream=stream, bias=self.sel_bias)
      self.ffn_gate_exps(s.sel, s.xn, s.act_e, jobs_per_x_row=k, up=self.ffn_up_exps, stream=stream)      # silu(gate_e x) * (up_e x) per slot
    self.ffn_down_exps(s.sel, s.act_e, s.y_e, jobs_per_x_row=1, stream=stream)
    n_sum = k
    if self.shared:
      # the shared expert (model.py:131-134) is one more row of the weighted sum: its output goes to row k of y_e, its weight (1, or the
      # sigmoid gate) to probs[k]
      qlinear_multi([self.sh_gate, self.sh_up], s.xn, [s.act_sh], epilogue=2, stream=stream, stage_out_for=self.sh_down if self.stage_sh else None)
      qlinear_multi([self.sh_down], s.act_sh, [s.y_sh], stream=stream, x_staged=self.stage_sh)
      if self.sh_gate_inp is not None:
        self.sh_gate_inp(s.xn, out=s.sh_logit, stream=stream)
        moe_gate(s.sh_logit, 1, 1, 1, s.sh_sel, s.p_sh, 2, False, 1.0, stream=stream)     # sigmoid of the one logit
      n_sum = k + 1
    if defer: return x, n_sum                                           # the consumer of the completed row adds sum_j probs_j y_j + x itself
    moe_combine(s.y_e, s.probs, x, 1, n_sum, c.dim, x, stream=stream)
    return x, 0

class _Shared:
  """Activation buffers shared by all blocks (batch 1)."""
  def __init__(self, c: TransformerConfig, max_new: int):
    f32, f16 = np.float32, np.float16
    self.state = Buffer((16,), np.int32).zero_()
    self.x = Buffer((1, c.dim), f32)
    self.x2 = Buffer((1, c.dim), f32)                                    # second residual row: a launch that completes x + sum_j p_j y_j writes here
    self.xn = Buffer((1, c.dim), f16)
    nq, nkv = c.n_heads * c.head_dim, c.n_kv_heads * c.head_dim
    self.qkv = Buffer((1, nq + 2 * nkv), f32)                          # q | k | v
    self.q, self.k, self.v = self.qkv.view(0, (1, nq), f32), self.qkv.view(4 * nq, (1, nkv), f32), self.qkv.view(4 * (nq + nkv), (1, nkv), f32)
    self.attn = Buffer((1, c.n_heads * c.head_dim), f16)
    self.attn_part = Buffer((c.n_heads * max(((c.max_context + 63) // 64) * (c.head_dim + 2), 6 * c.head_dim + 16),), f32).zero_()   # (two-launch layout or up to six split partials + their (max, sum) pairs)
    self.act = Buffer((1, max(c.hidden_dim, c.dense_hidden_dim)), f16)
    if c.num_experts:
      k = c.num_experts_per_tok
      self.router, self.sel = Buffer((1, c.num_experts + 1), f32).zero_(), Buffer((k,), np.int32)     # logits + arrival counter
      self.probs = Buffer.from_numpy(np.ones(k + 1, dtype=f32))           # k routed weights + the shared expert's (1 unless it is gated)
      self.act_e, self.y_e = Buffer((k, c.hidden_dim), f16), Buffer((k + 1, c.dim), f32)
      self.y_sh, self.p_sh = self.y_e.view(4 * k * c.dim, (1, c.dim), f32), self.probs.view(4 * k, (1,), f32)
      self.act_sh = Buffer((1, max(1, c.shared_expert_dim)), f16)
      self.sh_logit, self.sh_sel = Buffer((1, 1), f32), Buffer((1,), np.int32)
    self.logits = Buffer((1, c.vocab_size), f32)
    self.am_v, self.am_i = Buffer((256,), f32), Buffer((256,), np.int32)
    self.rope = Buffer.from_numpy(rope_table(c.head_dim, c.rope_dim or c.head_dim, c.max_context, c.rope_theta))
    self.prompt = Buffer((c.max_context,), np.int32).zero_()
    self.out_tokens = Buffer((max(1, max_new),), np.int32).zero_()

class Transformer:
  def __init__(self, config: TransformerConfig, state_dict: dict, max_new: int = 4096):
    """One launch per op (six per dense block, seven per MoE block; attention is two), captured once per token kind and replayed."""
    self.config = c = config
    self.s = _Shared(c, max_new)
    self.max_new = max_new
    emb = state_dict["token_embd.weight"]
    self.token_embd, self.embd_type = emb[0], emb[1]
    self.blk = [TransformerBlock(c, state_dict, i, self.s) for i in range(c.num_blocks)]
    self.output_norm = state_dict["output_norm.weight"][0]
    out = state_dict.get("output.weight", emb)                       # tied embeddings: model.py:379
    self.output = QuantLinear(out[0], out[1], *out[2])
    self.fuse_head_norm = fast_k(out[1], c.dim) and out[0].ptr % 4 == 0
    self.can_fold_head = self.fuse_head_norm and c.dim <= 2048 and 0 < c.n_summands <= 8
    self.stream = rt.Stream()
    self._graphs = {}
    self._n_prompt, self._steps_done = 0, 0                          # host mirror of the device-side position bookkeeping (for the context guard)
    self._cached_tokens, self._last_input, self.prefill_steps = [], None, 0   # tokens whose K / V rows the cache holds (KV-prefix reuse, model.py:455-462)
    self.replay = "cmdlist"                                          # how a captured step is replayed: "cmdlist" (plain launches in capture order) or "graph" (hipGraphLaunch)
    self._state_dict, self._chunker, self._tail_chunkers = state_dict, None, {}   # (references to the weight buffers: the chunked prefill builds its linears over the same bytes)
    self.prefill_chunk = 128                                         # prompt positions per prefill step, 2..128 (the reference's chunks hold 32, model.py:464; MoE models: at most 16); 1: token by token

  def check_state(self):
    """Raises when a kernel of the last steps refused its input (state.error: bit 0 = a token id outside the vocabulary reached the embedding
    lookup, bit 1 = a position at or beyond max_context reached the attention launch).  The kernels clamp / skip instead of faulting."""
    err = int(self.s.state.numpy()[4])
    if err:
      st = self.s.state.numpy(); st[4] = 0; self.s.state.copyin(st)
      raise RuntimeError(f"decode state error {err}: " + ", ".join(m for b, m in ((1, "token id outside the vocabulary"), (2, "position beyond max_context")) if err & b))

  # one token through all blocks; with_head adds output_norm + output + argmax (model.py:358-364)
  def _step(self, with_head: bool, on_block=None):
    """The launches of one token.  on_block(i): called when block i's launches have been issued (eager stepping only; e.g. to read back s.sel, the
    experts block i selected, after a synchronisation)."""
    c, s, L, st = self.config, self.s, rt.lib(), self.stream.handle
    rt.check(L.tga_embed_row(self.token_embd.ptr, self.embd_type, c.dim, s.state.ptr, s.x.ptr, st))
    x, pending = s.x, 0
    nb = len(self.blk)
    for i, b in enumerate(self.blk):
      nxt = self.blk[i + 1].can_fold_combine if i + 1 < nb else (with_head and self.can_fold_head)
      x, pending = b(x, st, pending, defer=nxt)
      if on_block is not None: on_block(i)
    if with_head:
      if pending:                                                      # the last block's weighted sum completed inside the lm-head launch
        x_new = s.x2 if x.ptr == s.x.ptr else s.x
        qlinear_multi([self.output], x, [s.logits], stream=st, norm=(self.output_norm, c.norm_eps), combine=(s.y_e, s.probs, pending, x_new))
        x = x_new
      elif self.fuse_head_norm:                                        # output_norm inside the lm-head launch (model.py:362)
        qlinear_multi([self.output], x, [s.logits], stream=st, norm=(self.output_norm, c.norm_eps))
      else:
        rt.check(L.tga_rmsnorm(x.ptr, self.output_norm.ptr, c.dim, c.norm_eps, s.xn.ptr, None, 0, st))
        self.output(s.xn, out=s.logits, stream=st)
      rt.check(L.tga_argmax_step(s.logits.ptr, c.vocab_size, s.am_v.ptr, s.am_i.ptr, s.state.ptr, s.prompt.ptr, s.out_tokens.ptr, self.max_new, st))
    else:
      rt.check(L.tga_advance_prompt(s.state.ptr, s.prompt.ptr, st))

  def _graph(self, with_head: bool):
    if with_head not in self._graphs:
      g = (rt.CommandList if self.replay == "cmdlist" else rt.Graph)(self.stream)
      with g: self._step(with_head)
      self._graphs[with_head] = g
    return self._graphs[with_head]

  @staticmethod
  def from_gguf(gguf, max_context: int | None = None, max_new: int = 4096) -> tuple["Transformer", dict]:
    """Transformer.from_gguf (tinygrad/llm/model.py:370-451) for the architectures on the path (dense llama-family and MoE with
    qk-norm).  Weights stay in their GGUF blocks on the device; F32 / BF16 matrices are cast to fp16 on the host (the reference
    casts every weight to fp16, model.py:376); for arch == 'llama' the rows of attn_q / attn_k are permuted from the interleaved
    to the half-split RoPE layout (model.py:409-419) by moving whole block rows."""
    from tinygrad_amd.gguf import gguf_load, ggml_data_to_tensor, GGUF_F32_LIKE
    kv, ts = gguf_load(gguf)
    arch = kv["general.architecture"]
    ctx = kv[f"{arch}.context_length"]
    max_context = min(max_context, ctx) if max_context is not None else ctx
    n_heads, n_kv = kv[f"{arch}.attention.head_count"], kv[f"{arch}.attention.head_count_kv"]
    dim = kv[f"{arch}.embedding_length"]
    head_dim = kv.get(f"{arch}.attention.key_length_mla", kv.get(f"{arch}.attention.key_length", dim // n_heads))
    num_blocks = kv[f"{arch}.block_count"] - kv.get(f"{arch}.nextn_predict_layers", 0)     # trailing next-token-prediction layers are not part of the decoder (model.py:424)
    rope_dim = kv.get(f"{arch}.rope.dimension_count", head_dim)
    v_head_dim = kv.get(f"{arch}.attention.value_length_mla", kv.get(f"{arch}.attention.value_length", head_dim))     # model.py from_gguf: v_head_dim
    if v_head_dim != head_dim: raise NotImplementedError(f"value heads of {v_head_dim} values beside key heads of {head_dim} are not built")
    if rope_dim != head_dim and (arch == "llama" or rope_dim % 2 or (head_dim - rope_dim) % 2 or not 0 < rope_dim < head_dim):
      raise NotImplementedError(f"rope dimension {rope_dim} of head_dim {head_dim} for architecture {arch} is not built")
    if kv.get(f"{arch}.attention.kv_lora_rank", 0) or arch in ("qwen35", "qwen35moe", "kimi-linear"): raise NotImplementedError(f"architecture {arch} is outside the built path")
    sd = {}
    for name, t in ts.items():
      if name == "rope_freqs.weight": continue                         # unused by the reference too (model.py:446)
      if name.startswith("blk.") and int(name.split(".")[1]) >= num_blocks: continue     # next-token-prediction layers
      if arch == "glm4moe": name = name.replace("post_attention_norm", "ffn_norm")       # model.py:403-404
      rows, cols = (int(np.prod(t.shape[:-1])), t.shape[-1]) if len(t.shape) > 1 else (1, t.shape[0])
      typ, buf, data = t.ggml_type, t.buffer, t.data
      is_norm = name.endswith("_norm.weight") or name.endswith(".bias")
      if is_norm:                                                      # norm weights and biases: float32 rows holding the reference's fp16 values (model.py:376)
        data = _to_f32(data, typ).astype(np.float16).astype(np.float32); buf = Buffer.from_numpy(data.view(np.uint8)); typ = rt.F32
      elif typ in GGUF_F32_LIKE:                                       # F32 / BF16 matrices -> fp16 (model.py:376)
        data = _to_f32(data, typ).astype(np.float16); buf = Buffer.from_numpy(data.view(np.uint8)); typ = rt.F16
      if arch == "llama" and (name.endswith("attn_q.weight") or name.endswith("attn_k.weight")):
        h = n_heads if name.endswith("attn_q.weight") else n_kv
        raw = np.ascontiguousarray(data).view(np.uint8).reshape(rows, -1)
        per = rows // h
        idx = np.arange(rows).reshape(h, per // 2, 2).transpose(0, 2, 1).reshape(-1)   # "n (h two) d -> n (two h) d"
        buf = Buffer.from_numpy(np.ascontiguousarray(raw[idx]).reshape(-1))
      shape = (rows, cols) if len(t.shape) <= 2 else tuple(t.shape)
      if rope_dim != head_dim and name.split(".")[-2] in ("attn_q", "attn_k", "attn_q_norm", "attn_k_norm"):
        # partial rotary: reorder every head's rows (or per-value weights) so that the kernel's pairs (i, i + head_dim/2) are the reference's
        raw = np.ascontiguousarray(buf.numpy() if data is None else data).view(np.uint8).reshape(rows if len(t.shape) > 1 else cols, -1)
        idx = (np.arange(raw.shape[0]).reshape(-1, head_dim)[:, partial_rope_order(head_dim, rope_dim)]).reshape(-1)
        buf = Buffer.from_numpy(np.ascontiguousarray(raw[idx]).reshape(-1))
      sd[name] = (buf, typ, shape)
    if "output.weight" not in sd: sd["output.weight"] = sd["token_embd.weight"]        # tied embeddings, model.py:379
    config = TransformerConfig(
      num_blocks=num_blocks, dim=dim,
      hidden_dim=kv.get(f"{arch}.expert_feed_forward_length", kv.get(f"{arch}.feed_forward_length", 0)),
      n_heads=n_heads, n_kv_heads=n_kv, norm_eps=kv[f"{arch}.attention.layer_norm_rms_epsilon"], vocab_size=len(kv["tokenizer.ggml.tokens"]),
      head_dim=head_dim, rope_theta=kv[f"{arch}.rope.freq_base"], max_context=max_context,
      qk_norm=int(sd["blk.0.attn_q_norm.weight"][2][-1]) if "blk.0.attn_q_norm.weight" in sd else 0,
      num_experts=kv.get(f"{arch}.expert_count", 0), num_experts_per_tok=kv.get(f"{arch}.expert_used_count", 0),
      norm_topk_prob=kv.get(f"{arch}.expert_weights_norm", arch in ("qwen3moe",)),
      expert_gating_func=kv.get(f"{arch}.expert_gating_func", 1), routed_scaling_factor=kv.get(f"{arch}.expert_weights_scale", 1.0),
      rope_dim=rope_dim if rope_dim != head_dim else 0,
      leading_dense_blocks=(lead := kv.get(f"{arch}.leading_dense_block_count", 0)),
      dense_hidden_dim=kv.get(f"{arch}.feed_forward_length", 0) if lead else 0,
      shared_expert_dim=kv.get(f"{arch}.expert_shared_feed_forward_length", kv.get(f"{arch}.expert_shared_count", 0) * kv.get(f"{arch}.expert_feed_forward_length", 0)),
      shared_expert_gate=f"blk.{lead}.ffn_gate_inp_shexp.weight" in sd, expert_bias=f"blk.{lead}.exp_probs_b.bias" in sd)
    sd = _Consumed(sd)
    model = Transformer(config, sd, max_new=max_new)
    if (left := sorted(set(sd) - sd.used)):                            # nothing a file carries is silently dropped
      raise NotImplementedError(f"tensors the built path does not consume: {left[:8]}{' ...' if len(left) > 8 else ''}")
    return model, kv

  def get_start_pos(self, tokens: list[int]) -> int:
    """How many leading positions of the KV cache can be kept for this prompt (Transformer.get_start_pos, model.py:455-462): the longest common
    prefix of tokens[:-1] and the tokens whose keys and values the cache holds."""
    n = 0
    for a, b in zip(tokens[:-1], self._cached_tokens):
      if a != b: break
      n += 1
    return n

  def reset(self, tokens: list[int], start_pos: int = 0):
    """Start a sequence at position start_pos (the cache rows below it are kept): the prompt table, the position and the first input token."""
    c, s = self.config, self.s
    if not 1 <= len(tokens) < c.max_context: raise ValueError(f"prompt of {len(tokens)} tokens does not fit max_context {c.max_context}")
    if min(tokens) < 0 or max(tokens) >= c.vocab_size: raise ValueError(f"token id outside the vocabulary of {c.vocab_size}")
    if not 0 <= start_pos < len(tokens): raise ValueError(f"start position {start_pos} outside the prompt of {len(tokens)} tokens")
    prompt = np.zeros(c.max_context, dtype=np.int32); prompt[:len(tokens)] = tokens
    s.prompt.copyin(prompt)
    st = np.zeros(16, dtype=np.int32); st[0], st[1], st[3], st[5] = start_pos, tokens[start_pos], len(tokens), c.vocab_size
    s.state.copyin(st)
    self._n_prompt, self._steps_done = len(tokens), start_pos
    self._cached_tokens = list(tokens[:start_pos])

  def prefill(self, tokens: list[int], use_graph: bool = True, reuse_cache: bool = True, on_block=None):
    """Feeds all but the last prompt token (KV cache fill); the last one is consumed by the first decode step.  Like the reference's generate
    (model.py:472-473) the positions whose tokens equal what the cache already holds are not recomputed.  on_block: token by token with eager launches,
    on_block(i) after the launches of block i of every position (see _step)."""
    start = self.get_start_pos(tokens) if reuse_cache else 0
    self.prefill_steps = len(tokens) - 1 - start                        # (positions the last call actually computed)
    self._cached_tokens = self._cached_tokens[:start]                   # the rows from here on are about to be overwritten: if a step below raises, they are not claimed
    B = self.prefill_chunk if on_block is None else 1
    if B > 16 and self.config.num_experts: B = 16                       # (MoE blocks keep steps of sixteen positions: longer ones are not measured there)
    # Whole chunks as small-batch steps (model.py:476-481) of the largest size that the prompt holds (the chosen one, else 64, 32, 16, 8 or 4 positions).  Dense models: what
    # they leave is ONE more chunk that ends at the last position and computes some positions again - every row of a step depends on the cache and on its own token
    # only, so the same values are written again - instead of a ladder of smaller steps and up to three single ones (seven steps, a tenth of a 1023-position prefill).
    # MoE models keep the ladder (one step each of 8 and / or 4 positions, then single ones).
    overlap = not self.config.num_experts
    for b in [B] + [t for t in (64, 32, 16, 8, 4) if t < B]:
      total = len(tokens) - 1 - start
      if not 2 <= b <= 128 or total < b: continue
      if b == B:
        if self._chunker is None or self._chunker.batch != B: self._chunker = BatchedTransformer(self.config, self._state_dict, B, max_new=1, chunk_of=self)
        chunker = self._chunker
      else:
        if b not in self._tail_chunkers: self._tail_chunkers[b] = BatchedTransformer(self.config, self._state_dict, b, max_new=1, chunk_of=self)
        chunker = self._tail_chunkers[b]
      start += chunker.prefill_chunks(tokens, start, total // b, use_graph)
      if overlap:
        if start < len(tokens) - 1: chunker.prefill_chunks(tokens, len(tokens) - 1 - b, 1, use_graph); start = len(tokens) - 1
        break
    self.reset(tokens, start)
    for _ in range(len(tokens) - 1 - start):
      if use_graph and on_block is None: self._graph(False).launch()
      else: self._step(False, on_block)
    self._steps_done = len(tokens) - 1
    self._cached_tokens = list(tokens[:-1])
    self._last_input = tokens[-1]
    self.stream.synchronize()

  def decode_step(self, use_graph: bool = True, sync: bool = True, on_block=None):
    """One token.  The position it occupies must exist in the KV cache and the rotation table: like the reference's generate loop
    (`while len(tokens) < self.max_context`, tinygrad/llm/model.py:475) the sequence ends at max_context.  on_block: eager launches with that hook (see _step)."""
    if self._steps_done >= self.config.max_context: raise RuntimeError(f"context full: position {self._steps_done} is beyond max_context {self.config.max_context}")
    if use_graph and on_block is None: self._graph(True).launch()
    else: self._step(True, on_block)
    self._steps_done += 1
    self._cached_tokens.append(self._last_input); self._last_input = None    # this step wrote its input token's keys and values; the next input is on the device
    if sync: self.stream.synchronize()

  def generate(self, tokens: list[int], max_new_tokens: int, use_graph: bool = True):
    """Greedy decoding (temperature 0): yields one token id per step, like Transformer.generate (model.py:464-484), and like it stops when
    the context is full (model.py:475)."""
    self.prefill(tokens, use_graph)
    for i in range(min(max_new_tokens, self.config.max_context - len(tokens), self.max_new)):
      self.decode_step(use_graph, sync=True)                          # the reference syncs once per token too (out.item(), model.py:482)
      tok = int(self.s.out_tokens.view(4 * i, (1,), np.int32).numpy()[0])
      self._last_input = tok                                          # (model.py:483: the cache then holds tokens[:-1])
      yield tok
    self.check_state()

  def logits(self) -> np.ndarray: return self.s.logits.numpy().reshape(-1)

  def weight_bytes_per_token(self) -> int:
    """Packed weight bytes one decode step streams (all block linears + lm-head), the reference's GB/s accounting (cli.py:179-181)."""
    n = self.output.nbytes
    for b in self.blk:
      n += sum(l.nbytes for l in (b.attn_q, b.attn_k, b.attn_v, b.attn_output))
      if b.moe:
        n += b.ffn_gate_inp.nbytes + self.config.num_experts_per_tok * sum(e.expert_nbytes for e in (b.ffn_gate_exps, b.ffn_up_exps, b.ffn_down_exps))
        if b.shared: n += sum(l.nbytes for l in (b.sh_gate, b.sh_up, b.sh_down))
      else: n += sum(l.nbytes for l in (b.ffn_gate, b.ffn_up, b.ffn_down))
    return n


class BatchedTransformer:
  """2..8 sequences decoded in lockstep at one shared position: the reference's forward over a (B, 1) token batch (tinygrad/llm/model.py:358-364).
  Dense linears run as small-batch GEMMs over the GGUF blocks (M = B); in a MoE block the B * k (token, slot) jobs are grouped by expert, so an
  expert selected by several tokens is streamed once (ExpertWeights over a (B, T, k) selection, model.py:21-27, 110-135).  Same state dict and
  config as Transformer; every sequence has its own KV cache; prompts of one batch have equal length."""
  def __init__(self, config: TransformerConfig, state_dict: dict, batch: int, max_new: int = 1024, chunk_of: "Transformer | None" = None):
    """chunk_of: the rows are `batch` consecutive prompt positions of that Transformer's sequence instead of `batch` sequences (chunked prefill,
    model.py:464, 476-481): its KV caches and rotation table are used, the attention is causal inside the chunk, no token is sampled."""
    if not 1 <= batch <= (16 if chunk_of is None else 128): raise ValueError(f"batch of {batch} sequences is outside the decode range 1..16")
    self.config, self.batch, self.max_new = config, batch, max_new
    # (no reference back to the Transformer: a cycle would leave its buffers to the cycle collector, which may free them in the middle of a stream capture)
    self.chunked, self._owner_stream = chunk_of is not None, (chunk_of.stream if chunk_of is not None else None)
    c, B = config, batch
    f32, f16 = np.float32, np.float16
    lin = lambda name: QuantLinear(state_dict[name][0], state_dict[name][1], *state_dict[name][2])
    emb = state_dict["token_embd.weight"]
    self.token_embd, self.embd_type = emb[0], emb[1]
    self.output_norm = state_dict["output_norm.weight"][0]
    out = state_dict.get("output.weight", emb)
    self.output = QuantLinear(out[0], out[1], *out[2])
    self.blk = []
    nq, nkv = c.n_heads * c.head_dim, c.n_kv_heads * c.head_dim
    for i in range(c.num_blocks):
      p, b = f"blk.{i}.", {}
      for nm in ("attn_q", "attn_k", "attn_v", "attn_output"): b[nm] = lin(p + nm + ".weight")
      b["attn_norm"], b["ffn_norm"] = state_dict[p + "attn_norm.weight"][0], state_dict[p + "ffn_norm.weight"][0]
      b["q_norm"] = state_dict[p + "attn_q_norm.weight"][0] if c.qk_norm else None
      b["k_norm"] = state_dict[p + "attn_k_norm.weight"][0] if c.qk_norm else None
      if p + "attn_q.bias" in state_dict:                                # Linear(bias=qkv_bias), model.py:161-163: one bias row per sequence for the additive epilogue
        b["bias"] = [Buffer.from_numpy(np.tile(state_dict[p + f"attn_{n}.bias"][0].numpy().view(np.uint8).view(f32).reshape(1, -1), (B, 1))) for n in "qkv"]
      b["moe"] = c.num_experts > 0 and i >= c.leading_dense_blocks       # leading blocks of an MoE model are dense (model.py:84)
      if b["moe"]:
        ex = lambda name: ExpertWeights(state_dict[p + name][0], state_dict[p + name][1], *state_dict[p + name][2])
        b["router"] = lin(p + "ffn_gate_inp.weight")
        b["gate_exps"], b["up_exps"], b["down_exps"] = ex("ffn_gate_exps.weight"), ex("ffn_up_exps.weight"), ex("ffn_down_exps.weight")
        b["sel_bias"] = state_dict[p + "exp_probs_b.bias"][0] if c.expert_bias else None
        if c.shared_expert_dim:                                          # model.py:99-103, 131-134
          for nm in ("ffn_gate_shexp", "ffn_up_shexp", "ffn_down_shexp"): b[nm] = lin(p + nm + ".weight")
          b["gate_inp_shexp"] = lin(p + "ffn_gate_inp_shexp.weight") if c.shared_expert_gate else None
          if b["ffn_gate_shexp"].ggml_type != b["ffn_up_shexp"].ggml_type: raise NotImplementedError("ffn_gate_shexp and ffn_up_shexp of different ggml types are not built")
      else:
        for nm in ("ffn_gate", "ffn_up", "ffn_down"): b[nm] = lin(p + nm + ".weight")
      if chunk_of is not None: b["cache_k"], b["cache_v"] = chunk_of.blk[i].cache_k, chunk_of.blk[i].cache_v
      else:
        b["cache_k"] = Buffer((B, c.n_kv_heads, c.max_context, c.head_dim), f16).zero_()
        b["cache_v"] = Buffer((B, c.n_kv_heads, c.max_context, c.head_dim), f16).zero_()
      self.blk.append(b)
    k = max(1, c.num_experts_per_tok)
    self.state = Buffer((16,), np.int32).zero_()
    self.tokens = Buffer((B,), np.int32).zero_()
    self.x, self.xn = Buffer((B, c.dim), f32), Buffer((B, c.dim), f16)
    self.q, self.k, self.v = Buffer((B, nq), f32), Buffer((B, nkv), f32), Buffer((B, nkv), f32)
    self.attn = Buffer((B, nq), f16)
    self.attn_part = Buffer((B * c.n_heads * ((c.max_context + 63) // 64) * (c.head_dim + 2),), f32).zero_()
    self.act = Buffer((B, max(1, c.hidden_dim, c.dense_hidden_dim)), f16)
    if any(not b["moe"] and b["ffn_gate"].ggml_type != b["ffn_up"].ggml_type for b in self.blk):      # (gate and up rows of such a block, before silu(gate) * up)
      self.gate32, self.up32 = Buffer((B, max(c.hidden_dim, c.dense_hidden_dim)), f32), Buffer((B, max(c.hidden_dim, c.dense_hidden_dim)), f32)
    if c.shared_expert_dim:
      self.act_sh, self.y_sh = Buffer((B, c.shared_expert_dim), f16), Buffer((B, c.dim), f32)
      self.p_sh, self.sh_logit, self.sh_sel = Buffer.from_numpy(np.ones(B, dtype=f32)), Buffer((B, 1), f32), Buffer((B,), np.int32)   # weight 1 unless the shared expert is gated
    if c.num_experts:
      self.router_logits, self.sel, self.probs = Buffer((B, c.num_experts), f32), Buffer((B * k,), np.int32), Buffer((B * k,), f32)
      self.job_table, self.job_flags = Buffer((c.num_experts, 16), np.int32).zero_(), Buffer((1,), np.int32).zero_()
      self.act_e, self.y_e = Buffer((B * k, c.hidden_dim), f16), Buffer((B * k, c.dim), f32)
    self.logits_buf = Buffer((B, c.vocab_size), f32) if chunk_of is None else None
    self.rope = Buffer.from_numpy(rope_table(c.head_dim, c.rope_dim or c.head_dim, c.max_context, c.rope_theta)) if chunk_of is None else chunk_of.s.rope
    self.prompts = Buffer((B if chunk_of is None else 1, c.max_context), np.int32).zero_()
    self.out_tokens = Buffer((max(1, max_new), B), np.int32).zero_()
    self.stream = rt.Stream()
    self._graphs, self._steps_done = {}, 0
    self.replay = "cmdlist"                                          # as Transformer.replay
    self.expert_path = os.environ.get("TGA_EXPERT_PATH", "jobs")      # "jobs": one GEMV per (sequence, slot); "grouped": one small-batch GEMM per selected expert
    # Prefill steps of 17 .. 128 positions of a dense model: the rows pass from launch to launch in the layout the prefill GEMM multiplies from (norm -> q/k/v and gate/up,
    # attention -> attn_output, SwiGLU -> ffn_down: no staging launches) and the split-K sums of attn_output / ffn_down are completed by the norm launch behind them
    self.rows64 = 0
    if self.chunked and 17 <= B <= 128 and not c.num_experts and os.environ.get("TGA_ROWS64", "1") == "1":
      def ncg_of(l):
        n = ctypes.c_int(0); rt.check(rt.lib().tga_rows_staged_plan(l.ggml_type, l.in_features, B, ctypes.byref(n))); return n.value
      ok = all("bias" not in b and not b["moe"] and b["ffn_gate"].ggml_type == b["ffn_up"].ggml_type
               and all(ncg_of(b[nm]) for nm in ("attn_q", "attn_k", "attn_v", "attn_output", "ffn_gate", "ffn_up", "ffn_down"))
               and all(b[nm].out_features % 16 == 0 for nm in ("attn_q", "attn_k", "attn_v")) for b in self.blk)
      if ok and c.dim % 256 == 0 and c.hidden_dim % 256 == 0 and nq % 256 == 0:
        self.rows64 = 2 if B <= 32 else 4 if B <= 64 else 8             # column groups of sixteen rows in the layout
        R = 16 * self.rows64
        self.xn_st, self.attn_st, self.act_st = Buffer((R, c.dim), f16).zero_(), Buffer((R, nq), f16).zero_(), Buffer((R, c.hidden_dim), f16).zero_()

  def _linear(self, layers, x, outs, **kw): qlinear_multi(layers, x, outs, stream=self.stream.handle, **kw)

  def _step(self, with_head: bool, on_block=None):
    c, B, L, st = self.config, self.batch, rt.lib(), self.stream.handle
    rt.check(L.tga_embed_rows(self.token_embd.ptr, self.embd_type, c.dim, self.tokens.ptr, B, self.state.ptr, self.x.ptr, st))
    # The weighted sum over a block's selected experts plus its residual (model.py:130, 150) is completed by the NEXT norm's launch (the next block's attn_norm
    # or output_norm): `pending` says that x still lacks it.
    pending = False
    def norm(weight):
      nonlocal pending
      if pending: rt.check(L.tga_moe_combine_rmsnorm_rows(self.y_e.ptr, self.probs.ptr, self.x.ptr, weight.ptr, B, c.num_experts_per_tok, c.dim, c.norm_eps, self.xn.ptr, None, st))
      else: rt.check(L.tga_rmsnorm_rows(self.x.ptr, weight.ptr, B, c.dim, c.norm_eps, self.xn.ptr, None, 0, st))
      pending = False
    done = (lambda i: on_block(i)) if on_block is not None else (lambda i: None)     # on_block(i): block i's launches have been issued (eager stepping only; e.g. to read back self.sel)
    if self.rows64:
      self._blocks_rows64(done)
      rt.check(L.tga_chunk_advance(self.state.ptr, self.prompts.ptr, B, self.tokens.ptr, c.max_context, st))
      return
    for bi, b in enumerate(self.blk):
      # h = x + attention(attn_norm(x))                                                   model.py:149
      qkv, outs, i = [b["attn_q"], b["attn_k"], b["attn_v"]], [self.q, self.k, self.v], 0
      # the norm inside the launch where the kernel can: always for one run of equal block types (the call norms first where it cannot), for several runs
      # (a Q4_K_M file keeps attn_v as Q6_K in half of the blocks) only in the range where every run's kernel folds it
      same = all(l.ggml_type == qkv[0].ggml_type for l in qkv)
      fold = not pending and (same or (2 <= B <= 8 and c.dim <= 4096 and c.dim % 2048 == 0 and all(l.out_features % 16 == 0 for l in qkv)))
      if not fold: norm(b["attn_norm"])
      while i < 3:                                                     # one launch per run of equal block types
        j = i + 1
        while j < 3 and qkv[j].ggml_type == qkv[i].ggml_type: j += 1
        bias = dict(epilogue=1, resid=b["bias"][i:j]) if "bias" in b else {}
        if fold: self._linear(qkv[i:j], self.x, outs[i:j], norm=(b["attn_norm"], c.norm_eps, self.xn), **bias)
        else: self._linear(qkv[i:j], self.xn, outs[i:j], **bias)
        i = j
      attention = L.tga_attention_prefill_chunk if self.chunked else L.tga_attention_decode_batched
      rt.check(attention(B, self.q.ptr, self.k.ptr, self.v.ptr, b["q_norm"].ptr if c.qk_norm else None, b["k_norm"].ptr if c.qk_norm else None,
                         c.norm_eps, int(c.qk_norm == c.head_dim), b["cache_k"].ptr, b["cache_v"].ptr, self.attn_part.ptr, self.state.ptr,
                         c.n_heads, c.n_kv_heads, c.head_dim, c.max_context, self.rope.ptr, self.attn.ptr, None, st))
      self._linear([b["attn_output"]], self.attn, [self.x], epilogue=1, resid=[self.x])
      # x = h + feed_forward(ffn_norm(h))                                                   model.py:150
      fused_router = b["moe"] and b["router"].ggml_type == rt.F16 and c.dim % 8 == 0 and c.num_experts <= 1024   # ffn_norm and the router logits in one launch (as the batch-1 step)
      if fused_router:
        rt.check(L.tga_moe_router_rows(self.x.ptr, b["ffn_norm"].ptr, c.norm_eps, b["router"].blocks.ptr, B, c.dim, c.num_experts, self.xn.ptr, self.router_logits.ptr, st))
      elif b["moe"]:
        rt.check(L.tga_rmsnorm_rows(self.x.ptr, b["ffn_norm"].ptr, B, c.dim, c.norm_eps, self.xn.ptr, None, 0, st))
      if not b["moe"]:
        if b["ffn_gate"].ggml_type != b["ffn_up"].ggml_type:             # two launches and an elementwise silu(gate) * up (the SwiGLU epilogue pairs rows of one block type)
          rt.check(L.tga_rmsnorm_rows(self.x.ptr, b["ffn_norm"].ptr, B, c.dim, c.norm_eps, self.xn.ptr, None, 0, st))
          h = b["ffn_gate"].out_features
          g32, u32 = self.gate32.view(0, (B, h), np.float32), self.up32.view(0, (B, h), np.float32)
          self._linear([b["ffn_gate"]], self.xn, [g32]); self._linear([b["ffn_up"]], self.xn, [u32])
          rt.check(L.tga_silu_mul(g32.ptr, u32.ptr, B * h, self.act.ptr, st))
        else: self._linear([b["ffn_gate"], b["ffn_up"]], self.x, [self.act], epilogue=2, norm=(b["ffn_norm"], c.norm_eps, self.xn))
        self._linear([b["ffn_down"]], self.act, [self.x], epilogue=1, resid=[self.x])
        done(bi); continue
      k = c.num_experts_per_tok                                         # model.py:110-135
      if not fused_router: b["router"](self.xn, out=self.router_logits, stream=st)
      self_gated = self.expert_path != "grouped" and b["sel_bias"] is None and self.xn.dtype == np.float16 and c.dim <= 4096   # the gate/up launch gates for itself (as the batch-1 step does)
      if not self_gated:
        moe_gate(self.router_logits, B, c.num_experts, k, self.sel, self.probs, c.expert_gating_func, c.norm_topk_prob, c.routed_scaling_factor, stream=st, bias=b["sel_bias"])
      if self.expert_path == "grouped" and B > 8: raise ValueError("the grouped expert path keeps at most eight rows per expert (one per sequence): batch <= 8")
      if self.expert_path == "grouped":                                # one small-batch GEMM per selected expert (its weights read once by the kernel)
        expert_jobs(self.sel, c.num_experts, self.job_table, self.job_flags, stream=st)
        experts_grouped(b["gate_exps"], self.job_table, B * k, self.xn, self.act_e, jobs_per_x_row=k, up=b["up_exps"], stream=st)
        experts_grouped(b["down_exps"], self.job_table, B * k, self.act_e, self.y_e, jobs_per_x_row=1, stream=st)
      else:                                                              # one GEMV per (sequence, slot) job; an expert picked twice is read twice, the second time from cache
        route = (self.router_logits, c.expert_gating_func, c.norm_topk_prob, c.routed_scaling_factor, self.probs) if self_gated else None
        b["gate_exps"](self.sel, self.xn, self.act_e, jobs_per_x_row=k, up=b["up_exps"], stream=st, route=route)
        b["down_exps"](self.sel, self.act_e, self.y_e, jobs_per_x_row=1, stream=st)
      if not c.shared_expert_dim: pending = True; done(bi); continue  # x + sum_j p_j y_j: left to the next norm's launch
      moe_combine(self.y_e, self.probs, self.x, B, k, c.dim, self.x, stream=st)
      if c.shared_expert_dim:                                            # + shared expert, each row scaled by 1 or by sigmoid(xn . ffn_gate_inp_shexp)
        self._linear([b["ffn_gate_shexp"], b["ffn_up_shexp"]], self.xn, [self.act_sh], epilogue=2)
        self._linear([b["ffn_down_shexp"]], self.act_sh, [self.y_sh])
        if b["gate_inp_shexp"] is not None:
          b["gate_inp_shexp"](self.xn, out=self.sh_logit, stream=st)
          moe_gate(self.sh_logit, B, 1, 1, self.sh_sel, self.p_sh, 2, False, 1.0, stream=st)
        moe_combine(self.y_sh, self.p_sh, self.x, B, 1, c.dim, self.x, stream=st)
      done(bi)
    if with_head:                                                        # output(output_norm(x)) and the greedy token of every sequence, model.py:362-364
      if pending or not 2 <= B <= 8: norm(self.output_norm); self.output(self.xn, out=self.logits_buf, stream=st)
      else: self._linear([self.output], self.x, [self.logits_buf], norm=(self.output_norm, c.norm_eps, self.xn))
    elif pending:                                                        # (a prompt step ends with the last block: nothing reads x afterwards, but keep it whole)
      moe_combine(self.y_e, self.probs, self.x, B, c.num_experts_per_tok, c.dim, self.x, stream=st)
    if self.chunked:                                                     # the next B prompt tokens, B positions on
      rt.check(L.tga_chunk_advance(self.state.ptr, self.prompts.ptr, B, self.tokens.ptr, c.max_context, st))
      return
    rt.check(L.tga_argmax_rows_step(self.logits_buf.ptr if with_head else None, B, c.vocab_size, self.state.ptr, self.prompts.ptr, c.max_context, self.tokens.ptr,
                                    self.out_tokens.ptr, self.max_new, st))

  def _blocks_rows64(self, done):
    """The blocks of a prefill step of 17 .. 128 rows (see rows64 in __init__): per block norm (+ the pending split-K sums of the linear before it) -> q/k/v -> attention ->
    attn_output (sums deferred) -> norm -> gate/up + SwiGLU -> ffn_down (sums deferred); what the last block leaves pending is added at the end."""
    c, B, L, st = self.config, self.batch, rt.lib(), self.stream.handle
    VP2, I2 = ctypes.c_void_p * 2, ctypes.c_int64 * 2
    pend = (None, 0, 0)                                                # partial tiles still to be added to self.x: (pointer, splits, row pitch)
    def norm_stage(weight, consumer):
      nonlocal pend
      rt.check(L.tga_rmsnorm_rows_stage(self.x.ptr, pend[0], pend[1], pend[2], weight.ptr, c.norm_eps, B, c.dim, consumer.ggml_type, None, self.xn_st.ptr, st))
      pend = (None, 0, 0)
    def deferred(layer, x_st):
      nonlocal pend
      part, ks, np_ = ctypes.c_void_p(), ctypes.c_int(0), ctypes.c_int(0)
      rt.check(L.tga_qlinear_rows_deferred(layer.ggml_type, layer.blocks.ptr, layer.out_features, layer.in_features, x_st.ptr, B, self.x.ptr,
                                           ctypes.byref(part), ctypes.byref(ks), ctypes.byref(np_), st))
      pend = (part.value, ks.value, np_.value) if ks.value else (None, 0, 0)
    for bi, b in enumerate(self.blk):
      qkv, outs, i = [b["attn_q"], b["attn_k"], b["attn_v"]], [self.q, self.k, self.v], 0
      while i < 3:                                                     # one launch per run of equal block types (a Q4_K_M file keeps attn_v as Q6_K in half of the blocks), each over
        j = i + 1                                                      # the rows in ITS type's layout: the norm launch runs once per run (the first completes the pending sums)
        while j < 3 and qkv[j].ggml_type == qkv[i].ggml_type: j += 1
        norm_stage(b["attn_norm"], qkv[i])
        n = j - i
        rt.check(L.tga_qlinear_multi(qkv[i].ggml_type, n, (ctypes.c_void_p * n)(*[l.blocks.ptr for l in qkv[i:j]]), (ctypes.c_void_p * n)(*[o.ptr for o in outs[i:j]]),
                                     (ctypes.c_int64 * n)(*[l.out_features for l in qkv[i:j]]), self.xn_st.ptr, rt.F16_STAGED, rt.F32, B, qkv[i].in_features, 0, None, 0, 0, st))
        i = j
      ao = b["attn_output"]
      rt.check(L.tga_attention_prefill_chunk_staged(B, self.q.ptr, self.k.ptr, self.v.ptr, b["q_norm"].ptr if c.qk_norm else None, b["k_norm"].ptr if c.qk_norm else None,
                                                    c.norm_eps, int(c.qk_norm == c.head_dim), b["cache_k"].ptr, b["cache_v"].ptr, self.attn_part.ptr, self.state.ptr,
                                                    c.n_heads, c.n_kv_heads, c.head_dim, c.max_context, self.rope.ptr, self.attn_st.ptr, ao.ggml_type, st))
      deferred(ao, self.attn_st)
      g, u, d = b["ffn_gate"], b["ffn_up"], b["ffn_down"]
      norm_stage(b["ffn_norm"], g)
      rt.check(L.tga_qlinear_multi(g.ggml_type, 2, VP2(g.blocks.ptr, u.blocks.ptr), VP2(self.act_st.ptr, None), I2(g.out_features, u.out_features),
                                   self.xn_st.ptr, rt.F16_STAGED, rt.F16, B, g.in_features, 2, None, d.ggml_type, d.in_features, st))
      deferred(d, self.act_st)
      done(bi)
    if pend[1]: rt.check(L.tga_rows_add_partials(self.x.ptr, pend[0], pend[1], pend[2], B, c.dim, st))

  def _graph(self, with_head: bool):
    if with_head not in self._graphs:
      g = (rt.CommandList if self.replay == "cmdlist" else rt.Graph)(self.stream)
      with g: self._step(with_head)
      self._graphs[with_head] = g
    return self._graphs[with_head]

  def prefill_chunks(self, tokens: list[int], start: int, n_chunks: int, use_graph: bool = True) -> int:
    """Chunked prefill for `chunk_of`: computes the positions start .. start + n_chunks * batch - 1 of the prompt, `batch` at a time, into its KV caches.
    Returns the number of positions done."""
    c, B = self.config, self.batch
    if not self.chunked: raise RuntimeError("prefill_chunks needs a model built with chunk_of")
    if n_chunks <= 0: return 0
    if not (0 <= start and start + n_chunks * B <= len(tokens) < c.max_context): raise ValueError(f"chunks {start}+{n_chunks}x{B} outside the prompt of {len(tokens)} tokens")
    if min(tokens) < 0 or max(tokens) >= c.vocab_size: raise ValueError(f"token id outside the vocabulary of {c.vocab_size}")
    pr = np.zeros((1, c.max_context), np.int32); pr[0, :len(tokens)] = tokens
    self.prompts.copyin(pr)
    self.tokens.copyin(np.ascontiguousarray(pr[0, start:start + B]))
    st = np.zeros(16, np.int32); st[0], st[3], st[5] = start, len(tokens), c.vocab_size
    self.state.copyin(st)
    self._owner_stream.synchronize()
    for _ in range(n_chunks):
      if use_graph: self._graph(False).launch()
      else: self._step(False)
    self.stream.synchronize()
    self.check_state()
    return n_chunks * B

  def prefill(self, prompts: list[list[int]], use_graph: bool = True, on_block=None):
    c, B = self.config, self.batch
    n = len(prompts[0])
    if len(prompts) != B or any(len(p) != n for p in prompts): raise ValueError(f"need {B} prompts of equal length")
    if not 1 <= n < c.max_context: raise ValueError(f"prompt of {n} tokens does not fit max_context {c.max_context}")
    if min(map(min, prompts)) < 0 or max(map(max, prompts)) >= c.vocab_size: raise ValueError(f"token id outside the vocabulary of {c.vocab_size}")
    pr = np.zeros((B, c.max_context), np.int32); pr[:, :n] = np.array(prompts, np.int32)
    self.prompts.copyin(pr)
    self.tokens.copyin(np.ascontiguousarray(pr[:, 0]))
    st = np.zeros(16, np.int32); st[3], st[5] = n, c.vocab_size
    self.state.copyin(st)
    for _ in range(n - 1):
      if use_graph and on_block is None: self._graph(False).launch()
      else: self._step(False, on_block)
    self._steps_done = n - 1
    self.stream.synchronize()

  def decode_step(self, use_graph: bool = True, sync: bool = True, on_block=None):
    if self._steps_done >= self.config.max_context: raise RuntimeError(f"context full: position {self._steps_done} is beyond max_context {self.config.max_context}")
    if use_graph and on_block is None: self._graph(True).launch()
    else: self._step(True, on_block)
    self._steps_done += 1
    if sync: self.stream.synchronize()

  def generate(self, prompts: list[list[int]], max_new_tokens: int, use_graph: bool = True):
    """Greedy decoding of every sequence: yields the list of B token ids of each step."""
    self.prefill(prompts, use_graph)
    for i in range(min(max_new_tokens, self.config.max_context - len(prompts[0]), self.max_new)):
      self.decode_step(use_graph)
      yield [int(t) for t in self.out_tokens.view(4 * i * self.batch, (self.batch,), np.int32).numpy()]
    self.check_state()

  def check_state(self):
    err = int(self.state.numpy()[4])
    flags = int(self.job_flags.numpy()[0]) if self.config.num_experts else 0
    if err or flags:                                                    # cleared before raising, so that the next check reports the next steps only
      st = self.state.numpy(); st[4] = 0; self.state.copyin(st)
      if flags: self.job_flags.zero_()
      raise RuntimeError(f"batched decode refused an input: state error {err}, expert grouping flags {flags}")

  def logits(self) -> np.ndarray: return self.logits_buf.numpy()
