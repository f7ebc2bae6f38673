"""oracle.llm.Model for models too large to dequantize whole: the same one-token-at-a-time restatement of tinygrad/llm/model.py (forward :358-364,
FFNBlock :110-151, TransformerBlock._attention :167-198), with every quantized matrix left in its GGUF blocks and multiplied by the C restatement
(oracle/c: dequantize a row, round it to fp16 like model.py:376, float32 multiply-accumulate) and only the selected experts of a MoE block touched.
Test infrastructure only.  Pinned by tests/test_oracle_packed.py: logits equal to oracle.llm.Model's on small dense and MoE models (which the closed forms of
tests/test_oracle_pins.py pin) up to the summation order of a float32 dot product."""
import numpy as np
from oracle import cref, llm as ollm, moe as omoe, ggml

class PackedModel:
  def __init__(self, cfg: dict, tensors: dict, max_context: int, threads: int = 1, kv_dtype=np.float16, act_round_f16: bool = False):
    """tensors: {name: (raw bytes ndarray, ggml_type, shape)} as the GPU tests read them back.  F32 / F16 tensors are kept as float32 arrays (norms, dense
    weights of MoE models: the fp16 values the reference holds after its cast); block types stay packed."""
    self.c, self.max_context, self.kv_dtype, self.threads = cfg, max_context, kv_dtype, threads
    self.act16 = act_round_f16        # additionally round the activation entering each linear to fp16 (what the GPU build does): separates that known deviation from others
    self.t = {}
    for name, (raw, typ, shp) in tensors.items():
      raw = np.ascontiguousarray(raw).view(np.uint8).reshape(-1)
      if typ == 0: self.t[name] = ("f", raw.view(np.float32).reshape(shp).astype(np.float32))
      elif typ == 1: self.t[name] = ("f", raw.view(np.float16).reshape(shp).astype(np.float32))
      else: self.t[name] = ("q", raw, typ, tuple(int(s) for s in shp))
    if "output.weight" not in self.t: self.t["output.weight"] = self.t["token_embd.weight"]      # tied embeddings, model.py:379
    self.rd = cfg.get("rope_dim") or cfg["head_dim"]
    self.fc = ollm.precompute_freqs_cis(self.rd, max_context, cfg["rope_theta"])
    L, kv, hd = cfg["num_blocks"], cfg["n_kv_heads"], cfg["head_dim"]
    self.ck = np.zeros((L, kv, max_context, hd), dtype=kv_dtype)
    self.cv = np.zeros((L, kv, max_context, hd), dtype=kv_dtype)
    self.min_route_gap, self.ties_followed, self.trace = np.inf, 0, None

  def clone(self) -> "PackedModel":
    """Another sequence over the same tensors: its own (empty) KV cache and counters."""
    m = object.__new__(PackedModel)
    m.__dict__.update(self.__dict__)
    m.ck, m.cv = np.zeros_like(self.ck), np.zeros_like(self.cv)
    m.min_route_gap, m.ties_followed = np.inf, 0
    return m

  def _vec(self, name): return self.t[name][1].reshape(-1)

  def _lin(self, name, x, expert=None):
    """x (K,) float32 -> (N,) float32: x @ W^T for the named matrix, or for one expert of a stacked (E, N, K) tensor."""
    e = self.t[name]
    if self.act16: x = x.astype(np.float16).astype(np.float32)
    if e[0] == "f":
      w = e[1] if expert is None else e[1][expert]
      return w @ x.astype(np.float32)                                      # (float32 BLAS: a float64 copy of a 50304 x 2048 table per token would dominate the run)
    _, raw, typ, shp = e
    n, k = shp[-2], shp[-1]
    nel, nby = cref._GEOM[typ]
    mat_bytes = n * k // nel * nby
    w = raw if expert is None else raw[expert * mat_bytes:(expert + 1) * mat_bytes]
    return cref.linear(typ, w, np.ascontiguousarray(x, dtype=np.float32).reshape(1, -1), n, k, w_round_f16=True, threads=self.threads)[0]

  def _embed(self, token):
    e = self.t["token_embd.weight"]
    if e[0] == "f": return e[1][token].astype(np.float32)
    _, raw, typ, shp = e
    nel, nby = cref._GEOM[typ]
    rb = shp[-1] // nel * nby
    return ggml.ggml_data_to_tensor(raw[token * rb:(token + 1) * rb], shp[-1], typ).astype(np.float16).astype(np.float32)   # the table is cast to fp16 like every weight (model.py:376)

  def forward(self, token: int, pos: int, follow_sel=None, tie: float = 0.0) -> np.ndarray:
    """One token at position pos -> float32 logits.  follow_sel: per block, the expert selection another implementation made for this token (None for
    dense blocks); it is adopted where it differs from the own one only by a near-tie of router logits within `tie` (oracle.moe.follow_selection),
    anything else raises.  self.ties_followed counts the adoptions."""
    c = self.c
    H, KV, hd, eps = c["n_heads"], c["n_kv_heads"], c["head_dim"], c["norm_eps"]
    x = self._embed(token)
    for i in range(c["num_blocks"]):
      p = f"blk.{i}."
      n = ollm.rmsnorm(x, self._vec(p + "attn_norm.weight"), eps)
      q, k, v = self._lin(p + "attn_q.weight", n), self._lin(p + "attn_k.weight", n), self._lin(p + "attn_v.weight", n)
      if c.get("qk_norm", 0) and c["qk_norm"] != hd:                        # model.py:169
        q, k = ollm.rmsnorm(q, self._vec(p + "attn_q_norm.weight"), eps), ollm.rmsnorm(k, self._vec(p + "attn_k_norm.weight"), eps)
      q, k, v = q.reshape(H, hd), k.reshape(KV, hd), v.reshape(KV, hd)
      if c.get("qk_norm", 0) == hd:                                         # model.py:180
        q, k = ollm.rmsnorm(q, self._vec(p + "attn_q_norm.weight"), eps), ollm.rmsnorm(k, self._vec(p + "attn_k_norm.weight"), eps)
      rd = self.rd
      q = np.concatenate([ollm.apply_rope(q[:, :rd], self.fc[pos]), q[:, rd:]], axis=-1)
      k = np.concatenate([ollm.apply_rope(k[:, :rd], self.fc[pos]), k[:, rd:]], axis=-1)
      self.ck[i, :, pos], self.cv[i, :, pos] = k.astype(self.kv_dtype), v.astype(self.kv_dtype)
      K = np.repeat(self.ck[i, :, :pos + 1].astype(np.float32), H // KV, axis=0)
      V = np.repeat(self.cv[i, :, :pos + 1].astype(np.float32), H // KV, axis=0)
      sc = np.einsum("hd,htd->ht", q, K).astype(np.float32) / np.float32(np.sqrt(hd))
      e = np.exp(sc - sc.max(axis=-1, keepdims=True)); pr = e * (np.float32(1.0) / e.sum(axis=-1, keepdims=True))
      attn = np.einsum("ht,htd->hd", pr, V).astype(np.float32).reshape(-1)
      h = x + self._lin(p + "attn_output.weight", attn)
      n2 = ollm.rmsnorm(h, self._vec(p + "ffn_norm.weight"), eps)
      if c.get("num_experts", 0) and i >= c.get("leading_dense_blocks", 0):
        kx = c["num_experts_per_tok"]
        logits = self._lin(p + "ffn_gate_inp.weight", n2)
        sel, probs = omoe.gate_probs(logits[None, :], kx, c.get("expert_gating_func", 1), c.get("norm_topk_prob", False), c.get("routed_scaling_factor", 1.0))
        if follow_sel is not None and follow_sel[i] is not None:
          s1, p1, followed = omoe.follow_selection(logits, follow_sel[i], kx, c.get("expert_gating_func", 1), c.get("norm_topk_prob", False), c.get("routed_scaling_factor", 1.0), tie)
          sel, probs = s1[None, :], p1[None, :]
          self.ties_followed += int(followed)
        srt = np.sort(logits)
        self.min_route_gap = min(self.min_route_gap, float(srt[-kx] - srt[-kx - 1]) if logits.size > kx else np.inf)
        acc = np.zeros_like(x, dtype=np.float64)
        for sl in range(kx):
          ex = int(sel[0, sl])
          a = ollm.silu(self._lin(p + "ffn_gate_exps.weight", n2, ex)) * self._lin(p + "ffn_up_exps.weight", n2, ex)
          acc += np.float64(probs[0, sl]) * self._lin(p + "ffn_down_exps.weight", a, ex)
        x = h + acc.astype(np.float32)
        self.last_sel = sel[0]
      else:
        x = h + self._lin(p + "ffn_down.weight", ollm.silu(self._lin(p + "ffn_gate.weight", n2)) * self._lin(p + "ffn_up.weight", n2))
      if self.trace is not None: self.trace.append((h.copy(), x.copy()))     # (debugging aid: the residual row after the attention and after the block)
    return self._lin("output.weight", ollm.rmsnorm(x, self._vec("output_norm.weight"), eps))
