"""numpy restatement of one-token-at-a-time decoding in tinygrad/llm/model.py (dense llama path).  Test infrastructure only.

Follows: Transformer.forward model.py:358-364; FFNBlock.__call__ :144-151; TransformerBlock._attention :167-198; apply_rope :29-33;
precompute_freqs_cis :16-19; nn.RMSNorm tinygrad/nn/__init__.py:296-304; SDPA tinygrad/mixin/rand.py:298-327; silu
tinygrad/mixin/elementwise.py:682-690; argmax tinygrad/mixin/op.py:866-891 (first index of the maximum).
Weights are the float32 dequantization of the same GGUF bytes, cast to fp16 like model.py:376 (w_round_f16) - the model path.
kv_dtype: the reference's cache is float32 by default (model.py:202); benchmark configuration 3 asks for fp16, which is what the build runs."""
import numpy as np
from oracle import ggml, moe as omoe

def precompute_freqs_cis(dim, end, theta):
  freqs = (np.float32(1.0) / (np.float32(theta) ** (np.arange(0, dim, 2, dtype=np.float32)[:dim // 2] / np.float32(dim)))).astype(np.float32)
  ang = (np.arange(end, dtype=np.float32)[:, None] * freqs[None, :]).astype(np.float32)
  return np.concatenate([np.cos(ang), np.sin(ang)], axis=-1).astype(np.float32)

def rmsnorm(x, w, eps):
  x = x.astype(np.float32)
  return (x * (np.float32(1.0) / np.sqrt(np.mean(x * x, axis=-1, keepdims=True, dtype=np.float32) + np.float32(eps)))).astype(np.float32) * w

def apply_rope(x, fc):
  """x: (H, hd); fc: (hd,) = cos half | sin half for this position."""
  half = x.shape[-1] // 2
  cos, sin = fc[:half], fc[half:]
  x1, x2 = x[..., :half], x[..., half:]
  return np.concatenate([x1 * cos - x2 * sin, x2 * cos + x1 * sin], axis=-1)

def silu(x): return x * (np.float32(1.0) / (np.float32(1.0) + np.exp(-x.astype(np.float32))))

class Model:
  def __init__(self, cfg: dict, tensors: dict, max_context: int, w_round_f16=True, kv_dtype=np.float16, act_round_f16=False):
    """tensors: {name: (raw bytes ndarray, ggml_type, (rows, cols))}.  act_round_f16 additionally rounds the activation entering
    each linear to fp16 (what the GPU build does) - used only to separate that known deviation from real discrepancies."""
    self.c, self.max_context, self.kv_dtype, self.act16 = cfg, max_context, kv_dtype, act_round_f16
    def deq(name):
      raw, t, shp = tensors[name]
      w = ggml.ggml_data_to_tensor(raw, int(np.prod(shp)), t).reshape(shp)
      return w.astype(np.float16).astype(np.float32) if (w_round_f16 and t not in (0,)) else w.astype(np.float32)
    self.w = {name: (deq(name) if isinstance(tensors[name], tuple) else np.asarray(tensors[name], dtype=np.float32)) for name in tensors}
    if "output.weight" not in self.w: self.w["output.weight"] = self.w["token_embd.weight"]
    self.rd = cfg.get("rope_dim") or cfg["head_dim"]                        # model.py:63, 204
    self.fc = precompute_freqs_cis(self.rd, max_context, cfg["rope_theta"])
    L, kv, hd = cfg["num_blocks"], cfg["n_kv_heads"], cfg["head_dim"]
    self.ck = np.zeros((L, kv, max_context, hd), dtype=kv_dtype)
    self.cv = np.zeros((L, kv, max_context, hd), dtype=kv_dtype)

  def _lin(self, name, x):
    if self.act16: x = x.astype(np.float16).astype(np.float32)
    return (x.astype(np.float64) @ self.w[name].astype(np.float64).T).astype(np.float32)

  def forward(self, token: int, pos: int) -> np.ndarray:
    """One token at position pos -> float32 logits (vocab,)."""
    c = self.c
    H, KV, hd, eps = c["n_heads"], c["n_kv_heads"], c["head_dim"], c["norm_eps"]
    x = self.w["token_embd.weight"][token].astype(np.float32)
    for i in range(c["num_blocks"]):
      p = f"blk.{i}."
      n = rmsnorm(x, self.w[p + "attn_norm.weight"].reshape(-1), eps)
      q, k = self._lin(p + "attn_q.weight", n), self._lin(p + "attn_k.weight", n)
      if p + "attn_q.bias" in self.w: q, k = q + self.w[p + "attn_q.bias"].reshape(-1), k + self.w[p + "attn_k.bias"].reshape(-1)   # Linear(bias=qkv_bias), model.py:161-163
      if c.get("qk_norm", 0) and c["qk_norm"] != hd:                        # model.py:169: full-width q/k norm before the head split
        q, k = rmsnorm(q, self.w[p + "attn_q_norm.weight"].reshape(-1), eps), rmsnorm(k, self.w[p + "attn_k_norm.weight"].reshape(-1), eps)
      q, k = q.reshape(H, hd), k.reshape(KV, hd)
      if c.get("qk_norm", 0) == hd:                                         # model.py:180: per-head q/k norm after the head split
        q, k = rmsnorm(q, self.w[p + "attn_q_norm.weight"].reshape(-1), eps), rmsnorm(k, self.w[p + "attn_k_norm.weight"].reshape(-1), eps)
      rd = self.rd                                                          # model.py:180-181: only the first rope_dim values of a head rotate
      q = np.concatenate([apply_rope(q[:, :rd], self.fc[pos]), q[:, rd:]], axis=-1)
      k = np.concatenate([apply_rope(k[:, :rd], self.fc[pos]), k[:, rd:]], axis=-1)
      v = self._lin(p + "attn_v.weight", n)
      if p + "attn_v.bias" in self.w: v = v + self.w[p + "attn_v.bias"].reshape(-1)
      v = v.reshape(KV, hd)
      self.ck[i, :, pos], self.cv[i, :, pos] = k.astype(self.kv_dtype), v.astype(self.kv_dtype)
      K = np.repeat(self.ck[i, :, :pos + 1].astype(np.float32), H // KV, axis=0)      # (H, T, hd)  GQA repeat_interleave
      V = np.repeat(self.cv[i, :, :pos + 1].astype(np.float32), H // KV, axis=0)
      sc = np.einsum("hd,htd->ht", q, K).astype(np.float32) / np.float32(np.sqrt(hd))
      e = np.exp(sc - sc.max(axis=-1, keepdims=True)); pr = e * (np.float32(1.0) / e.sum(axis=-1, keepdims=True))
      attn = np.einsum("ht,htd->hd", pr, V).astype(np.float32).reshape(-1)
      h = x + self._lin(p + "attn_output.weight", attn)
      n2 = rmsnorm(h, self.w[p + "ffn_norm.weight"].reshape(-1), eps)
      if c.get("num_experts", 0) and i >= c.get("leading_dense_blocks", 0):   # model.py:84 (leading blocks stay dense), 110-135
        kx = c["num_experts_per_tok"]
        logits = self._lin(p + "ffn_gate_inp.weight", n2)
        bias = self.w[p + "exp_probs_b.bias"].reshape(-1) if p + "exp_probs_b.bias" in self.w else None     # model.py:113, 123: ranks by score + bias
        sel, probs = omoe.gate_probs(logits[None, :], kx, c.get("expert_gating_func", 1), c.get("norm_topk_prob", False), c.get("routed_scaling_factor", 1.0), bias=bias)
        # how far the selection is from a tie: gap between the k-th and the (k+1)-th router logit (a test that compares token streams reports
        # it: top-k is discontinuous, an input within rounding noise of a tie may legitimately select another expert)
        srt = np.sort(logits if bias is None else omoe.gate_scores(logits, c.get("expert_gating_func", 1)) + bias)
        self.min_route_gap = min(getattr(self, "min_route_gap", np.inf), float(srt[-kx] - srt[-kx - 1]) if logits.size > kx else np.inf)
        n2l = n2.astype(np.float16).astype(np.float32) if self.act16 else n2
        acc = np.zeros_like(x, dtype=np.float64)
        for sl in range(kx):
          e = int(sel[0, sl])
          g = (n2l.astype(np.float64) @ self.w[p + "ffn_gate_exps.weight"][e].astype(np.float64).T).astype(np.float32)
          u = (n2l.astype(np.float64) @ self.w[p + "ffn_up_exps.weight"][e].astype(np.float64).T).astype(np.float32)
          a = silu(g) * u
          if self.act16: a = a.astype(np.float16).astype(np.float32)
          acc += np.float64(probs[0, sl]) * (a.astype(np.float64) @ self.w[p + "ffn_down_exps.weight"][e].astype(np.float64).T).astype(np.float32)
        out = acc.astype(np.float32)
        if p + "ffn_gate_shexp.weight" in self.w:                             # model.py:131-134: the shared expert, optionally scaled by a sigmoid gate
          sh = self._lin(p + "ffn_down_shexp.weight", silu(self._lin(p + "ffn_gate_shexp.weight", n2)) * self._lin(p + "ffn_up_shexp.weight", n2))
          if p + "ffn_gate_inp_shexp.weight" in self.w:
            gl = self._lin(p + "ffn_gate_inp_shexp.weight", n2).reshape(-1)[0]          # (x * w).sum(-1)
            sh = sh * (np.float32(1.0) / (np.float32(1.0) + np.exp(-gl)))
          out = out + sh
        x = h + out
        self.last_sel = sel[0]
      else:
        x = h + self._lin(p + "ffn_down.weight", silu(self._lin(p + "ffn_gate.weight", n2)) * self._lin(p + "ffn_up.weight", n2))
    return self._lin("output.weight", rmsnorm(x, self.w["output_norm.weight"].reshape(-1), eps))

  def generate(self, tokens, max_new):
    """Greedy: returns (generated tokens, per-step top-2 logit margins)."""
    out, margins, pos = [], [], 0
    for t in tokens[:-1]: self.forward(t, pos); pos += 1
    cur = tokens[-1]
    for _ in range(max_new):
      lg = self.forward(cur, pos); pos += 1
      cur = int(np.argmax(lg))                      # first index of the maximum
      top2 = np.partition(lg, -2)[-2:]
      margins.append(float(top2[1] - top2[0]))
      out.append(cur)
    return out, margins
