"""numpy restatement of the MoE routing / feed-forward pieces.  Test infrastructure only.

pairwise_topk, ExpertGating, FFNBlock._feed_forward (MoE branch): tinygrad/llm/model.py:9-13, 35-41, 110-135.
route / dispatch / combine / m_max_for / Routing.rows_e: extra/gemm/moe_routing.py:89-131 (single device group, G = 1).
The reference holds no test for route / dispatch / combine; they are pinned by a hand-worked case and invariants (tests/test_oracle_pins.py)."""
import numpy as np

BLOCK_ROW = 256
SOFTMAX, SIGMOID, SOFTMAX_WEIGHT, SQRT_SOFTPLUS = 1, 2, 3, 4

def pairwise_topk(x: np.ndarray, k: int):
  """model.py:35-41: rank_i = #{j: x_i > x_j or (x_i == x_j and i < j)}; element of rank r sits at position r; the last k
  positions are returned (ascending: the largest last; among equals the LOWER index ranks higher)."""
  n = x.shape[-1]
  i, j = np.arange(n)[:, None], np.arange(n)[None, :]
  cmp = (x[..., :, None] > x[..., None, :]) | ((x[..., :, None] == x[..., None, :]) & (i < j))
  rank = cmp.sum(axis=-1)
  sel = np.zeros(x.shape, dtype=np.int32)
  np.put_along_axis(sel, rank, np.broadcast_to(np.arange(n, dtype=np.int32), x.shape), axis=-1)
  sel = sel[..., n - k:]
  return np.take_along_axis(x, sel, axis=-1), sel

def softmax(x, axis=-1):
  e = np.exp(x - x.max(axis=axis, keepdims=True))
  return e * (1.0 / e.sum(axis=axis, keepdims=True))

def gate_scores(logits: np.ndarray, gating=SOFTMAX) -> np.ndarray:
  """The scores the selection bias is added to (model.py:118-121)."""
  logits = logits.astype(np.float32)
  if gating == SOFTMAX_WEIGHT: return logits
  if gating == SOFTMAX: return softmax(logits)
  if gating == SIGMOID: return 1.0 / (1.0 + np.exp(-logits))
  return np.sqrt(np.log1p(np.exp(logits)))

def gate_probs(logits: np.ndarray, k: int, gating=SOFTMAX, norm_topk_prob=False, scale=1.0, bias=None):
  """model.py:112-128 -> (sel (.., k) int32, probs (.., k) float32)."""
  logits = logits.astype(np.float32)
  if gating == SOFTMAX and bias is None and norm_topk_prob: gating, norm_topk_prob = SOFTMAX_WEIGHT, False
  if gating == SOFTMAX_WEIGHT: scores = logits
  elif gating == SOFTMAX: scores = softmax(logits)
  elif gating == SIGMOID: scores = 1.0 / (1.0 + np.exp(-logits))
  else: scores = np.sqrt(np.log1p(np.exp(logits)))
  _, sel = pairwise_topk(scores if bias is None else scores + bias, k)
  return sel, selection_probs(scores, sel, gating, norm_topk_prob, scale)

def selection_probs(scores: np.ndarray, sel: np.ndarray, gating, norm_topk_prob, scale) -> np.ndarray:
  """The weights of a given selection (model.py:124-128): the selected scores, softmaxed over the selection for SOFTMAX_WEIGHT, optionally normalised
  to sum 1, times the routed scaling factor.  gating / norm_topk_prob as gate_probs has resolved them."""
  probs = np.take_along_axis(scores, sel, axis=-1)
  if gating == SOFTMAX_WEIGHT: probs = softmax(probs)
  if norm_topk_prob: probs = probs / probs.sum(axis=-1, keepdims=True)
  return (probs * scale).astype(np.float32)

def follow_selection(logits: np.ndarray, forced, k: int, gating=SOFTMAX, norm_topk_prob=False, scale=1.0, tie=0.0):
  """gate_probs of one token's router logits (E,), except that a given selection is adopted where it differs from the own top-k only in experts whose
  router logits lie within `tie` of each other (a near-tie may fall either way between two correct implementations).  Returns (sel (k,), probs (k,),
  followed: the own selection was replaced).  Raises when the given selection differs beyond that."""
  logits = logits.astype(np.float32)
  sel, probs = gate_probs(logits[None, :], k, gating, norm_topk_prob, scale)
  forced = np.asarray(forced).astype(np.int64).reshape(-1)
  if set(forced.tolist()) == set(sel[0].tolist()): return sel[0], probs[0], False
  diff = sorted(set(forced.tolist()) ^ set(sel[0].tolist()))
  spread = float(logits[diff].max() - logits[diff].min())
  if len(forced) != k or len(set(forced.tolist())) != k or spread > tie:
    raise AssertionError(f"expert selection {sorted(forced.tolist())} differs from the own {sorted(sel[0].tolist())} beyond a near-tie: router logits of {diff} spread {spread:.3e} > {tie:.1e}")
  if gating == SOFTMAX and norm_topk_prob: gating, norm_topk_prob = SOFTMAX_WEIGHT, False
  scores = gate_scores(logits, gating)
  order = np.array(sorted(forced.tolist(), key=lambda e: (scores[e], -e)), dtype=np.int32)      # ascending, the lower index ranks higher among equals
  return order, selection_probs(scores[None, :], order[None, :], gating, norm_topk_prob, scale)[0], True

def silu(x): return x * (1.0 / (1.0 + np.exp(-x)))

def moe_feed_forward(x, router_w, gate_w, up_w, down_w, k, gating=SOFTMAX, norm_topk_prob=False, scale=1.0):
  """model.py:110-135 without shared experts.  x (T, D); router_w (E, D); gate_w/up_w (E, H, D); down_w (E, D, H) float."""
  logits = (x.astype(np.float64) @ router_w.astype(np.float64).T).astype(np.float32)
  sel, probs = gate_probs(logits, k, gating, norm_topk_prob, scale)
  out = np.zeros_like(x, dtype=np.float32)
  for t in range(x.shape[0]):
    acc = np.zeros(x.shape[1], dtype=np.float64)
    for s in range(k):
      e = sel[t, s]
      h = silu(gate_w[e].astype(np.float64) @ x[t]) * (up_w[e].astype(np.float64) @ x[t])
      acc += probs[t, s] * (down_w[e].astype(np.float64) @ h)
    out[t] = acc
  return out, sel, probs

# ---- token-sorted expert grouping (extra/gemm/moe_routing.py) ----
def m_max_for(t_local, experts_per_tok, n_experts):            # moe_routing.py:89-90
  return (-(-t_local * experts_per_tok // BLOCK_ROW) + n_experts) * BLOCK_ROW

def route(logits: np.ndarray, k: int, n_experts: int):
  """moe_routing.py:109-122 -> dict(weights (T,k), topi (T,k), dest_row (T*k,), off (E+1,), m_l).
  topk here is Tensor.topk: descending values, the lower index first among equals."""
  T, E = logits.shape
  order = np.argsort(-logits, axis=-1, kind="stable")[:, :k]
  topv = np.take_along_axis(logits, order, axis=-1)
  weights = softmax(topv.astype(np.float32))
  flat = order.reshape(-1)
  m = np.zeros((T * k, E), dtype=np.int32); m[np.arange(T * k), flat] = 1
  cnt = m.sum(0)
  pad = ((cnt + BLOCK_ROW - 1) // BLOCK_ROW) * BLOCK_ROW
  off = np.concatenate([[0], np.cumsum(pad)]).astype(np.int32)
  dest_row = ((np.cumsum(m, axis=0) + off[:E][None, :]) * m).sum(-1) - 1
  return dict(weights=weights, topi=order.astype(np.int32), dest_row=dest_row.astype(np.int32), off=off, m_l=m_max_for(T, k, E))

def rows_e(off: np.ndarray, m_l: int) -> np.ndarray:
  """moe_routing.py:98-104: expert of every 256-row tile = #(off[:E] <= 256 t) - 1."""
  E = off.shape[0] - 1
  tr = np.arange(m_l // BLOCK_ROW) * BLOCK_ROW
  return ((tr[:, None] >= off[None, :E]).sum(-1) - 1).astype(np.int32)

def dispatch(x: np.ndarray, r: dict, k: int) -> np.ndarray:
  """moe_routing.py:124-126: xg[dest_row[j]] = x[j // k] into a zeroed (m_l, D) buffer."""
  xg = np.zeros((r["m_l"], x.shape[1]), dtype=x.dtype)
  xg[r["dest_row"]] = x[np.arange(r["dest_row"].size) // k]
  return xg

def combine(y: np.ndarray, r: dict, n_tokens: int, k: int) -> np.ndarray:
  """moe_routing.py:128-131: out[t] = sum_s weights[t,s] * y[dest_row[t*k+s]] (weights cast to y's dtype first)."""
  sel = y[r["dest_row"]].reshape(n_tokens, k, -1)
  return (sel * r["weights"].reshape(n_tokens, k, 1).astype(sel.dtype)).sum(1)
