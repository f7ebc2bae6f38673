"""Pins for the oracle functions that no reference test covers: route / rows_e on a hand-computed case, grouped_mx_gemm_ref against a
brute-force loop in exact rational arithmetic, and the wiring of llm.Model.forward through closed forms (each one built so that a
plausible mistake - a tile too many, weights permuted against their experts, a transposed operand, np.tile for np.repeat, a cache
row written at the wrong position, the FFN fed from the wrong residual - changes the expected numbers)."""
from fractions import Fraction
import struct
import numpy as np
from oracle import moe as omoe, mxfp8 as omx, llm as ollm

# ------------------------------------------------------------------------------------------------ route (extra/gemm/moe_routing.py:109-122)
def test_route_hand_computed_tie_and_empty_expert():
  """T = 3, E = 4, k = 2.  Worked by hand from moe_routing.py:109-122 and Tensor.topk's order (descending, lower index first among equals):
    token 0 logits [1, 1, 0, -1]      -> experts (0, 1), a tie, weights softmax(1, 1) = (1/2, 1/2)
    token 1 logits [0, 3, -5, 2]      -> experts (1, 3), weights softmax(3, 2) = (e/(1+e), 1/(1+e))
    token 2 logits [.5, -1, -2, .5]   -> experts (0, 3), a tie across a gap, weights (1/2, 1/2)
  flattened assignments j = 0..5 go to experts 0, 1, 1, 3, 0, 3; expert 2 gets nothing.  counts (2, 2, 0, 2) -> padded (256, 256, 0, 256)
  -> off = (0, 256, 512, 512, 768); dest_row = off[e] + (rank of j among the assignments of e) = (0, 256, 257, 512, 1, 513);
  m_l = (ceil(6 / 256) + 4) * 256 = 1280; tile -> expert = #(off[:4] <= 256 t) - 1 = (0, 1, 3, 3, 3): the empty expert owns no tile."""
  lg = np.array([[1, 1, 0, -1], [0, 3, -5, 2], [0.5, -1, -2, 0.5]], dtype=np.float32)
  r = omoe.route(lg, 2, 4)
  np.testing.assert_array_equal(r["topi"], [[0, 1], [1, 3], [0, 3]])
  e = np.e
  np.testing.assert_allclose(r["weights"], [[0.5, 0.5], [e / (1 + e), 1 / (1 + e)], [0.5, 0.5]], rtol=1e-6)
  np.testing.assert_array_equal(r["off"], [0, 256, 512, 512, 768])
  np.testing.assert_array_equal(r["dest_row"], [0, 256, 257, 512, 1, 513])
  assert r["m_l"] == 1280 and omoe.m_max_for(3, 2, 4) == 1280
  np.testing.assert_array_equal(omoe.rows_e(r["off"], r["m_l"]), [0, 1, 3, 3, 3])
  # dispatch / combine on rows that identify their token: xg holds token j // k at dest_row[j], zero elsewhere; combine weighs slot s by weights[t, s]
  x = np.array([[1.0, 10.0], [2.0, 20.0], [3.0, 30.0]], dtype=np.float32)
  xg = omoe.dispatch(x, r, 2)
  assert xg.shape == (1280, 2)
  for row, tok in {0: 0, 1: 2, 256: 0, 257: 1, 512: 1, 513: 2}.items(): np.testing.assert_array_equal(xg[row], x[tok])
  assert np.count_nonzero(xg.any(axis=1)) == 6
  y = np.zeros((1280, 1), dtype=np.float32); y[[0, 256, 257, 512, 1, 513], 0] = [100, 200, 300, 400, 500, 600]   # y[dest_row[j]] = 100 (j + 1)
  out = omoe.combine(y, r, 3, 2)
  np.testing.assert_allclose(out[:, 0], [150.0, (300 * e + 400) / (1 + e), 550.0], rtol=1e-6)

def test_route_padding_is_minimal_at_tile_boundaries():
  """256 assignments to one expert need exactly one tile, 257 need two (off by one in the ceil would show here)."""
  for n, tiles in ((255, 1), (256, 1), (257, 2), (512, 2), (513, 3)):
    lg = np.full((n, 3), -1.0, dtype=np.float32); lg[:, 1] = 1.0
    r = omoe.route(lg, 1, 3)
    np.testing.assert_array_equal(r["off"], [0, 0, 256 * tiles, 256 * tiles])
    np.testing.assert_array_equal(r["dest_row"], np.arange(n))
    np.testing.assert_allclose(r["weights"], 1.0)

# ------------------------------------------------------------------------------------------------ grouped_mx_gemm_ref
def _e4m3_value(b: int) -> Fraction:
  """OCP E4M3 (fn) by its definition: sign, 4-bit exponent with bias 7, 3-bit mantissa; exponent 0 = subnormal m / 8 * 2^-6."""
  s, ex, m = -1 if b & 0x80 else 1, (b >> 3) & 0xF, b & 7
  v = Fraction(m, 8) * Fraction(1, 64) if ex == 0 else (1 + Fraction(m, 8)) * (Fraction(2) ** (ex - 7))
  return s * v

def _bf16_rne(v: float) -> float:
  """float32 -> bfloat16, round to nearest even, through the bit pattern."""
  (u,) = struct.unpack("<I", struct.pack("<f", v))
  u = (u + 0x7FFF + ((u >> 16) & 1)) & 0xFFFF0000
  return struct.unpack("<f", struct.pack("<I", u))[0]

def test_grouped_mx_gemm_ref_against_exact_brute_force():
  """Three 256-row tiles, three experts of which the middle one is empty and the last tile lies beyond expert_off[E] (rows_e gives it to the
  last expert, moe_routing.py:98-104); every output element recomputed as an exact rational sum over k of
  e4m3(x) 2^(ex-127) e4m3(w[e]) 2^(ew-127) with e chosen by the row's offset range, then rounded float32 -> bf16."""
  rng = np.random.default_rng(7)
  M, N, K, E = 768, 3, 64, 3
  off = np.array([0, 256, 256, 512], dtype=np.int32)
  codes = np.array([c for c in range(256) if (c & 0x7F) != 0x7F], dtype=np.uint8)          # every finite E4M3 code
  xq, wq = rng.choice(codes, (M, K)), rng.choice(codes, (E, N, K))
  xe, we = rng.integers(120, 131, (M, K // 32), dtype=np.uint8), rng.integers(120, 131, (E, N, K // 32), dtype=np.uint8)
  got = omx.grouped_mx_gemm_ref(xq, xe, wq, we, off)
  val = [_e4m3_value(c) for c in range(256)]
  rows = list(range(0, 8)) + [255, 256, 257, 300, 511, 512, 700, 767]                        # both sides of the expert boundary, and the tile beyond off[E]
  exact, ulp_off = 0, 0
  for r in rows:
    e = 0 if r < 256 else 2                                                                  # (row 512 and beyond: off[E] = 512, so the last expert)
    for n in range(N):
      acc = Fraction(0)
      for k in range(K):
        acc += val[xq[r, k]] * Fraction(2) ** (int(xe[r, k // 32]) - 127) * val[wq[e, n, k]] * Fraction(2) ** (int(we[e, n, k // 32]) - 127)
      want = _bf16_rne(float(np.float32(float(acc))))
      if got[r, n] == want: exact += 1
      else:
        assert abs(got[r, n] - want) <= abs(want) * 2.0 ** -7, (r, n, got[r, n], want)      # one bf16 ulp (float64 vs exact accumulation before the rounding)
        ulp_off += 1
  assert exact >= 0.95 * len(rows) * N, (exact, ulp_off)
  # a transposed or mis-scaled operand is far outside a bf16 ulp: the check above has teeth
  bad = omx.grouped_mx_gemm_ref(xq, xe, wq[::-1], we[::-1], off)
  assert np.abs(bad[:8] - got[:8]).max() > 2.0 ** -6 * np.abs(got[:8]).max()

def test_tile_experts_bias_and_swiglu_closed_forms():
  off = np.array([0, 256, 256, 512], dtype=np.int32)
  np.testing.assert_array_equal(omx.tile_experts(off, 1024), [0, 2, 2, 2])                   # empty expert 1 owns nothing; tiles beyond off[E] -> E - 1
  h = np.zeros((1024, 2), np.float32); bias = np.array([[1.0, 2.0], [10.0, 20.0], [100.0, 200.0]], np.float32)
  hb = omx.add_expert_bias(h, bias, off)
  np.testing.assert_array_equal(hb[[0, 255, 256, 511, 512, 1023]], [[1, 2], [1, 2], [100, 200], [100, 200], [100, 200], [100, 200]])
  # swiglu: interleaved (glu, linear) pairs, glu clamped above only, linear on both sides; float64 closed form within bf16 rounding of the chain
  rng = np.random.default_rng(5)
  hh = omx.to_bf16((rng.standard_normal((7, 16)) * 5).astype(np.float32))
  glu, lin = np.minimum(hh[:, ::2].astype(np.float64), 7.0), np.clip(hh[:, 1::2].astype(np.float64), -7.0, 7.0)
  want = glu / (1 + np.exp(-1.702 * glu)) * (lin + 1)
  # (rounding alpha * glu to bf16 moves the sigmoid's argument by up to |alpha glu| 2^-9 <= 2.3 %, the three products add 2^-9 each)
  np.testing.assert_allclose(omx.swiglu_interleaved(hh), want, rtol=0.035, atol=1e-6)
  big = np.array([[100.0, 100.0, -100.0, -100.0]], np.float32)
  np.testing.assert_allclose(omx.swiglu_interleaved(big), [[7.0 * 8.0, -0.0]], atol=1e-30)   # glu 100 -> 7, lin 100 -> 7 (+1); glu -100 * sigmoid(-170) = -0

def test_moe_feed_forward_loop_against_float64_closed_form():
  """The per-expert loop (gpt_oss.py:227-238) on operands that MXFP8 holds exactly: the result must be the float64 value of
  sum over the top-k experts of softmax_topk(logits)_e * (swiglu(x Wgu_e^T + bgu_e) Wdn_e^T + bdn_e), up to the bf16 roundings of the chain."""
  rng = np.random.default_rng(9)
  T, D, I, E, k = 5, 32, 32, 4, 2
  vals = np.array([0, 0.5, 1, 1.5, 2, -0.5, -1, -1.5, -2], np.float32)
  x = rng.choice(vals, (T, D)); wgu = rng.choice(vals, (E, 2 * I, D)) * 0.25; wdn = rng.choice(vals, (E, D, I)) * 0.25
  bgu = rng.choice(vals, (E, 2 * I)); bdn = rng.choice(vals, (E, D))
  logits = rng.standard_normal((T, E)).astype(np.float32)
  (gq, ge), (dq, de) = omx.quantize_mxfp8(wgu), omx.quantize_mxfp8(wdn)
  np.testing.assert_array_equal(omx.dequant_mxfp8(gq, ge), wgu)                               # exactly representable: no quantization error in the operands
  got = omx.moe_feed_forward_loop(x, logits, k, gq, ge, bgu, dq, de, bdn)
  want = np.zeros((T, D))
  for t in range(T):
    top = np.argsort(-logits[t])[:k]
    w = np.exp(logits[t, top] - logits[t, top].max()); w /= w.sum()
    for wi, e in zip(w, top):
      gu = wgu[e].astype(np.float64) @ x[t] + bgu[e]
      glu, lin = np.minimum(gu[::2], 7.0), np.clip(gu[1::2], -7.0, 7.0)
      y = glu / (1 + np.exp(-1.702 * glu)) * (lin + 1)
      yq = omx.dequant_mxfp8(*omx.quantize_mxfp8(omx.to_bf16(y.astype(np.float32))[None, :]))[0]      # the activation of the second GEMM is MXFP8 too
      want[t] += wi * (wdn[e].astype(np.float64) @ yq + bdn[e])
  assert np.abs(got - want).max() <= 0.03 * np.abs(want).max()
  # teeth: using the wrong expert's down projection is far outside that bound
  wrong = omx.moe_feed_forward_loop(x, logits, k, gq, ge, bgu, dq[::-1], de[::-1], bdn)
  assert np.abs(wrong - want).max() > 0.2 * np.abs(want).max()

# ------------------------------------------------------------------------------------------------ llm.Model.forward wiring
def _model(H=4, KV=2, hd=8, dim=32, hidden=32, vocab=16, blocks=1, seed=0, **over):
  """A float32 (ggml type 0) model whose matrices are set by the caller: {name: array} overrides on top of zeros / identities."""
  rng = np.random.default_rng(seed)
  cfg = dict(num_blocks=blocks, dim=dim, hidden_dim=hidden, n_heads=H, n_kv_heads=KV, norm_eps=1e-5, vocab_size=vocab, head_dim=hd, rope_theta=10000.0)
  t = {"token_embd.weight": rng.standard_normal((vocab, dim)).astype(np.float32), "output_norm.weight": np.ones((1, dim), np.float32),
       "output.weight": np.eye(vocab, dim, dtype=np.float32)}
  for i in range(blocks):
    p = f"blk.{i}."
    t.update({p + "attn_norm.weight": np.ones((1, dim), np.float32), p + "ffn_norm.weight": np.ones((1, dim), np.float32),
              p + "attn_q.weight": rng.standard_normal((H * hd, dim)).astype(np.float32), p + "attn_k.weight": rng.standard_normal((KV * hd, dim)).astype(np.float32),
              p + "attn_v.weight": rng.standard_normal((KV * hd, dim)).astype(np.float32), p + "attn_output.weight": np.zeros((dim, H * hd), np.float32),
              p + "ffn_gate.weight": rng.standard_normal((hidden, dim)).astype(np.float32), p + "ffn_up.weight": rng.standard_normal((hidden, dim)).astype(np.float32),
              p + "ffn_down.weight": np.zeros((dim, hidden), np.float32)})
  t.update(over)
  tensors = {k: (np.ascontiguousarray(v).view(np.uint8).reshape(-1), 0, v.shape) for k, v in t.items()}
  return ollm.Model(cfg, tensors, 16, w_round_f16=False, kv_dtype=np.float32), t, cfg

def _rms(x, eps=1e-5): return x / np.sqrt(np.mean(x * x) + eps)

def test_forward_residual_passes_through_when_projections_are_zero():
  """attn_output = 0 and ffn_down = 0 in both blocks: the row that reaches output_norm is the embedding row itself."""
  m, t, cfg = _model(blocks=2)
  for tok, pos in ((3, 0), (7, 1), (3, 2)):
    lg = m.forward(tok, pos)
    np.testing.assert_allclose(lg, _rms(t["token_embd.weight"][tok])[:cfg["vocab_size"]], rtol=1e-5, atol=1e-6)

def test_forward_single_position_returns_v_with_gqa_mapping():
  """Position 0 holds one key: softmax over one score is 1, so head h outputs the value row of kv head h // (H / KV).  The values are made
  constant per kv head through attn_v.bias (weight 0), attn_output is the identity, so the logits show x + c[h // group] block by block."""
  H, KV, hd, dim = 4, 2, 8, 32
  c = np.array([5.0, -3.0], dtype=np.float32)
  m, t, cfg = _model(H, KV, hd, dim, **{"blk.0.attn_v.weight": np.zeros((KV * hd, dim), np.float32), "blk.0.attn_q.bias": np.zeros((1, H * hd), np.float32),
                                        "blk.0.attn_k.bias": np.zeros((1, KV * hd), np.float32), "blk.0.attn_v.bias": np.repeat(c, hd)[None, :].astype(np.float32),
                                        "blk.0.attn_output.weight": np.eye(dim, H * hd, dtype=np.float32), "output.weight": np.eye(dim, dim, dtype=np.float32),
                                        "token_embd.weight": np.random.default_rng(1).standard_normal((32, dim)).astype(np.float32)}, vocab=32)
  x = t["token_embd.weight"][9]
  want = x + np.repeat(c[[0, 0, 1, 1]], hd)                       # heads 0, 1 -> kv head 0; heads 2, 3 -> kv head 1 (repeat_interleave, not tile)
  np.testing.assert_allclose(m.forward(9, 0), _rms(want), rtol=1e-5, atol=1e-6)

def test_forward_uniform_attention_averages_the_cached_values():
  """attn_k = 0: every score is 0, the softmax is uniform over positions 0..pos, so the attention output at position p is the mean of the values
  written at 0..p - each token's value row must have been written at its own position and all of them read back."""
  H, KV, hd, dim = 2, 2, 8, 16
  rng = np.random.default_rng(2)
  Wv = rng.standard_normal((KV * hd, dim)).astype(np.float32)
  m, t, cfg = _model(H, KV, hd, dim, hidden=16, vocab=16, **{"blk.0.attn_k.weight": np.zeros((KV * hd, dim), np.float32), "blk.0.attn_v.weight": Wv,
                                                              "blk.0.attn_output.weight": np.eye(dim, H * hd, dtype=np.float32), "output.weight": np.eye(dim, dim, dtype=np.float32)})
  toks = [4, 11, 6, 11]
  vals = []
  for pos, tok in enumerate(toks):
    x = t["token_embd.weight"][tok]
    vals.append(Wv @ _rms(x))
    want = x + np.mean(vals, axis=0)
    np.testing.assert_allclose(m.forward(tok, pos), _rms(want), rtol=2e-5, atol=2e-6)

def test_forward_attention_prefers_the_matching_key_across_positions():
  """RoPE makes q . k depend on the distance only: with q = k projections (one head) and a sharp scale, the token attends to the cached position
  that holds the SAME token at distance 0 (itself) rather than to a different token, and the rotation keeps |q . k| of the self score at |k|^2."""
  H = KV = 1; hd = dim = 16
  rng = np.random.default_rng(3)
  P = (rng.standard_normal((hd, dim)) * 4).astype(np.float32)
  m, t, cfg = _model(H, KV, hd, dim, hidden=16, vocab=16, **{"blk.0.attn_q.weight": P, "blk.0.attn_k.weight": P, "blk.0.attn_v.weight": np.eye(hd, dim, dtype=np.float32),
                                                              "blk.0.attn_output.weight": np.eye(dim, hd, dtype=np.float32), "output.weight": np.eye(dim, dim, dtype=np.float32)})
  a, b = t["token_embd.weight"][1], t["token_embd.weight"][2]
  m.forward(1, 0)
  lg = m.forward(2, 1)                                             # scores: (q_b . R(-1) k_a, |k_b|^2) / 4; the self score dominates by construction of the scale
  qa, qb = P @ _rms(a), P @ _rms(b)
  self_score = float(qb @ qb) / 4
  assert self_score > 40                                           # the softmax is saturated unless the self score were computed wrongly
  np.testing.assert_allclose(lg, _rms(b + _rms(b)), rtol=1e-4, atol=1e-5)   # value = eye @ rms(b): attention returns (almost exactly) the token's own value

def test_forward_ffn_reads_the_post_attention_residual():
  """h = x + attention, out = h + down(silu(gate n) * up n) with n = rmsnorm(h): gate = up = down = identity make the FFN term silu(n) * n, and
  a non-zero attention term (constant value rows, single position) separates h from x."""
  H = KV = 2; hd = 8; dim = 16
  c = np.array([2.0, -1.0], dtype=np.float32)
  I = np.eye(dim, dtype=np.float32)
  m, t, cfg = _model(H, KV, hd, dim, hidden=dim, vocab=16, **{"blk.0.attn_v.weight": np.zeros((KV * hd, dim), np.float32), "blk.0.attn_q.bias": np.zeros((1, H * hd), np.float32),
                                                               "blk.0.attn_k.bias": np.zeros((1, KV * hd), np.float32), "blk.0.attn_v.bias": np.repeat(c, hd)[None, :].astype(np.float32),
                                                               "blk.0.attn_output.weight": I, "blk.0.ffn_gate.weight": I, "blk.0.ffn_up.weight": I, "blk.0.ffn_down.weight": I,
                                                               "output.weight": I})
  x = t["token_embd.weight"][5]
  h = x + np.repeat(c, hd)
  n = _rms(h)
  want = h + (n / (1 + np.exp(-n))) * n
  np.testing.assert_allclose(m.forward(5, 0), _rms(want), rtol=1e-5, atol=1e-6)
  wrong = x + (_rms(x) / (1 + np.exp(-_rms(x)))) * _rms(x) + np.repeat(c, hd)          # FFN fed from x instead of h: measurably different
  assert np.abs(_rms(wrong) - _rms(want)).max() > 1e-2

def test_generate_is_greedy_first_maximum():
  """generate() feeds prompt tokens at consecutive positions and picks the FIRST index of the maximum (a tie is made with a duplicated output row)."""
  dim = 16
  out_w = np.eye(16, dim, dtype=np.float32); out_w[9] = out_w[4]                          # rows 4 and 9 always tie
  emb = np.zeros((16, dim), np.float32)
  for tok in range(16): emb[tok, 4 if tok % 2 == 0 else (tok + 1) % 16] = 1.0             # even tokens point at the tied pair, odd token t at t + 1
  m, t, cfg = _model(2, 2, 8, dim, hidden=16, vocab=16, **{"token_embd.weight": emb, "output.weight": out_w})
  toks, margins = m.generate([1], 3)
  assert toks == [2, 4, 4] and margins[1] == 0.0                                          # 1 -> 2; 2 -> tie(4, 9) -> 4; 4 -> tie -> 4

# ---- expert selection bias, shared expert and leading dense blocks of FFNBlock._feed_forward (model.py:84, 113, 123, 131-134) ----

def test_selection_bias_ranks_but_does_not_weigh():
  """Hand case, SIGMOID gating (no softmax coupling): logits 0, ln 3, -ln 3, ln 1 -> scores 1/2, 3/4, 1/4, 1/2.  Without a bias the top-2 is
  {1, then the lower index of the tie 0 / 3}; a bias of +1 on expert 2 must SELECT expert 2 yet weigh it with its unbiased score 1/4."""
  lg = np.array([[0.0, np.log(3.0), -np.log(3.0), 0.0]], np.float32)
  sel, p = omoe.gate_probs(lg, 2, gating=omoe.SIGMOID)
  assert sel.tolist() == [[0, 1]]                        # ascending rank: expert 0 (tie with 3, lower index ranks higher), then expert 1
  np.testing.assert_allclose(p, [[0.5, 0.75]], rtol=1e-6)
  bias = np.array([0.0, 0.0, 1.0, 0.0], np.float32)
  sel, p = omoe.gate_probs(lg, 2, gating=omoe.SIGMOID, bias=bias)
  assert sel.tolist() == [[1, 2]]                        # biased scores 0.5, 0.75, 1.25, 0.5: expert 2 on top, then expert 1
  np.testing.assert_allclose(p, [[0.75, 0.25]], rtol=1e-6)
  sel, p = omoe.gate_probs(lg, 2, gating=omoe.SIGMOID, norm_topk_prob=True, scale=2.0, bias=bias)
  np.testing.assert_allclose(p, [[1.5, 0.5]], rtol=1e-6)  # normalised over the unbiased scores of the selection, then scaled
  # with a bias the SOFTMAX + normalise shortcut of model.py:116-117 must NOT be taken: weights are softmax scores renormalised, not a softmax of logits
  lg2 = np.array([[2.0, 1.0, 0.0]], np.float32)
  sc = np.exp(lg2[0]) / np.exp(lg2[0]).sum()
  sel, p = omoe.gate_probs(lg2, 2, gating=omoe.SOFTMAX, norm_topk_prob=True, bias=np.array([0.0, 0.0, 5.0], np.float32))
  assert sel.tolist() == [[0, 2]]
  np.testing.assert_allclose(p[0], np.array([sc[0], sc[2]]) / (sc[0] + sc[2]), rtol=1e-6)

def _tiny_moe_weights(rng, L=2, D=8, H=4, E=3, lead=0, shared=0, gate=False, bias=False, vocab=16, hd=4):
  w = {"token_embd.weight": rng.standard_normal((vocab, D)).astype(np.float32), "output_norm.weight": np.ones(D, np.float32), "output.weight": rng.standard_normal((vocab, D)).astype(np.float32)}
  for i in range(L):
    p = f"blk.{i}."
    w.update({p + "attn_norm.weight": np.ones(D, np.float32), p + "ffn_norm.weight": np.ones(D, np.float32),
              p + "attn_q.weight": rng.standard_normal((2 * hd, D)).astype(np.float32), p + "attn_k.weight": rng.standard_normal((hd, D)).astype(np.float32),
              p + "attn_v.weight": rng.standard_normal((hd, D)).astype(np.float32), p + "attn_output.weight": np.zeros((D, 2 * hd), np.float32)})
    if i < lead:
      w.update({p + "ffn_gate.weight": rng.standard_normal((6, D)).astype(np.float32), p + "ffn_up.weight": rng.standard_normal((6, D)).astype(np.float32),
                p + "ffn_down.weight": rng.standard_normal((D, 6)).astype(np.float32)})
      continue
    w.update({p + "ffn_gate_inp.weight": rng.standard_normal((E, D)).astype(np.float32), p + "ffn_gate_exps.weight": rng.standard_normal((E, H, D)).astype(np.float32),
              p + "ffn_up_exps.weight": rng.standard_normal((E, H, D)).astype(np.float32), p + "ffn_down_exps.weight": np.zeros((E, D, H), np.float32)})
    if shared:
      w.update({p + "ffn_gate_shexp.weight": rng.standard_normal((shared, D)).astype(np.float32), p + "ffn_up_shexp.weight": rng.standard_normal((shared, D)).astype(np.float32),
                p + "ffn_down_shexp.weight": rng.standard_normal((D, shared)).astype(np.float32)})
      if gate: w[p + "ffn_gate_inp_shexp.weight"] = np.zeros((1, D), np.float32)
    if bias: w[p + "exp_probs_b.bias"] = rng.standard_normal(E).astype(np.float32)
  return w

def test_shared_expert_and_leading_dense_block_wiring():
  """attn_output = 0 and routed ffn_down_exps = 0, so a block adds exactly its always-on feed-forward to the residual row:
  block 0 (leading dense block) x += ffn_down(silu(ffn_gate n) * ffn_up n), block 1 (MoE) x += shared expert, halved by its zero-weight gate
  (sigmoid(0) = 1/2).  Computed here in float64 from the definitions; a block that took the wrong branch, dropped the shared expert or ignored the
  gate misses by O(1)."""
  rng = np.random.default_rng(12)
  cfg = dict(num_blocks=2, dim=8, hidden_dim=4, n_heads=2, n_kv_heads=1, norm_eps=1e-5, vocab_size=16, head_dim=4, rope_theta=10000.0,
             num_experts=3, num_experts_per_tok=2, leading_dense_blocks=1)
  for gate in (False, True):
    w = _tiny_moe_weights(rng, lead=1, shared=5, gate=gate)
    m = ollm.Model(cfg, w, 8, w_round_f16=False, kv_dtype=np.float32)
    lg = m.forward(3, 0)
    f64 = lambda a: a.astype(np.float64)
    rms = lambda v: v / np.sqrt((v * v).mean() + 1e-5)
    silu = lambda v: v / (1 + np.exp(-v))
    x = f64(w["token_embd.weight"][3])
    n = rms(x); x = x + f64(w["blk.0.ffn_down.weight"]) @ (silu(f64(w["blk.0.ffn_gate.weight"]) @ n) * (f64(w["blk.0.ffn_up.weight"]) @ n))
    n = rms(x); sh = f64(w["blk.1.ffn_down_shexp.weight"]) @ (silu(f64(w["blk.1.ffn_gate_shexp.weight"]) @ n) * (f64(w["blk.1.ffn_up_shexp.weight"]) @ n))
    x = x + (0.5 * sh if gate else sh)
    ref = f64(w["output.weight"]) @ rms(x)
    np.testing.assert_allclose(lg, ref, rtol=2e-4, atol=2e-4)
