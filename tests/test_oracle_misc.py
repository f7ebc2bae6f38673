"""Pins the remaining oracle pieces without a GPU: linear modes, E4M3 / MXFP8, pairwise_topk and routing invariants, MoE closed form."""
import numpy as np, pytest
from oracle import linear as ol, mxfp8 as omx, moe as omoe, cref, ggml as og, llm as ollm

def test_linear_modes_agree_within_tolerance():
  rng = np.random.default_rng(1)
  n, k = 96, 512
  w = rng.integers(0, 256, size=(n * k // 32, 18), dtype=np.uint8)
  w[:, :2] = np.float16(np.abs(rng.standard_normal(n * k // 32)) * 0.003).view(np.uint8).reshape(-1, 2)
  x = rng.standard_normal((3, k)).astype(np.float32)
  W = ol.weight_f32(w, n, k, 2)
  # brute force of the textbook definition on a corner
  bf = np.array([[sum(float(x[m, j]) * float(W[r, j]) for j in range(k)) for r in range(4)] for m in range(3)])
  np.testing.assert_allclose(ol.linear_f64(x, W)[:, :4], bf, rtol=1e-12)
  assert ol.rel_err(cref.linear(2, w, x, n, k), ol.linear_f64(x, W)) < 1e-5
  assert ol.rel_err(cref.linear(2, w, x, n, k, w_round_f16=True), ol.linear_model(x, W)) < 1e-5
  xh = x.astype(np.float16)
  a = cref.linear(2, w, xh, n, k, w_round_f16=True, prod_round_f16=True).astype(np.float16)
  assert ol.rel_err(a, ol.linear_standalone_f16(xh, W)) < 2e-3
  # the model path's fp16 weight cast is lossy for Q4_0 (odd multiplier x 11-bit mantissa)
  assert (W.astype(np.float16).astype(np.float32) != W).mean() > 0.2

def test_e4m3_against_torch_and_round_trip():
  torch = pytest.importorskip("torch")
  rng = np.random.default_rng(0)
  x = np.concatenate([rng.standard_normal(100000) * np.exp2(rng.integers(-12, 10, 100000)),
                      [0, -0.0, 448, 449, 463.9, 464, 464.1, 480, 1e6, -1e6, 2 ** -9, 2 ** -10, 1.5 * 2 ** -10, 0.99 * 2 ** -10]]).astype(np.float32)
  ours = omx.float_to_e4m3(x)
  t = torch.tensor(x).clamp(-448, 448).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
  np.testing.assert_array_equal(ours, t)
  codes = np.arange(256, dtype=np.uint8)
  f = omx.e4m3_to_float(codes); tf = torch.tensor(codes).view(torch.float8_e4m3fn).float().numpy()
  assert ((f == tf) | (np.isnan(f) & np.isnan(tf))).all()
  ok = ~np.isnan(f)
  np.testing.assert_array_equal(omx.float_to_e4m3(f[ok]), codes[ok])             # exhaustive round trip

def test_e4m3_brute_force_nearest_even():
  grid = np.unique(np.abs(omx.e4m3_to_float(np.arange(0x7f, dtype=np.uint8))))
  rng = np.random.default_rng(2)
  for v in rng.uniform(0, 448, 3000):
    d = np.abs(grid - v); best = grid[d == d.min()]
    got = float(omx.e4m3_to_float(omx.float_to_e4m3(np.array([v], np.float32)))[0])
    assert got in best

def test_quantize_mxfp8_invariants():
  rng = np.random.default_rng(3)
  x = (rng.standard_normal((64, 256)) * np.exp2(rng.integers(-10, 10, (64, 1)))).astype(np.float32)
  q, e8 = omx.quantize_mxfp8(x)
  scaled_max = np.abs(x.reshape(64, 8, 32)).max(-1) * np.exp2(127.0 - e8)
  assert ((scaled_max >= 1) & (scaled_max < 2)).all()                            # no -emax bias: block max lands in [1, 2)
  d = omx.dequant_mxfp8(q, e8)
  big = np.abs(x) >= np.repeat(np.abs(x.reshape(64, 8, 32)).max(-1), 32, axis=-1) * 2.0 ** -6
  assert (np.abs(d - x)[big] <= np.abs(x)[big] * 2.0 ** -4).all()                # E4M3-normal values: rel err <= 2^-4
  p2 = np.exp2(rng.integers(-6, 6, (4, 64))).astype(np.float32) * np.sign(rng.standard_normal((4, 64))).astype(np.float32)
  qq, ee = omx.quantize_mxfp8(p2)
  keep = np.abs(p2) >= np.repeat(np.abs(p2.reshape(4, 2, 32)).max(-1), 32, axis=-1) * 2.0 ** -9
  np.testing.assert_array_equal(omx.dequant_mxfp8(qq, ee)[keep], p2[keep])       # powers of two round-trip exactly
  z, ze = omx.quantize_mxfp8(np.zeros((1, 32), np.float32)); assert (z == 0).all() and ze[0, 0] == 0
  assert omx.mx_pack(e8).shape == (2, 64) and omx.mx_pack(e8)[1, 5] == int.from_bytes(bytes(e8[5, 4:8]), "little")

def test_pairwise_topk_reference_vectors():
  # test/unit/test_attention.py:249-270
  v, s = omoe.pairwise_topk(np.array([[[1.0, 3.0, 2.0, 5.0, 4.0]]]), 3)
  np.testing.assert_array_equal(s, [[[1, 4, 3]]]); np.testing.assert_allclose(v, [[[3.0, 4.0, 5.0]]])
  v, s = omoe.pairwise_topk(np.array([[[5.0, 5.0, 3.0, 5.0]]]), 2)
  np.testing.assert_array_equal(s, [[[1, 0]]])
  np.random.seed(42)
  data = np.random.randn(4, 2, 16).astype(np.float32)
  v, s = omoe.pairwise_topk(data, 5)
  for b in range(4):
    for t in range(2): assert set(s[b, t].tolist()) == set(np.argsort(-data[b, t])[:5].tolist())

def test_routing_invariants():
  rng = np.random.default_rng(4)
  T, E, k, D = 500, 32, 4, 16
  lg = rng.standard_normal((T, E)).astype(np.float32)
  r = omoe.route(lg, k, E)
  d, off = r["dest_row"], r["off"]
  assert len(set(d.tolist())) == T * k and (off % 256 == 0).all() and (np.diff(off) >= 0).all() and off[-1] <= r["m_l"]
  e = r["topi"].reshape(-1)
  assert ((d >= off[e]) & (d < off[e + 1])).all()
  for ex in range(E):                                                             # stable: rank order = flattened (token, slot) order
    rows = d[e == ex]; assert (np.diff(rows) == 1).all() and (rows.size == 0 or rows[0] == off[ex])
  x = rng.standard_normal((T, D)).astype(np.float32)
  out = omoe.combine(omoe.dispatch(x, r, k), r, T, k)
  np.testing.assert_allclose(out, x, rtol=1e-5, atol=1e-6)                        # identity experts: x * sum(weights) = x
  te = omoe.rows_e(off, r["m_l"])
  for t in range(off[-1] // 256): assert off[te[t]] <= 256 * t < off[te[t] + 1]

def test_moe_feed_forward_reference_closed_form():
  # test/unit/test_llm_moe.py:15-34: gate scales by (expert+1), up/down identity, router prefers experts 0 and 2
  dim, hidden, E, k = 8, 16, 4, 2
  gate = np.stack([np.eye(hidden, dim) * (i + 1) for i in range(E)]); up = np.stack([np.eye(hidden, dim)] * E); down = np.stack([np.eye(dim, hidden)] * E)
  router = np.array([[1, 0, 1, 0]] * dim, dtype=np.float32).T
  x = ollm.rmsnorm(np.ones((1, dim), np.float32), np.ones(dim, np.float32), 1e-5)
  out, sel, probs = omoe.moe_feed_forward(x, router, gate, up, down, k)
  silu = lambda v: v / (1 + np.exp(-v))
  np.testing.assert_allclose(out[0, 0], (silu(1.0) + silu(3.0)) / 2, rtol=1e-2)
  assert set(sel[0].tolist()) == {0, 2}

def test_rope_and_softmax_closed_forms():
  fc = ollm.precompute_freqs_cis(64, 16, 10000.0)
  x = np.random.default_rng(0).standard_normal((3, 64)).astype(np.float32)
  y = ollm.apply_rope(x, fc[5])
  np.testing.assert_allclose(np.linalg.norm(y, axis=-1), np.linalg.norm(x, axis=-1), rtol=1e-5)   # a rotation
  np.testing.assert_allclose(ollm.apply_rope(x, fc[0]), x, atol=1e-7)                               # position 0: identity
  np.testing.assert_allclose(fc[3, :32], np.cos(3 * 10000.0 ** (-np.arange(0, 64, 2) / 64)), rtol=1e-5)
