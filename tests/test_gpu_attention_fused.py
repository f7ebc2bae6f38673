"""The attention of one token as ONE launch whose split partials the attn_output linear merges (tga_attention_decode_split + tga_attn_merge_qlinear)
against the two-launch attention followed by the plain linear, and both against a float64 restatement of TransformerBlock._attention
(tinygrad/llm/model.py:180-198: half-split RoPE, KV append, scaled-dot-product attention over positions 0..pos, attn_output + residual); and the
q / k / v launch that also touches the cache rows for that attention (tga_rmsnorm_qlinear_multi_touch), which must change no result."""
import ctypes
import numpy as np, pytest
from oracle import ggml as og, linear as ol

pytestmark = pytest.mark.gpu

def _rope_table(hd, n, theta=500000.0):
  f = (np.float32(1.0) / (np.float32(theta) ** (np.arange(0, hd, 2, dtype=np.float32) / np.float32(hd)))).astype(np.float32)
  ang = (np.arange(n, dtype=np.float32)[:, None] * f[None, :]).astype(np.float32)
  return np.concatenate([np.cos(ang), np.sin(ang)], -1).astype(np.float32)

def _rot(x, row):
  h = x.shape[-1] // 2
  c, s = row[:h], row[h:]
  return np.concatenate([x[..., :h] * c - x[..., h:] * s, x[..., h:] * c + x[..., :h] * s], -1)

def _attention_f64(q, k, v, ck, cv, pos, rope):
  """q (H, hd), k / v (KV, hd) float32 of this token; ck / cv (KV, ctx, hd) the cache as fp16 values; returns the attention row (H * hd) in float64 and the
  fp16 rows appended at pos."""
  H, hd = q.shape
  KV = k.shape[0]
  qr, kr = _rot(q.astype(np.float32), rope[pos]), _rot(k.astype(np.float32), rope[pos])
  k16, v16 = kr.astype(np.float16), v.astype(np.float16)
  K = ck[:, :pos + 1].astype(np.float64).copy(); V = cv[:, :pos + 1].astype(np.float64).copy()
  K[:, pos], V[:, pos] = k16.astype(np.float64), v16.astype(np.float64)
  out = np.zeros((H, hd))
  for h in range(H):
    g = h // (H // KV)
    sc = K[g] @ qr[h].astype(np.float64) / np.sqrt(hd)
    p = np.exp(sc - sc.max()); p /= p.sum()
    out[h] = p @ V[g]
  return out.reshape(-1), k16, v16

CASES = [  # n_heads, n_kv, head_dim, max_ctx, positions
  (32, 8, 128, 1152, [0, 1, 255, 256, 257, 700, 1151]),          # the 8B shape: five splits of 256 positions
  (64, 8, 64, 300, [0, 127, 128, 299]),                          # head_dim 64, three splits of 128
  (16, 4, 256, 64, [0, 5, 63]),                                  # head_dim 256, one split, kv heads not a multiple of 8
  (24, 8, 128, 3072, [3071, 2000, 511, 512]),                    # four tiles per wave, six splits of 512
]

@pytest.mark.parametrize("H,KV,hd,ctx,positions", CASES)
def test_one_launch_attention_and_merging_linear(gpu, H, KV, hd, ctx, positions):
  rt, L = gpu, gpu.lib()
  from tinygrad_amd import synth
  rng = np.random.default_rng(H * 1000 + hd + ctx)
  K, N = H * hd, 512
  ns = ctypes.c_int(0)
  rt.check(L.tga_attention_split_plan(ctx, ctypes.byref(ns)))
  assert 1 <= ns.value <= 6
  w = synth.random_blocks(rng, rt.Q4_0, N, K)
  wf = og.ggml_data_to_tensor(w, N * K, rt.Q4_0).reshape(N, K).astype(np.float64)
  wb = rt.Buffer.from_numpy(w)
  rope = _rope_table(hd, ctx)
  ck0 = (rng.standard_normal((KV, ctx, hd)) * 0.7).astype(np.float16)
  cv0 = rng.standard_normal((KV, ctx, hd)).astype(np.float16)
  part_old = rt.Buffer((H * ((ctx + 63) // 64) * (hd + 2),), np.float32).zero_()
  part_new = rt.Buffer((H * (ns.value * hd + 16),), np.float32).zero_()
  ropeb = rt.Buffer.from_numpy(rope)
  for pos in positions:
    q = rng.standard_normal((H, hd)).astype(np.float32); k = rng.standard_normal((KV, hd)).astype(np.float32); v = rng.standard_normal((KV, hd)).astype(np.float32)
    x = rng.standard_normal((1, N)).astype(np.float32)
    st = np.zeros(16, np.int32); st[0] = pos
    ref_row, k16, v16 = _attention_f64(q, k, v, ck0, cv0, pos, rope)
    y_ref = x[0] + wf @ ref_row
    res = {}
    for name in ("two launches", "one launch"):
      cK, cV, stb = rt.Buffer.from_numpy(ck0), rt.Buffer.from_numpy(cv0), rt.Buffer.from_numpy(st)
      qb, kb, vb, y = rt.Buffer.from_numpy(q), rt.Buffer.from_numpy(k), rt.Buffer.from_numpy(v), rt.Buffer.from_numpy(x.copy())
      if name == "two launches":
        attn = rt.Buffer((1, K), np.float16)
        rt.check(L.tga_attention_decode(qb.ptr, kb.ptr, vb.ptr, cK.ptr, cV.ptr, part_old.ptr, stb.ptr, H, KV, hd, ctx, ropeb.ptr, attn.ptr, None, 0, None))
        wv, yv, rv, nv = (ctypes.c_void_p * 1)(wb.ptr), (ctypes.c_void_p * 1)(y.ptr), (ctypes.c_void_p * 1)(y.ptr), (ctypes.c_int64 * 1)(N)
        rt.check(L.tga_qlinear_multi(rt.Q4_0, 1, wv, yv, nv, attn.ptr, rt.dtype_code(np.float16), rt.dtype_code(np.float32), 1, K, 1, rv, 0, 0, None))
      else:
        rt.check(L.tga_attention_decode_split(qb.ptr, kb.ptr, vb.ptr, cK.ptr, cV.ptr, part_new.ptr, stb.ptr, H, KV, hd, ctx, ropeb.ptr, None))
        rt.check(L.tga_attn_merge_qlinear(rt.Q4_0, wb.ptr, y.ptr, N, K, y.ptr, part_new.ptr, ns.value, hd, None))
      rt.synchronize()
      assert int(stb.numpy()[4]) == 0
      res[name] = (y.numpy()[0].copy(), cK.numpy(), cV.numpy())
      e = ol.rel_err(res[name][0], y_ref)
      assert e <= 1e-3, f"{name} at position {pos}: rel-err {e:.2e} against the float64 attention + linear"
      # the appended rows: the float32 rotation rounded to fp16 (the kernel may contract x1 c - x2 s into a fused multiply-add: one fp16 ulp); every other
      # cache row untouched
      np.testing.assert_allclose(res[name][1][:, pos].astype(np.float32), k16.astype(np.float32), rtol=2e-3, atol=2e-3); np.testing.assert_array_equal(res[name][2][:, pos], v16)
      keep = np.ones(ctx, bool); keep[pos] = False
      np.testing.assert_array_equal(res[name][1][:, keep], ck0[:, keep]); np.testing.assert_array_equal(res[name][2][:, keep], cv0[:, keep])
    np.testing.assert_array_equal(res["one launch"][1], res["two launches"][1])      # both paths append the same key bits
    # the two paths group their sums differently, so an fp16 activation may round the other way: close, not bit-equal
    assert ol.rel_err(res["one launch"][0], res["two launches"][0]) <= 2e-4

@pytest.mark.parametrize("H,KV,hd,ctx,per_head", [(16, 16, 128, 576, 0), (8, 2, 128, 300, 1), (32, 8, 128, 1152, 1), (16, 4, 64, 200, 0), (4, 2, 256, 128, 1)],
                         ids=["olmoe-whole-row", "qwen3-per-head-k1024", "per-head-k4096", "whole-row-hd64", "per-head-hd256"])
def test_one_launch_attention_with_qk_norm(gpu, H, KV, hd, ctx, per_head):
  """tga_attention_decode_split_normed + tga_attn_merge_qlinear against tga_attention_decode_normed followed by the plain linear: the q / k RMSNorm over the whole
  rows (model.py:169) or per head (model.py:180), attn_output rows of 1024 .. 4096 values (rows of at most 32 units take the whole-wave kernel with idle lanes),
  and both against the float64 attention of the normalised rows."""
  rt, L = gpu, gpu.lib()
  from tinygrad_amd import synth
  rng = np.random.default_rng(H * 100 + hd + ctx + per_head)
  K, N = H * hd, 384
  ns = ctypes.c_int(0)
  rt.check(L.tga_attention_split_plan(ctx, ctypes.byref(ns)))
  w = synth.random_blocks(rng, rt.Q8_0, N, K)
  wf = og.ggml_data_to_tensor(w, N * K, rt.Q8_0).reshape(N, K).astype(np.float64)
  wb = rt.Buffer.from_numpy(w)
  rope = _rope_table(hd, ctx); ropeb = rt.Buffer.from_numpy(rope)
  ck0 = (rng.standard_normal((KV, ctx, hd)) * 0.7).astype(np.float16); cv0 = rng.standard_normal((KV, ctx, hd)).astype(np.float16)
  qw = (1 + 0.3 * rng.standard_normal(hd if per_head else H * hd)).astype(np.float32); kw = (1 + 0.3 * rng.standard_normal(hd if per_head else KV * hd)).astype(np.float32)
  qwb, kwb = rt.Buffer.from_numpy(qw), rt.Buffer.from_numpy(kw)
  eps = 1e-6
  def normed(x, wgt):                                                        # float32 RMSNorm as the kernels take it: (x * rsqrt(mean(x^2) + eps)) * weight
    if per_head: return ((x / np.sqrt((x.astype(np.float64) ** 2).mean(-1, keepdims=True) + eps)) * wgt).astype(np.float32)
    flat = x.reshape(-1)
    return ((flat / np.sqrt((flat.astype(np.float64) ** 2).mean() + eps)) * wgt).astype(np.float32).reshape(x.shape)
  part_old = rt.Buffer((H * ((ctx + 63) // 64) * (hd + 2),), np.float32).zero_()
  part_new = rt.Buffer((H * (ns.value * hd + 16),), np.float32).zero_()
  for pos in (0, 1, min(127, ctx - 1), min(130, ctx - 1), ctx - 1):
    q = (rng.standard_normal((H, hd)) * 2).astype(np.float32); k = (rng.standard_normal((KV, hd)) * 3).astype(np.float32); v = rng.standard_normal((KV, hd)).astype(np.float32)
    x = rng.standard_normal((1, N)).astype(np.float32)
    st = np.zeros(16, np.int32); st[0] = pos
    ref_row, k16, v16 = _attention_f64(normed(q, qw), normed(k, kw), v, ck0, cv0, pos, rope)
    y_ref = x[0] + wf @ ref_row
    res = {}
    for name in ("two launches", "one launch"):
      cK, cV, stb = rt.Buffer.from_numpy(ck0), rt.Buffer.from_numpy(cv0), rt.Buffer.from_numpy(st)
      qb, kb, vb, y = rt.Buffer.from_numpy(q), rt.Buffer.from_numpy(k), rt.Buffer.from_numpy(v), rt.Buffer.from_numpy(x.copy())
      if name == "two launches":
        attn = rt.Buffer((1, K), np.float16)
        rt.check(L.tga_attention_decode_normed(qb.ptr, kb.ptr, vb.ptr, qwb.ptr, kwb.ptr, eps, per_head, cK.ptr, cV.ptr, part_old.ptr, stb.ptr, H, KV, hd, ctx, ropeb.ptr, attn.ptr, None, 0, None))
        wv, yv, rv, nv = (ctypes.c_void_p * 1)(wb.ptr), (ctypes.c_void_p * 1)(y.ptr), (ctypes.c_void_p * 1)(y.ptr), (ctypes.c_int64 * 1)(N)
        rt.check(L.tga_qlinear_multi(rt.Q8_0, 1, wv, yv, nv, attn.ptr, rt.dtype_code(np.float16), rt.dtype_code(np.float32), 1, K, 1, rv, 0, 0, None))
      else:
        rt.check(L.tga_attention_decode_split_normed(qb.ptr, kb.ptr, vb.ptr, qwb.ptr, kwb.ptr, eps, per_head, cK.ptr, cV.ptr, part_new.ptr, stb.ptr, H, KV, hd, ctx, ropeb.ptr, None))
        rt.check(L.tga_attn_merge_qlinear(rt.Q8_0, wb.ptr, y.ptr, N, K, y.ptr, part_new.ptr, ns.value, hd, None))
      rt.synchronize()
      assert int(stb.numpy()[4]) == 0
      res[name] = (y.numpy()[0].copy(), cK.numpy(), cV.numpy())
      e = ol.rel_err(res[name][0], y_ref)
      assert e <= 1e-3, f"{name} at position {pos}: rel-err {e:.2e} against the float64 attention + linear"
      np.testing.assert_allclose(res[name][1][:, pos].astype(np.float32), k16.astype(np.float32), rtol=2e-3, atol=2e-3); np.testing.assert_array_equal(res[name][2][:, pos], v16)
      keep = np.ones(ctx, bool); keep[pos] = False
      np.testing.assert_array_equal(res[name][1][:, keep], ck0[:, keep]); np.testing.assert_array_equal(res[name][2][:, keep], cv0[:, keep])
    assert ol.rel_err(res["one launch"][0], res["two launches"][0]) <= 2e-4
    # (the two kernels sum the squares in different orders: an appended key may differ by one fp16 ulp)
    np.testing.assert_allclose(res["one launch"][1][:, pos].astype(np.float32), res["two launches"][1][:, pos].astype(np.float32), rtol=2e-3, atol=2e-3)

def test_one_launch_attention_refuses_what_it_cannot_serve(gpu):
  rt, L = gpu, gpu.lib()
  ns = ctypes.c_int(7)
  rt.check(L.tga_attention_split_plan(3073, ctypes.byref(ns)))
  assert ns.value == 0                                                      # more than six splits of 512 positions: the caller keeps the two-launch attention
  b = rt.Buffer((4096,), np.float32).zero_()
  st = rt.Buffer.from_numpy(np.zeros(16, np.int32))
  assert L.tga_attention_decode_split(b.ptr, b.ptr, b.ptr, b.ptr, b.ptr, b.ptr, st.ptr, 8, 8, 128, 4096, b.ptr, None) != 0
  assert L.tga_attention_decode_split(b.ptr, b.ptr, b.ptr, b.ptr, b.ptr, b.ptr, st.ptr, 8, 3, 128, 64, b.ptr, None) != 0      # heads not a multiple of kv heads
  assert L.tga_attn_merge_qlinear(rt.Q4_0, b.ptr, b.ptr, 64, 8192, b.ptr, b.ptr, 2, 128, None) != 0                              # rows of more than 64 units
  assert L.tga_attn_merge_qlinear(rt.Q4_0, b.ptr, b.ptr, 64, 4096, b.ptr, b.ptr, 7, 128, None) != 0                              # more than six splits
  # a position outside the cache: flag, nothing written
  st2 = np.zeros(16, np.int32); st2[0] = 64
  stb = rt.Buffer.from_numpy(st2)
  ck = rt.Buffer.from_numpy(np.ones((8, 64, 128), np.float16)); part = rt.Buffer((8 * (1 * 128 + 16),), np.float32).zero_()
  rt.check(L.tga_attention_decode_split(b.ptr, b.ptr, b.ptr, ck.ptr, ck.ptr, part.ptr, stb.ptr, 8, 8, 128, 64, b.ptr, None))
  rt.synchronize()
  assert int(stb.numpy()[4]) == 2 and np.all(ck.numpy() == 1) and not part.numpy().any()

def test_qkv_launch_with_cache_touch_changes_nothing(gpu):
  rt, L = gpu, gpu.lib()
  from tinygrad_amd import synth
  from tinygrad_amd.nn import QuantLinear, qlinear_multi
  rng = np.random.default_rng(5)
  K, KV, hd, ctx = 4096, 8, 128, 1152
  lins = [QuantLinear(rt.Buffer.from_numpy(synth.random_blocks(rng, rt.Q4_0, n, K)), rt.Q4_0, n, K) for n in (4096, 1024, 1024)]
  x = rt.Buffer.from_numpy((rng.standard_normal((1, K)) * 2).astype(np.float32))
  nw = rt.Buffer.from_numpy(rng.uniform(0.5, 1.5, K).astype(np.float32))
  ck = rt.Buffer.from_numpy(rng.standard_normal((KV, ctx, hd)).astype(np.float16)); cv = rt.Buffer.from_numpy(rng.standard_normal((KV, ctx, hd)).astype(np.float16))
  rope = rt.Buffer.from_numpy(_rope_table(hd, ctx))
  outs = {}
  for pos in (None, 0, 1, 700, ctx - 1, ctx + 5, -3):                       # (positions outside the cache are clamped: the touch never leaves the buffers)
    o = [rt.Buffer((1, l.out_features), np.float32) for l in lins]
    if pos is None: qlinear_multi(lins, x, o, norm=(nw, 1e-5))
    else:
      st = np.zeros(16, np.int32); st[0] = pos
      qlinear_multi(lins, x, o, norm=(nw, 1e-5), touch=(rt.Buffer.from_numpy(st), ck, cv, rope, KV, hd, ctx))
    rt.synchronize()
    outs[pos] = np.concatenate([b.numpy()[0] for b in o])
  for pos in outs: np.testing.assert_array_equal(outs[pos], outs[None])

WIDE = dict(num_blocks=2, dim=512, hidden_dim=1024, n_heads=32, n_kv_heads=8, norm_eps=1e-5, vocab_size=512, head_dim=128, rope_theta=500000.0)

def test_model_on_the_one_launch_attention_vs_oracle(gpu):
  """A model whose attention width (32 heads of 128) puts it on the one-launch attention with the cache touch: 32 greedy tokens and the logits of
  every step against the oracle run with the reference's numerics, over a prompt that crosses a split boundary."""
  from tinygrad_amd.llm import Transformer, TransformerConfig, synth_state
  from oracle import llm as ollm
  from decode_helpers import greedy_vs_reference_numerics
  c = TransformerConfig(max_context=320, **WIDE)                             # three splits of 128 positions
  sd = synth_state(c, seed=11)
  gpu.synchronize()
  host = {k: (b.numpy(), t, shp) for k, (b, t, shp) in sd.items()}
  model = Transformer(c, sd, max_new=64)
  assert model.blk[0].fused_attn == 3 and model.blk[0].kv_touch
  rng = np.random.default_rng(12)
  prompt = [int(t) for t in rng.integers(0, WIDE["vocab_size"], size=120)]
  oref = ollm.Model(WIDE, host, 320, act_round_f16=False)
  got, ref, worst, margin, rms = greedy_vs_reference_numerics(model, oref, prompt, 32)
  print(f"min top-2 margin {margin:.4f} (logit rms {rms:.4f}); worst logits rel-err {worst:.2e}")
  assert got == ref
  assert worst <= 1e-3
