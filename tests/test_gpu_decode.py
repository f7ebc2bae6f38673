"""Greedy decode of a small llama-architecture model on the GPU vs the numpy restatement of tinygrad/llm/model.py.

The weights are written on the GPU as GGUF blocks; the SAME bytes are read back and given to the oracle, which runs the REFERENCE's
numerics (float32 activations into fp16-rounded weights, model.py:359, 376; fp16 KV cache as benchmark configuration 3 states).  Bars:
the first 32 greedy tokens equal the oracle's (its minimum top-2 margin is printed), and the logits of every one of those steps
within rel-err 1e-3 of the oracle's logits for the same token history."""
import numpy as np, pytest
from oracle import llm as ollm, linear as ol
from decode_helpers import greedy_vs_reference_numerics

pytestmark = pytest.mark.gpu

SMALL = dict(num_blocks=2, dim=256, hidden_dim=512, n_heads=4, n_kv_heads=2, norm_eps=1e-5, vocab_size=512, head_dim=64, rope_theta=500000.0)

def _build(gpu, cfg, max_context, seed=1003, linear_type=None):
  from tinygrad_amd.llm import Transformer, TransformerConfig, synth_state
  from tinygrad_amd import runtime as rt
  c = TransformerConfig(max_context=max_context, **cfg)
  sd = synth_state(c, seed=seed, linear_type=rt.Q4_0 if linear_type is None else linear_type)
  gpu.synchronize()
  host = {k: (b.numpy(), t, shp) for k, (b, t, shp) in sd.items()}
  return Transformer(c, sd, max_new=64), host

def test_small_model_logits_and_tokens(gpu):
  model, host = _build(gpu, SMALL, 128)
  rng = np.random.default_rng(1003)
  prompt = [int(t) for t in rng.integers(0, SMALL["vocab_size"], size=70)]      # spans two 64-position attention splits
  oref = ollm.Model(SMALL, host, 128, act_round_f16=False)                      # the reference's numerics: nothing of the build's rounding
  got, ref, worst, margin, rms = greedy_vs_reference_numerics(model, oref, prompt, 32)
  print(f"oracle (reference numerics) min top-2 logit margin over 32 steps: {margin:.4f} (logit rms {rms:.4f}); worst logits rel-err {worst:.2e}")
  assert got == ref
  assert worst <= 1e-3

def test_context_and_token_guards(gpu):
  """The sequence ends at max_context like the reference's generate loop (tinygrad/llm/model.py:475), ids outside the vocabulary are refused on
  the host, and the kernels themselves refuse (flag, no access) a position or token outside their tables."""
  model, _ = _build(gpu, SMALL, 64, seed=3)
  out = list(model.generate([1, 2, 3], 1000))
  assert len(out) == 61                                                          # 3 prompt tokens + 61 generated = max_context
  model.decode_step()                                                            # the last cache position (63) can still be processed ...
  with pytest.raises(RuntimeError, match="context full"): model.decode_step()    # ... position 64 does not exist
  with pytest.raises(ValueError): model.reset([SMALL["vocab_size"]])
  with pytest.raises(ValueError): model.reset([-1])
  with pytest.raises(ValueError): model.reset(list(range(64)))
  # device-side refusal: a state record whose position / token lie outside the tables
  model.reset([1, 2])
  st = model.s.state.numpy(); st[0] = 64; model.s.state.copyin(st)             # pos == max_context
  before = model.blk[0].cache_k.numpy().copy()
  model._step(True); model.stream.synchronize()
  np.testing.assert_array_equal(model.blk[0].cache_k.numpy(), before)
  with pytest.raises(RuntimeError, match="position beyond max_context"): model.check_state()
  model.reset([1, 2])
  st = model.s.state.numpy(); st[1] = 1 << 30; model.s.state.copyin(st)        # token id far outside the table
  model._step(True); model.stream.synchronize()
  with pytest.raises(RuntimeError, match="token id outside the vocabulary"): model.check_state()
  # NaN logits: the argmax stays inside the row (index 0), never 2^31 - 1
  lg = np.full(SMALL["vocab_size"], np.nan, np.float32)
  stb = gpu.Buffer.from_numpy(np.zeros(16, np.int32)); outt = gpu.Buffer((4,), np.int32).zero_(); pr = gpu.Buffer((8,), np.int32).zero_()
  lgb, sv, si = gpu.Buffer.from_numpy(lg), gpu.Buffer((256,), np.float32), gpu.Buffer((256,), np.int32)
  gpu.check(gpu.lib().tga_argmax_step(lgb.ptr, lg.size, sv.ptr, si.ptr, stb.ptr, pr.ptr, outt.ptr, 4, None))
  assert outt.numpy()[0] == 0

@pytest.mark.parametrize("replay", ["cmdlist", "graph"])
def test_graph_replay_equals_eager(gpu, replay):
  """The captured step replayed as plain launches in capture order (tga_cmdlist_*) and through hipGraphLaunch: same tokens and logits as eager
  launches, over several replays with host synchronisation between them."""
  model, _ = _build(gpu, SMALL, 128, seed=77)
  model.replay = replay
  prompt = [5, 17, 300, 42, 8]
  a = list(model.generate(prompt, 16, use_graph=False))
  la = model.logits().copy()
  b = list(model.generate(prompt, 16, use_graph=True))
  assert a == b
  np.testing.assert_array_equal(la, model.logits())
  if replay == "cmdlist": assert len(model._graph(True)) > 10                          # one entry per kernel of the step

def test_kv_prefix_reuse_equals_fresh_model(gpu):
  """A prompt that shares a prefix with what the KV cache holds is prefilled from the first differing position only (Transformer.get_start_pos,
  tinygrad/llm/model.py:455-462, used at 472-473), with the tokens and logits of a model that starts from nothing; a follow-up turn (prompt +
  reply + new tokens) runs only the new tokens."""
  model, _ = _build(gpu, SMALL, 128, seed=11)
  fresh, _ = _build(gpu, SMALL, 128, seed=11)
  model.prefill_chunk = fresh.prefill_chunk = 1                                          # token by token on both sides: the comparison below is bit for bit
  rng = np.random.default_rng(11)
  p1 = [int(t) for t in rng.integers(0, SMALL["vocab_size"], size=70)]
  p2 = p1[:40] + [int(t) for t in rng.integers(0, SMALL["vocab_size"], size=12)]
  if p2[40] == p1[40]: p2[40] = (p2[40] + 1) % SMALL["vocab_size"]
  list(model.generate(p1, 8))
  assert model.prefill_steps == 69
  assert model.get_start_pos(p2) == 40
  got = list(model.generate(p2, 8)); lg = model.logits().copy()
  assert model.prefill_steps == len(p2) - 1 - 40
  want = list(fresh.generate(p2, 8))
  assert fresh.prefill_steps == len(p2) - 1
  assert got == want
  np.testing.assert_array_equal(lg, fresh.logits())
  p3 = p2 + got + [7, 9, 11]                                                            # the next turn of a conversation
  got3 = list(model.generate(p3, 8)); lg3 = model.logits().copy()
  assert model.prefill_steps == 3
  fresh2, _ = _build(gpu, SMALL, 128, seed=11)
  fresh2.prefill_chunk = 1
  assert got3 == list(fresh2.generate(p3, 8))
  np.testing.assert_array_equal(lg3, fresh2.logits())
  assert model.get_start_pos(p3) == len(p3) - 1                                          # the same prompt again: nothing to prefill
  assert list(model.generate(p3, 8)) == got3 and model.prefill_steps == 0
  model.prefill(p3, reuse_cache=False)
  assert model.prefill_steps == len(p3) - 1

@pytest.mark.parametrize("chunk", [8, 16, 5, 32, 24, 64, 128, 100])
@pytest.mark.parametrize("n_prompt", [9, 17, 61, 70, 131, 180])
def test_chunked_prefill_vs_token_by_token_and_oracle(gpu, n_prompt, chunk):
  """Prompt positions computed eight, sixteen or thirty-two (or five, or twenty-four) at a time (small-batch linears, causal attention inside the chunk: Transformer.generate's chunked prefill,
  tinygrad/llm/model.py:464, 476-481) against the same model prefilled token by token and against the oracle: the KV caches agree to fp16 rounding of
  slightly different float32 results, the logits of the following decode steps stay within 1e-3 of the oracle's for the same token history, and the
  greedy tokens are the oracle's.  Prompt lengths that leave 0..7 positions behind the whole chunks (computed by one more chunk that ends at the last position) and cross the 64-position splits."""
  model, host = _build(gpu, SMALL, 192, seed=21)
  single, _ = _build(gpu, SMALL, 192, seed=21)
  model.prefill_chunk, single.prefill_chunk = chunk, 1
  rng = np.random.default_rng(21 + n_prompt)
  prompt = [int(t) for t in rng.integers(0, SMALL["vocab_size"], size=n_prompt)]
  model.prefill(prompt); single.prefill(prompt)
  assert model.prefill_steps == single.prefill_steps == n_prompt - 1
  assert (model._chunker is not None) == (n_prompt - 1 >= chunk) and single._chunker is None
  for bm, bs in zip(model.blk, single.blk):
    for cm, cs in ((bm.cache_k, bs.cache_k), (bm.cache_v, bs.cache_v)):
      a, b = cm.numpy().astype(np.float32)[:, :n_prompt - 1], cs.numpy().astype(np.float32)[:, :n_prompt - 1]
      assert ol.rel_err(a, b) <= 2e-3
      assert not cm.numpy()[:, n_prompt - 1:].any()                                    # nothing beyond the prompt was written
  oref = ollm.Model(SMALL, host, 192, act_round_f16=False)
  got, ref, worst, margin, rms = greedy_vs_reference_numerics(model, oref, prompt, 12)
  print(f"prompt {n_prompt}: min top-2 margin {margin:.4f}, worst logits rel-err {worst:.2e}")
  assert got == ref and worst <= 1e-3

@pytest.mark.parametrize("ltype,chunk", [("Q4_0", 64), ("Q8_0", 24), ("Q4_K", 40), ("Q6_K", 32), ("Q4_K_M", 48), ("Q4_0", 128), ("Q4_K_M", 100), ("Q8_0", 72)])
def test_prefill_steps_with_rows_in_the_multiplying_layout_equal_the_plain_steps(gpu, monkeypatch, ltype, chunk):
  """A prefill in steps of 17 .. 128 positions hands its rows from launch to launch in the layout the prefill kernel multiplies from and lets the norm launches complete
  the split-K sums (BatchedTransformer.rows64); with TGA_ROWS64=0 the same steps run on plain rows.  Same kernels on the same fp16 values: the KV caches agree to the order
  of a float32 sum, the decode steps that follow give the same tokens."""
  from tinygrad_amd import runtime as rt
  cfg = dict(SMALL, dim=512, hidden_dim=1024, n_heads=8, n_kv_heads=2) if ltype in ("Q4_K", "Q6_K", "Q4_K_M") else SMALL
  rng = np.random.default_rng(64 + chunk)
  prompt = [int(t) for t in rng.integers(0, cfg["vocab_size"], size=150)]
  caches, toks = [], []
  for flag in ("1", "0"):
    monkeypatch.setenv("TGA_ROWS64", flag)
    if ltype == "Q4_K_M":                                                                # Q4_K with attn_v / ffn_down as Q6_K in half of the blocks: q / k and v are two launches
      from tinygrad_amd.llm import Transformer, TransformerConfig, synth_state
      c = TransformerConfig(max_context=192, **cfg)
      model = Transformer(c, synth_state(c, seed=33, q4_k_m=True), max_new=64)
    else: model, _ = _build(gpu, cfg, 192, seed=33, linear_type=getattr(rt, ltype))
    model.prefill_chunk = chunk
    model.prefill(prompt)
    assert bool(model._chunker.rows64) == (flag == "1")
    caches.append([(b.cache_k.numpy().astype(np.float32), b.cache_v.numpy().astype(np.float32)) for b in model.blk])
    toks.append(list(model.generate(prompt, 8)))
  for (k1, v1), (k0, v0) in zip(*caches):
    assert ol.rel_err(k1, k0) <= 1e-3 and ol.rel_err(v1, v0) <= 1e-3
  assert toks[0] == toks[1]

def test_attention_prefill_chunk_kernel_vs_numpy(gpu):
  """tga_attention_prefill_chunk alone: eight consecutive positions per call over one cache (per-head q/k norm, GQA), each row against numpy attention over
  the positions up to its own; tga_chunk_advance moves the position and loads the next ids."""
  from tinygrad_amd.llm import precompute_freqs_cis
  H, KV, hd, ctx, B = 8, 2, 128, 256, 8
  rng = np.random.default_rng(88)
  rope = precompute_freqs_cis(hd, ctx, 10000.0)
  ck, cv = gpu.Buffer((KV, ctx, hd), np.float16).zero_(), gpu.Buffer((KV, ctx, hd), np.float16).zero_()
  part = gpu.Buffer((B * H * ((ctx + 63) // 64) * (hd + 2),), np.float32).zero_()
  ropeb = gpu.Buffer.from_numpy(rope)
  out = gpu.Buffer((B, H * hd), np.float32)
  qw, kw = rng.standard_normal(hd).astype(np.float32), rng.standard_normal(hd).astype(np.float32)
  qwb, kwb = gpu.Buffer.from_numpy(qw), gpu.Buffer.from_numpy(kw)
  prompt = np.arange(ctx, dtype=np.int32) * 3 % 101
  pb, tokb = gpu.Buffer.from_numpy(prompt), gpu.Buffer((B,), np.int32).zero_()
  st = np.zeros(16, np.int32); st[0] = 0
  stb = gpu.Buffer.from_numpy(st)
  rk, rv = np.zeros((KV, ctx, hd), np.float16), np.zeros((KV, ctx, hd), np.float16)
  for chunk in range(18):                                                              # positions 0 .. 143: across two split boundaries
    pos0 = chunk * B
    q, k, v = (rng.standard_normal((B, n)).astype(np.float32) * 1.5 for n in (H * hd, KV * hd, KV * hd))
    qb, kb, vb = (gpu.Buffer.from_numpy(t) for t in (q, k, v))
    gpu.check(gpu.lib().tga_attention_prefill_chunk(B, qb.ptr, kb.ptr, vb.ptr, qwb.ptr, kwb.ptr, 1e-5, 1, ck.ptr, cv.ptr, part.ptr, stb.ptr, H, KV, hd, ctx, ropeb.ptr,
                                                    None, out.ptr, None))
    gpu.check(gpu.lib().tga_chunk_advance(stb.ptr, pb.ptr, B, tokb.ptr, ctx, None))
    gpu.synchronize()
    o = out.numpy()
    for r in range(B):
      pos = pos0 + r
      qn, kn = ollm.rmsnorm(q[r].reshape(H, hd), qw, 1e-5), ollm.rmsnorm(k[r].reshape(KV, hd), kw, 1e-5)
      qr, kr = ollm.apply_rope(qn, rope[pos]), ollm.apply_rope(kn, rope[pos])
      rk[:, pos], rv[:, pos] = kr.astype(np.float16), v[r].reshape(KV, hd).astype(np.float16)
      K = np.repeat(rk[:, :pos + 1].astype(np.float32), H // KV, axis=0); V = np.repeat(rv[:, :pos + 1].astype(np.float32), H // KV, axis=0)
      sc = np.einsum("hd,htd->ht", qr, K) / np.sqrt(hd)
      e = np.exp(sc - sc.max(-1, keepdims=True)); p = e / e.sum(-1, keepdims=True)
      assert ol.rel_err(o[r], np.einsum("ht,htd->hd", p, V).reshape(-1)) <= 1e-4, pos
    assert int(stb.numpy()[0]) == pos0 + B
    np.testing.assert_array_equal(tokb.numpy(), prompt[np.minimum(pos0 + B + np.arange(B), ctx - 1)])
  assert ol.rel_err(ck.numpy().astype(np.float32), rk.astype(np.float32)) < 2e-3

@pytest.mark.parametrize("H,KV,hd,B,ctx", [(8, 2, 128, 16, 256), (8, 2, 128, 37, 256), (4, 4, 64, 64, 256), (16, 2, 64, 24, 256), (8, 8, 128, 17, 256), (8, 1, 128, 9, 256), (8, 2, 128, 128, 256),
                                           (4, 4, 64, 100, 256), (8, 2, 128, 16, 192), (8, 2, 64, 37, 320)])
def test_attention_prefill_chunk_on_the_matrix_cores_vs_numpy(gpu, H, KV, hd, B, ctx):
  """tga_attention_prefill_chunk for more than eight rows without q / k norm (the launch that attends multiplies on the matrix cores: workgroup per kv head, split of two
  64-position tiles walked with a running maximum, and tile of sixteen rows, wave per query head of the group): steps of B consecutive positions over one cache up to
  position 150 and beyond two split boundaries, caches of an odd number of tiles (192, 320 positions: the last split's second tile lies beyond the cache), groups of 1, 4 and 8 query heads per kv head (8: two passes of the four waves), row counts that end inside a tile; every row against numpy attention over the
  positions up to its own.  The rotated queries and the probabilities are rounded to fp16 there: the bar is the linears' 1e-3."""
  from tinygrad_amd.llm import precompute_freqs_cis
  rng = np.random.default_rng(1000 * H + 10 * KV + B)
  rope = precompute_freqs_cis(hd, ctx, 10000.0)
  ck, cv = gpu.Buffer((KV, ctx, hd), np.float16).zero_(), gpu.Buffer((KV, ctx, hd), np.float16).zero_()
  part = gpu.Buffer((B * H * ((ctx + 63) // 64) * (hd + 2),), np.float32).zero_()
  ropeb = gpu.Buffer.from_numpy(rope)
  out = gpu.Buffer((B, H * hd), np.float32)
  out16 = gpu.Buffer((B, H * hd), np.float16)
  prompt = np.arange(ctx, dtype=np.int32)
  pb, tokb = gpu.Buffer.from_numpy(prompt), gpu.Buffer((B,), np.int32).zero_()
  stb = gpu.Buffer.from_numpy(np.zeros(16, np.int32))
  rk, rv = np.zeros((KV, ctx, hd), np.float16), np.zeros((KV, ctx, hd), np.float16)
  worst, pos0 = 0.0, 0
  while pos0 + B <= (150 if ctx == 256 else ctx) + B and pos0 + B < ctx:
    q, k, v = (rng.standard_normal((B, n)).astype(np.float32) * 1.5 for n in (H * hd, KV * hd, KV * hd))
    qb, kb, vb = (gpu.Buffer.from_numpy(t) for t in (q, k, v))
    gpu.check(gpu.lib().tga_attention_prefill_chunk(B, qb.ptr, kb.ptr, vb.ptr, None, None, 0.0, 0, ck.ptr, cv.ptr, part.ptr, stb.ptr, H, KV, hd, ctx, ropeb.ptr,
                                                    out16.ptr, out.ptr, None))
    gpu.check(gpu.lib().tga_chunk_advance(stb.ptr, pb.ptr, B, tokb.ptr, ctx, None))
    gpu.synchronize()
    o = out.numpy()
    np.testing.assert_array_equal(out16.numpy(), o.astype(np.float16))
    for r in range(B):
      pos = pos0 + r
      qr, kr = ollm.apply_rope(q[r].reshape(H, hd), rope[pos]), ollm.apply_rope(k[r].reshape(KV, hd), rope[pos])
      rk[:, pos], rv[:, pos] = kr.astype(np.float16), v[r].reshape(KV, hd).astype(np.float16)
      K = np.repeat(rk[:, :pos + 1].astype(np.float32), H // KV, axis=0); V = np.repeat(rv[:, :pos + 1].astype(np.float32), H // KV, axis=0)
      sc = np.einsum("hd,htd->ht", qr, K) / np.sqrt(hd)
      e = np.exp(sc - sc.max(-1, keepdims=True)); p = e / e.sum(-1, keepdims=True)
      worst = max(worst, ol.rel_err(o[r], np.einsum("ht,htd->hd", p, V).reshape(-1)))
    pos0 += B
    assert int(stb.numpy()[0]) == pos0
  print(f"H {H} KV {KV} hd {hd} B {B}: worst rel-err {worst:.2e}")
  assert worst <= 1e-3, worst
  assert ol.rel_err(ck.numpy().astype(np.float32), rk.astype(np.float32)) < 2e-3
  assert not ck.numpy()[:, pos0:].any() and not cv.numpy()[:, pos0:].any()

def test_command_list_takes_kernel_launches_only(gpu):
  """A capture that holds anything but kernel launches (here a device-to-device copy, which the capture records as a copy node; the graph is never
  instantiated) is refused when the list is built; the stream stays usable."""
  from tinygrad_amd import runtime as rt
  s = rt.Stream()
  buf, src = gpu.Buffer((256,), np.float32), gpu.Buffer((256,), np.float32).zero_()
  cl = rt.CommandList(s)
  with pytest.raises(RuntimeError, match="not a kernel launch"):
    with cl: gpu.check(gpu.lib().tga_memcpy_d2d(buf.ptr, src.ptr, buf.nbytes, s.handle))
  ok = rt.CommandList(s)
  with ok: gpu.check(gpu.lib().tga_synth_weights(0, buf.ptr, 256, 1, 3.0, s.handle))    # a fill kernel: float32 "weights" are a constant fill
  assert len(ok) == 1
  for _ in range(3): ok.launch()
  s.synchronize()
  assert (buf.numpy() == 3.0).all()

# wider shapes: head_dim 128, K split over four waves (K > 4096), Q8_0
WIDE = dict(num_blocks=2, dim=1024, hidden_dim=4608, n_heads=8, n_kv_heads=1, norm_eps=1e-5, vocab_size=512, head_dim=128, rope_theta=10000.0)
WIDE_D = dict(num_blocks=2, dim=4352, hidden_dim=256, n_heads=34, n_kv_heads=17, norm_eps=1e-5, vocab_size=256, head_dim=128, rope_theta=10000.0)

@pytest.mark.parametrize("cfg,ltype", [(WIDE, "Q4_0"), (WIDE, "Q8_0"), (WIDE_D, "Q4_0"), (SMALL, "Q8_0")], ids=["wide-hidden-q4", "wide-hidden-q8", "wide-dim-q4", "small-q8"])
def test_wider_models_vs_reference_numerics(gpu, cfg, ltype):
  from tinygrad_amd import runtime as rt
  model, host = _build(gpu, cfg, 192, seed=11, linear_type=getattr(rt, ltype))
  rng = np.random.default_rng(3)
  prompt = [int(t) for t in rng.integers(0, cfg["vocab_size"], size=67)]
  got, ref, worst, margin, rms = greedy_vs_reference_numerics(model, ollm.Model(cfg, host, 192, act_round_f16=False), prompt, 12)
  print(f"min top-2 margin {margin:.4f}, logit rms {rms:.4f}, worst logits rel-err {worst:.2e}")
  assert got == ref and worst <= 1e-3

@pytest.mark.parametrize("H,KV,hd,normed", [(8, 2, 128, 0), (4, 4, 64, 1), (12, 2, 128, 1), (4, 2, 256, 0), (16, 16, 128, 1), (16, 8, 128, 2), (6, 2, 64, 2)],
                         ids=["gqa4-hd128", "mha-hd64-qknorm", "gqa6-hd128-qknorm", "gqa2-hd256", "mha16-hd128-qknorm", "gqa2-hd128-headnorm", "gqa3-hd64-headnorm"])
def test_attention_decode_kernel_vs_numpy(gpu, H, KV, hd, normed):
  """tga_attention_decode(_normed) alone: (full-width q/k RMSNorm,) RoPE + fp16 KV append + GQA softmax attention at several positions."""
  from tinygrad_amd.llm import precompute_freqs_cis
  ctx = 256
  rng = np.random.default_rng(5 + H)
  rope = precompute_freqs_cis(hd, ctx, 10000.0)
  ck, cv = gpu.Buffer((KV, ctx, hd), np.float16).zero_(), gpu.Buffer((KV, ctx, hd), np.float16).zero_()
  part = gpu.Buffer((H * ((ctx + 63) // 64) * (hd + 2),), np.float32).zero_()
  ropeb = gpu.Buffer.from_numpy(rope)
  out = gpu.Buffer((H * hd,), np.float32)
  # normed: 0 none, 1 full-width q/k norm (weights over all heads), 2 per-head norm (weights of head_dim values)
  qw, kw = (rng.standard_normal(n).astype(np.float32) for n in ((H * hd, KV * hd) if normed != 2 else (hd, hd)))
  qwb, kwb = gpu.Buffer.from_numpy(qw), gpu.Buffer.from_numpy(kw)
  rk, rv = np.zeros((KV, ctx, hd), np.float16), np.zeros((KV, ctx, hd), np.float16)
  for pos in range(0, 140):
    q, k, v = (rng.standard_normal(n).astype(np.float32) * 1.5 for n in (H * hd, KV * hd, KV * hd))
    st = np.zeros(16, np.int32); st[0] = pos
    qb, kb, vb, stb = (gpu.Buffer.from_numpy(t) for t in (q, k, v, st))       # keep the device buffers alive across the launch
    if normed:
      gpu.check(gpu.lib().tga_attention_decode_normed(qb.ptr, kb.ptr, vb.ptr, qwb.ptr, kwb.ptr, 1e-5, int(normed == 2), ck.ptr, cv.ptr, part.ptr, stb.ptr,
                                                      H, KV, hd, ctx, ropeb.ptr, None, out.ptr, 0, None))
      if normed == 2: q, k = ollm.rmsnorm(q.reshape(H, hd), qw, 1e-5).reshape(-1), ollm.rmsnorm(k.reshape(KV, hd), kw, 1e-5).reshape(-1)
      else: q, k = ollm.rmsnorm(q, qw, 1e-5), ollm.rmsnorm(k, kw, 1e-5)
    else:
      gpu.check(gpu.lib().tga_attention_decode(qb.ptr, kb.ptr, vb.ptr, ck.ptr, cv.ptr, part.ptr, stb.ptr, H, KV, hd, ctx, ropeb.ptr, None, out.ptr, 0, None))
    gpu.synchronize()
    qr = ollm.apply_rope(q.reshape(H, hd), rope[pos]); kr = ollm.apply_rope(k.reshape(KV, hd), rope[pos])
    rk[:, pos], rv[:, pos] = kr.astype(np.float16), v.reshape(KV, hd).astype(np.float16)
    if pos in (0, 1, 15, 16, 17, 63, 64, 65, 127, 128, 139):
      K = np.repeat(rk[:, :pos + 1].astype(np.float32), H // KV, axis=0); V = np.repeat(rv[:, :pos + 1].astype(np.float32), H // KV, axis=0)
      sc = np.einsum("hd,htd->ht", qr, K) / np.sqrt(hd)
      e = np.exp(sc - sc.max(-1, keepdims=True)); p = e / e.sum(-1, keepdims=True)
      ref = np.einsum("ht,htd->hd", p, V).reshape(-1)
      assert ol.rel_err(out.numpy(), ref) <= 1e-4, pos
  assert ck.numpy().tobytes() == rk.tobytes() or ol.rel_err(ck.numpy().astype(np.float32), rk.astype(np.float32)) < 2e-3

def test_rmsnorm_argmax_embed(gpu):
  rng = np.random.default_rng(9)
  x = rng.standard_normal(4096).astype(np.float32) * 3; w = rng.standard_normal(4096).astype(np.float32)
  o32 = gpu.Buffer((4096,), np.float32); o16 = gpu.Buffer((4096,), np.float16)
  xb, wb = gpu.Buffer.from_numpy(x), gpu.Buffer.from_numpy(w)
  gpu.check(gpu.lib().tga_rmsnorm(xb.ptr, wb.ptr, 4096, 1e-5, o16.ptr, o32.ptr, 0, None))
  ref = ollm.rmsnorm(x, w, 1e-5)
  np.testing.assert_allclose(o32.numpy(), ref, rtol=2e-6, atol=1e-6)
  assert o16.numpy().tobytes() == o32.numpy().astype(np.float16).tobytes()
  # argmax: first index of the maximum, ties included
  lg = rng.standard_normal(128256).astype(np.float32); lg[[777, 90001]] = 9.0
  st = np.zeros(16, np.int32); st[3] = 0
  stb = gpu.Buffer.from_numpy(st); outt = gpu.Buffer((4,), np.int32).zero_(); pr = gpu.Buffer((8,), np.int32).zero_()
  lgb, sv, si = gpu.Buffer.from_numpy(lg), gpu.Buffer((256,), np.float32), gpu.Buffer((256,), np.int32)
  gpu.check(gpu.lib().tga_argmax_step(lgb.ptr, lg.size, sv.ptr, si.ptr, stb.ptr, pr.ptr, outt.ptr, 4, None))
  assert outt.numpy()[0] == 777 and list(stb.numpy()[:3]) == [1, 777, 1]

@pytest.mark.parametrize("n", [128256, 50257, 1023, 7])
def test_argmax_of_several_rows(gpu, n):
  """tga_argmax_rows_step: the first index of every row's maximum (ties, a maximum in the last elements, rows that start off a 16-byte boundary when n is
  odd, NaN entries that never win) is fed back and stored at out_tokens[step][b]; the shared state moves on once."""
  rng = np.random.default_rng(n)
  B = 5
  lg = rng.standard_normal((B, n)).astype(np.float32)
  lg[0, [n // 3, n - 1]] = 9.0                                       # a tie: the first wins
  lg[1, n - 1] = 11.0                                                # the last element
  lg[2, 0] = 12.0
  lg[3, n // 2] = np.nan; lg[3, n - 2] = 10.0
  lg[4, :] = -np.inf                                                 # nothing compares greater: index 0
  ref = [n // 3, n - 1, 0, n - 2, 0]
  st = np.zeros(16, np.int32)                                        # pos 0, no prompt left (n_prompt 0): every row samples
  stb = gpu.Buffer.from_numpy(st); pr = gpu.Buffer((B, 8), np.int32).zero_()
  toks = gpu.Buffer((B,), np.int32).zero_(); outt = gpu.Buffer((4, B), np.int32).zero_()
  lgb = gpu.Buffer.from_numpy(lg)
  gpu.check(gpu.lib().tga_argmax_rows_step(lgb.ptr, B, n, stb.ptr, pr.ptr, 8, toks.ptr, outt.ptr, 4, None))
  assert list(toks.numpy()) == ref and list(outt.numpy()[0]) == ref
  after = stb.numpy()
  assert after[0] == 1 and after[2] == 1                             # pos and step moved on by one

def test_copy_kernel_and_mfma_peak_run(gpu):
  from tinygrad_amd import runtime as rt
  L = rt.lib()
  a = rt.Buffer.from_numpy(np.arange(1 << 16, dtype=np.uint32)); b = rt.Buffer((1 << 16,), np.uint32).zero_()
  rt.check(L.tga_copy_kernel(b.ptr, a.ptr, a.nbytes, None))
  np.testing.assert_array_equal(b.numpy(), a.numpy())
  assert L.tga_copy_kernel(b.ptr, a.ptr, 24, None) != 0
  scratch = rt.Buffer((64,), np.float32).zero_()
  rt.check(L.tga_mfma_peak(8, 2, scratch.ptr, None)); rt.synchronize()
