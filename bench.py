#!/usr/bin/env python3
"""Headline benchmark: Q4_0 Llama-3-8B-architecture greedy decode at batch 1 on one MI355X (benchmark configuration 3).

A step is one decoded token.  Random-init weights are written on the GPU as GGUF blocks (Q4_0 linears and embedding, Q6_K
lm-head), the fp16 KV cache is prefilled with 1024 random token ids through the model itself, then --warmup + --steps tokens
are decoded greedily, one captured launch sequence per token with a host sync per token (as the reference's generate loop does).
Prints ONE JSON line: tok/s, the roofline of the dominant kernel from HIP-event timings taken live (the fused ffn_norm + ffn_gate + ffn_up +
SwiGLU dequant-GEMV, one of five launches per block), the same figures for the other kernels of a block, a parity gate (outside the timed
region: one more decoded token of the SAME model recomputed on the CPU from the GPU's own KV cache, and every linear of layer 0 on a fresh
row; the run exits non-zero when a bar is missed), a CPU baseline (C restatement of the reference arithmetic on a bounded sample of the
same weights) and the kernel-level figures of the other benchmark configurations measured in the same process."""
import argparse, json, os, sys, time
import numpy as np

HBM_PEAK_GBS = 8000.0
# HBM bytes per launch of the dominant kernel from two rocprofv3 --pmc runs (FETCH_SIZE, then WRITE_SIZE) of
# `python -m tinygrad_amd.benchmarks --traffic`, each scaled by what the same counter reads for a 1 GiB copy kernel (x2.0000 and x1.0000):
# 66 509 824 B fetched + 71 680 B written.  A recorded figure (profiles/qgemv1_gate_up_hbm_traffic.md), not re-measured by this run.
GATE_UP_TRAFFIC_BYTES = 66581504
GATE_UP_ROCPROF_AVG_US = 15.17    # rocprofv3 --kernel-trace --stats average of the same kernel over every call of an eagerly launched run (profiles/decode_llama3_8b_q4_0_kernel_stats.md)
GATE_UP_ROCPROF_B2B_US = 14.40    # the same trace, only the passes that issue the 32 launches back to back (the region the HIP events below bracket)
PARITY_TOL = 1e-3

def _host_layer(model, i):
  b = model.blk[i]
  lins = dict(attn_q=b.attn_q, attn_k=b.attn_k, attn_v=b.attn_v, attn_output=b.attn_output, ffn_gate=b.ffn_gate, ffn_up=b.ffn_up, ffn_down=b.ffn_down)
  return {k: (l.ggml_type, l.blocks.view(0, (l.nbytes,), np.uint8).numpy(), l.out_features, l.in_features) for k, l in lins.items()}

def parity_gate(model, c, threads):
  """Checks, against the C / numpy restatement of the reference's model-path numerics (fp32 activations, fp16-rounded weights, fp32 accumulate,
  fp16 KV cache), (1) the seven linears of layer 0 and 4096 spread rows of the lm-head on a fresh random row, through the same fused entry
  points the decode step uses, and (2) one more decoded token of the benchmark model itself: the CPU recomputes the whole step for the same
  input token from the GPU's own KV cache of the earlier positions and must arrive at the same greedy token with logits within the bar."""
  from oracle import cref, llm as ollm, linear as ol
  from tinygrad_amd import runtime as rt
  from tinygrad_amd.nn import qlinear_multi, stage_activation
  lin = lambda t, w, x, n, k: cref.linear(t, w, np.ascontiguousarray(x, dtype=np.float32).reshape(1, -1), n, k, w_round_f16=True, threads=threads)[0]
  rng = np.random.default_rng(7)
  B = rt.Buffer.from_numpy
  f32 = lambda buf: np.ascontiguousarray(buf.numpy()).view(np.uint8).view(np.float32).reshape(-1)      # norm weights are float32 rows kept in byte buffers
  b0, host0 = model.blk[0], _host_layer(model, 0)
  checked, worst = [], 0.0
  def note(name, got, ref):
    nonlocal worst
    e = ol.rel_err(np.asarray(got).reshape(-1), np.asarray(ref).reshape(-1)); worst = max(worst, e); checked.append({"what": name, "rel_err": float(f"{e:.3e}")})
  # ---- (1) layer 0's launches on a fresh row
  x = (rng.standard_normal((1, c.dim)) * 2).astype(np.float32)
  an, fn = f32(b0.attn_norm), f32(b0.ffn_norm)
  xn = ollm.rmsnorm(x, an, c.norm_eps)
  q, k, v = (rt.Buffer((1, n), np.float32) for n in (b0.attn_q.out_features, b0.attn_k.out_features, b0.attn_v.out_features))
  qlinear_multi([b0.attn_q, b0.attn_k, b0.attn_v], B(x), [q, k, v], norm=(b0.attn_norm, c.norm_eps))
  for nm, got in (("attn_q", q), ("attn_k", k), ("attn_v", v)): note("blk.0." + nm, got.numpy(), lin(*host0[nm][:2], xn, *host0[nm][2:]))
  attn = rng.standard_normal((1, b0.attn_output.in_features)).astype(np.float16)
  h = B(x.copy())
  qlinear_multi([b0.attn_output], stage_activation(b0.attn_output, B(attn)) if b0.stage_attn else B(attn), [h], epilogue=1, resid=[h], x_staged=b0.stage_attn)
  note("blk.0.attn_output + residual", h.numpy(), x[0] + lin(*host0["attn_output"][:2], attn, *host0["attn_output"][2:]))
  act = rt.Buffer((1, c.hidden_dim), np.float16)
  qlinear_multi([b0.ffn_gate, b0.ffn_up], h, [act], epilogue=2, norm=(b0.ffn_norm, c.norm_eps))
  hn = ollm.rmsnorm(h.numpy(), fn, c.norm_eps)
  aref = ollm.silu(lin(*host0["ffn_gate"][:2], hn, *host0["ffn_gate"][2:])) * lin(*host0["ffn_up"][:2], hn, *host0["ffn_up"][2:])
  note("blk.0.silu(ffn_gate) * ffn_up", act.numpy(), aref)
  a16 = aref.astype(np.float16).reshape(1, -1)
  out = B(h.numpy())
  qlinear_multi([b0.ffn_down], stage_activation(b0.ffn_down, B(a16)) if b0.stage_act else B(a16), [out], epilogue=1, resid=[out], x_staged=b0.stage_act)
  note("blk.0.ffn_down + residual", out.numpy(), h.numpy()[0] + lin(*host0["ffn_down"][:2], a16, *host0["ffn_down"][2:]))
  head = model.output
  row_bytes = head.nbytes // head.out_features
  lg = rt.Buffer((1, c.vocab_size), np.float32)
  qlinear_multi([head], B(x), [lg], norm=(model.output_norm, c.norm_eps))
  xo = ollm.rmsnorm(x, f32(model.output_norm), c.norm_eps)
  lgh = lg.numpy()[0]
  got_rows, ref_rows = [], []
  for r0 in np.linspace(0, c.vocab_size - 512, 8).astype(int):
    r0 = int(r0) & ~1
    wslice = head.blocks.view(r0 * row_bytes, (512 * row_bytes,), np.uint8).numpy()
    ref_rows.append(lin(head.ggml_type, wslice, xo, 512, c.dim)); got_rows.append(lgh[r0:r0 + 512])
  note("output_norm + lm-head (8 x 512 spread rows)", np.concatenate(got_rows), np.concatenate(ref_rows))
  # ---- (2) one more token of the benchmark model, recomputed on the CPU from the GPU's KV cache
  st = model.s.state.numpy()
  pos, tok = int(st[0]), int(st[1])
  model.decode_step(True)
  lg_gpu, tok_gpu = model.logits(), int(model.s.state.numpy()[1])
  H, KV, hd = c.n_heads, c.n_kv_heads, c.head_dim
  fc = ollm.precompute_freqs_cis(hd, pos + 1, c.rope_theta)[pos]
  emb_row_bytes = model.token_embd.nbytes // c.vocab_size
  from oracle import ggml as og
  xr = og.ggml_data_to_tensor(model.token_embd.view(tok * emb_row_bytes, (emb_row_bytes,), np.uint8).numpy(), c.dim, model.embd_type).astype(np.float16).astype(np.float32)   # the table is an fp16 weight (model.py:376)
  cpu_s = 0.0                                                    # CPU time of the recomputed step itself (weights and KV rows already copied to the host)
  for i, b in enumerate(model.blk):
    hl = _host_layer(model, i)
    ck, cv = b.cache_k.numpy()[:, :pos + 1].astype(np.float32), b.cache_v.numpy()[:, :pos + 1].astype(np.float32)
    an_w, fn_w = f32(b.attn_norm), f32(b.ffn_norm)
    t0 = time.perf_counter()
    n1 = ollm.rmsnorm(xr, an_w, c.norm_eps)
    qv, kv_, vv = (lin(*hl[nm][:2], n1, *hl[nm][2:]) for nm in ("attn_q", "attn_k", "attn_v"))
    qr, kr = ollm.apply_rope(qv.reshape(H, hd), fc), ollm.apply_rope(kv_.reshape(KV, hd), fc)
    ck[:, pos], cv[:, pos] = kr.astype(np.float16).astype(np.float32), vv.reshape(KV, hd).astype(np.float16).astype(np.float32)   # this token's own rows, recomputed
    Kh, Vh = np.repeat(ck, H // KV, axis=0), np.repeat(cv, H // KV, axis=0)
    sc = np.einsum("hd,htd->ht", qr, Kh).astype(np.float32) / np.float32(np.sqrt(hd))
    e = np.exp(sc - sc.max(-1, keepdims=True)); pr = e / e.sum(-1, keepdims=True)
    at = np.einsum("ht,htd->hd", pr, Vh).astype(np.float32).reshape(-1)
    hh = xr + lin(*hl["attn_output"][:2], at, *hl["attn_output"][2:])
    n2 = ollm.rmsnorm(hh, fn_w, c.norm_eps)
    ff = ollm.silu(lin(*hl["ffn_gate"][:2], n2, *hl["ffn_gate"][2:])) * lin(*hl["ffn_up"][:2], n2, *hl["ffn_up"][2:])
    xr = hh + lin(*hl["ffn_down"][:2], ff, *hl["ffn_down"][2:])
    cpu_s += time.perf_counter() - t0
  head_w = head.blocks.view(0, (head.nbytes,), np.uint8).numpy()
  t0 = time.perf_counter()
  xo = ollm.rmsnorm(xr, f32(model.output_norm), c.norm_eps)
  lg_cpu = lin(head.ggml_type, head_w, xo, c.vocab_size, c.dim)
  cpu_s += time.perf_counter() - t0
  note(f"full decode step at position {pos} ({c.num_blocks} blocks + lm-head): logits", lg_gpu, lg_cpu)
  top2 = np.partition(lg_cpu, -2)[-2:]
  tok_cpu = int(np.argmax(lg_cpu))
  res = {"bar_rel_err": PARITY_TOL, "max_rel_err": float(f"{worst:.3e}"), "greedy_token_gpu": tok_gpu, "greedy_token_cpu": tok_cpu,
         "cpu_top2_margin": float(f"{float(top2[1] - top2[0]):.4e}"), "checked": checked,
         "cpu_full_step": {"seconds": round(cpu_s, 3), "tok_s": round(1.0 / cpu_s, 4), "threads": int(threads), "context": pos + 1,
                           "what": "the whole recomputed token (32 blocks with attention and norms + lm-head) on the host, one pass, weights and KV rows already in host memory"},
         "ok": bool(worst <= PARITY_TOL and tok_gpu == tok_cpu)}
  return res

def cpu_baseline(model, cfg, threads_all, parity=None):
  """Times oracle/c (scalar C restatement of dequant + fp32-accumulate matmul, model-path numerics) on the GPU box's host
  cores: the 7 linears of layer 0 plus a 1/32 row slice of the lm-head, extrapolated to one token (32 layers + full head).  Protocol: 2 warm-up
  passes, then the median of 5 timed passes (7 on one thread when they fit 20 s), wall clock."""
  from oracle import cref
  host = list(_host_layer(model, 0).values())
  head = model.output
  hrows = head.out_features // 32
  hbytes = hrows * (head.nbytes // head.out_features)
  hw = head.blocks.view(0, (hbytes,), np.uint8).numpy()
  rng = np.random.default_rng(0)
  def one_pass(threads):
    t0 = time.perf_counter()
    for t, w, n, k in host: cref.linear(t, w, rng.standard_normal((1, k)).astype(np.float32), n, k, w_round_f16=True, threads=threads)
    t1 = time.perf_counter()
    cref.linear(head.ggml_type, hw, rng.standard_normal((1, head.in_features)).astype(np.float32), hrows, head.in_features, w_round_f16=True, threads=threads)
    t2 = time.perf_counter()
    return (t1 - t0), (t2 - t1) * 32
  def measure(threads, budget_s):
    one_pass(threads); one_pass(threads)                  # two warm-ups
    reps, t_start = [], time.perf_counter()
    while len(reps) < 5 or (len(reps) < 7 and time.perf_counter() - t_start < budget_s): reps.append(one_pass(threads))
    return 1.0 / (cfg["num_blocks"] * np.median([r[0] for r in reps]) + np.median([r[1] for r in reps])), len(reps)
  tok_s_1, n1 = measure(1, 12.0)
  tok_s_n, nn = measure(threads_all, 4.0)
  full = (parity or {}).get("cpu_full_step")
  return {"value": round(tok_s_1, 4), "unit": "tok/s", "cores": 1, "kind": "port", **({"measured_whole_token_all_cores": full} if full else {}),
          "sample": f"oracle/c scalar restatement (dequant -> fp16-rounded weight -> fp32 MAC), 1 thread: the 7 linears of layer 0 + 1/32 of the "
                    f"lm-head rows, 2 warm-ups then the median of {n1} passes, extrapolated to {cfg['num_blocks']} layers + full lm-head (attention/norms excluded)",
          "all_cores": {"value": round(tok_s_n, 4), "cores": int(threads_all), "passes": nn}}

def moe_step_gate(model, sd, c):
  """One more decode step of a timed configuration-4 model (one sequence, or sequences in lockstep), launched eagerly so that every block's expert selection
  can be read back, recomputed on the CPU by oracle.packed.PackedModel (the reference's numerics) from the GPU's own KV cache of the earlier positions: logits
  within 4e-3 (this configuration's bar, see tests/test_zy_real_size_parity.py) and the greedy token equal or inside that bar of the oracle's; the oracle
  follows the GPU's selection only across router near-ties (logits within 1e-2 of each other)."""
  from oracle import cref, linear as ol
  from oracle.packed import PackedModel
  from tinygrad_amd.llm import OLMOE
  batched = hasattr(model, "batch")
  B, k, nb = (model.batch if batched else 1), c.num_experts_per_tok, c.num_blocks
  state = (model.state if batched else model.s.state).numpy()
  pos = int(state[0])
  toks_in = model.tokens.numpy().copy() if batched else np.array([int(state[1])])
  sels, cur = [], []
  def on_block(i):
    model.stream.synchronize()
    cur.append((model.sel if batched else model.s.sel).numpy().reshape(B, k).copy())
  model.decode_step(on_block=on_block)
  lg_gpu = np.array(model.logits()).reshape(B, -1)
  toks_out = (model.tokens.numpy().copy() if batched else np.array([int(model.s.state.numpy()[1])]))
  host = {kk: (b.numpy(), t, shp) for kk, (b, t, shp) in sd.items()}
  base = PackedModel(OLMOE, host, c.max_context, threads=min(16, cref.max_threads()))
  worst, flips, ties = 0.0, 0, 0
  for b in range(B):
    o = base if b == 0 else base.clone()
    for i in range(nb):
      blk = model.blk[i]
      ck = (blk["cache_k"].numpy()[b] if batched else blk.cache_k.numpy()); cv = (blk["cache_v"].numpy()[b] if batched else blk.cache_v.numpy())
      o.ck[i, :, :pos], o.cv[i, :, :pos] = ck[:, :pos], cv[:, :pos]
    lg = o.forward(int(toks_in[b]), pos, follow_sel=[s[b] for s in cur], tie=1e-2)
    worst = max(worst, ol.rel_err(lg_gpu[b], lg)); ties += o.ties_followed
    if int(toks_out[b]) != int(np.argmax(lg)):
      flips += 1
      if float(lg[int(np.argmax(lg))] - lg[int(toks_out[b])]) > 2 * 4e-3 * float(np.abs(lg).max()): worst = np.inf
  return {"bar_rel_err": 4e-3, "max_rel_err": float(f"{worst:.3e}"), "sequences": B, "position": pos, "tokens_across_an_oracle_near_tie": flips,
          "routings_followed_across_a_near_tie": ties, "ok": bool(worst <= 4e-3)}

def other_configs():
  """Kernel-level figures of benchmark configurations 1, 2, 4 and 5 (python -m tinygrad_amd.benchmarks) measured in this process."""
  from tinygrad_amd import benchmarks as bm
  out = {}
  for name, fn in (("config1", bm.config1), ("config2", bm.config2), ("config4", lambda: bm.config4(gate=moe_step_gate)), ("config5", bm.config5)):
    try: out[name] = [{k: v for k, v in row.items() if k != "config"} for row in fn()]
    except Exception as e: out[name] = {"error": f"{type(e).__name__}: {e}"}
  return out

def main():
  ap = argparse.ArgumentParser()
  ap.add_argument("--gpus", type=int, default=1)
  ap.add_argument("--steps", type=int, default=128)
  ap.add_argument("--warmup", type=int, default=8)
  ap.add_argument("--prefill", type=int, default=1024)
  ap.add_argument("--layers", type=int, default=32, help="reduce only for smoke runs; the reported config then says so")
  ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
  ap.add_argument("--no-parity", action="store_true", help="skip the parity gate (profiling runs)")
  ap.add_argument("--no-other", action="store_true", help="skip the kernel-level figures of the other configurations")
  ap.add_argument("--replay", choices=("cmdlist", "graph"), default="cmdlist", help="how the captured step is replayed: plain launches in capture order, or hipGraphLaunch")
  ap.add_argument("--no-graph", action="store_true", help="eager launches instead of graph replay (for kernel-trace profiling)")
  args = ap.parse_args()
  if args.gpus != 1:
    print("bench.py: this build measures one GPU only (no collectives, no sharding in this run); use --gpus 1", file=sys.stderr)
    sys.exit(2)

  from tinygrad_amd import runtime as rt
  from tinygrad_amd.llm import Transformer, TransformerConfig, synth_state, LLAMA3_8B
  rt.init(0)
  cfg = dict(LLAMA3_8B); cfg["num_blocks"] = args.layers
  max_new = args.steps + args.warmup + 16                    # + the parity step and the eager steps of the per-kernel timing below
  max_ctx = ((args.prefill + max_new + 63) // 64) * 64
  c = TransformerConfig(max_context=max_ctx, **cfg)
  sd = synth_state(c, seed=1003)
  model = Transformer(c, sd, max_new=max_new)
  model.replay = args.replay
  rt.synchronize()

  rng = np.random.default_rng(1003)
  prompt = [int(t) for t in rng.integers(0, c.vocab_size, size=args.prefill)]
  ug = not args.no_graph
  model.prefill(prompt, ug)                                    # fills positions 0..prefill-2; the last prompt token is the first decode input
  rt.synchronize()
  tp = time.perf_counter()
  model.prefill(prompt, ug, reuse_cache=False)                 # the same prompt once more, now with every step kind recorded: the prefill rate (extra/benchmark_llm.py reports it beside the decode rate)
  rt.synchronize()
  prefill_s = time.perf_counter() - tp
  for _ in range(args.warmup): model.decode_step(ug)
  rt.synchronize()
  t0 = time.perf_counter()
  for _ in range(args.steps): model.decode_step(ug)          # graph launch + stream sync per token
  rt.synchronize()
  dt = time.perf_counter() - t0
  model.check_state()
  ms_per_step = dt / args.steps * 1e3
  tok_s = args.steps / dt
  threads_all = min(len(os.sched_getaffinity(0)), 64)
  parity = None
  if not args.no_parity:
    from oracle import cref
    parity = parity_gate(model, c, min(threads_all, cref.max_threads()))

  # ---- the per-op kernels on the same weights, timed with HIP events on the model's stream (the five launches of TransformerBlock.__call__:
  #      q/k/v with attn_norm folded in (it also touches the cache rows the attention will read), the attention as one launch that leaves split
  #      partials, attn_output + residual merging those partials while it stages its row, gate/up with ffn_norm folded in + SwiGLU, down + residual) ----
  st = model.stream.handle
  L = rt.lib()
  from tinygrad_amd.nn import qlinear_multi
  durs = {"gate_up": [], "down": [], "qkv": [], "attn_output": [], "attention": []}
  s = model.s
  b_first = model.blk[0]
  fused = bool(b_first.fused_attn)                             # the attention as one launch whose partials attn_output merges (TransformerBlock.__call__)
  touch = lambda b: (s.state, b.cache_k, b.cache_v, s.rope, c.n_kv_heads, c.head_dim, c.max_context) if b.kv_touch else None
  ops = {
    "qkv": lambda b: qlinear_multi([b.attn_q, b.attn_k, b.attn_v], s.x, [s.q, s.k, s.v], stream=st, norm=(b.attn_norm, c.norm_eps), touch=touch(b)),
    "attention": (lambda b: rt.check(L.tga_attention_decode_split(s.q.ptr, s.k.ptr, s.v.ptr, b.cache_k.ptr, b.cache_v.ptr, s.attn_part.ptr, s.state.ptr, c.n_heads, c.n_kv_heads,
                                     c.head_dim, c.max_context, s.rope.ptr, st))) if fused else
                 (lambda b: rt.check(L.tga_attention_decode(s.q.ptr, s.k.ptr, s.v.ptr, b.cache_k.ptr, b.cache_v.ptr, s.attn_part.ptr, s.state.ptr,
                                     c.n_heads, c.n_kv_heads, c.head_dim, c.max_context, s.rope.ptr, s.attn.ptr, None, b.attn_output.ggml_type if b.stage_attn else 0, st))),
    "attn_output": (lambda b: rt.check(L.tga_attn_merge_qlinear(b.attn_output.ggml_type, b.attn_output.blocks.ptr, s.x.ptr, b.attn_output.out_features, b.attn_output.in_features,
                                       s.x.ptr, s.attn_part.ptr, b.fused_attn, c.head_dim, st))) if fused else
                   (lambda b: qlinear_multi([b.attn_output], s.attn, [s.x], epilogue=1, resid=[s.x], stream=st, x_staged=b.stage_attn)),
    "gate_up": lambda b: qlinear_multi([b.ffn_gate, b.ffn_up], s.x, [s.act], epilogue=2, stream=st, norm=(b.ffn_norm, c.norm_eps), stage_out_for=b.ffn_down if b.stage_act else None),
    "down": lambda b: qlinear_multi([b.ffn_down], s.act, [s.x], epilogue=1, resid=[s.x], stream=st, x_staged=b.stage_act),
  }
  order = ("qkv", "attention", "attn_output", "gate_up", "down")
  # One op at a time over all blocks, back to back between ONE pair of events: every launch reads its own block's weights (32 x 66 MB for
  # gate/up, nothing is served from a cache), and the figure is the average launch duration including the dispatch gap between launches, without
  # an event packet in front of and behind every kernel (bracketing single launches adds about 2 us to each).  A long kernel that touches
  # nothing of the model (it writes a Q6_K matrix into a scratch buffer, about 30 ms) goes first, so that the launches queue up behind it
  # and then run as fast as the GPU takes them rather than as fast as the host enqueues them.
  blocker = rt.Buffer((model.output.nbytes,), np.uint8)
  for it in range(4):                                          # the first pass is a warm-up (first launches load code objects), not timed
    rt.check(L.tga_embed_row(model.token_embd.ptr, model.embd_type, c.dim, model.s.state.ptr, model.s.x.ptr, st))
    for b in model.blk:                                        # one real step first: every buffer holds values of the right scale
      for k in order: ops[k](b)
    rt.check(L.tga_synth_weights(model.output.ggml_type, blocker.ptr, model.output.out_features * model.output.in_features, 4242, 0.02, st))
    ev = {}
    for k in order:
      e0, e1 = rt.Event(), rt.Event(); e0.record(st)
      for b in model.blk: ops[k](b)
      e1.record(st); ev[k] = (e0, e1)
    rt.check(L.tga_advance_prompt(model.s.state.ptr, model.s.prompt.ptr, st))
    model.stream.synchronize()
    if it > 0:
      for k in durs: durs[k].append(ev[k][0].elapsed_ms(ev[k][1]) * 1e3 / len(model.blk))
  b0 = model.blk[0]
  ctx_now = int(model.s.state.numpy()[0])
  alg = {"gate_up": b0.ffn_gate.nbytes + b0.ffn_up.nbytes + c.dim * 8 + c.hidden_dim * 2,            # weights + fp32 row + norm weight + fp16 out
         "down": b0.ffn_down.nbytes + c.hidden_dim * 2 + c.dim * 8,
         "qkv": b0.attn_q.nbytes + b0.attn_k.nbytes + b0.attn_v.nbytes + c.dim * 8 + (c.n_heads + 2 * c.n_kv_heads) * c.head_dim * 4,
         "attn_output": b0.attn_output.nbytes + c.dim * 2 + c.dim * 8,
         "attention": 2 * c.n_kv_heads * c.head_dim * ctx_now * 2}                                     # fp16 K and V rows read at this context
  kern = {k: {"avg_us": round(float(np.mean(v)), 3), "alg_bytes": int(alg[k]), "GBps": round(alg[k] / np.mean(v) / 1e3, 1),
              "frac_hbm": round(alg[k] / np.mean(v) / 1e3 / HBM_PEAK_GBS, 4)} for k, v in durs.items()}
  wbytes = model.weight_bytes_per_token()
  ctx_mid = args.prefill + args.warmup + args.steps // 2
  kv_bytes = 2 * c.num_blocks * c.n_kv_heads * c.head_dim * ctx_mid * 2
  out = {
    "metric": "Q4_0 8B-arch decode tok/s @bs1; dequant-GEMV GB/s as % of HBM peak", "value": round(tok_s, 2), "unit": "tok/s",
    "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4), "higher_is_better": True,
    "scaling": "weak", "vs_baseline": None, "dtype": "f16 x q4_0/q6_k -> f32 accumulate", "data": "synthetic",
    "config": {"workload": f"benchmark configuration 3: Llama-3-8B-arch ({c.num_blocks} layers) Q4_0 linears + Q6_K lm-head, random-init, batch 1, "
                           f"fp16 KV prefilled with {args.prefill} random ids, greedy decode", "device": rt.device_name(),
               "weight_bytes_per_token": int(wbytes), "stream_GBps_over_whole_step": round((wbytes + kv_bytes) / (ms_per_step * 1e-3) / 1e9, 1),
               "frac_hbm_over_whole_step": round((wbytes + kv_bytes) / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)},
  }
  dom = kern["gate_up"]
  per_block = sum(v["avg_us"] for v in kern.values())
  out["roofline"] = {"bound": "hbm", "kernel": "qgemv1_kernel<Q4_0 pair, R=2, WK=1, WR=8, SwiGLU, norm prologue> (ffn_norm + ffn_gate + ffn_up + silu*mul in one launch, 2 x 14336 x 4096; "
                                               "one of five launches per block)",
                     "achieved": dom["GBps"], "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": dom["frac_hbm"],
                     "traffic": GATE_UP_TRAFFIC_BYTES if c.num_blocks == 32 else None,
                     "traffic_source": "recorded rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs (profiles/qgemv1_gate_up_hbm_traffic.md), not re-measured by this run",
                     "avg_launch_us": dom["avg_us"], "alg_bytes_per_launch": dom["alg_bytes"],
                     "rocprof_avg_us": GATE_UP_ROCPROF_AVG_US if c.num_blocks == 32 else None,
                     "frac_by_rocprof_avg": round(dom["alg_bytes"] / GATE_UP_ROCPROF_AVG_US / 1e3 / HBM_PEAK_GBS, 4) if c.num_blocks == 32 else None,
                     "rocprof_back_to_back_avg_us": GATE_UP_ROCPROF_B2B_US if c.num_blocks == 32 else None,
                     "timing": "achieved / frac: HIP events on the launch stream around the 32 gate/up launches of all blocks issued back to back, three repetitions (live, this run); "
                               "rocprof_avg_us / frac_by_rocprof_avg: the recorded rocprofv3 kernel-trace average of the same kernel over every call of an eagerly launched decode, "
                               "rocprof_back_to_back_avg_us: the same trace restricted to the back-to-back passes that the HIP events bracket "
                               "(profiles/decode_llama3_8b_q4_0_kernel_stats.md), neither re-measured by this run",
                     "share_of_block_time": round(dom["avg_us"] / per_block, 3),
                     "per_op_kernels": {k: v for k, v in kern.items() if k != "gate_up"}}
  out["prefill"] = {"positions": args.prefill - 1, "ms": round(prefill_s * 1e3, 2), "positions_per_s": round((args.prefill - 1) / prefill_s, 1), "positions_per_step": int(model.prefill_chunk),
                    "what": "the prompt prefilled once more before the timed decode steps (recorded steps replayed; one pass over the weights per step of positions_per_step rows), host wall clock; not part of `value`"}
  if parity is not None: out["parity"] = parity
  if not args.no_cpu:
    from oracle import cref
    out["cpu_baseline"] = cpu_baseline(model, cfg, min(threads_all, cref.max_threads()), parity)
  if not args.no_other:
    out["other_configs"] = other_configs()
  print(json.dumps(out))
  bad = [row.get("case", "?") for rows in (out.get("other_configs") or {}).values() if isinstance(rows, list) for row in rows if isinstance(row.get("parity"), dict) and not row["parity"]["ok"]]
  if bad:
    print(f"bench.py: PARITY GATE FAILED for {bad}", file=sys.stderr)
    sys.exit(1)
  if parity is not None and not parity["ok"]:
    print(f"bench.py: PARITY GATE FAILED: max rel-err {parity['max_rel_err']} (bar {PARITY_TOL}), greedy token gpu {parity['greedy_token_gpu']} cpu {parity['greedy_token_cpu']}", file=sys.stderr)
    sys.exit(1)

if __name__ == "__main__":
  main()
