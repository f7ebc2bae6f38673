#!/usr/bin/env python3
"""Headline benchmark: Q4_0 Llama-3-8B-architecture greedy decode at batch 1 on one MI355X (benchmark configuration 3).

A step is one decoded token.  Random-init weights are written on the GPU as GGUF blocks (Q4_0 linears and embedding, Q6_K
lm-head), the fp16 KV cache is prefilled with 1024 random token ids through the model itself, then --warmup + --steps tokens
are decoded greedily, one captured launch sequence per token with a host sync per token (as the reference's generate loop does).
Prints ONE JSON line: tok/s, the roofline of the dominant kernel from HIP-event timings taken live, the same figures for the other
kernels of a block, and a CPU baseline (C restatement of the reference arithmetic on a bounded sample of the same weights).
Default path: one launch per op (six per block, attention being two); the dominant kernel is then the fused ffn_gate + ffn_up dequant-GEMV with the
ffn_norm folded in.  --fused: all 32 blocks of a token in one persistent launch (tga_decode_layers), which is then the kernel reported."""
import argparse, json, os, sys, time
import numpy as np

HBM_PEAK_GBS = 8000.0
GATE_UP_TRAFFIC_BYTES = 66702500   # 66 609 152 B fetched + 93 389 B written per launch (counter runs summarised in profiles/qgemv1_gate_up_hbm_traffic.md)

def cpu_baseline(model, cfg, seconds_budget=20.0):
  """Times oracle/c (scalar C restatement of dequant + fp32-accumulate matmul, model-path numerics) on the GPU box's host
  cores: the 7 linears of layer 0 plus a 1/32 row slice of the lm-head, extrapolated to one token (32 layers + full head)."""
  from oracle import cref
  b = model.blk[0]
  lins = [("attn_q", b.attn_q), ("attn_k", b.attn_k), ("attn_v", b.attn_v), ("attn_output", b.attn_output),
          ("ffn_gate", b.ffn_gate), ("ffn_up", b.ffn_up), ("ffn_down", b.ffn_down)]
  host = [(l.ggml_type, l.blocks.view(0, (l.nbytes,), np.uint8).numpy(), l.out_features, l.in_features) for _, l in lins]
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
  one_pass(1)                                             # warm-up (page in, build)
  reps = []
  t_start = time.perf_counter()
  while len(reps) < 3 or (time.perf_counter() - t_start < seconds_budget / 2 and len(reps) < 9): reps.append(one_pass(1))
  layer_s, head_s = np.median([r[0] for r in reps]), np.median([r[1] for r in reps])
  tok_s_1 = 1.0 / (cfg["num_blocks"] * layer_s + head_s)
  cores = len(os.sched_getaffinity(0))
  nthr = min(cores, cref.max_threads())
  one_pass(nthr)
  repn = [one_pass(nthr) for _ in range(3)]
  tok_s_n = 1.0 / (cfg["num_blocks"] * np.median([r[0] for r in repn]) + np.median([r[1] for r in repn]))
  return {"value": round(tok_s_1, 4), "unit": "tok/s", "cores": 1, "kind": "port",
          "sample": "oracle/c scalar restatement (dequant -> fp16-rounded weight -> fp32 MAC), 1 thread: the 7 linears of layer 0 + 1/32 of the "
                    "lm-head rows, median of >=3 passes, extrapolated to 32 layers + full lm-head (attention/norms excluded)",
          "all_cores": {"value": round(tok_s_n, 4), "cores": int(nthr)}}

def main():
  ap = argparse.ArgumentParser()
  ap.add_argument("--gpus", type=int, default=1)
  ap.add_argument("--steps", type=int, default=128)
  ap.add_argument("--warmup", type=int, default=8)
  ap.add_argument("--prefill", type=int, default=1024)
  ap.add_argument("--layers", type=int, default=32, help="reduce only for smoke runs; the reported config then says so")
  ap.add_argument("--no-cpu", action="store_true")
  ap.add_argument("--no-graph", action="store_true", help="eager launches instead of graph replay (for kernel-trace profiling)")
  ap.add_argument("--fused", action="store_true", help="all blocks of a token in one persistent launch instead of one launch per op")
  ap.add_argument("--per-op", action="store_true", help="(the default; kept so that older command lines still run)")
  args = ap.parse_args()
  if args.gpus != 1:
    print("bench.py: this build measures one GPU only (no collectives, no sharding in this run); use --gpus 1", file=sys.stderr)
    sys.exit(2)

  from tinygrad_amd import runtime as rt
  from tinygrad_amd.llm import Transformer, TransformerConfig, synth_state, LLAMA3_8B
  rt.init(0)
  cfg = dict(LLAMA3_8B); cfg["num_blocks"] = args.layers
  max_new = args.steps + args.warmup + 16                    # + the eager steps of the per-kernel timing below
  max_ctx = ((args.prefill + max_new + 63) // 64) * 64
  c = TransformerConfig(max_context=max_ctx, **cfg)
  sd = synth_state(c, seed=1003)
  model = Transformer(c, sd, max_new=max_new, fused=args.fused)
  rt.synchronize()

  rng = np.random.default_rng(1003)
  prompt = [int(t) for t in rng.integers(0, c.vocab_size, size=args.prefill)]
  ug = not args.no_graph
  model.prefill(prompt, ug)                                    # fills positions 0..prefill-2; the last prompt token is the first decode input
  for _ in range(args.warmup): model.decode_step(ug)
  rt.synchronize()
  t0 = time.perf_counter()
  for _ in range(args.steps): model.decode_step(ug)          # graph launch + stream sync per token
  rt.synchronize()
  dt = time.perf_counter() - t0
  ms_per_step = dt / args.steps * 1e3
  tok_s = args.steps / dt

  # ---- live timing of the dominant kernel: HIP events (on the model's stream) around the one-launch block kernel of eager steps ----
  st = model.stream.handle
  L = rt.lib()
  fused_us, phase = [], None
  if model.layer_table is not None:
    s_ = model.s
    tb = rt.Buffer((8 * 11 * c.num_blocks,), np.uint64).zero_()
    for it in range(8):
      rt.check(L.tga_embed_row(model.token_embd.ptr, model.embd_type, c.dim, s_.state.ptr, s_.x.ptr, st))
      if it == 7: rt.check(L.tga_decode_layers_trace(tb.ptr))
      e0, e1 = rt.Event(), rt.Event(); e0.record(st)
      rt.check(L.tga_decode_layers(model.layer_table.ptr, c.num_blocks, model.layer_type, s_.x.ptr, s_.qkv.ptr, s_.attn.ptr, s_.act.ptr, s_.attn_part.ptr,
                                   s_.state.ptr, s_.rope.ptr, s_.sync.ptr, c.dim, c.hidden_dim, c.n_heads, c.n_kv_heads, c.head_dim, c.max_context, c.norm_eps, st))
      e1.record(st)
      rt.check(L.tga_advance_prompt(s_.state.ptr, s_.prompt.ptr, st))
      model.stream.synchronize()
      fused_us.append(e0.elapsed_ms(e1) * 1e3)
    rt.check(L.tga_decode_layers_trace(None))
    model.check_fused()
    if c.num_blocks > 2:
      # wall-clock stamps (100 MHz) of workgroups 0, 73, ... at the phase boundaries of every block: time from the start of a
      # phase (all workgroups past the barrier) to the last sampled workgroup finishing it, median over the inner blocks
      T = tb.numpy().astype(np.int64).reshape(8, c.num_blocks, 11)[:, 1:-1]
      span = lambda i0, i1: float(np.median(T[:, :, i1].max(0) - T[:, :, i0].min(0)) * 0.01)
      phase = {"qkv_after_staging_us": round(span(0, 1), 2),
               "attention_us": round(span(2, 3), 2), "attn_output_us": round(span(4, 5), 2), "gate_up_us": round(span(6, 7), 2), "down_us": round(span(8, 9), 2),
               "block_us": round(float(np.median(np.diff(T[0, :, 0])) * 0.01), 2)}
  # ---- the per-op kernels on the same weights, timed with HIP events on the model's stream (the launches of TransformerBlock.__call__:
  #      q/k/v with attn_norm folded in, attention, attn_output + residual, gate/up with ffn_norm folded in + SwiGLU, down + residual) ----
  from tinygrad_amd.nn import qlinear_multi
  durs = {"gate_up": [], "down": [], "qkv": [], "attn_output": [], "attention": []}
  s = model.s
  ops = {
    "qkv": lambda b: qlinear_multi([b.attn_q, b.attn_k, b.attn_v], s.x, [s.q, s.k, s.v], stream=st, norm=(b.attn_norm, c.norm_eps)),
    "attention": lambda b: rt.check(L.tga_attention_decode(s.q.ptr, s.k.ptr, s.v.ptr, b.cache_k.ptr, b.cache_v.ptr, s.attn_part.ptr, s.state.ptr,
                                    c.n_heads, c.n_kv_heads, c.head_dim, c.max_context, s.rope.ptr, s.attn.ptr, None, b.attn_output.ggml_type if b.stage_attn else 0, st)),
    "attn_output": lambda b: qlinear_multi([b.attn_output], s.attn, [s.x], epilogue=1, resid=[s.x], stream=st, x_staged=b.stage_attn),
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
  ctx_now = args.prefill + args.warmup + args.steps
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
  if fused_us:
    # algorithmic bytes of one launch: the seven Q4_0 matrices of every block + the fp16 K/V rows read at this context length
    blk_w = sum(l.nbytes for b in model.blk for l in (b.attn_q, b.attn_k, b.attn_v, b.attn_output, b.ffn_gate, b.ffn_up, b.ffn_down))
    alg_f = blk_w + 2 * c.num_blocks * c.n_kv_heads * c.head_dim * ctx_now * 2
    avg = float(np.mean(fused_us[1:]))
    out["roofline"] = {"bound": "hbm", "kernel": f"decode_layers_kernel<Q4_0 pair> (all {c.num_blocks} blocks of one token in one persistent launch: 4 dequant-GEMV phases + attention per block)",
                       "achieved": round(alg_f / avg / 1e3, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(alg_f / avg / 1e3 / HBM_PEAK_GBS, 4),
                       # HBM bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of tinygrad_amd/traffic_probe.py at context 1024
                       # (counters scaled by a 1 GiB copy kernel: x2.0000 and x1.0000): 4 100.5 MB fetched + 43.0 MB written
                       "traffic": 4143500000 if c.num_blocks == 32 else None,
                       "avg_launch_us": round(avg, 2), "alg_bytes_per_launch": int(alg_f), "phase_us_inside_launch": phase,
                       "per_op_kernels": kern}
    if phase:
      out["roofline"]["gate_up_phase_GBps"] = round(alg["gate_up"] / phase["gate_up_us"] / 1e3, 1)
      out["roofline"]["down_phase_GBps"] = round(alg["down"] / phase["down_us"] / 1e3, 1)
  else:
    dom = kern["gate_up"]
    per_block = sum(v["avg_us"] for v in kern.values())
    out["roofline"] = {"bound": "hbm", "kernel": "qgemv1_kernel<Q4_0 pair, R=2, WK=1, WR=8, SwiGLU, norm prologue> (ffn_norm + ffn_gate + ffn_up + silu*mul in one launch, 2 x 14336 x 4096; "
                                                 "one of six launches per block)",
                       "achieved": dom["GBps"], "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": dom["frac_hbm"],
                       # HBM bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of tinygrad_amd/traffic_probe.py (counters scaled by a
                       # 1 GiB copy kernel: x2.0000 and x1.0000)
                       "traffic": GATE_UP_TRAFFIC_BYTES if c.num_blocks == 32 else None,
                       "avg_launch_us": dom["avg_us"], "alg_bytes_per_launch": dom["alg_bytes"],
                       "share_of_block_time": round(dom["avg_us"] / per_block, 3),
                       "per_op_kernels": {k: v for k, v in kern.items() if k != "gate_up"}}
  if not args.no_cpu:
    out["cpu_baseline"] = cpu_baseline(model, cfg)
  print(json.dumps(out))

if __name__ == "__main__":
  main()
