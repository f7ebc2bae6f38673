"""Kernel-level measurements on one MI355X for the configurations that are not the headline benchmark:
  config 1  Q4_0 4096x4096 GEMV, batch 1
  config 2  Q8_0 / Q6_K small-batch sweep, M in {1, 2, 4, 8}
  config 4  OLMoE-architecture MXFP4 expert decode, batch 1 (tok/s and expert-GEMV GB/s)
  config 5  MXFP8 grouped GEMM at T = 4096, E = 128, k = 8 with Zipf routing (MFMA utilisation and GB/s), plus the measured
            register-only peak of the scaled FP8 MFMA

  config 6  Q4_K / Q5_K and Q4_1 / Q5_0 / Q5_1 dequant-GEMV at the same linear shapes (not one of the benchmark's configurations)

  config 7  Llama-3-8B-architecture decode with the tensor-type mix of a Q4_K_M file (Q4_K, Q6_K for part of attn_v / ffn_down, Q6_K lm-head)

    python -m tinygrad_amd.benchmarks [--config N ...]        prints one JSON object per measurement

Timing: HIP events around >= 100 back-to-back launches; weights are rotated over enough distinct copies to exceed the 256 MB
Infinity Cache (a single matrix that is re-read every launch would be served from that cache, not from HBM).  Weights for
configs 1 / 2 / 4 are written on the GPU as valid GGUF blocks by tga_synth_weights; timing does not depend on their values (the
parity tests use the seeded host generators)."""
from __future__ import annotations
import argparse, json, sys
import numpy as np
from tinygrad_amd import runtime as rt
from tinygrad_amd.runtime import Buffer
from tinygrad_amd.nn import QuantLinear, ExpertWeights

HBM_PEAK_GBS = 8000.0
MFMA_FP8_PEAK_TFLOPS = 5000.0
MALL_BYTES = 256 << 20

def _time_launches(fn, n_variants: int, iters: int, stream: rt.Stream) -> float:
  """Average microseconds per call of fn(i % n_variants) over `iters` back-to-back launches (one warm-up pass first)."""
  for i in range(n_variants): fn(i)
  stream.synchronize()
  e0, e1 = rt.Event(), rt.Event()
  e0.record(stream.handle)
  for i in range(iters): fn(i % n_variants)
  e1.record(stream.handle); e1.synchronize()
  return e0.elapsed_ms(e1) * 1e3 / iters

def gemv_case(ggml_type: int, n: int, k: int, m: int, iters: int = 200) -> dict:
  nel, nby = rt.GGML_QUANT.get(ggml_type, (1, 2))                      # (fp16 rows otherwise)
  wbytes = n * (k // nel) * nby
  copies = max(2, -(-int(1.25 * MALL_BYTES) // wbytes))
  big = Buffer((copies * wbytes,), np.uint8)
  if ggml_type in (rt.Q4_K, rt.Q5_K, rt.Q4_1, rt.Q5_0, rt.Q5_1, rt.IQ4_XS, rt.IQ3_XXS, rt.IQ3_S, rt.IQ2_S, rt.Q1_0):       # no device-side writer for these: seeded host blocks, one upload per copy
    from tinygrad_amd import synth
    host = synth.random_blocks(np.random.default_rng(1002), ggml_type, n, k)
    for c in range(copies): big.view(c * wbytes, (wbytes,), np.uint8).copyin(host)
  else:
    for c in range(copies): rt.check(rt.lib().tga_synth_weights(ggml_type, big.ptr + c * wbytes, n * k, 1000 + c, k ** -0.5, None))
  rt.synchronize()
  lins = [QuantLinear(big.view(c * wbytes, (wbytes,), np.uint8), ggml_type, n, k) for c in range(copies)]
  rng = np.random.default_rng(1002)
  x = Buffer.from_numpy(rng.standard_normal((m, k)).astype(np.float16)); y = Buffer((m, n), np.float16)
  s = rt.Stream()
  us = _time_launches(lambda i: lins[i](x, out=y, stream=s.handle), copies, iters, s)
  alg = wbytes + m * k * 2 + m * n * 2
  name = {rt.Q4_0: "Q4_0", rt.Q8_0: "Q8_0", rt.Q4_1: "Q4_1", rt.Q5_0: "Q5_0", rt.Q5_1: "Q5_1", rt.Q4_K: "Q4_K", rt.Q5_K: "Q5_K", rt.Q6_K: "Q6_K", rt.IQ4_XS: "IQ4_XS", rt.MXFP4: "MXFP4", rt.F16: "F16",
          rt.IQ3_XXS: "IQ3_XXS", rt.IQ3_S: "IQ3_S", rt.IQ2_S: "IQ2_S", rt.Q1_0: "Q1_0"}[ggml_type]
  return {"case": f"{name} {n}x{k} M={m}", "avg_us": round(us, 2), "alg_bytes": alg, "GBps": round(alg / us / 1e3, 1),
          "frac_hbm_peak": round(alg / us / 1e3 / HBM_PEAK_GBS, 4), "weight_copies_rotated": copies, "launches": iters}

def config1(): return [dict(config=1, **gemv_case(rt.Q4_0, 4096, 4096, 1, iters=400))]

def config2():
  out = []
  for t, n, k in ((rt.Q8_0, 4096, 4096), (rt.Q8_0, 14336, 4096), (rt.Q8_0, 4096, 14336), (rt.Q6_K, 128256, 4096)):
    for m in (1, 2, 4, 8): out.append(dict(config=2, **gemv_case(t, n, k, m, iters=100 if n > 100000 else 200)))
  return out

def kquants():
  """Q4_K / Q5_K (the block types of Q4_K_M / Q5_K_M model files) and the older Q4_1 / Q5_0 / Q5_1 blocks at the Llama-3-8B linear
  shapes, M in {1, 8} (Q4_K / Q5_K: and 4, 16), and the Q6_K ffn_down of a Q4_K_M file."""
  out = []
  for t in (rt.Q4_K, rt.Q5_K, rt.Q4_1, rt.Q5_0, rt.Q5_1, rt.IQ4_XS):
    for n, k in ((4096, 4096), (14336, 4096), (4096, 14336)):
      for m in ((1, 4, 8, 16) if t in (rt.Q4_K, rt.Q5_K) else (1, 8)): out.append(dict(config="k-quants", **gemv_case(t, n, k, m, iters=200)))
  for m in (1, 4, 8, 16): out.append(dict(config="k-quants", **gemv_case(rt.Q6_K, 4096, 14336, m, iters=200)))
  return out

def codebooks():
  """IQ3_XXS / IQ3_S / IQ2_S / Q1_0 read in place at the Llama-3-8B linear shapes, M in {1, 8}, beside the fp16 matrix of the same shape (what a load-time expansion would stream)."""
  out = []
  for n, k in ((4096, 4096), (14336, 4096), (4096, 14336)):
    out.append(dict(config="codebooks", **gemv_case(rt.F16, n, k, 1, iters=200)))
    for t in (rt.IQ3_XXS, rt.IQ3_S, rt.IQ2_S, rt.Q1_0):
      for m in (1, 8): out.append(dict(config="codebooks", **gemv_case(t, n, k, m, iters=200)))
  return out

def config7(steps: int = 64, ctx: int = 1024, use_graph: bool = True):
  """The 8B architecture of benchmark configuration 3 with the tensor types of a Q4_K_M file, same procedure as bench.py (prefill through the model,
  graph replay + sync per token); then the prefill alone (16 positions per step) and 2 / 4 / 8 sequences decoded in lockstep."""
  from tinygrad_amd.llm import Transformer, BatchedTransformer, TransformerConfig, synth_state, LLAMA3_8B
  import time
  c = TransformerConfig(max_context=((ctx + steps + 16 + 63) // 64) * 64, **LLAMA3_8B)
  sd = synth_state(c, seed=1007, q4_k_m=True)
  model = Transformer(c, sd, max_new=steps + 16)
  rt.synchronize()
  rng = np.random.default_rng(1007)
  prompt = [int(t) for t in rng.integers(0, c.vocab_size, size=ctx)]
  model.prefill(prompt, use_graph)
  for _ in range(8): model.decode_step(use_graph)
  rt.synchronize()
  t0 = time.perf_counter()
  for _ in range(steps): model.decode_step(use_graph)
  rt.synchronize()
  dt = (time.perf_counter() - t0) / steps
  wb = model.weight_bytes_per_token()
  mix = "Q4_K_M tensor-type mix (Q4_K + Q6_K)"
  res = [{"config": 7, "case": f"Llama-3-8B-arch decode B=1 ctx {ctx}, {mix}, {'graph replay' if use_graph else 'eager launches'} + sync per token",
          "tok_s": round(1.0 / dt, 1), "ms_per_token": round(dt * 1e3, 4), "weight_bytes_per_token": wb, "weight_GBps_over_step": round(wb / dt / 1e9, 1)}]
  if not use_graph: return res                                          # (a profiler's run: the single-sequence step is what it is after)
  t0 = time.perf_counter()
  model.prefill(prompt, reuse_cache=False)                               # (every step kind was captured by the first prefill)
  dtp = time.perf_counter() - t0
  res.append({"config": 7, "case": f"Llama-3-8B-arch prefill of {ctx - 1} positions, {model.prefill_chunk} per step, {mix}", "ms": round(dtp * 1e3, 1), "positions_per_s": round((ctx - 1) / dtp, 1)})
  del model
  for B in (2, 4, 8, 16):
    bm = BatchedTransformer(c, sd, B, max_new=steps + 16)
    bm.prefill([[int(t) for t in rng.integers(0, c.vocab_size, size=ctx)] for _ in range(B)])
    for _ in range(4): bm.decode_step()
    rt.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps): bm.decode_step()
    rt.synchronize()
    dtb = (time.perf_counter() - t0) / steps
    bm.check_state()
    res.append({"config": 7, "case": f"Llama-3-8B-arch decode B={B} ctx {ctx} (sequences in lockstep), {mix}", "tok_s": round(B / dtb, 1), "ms_per_step": round(dtb * 1e3, 4)})
    del bm
  return res

def config8(steps: int = 32, ctx: int = 1024):
  """Not a BASELINE configuration: the 8B architecture of configuration 3 (Q4_0, Q6_K lm-head) prefilled in chunks of 64 / 32 / 16 / 8 / 4 / 2 / 1 positions, and decoded
  with 2, 4, 8 and 16 sequences in lockstep (dense linears as small-batch GEMMs)."""
  from tinygrad_amd.llm import Transformer, BatchedTransformer, TransformerConfig, synth_state, LLAMA3_8B
  import time
  c = TransformerConfig(max_context=((ctx + steps + 16 + 63) // 64) * 64, **LLAMA3_8B)
  sd = synth_state(c, seed=1003)
  model = Transformer(c, sd, max_new=16)
  rt.synchronize()
  rng = np.random.default_rng(1003)
  prompt = [int(t) for t in rng.integers(0, c.vocab_size, size=ctx)]
  res = []
  for chunk in (128, 96, 64, 32, 16, 8, 4, 2, 1):
    model.prefill_chunk = chunk
    model.prefill(prompt[:2 * 64 + 64], reuse_cache=False)             # captures the step kinds this chunk size uses (whole chunks, the tail steps of sixteen, eight and four, single positions)
    t0 = time.perf_counter()
    model.prefill(prompt, reuse_cache=False)
    dt = time.perf_counter() - t0
    res.append({"config": 8, "case": f"Llama-3-8B-arch Q4_0 prefill of {ctx - 1} positions, {chunk} per step", "ms": round(dt * 1e3, 1), "positions_per_s": round((ctx - 1) / dt, 1)})
  del model
  for B in (2, 4, 8, 16):
    bm = BatchedTransformer(c, sd, B, max_new=steps + 16)
    bm.prefill([[int(t) for t in rng.integers(0, c.vocab_size, size=ctx)] for _ in range(B)])
    for _ in range(4): bm.decode_step()
    rt.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps): bm.decode_step()
    rt.synchronize()
    dtb = (time.perf_counter() - t0) / steps
    bm.check_state()
    res.append({"config": 8, "case": f"Llama-3-8B-arch Q4_0 decode B={B} ctx {ctx} (sequences in lockstep)", "tok_s": round(B / dtb, 1), "ms_per_step": round(dtb * 1e3, 4)})
    del bm
  return res

def config4(steps: int = 64, ctx: int = 512, use_graph: bool = True, gate=None):
  """gate(model, state dict, config) -> dict: called with the timed batch-1 model and the timed eight-sequence model after their runs; its result is reported
  with the figures (bench.py passes a one-step check against the CPU restatement; this package itself holds no checker)."""
  from tinygrad_amd.llm import Transformer, TransformerConfig, synth_state_moe, OLMOE
  import time
  c = TransformerConfig(max_context=((ctx + steps + 16 + 63) // 64) * 64, **OLMOE)
  model_sd = synth_state_moe(c, seed=1004)
  model = Transformer(c, model_sd, max_new=steps + 16)
  rt.synchronize()
  rng = np.random.default_rng(1004)
  model.prefill([int(t) for t in rng.integers(0, c.vocab_size, size=ctx)], use_graph)
  for _ in range(8): model.decode_step(use_graph)
  rt.synchronize()
  t0 = time.perf_counter()
  for _ in range(steps): model.decode_step(use_graph)
  rt.synchronize()
  dt = (time.perf_counter() - t0) / steps
  expert_bytes = c.num_blocks * c.num_experts_per_tok * sum(e.expert_nbytes for e in (model.blk[0].ffn_gate_exps, model.blk[0].ffn_up_exps, model.blk[0].ffn_down_exps))
  res = [{"config": 4, "case": f"OLMoE-arch decode B=1 ctx {ctx} (MXFP4 experts exponents 119..123, fp16 dense weights, {'graph replay' if use_graph else 'eager launches'} + sync per token)",
          "tok_s": round(1.0 / dt, 1), "ms_per_token": round(dt * 1e3, 4), "expert_bytes_per_token": expert_bytes, "weight_bytes_per_token": model.weight_bytes_per_token(),
          "weight_GBps_over_step": round(model.weight_bytes_per_token() / dt / 1e9, 1)}]
  if gate is not None: res[0]["parity"] = gate(model, model_sd, c)
  # batched decode: B sequences in lockstep (dense linears as small-batch GEMMs, one expert GEMV per (sequence, slot) job)
  from tinygrad_amd.llm import BatchedTransformer
  sd = {k: v for k, v in model_sd.items()}
  for B in (2, 4, 8, 16):
    bm = BatchedTransformer(c, sd, B, max_new=steps + 16)
    bm.prefill([[int(t) for t in rng.integers(0, c.vocab_size, size=ctx)] for _ in range(B)], use_graph)
    for _ in range(4): bm.decode_step(use_graph)
    rt.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps): bm.decode_step(use_graph)
    rt.synchronize()
    dtb = (time.perf_counter() - t0) / steps
    bm.check_state()
    distinct = float(np.mean([len(np.unique(bm.sel.numpy()))]))
    res.append({"config": 4, "case": f"OLMoE-arch decode B={B} ctx {ctx} (sequences in lockstep, one expert GEMV per (sequence, slot) job; last layer of the last step: {int(distinct)} distinct experts for {B * c.num_experts_per_tok} jobs)",
                "tok_s": round(B / dtb, 1), "ms_per_step": round(dtb * 1e3, 4)})
    if gate is not None and B == 8: res[-1]["parity"] = gate(bm, sd, c)
    del bm
  # the expert GEMVs alone: B tokens x 8 experts, gate/up fused then down, distinct experts per slot, layers rotated
  k, s = c.num_experts_per_tok, rt.Stream()
  for B in (1, 2, 4, 8):
    sel_host = np.stack([rng.permutation(c.num_experts)[:k] for _ in range(B)]).astype(np.int32).reshape(-1)
    sel = Buffer.from_numpy(sel_host)
    x = Buffer.from_numpy(rng.standard_normal((B, c.dim)).astype(np.float16))
    act, y = Buffer((B * k, c.hidden_dim), np.float16), Buffer((B * k, c.dim), np.float32)
    blks = model.blk
    def run(i):
      b = blks[i]
      b.ffn_gate_exps(sel, x, act, jobs_per_x_row=k, up=b.ffn_up_exps, stream=s.handle)
      b.ffn_down_exps(sel, act, y, jobs_per_x_row=1, stream=s.handle)
    us = _time_launches(run, len(blks), 320, s)
    per_e = sum(e.expert_nbytes for e in (blks[0].ffn_gate_exps, blks[0].ffn_up_exps, blks[0].ffn_down_exps))
    nbytes = B * k * per_e                                                  # every (token, slot) job streams its expert once
    res.append({"config": 4, "case": f"expert GEMVs of one layer, B={B} ({B * k} jobs, {len(np.unique(sel_host))} distinct experts)", "avg_us": round(us, 2),
                "alg_bytes": nbytes, "GBps": round(nbytes / us / 1e3, 1), "frac_hbm_peak": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4)})
  return res

def mfma_peak() -> dict:
  L, s = rt.lib(), rt.Stream()
  scratch = Buffer((64,), np.float32).zero_()
  wgs, loops = 256 * 4, 2000
  rt.check(L.tga_mfma_peak(wgs, 10, scratch.ptr, s.handle)); s.synchronize()
  e0, e1 = rt.Event(), rt.Event(); e0.record(s.handle)
  rt.check(L.tga_mfma_peak(wgs, loops, scratch.ptr, s.handle))
  e1.record(s.handle); e1.synchronize()
  ms = e0.elapsed_ms(e1)
  flops = wgs * 4 * loops * 200 * 65536
  return {"config": 5, "case": "register-only v_mfma_scale_f32_16x16x128_f8f6f4 (1024 workgroups x 4 waves x 2000 x 200)", "ms": round(ms, 3),
          "TFLOPs": round(flops / ms / 1e9, 1), "frac_of_5_PFLOPs": round(flops / ms / 1e9 / MFMA_FP8_PEAK_TFLOPS, 4)}

def config5():
  """Grouped MXFP8 GEMM of the MoE prefill: T = 4096 tokens, E = 128, k = 8, d = 2048, gate/up (128, 1536, 2048), down (128, 2048, 768)."""
  from tinygrad_amd import moe
  L = rt.lib()
  T, E, k, D, I2, I = 4096, 128, 8, 2048, 1536, 768
  rng = np.random.default_rng(1005)
  # Zipf(1.1) expert popularity over a fixed random permutation, no duplicate expert within a token: logits = log(popularity) + Gumbel
  pop = 1.0 / np.arange(1, E + 1) ** 1.1
  logits = (np.log(pop[rng.permutation(E)])[None, :] + rng.gumbel(size=(T, E))).astype(np.float32)
  s = rt.Stream()
  r = moe.route(Buffer.from_numpy(logits), k, E, stream=s.handle)
  s.synchronize()
  off = r.off.numpy(); counts = r.counts.numpy()
  m_used = int(off[-1])
  def rand_mx(shape_rows, K):
    q = rng.integers(0, 256, size=(shape_rows, K), dtype=np.uint8); q[(q & 0x7F) == 0x7F] = 0x38      # no E4M3 NaN codes
    e8 = rng.integers(121, 126, size=(shape_rows, K // 32), dtype=np.uint8)
    return Buffer.from_numpy(q), Buffer.from_numpy(e8)
  res = [mfma_peak()]
  for name, N, K in (("gate/up", I2, D), ("down", D, I)):
    wq, we = rand_mx(E * N, K)
    xq, xe = rand_mx(r.m_l, K)
    out = Buffer((r.m_l, N), np.uint16)
    # the launch moe.moe_feed_forward makes: routed tiles only (combine never reads the rows beyond expert_off[E]); the reference's kernel also
    # multiplies the m_l - off[E] worst-case padding rows with the last expert, which tga_grouped_mxfp8_gemm does too (timed second)
    fn = lambda i: rt.check(L.tga_grouped_mxfp8_gemm_routed(out.ptr, xq.ptr, wq.ptr, xe.ptr, we.ptr, r.off.ptr, r.m_l, N, K, E, s.handle))
    us = _time_launches(fn, 1, 50, s)
    fn_all = lambda i: rt.check(L.tga_grouped_mxfp8_gemm(out.ptr, xq.ptr, wq.ptr, None, None, xe.ptr, we.ptr, r.off.ptr, r.m_l, N, K, E, s.handle))
    us_all = _time_launches(fn_all, 1, 50, s)
    fn_cnt = lambda i: rt.check(L.tga_grouped_mxfp8_gemm_counts(out.ptr, xq.ptr, wq.ptr, xe.ptr, we.ptr, r.off.ptr, r.counts.ptr, r.m_l, N, K, E, s.handle))
    us_cnt = _time_launches(fn_cnt, 1, 50, s)
    flops_unpadded = 2 * T * k * N * K
    flops_padded = 2 * m_used * N * K
    nbytes = E * N * K + E * N * K // 32 + T * k * K + T * k * K // 32 + T * k * N * 2
    res.append({"config": 5, "case": f"grouped MXFP8 GEMM {name}: {T * k} routed rows ({m_used} after 256-row padding), N={N}, K={K}, E={E}, Zipf(1.1) routing "
                f"(busiest expert {int(counts.max())} rows, idlest {int(counts.min())})", "avg_us": round(us, 1),
                "TFLOPs_unpadded": round(flops_unpadded / us / 1e6, 1), "mfma_utilisation_vs_5_PFLOPs": round(flops_unpadded / us / 1e6 / MFMA_FP8_PEAK_TFLOPS, 4),
                "TFLOPs_with_padding_rows": round(flops_padded / us / 1e6, 1), "alg_bytes": nbytes, "GBps": round(nbytes / us / 1e3, 1),
                "frac_hbm_peak": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4),
                "avg_us_all_tiles_of_m_l": round(us_all, 1), "rows_m_l": int(r.m_l),
                "avg_us_routed_rows_only": round(us_cnt, 1), "mfma_utilisation_routed_rows_only": round(flops_unpadded / us_cnt / 1e6 / MFMA_FP8_PEAK_TFLOPS, 4)})
  return res

def traffic(steps: int = 4):
  """Workload for the HBM-traffic counter runs (rocprofv3 --pmc FETCH_SIZE, then --pmc WRITE_SIZE, one run each):

      rocprofv3 --pmc FETCH_SIZE --output-format csv -d out -o t -- python3 -m tinygrad_amd.benchmarks --traffic

  one 1 GiB plain copy kernel (the yardstick: it must read 1 GiB and write 1 GiB), then a few eager decode steps of the benchmark model
  after a two-token prompt.  The dequant-GEMV launches do not depend on the context length, so the KV cache is not prefilled: a counter run
  intercepts every dispatch, and a 1024-token prefill would be 200 000 of them."""
  from tinygrad_amd.llm import Transformer, TransformerConfig, synth_state, LLAMA3_8B
  n = 1 << 30
  a, b = Buffer((n,), np.uint8).zero_(), Buffer((n,), np.uint8)
  rt.check(rt.lib().tga_copy_kernel(b.ptr, a.ptr, n, None)); rt.synchronize()
  c = TransformerConfig(max_context=64, **LLAMA3_8B)
  model = Transformer(c, synth_state(c, seed=1003), max_new=16)
  model.prefill([17, 4242], use_graph=False)
  for _ in range(steps): model.decode_step(use_graph=False)
  model.check_state()
  return [{"traffic_probe": "done", "copy_bytes": n, "decode_steps": steps}]

def prefill_trace(chunk: int = 64):
  """Workload for the kernel trace of a chunked prefill (rocprofv3 --kernel-trace --stats -- python3 -m tinygrad_amd.benchmarks --prefill 64): the 8B architecture
  of configuration 3 (Q4_0, Q6_K lm-head), 1023 positions in steps of `chunk`, launched eagerly twice (the first pass also sizes the step models); the
  wall time of the second pass is reported (eager launches: the replayed steps of configuration 8 are faster)."""
  from tinygrad_amd.llm import Transformer, TransformerConfig, synth_state, LLAMA3_8B
  import time
  c = TransformerConfig(max_context=1152, **LLAMA3_8B)
  model = Transformer(c, synth_state(c, seed=1003), max_new=4)
  model.prefill_chunk = chunk
  rng = np.random.default_rng(1003)
  prompt = [int(t) for t in rng.integers(0, c.vocab_size, size=1024)]
  model.prefill(prompt, False, reuse_cache=False)
  rt.synchronize()
  t0 = time.perf_counter()
  model.prefill(prompt, False, reuse_cache=False)
  rt.synchronize()
  return [{"prefill_trace": "done", "positions": 1023, "per_step": chunk, "eager_ms": round((time.perf_counter() - t0) * 1e3, 1)}]

def main():
  ap = argparse.ArgumentParser()
  ap.add_argument("--config", type=int, nargs="*", default=[1, 2, 4, 5], help="1, 2, 4, 5 = the benchmark's configurations; 6 = Q4_K / Q5_K / Q4_1 / Q5_0 / Q5_1 / IQ4_XS GEMV shapes; 9 = IQ3_XXS / IQ3_S / IQ2_S / Q1_0 GEMV shapes; 7 = 8B decode with the Q4_K_M type mix; 8 = 8B chunked prefill and batched dense decode")
  ap.add_argument("--no-graph", action="store_true", help="configs 4 and 7: launch eagerly instead of replaying a captured graph (for profilers)")
  ap.add_argument("--traffic", action="store_true", help="only the workload of the HBM-traffic counter runs (see traffic())")
  ap.add_argument("--prefill", type=int, default=0, metavar="CHUNK", help="only the workload of the prefill kernel trace, CHUNK positions per step (see prefill_trace())")
  args = ap.parse_args()
  rt.init(0)
  print(json.dumps({"device": rt.device_name()}), flush=True)
  if args.traffic:
    for row in traffic(): print(json.dumps(row), flush=True)
    return
  if args.prefill:
    for row in prefill_trace(args.prefill): print(json.dumps(row), flush=True)
    return
  for cfg in args.config:
    fn = {1: config1, 2: config2, 4: config4, 5: config5, 6: kquants, 7: config7, 8: config8, 9: codebooks}[cfg]
    for row in (fn(use_graph=not args.no_graph) if cfg in (4, 7) else fn()): print(json.dumps(row), flush=True)

if __name__ == "__main__":
  main()
