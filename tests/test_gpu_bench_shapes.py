"""The benchmark's own kernel instantiations at the benchmark's own sizes, against the C restatement of the reference's model-path numerics
(oracle/c: dequant -> fp16-rounded weight (model.py:376) -> float32 accumulate), rel-err <= 1e-3 (the bar benchmark configuration 2 and the
reference's test/unit/test_gguf.py:193-233 protocol state):
  * the lm-head launch of the decode step: Q6_K 128256 x 4096 with output_norm folded in, M = 1, and the plain linear at M in {1, 2, 4, 8}
  * configuration 2's Q8_0 shapes 4096 x 4096, 14336 x 4096, 4096 x 14336 at M in {1, 2, 4, 8}
  * the four Q4_0 launches of a Llama-3-8B block (q/k/v with attn_norm, attn_output + residual, gate/up + SwiGLU with ffn_norm, down + residual)
  * configuration 5's grouped MXFP8 GEMMs (E = 128, Zipf(1.1) routing, N x K = 1536 x 2048 and 2048 x 768) on sampled rows of every kind of tile."""
import os
import numpy as np, pytest
from oracle import cref, linear as ol, llm as ollm, mxfp8 as omx
from tinygrad_amd import synth

pytestmark = pytest.mark.gpu
TOL = 1e-3
THREADS = min(16, len(os.sched_getaffinity(0)))

def _ref(t, w, x, n, k): return cref.linear(t, w, np.ascontiguousarray(x, dtype=np.float32), n, k, w_round_f16=True, threads=THREADS)

def test_lm_head_q6_k_full_size(gpu):
  """128256 x 4096 Q6_K (configuration 2's lm-head, 431 MB): the decode step's launch with the RMSNorm folded in (two rows per step, eight
  interleaved row teams per workgroup) and the plain linear at every batch size of the sweep."""
  from tinygrad_amd.nn import QuantLinear, qlinear_multi
  rng = np.random.default_rng(1002)
  n, k = 128256, 4096
  w = synth.random_blocks(rng, 14, n, k)
  lin = QuantLinear(gpu.Buffer.from_numpy(w), 14, n, k)
  # M = 1 with output_norm folded in (model.py:362): x is the float32 residual row, the kernel multiplies W by fp16(rmsnorm(x) * weight)
  x = (rng.standard_normal((1, k)) * 3).astype(np.float32); nw = (1 + 0.1 * rng.standard_normal(k)).astype(np.float32)
  y = gpu.Buffer((1, n), np.float32)
  qlinear_multi([lin], gpu.Buffer.from_numpy(x), [y], norm=(gpu.Buffer.from_numpy(nw), 1e-5))
  ref = _ref(14, w, ollm.rmsnorm(x, nw, 1e-5), n, k)
  e = ol.rel_err(y.numpy(), ref)
  print(f"lm-head with folded norm, M=1: rel-err {e:.2e}")
  assert e <= TOL
  for m in (1, 2, 4, 8):
    xm = synth.activations(rng, m, k, np.float16)
    ym = lin(gpu.Buffer.from_numpy(xm), out_dtype=np.float32).numpy()
    e = ol.rel_err(ym, _ref(14, w, xm, n, k))
    print(f"lm-head plain, M={m}: rel-err {e:.2e}")
    assert e <= TOL, m

@pytest.mark.parametrize("n,k", [(4096, 4096), (14336, 4096), (4096, 14336)])
def test_config2_q8_0_shapes(gpu, n, k):
  from tinygrad_amd.nn import QuantLinear
  rng = np.random.default_rng(1002 + n + k)
  w = synth.random_blocks(rng, 8, n, k)
  lin = QuantLinear(gpu.Buffer.from_numpy(w), 8, n, k)
  for m in (1, 2, 4, 8):
    xm = synth.activations(rng, m, k, np.float16)
    ym = lin(gpu.Buffer.from_numpy(xm), out_dtype=np.float32).numpy()
    e = ol.rel_err(ym, _ref(8, w, xm, n, k))
    print(f"Q8_0 {n}x{k} M={m}: rel-err {e:.2e}")
    assert e <= TOL, m

def test_llama3_8b_block_launches_q4_0(gpu):
  """The four dequant-GEMV launches of one Llama-3-8B block exactly as TransformerBlock.__call__ issues them (same entry points, same staging
  hand-overs), on seeded Q4_0 matrices, each against the C restatement fed the same fp32 row."""
  from tinygrad_amd.nn import QuantLinear, qlinear_multi
  rng = np.random.default_rng(1003)
  dim, hidden, nq, nkv = 4096, 14336, 4096, 1024
  mk = lambda n, k: synth.random_blocks(rng, 2, n, k)
  wq, wk, wv, wo, wg, wu, wd = mk(nq, dim), mk(nkv, dim), mk(nkv, dim), mk(dim, nq), mk(hidden, dim), mk(hidden, dim), mk(dim, hidden)
  L = lambda w, n, k: QuantLinear(gpu.Buffer.from_numpy(w), 2, n, k)
  lq, lk, lv, lo, lg, lu, ld = L(wq, nq, dim), L(wk, nkv, dim), L(wv, nkv, dim), L(wo, dim, nq), L(wg, hidden, dim), L(wu, hidden, dim), L(wd, dim, hidden)
  x = (rng.standard_normal((1, dim)) * 2).astype(np.float32)
  nw = (1 + 0.1 * rng.standard_normal(dim)).astype(np.float32)
  xb, nwb = gpu.Buffer.from_numpy(x), gpu.Buffer.from_numpy(nw)
  xn = ollm.rmsnorm(x, nw, 1e-5)
  # attn_norm -> q / k / v, one launch
  q, kk, v = gpu.Buffer((1, nq), np.float32), gpu.Buffer((1, nkv), np.float32), gpu.Buffer((1, nkv), np.float32)
  qlinear_multi([lq, lk, lv], xb, [q, kk, v], norm=(nwb, 1e-5))
  for got, w, n in ((q, wq, nq), (kk, wk, nkv), (v, wv, nkv)): assert ol.rel_err(got.numpy(), _ref(2, w, xn, n, dim)) <= TOL
  # attn_output + residual on an fp16 row staged by its producer (the attention merge writes this order; here tga_stage_activation does)
  from tinygrad_amd.nn import stage_activation
  attn = synth.activations(rng, 1, nq, np.float16)
  staged = stage_activation(lo, gpu.Buffer.from_numpy(attn))
  h = gpu.Buffer.from_numpy(x.copy())
  qlinear_multi([lo], staged, [h], epilogue=1, resid=[h], x_staged=True)
  href = x + _ref(2, wo, attn, dim, nq)
  assert ol.rel_err(h.numpy(), href) <= TOL
  # ffn_norm -> gate / up -> SwiGLU, written in the staged order of ffn_down; then down + residual
  act = gpu.Buffer((1, hidden), np.float16)
  qlinear_multi([lg, lu], h, [act], epilogue=2, norm=(nwb, 1e-5), stage_out_for=ld)
  hn = ollm.rmsnorm(h.numpy(), nw, 1e-5)
  g, u = _ref(2, wg, hn, hidden, dim), _ref(2, wu, hn, hidden, dim)
  aref = ollm.silu(g) * u
  out = gpu.Buffer.from_numpy(h.numpy())
  qlinear_multi([ld], act, [out], epilogue=1, resid=[out], x_staged=True)
  oref = h.numpy() + _ref(2, wd, aref, dim, hidden)
  assert ol.rel_err(out.numpy() - h.numpy(), oref - h.numpy()) <= 2 * TOL       # two chained linears: each within the bar
  assert ol.rel_err(out.numpy(), oref) <= TOL

def _zipf_routing(gpu, T=4096, E=128, k=8, seed=1005):
  from tinygrad_amd import moe
  rng = np.random.default_rng(seed)
  pop = 1.0 / np.arange(1, E + 1) ** 1.1
  logits = (np.log(pop[rng.permutation(E)])[None, :] + rng.gumbel(size=(T, E))).astype(np.float32)
  r = moe.route(gpu.Buffer.from_numpy(logits), k, E)
  gpu.synchronize()
  return r, rng

@pytest.mark.parametrize("N,K", [(1536, 2048), (2048, 768)], ids=["gate_up", "down"])
def test_config5_grouped_gemm_full_size(gpu, N, K):
  """E = 128 experts, 32768 Zipf-routed rows padded per expert to 256 inside an m_l = 65536 row buffer: sampled rows of the first, a middle and the
  last tile of several experts, of the busiest and the idlest expert, and of the tiles beyond expert_off[E] (expert E - 1 by rows_e) against the
  oracle; then the routed-only variant leaves exactly the rows beyond expert_off[E] alone and agrees everywhere else."""
  from tinygrad_amd import moe
  E = 128
  r, rng = _zipf_routing(gpu)
  off, counts, M = r.off.numpy(), r.counts.numpy(), r.m_l
  assert M == 65536 and off[-1] < M
  def rand_mx(rows):
    q = rng.integers(0, 256, size=(rows, K), dtype=np.uint8); q[(q & 0x7F) == 0x7F] = 0x38            # no NaN codes
    return q, rng.integers(121, 126, size=(rows, K // 32), dtype=np.uint8)
  xq, xe = rand_mx(M); wq, we = rand_mx(E * N)
  bufs = [gpu.Buffer.from_numpy(a) for a in (xq, wq, xe, we)]
  C = gpu.Buffer((M, N), np.uint16)
  gpu.check(gpu.lib().tga_memset(C.ptr, 0xAB, C.nbytes, None))
  gpu.check(gpu.lib().tga_grouped_mxfp8_gemm(C.ptr, bufs[0].ptr, bufs[1].ptr, None, None, bufs[2].ptr, bufs[3].ptr, r.off.ptr, M, N, K, E, None))
  got = moe.from_bf16_bits(C.numpy())
  te = omx.tile_experts(off, M)
  busiest, idlest = int(np.argmax(counts)), int(np.argmin(np.where(counts > 0, counts, 1 << 30)))
  rows = set()
  for e in (0, 1, 63, 127, busiest, idlest):
    if off[e + 1] > off[e]: rows.update({int(off[e]), int(off[e]) + 255, int(off[e + 1]) - 1, int(off[e] + off[e + 1]) // 2})
  rows.update({int(off[-1]), int(off[-1]) + 300, M - 1})                                               # beyond the routed range
  wq3, we3 = wq.reshape(E, N, K), we.reshape(E, N, K // 32)
  for row in sorted(rows):
    e = int(te[row // 256])
    xd = omx.to_bf16(omx.dequant_mxfp8(xq[row:row + 1], xe[row:row + 1])).astype(np.float64)
    wd = omx.to_bf16(omx.dequant_mxfp8(wq3[e], we3[e])).astype(np.float64)
    ref = omx.to_bf16((xd @ wd.T).astype(np.float32))[0]
    np.testing.assert_allclose(got[row], ref, rtol=2 ** -7, atol=1e-3 * np.abs(ref).max(), err_msg=f"row {row} expert {e}")
  assert np.isfinite(got).all()
  C2 = gpu.Buffer((M, N), np.uint16)
  gpu.check(gpu.lib().tga_memset(C2.ptr, 0xAB, C2.nbytes, None))
  gpu.check(gpu.lib().tga_grouped_mxfp8_gemm_routed(C2.ptr, bufs[0].ptr, bufs[1].ptr, bufs[2].ptr, bufs[3].ptr, r.off.ptr, M, N, K, E, None))
  c1, c2 = C.numpy(), C2.numpy()
  np.testing.assert_array_equal(c2[:off[-1]], c1[:off[-1]])
  assert (c2[off[-1]:] == 0xABAB).all()
