"""Fused dequant-GEMV / small-batch GEMM on the GPU vs the oracle.

Bar: rel-err = max|y - ref| / max|ref| <= 1e-3 against the float64 textbook product of the exact dequantized weights, and the
same bound against the restatement of the reference's own numerics (model path: fp16-rounded weights; standalone: fp16 products).
fp16 outputs must equal the RNE cast of the float32 output of the same kernel."""
import numpy as np, pytest
from oracle import ggml as og, linear as ol, cref
from tinygrad_amd import synth
from tinygrad_amd.runtime import GGML_QUANT

pytestmark = pytest.mark.gpu
TOL = 1e-3

def _run(gpu, t, w, x, n, k, ydt=np.float32):
  from tinygrad_amd.nn import QuantLinear
  lin = QuantLinear(gpu.Buffer.from_numpy(w), t, n, k)
  return lin(gpu.Buffer.from_numpy(x), out_dtype=ydt).numpy()

def _check(y, x, W):
  ref64 = ol.linear_f64(x.astype(np.float32), W)
  e = ol.rel_err(y, ref64)
  assert e <= TOL, f"rel-err {e:.3e} vs float64 anchor"
  # elementwise: allclose in the sense of the reference's VALIDATE_WITH_CPU harness (engine/realize.py:192-201), atol scaled to the output rms.
  # The anchor is the exact-weight result or the result with weights rounded to fp16 (the reference's model path casts every weight to
  # fp16, model.py:376; the matrix-core kernel for M >= 3 rounds them the same way, the dot2 kernels use them exactly)
  atol = TOL * float(np.sqrt(np.mean(ref64 ** 2)))
  with np.errstate(over="ignore"): ref16 = ol.linear_f64(x.astype(np.float32), W.astype(np.float16).astype(np.float32))
  close = np.isclose(y, ref64, rtol=TOL, atol=atol) | np.isclose(y, ref16, rtol=TOL, atol=atol)
  assert close.all(), f"{np.count_nonzero(~close)} of {close.size} outputs outside rtol/atol {TOL}"
  return e

@pytest.mark.parametrize("t", [2, 3, 6, 7, 8, 12, 13, 14, 23, 39, 18, 21, 22, 41])
@pytest.mark.parametrize("m", [1, 2, 3, 4, 5, 6, 7, 8])
def test_small_shapes_all_batches(gpu, t, m):
  rng = np.random.default_rng(1000 * t + m)
  n, k = 257, 1024                       # odd row count: the last row group is ragged
  w = synth.random_blocks(rng, t, n, k)
  x = synth.activations(rng, m, k, np.float16)
  W = ol.weight_f32(w, n, k, t)
  y = _run(gpu, t, w, x, n, k)
  _check(y, x, W)
  # against the C restatement of the reference's model path (fp16-rounded weights, float32 accumulate)
  ym = cref.linear(t, w, x, n, k, w_round_f16=True)
  assert ol.rel_err(y, ym) <= TOL

@pytest.mark.parametrize("t,k", [(2, 32), (2, 96), (2, 4096 + 32), (8, 32), (8, 160), (39, 32), (39, 2048 + 64), (14, 256), (14, 768), (14, 4096 + 256), (12, 256), (12, 4096 + 256), (23, 256), (23, 768), (23, 4096 + 256), (23, 16384), (13, 768), (13, 8192 + 512),
                                 (3, 64), (3, 4096 + 64), (6, 192), (6, 2048 + 128), (7, 64), (7, 8192 + 64),
                                 (18, 256), (18, 4096 + 256), (21, 768), (21, 16384), (22, 256), (22, 8192 + 512), (41, 128), (41, 4096 + 128), (41, 32768 + 128)])
def test_ragged_k(gpu, t, k):
  """K that is not a multiple of 64 units per row: partially filled waves."""
  rng = np.random.default_rng(k + t)
  n = 130
  w = synth.random_blocks(rng, t, n, k)
  x = synth.activations(rng, 2, k, np.float16)
  _check(_run(gpu, t, w, x, n, k), x, ol.weight_f32(w, n, k, t))

@pytest.mark.parametrize("t", [2, 3, 6, 7, 8, 12, 13, 14, 23, 39, 18, 21, 22, 41])
def test_f32_activations_and_f16_output(gpu, t):
  rng = np.random.default_rng(31 + t)
  n, k = 512, 2048
  w = synth.random_blocks(rng, t, n, k)
  x32 = synth.activations(rng, 1, k, np.float32)
  W = ol.weight_f32(w, n, k, t)
  y32 = _run(gpu, t, w, x32, n, k, np.float32)
  _check(y32, x32, W)                       # fp32 x is rounded to fp16 inside the kernel: still inside the 1e-3 bar
  assert ol.rel_err(y32, ol.linear_model(x32, W)) <= TOL
  y16 = _run(gpu, t, w, x32, n, k, np.float16)
  assert y16.tobytes() == y32.astype(np.float16).tobytes()

def test_config1_q4_0_4096(gpu):
  """benchmark configuration 1 at full size: W 4096x4096 Q4_0, x fp16 [1,4096], fp32 accumulate, fp16 out (seed 1001)."""
  w, x, (n, k) = synth.config1()
  W = ol.weight_f32(w, n, k, 2)
  y32 = _run(gpu, 2, w, x, n, k, np.float32)
  e = _check(y32, x, W)
  y16 = _run(gpu, 2, w, x, n, k, np.float16)
  assert y16.tobytes() == y32.astype(np.float16).tobytes()
  # the reference's own standalone numerics (fp16 products, fp32 accumulate, fp16 out): within 1e-3 + one fp16 ulp of the output
  ref16 = ol.linear_standalone_f16(x, W).astype(np.float32)
  tol = TOL * np.abs(ref16).max() + np.spacing(np.abs(ref16).astype(np.float16)).astype(np.float32)
  assert (np.abs(y16.astype(np.float32) - ref16) <= tol).all()
  print(f"config1 rel-err vs f64 anchor {e:.2e}")

@pytest.mark.parametrize("t,n,k,m", [(8, 4096, 14336, 8), (8, 512, 14336, 5), (2, 300, 14336, 8), (14, 200, 8192, 8), (12, 200, 14336, 8), (13, 136, 8192, 6), (23, 200, 14336, 8), (23, 4096, 4096, 5),
                                     (3, 200, 14336, 8), (6, 136, 14336, 7), (7, 200, 8192, 8), (22, 200, 14336, 8), (18, 136, 14336, 2), (21, 264, 16384, 7), (41, 200, 14336, 8)])
def test_chunked_k_large_batch(gpu, t, n, k, m):
  """M*K activations beyond the LDS budget: the kernel walks K in chunks."""
  rng = np.random.default_rng(n + k + m)
  w = synth.random_blocks(rng, t, n, k)
  x = synth.activations(rng, m, k, np.float16)
  y = _run(gpu, t, w, x, n, k)
  ref = cref.linear(t, w, x, n, k, threads=8)
  assert ol.rel_err(y, ref) <= TOL

def test_multi_segment_and_epilogues(gpu):
  from tinygrad_amd.nn import QuantLinear, qlinear_multi
  rng = np.random.default_rng(77)
  k = 1024
  ns = [512, 128, 130]
  ws = [synth.random_blocks(rng, 2, n, k) for n in ns]
  x = synth.activations(rng, 1, k, np.float16)
  layers = [QuantLinear(gpu.Buffer.from_numpy(w), 2, n, k) for w, n in zip(ws, ns)]
  xb = gpu.Buffer.from_numpy(x)
  outs = [gpu.Buffer((1, n), np.float32) for n in ns]
  qlinear_multi(layers, xb, outs)
  refs = [ol.linear_f64(x.astype(np.float32), ol.weight_f32(w, n, k, 2)) for w, n in zip(ws, ns)]
  for o, r in zip(outs, refs): assert ol.rel_err(o.numpy(), r) <= TOL
  # residual epilogue, in place
  res = [rng.standard_normal((1, n)).astype(np.float32) for n in ns]
  rb = [gpu.Buffer.from_numpy(r) for r in res]
  qlinear_multi(layers, xb, rb, epilogue=1, resid=rb)
  for o, r0, r in zip(rb, res, refs): assert ol.rel_err(o.numpy(), r0 + r) <= TOL
  # SwiGLU epilogue: silu(gate) * up (tinygrad/llm/model.py:137)
  g = [QuantLinear(gpu.Buffer.from_numpy(ws[1]), 2, 128, k), QuantLinear(gpu.Buffer.from_numpy(synth.random_blocks(rng, 2, 128, k)), 2, 128, k)]
  out = gpu.Buffer((1, 128), np.float32)
  qlinear_multi(g, xb, [out], epilogue=2)
  a = ol.linear_f64(x.astype(np.float32), ol.weight_f32(g[0].blocks.numpy(), 128, k, 2))
  b = ol.linear_f64(x.astype(np.float32), ol.weight_f32(g[1].blocks.numpy(), 128, k, 2))
  ref = a / (1 + np.exp(-a)) * b
  assert ol.rel_err(out.numpy(), ref) <= TOL

@pytest.mark.parametrize("t", [2, 8, 14, 1, 39, 21, 22], ids=["q4_0", "q8_0", "q6_k", "f16", "mxfp4", "iq3_s", "iq2_s"])
@pytest.mark.parametrize("m", [2, 3, 5, 8])
def test_multi_segment_small_batch(gpu, t, m):
  """q / k / v in one launch at 2..8 activation rows: from three rows on the matrix-core kernel walks all three matrices (every one a multiple of
  16 rows); a segment that is not (130 rows) sends the call to the dot2 kernel.  Both against the float64 anchor."""
  from tinygrad_amd.nn import QuantLinear, qlinear_multi
  rng = np.random.default_rng(770 + t + m)
  k = 1024
  for ns in ([512, 128, 144], [512, 128, 130]):
    mk = lambda n: (rng.standard_normal((n, k)) * k ** -0.5).astype(np.float16).view(np.uint8).reshape(-1) if t == 1 else synth.random_blocks(rng, t, n, k)
    ws = [mk(n) for n in ns]
    x = synth.activations(rng, m, k, np.float16)
    layers = [QuantLinear(gpu.Buffer.from_numpy(w), t, n, k) for w, n in zip(ws, ns)]
    outs = [gpu.Buffer((m, n), np.float32) for n in ns]
    for o in outs: gpu.check(gpu.lib().tga_memset(o.ptr, 0xFF, o.nbytes, None))
    qlinear_multi(layers, gpu.Buffer.from_numpy(x), outs)
    for o, w, n in zip(outs, ws, ns):
      wf = w.view(np.float16).astype(np.float32).reshape(n, k) if t == 1 else ol.weight_f32(w, n, k, t)
      assert ol.rel_err(o.numpy(), ol.linear_f64(x.astype(np.float32), wf)) <= TOL, (ns, n)

@pytest.mark.parametrize("t", [2, 8], ids=["q4_0", "q8_0"])
@pytest.mark.parametrize("n,k,m", [(16, 1024, 3), (4096 + 48, 1024, 8), (14336, 4096, 4), (4112, 4096, 8), (512, 2048, 5), (1040, 8192, 4), (272, 8192, 8), (4096, 3072, 7)])
def test_small_batch_weights_through_lds(gpu, t, n, k, m):
  """The matrix-core kernel that streams the weights into LDS with contiguous 16-byte pieces (Q4_0 / Q8_0 pairs, K a multiple of 1024, rows a
  multiple of 16): one stage per row group (K = 1024) up to eight, one row group per workgroup up to several with a ragged share, the largest
  activation blocks that still leave room for a ring of three stages, and (8192, M = 8) which does not and takes the register-fed kernel.
  Against the C restatement (exact weights, float32 accumulate) and, for the first rows, the float64 anchor; float32 and fp16 activations."""
  rng = np.random.default_rng(n + k + m + t)
  w = synth.random_blocks(rng, t, n, k)
  x = synth.activations(rng, m, k, np.float16)
  y = _run(gpu, t, w, x, n, k)
  ref = cref.linear(t, w, x, n, k, threads=8)
  assert ol.rel_err(y, ref) <= TOL
  rows = min(n, 64)
  nel, nby = GGML_QUANT[t]
  W = ol.weight_f32(w[:rows * (k // nel) * nby], rows, k, t)
  assert ol.rel_err(y[:, :rows], ol.linear_f64(x.astype(np.float32), W)) <= TOL
  y32 = _run(gpu, t, w, x.astype(np.float32), n, k)                      # float32 activations are rounded to fp16 while they are staged
  np.testing.assert_array_equal(y32, y)
  y16 = _run(gpu, t, w, x, n, k, ydt=np.float16)
  assert y16.tobytes() == y.astype(np.float16).tobytes()

@pytest.mark.parametrize("t", [2, 8, 14], ids=["q4_0", "q8_0", "q6_k"])
@pytest.mark.parametrize("n,k", [(8192 + 3, 4096), (14336, 4096), (2400, 14336), (5500, 6144), (15889, 2112), (300, 4096)])
def test_two_rows_on_the_single_row_kernel(gpu, t, n, k):
  if t == 14 and k % 256: k = k // 256 * 256 + 256                       # Q6_K rows are whole 256-value superblocks
  """M = 2 for Q4_0 / Q8_0 rows of more than 32 block pairs runs on the single-row kernel's walk with two sets of activations in registers:
  rows that one wave covers (K <= 4096) and K split over four waves, ragged row counts, more row groups than teams (from 2^25 weights on; the last,
  smaller shape stays on the LDS-staged kernel).  Exact weights, so the bar is
  the float64 anchor of the exact dequantized weights (first rows) and the C restatement (all rows); fp32 activations and fp16 outputs as well."""
  rng = np.random.default_rng(2 * n + k + t)
  w = synth.random_blocks(rng, t, n, k)
  x = synth.activations(rng, 2, k, np.float16)
  y = _run(gpu, t, w, x, n, k)
  assert ol.rel_err(y, cref.linear(t, w, x, n, k, threads=8)) <= TOL
  rows = min(n, 64)
  nel, nby = GGML_QUANT[t]
  W = ol.weight_f32(w[:rows * (k // nel) * nby], rows, k, t)
  assert ol.rel_err(y[:, :rows], ol.linear_f64(x.astype(np.float32), W)) <= TOL
  np.testing.assert_array_equal(_run(gpu, t, w, x.astype(np.float32), n, k), y)
  assert _run(gpu, t, w, x, n, k, ydt=np.float16).tobytes() == y.astype(np.float16).tobytes()

def test_two_rows_segments_and_residual(gpu):
  """q / k / v in one launch at M = 2 (K = 4096: the two-row walk over three matrices, teams crossing from one matrix into the next) and the
  residual epilogue in place."""
  from tinygrad_amd.nn import QuantLinear, qlinear_multi
  rng = np.random.default_rng(2424)
  k, m = 4096, 2
  ns = [8192, 136, 130]
  for t in (2, 8):
    ws = [synth.random_blocks(rng, t, n, k) for n in ns]
    x = synth.activations(rng, m, k, np.float16)
    layers = [QuantLinear(gpu.Buffer.from_numpy(w), t, n, k) for w, n in zip(ws, ns)]
    outs = [gpu.Buffer((m, n), np.float32) for n in ns]
    for o in outs: gpu.check(gpu.lib().tga_memset(o.ptr, 0xFF, o.nbytes, None))
    xb = gpu.Buffer.from_numpy(x)
    qlinear_multi(layers, xb, outs)
    refs = [ol.linear_f64(x.astype(np.float32), ol.weight_f32(w, n, k, t)) for w, n in zip(ws, ns)]
    for o, r in zip(outs, refs): assert ol.rel_err(o.numpy(), r) <= TOL
    res = [rng.standard_normal((m, n)).astype(np.float32) for n in ns]
    rb = [gpu.Buffer.from_numpy(r) for r in res]
    qlinear_multi(layers, xb, rb, epilogue=1, resid=rb)
    for o, r0, r in zip(rb, res, refs): assert ol.rel_err(o.numpy(), r0 + r) <= TOL

@pytest.mark.parametrize("t", [2, 8], ids=["q4_0", "q8_0"])
@pytest.mark.parametrize("n,k,m", [(8, 1024, 3), (264, 2048, 8), (2056, 3072, 5), (14336, 4096, 8), (4096, 4096, 4), (14336, 4096, 2), (8200 + 1, 4096, 2), (2400, 14336, 2), (300, 4096, 2)])
def test_small_batch_swiglu_through_lds(gpu, t, n, k, m):
  """silu(gate) * up (tinygrad/llm/model.py:137) at 3..8 activation rows on the LDS-fed matrix-core kernel: a row group is eight gate rows and the same
  eight up rows.  At two rows (from 2^25 weights per matrix on) the single-row kernel's walk with two sets of activations forms the product, rows that one
  wave covers and K split over four waves.  Against the float64 product of the exact dequantized weights; fp16 and float32 outputs."""
  from tinygrad_amd.nn import QuantLinear, qlinear_multi
  rng = np.random.default_rng(n + k + m + 7 * t)
  wg, wu = synth.random_blocks(rng, t, n, k), synth.random_blocks(rng, t, n, k)
  x = synth.activations(rng, m, k, np.float16)
  layers = [QuantLinear(gpu.Buffer.from_numpy(wg), t, n, k), QuantLinear(gpu.Buffer.from_numpy(wu), t, n, k)]
  xb = gpu.Buffer.from_numpy(x)
  a = ol.linear_f64(x.astype(np.float32), ol.weight_f32(wg, n, k, t)); b = ol.linear_f64(x.astype(np.float32), ol.weight_f32(wu, n, k, t))
  ref = a / (1 + np.exp(-a)) * b
  for ydt in (np.float32, np.float16):
    out = gpu.Buffer((m, n), ydt)
    gpu.check(gpu.lib().tga_memset(out.ptr, 0xFF, out.nbytes, None))
    qlinear_multi(layers, xb, [out], epilogue=2)
    y = out.numpy().astype(np.float32)
    assert ol.rel_err(y, ref) <= (TOL if ydt == np.float32 else 2 * TOL), ydt

@pytest.mark.parametrize("t,n,k,m", [(2, 4096, 4096, 16), (2, 528, 2048, 9), (8, 14336, 4096, 13), (8, 64, 1024, 16), (2, 200, 14336, 16), (14, 300, 4096, 11), (2, 257, 1024, 12), (1, 96, 2048, 16), (23, 528, 4096, 16), (23, 300, 14336, 9), (21, 300, 4096, 11), (41, 528, 2048, 16)])
def test_nine_to_sixteen_rows(gpu, t, n, k, m):
  """Prefill chunks of up to sixteen rows: one launch of the LDS-fed kernel where it applies (all sixteen columns of the MFMA tile), otherwise two
  calls of at most eight rows (K beyond 4096, other formats, ragged row counts).  Against the C restatement run in blocks of eight rows."""
  rng = np.random.default_rng(3 * n + k + m + t)
  if t == 1: w = (rng.standard_normal((n, k)) * k ** -0.5).astype(np.float16).view(np.uint8).reshape(-1)
  else: w = synth.random_blocks(rng, t, n, k)
  x = synth.activations(rng, m, k, np.float16)
  y = _run(gpu, t, w, x, n, k)
  if t == 1: ref = ol.linear_f64(x.astype(np.float32), w.view(np.float16).astype(np.float32).reshape(n, k))
  else: ref = np.concatenate([cref.linear(t, w, x[i:i + 8], n, k, threads=8) for i in range(0, m, 8)])
  assert y.shape == (m, n) and ol.rel_err(y, ref) <= TOL
  np.testing.assert_array_equal(_run(gpu, t, w, x.astype(np.float32), n, k), y)

@pytest.mark.parametrize("t,n,k,m", [(2, 4096, 4096, 32), (12, 528, 2048, 24), (8, 200, 14336, 40), (14, 1024, 4096, 64), (2, 512, 14336, 17), (13, 300, 4096, 48), (23, 528, 4096, 64), (12, 4096, 4096, 17),
                                     (8, 1000, 1024, 33), (14, 72, 256, 50), (2, 200, 2048 + 32, 40), (3, 200, 2048, 40), (39, 256, 2048, 24), (18, 528, 2048, 24), (22, 300, 4096, 40),
                                     (2, 4096, 4096, 128), (12, 528, 2048, 100), (8, 200, 14336, 65), (14, 1024, 4096, 128), (23, 528, 4096, 96), (13, 300, 4096, 80), (39, 256, 2048, 70)])
def test_seventeen_to_sixty_four_rows(gpu, t, n, k, m):
  """Prefill chunks of 17 .. 128 rows: one pass of the prefill kernel where it applies (K a multiple of 256, its formats), otherwise blocks of sixteen (and a rest)
  through the small-batch kernels: plain, with the residual in place and with the norm in front (tga_rmsnorm_qlinear_rows), against the C restatement run in
  blocks of eight rows."""
  from tinygrad_amd.nn import QuantLinear, qlinear_multi
  rng = np.random.default_rng(3 * n + k + m + t)
  w = synth.random_blocks(rng, t, n, k)
  x = synth.activations(rng, m, k, np.float16)
  ref = np.concatenate([cref.linear(t, w, x[i:i + 8], n, k, threads=8) for i in range(0, m, 8)])
  y = _run(gpu, t, w, x, n, k)
  assert y.shape == (m, n) and ol.rel_err(y, ref) <= TOL
  assert ol.rel_err(y[:16], _run(gpu, t, w, x[:16], n, k)) <= 1e-4        # (the sixteen-row kernels sum K in another order)
  np.testing.assert_array_equal(_run(gpu, t, w, x.astype(np.float32), n, k), y)
  layer = QuantLinear(gpu.Buffer.from_numpy(w), t, n, k)
  res = rng.standard_normal((m, n)).astype(np.float32)
  rb = gpu.Buffer.from_numpy(res)
  qlinear_multi([layer], gpu.Buffer.from_numpy(x), [rb], epilogue=1, resid=[rb])
  assert ol.rel_err(rb.numpy(), res + ref) <= TOL
  x32 = (rng.standard_normal((m, k)) * 2).astype(np.float32); nw = (1 + 0.2 * rng.standard_normal(k)).astype(np.float32)
  xn = gpu.Buffer((m, k), np.float16); nb = gpu.Buffer.from_numpy(nw); out = gpu.Buffer((m, n), np.float32)
  qlinear_multi([layer], gpu.Buffer.from_numpy(x32), [out], norm=(nb, 1e-5, xn))
  h = xn.numpy()
  hn = x32 / np.sqrt((x32.astype(np.float64) ** 2).mean(-1, keepdims=True) + 1e-5) * nw
  assert ol.rel_err(h.astype(np.float32), hn.astype(np.float32)) <= 1e-3
  refn = np.concatenate([cref.linear(t, w, h[i:i + 8], n, k, threads=8) for i in range(0, m, 8)])
  assert ol.rel_err(out.numpy(), refn) <= TOL

@pytest.mark.parametrize("t,dim,hidden,m", [(2, 1024, 2048, 40), (8, 512, 1024, 17), (12, 1024, 2304, 64), (14, 512, 1024, 33), (23, 1024, 1024, 24), (13, 256, 512, 50), (2, 1024, 2048, 128), (12, 1024, 2304, 80), (14, 512, 1024, 100)])
def test_rows_in_the_multiplying_layout_equal_plain_rows(gpu, t, dim, hidden, m):
  """The entry points of a prefill step that hands its rows from launch to launch in the layout the prefill kernel multiplies from (tga_rmsnorm_rows_stage ->
  tga_qlinear_multi with staged x -> SwiGLU written for its consumer -> tga_qlinear_rows_deferred -> partial sums completed by the next norm or by
  tga_rows_add_partials) against the same linears on plain rows (tga_rmsnorm_qlinear_rows, tga_qlinear_multi): the same kernels multiply the same fp16 values, so the
  results agree to 1e-5 with the plain rows and bit for bit among the staged variants, except where a sum is taken in another order (residual first instead of last: 1e-6)."""
  import ctypes
  from tinygrad_amd.nn import QuantLinear, qlinear_multi
  from tinygrad_amd import runtime as rt
  L = gpu.lib()
  rng = np.random.default_rng(7 * t + m)
  ncg = ctypes.c_int(0)
  gpu.check(L.tga_rows_staged_plan(t, dim, m, ctypes.byref(ncg)))
  assert ncg.value == (2 if m <= 32 else 4 if m <= 64 else 8)
  gpu.check(L.tga_rows_staged_plan(39, 2048, m, ctypes.byref(ncg))); assert ncg.value == 0          # (MXFP4: no prefill kernel)
  gpu.check(L.tga_rows_staged_plan(t, dim, 16, ctypes.byref(ncg))); assert ncg.value == 0
  R = 16 * (2 if m <= 32 else 4 if m <= 64 else 8)
  gate, up = (QuantLinear(gpu.Buffer.from_numpy(synth.random_blocks(rng, t, hidden, dim)), t, hidden, dim) for _ in range(2))
  down = QuantLinear(gpu.Buffer.from_numpy(synth.random_blocks(rng, t, dim, hidden)), t, dim, hidden)
  x = (rng.standard_normal((m, dim)) * 2).astype(np.float32)
  nw = gpu.Buffer.from_numpy(((1 + 0.2 * rng.standard_normal(dim)) * (0.01 if t in (12, 13, 14, 23) else 1.0)).astype(np.float32))   # (random superblock scales are large: keep silu(g) * u inside fp16)
  # plain rows: norm + gate/up + SwiGLU, then down + residual in place
  xb, xn, act = gpu.Buffer.from_numpy(x), gpu.Buffer((m, dim), np.float16), gpu.Buffer((m, hidden), np.float16)
  qlinear_multi([gate, up], xb, [act], epilogue=2, norm=(nw, 1e-5, xn))
  qlinear_multi([down], act, [xb], epilogue=1, resid=[xb])
  ref = xb.numpy()
  # rows in the multiplying layout
  xs = gpu.Buffer.from_numpy(x)
  xn_st, act_st, xn2 = gpu.Buffer((R, dim), np.float16), gpu.Buffer((R, hidden), np.float16), gpu.Buffer((m, dim), np.float16)
  for b in (xn_st, act_st): gpu.check(L.tga_memset(b.ptr, 0xFF, b.nbytes, None))
  gpu.check(L.tga_rmsnorm_rows_stage(xs.ptr, None, 0, 0, nw.ptr, 1e-5, m, dim, t, xn2.ptr, xn_st.ptr, None))
  np.testing.assert_array_equal(xn2.numpy(), xn.numpy())
  VP2, I2 = ctypes.c_void_p * 2, ctypes.c_int64 * 2
  gpu.check(L.tga_qlinear_multi(t, 2, VP2(gate.blocks.ptr, up.blocks.ptr), VP2(act_st.ptr, None), I2(hidden, hidden), xn_st.ptr, rt.F16_STAGED, rt.F16, m, dim, 2, None, t, hidden, None))
  VP1, I1 = ctypes.c_void_p * 1, ctypes.c_int64 * 1
  yb = gpu.Buffer.from_numpy(x)                                                           # down + residual over the staged rows, sum taken by the call itself
  gpu.check(L.tga_qlinear_multi(t, 1, VP1(down.blocks.ptr), VP1(yb.ptr), I1(dim), act_st.ptr, rt.F16_STAGED, rt.F32, m, hidden, 1, VP1(yb.ptr), 0, 0, None))
  staged = yb.numpy()
  assert ol.rel_err(staged, ref) <= 1e-4                                                  # (the two SwiGLU epilogues are separate builds of silu(g) * u: a product may round the other way)
  part, ks, npitch = ctypes.c_void_p(), ctypes.c_int(-1), ctypes.c_int(-1)
  gpu.check(L.tga_qlinear_rows_deferred(t, down.blocks.ptr, dim, hidden, act_st.ptr, m, xs.ptr, ctypes.byref(part), ctypes.byref(ks), ctypes.byref(npitch), None))
  if ks.value:
    gpu.synchronize()
    np.testing.assert_array_equal(xs.numpy(), x)                                          # the sum is pending: y untouched
    xs2 = gpu.Buffer.from_numpy(x)
    gpu.check(L.tga_rows_add_partials(xs2.ptr, part.value, ks.value, npitch.value, m, dim, None))
    np.testing.assert_array_equal(xs2.numpy(), staged)
    # ... or completed by the next norm's launch, which also normalises the completed rows
    st2, xn3 = gpu.Buffer((R, dim), np.float16), gpu.Buffer((m, dim), np.float16)
    gpu.check(L.tga_rmsnorm_rows_stage(xs.ptr, part.value, ks.value, npitch.value, nw.ptr, 1e-5, m, dim, t, xn3.ptr, st2.ptr, None))
    assert ol.rel_err(xs.numpy(), staged) <= 1e-6
    h = xs.numpy(); hn = h / np.sqrt((h.astype(np.float64) ** 2).mean(-1, keepdims=True) + 1e-5) * nw.numpy()
    assert ol.rel_err(xn3.numpy().astype(np.float32), hn.astype(np.float32)) <= 1e-3
  else:
    np.testing.assert_array_equal(xs.numpy(), staged)
  # a staged call outside the kernel's range is refused, not run on other rows
  assert L.tga_qlinear_multi(39, 2, VP2(gate.blocks.ptr, up.blocks.ptr), VP2(act_st.ptr, None), I2(hidden, hidden), xn_st.ptr, rt.F16_STAGED, rt.F16, m, dim, 2, None, 0, 0, None) != 0

def test_seventeen_rows_on_more_streams_than_workspace_slots(gpu):
  """The prefill kernel keeps its staged activations and split-K partial tiles in a per-device workspace of a few slots, one per stream; a call on a
  further stream runs blocks of sixteen rows instead.  Six streams, two calls each (the second finds its stream's slot again): every result within the bar,
  and equal between the two calls of a stream."""
  from tinygrad_amd.nn import QuantLinear, qlinear_multi
  from tinygrad_amd import runtime as rt
  rng = np.random.default_rng(64)
  t, n, k, m = 2, 1024, 4096, 40
  w = synth.random_blocks(rng, t, n, k)
  layer = QuantLinear(gpu.Buffer.from_numpy(w), t, n, k)
  streams = [rt.Stream() for _ in range(6)]
  for st in streams:
    x = synth.activations(rng, m, k, np.float16)
    ref = np.concatenate([cref.linear(t, w, x[i:i + 8], n, k, threads=8) for i in range(0, m, 8)])
    xb = gpu.Buffer.from_numpy(x)
    outs = [gpu.Buffer((m, n), np.float32) for _ in range(2)]
    for o in outs: qlinear_multi([layer], xb, [o], stream=st.handle)
    st.synchronize()
    assert ol.rel_err(outs[0].numpy(), ref) <= TOL
    np.testing.assert_array_equal(outs[0].numpy(), outs[1].numpy())

@pytest.mark.parametrize("t,n,k,m", [(2, 4096, 14336, 16), (8, 4096, 14336, 8), (2, 256, 5120, 3), (8, 48, 14336, 9), (2, 4112, 8192, 13), (8, 1024, 6144, 16),
                                       (14, 4096, 14336, 8), (14, 48, 8192, 3), (14, 1040, 6144, 16), (14, 64, 5120, 5), (14, 272, 14336, 7)])
def test_small_batch_long_rows_through_lds(gpu, t, n, k, m):
  """K beyond 4096 on the LDS-fed kernel (one matrix): the activations stream beside the weights, whole lines per load, and reach
  the operand layout through a wave-private piece of LDS; float32 activations are rounded on the way into it.  Q6_K: slots of four superblocks (840 bytes) fetched
  as windows of 53 aligned pieces, the second slot of a stage 8 bytes into its window (K a multiple of 2048; beyond eight rows the ring holds two stages instead of three;
  K = 5120 takes the register-fed kernel).  Plain and with the residual added in place, against the C restatement run in blocks of eight rows."""
  from tinygrad_amd.nn import QuantLinear, qlinear_multi
  rng = np.random.default_rng(7 * n + k + m + t)
  w = synth.random_blocks(rng, t, n, k)
  x = synth.activations(rng, m, k, np.float16)
  ref = np.concatenate([cref.linear(t, w, x[i:i + 8], n, k, threads=8) for i in range(0, m, 8)])
  y = _run(gpu, t, w, x, n, k)
  assert y.shape == (m, n) and ol.rel_err(y, ref) <= TOL
  np.testing.assert_array_equal(_run(gpu, t, w, x.astype(np.float32), n, k), y)
  layer = QuantLinear(gpu.Buffer.from_numpy(w), t, n, k)
  res = rng.standard_normal((m, n)).astype(np.float32)
  rb = gpu.Buffer.from_numpy(res)
  qlinear_multi([layer], gpu.Buffer.from_numpy(x), [rb], epilogue=1, resid=[rb])
  assert ol.rel_err(rb.numpy(), res + ref) <= TOL

@pytest.mark.parametrize("t", [12, 13, 3, 6, 7], ids=["q4_k", "q5_k", "q4_1", "q5_0", "q5_1"])
@pytest.mark.parametrize("n,k,m", [(16, 2048, 3), (4096 + 48, 4096, 8), (1024, 4096, 16), (4112, 2048, 5), (272, 4096, 11), (1040, 14336, 8), (64, 5120, 13), (2048, 8192, 2), (512, 4096, 2)])
def test_small_batch_q4_k_q5_k_through_lds(gpu, t, n, k, m):
  """Q4_K / Q5_K on the kernel that streams the weights into LDS: a slot is eight superblocks of 144 / 176 bytes per row (K = 2048 or 4096), four with
  the activations streamed beside the weights (K beyond 4096, one matrix); a wave's step is one superblock per row.  Q4_1 / Q5_0 / Q5_1: slots of sixteen
  block pairs of 40 / 44 / 48 bytes.  Plain, with the residual, as the
  SwiGLU pair and as three matrices of one launch; fp16 and float32 activations; against the C restatement run in blocks of eight rows and the float64 anchor."""
  from tinygrad_amd.nn import QuantLinear, qlinear_multi
  rng = np.random.default_rng(5 * n + k + m + t)
  w = synth.random_blocks(rng, t, n, k)
  x = synth.activations(rng, m, k, np.float16)
  ref = np.concatenate([cref.linear(t, w, x[i:i + 8], n, k, threads=8) for i in range(0, m, 8)])
  y = _run(gpu, t, w, x, n, k)
  assert y.shape == (m, n) and ol.rel_err(y, ref) <= TOL
  rows = min(n, 64)
  nel, nby = GGML_QUANT[t]
  W = ol.weight_f32(w[:rows * (k // nel) * nby], rows, k, t)
  assert ol.rel_err(y[:, :rows], ol.linear_f64(x.astype(np.float32), W)) <= TOL
  np.testing.assert_array_equal(_run(gpu, t, w, x.astype(np.float32), n, k), y)
  layer = QuantLinear(gpu.Buffer.from_numpy(w), t, n, k)
  xb = gpu.Buffer.from_numpy(x)
  res = rng.standard_normal((m, n)).astype(np.float32)
  rb = gpu.Buffer.from_numpy(res)
  qlinear_multi([layer], xb, [rb], epilogue=1, resid=[rb])
  assert ol.rel_err(rb.numpy(), res + ref) <= TOL
  if k <= 4096:
    n2 = max(16, n // 4 // 16 * 16)
    w2 = synth.random_blocks(rng, t, n2, k)
    ref2 = np.concatenate([cref.linear(t, w2, x[i:i + 8], n2, k, threads=8) for i in range(0, m, 8)])
    l2 = QuantLinear(gpu.Buffer.from_numpy(w2), t, n2, k)
    outs = [gpu.Buffer((m, n), np.float32), gpu.Buffer((m, n2), np.float32), gpu.Buffer((m, n2), np.float16)]
    for o in outs: gpu.check(gpu.lib().tga_memset(o.ptr, 0xFF, o.nbytes, None))
    qlinear_multi([layer, l2], xb, outs[:2])
    np.testing.assert_array_equal(outs[0].numpy(), y)
    assert ol.rel_err(outs[1].numpy(), ref2) <= TOL
    r1 = ref2[:, :n2]; g = ref[:, :n2].astype(np.float64)
    lg = QuantLinear(gpu.Buffer.from_numpy(w[:n2 * (k // nel) * nby].copy()), t, n2, k)
    qlinear_multi([lg, l2], xb, [outs[2]], epilogue=2)
    assert ol.rel_err(outs[2].numpy().astype(np.float32), g / (1 + np.exp(-g)) * r1) <= 2 * TOL

@pytest.mark.parametrize("n,k,m", [(16, 2048, 3), (4096 + 48, 4096, 8), (1024, 4096, 16), (4112, 2048, 5), (272, 4096, 11)])
def test_small_batch_q6_k_through_lds(gpu, n, k, m):
  """Q6_K on the kernel that streams the weights into LDS (one matrix, K = 2048 or 4096, rows a multiple of 16): a slot is eight superblocks of 210
  bytes per row, a wave's step one superblock read at 2-byte alignment.  Plain and with the residual, fp16 and float32 activations, against the C
  restatement run in blocks of eight rows and, for the first rows, the float64 anchor."""
  from tinygrad_amd.nn import QuantLinear, qlinear_multi
  t = 14
  rng = np.random.default_rng(6 * n + k + m)
  w = synth.random_blocks(rng, t, n, k)
  x = synth.activations(rng, m, k, np.float16)
  ref = np.concatenate([cref.linear(t, w, x[i:i + 8], n, k, threads=8) for i in range(0, m, 8)])
  y = _run(gpu, t, w, x, n, k)
  assert y.shape == (m, n) and ol.rel_err(y, ref) <= TOL
  rows = min(n, 64)
  nel, nby = GGML_QUANT[t]
  W = ol.weight_f32(w[:rows * (k // nel) * nby], rows, k, t)
  assert ol.rel_err(y[:, :rows], ol.linear_f64(x.astype(np.float32), W)) <= TOL
  np.testing.assert_array_equal(_run(gpu, t, w, x.astype(np.float32), n, k), y)
  layer = QuantLinear(gpu.Buffer.from_numpy(w), t, n, k)
  res = rng.standard_normal((m, n)).astype(np.float32)
  rb = gpu.Buffer.from_numpy(res)
  qlinear_multi([layer], gpu.Buffer.from_numpy(x), [rb], epilogue=1, resid=[rb])
  assert ol.rel_err(rb.numpy(), res + ref) <= TOL

@pytest.mark.parametrize("t,k,ns,m,epi", [(2, 4096, [512, 128, 128], 16, 0), (2, 2048, [256, 64, 64], 5, 0), (8, 4096, [1024, 1024], 8, 2), (2, 4096, [448, 448], 3, 2),
                                            (14, 4096, [272], 4, 0), (2, 4096, [512, 128, 128], 2, 0), (8, 4096, [256, 256], 2, 2), (12, 4096, [256, 64, 64], 6, 0), (13, 2048, [264, 264], 7, 2),
                                            (3, 4096, [256, 64, 64], 6, 0), (8, 1024, [64], 16, 0), (39, 4096, [256, 64, 64], 6, 0), (2, 8192, [128], 8, 0), (2, 4096, [200], 2, 0)])
def test_norm_folded_into_the_small_batch_kernel(gpu, t, k, ns, m, epi):
  """tga_rmsnorm_qlinear_rows (the RMSNorm in front of q/k/v or gate/up folded into the LDS-fed small-batch kernel's prologue) against tga_rmsnorm_rows
  followed by tga_qlinear_multi, and against the float64 anchor of the normalised fp16 rows.  The last cases are outside the kernel that folds the norm
  (more than eight rows, MXFP4, K beyond 4096, ragged row counts): there the call IS the two launches, bit for bit."""
  from tinygrad_amd.nn import QuantLinear, qlinear_multi
  L = gpu.lib()
  rng = np.random.default_rng(sum(ns) + k + m + t)
  ws = [synth.random_blocks(rng, t, n, k) for n in ns]
  layers = [QuantLinear(gpu.Buffer.from_numpy(w), t, n, k) for w, n in zip(ws, ns)]
  x = (rng.standard_normal((m, k)) * np.exp(rng.standard_normal((m, 1)))).astype(np.float32)       # rows of different magnitudes
  nw = (1 + 0.2 * rng.standard_normal(k)).astype(np.float32)
  xb, nb = gpu.Buffer.from_numpy(x), gpu.Buffer.from_numpy(nw)
  nout = 1 if epi == 2 else len(ns)
  xn0 = gpu.Buffer((m, k), np.float16)
  gpu.check(L.tga_rmsnorm_rows(xb.ptr, nb.ptr, m, k, 1e-5, xn0.ptr, None, 0, None))
  o0 = [gpu.Buffer((m, ns[i]), np.float32) for i in range(nout)]
  qlinear_multi(layers, xn0, o0, epilogue=epi)
  o1 = [gpu.Buffer((m, ns[i]), np.float32) for i in range(nout)]
  for o in o1: gpu.check(L.tga_memset(o.ptr, 0xFF, o.nbytes, None))
  scratch = gpu.Buffer((m, k), np.float16)
  gpu.check(L.tga_memset(scratch.ptr, 0xFF, scratch.nbytes, None))
  qlinear_multi(layers, xb, o1, epilogue=epi, norm=(nb, 1e-5, scratch))
  folded = t in (2, 8, 12, 13, 14, 3, 6, 7) and k <= 4096 and 2 <= m <= 8 and all(n % (8 if epi == 2 else 16) == 0 for n in ns)
  assert (scratch.numpy().view(np.uint16) == 0xFFFF).all() == folded       # one launch: the scratch rows were not needed
  h = xn0.numpy().astype(np.float32)
  refs = [ol.linear_f64(h, ol.weight_f32(w, n, k, t)) for w, n in zip(ws, ns)]
  if epi == 2: refs = [refs[0] / (1 + np.exp(-refs[0])) * refs[1]]
  for a, b, ref in zip(o1, o0, refs):
    if folded: assert ol.rel_err(a.numpy(), b.numpy()) <= 2e-4 and ol.rel_err(a.numpy(), ref) <= TOL      # the sum of squares is associated differently: an fp16 value may round the other way
    else: np.testing.assert_array_equal(a.numpy(), b.numpy())

@pytest.mark.parametrize("types,k,ns", [((12, 12, 14), 4096, [4096, 1024, 1024]), ((13, 13, 14), 2560, [512, 128, 128]), ((12, 12, 14), 2304, [48, 9, 7]), ((12, 14), 4096, [6000, 200]),
                                        ((2, 2, 8), 4096, [256, 64, 64]), ((12, 14, 12), 4096, [256, 64, 64]), ((12, 12, 14), 8192, [128, 64, 64]), ((14, 14, 14), 4096, [256, 64, 64]),
                                        ((12, 12, 14), 2048, [128, 64, 64])])
def test_norm_and_linears_of_mixed_block_types(gpu, types, k, ns):
  """tga_rmsnorm_qlinear_mixed (Q4_K / Q5_K attn_q, attn_k and a Q6_K attn_v of one block in ONE launch of the single-row kernel: the first workgroups walk the first
  set, the others the second) against tga_rmsnorm_qlinear_multi per run of equal types (to float32 rounding of the sums: 2e-6 of the largest output), and against the float64 anchor of the normalised fp16 row.
  The later cases are outside the shared launch (other type pairs, three runs, K beyond 4096 or rows of at most 32 units, a single run): there the call IS one launch per run."""
  from tinygrad_amd.nn import QuantLinear, qlinear_multi, qlinear_mixed
  rng = np.random.default_rng(sum(ns) + k + sum(types))
  ws = [synth.random_blocks(rng, t, n, k) for t, n in zip(types, ns)]
  layers = [QuantLinear(gpu.Buffer.from_numpy(w), t, n, k) for w, t, n in zip(ws, types, ns)]
  x = (rng.standard_normal((1, k)) * 3).astype(np.float32)
  nw = (1 + 0.2 * rng.standard_normal(k)).astype(np.float32)
  xb, nb = gpu.Buffer.from_numpy(x), gpu.Buffer.from_numpy(nw)
  o0 = [gpu.Buffer((1, n), np.float32) for n in ns]
  i = 0
  while i < len(ns):
    j = i + 1
    while j < len(ns) and types[j] == types[i]: j += 1
    qlinear_multi(layers[i:j], xb, o0[i:j], norm=(nb, 1e-5))
    i = j
  for ydt in (np.float32, np.float16):
    o1 = [gpu.Buffer((1, n), ydt) for n in ns]
    for o in o1: gpu.check(gpu.lib().tga_memset(o.ptr, 0xFF, o.nbytes, None))
    qlinear_mixed(layers, xb, o1, norm=(nb, 1e-5))
    shared = len(set(types)) == 2 and types[-1] == 14 and types[0] in (12, 13) and list(types) == sorted(types) and 2048 < k <= 4096
    for a, b in zip(o1, o0):
      if not shared: assert a.numpy().tobytes() == b.numpy().astype(ydt).tobytes()
      else:                                                          # another build of the same walk: the compiler contracts the float32 sums differently
        e = ol.rel_err(a.numpy().astype(np.float32), b.numpy())
        assert e <= (2e-6 if ydt == np.float32 else 1e-3), (e, ydt)
  xn = gpu.Buffer((1, k), np.float16)
  gpu.check(gpu.lib().tga_rmsnorm(xb.ptr, nb.ptr, k, 1e-5, xn.ptr, None, 0, None))
  h = xn.numpy().astype(np.float32)
  for o, o16, w, t, n in zip(o0, o1, ws, types, ns):
    ref = ol.linear_f64(h, ol.weight_f32(w, n, k, t))
    assert ol.rel_err(o.numpy(), ref) <= TOL and ol.rel_err(o16.numpy().astype(np.float32), ref) <= 2 * TOL

@pytest.mark.parametrize("m", [16, 17, 37, 64, 65, 100, 128])
def test_sixteen_and_more_rows_segments_residual_and_swiglu(gpu, m):
  """q / k / v in one launch, the residual epilogue in place and silu(gate) * up at sixteen rows (on the LDS-fed kernel's range and outside it) and at
  17 .. 128 rows (the prefill kernel; segments that are no multiple of sixteen rows go through blocks of sixteen)."""
  from tinygrad_amd.nn import QuantLinear, qlinear_multi
  rng = np.random.default_rng(1616 + m)
  for t, k, ns in ((2, 2048, [2048, 512, 512]), (8, 1024, [512, 128, 130]), (14, 1024, [64, 32, 32]), (12, 2048, [272, 48, 48]), (13, 1024, [100, 100]), (23, 1024, [80, 16, 16])):
    if len(ns) == 2: ns = [ns[0], ns[1], ns[1]]
    ws = [synth.random_blocks(rng, t, n, k) for n in ns]
    x = synth.activations(rng, m, k, np.float16)
    layers = [QuantLinear(gpu.Buffer.from_numpy(w), t, n, k) for w, n in zip(ws, ns)]
    outs = [gpu.Buffer((m, n), np.float32) for n in ns]
    for o in outs: gpu.check(gpu.lib().tga_memset(o.ptr, 0xFF, o.nbytes, None))
    xb = gpu.Buffer.from_numpy(x)
    qlinear_multi(layers, xb, outs)
    refs = [ol.linear_f64(x.astype(np.float32), ol.weight_f32(w, n, k, t)) for w, n in zip(ws, ns)]
    for o, r in zip(outs, refs): assert ol.rel_err(o.numpy(), r) <= TOL, (t, k)
    res = [rng.standard_normal((m, n)).astype(np.float32) for n in ns]
    rb = [gpu.Buffer.from_numpy(r) for r in res]
    qlinear_multi(layers, xb, rb, epilogue=1, resid=rb)
    for o, r0, r in zip(rb, res, refs): assert ol.rel_err(o.numpy(), r0 + r) <= TOL, (t, k)
    g = [layers[1], QuantLinear(gpu.Buffer.from_numpy(synth.random_blocks(rng, t, ns[1], k)), t, ns[1], k)]
    out = gpu.Buffer((m, ns[1]), np.float32)                              # (float32: products of random Q6_K rows leave the fp16 range)
    qlinear_multi(g, xb, [out], epilogue=2)
    a, b = refs[1], ol.linear_f64(x.astype(np.float32), ol.weight_f32(g[1].blocks.numpy(), ns[1], k, t))
    assert ol.rel_err(out.numpy(), a / (1 + np.exp(-a)) * b) <= TOL, (t, k)

@pytest.mark.parametrize("t,k,m,f32", [(8, 4096, 2, False), (8, 4096, 3, True), (8, 2048, 5, False), (8, 4096, 8, True), (8, 2048, 9, True), (8, 4096, 13, False), (8, 4096, 16, True), (8, 2048, 16, False),
                                       (1, 2048, 2, False), (1, 2048, 4, True), (1, 2048, 8, False), (1, 2048, 11, True), (1, 2048, 16, False),
                                       (2, 4096, 8, False), (2, 2048, 16, True), (12, 4096, 6, True), (12, 2048, 16, False), (13, 4096, 8, False), (13, 2048, 3, True),
                                       (3, 4096, 5, False), (6, 2048, 8, True), (7, 4096, 16, False)])
def test_small_batch_on_wave_private_rings(gpu, t, k, m, f32):
  """The small-batch kernel whose waves stream their own slices of K (qgemm_wp.hip: block pairs and Q4_K / Q5_K at K = 2048 / 4096, fp16 weights at K = 2048, 2 .. 16
  rows): q / k / v in one launch, the residual epilogue in place, silu(gate) * up (not for fp16 weights), and a matrix of 14336 rows (three or four row groups per workgroup, so the rings wrap and both
  tile sets are reused), fp16 and float32 activations, against the float64 anchor; twice, to see that a launch leaves nothing behind that the next one reads."""
  from tinygrad_amd.nn import QuantLinear, qlinear_multi
  rng = np.random.default_rng(88 + k + m)
  ns = [1024, 256, 256]
  mkw = lambda n: synth.random_blocks(rng, t, n, k) if t != 1 else (rng.standard_normal((n, k)) * 0.02).astype(np.float16).view(np.uint8).reshape(-1)
  wf32 = lambda w, n: ol.weight_f32(w, n, k, t) if t != 1 else w.view(np.float16).reshape(n, k).astype(np.float32)
  ws = [mkw(n) for n in ns]
  x = synth.activations(rng, m, k, np.float32 if f32 else np.float16)
  xf = x.astype(np.float32) if f32 else x.astype(np.float32)
  h = xf.astype(np.float16).astype(np.float32)                          # the kernel rounds float32 rows to fp16 operands
  layers = [QuantLinear(gpu.Buffer.from_numpy(w), t, n, k) for w, n in zip(ws, ns)]
  xb = gpu.Buffer.from_numpy(x)
  refs = [ol.linear_f64(h, wf32(w, n)) for w, n in zip(ws, ns)]
  for rep in range(2):
    outs = [gpu.Buffer((m, n), np.float32) for n in ns]
    for o in outs: gpu.check(gpu.lib().tga_memset(o.ptr, 0xFF, o.nbytes, None))
    qlinear_multi(layers, xb, outs)
    for o, r in zip(outs, refs): assert ol.rel_err(o.numpy(), r) <= TOL, (k, m, rep)
    res = [rng.standard_normal((m, n)).astype(np.float32) for n in ns]
    rb = [gpu.Buffer.from_numpy(r) for r in res]
    qlinear_multi(layers[:1], xb, rb[:1], epilogue=1, resid=rb[:1])
    assert ol.rel_err(rb[0].numpy(), res[0] + refs[0]) <= TOL, (k, m, rep)
    if t == 1: continue                                                 # (fp16 weights: no SwiGLU pair on this kernel)
    g = [layers[1], layers[2]]
    out = gpu.Buffer((m, ns[1]), np.float32)
    qlinear_multi(g, xb, [out], epilogue=2)
    assert ol.rel_err(out.numpy(), refs[1] / (1 + np.exp(-refs[1])) * refs[2]) <= TOL, (k, m, rep)
    out16 = gpu.Buffer((m, ns[1]), np.float16)
    qlinear_multi(g, xb, [out16], epilogue=2)
    assert ol.rel_err(out16.numpy().astype(np.float32), refs[1] / (1 + np.exp(-refs[1])) * refs[2]) <= 2 * TOL, (k, m, rep)
  if (t, k) in ((8, 4096), (1, 2048), (2, 4096), (13, 4096)) and m in (8, 16):
    n = 14336
    w = mkw(n)
    lin = QuantLinear(gpu.Buffer.from_numpy(w), t, n, k)
    ref = ol.linear_f64(h, wf32(w, n))
    for rep in range(2):
      o = gpu.Buffer((m, n), np.float16)
      gpu.check(gpu.lib().tga_memset(o.ptr, 0xFF, o.nbytes, None))
      lin(xb, out=o)
      assert ol.rel_err(o.numpy().astype(np.float32), ref) <= TOL, (m, rep)

def test_small_batch_through_lds_segments_and_residual(gpu):
  """q / k / v of a llama block shape in one launch at M = 4 and the residual epilogue in place, on the LDS-fed kernel's range."""
  from tinygrad_amd.nn import QuantLinear, qlinear_multi
  rng = np.random.default_rng(4242)
  k, m = 2048, 4
  ns = [2048, 512, 512]
  for t in (2, 8):
    ws = [synth.random_blocks(rng, t, n, k) for n in ns]
    x = synth.activations(rng, m, k, np.float16)
    layers = [QuantLinear(gpu.Buffer.from_numpy(w), t, n, k) for w, n in zip(ws, ns)]
    outs = [gpu.Buffer((m, n), np.float32) for n in ns]
    for o in outs: gpu.check(gpu.lib().tga_memset(o.ptr, 0xFF, o.nbytes, None))
    xb = gpu.Buffer.from_numpy(x)
    qlinear_multi(layers, xb, outs)
    refs = [ol.linear_f64(x.astype(np.float32), ol.weight_f32(w, n, k, t)) for w, n in zip(ws, ns)]
    for o, r in zip(outs, refs): assert ol.rel_err(o.numpy(), r) <= TOL
    res = [rng.standard_normal((m, n)).astype(np.float32) for n in ns]
    rb = [gpu.Buffer.from_numpy(r) for r in res]
    qlinear_multi(layers, xb, rb, epilogue=1, resid=rb)
    for o, r0, r in zip(rb, res, refs): assert ol.rel_err(o.numpy(), r0 + r) <= TOL

def test_argument_errors(gpu):
  from tinygrad_amd.nn import QuantLinear
  w = gpu.Buffer.from_numpy(np.zeros(18 * 4, dtype=np.uint8))
  with pytest.raises(ValueError): QuantLinear(w, 1337, 4, 32)
  lin = QuantLinear(w, 2, 4, 32)
  with pytest.raises(AssertionError): lin(gpu.Buffer((129, 32), np.float16))
  with pytest.raises(RuntimeError, match="out of range 1..128"): gpu.check(gpu.lib().tga_qlinear(2, w.ptr, w.ptr, 0, w.ptr, 0, 129, 4, 32, None))
  with pytest.raises(RuntimeError): gpu.check(gpu.lib().tga_qlinear(2, w.ptr, w.ptr, 0, w.ptr, 0, 1, 4, 33, None))
  # Q4_1 / Q5_0 / Q5_1 rows are read as block pairs: an odd number of blocks per row is refused
  with pytest.raises(RuntimeError, match="multiple of 64"): gpu.check(gpu.lib().tga_qlinear(3, w.ptr, w.ptr, 1, w.ptr, 0, 1, 1, 96, None))
  # the entry points of the batched steps refuse what they cannot launch
  L, f = gpu.lib(), gpu.Buffer((64,), np.float32).zero_()
  with pytest.raises(RuntimeError, match="null pointer"): gpu.check(L.tga_rmsnorm_qlinear_rows(f.ptr, 1e-5, 2, 1, None, None, None, f.ptr, None, 1, 4, 32, 0, None, None))
  with pytest.raises(RuntimeError, match="1..128"): gpu.check(L.tga_rmsnorm_qlinear_rows(f.ptr, 1e-5, 2, 1, None, None, None, f.ptr, f.ptr, 1, 129, 32, 0, None, None))
  with pytest.raises(RuntimeError, match="multiple of 8"): gpu.check(L.tga_moe_router_rows(f.ptr, f.ptr, 1e-5, f.ptr, 2, 20, 4, f.ptr, f.ptr, None))
  with pytest.raises(RuntimeError, match="rows=0"): gpu.check(L.tga_moe_combine_rmsnorm_rows(f.ptr, f.ptr, f.ptr, f.ptr, 0, 2, 16, 1e-5, f.ptr, None, None))
  with pytest.raises(RuntimeError, match="exceed one launch"):
    gpu.check(L.tga_qlinear_experts_routed_rows(2, w.ptr, w.ptr, 8, f.ptr, 40000, 2, 1, 0, 1.0, f.ptr, f.ptr, f.ptr, f.ptr, 1, 4, 64, None))

@pytest.mark.parametrize("t,k", [(2, 4096), (2, 14336), (8, 4096), (14, 4096), (39, 2048), (1, 2048), (12, 4096), (13, 2048), (3, 2048), (6, 4096), (7, 1024), (23, 4096), (23, 14336), (18, 4096), (21, 2048), (22, 14336), (41, 2048)])
def test_staged_activations_equal_plain_path(gpu, t, k):
  """tga_stage_activation + TGA_F16_STAGED gives the plain path's result (same products; only the order the per-block offset
  correction is summed in differs), and a SwiGLU output staged for a consumer feeds that consumer correctly."""
  from tinygrad_amd.nn import QuantLinear, qlinear_multi, stage_activation
  rng = np.random.default_rng(k + t)
  n = 384
  w = synth.random_blocks(rng, t, n, k) if t != 1 else (rng.standard_normal((n, k)) * 0.02).astype(np.float16).view(np.uint8).reshape(-1)
  lin = QuantLinear(gpu.Buffer.from_numpy(w), t, n, k)
  x = synth.activations(rng, 1, k, np.float16)
  xb = gpu.Buffer.from_numpy(x)
  plain = lin(xb, out_dtype=np.float32).numpy()
  xs = stage_activation(lin, xb)
  assert sorted(xs.numpy().reshape(-1).view(np.uint16).tolist()) == sorted(x.reshape(-1).view(np.uint16).tolist())   # a permutation of the row
  out = gpu.Buffer((1, n), np.float32)
  qlinear_multi([lin], xs, [out], x_staged=True)
  assert ol.rel_err(out.numpy(), plain) <= 1e-5
  # fp32 input staged (rounded to fp16 on the way)
  xs32 = stage_activation(lin, gpu.Buffer.from_numpy(x.astype(np.float32)))
  assert xs32.numpy().tobytes() == xs.numpy().tobytes()

def test_swiglu_output_staged_for_the_down_projection(gpu):
  from tinygrad_amd.nn import QuantLinear, qlinear_multi
  rng = np.random.default_rng(8)
  d, hdim = 512, 1024
  g, u, dn = (QuantLinear(gpu.Buffer.from_numpy(synth.random_blocks(rng, 2, r, c)), 2, r, c) for r, c in ((hdim, d), (hdim, d), (d, hdim)))
  x = gpu.Buffer.from_numpy(synth.activations(rng, 1, d, np.float16))
  act_n, act_s = gpu.Buffer((1, hdim), np.float16), gpu.Buffer((1, hdim), np.float16)
  y_n, y_s = gpu.Buffer((1, d), np.float32), gpu.Buffer((1, d), np.float32)
  qlinear_multi([g, u], x, [act_n], epilogue=2)
  qlinear_multi([dn], act_n, [y_n])
  qlinear_multi([g, u], x, [act_s], epilogue=2, stage_out_for=dn)
  qlinear_multi([dn], act_s, [y_s], x_staged=True)
  assert ol.rel_err(y_s.numpy(), y_n.numpy()) <= 1e-5

@pytest.mark.parametrize("t,k", [(2, 2048), (8, 512), (14, 1024), (39, 2048), (1, 2048), (2, 8192), (12, 4096), (13, 1024), (3, 1024), (6, 2048), (7, 4096), (23, 4096), (18, 4096), (21, 1024), (22, 2048), (41, 4096)],
                         ids=["q4_0", "q8_0", "q6_k", "mxfp4", "f16", "q4_0-k8192", "q4_k", "q5_k", "q4_1", "q5_0", "q5_1", "iq4_xs", "iq3_xxs", "iq3_s", "iq2_s", "q1_0"])
def test_rmsnorm_folded_into_the_linear(gpu, t, k):
  """tga_rmsnorm_qlinear_multi against tga_rmsnorm followed by tga_qlinear_multi (same fp16 activation up to the summation order of
  the mean square) and against the float64 anchor on the fp16-rounded normalised row."""
  from tinygrad_amd.nn import QuantLinear, qlinear_multi
  from tinygrad_amd import runtime as rt
  from oracle import llm as ollm
  rng = np.random.default_rng(t * 1000 + k)
  ns = [192, 64]
  if t == 1: ws = [rng.standard_normal((n, k)).astype(np.float16).view(np.uint8).reshape(-1) * 1 for n in ns]
  else: ws = [synth.random_blocks(rng, t, n, k) for n in ns]
  layers = [QuantLinear(gpu.Buffer.from_numpy(w), t, n, k) for w, n in zip(ws, ns)]
  x = (rng.standard_normal((1, k)) * 3).astype(np.float32); nw = rng.standard_normal(k).astype(np.float32)
  xb, nwb = gpu.Buffer.from_numpy(x), gpu.Buffer.from_numpy(nw)
  fused = [gpu.Buffer((1, n), np.float32) for n in ns]
  qlinear_multi(layers, xb, fused, norm=(nwb, 1e-5))
  xn = gpu.Buffer((1, k), np.float16)
  gpu.check(gpu.lib().tga_rmsnorm(xb.ptr, nwb.ptr, k, 1e-5, xn.ptr, None, 0, None))
  plain = [gpu.Buffer((1, n), np.float32) for n in ns]
  qlinear_multi(layers, xn, plain)
  h = ollm.rmsnorm(x[0], nw, 1e-5).astype(np.float16).astype(np.float32)[None]
  for f, p, w, n in zip(fused, plain, ws, ns):
    W = w.view(np.float16).astype(np.float32).reshape(n, k) if t == 1 else ol.weight_f32(w, n, k, t)
    assert ol.rel_err(f.numpy(), p.numpy()) <= 2e-4
    assert ol.rel_err(f.numpy(), ol.linear_f64(h, W)) <= TOL
  # SwiGLU epilogue with the folded norm (ffn_norm -> ffn_gate / ffn_up)
  pair = [QuantLinear(layers[1].blocks, t, 64, k), QuantLinear(gpu.Buffer.from_numpy(ws[0][: len(ws[0]) // 3]), t, 64, k)]
  o1, o2 = gpu.Buffer((1, 64), np.float32), gpu.Buffer((1, 64), np.float32)
  qlinear_multi(pair, xb, [o1], epilogue=2, norm=(nwb, 1e-5))
  qlinear_multi(pair, xn, [o2], epilogue=2)
  assert ol.rel_err(o1.numpy(), o2.numpy()) <= 1e-3
  # outside the fast path the call is refused with a message
  bad = QuantLinear(gpu.Buffer.from_numpy(synth.random_blocks(rng, 2, 8, 96)), 2, 8, 96)
  with pytest.raises(RuntimeError, match="fast path"):
    qlinear_multi([bad], gpu.Buffer.from_numpy(x[:, :96].copy()), [gpu.Buffer((1, 8), np.float32)], norm=(nwb, 1e-5))


@pytest.mark.parametrize("case", ["interleaved_ragged", "interleaved_residual", "swiglu_pair", "split_k_skewed", "fewer_groups_than_teams"])
def test_row_team_schedules_write_every_row(gpu, case):
  """The M = 1 launches hand row groups to their wave teams in three ways on a 256-CU part: interleaved (team t owns groups t, t + teams, ...),
  contiguous with the first pass of workgroups owning one group more than the second (two workgroups per CU), and contiguous and equal.
  Row counts here leave remainders everywhere (teams with unequal counts, a last group of one row); outputs start as NaN so that a row
  nobody wrote, or wrote twice with different values, shows."""
  from tinygrad_amd.nn import QuantLinear, qlinear_multi
  rng = np.random.default_rng(4242)
  t = 2
  n, k = {"interleaved_ragged": (13843, 4096), "interleaved_residual": (13843, 4096), "swiglu_pair": (7001, 4096),
          "split_k_skewed": (4603, 14336), "fewer_groups_than_teams": (100, 4096)}[case]
  x = synth.activations(rng, 1, k, np.float16)
  xb = gpu.Buffer.from_numpy(x)
  w = synth.random_blocks(rng, t, n, k)
  lin = QuantLinear(gpu.Buffer.from_numpy(w), t, n, k)
  ref = ol.linear_f64(x.astype(np.float32), ol.weight_f32(w, n, k, t))
  nan = np.full((1, n), np.nan, np.float32)
  if case in ("interleaved_ragged", "fewer_groups_than_teams"):
    out = gpu.Buffer.from_numpy(nan)
    qlinear_multi([lin], xb, [out])
    y = out.numpy()
  elif case in ("interleaved_residual", "split_k_skewed"):
    res = rng.standard_normal((1, n)).astype(np.float32)
    out = gpu.Buffer.from_numpy(res)
    qlinear_multi([lin], xb, [out], epilogue=1, resid=[out])
    y = out.numpy(); ref = ref + res
  else:
    w2 = synth.random_blocks(rng, t, n, k)
    lin2 = QuantLinear(gpu.Buffer.from_numpy(w2), t, n, k)
    out = gpu.Buffer.from_numpy(nan)
    qlinear_multi([lin, lin2], xb, [out], epilogue=2)
    y = out.numpy()
    up = ol.linear_f64(x.astype(np.float32), ol.weight_f32(w2, n, k, t))
    ref = ref / (1 + np.exp(-ref)) * up
  assert np.isfinite(y).all(), f"{np.count_nonzero(~np.isfinite(y))} rows not written"
  assert ol.rel_err(y, ref) <= TOL
  atol = TOL * float(np.sqrt(np.mean(ref ** 2)))
  assert np.isclose(y, ref, rtol=TOL, atol=atol).all()
