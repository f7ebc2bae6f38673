"""MXFP8 MoE prefill path on the GPU vs the oracle: quantize_mxfp8 bit-exact, route/dispatch/combine exact (integer / byte work),
grouped GEMM within the reference's own error bars (test/backend/test_asm_gemm.py:310-313: mean-rel-err < 1e-2 vs dequant-matmul)."""
import numpy as np, pytest
from oracle import mxfp8 as omx, moe as omoe

pytestmark = pytest.mark.gpu

def test_quantize_mxfp8_bit_exact(gpu):
  from tinygrad_amd import moe
  rng = np.random.default_rng(1)
  x = (rng.standard_normal((300, 512)) * np.exp2(rng.integers(-20, 12, size=(300, 1)))).astype(np.float32)
  x[0, :32] = 0; x[1, :64] = 2.0 ** -3; x[2, 5] = 448.0; x[3, :32] = 1e-30
  q, e8, packed = moe.quantize_mxfp8(gpu.Buffer.from_numpy(x))
  rq, re8 = omx.quantize_mxfp8(x)
  np.testing.assert_array_equal(e8.numpy(), re8)
  np.testing.assert_array_equal(q.numpy(), rq)
  np.testing.assert_array_equal(packed.numpy(), omx.mx_pack(re8))
  # bf16 input
  xb = moe.to_bf16_bits(x)
  q2, e82, _ = moe.quantize_mxfp8(gpu.Buffer.from_numpy(xb))
  rq2, re82 = omx.quantize_mxfp8(moe.from_bf16_bits(xb))
  np.testing.assert_array_equal(e82.numpy(), re82); np.testing.assert_array_equal(q2.numpy(), rq2)

@pytest.mark.parametrize("M,N", [(256, 512), (96, 64), (384, 320)])
def test_transpose_quantize_mxfp8_bit_exact(gpu, M, N):
  """transpose_quantize_mxfp8(g) == quantize_mxfp8(g.T) (extra/llama_kernels/transpose_quantize_mxfp8/__init__.py:24-25): bit-exact against the
  oracle and against this library's own row-wise quantizer fed the transposed matrix; M = 96 has a partial 128-row tile and no packed scales."""
  from tinygrad_amd import moe
  rng = np.random.default_rng(M + N)
  g = (rng.standard_normal((M, N)) * np.exp2(rng.integers(-20, 12, size=(1, N)))).astype(np.float32)
  g[:32, 0] = 0; g[32:64, 1] = 2.0 ** -3; g[5, 2] = 448.0; g[:32, 3] = 1e-30
  gb = moe.to_bf16_bits(g)
  q, e8, si = moe.transpose_quantize_mxfp8(gpu.Buffer.from_numpy(gb))
  rq, re8, rsi = omx.transpose_quantize_mxfp8(moe.from_bf16_bits(gb))
  assert q.shape == (N, M) and e8.shape == (N, M // 32)
  np.testing.assert_array_equal(e8.numpy(), re8); np.testing.assert_array_equal(q.numpy(), rq)
  if M % 128 == 0: np.testing.assert_array_equal(si.numpy(), rsi)
  else: assert si is None and rsi is None
  q2, e82, si2 = moe.quantize_mxfp8(gpu.Buffer.from_numpy(np.ascontiguousarray(gb.T)))
  np.testing.assert_array_equal(q2.numpy(), q.numpy()); np.testing.assert_array_equal(e82.numpy(), e8.numpy())
  if M % 128 == 0: np.testing.assert_array_equal(si2.numpy(), si.numpy())

def test_fused_silu_mul_quantize_mxfp8(gpu):
  """silu(x_w1) * x_w3 quantized without an intermediate tensor (extra/llama_kernels/fused_silu_mul_quantize_mxfp8).  The product is
  formed in float32 from exp2; where the device's exp2 differs from numpy's in the last ulp an E4M3 code may land on the other side of
  a rounding boundary, so the bar is: block exponents equal, codes equal except for a < 1e-4 fraction, and those within one code."""
  from tinygrad_amd import moe
  rng = np.random.default_rng(4)
  w1 = (rng.standard_normal((256, 768)) * 3).astype(np.float32); w3 = rng.standard_normal((256, 768)).astype(np.float32)
  w1[0, :32] = 0; w1[1, :32] = -40.0; w1[2, :32] = 30.0
  b1, b3 = moe.to_bf16_bits(w1), moe.to_bf16_bits(w3)
  q, e8, packed = moe.fused_silu_mul_quantize_mxfp8(gpu.Buffer.from_numpy(b1), gpu.Buffer.from_numpy(b3))
  rq, re8 = omx.silu_mul_quantize_mxfp8(moe.from_bf16_bits(b1), moe.from_bf16_bits(b3))
  ge8, gq = e8.numpy(), q.numpy()
  assert np.mean(ge8 != re8) < 1e-4 and np.abs(ge8.astype(int) - re8.astype(int)).max() <= 1
  same_block = np.repeat(ge8 == re8, 32, axis=-1)
  diff = (gq != rq) & same_block
  assert diff.mean() < 1e-4
  mag = lambda c: (c & 0x7F).astype(int)
  assert (np.abs(mag(gq[diff]) - mag(rq[diff])) <= 1).all()
  np.testing.assert_array_equal(packed.numpy(), omx.mx_pack(ge8))
  # against the unfused chain on the GPU itself (float32 product quantized by tga_quantize_mxfp8): same bar
  act = moe.from_bf16_bits(b1); act = (act * (1.0 / (1.0 + np.exp2(act * np.float32(-1.4426950408889634)))) * moe.from_bf16_bits(b3)).astype(np.float32)
  q2, e82, _ = moe.quantize_mxfp8(gpu.Buffer.from_numpy(act))
  assert np.mean(q2.numpy() != gq) < 1e-4

@pytest.mark.parametrize("T,E,k", [(300, 16, 4), (4096, 128, 8), (7, 5, 5)])
def test_route_dispatch_combine(gpu, T, E, k):
  from tinygrad_amd import moe
  rng = np.random.default_rng(T + E)
  logits = rng.standard_normal((T, E)).astype(np.float32)
  if T > 10: logits[3, 2] = logits[3, 7] = 9.0                                   # a tie inside the top-k
  if E == 128: logits[:, :64] -= 3.0                                             # skewed load, some experts (nearly) empty
  r = moe.route(gpu.Buffer.from_numpy(logits), k, E)
  ref = omoe.route(logits, k, E)
  np.testing.assert_array_equal(r.topi.numpy(), ref["topi"])
  np.testing.assert_array_equal(r.off.numpy(), ref["off"])
  np.testing.assert_array_equal(r.dest_row.numpy(), ref["dest_row"])
  np.testing.assert_allclose(r.weights.numpy(), ref["weights"], rtol=2e-6, atol=1e-8)
  assert r.m_l == ref["m_l"]
  # invariants: dest_row is injective into expert-contiguous 256-padded ranges
  d = r.dest_row.numpy(); off = r.off.numpy(); e = r.topi.numpy().reshape(-1)
  assert len(set(d.tolist())) == T * k and (off % 256 == 0).all() and ((d >= off[e]) & (d < off[e + 1])).all()
  D = 64
  x = moe.to_bf16_bits(rng.standard_normal((T, D)).astype(np.float32))
  xg = moe.dispatch(gpu.Buffer.from_numpy(x), r)
  np.testing.assert_array_equal(xg.numpy(), omoe.dispatch(x, ref, k))
  # identity experts: combine(dispatch(x)) = x * sum(weights) = x (up to bf16 rounding of the products)
  out = moe.combine(xg, r, T, k)
  xf = moe.from_bf16_bits(x)
  wb = moe.from_bf16_bits(moe.to_bf16_bits(ref["weights"]))
  exp = moe.to_bf16_bits(moe.from_bf16_bits(moe.to_bf16_bits(xf[:, None, :] * wb[:, :, None])).sum(1))
  np.testing.assert_array_equal(out.numpy(), exp)

@pytest.mark.parametrize("E,N,K,rows", [(4, 256, 128, [256, 0, 512, 256]), (8, 512, 2048, [256] * 8), (3, 256, 768, [512, 256, 0])])
def test_grouped_mxfp8_gemm(gpu, E, N, K, rows):
  from tinygrad_amd import moe
  rng = np.random.default_rng(N + K)
  off = np.concatenate([[0], np.cumsum(rows)]).astype(np.int32)
  M = int(off[-1]) + 256                                                          # one tile beyond expert_off[E]: expert E - 1's by rows_e (moe_routing.py:98-104)
  x = (rng.standard_normal((M, K)) * 0.5).astype(np.float32)
  w = (rng.standard_normal((E, N, K)) * 0.5).astype(np.float32)
  xq, xe8 = omx.quantize_mxfp8(x); wq, we8 = omx.quantize_mxfp8(w)
  C = gpu.Buffer((M, N), np.uint16).zero_()
  bufs = [gpu.Buffer.from_numpy(a) for a in (xq, wq, xe8, we8, off)]
  gpu.check(gpu.lib().tga_grouped_mxfp8_gemm(C.ptr, bufs[0].ptr, bufs[1].ptr, None, None, bufs[2].ptr, bufs[3].ptr, bufs[4].ptr, M, N, K, E, None))
  got = moe.from_bf16_bits(C.numpy())
  ref = omx.grouped_mx_gemm_ref(xq, xe8, wq, we8, off)
  used = M
  err_mx = np.abs(got[:used] - ref[:used]).mean() / np.abs(ref[:used]).mean()
  assert err_mx < 1e-2, err_mx                                                    # the reference's bar
  # tighter: bf16 output of a float32 accumulation of exactly representable products: within one bf16 ulp of the oracle
  np.testing.assert_allclose(got[:used], ref[:used], rtol=2 ** -7, atol=1e-3 * np.abs(ref).max())
  # the routed-only variant writes the same values below expert_off[E] and nothing beyond
  C2 = gpu.Buffer((M, N), np.uint16).zero_()
  gpu.check(gpu.lib().tga_grouped_mxfp8_gemm_routed(C2.ptr, bufs[0].ptr, bufs[1].ptr, bufs[2].ptr, bufs[3].ptr, bufs[4].ptr, M, N, K, E, None))
  np.testing.assert_array_equal(C2.numpy()[:off[-1]], C.numpy()[:off[-1]]); assert (C2.numpy()[off[-1]:] == 0).all()
  # the pointer-argument kernel a Tensor.custom_kernel PROGRAM would bind (arguments in sink order, then the scalars), launched like
  # HIPProgram.__call__ does: 512 threads x (M / 256) (N / 256) workgroups
  import ctypes
  fn = ctypes.c_void_p()
  gpu.check(gpu.lib().tga_kernel_symbol(b"tga_grouped_mxfp8_gemm_kernel", ctypes.byref(fn)))
  C3 = gpu.Buffer((M, N), np.uint16).zero_()
  vals = [ctypes.c_void_p(C3.ptr), ctypes.c_void_p(bufs[0].ptr), ctypes.c_void_p(bufs[1].ptr), ctypes.c_void_p(None), ctypes.c_void_p(None), ctypes.c_void_p(bufs[2].ptr),
          ctypes.c_void_p(bufs[3].ptr), ctypes.c_void_p(bufs[4].ptr), ctypes.c_int(M), ctypes.c_int(N), ctypes.c_int(K), ctypes.c_int(E)]
  args = (ctypes.c_void_p * len(vals))(*[ctypes.cast(ctypes.pointer(v), ctypes.c_void_p) for v in vals])
  grid, block = (ctypes.c_uint32 * 3)((M // 256) * (N // 256), 1, 1), (ctypes.c_uint32 * 3)(512, 1, 1)
  gpu.check(gpu.lib().tga_launch_kernel(fn, grid, block, args, None)); gpu.synchronize()
  np.testing.assert_array_equal(C3.numpy(), C.numpy())
  assert gpu.lib().tga_kernel_symbol(b"no_such_kernel", ctypes.byref(fn)) != 0
  # against the unquantized product: the reference's second bar (< 6e-2)
  full = np.zeros_like(ref)
  for e in range(E): full[off[e]:off[e + 1]] = x[off[e]:off[e + 1]] @ w[e].T
  full[off[-1]:] = x[off[-1]:] @ w[E - 1].T
  assert np.abs(got[:used] - full[:used]).mean() / np.abs(full[:used]).mean() < 6e-2

def test_dense_mx_gemm_and_expert_bias(gpu):
  """The dense MXFP8 GEMM (one expert owning every row) against the oracle's matmul_mx semantics, then the per-expert bias add of
  gpt_oss.py:219-224 on a grouped result (bias cast to bf16, bf16 add), bit for bit."""
  from tinygrad_amd import moe
  rng = np.random.default_rng(12)
  M, N, K = 512, 256, 256
  x = moe.to_bf16_bits((rng.standard_normal((M, K)) * 0.5).astype(np.float32))
  w = (rng.standard_normal((N, K)) * 0.5).astype(np.float32)
  wq, we8 = omx.quantize_mxfp8(w)
  out = moe.mx_gemm(gpu.Buffer.from_numpy(x), (gpu.Buffer.from_numpy(wq), gpu.Buffer.from_numpy(we8)))
  xq, xe8 = omx.quantize_mxfp8(moe.from_bf16_bits(x))
  ref = omx.grouped_mx_gemm_ref(xq, xe8, wq[None], we8[None], np.array([0, M], np.int32))
  got = moe.from_bf16_bits(out.numpy())
  np.testing.assert_allclose(got, ref, rtol=2 ** -7, atol=1e-3 * np.abs(ref).max())
  # bias by expert on three experts' tiles; the last tile lies beyond expert_off[E] and takes the last expert's bias (rows_e)
  E = 3
  off = np.array([0, 256, 256, 512], dtype=np.int32)                 # expert 1 owns no rows
  h = moe.to_bf16_bits(rng.standard_normal((768, N)).astype(np.float32))
  bias = rng.standard_normal((E, N)).astype(np.float32)
  hb = gpu.Buffer.from_numpy(h)
  moe.add_expert_bias(hb, gpu.Buffer.from_numpy(bias), gpu.Buffer.from_numpy(off))
  exp = omx.add_expert_bias(moe.from_bf16_bits(h), bias, off)
  np.testing.assert_array_equal(hb.numpy(), moe.to_bf16_bits(exp))
  assert (hb.numpy()[512:] != h[512:]).any()                         # rows beyond expert_off[E] got expert E - 1's bias

def test_swiglu_interleaved(gpu):
  """The clamped interleaved SwiGLU between the two grouped GEMMs (examples/mlperf/models/gpt_oss.py:94-98) on bf16 rows, bit for bit against the
  oracle's bf16 chain except where the device's exp differs by an ulp before the bf16 rounding (at most one bf16 ulp, a handful of elements)."""
  from tinygrad_amd import moe
  rng = np.random.default_rng(21)
  h = moe.to_bf16_bits((rng.standard_normal((300, 512)) * 4).astype(np.float32))
  h[0, :8] = moe.to_bf16_bits(np.array([100, 100, -100, -100, 7, -7, 0, 0], np.float32))
  y = moe.swiglu(gpu.Buffer.from_numpy(h)).numpy()
  ref = omx.swiglu_interleaved(moe.from_bf16_bits(h))
  got = moe.from_bf16_bits(y)
  assert y.shape == (300, 256)
  np.testing.assert_allclose(got, ref, rtol=2 ** -7, atol=1e-30)
  assert (moe.to_bf16_bits(ref) == y).mean() > 0.99

def test_moe_feed_forward_composition(gpu):
  """moe.moe_feed_forward (route -> dispatch -> grouped GEMM + bias -> SwiGLU -> grouped GEMM + bias -> combine, gpt_oss.py:213-226) against the
  reference's per-expert loop (gpt_oss.py:227-238) restated in the oracle; the reference has no test of its own for either branch, the
  loop is the definition (oracle pinned in tests/test_oracle_pins.py).  Bar: the reference's MXFP8 GEMM bar (mean rel-err < 1e-2), since the two
  branches round to bf16 at different points (the loop weighs and sums bf16 contributions expert by expert, the grouped branch weighs rows)."""
  from tinygrad_amd import moe
  rng = np.random.default_rng(33)
  T, D, I, E, k = 96, 256, 256, 6, 2
  inp = moe.to_bf16_bits(rng.standard_normal((T, D)).astype(np.float32))
  logits = rng.standard_normal((T, E)).astype(np.float32); logits[:, 4] = -30.0       # expert 4 is never selected: an empty range
  wgu, wdn = (rng.standard_normal((E, 2 * I, D)) * D ** -0.5).astype(np.float32), (rng.standard_normal((E, D, I)) * I ** -0.5).astype(np.float32)
  bgu, bdn = (rng.standard_normal((E, 2 * I)) * 0.1).astype(np.float32), (rng.standard_normal((E, D)) * 0.1).astype(np.float32)
  (gq, ge), (dq, de) = omx.quantize_mxfp8(wgu), omx.quantize_mxfp8(wdn)
  B = gpu.Buffer.from_numpy
  ref = omx.moe_feed_forward_loop(moe.from_bf16_bits(inp), logits, k, gq, ge, bgu, dq, de, bdn)
  for routed_only in (True, False):
    out = moe.moe_feed_forward(B(inp), B(logits), k, (B(gq), B(ge)), B(bgu), (B(dq), B(de)), B(bdn), routed_only=routed_only)
    got = moe.from_bf16_bits(out.numpy())
    assert got.shape == (T, D) and np.isfinite(got).all()
    err = np.abs(got - ref).mean() / np.abs(ref).mean()
    print(f"moe_feed_forward vs per-expert loop (routed_only={routed_only}): mean rel-err {err:.2e}")
    assert err < 1e-2
    np.testing.assert_allclose(got, ref, rtol=0.05, atol=0.02 * np.abs(ref).max())

def test_grouped_gemm_with_counts_skips_padding(gpu):
  """tga_grouped_mxfp8_gemm_counts: routed rows equal the routed-tiles product bit for bit; padding rows inside an expert's range come out as zeros even
  when A holds garbage there; rows beyond expert_off[E] keep their contents.  Experts of 1, 16, 17, 128, 129, 255, 256 and 300 rows and an empty one."""
  rng = np.random.default_rng(41)
  counts = np.array([1, 16, 17, 0, 128, 129, 255, 256, 300], np.int32)
  E, N, K = len(counts), 512, 384
  off = np.concatenate([[0], np.cumsum((counts + 255) // 256 * 256)]).astype(np.int32)
  M = int(off[-1]) + 512                                              # two tiles beyond the routed range
  def rand_mx(rows):
    q = rng.integers(0, 256, size=(rows, K), dtype=np.uint8); q[(q & 0x7F) == 0x7F] = 0x38
    return q, rng.integers(121, 126, size=(rows, K // 32), dtype=np.uint8)
  xq, xe = rand_mx(M); wq, we = rand_mx(E * N)                         # padding rows of A are random too: they must not reach the output
  bufs = [gpu.Buffer.from_numpy(a) for a in (xq, wq, xe, we)]
  offb, cntb = gpu.Buffer.from_numpy(off), gpu.Buffer.from_numpy(counts)
  C1, C2 = gpu.Buffer((M, N), np.uint16), gpu.Buffer((M, N), np.uint16)
  for C in (C1, C2): gpu.check(gpu.lib().tga_memset(C.ptr, 0xAB, C.nbytes, None))
  gpu.check(gpu.lib().tga_grouped_mxfp8_gemm_routed(C1.ptr, bufs[0].ptr, bufs[1].ptr, bufs[2].ptr, bufs[3].ptr, offb.ptr, M, N, K, E, None))
  gpu.check(gpu.lib().tga_grouped_mxfp8_gemm_counts(C2.ptr, bufs[0].ptr, bufs[1].ptr, bufs[2].ptr, bufs[3].ptr, offb.ptr, cntb.ptr, M, N, K, E, None))
  c1, c2 = C1.numpy(), C2.numpy()
  for e in range(E):
    lo, n, hi = int(off[e]), int(counts[e]), int(off[e + 1])
    np.testing.assert_array_equal(c2[lo:lo + n], c1[lo:lo + n], err_msg=f"routed rows of expert {e}")
    pad16 = lo + (n + 15) // 16 * 16                                  # rows of a 16-row group that also holds routed rows are multiplied like them
    np.testing.assert_array_equal(c2[lo + n:pad16], c1[lo + n:pad16])
    assert (c2[pad16:hi] == 0).all(), f"padding rows of expert {e}"
  assert (c2[off[-1]:] == 0xABAB).all()
