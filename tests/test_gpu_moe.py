"""MoE decode pieces on the GPU vs the oracle: expert gating/top-k (reference vectors test/unit/test_attention.py:249-270),
MXFP4 expert GEMVs with expert indirection (ExpertWeights, tinygrad/llm/model.py:21-27), the reference's MoE closed form
(test/unit/test_llm_moe.py:15-34) and a small OLMoE-architecture greedy decode."""
import numpy as np, pytest
from oracle import ggml as og, linear as ol, moe as omoe, llm as ollm
from tinygrad_amd import synth

pytestmark = pytest.mark.gpu

def _gate(gpu, logits, k, gating=1, norm=False, scale=1.0):
  from tinygrad_amd.nn import moe_gate
  T, E = logits.shape
  lb = gpu.Buffer.from_numpy(logits.astype(np.float32)); sel = gpu.Buffer((T, k), np.int32); pr = gpu.Buffer((T, k), np.float32)
  moe_gate(lb, T, E, k, sel, pr, gating, norm, scale)
  return sel.numpy(), pr.numpy()

def test_pairwise_topk_reference_vectors(gpu):
  sel, p = _gate(gpu, np.array([[1.0, 3.0, 2.0, 5.0, 4.0]]), 3, gating=3)          # SOFTMAX_WEIGHT: scores are the logits themselves
  assert sel.tolist() == [[1, 4, 3]]
  np.testing.assert_allclose(p[0], omoe.softmax(np.array([3.0, 4.0, 5.0])), rtol=1e-6)
  sel, _ = _gate(gpu, np.array([[5.0, 5.0, 3.0, 5.0]]), 2, gating=3)               # duplicates: the lower index ranks higher, output ascending
  assert sel.tolist() == [[1, 0]]

@pytest.mark.parametrize("gating", [1, 2, 3, 4])
@pytest.mark.parametrize("norm", [False, True])
def test_gating_modes_vs_oracle(gpu, gating, norm):
  rng = np.random.default_rng(10 * gating + norm)
  lg = rng.standard_normal((7, 64)).astype(np.float32) * 2
  lg[3, 10] = lg[3, 20] = lg[3].max() + 1                                          # an exact tie among the selected
  sel, p = _gate(gpu, lg, 8, gating, norm, 2.5)
  rs, rp = omoe.gate_probs(lg, 8, gating, norm, 2.5)
  np.testing.assert_array_equal(sel, rs)
  np.testing.assert_allclose(p, rp, rtol=2e-5, atol=1e-7)

@pytest.mark.parametrize("t,kdim,n", [(39, 2048, 1024), (39, 1024, 2048), (2, 512, 256), (8, 256, 192), (14, 512, 96), (12, 1024, 96), (13, 512, 128), (3, 512, 96), (6, 256, 128), (7, 1024, 64), (23, 1024, 96), (18, 512, 96), (21, 1024, 64), (22, 512, 128), (41, 256, 96)])
def test_expert_gemv_with_indirection(gpu, t, kdim, n):
  from tinygrad_amd.nn import ExpertWeights
  rng = np.random.default_rng(n + t)
  E, T, k = 6, 3, 4
  w = synth.random_blocks(rng, t, E * n, kdim)
  wu = synth.random_blocks(rng, t, E * n, kdim)
  W, WU = ol.weight_f32(w, E * n, kdim, t).reshape(E, n, kdim), ol.weight_f32(wu, E * n, kdim, t).reshape(E, n, kdim)
  x = synth.activations(rng, T, kdim, np.float16)
  sel = rng.integers(0, E, size=(T, k)).astype(np.int32)
  ew, eu = ExpertWeights(gpu.Buffer.from_numpy(w), t, E, n, kdim), ExpertWeights(gpu.Buffer.from_numpy(wu), t, E, n, kdim)
  selb, xb = gpu.Buffer.from_numpy(sel), gpu.Buffer.from_numpy(x)
  y = gpu.Buffer((T * k, n), np.float32)
  ew(selb, xb, y, jobs_per_x_row=k)
  ref = np.stack([ol.linear_f64(x[j // k][None].astype(np.float32), W[sel.reshape(-1)[j]])[0] for j in range(T * k)])
  assert ol.rel_err(y.numpy(), ref) <= 1e-3
  # SwiGLU pair: silu(gate_e x) * (up_e x)
  ew(selb, xb, y, jobs_per_x_row=k, up=eu)
  refu = np.stack([ol.linear_f64(x[j // k][None].astype(np.float32), WU[sel.reshape(-1)[j]])[0] for j in range(T * k)])
  assert ol.rel_err(y.numpy(), ref / (1 + np.exp(-ref)) * refu) <= 1e-3
  # one activation row per job (the down projection's case)
  xj = synth.activations(rng, T * k, kdim, np.float16)
  ew(selb, gpu.Buffer.from_numpy(xj), y, jobs_per_x_row=1)
  refj = np.stack([ol.linear_f64(xj[j][None].astype(np.float32), W[sel.reshape(-1)[j]])[0] for j in range(T * k)])
  assert ol.rel_err(y.numpy(), refj) <= 1e-3

@pytest.mark.parametrize("dim,E,k,gating,normw", [(2048, 64, 8, 1, True), (256, 8, 2, 3, True), (1024, 130, 6, 2, False)])
def test_router_in_one_launch(gpu, dim, E, k, gating, normw):
  """tga_moe_router (ffn_norm + router logits + gating + top-k) against the oracle fed with the float64 logits of the fp16-rounded row."""
  from tinygrad_amd.nn import QuantLinear, moe_router
  from tinygrad_amd import runtime as rt
  rng = np.random.default_rng(dim + E)
  x = (rng.standard_normal(dim) * 2).astype(np.float32); nw = rng.standard_normal(dim).astype(np.float32)
  wr = (rng.standard_normal((E, dim)) * dim ** -0.5).astype(np.float16)
  router = QuantLinear(gpu.Buffer.from_numpy(wr.view(np.uint8).reshape(-1)), rt.F16, E, dim)
  xn, lg = gpu.Buffer((dim,), np.float16), gpu.Buffer((E + 1,), np.float32).zero_()
  sel, pr = gpu.Buffer((k,), np.int32), gpu.Buffer((k,), np.float32)
  for _ in range(2):                                                     # twice: the arrival counter is left at zero
    moe_router(gpu.Buffer.from_numpy(x), gpu.Buffer.from_numpy(nw) if normw else None, 1e-5, router, k, sel, pr, lg, xn_out=xn, gating=gating,
               norm_topk_prob=True, scale=1.5)
  assert lg.numpy()[E:].view(np.int32)[0] == 0
  lgv = lg.numpy()[:E]
  h = (ollm.rmsnorm(x, nw, 1e-5) if normw else x).astype(np.float16)
  assert np.mean(xn.numpy() != h) < 0.01 and ol.rel_err(xn.numpy().astype(np.float32), h.astype(np.float32)) < 1e-3   # fp16 ties may round either way
  ref_lg = (h.astype(np.float64) @ wr.astype(np.float64).T).astype(np.float32)
  assert ol.rel_err(lgv, ref_lg) <= 1e-3
  rs, rp = omoe.gate_probs(lgv[None], k, gating, True, 1.5)        # selection on the kernel's own logits: exact
  np.testing.assert_array_equal(sel.numpy(), rs[0])
  np.testing.assert_allclose(pr.numpy(), rp[0], rtol=2e-5, atol=1e-7)

@pytest.mark.parametrize("T,dim,E", [(1, 2048, 64), (5, 2048, 64), (8, 256, 8), (3, 1024, 130)])
def test_router_logits_for_several_tokens(gpu, T, dim, E):
  """tga_moe_router_rows (ffn_norm + router logits of T tokens in one launch) against the single-token launch row by row: same fp16 rows, same logits, bit
  for bit; and the logits against float64."""
  from tinygrad_amd import runtime as rt
  L = gpu.lib()
  rng = np.random.default_rng(T + dim + E)
  x = (rng.standard_normal((T, dim)) * 2).astype(np.float32); nw = rng.standard_normal(dim).astype(np.float32)
  wr = (rng.standard_normal((E, dim)) * dim ** -0.5).astype(np.float16)
  xb, nb, wb = gpu.Buffer.from_numpy(x), gpu.Buffer.from_numpy(nw), gpu.Buffer.from_numpy(wr)
  xn, lg = gpu.Buffer((T, dim), np.float16), gpu.Buffer((T, E), np.float32)
  for b in (xn, lg): gpu.check(L.tga_memset(b.ptr, 0xFF, b.nbytes, None))
  gpu.check(L.tga_moe_router_rows(xb.ptr, nb.ptr, 1e-5, wb.ptr, T, dim, E, xn.ptr, lg.ptr, None))
  for t in range(T):
    xn1, lg1 = gpu.Buffer((dim,), np.float16), gpu.Buffer((E + 1,), np.float32).zero_()
    gpu.check(L.tga_moe_router(xb.ptr + 4 * t * dim, nb.ptr, 1e-5, wb.ptr, dim, E, 0, 1, 0, 1.0, xn1.ptr, lg1.ptr, None, None, None))
    assert xn.numpy()[t].tobytes() == xn1.numpy().tobytes()
    np.testing.assert_array_equal(lg.numpy()[t], lg1.numpy()[:E])
  ref = xn.numpy().astype(np.float64) @ wr.astype(np.float64).T
  assert ol.rel_err(lg.numpy(), ref.astype(np.float32)) <= 1e-3

@pytest.mark.parametrize("t,dim,k", [(1, 2048, 8), (2, 1024, 4), (14, 512, 1), (39, 2048, 6)])
def test_weighted_expert_sum_folded_into_the_next_linear(gpu, t, dim, k):
  """tga_moe_combine_rmsnorm_qlinear_multi against tga_moe_combine followed by tga_rmsnorm_qlinear_multi: same completed row (bit for
  bit: the same products in the same order), same linear outputs up to the summation order of the mean square."""
  from tinygrad_amd.nn import QuantLinear, qlinear_multi, moe_combine
  rng = np.random.default_rng(dim + k + t)
  ns = [192, 64]
  if t == 1: ws = [(rng.standard_normal((n, dim)) * dim ** -0.5).astype(np.float16).view(np.uint8).reshape(-1) for n in ns]
  else: ws = [synth.random_blocks(rng, t, n, dim) for n in ns]
  layers = [QuantLinear(gpu.Buffer.from_numpy(w), t, n, dim) for w, n in zip(ws, ns)]
  x = rng.standard_normal((1, dim)).astype(np.float32); y = rng.standard_normal((k, dim)).astype(np.float32); p = rng.random(k).astype(np.float32)
  nw = rng.standard_normal(dim).astype(np.float32)
  xb, yb, pb, nwb = (gpu.Buffer.from_numpy(a) for a in (x, y, p, nw))
  x_out = gpu.Buffer((1, dim), np.float32).zero_()
  fused = [gpu.Buffer((1, n), np.float32) for n in ns]
  qlinear_multi(layers, xb, fused, norm=(nwb, 1e-5), combine=(yb, pb, k, x_out))
  x_ref = gpu.Buffer((1, dim), np.float32)
  moe_combine(yb, pb, xb, 1, k, dim, x_ref)
  plain = [gpu.Buffer((1, n), np.float32) for n in ns]
  qlinear_multi(layers, x_ref, plain, norm=(nwb, 1e-5))
  np.testing.assert_allclose(x_out.numpy(), x_ref.numpy(), rtol=1e-6, atol=1e-6)
  np.testing.assert_allclose(x_out.numpy(), x + (y * p[:, None]).sum(0, keepdims=True), rtol=1e-5, atol=1e-5)
  assert xb.numpy().tobytes() == x.tobytes()                           # the input row is left alone
  for f, q in zip(fused, plain): assert ol.rel_err(f.numpy(), q.numpy()) <= 2e-4
  with pytest.raises(RuntimeError): qlinear_multi(layers, xb, fused, norm=(nwb, 1e-5), combine=(yb, pb, 9, x_out))

@pytest.mark.parametrize("T", [1, 3, 8])
@pytest.mark.parametrize("t,dim,n,E,k,gating", [(39, 2048, 256, 64, 8, 1), (2, 512, 128, 8, 2, 3), (1, 1024, 96, 130, 6, 2), (12, 1024, 64, 16, 4, 4)])
def test_expert_gate_up_that_gates_for_itself(gpu, t, dim, n, E, k, gating, T):
  """tga_qlinear_experts_routed / _routed_rows (scores, top-k and weights computed inside the expert gate/up launch from the router logits, every
  workgroup for its own token) against tga_moe_gate followed by tga_qlinear_experts: identical selection and weights, identical outputs, for
  one token and for several tokens in one launch."""
  from tinygrad_amd.nn import ExpertWeights, moe_gate
  rng = np.random.default_rng(dim + E + k + T)
  mk = (lambda: synth.random_blocks(rng, t, E * n, dim)) if t != 1 else (lambda: (rng.standard_normal((E * n, dim)) * dim ** -0.5).astype(np.float16).view(np.uint8).reshape(-1))
  ew, eu = ExpertWeights(gpu.Buffer.from_numpy(mk()), t, E, n, dim), ExpertWeights(gpu.Buffer.from_numpy(mk()), t, E, n, dim)
  x = gpu.Buffer.from_numpy(synth.activations(rng, T, dim, np.float16))
  lg = gpu.Buffer.from_numpy(rng.standard_normal((T, E)).astype(np.float32))
  sel0, p0, y0 = gpu.Buffer((T * k,), np.int32), gpu.Buffer((T * k,), np.float32), gpu.Buffer((T * k, n), np.float32)
  moe_gate(lg, T, E, k, sel0, p0, gating, True, 1.25)
  ew(sel0, x, y0, jobs_per_x_row=k, up=eu)
  sel1, p1, y1 = gpu.Buffer((T * k,), np.int32).zero_(), gpu.Buffer((T * k,), np.float32).zero_(), gpu.Buffer((T * k, n), np.float32).zero_()
  ew(sel1, x, y1, jobs_per_x_row=k, up=eu, route=(lg, gating, True, 1.25, p1))
  np.testing.assert_array_equal(sel1.numpy(), sel0.numpy())
  np.testing.assert_array_equal(p1.numpy(), p0.numpy())
  np.testing.assert_array_equal(y1.numpy(), y0.numpy())
  rs, rp = omoe.gate_probs(lg.numpy(), k, gating, True, 1.25)
  np.testing.assert_array_equal(sel1.numpy().reshape(T, k), rs)

def test_moe_combine(gpu):
  from tinygrad_amd.nn import moe_combine
  rng = np.random.default_rng(3)
  T, k, D = 3, 8, 2048
  y, p, r = rng.standard_normal((T, k, D)).astype(np.float32), rng.random((T, k)).astype(np.float32), rng.standard_normal((T, D)).astype(np.float32)
  out = gpu.Buffer((T, D), np.float32)
  moe_combine(gpu.Buffer.from_numpy(y), gpu.Buffer.from_numpy(p), gpu.Buffer.from_numpy(r), T, k, D, out)
  np.testing.assert_allclose(out.numpy(), r + (y * p[:, :, None]).sum(1), rtol=1e-5, atol=1e-5)

@pytest.mark.parametrize("T,k,D", [(3, 8, 2048), (8, 2, 256), (16, 8, 4096), (2, 3, 6152)])
def test_moe_combine_folded_into_the_next_norm(gpu, T, k, D):
  """tga_moe_combine_rmsnorm_rows against tga_moe_combine followed by tga_rmsnorm_rows: the completed rows and both norm outputs bit for bit (rows of up to
  2048 values stay in registers, longer ones are read back by the thread that completed them), and the rows against numpy."""
  from tinygrad_amd.nn import moe_combine
  L = gpu.lib()
  rng = np.random.default_rng(T + k + D)
  y, p = rng.standard_normal((T, k, D)).astype(np.float32), rng.random((T, k)).astype(np.float32)
  r, w = rng.standard_normal((T, D)).astype(np.float32), (1 + 0.1 * rng.standard_normal(D)).astype(np.float32)
  yb, pb, wb = gpu.Buffer.from_numpy(y), gpu.Buffer.from_numpy(p), gpu.Buffer.from_numpy(w)
  x0, h0, f0 = gpu.Buffer.from_numpy(r), gpu.Buffer((T, D), np.float16), gpu.Buffer((T, D), np.float32)
  moe_combine(yb, pb, x0, T, k, D, x0)
  gpu.check(L.tga_rmsnorm_rows(x0.ptr, wb.ptr, T, D, 1e-5, h0.ptr, f0.ptr, 0, None))
  x1, h1, f1 = gpu.Buffer.from_numpy(r), gpu.Buffer((T, D), np.float16), gpu.Buffer((T, D), np.float32)
  for b in (h1, f1): gpu.check(L.tga_memset(b.ptr, 0xFF, b.nbytes, None))
  gpu.check(L.tga_moe_combine_rmsnorm_rows(yb.ptr, pb.ptr, x1.ptr, wb.ptr, T, k, D, 1e-5, h1.ptr, f1.ptr, None))
  np.testing.assert_array_equal(x1.numpy(), x0.numpy())
  np.testing.assert_array_equal(f1.numpy(), f0.numpy())
  assert h1.numpy().tobytes() == h0.numpy().tobytes()
  full = r + (y * p[:, :, None]).sum(1)
  np.testing.assert_allclose(x1.numpy(), full, rtol=1e-5, atol=1e-5)
  ref = full / np.sqrt((full.astype(np.float64) ** 2).mean(1, keepdims=True) + 1e-5) * w
  np.testing.assert_allclose(f1.numpy(), ref, rtol=2e-5, atol=2e-5)

SMALL_MOE = dict(num_blocks=2, dim=256, hidden_dim=128, n_heads=4, n_kv_heads=4, norm_eps=1e-5, vocab_size=512, head_dim=64, rope_theta=10000.0,
                 qk_norm=256, num_experts=8, num_experts_per_tok=2, norm_topk_prob=False, expert_gating_func=1)

def test_small_olmoe_decode(gpu):
  """OLMoE-architecture (fp16 attention/router, MXFP4 experts, full-width qk norm) greedy decode vs the numpy restatement."""
  from tinygrad_amd.llm import Transformer, TransformerConfig, synth_state_moe
  c = TransformerConfig(max_context=128, **SMALL_MOE)
  sd = synth_state_moe(c, seed=1004)
  gpu.synchronize()
  host = {k: (b.numpy(), t, shp) for k, (b, t, shp) in sd.items()}
  model = Transformer(c, sd, max_new=64)
  rng = np.random.default_rng(1004)
  prompt = [int(t) for t in rng.integers(0, 512, size=20)]
  from decode_helpers import greedy_vs_reference_numerics
  got, ref, worst, margin, rms = greedy_vs_reference_numerics(model, ollm.Model(SMALL_MOE, host, 128, act_round_f16=False), prompt, 32)
  print(f"oracle (reference numerics) min top-2 margin over 32 steps {margin:.4f} (logit rms {rms:.4f}); worst logits rel-err {worst:.2e}")
  assert got == ref
  assert worst <= 1e-3

@pytest.mark.parametrize("gating", [1, 2, 3, 4])
@pytest.mark.parametrize("norm", [False, True])
def test_gating_with_selection_bias_vs_oracle(gpu, gating, norm):
  """exp_probs_b (model.py:113, 123): ranks by score + bias, weights from the unbiased scores; the hand case of tests/test_oracle_pins.py first."""
  from tinygrad_amd.nn import moe_gate
  def gate(lg, bias, k, g, nrm, scale):
    T, E = lg.shape
    sel, pr = gpu.Buffer((T, k), np.int32), gpu.Buffer((T, k), np.float32)
    moe_gate(gpu.Buffer.from_numpy(lg), T, E, k, sel, pr, g, nrm, scale, bias=gpu.Buffer.from_numpy(bias))
    return sel.numpy(), pr.numpy()
  sel, p = gate(np.array([[0.0, np.log(3.0), -np.log(3.0), 0.0]], np.float32), np.array([0.0, 0.0, 1.0, 0.0], np.float32), 2, 2, False, 1.0)
  assert sel.tolist() == [[1, 2]]
  np.testing.assert_allclose(p, [[0.75, 0.25]], rtol=1e-6)
  rng = np.random.default_rng(100 + 10 * gating + norm)
  lg = rng.standard_normal((9, 96)).astype(np.float32) * 2
  bias = rng.uniform(-0.5, 0.5, 96).astype(np.float32)
  sel, p = gate(lg, bias, 8, gating, norm, 1.75)
  rs, rp = omoe.gate_probs(lg, 8, gating, norm, 1.75, bias=bias)
  np.testing.assert_array_equal(sel, rs)
  np.testing.assert_allclose(p, rp, rtol=2e-5, atol=1e-7)
  assert (sel != omoe.gate_probs(lg, 8, gating, norm, 1.75)[0]).any()             # the bias changes at least one selection in this sample

GLM_LIKE = dict(num_blocks=3, dim=512, hidden_dim=256, n_heads=8, n_kv_heads=2, norm_eps=1e-5, vocab_size=512, head_dim=64, rope_theta=10000.0,
                num_experts=8, num_experts_per_tok=2, norm_topk_prob=True, expert_gating_func=2, routed_scaling_factor=1.5,
                leading_dense_blocks=1, dense_hidden_dim=768, shared_expert_dim=256, shared_expert_gate=True, expert_bias=True)

@pytest.mark.parametrize("gate", [True, False], ids=["gated_shared_expert", "plain_shared_expert"])
def test_small_glm4moe_like_decode(gpu, gate):
  """The model-zoo extras of FFNBlock (model.py:84, 99-103, 113, 131-134) together: a leading dense block, sigmoid gating with an expert selection
  bias, normalised and scaled top-k weights, and a shared expert (with and without its sigmoid gate) on every MoE block; 32 greedy tokens against
  the oracle on reference numerics."""
  from tinygrad_amd.llm import Transformer, TransformerConfig, synth_state_moe
  from decode_helpers import greedy_vs_reference_numerics
  cfg = dict(GLM_LIKE, shared_expert_gate=gate)
  c = TransformerConfig(max_context=128, **cfg)
  sd = synth_state_moe(c, seed=1009)
  gpu.synchronize()
  host = {k: (b.numpy(), t, shp) for k, (b, t, shp) in sd.items()}
  model = Transformer(c, sd, max_new=64)
  assert [b.moe for b in model.blk] == [False, True, True] and model.blk[1].shared and (model.blk[1].sh_gate_inp is not None) == gate
  rng = np.random.default_rng(1009)
  prompt = [int(t) for t in rng.integers(0, 512, size=20)]
  oracle = ollm.Model(cfg, host, 128, act_round_f16=False)
  got, ref, worst, margin, rms = greedy_vs_reference_numerics(model, oracle, prompt, 32)
  print(f"oracle (reference numerics) min top-2 margin over 32 steps {margin:.4f} (logit rms {rms:.4f}); worst logits rel-err {worst:.2e}; min biased-score gap {oracle.min_route_gap:.2e}")
  assert got == ref
  assert worst <= 1e-3
  # every extra matters: dropping any one of them moves the oracle's logits far away from the GPU's
  lg_gpu = model.logits()
  hist = prompt + got[:-1]
  for drop in ("exp_probs_b.bias", "ffn_gate_shexp.weight"):
    host2 = {k: v for k, v in host.items() if not k.endswith(drop)}
    if drop == "ffn_gate_shexp.weight": host2 = {k: v for k, v in host2.items() if "shexp" not in k}
    o2 = ollm.Model(cfg, host2, 128, act_round_f16=False)
    for pos, t in enumerate(hist): lg2 = o2.forward(t, pos)
    print(f"without {drop}: logits rel-err {ol.rel_err(lg2, lg_gpu):.3f}")
    assert ol.rel_err(lg2, lg_gpu) > 5e-3, drop                                    # five times the parity bar
