"""Batched decode (2..8 sequences in lockstep) on the GPU: the grouped expert GEMMs against the per-job expert GEMV and the C restatement, dense
fp16 linears at M > 1, and BatchedTransformer against the numpy restatement of tinygrad/llm/model.py run once PER SEQUENCE with the reference's
numerics (fp32 activations into fp16-rounded weights): equal greedy tokens for every sequence and logits within rel-err 1e-3 at every step."""
import numpy as np, pytest
from oracle import cref, linear as ol, llm as ollm
from tinygrad_amd import synth

pytestmark = pytest.mark.gpu
TOL = 1e-3

def _f16_weight(rng, n, k): return (rng.standard_normal((n, k)) * k ** -0.5).astype(np.float16)

@pytest.mark.parametrize("m", [2, 3, 5, 8])
def test_dense_f16_linear_small_batches(gpu, m):
  from tinygrad_amd.nn import QuantLinear
  rng = np.random.default_rng(40 + m)
  n, k = 300, 2048
  w = _f16_weight(rng, n, k)
  x = synth.activations(rng, m, k, np.float16)
  y = QuantLinear(gpu.Buffer.from_numpy(w.view(np.uint8).reshape(-1)), gpu.F16, n, k)(gpu.Buffer.from_numpy(x), out_dtype=np.float32).numpy()
  assert ol.rel_err(y, ol.linear_f64(x.astype(np.float32), w.astype(np.float32))) <= TOL

@pytest.mark.parametrize("t,dim,n,E,k,B", [(39, 2048, 1024, 64, 8, 8), (39, 1024, 2048, 64, 8, 5), (2, 512, 130, 8, 2, 3), (1, 1024, 96, 16, 4, 8), (12, 1024, 64, 16, 4, 2), (14, 512, 48, 6, 3, 1), (23, 1024, 64, 8, 2, 4), (21, 512, 96, 8, 2, 5), (22, 1024, 48, 6, 3, 3), (18, 512, 64, 8, 4, 2), (41, 512, 64, 8, 2, 3)])
def test_experts_grouped_against_per_job_gemv_and_oracle(gpu, t, dim, n, E, k, B):
  """Every (token, slot) job's row against the C restatement on that job's expert (model-path numerics: fp16-rounded weights), for the plain
  product with one activation row per job (the down projection's shape of call) and for silu(gate) * up with one row per token."""
  from tinygrad_amd.nn import ExpertWeights, expert_jobs, experts_grouped
  from tinygrad_amd.runtime import GGML_QUANT
  rng = np.random.default_rng(dim + E + k + B)
  if t == 1: mk = lambda: _f16_weight(rng, E * n, dim).view(np.uint8).reshape(-1); row_bytes = 2 * dim
  else: mk = lambda: synth.random_blocks(rng, t, E * n, dim, sigma=0.0002 if t in (23, 18, 21, 22) else 0.003); row_bytes = dim // GGML_QUANT[t][0] * GGML_QUANT[t][1]   # (small scales where a block's range is wide: silu(gate) * up is stored as fp16)
  wg, wu = mk(), mk()
  ew, eu = ExpertWeights(gpu.Buffer.from_numpy(wg), t, E, n, dim), ExpertWeights(gpu.Buffer.from_numpy(wu), t, E, n, dim)
  sel_host = np.stack([rng.permutation(E)[:k] for _ in range(B)]).astype(np.int32).reshape(-1)     # distinct experts inside a token, repeats across tokens
  if B > 1: sel_host[k] = sel_host[0]                                                                 # at least one expert shared by two tokens
  sel = gpu.Buffer.from_numpy(sel_host)
  table, flags = gpu.Buffer((E, 16), np.int32).zero_(), gpu.Buffer((1,), np.int32).zero_()
  expert_jobs(sel, E, table, flags)
  tab = table.numpy()
  assert flags.numpy()[0] == 0 and tab[:, 0].sum() == B * k
  for e in range(E): assert sorted(tab[e, 1:1 + tab[e, 0]].tolist()) == np.nonzero(sel_host == e)[0].tolist()
  def deq_lin(w, e, x): return cref.linear(t, w[e * n * row_bytes:(e + 1) * n * row_bytes], x.astype(np.float32).reshape(1, -1), n, dim, w_round_f16=True)[0] if t != 1 else \
      (x.astype(np.float64) @ w.view(np.float16).reshape(E, n, dim)[e].astype(np.float64).T).astype(np.float32)
  # plain product, one activation row per job
  xj = synth.activations(rng, B * k, dim, np.float16)
  y = gpu.Buffer((B * k, n), np.float32).zero_()
  experts_grouped(ew, table, B * k, gpu.Buffer.from_numpy(xj), y, jobs_per_x_row=1)
  ref = np.stack([deq_lin(wg, sel_host[j], xj[j]) for j in range(B * k)])
  assert ol.rel_err(y.numpy(), ref) <= TOL
  # silu(gate) * up, one activation row per token
  xt = synth.activations(rng, B, dim, np.float16)
  a = gpu.Buffer((B * k, n), np.float16).zero_()
  experts_grouped(ew, table, B * k, gpu.Buffer.from_numpy(xt), a, jobs_per_x_row=k, up=eu)
  refa = np.stack([ollm.silu(deq_lin(wg, sel_host[j], xt[j // k])) * deq_lin(wu, sel_host[j], xt[j // k]) for j in range(B * k)])
  assert ol.rel_err(a.numpy(), refa) <= TOL + 2.0 ** -11
  # and against the per-job GEMV of the batch-1 path on the same operands
  y1 = gpu.Buffer((B * k, n), np.float32)
  ew(sel, gpu.Buffer.from_numpy(xj), y1, jobs_per_x_row=1)
  assert ol.rel_err(y.numpy(), y1.numpy()) <= TOL

def test_expert_jobs_flags_overflow_and_bad_ids(gpu):
  from tinygrad_amd.nn import expert_jobs
  sel = gpu.Buffer.from_numpy(np.array([3] * 9 + [70, -1, 2], np.int32))
  table, flags = gpu.Buffer((8, 16), np.int32).zero_(), gpu.Buffer((1,), np.int32).zero_()
  expert_jobs(sel, 8, table, flags)
  assert flags.numpy()[0] == 3 and table.numpy()[3, 0] == 8 and table.numpy()[2, 0] == 1

def _per_sequence_check(gpu, model, cfg, host, prompts, n_new, max_context):
  """Steps the batch on the GPU and one oracle per sequence (fed the GPU's tokens); every row's greedy token and logits are compared."""
  B = len(prompts)
  oracles = [ollm.Model(cfg, host, max_context, act_round_f16=False) for _ in range(B)]
  model.prefill(prompts)
  pos = 0
  for i in range(len(prompts[0]) - 1):
    for b in range(B): oracles[b].forward(prompts[b][i], pos)
    pos += 1
  cur, worst, margin, near_ties = [p[-1] for p in prompts], 0.0, np.inf, 0
  for step in range(n_new):
    model.decode_step()
    lg_gpu = model.logits()
    toks = model.out_tokens.view(4 * step * B, (B,), np.int32).numpy()
    for b in range(B):
      lg = oracles[b].forward(cur[b], pos)
      top2 = np.partition(lg, -2)[-2:]; margin = min(margin, float(top2[1] - top2[0]))
      worst = max(worst, ol.rel_err(lg_gpu[b], lg))
      assert int(toks[b]) == int(np.argmax(lg_gpu[b])), (step, b, "the token is not the first maximum of the GPU's own logits")
      if int(toks[b]) != int(np.argmax(lg)):                              # the oracle may prefer another token only across a near-tie of its own logits (inside the logits bar)
        between = float(lg[int(np.argmax(lg))] - lg[int(toks[b])])
        assert between <= 2 * TOL * float(np.abs(lg).max()), (step, b, f"rel-err of this row {ol.rel_err(lg_gpu[b], lg):.2e}", f"oracle margin between the two candidates {between:.3e}",
                                                               f"logit max {np.abs(lg).max():.3f}", getattr(oracles[b], "last_sel", None))
        near_ties += 1
      cur[b] = int(toks[b])
    pos += 1
  model.check_state()
  print(f"batch {B}: worst logits rel-err {worst:.2e}, min oracle top-2 margin {margin:.4f}, {near_ties} of {B * n_new} tokens across an oracle near-tie")
  assert worst <= TOL and near_ties <= max(1, B * n_new // 50)

SMALL = dict(num_blocks=2, dim=256, hidden_dim=512, n_heads=4, n_kv_heads=2, norm_eps=1e-5, vocab_size=512, head_dim=64, rope_theta=500000.0)
SMALL_MOE = dict(num_blocks=2, dim=256, hidden_dim=128, n_heads=4, n_kv_heads=4, norm_eps=1e-5, vocab_size=512, head_dim=64, rope_theta=10000.0,
                 qk_norm=256, num_experts=8, num_experts_per_tok=2, norm_topk_prob=False, expert_gating_func=1)

@pytest.mark.parametrize("B", [2, 3, 8, 16, 11])
def test_batched_dense_decode(gpu, B):
  from tinygrad_amd.llm import BatchedTransformer, TransformerConfig, synth_state
  c = TransformerConfig(max_context=128, **SMALL)
  sd = synth_state(c, seed=1003)
  gpu.synchronize()
  host = {k: (b.numpy(), t, shp) for k, (b, t, shp) in sd.items()}
  rng = np.random.default_rng(B)
  prompts = [[int(t) for t in rng.integers(0, 512, size=66)] for _ in range(B)]          # past the first 64-position attention split
  _per_sequence_check(gpu, BatchedTransformer(c, sd, B, max_new=32), SMALL, host, prompts, 12, 128)

@pytest.mark.parametrize("path", ["jobs", "grouped"])
@pytest.mark.parametrize("B", [1, 2, 5, 8, 16])
def test_batched_olmoe_arch_decode(gpu, B, path):
  """Benchmark configuration 4's architecture (fp16 attention / router, MXFP4 experts, full-width q/k norm) at batch 1..16, with the experts as one
  GEMV per (sequence, slot) job and as one small-batch GEMM per selected expert."""
  from tinygrad_amd.llm import BatchedTransformer, TransformerConfig, synth_state_moe
  c = TransformerConfig(max_context=128, **SMALL_MOE)
  sd = synth_state_moe(c, seed=1004)
  gpu.synchronize()
  host = {k: (b.numpy(), t, shp) for k, (b, t, shp) in sd.items()}
  # top-k routing is discontinuous: a router logit gap below the rounding noise of the fp16 activations (about 1e-3 of the logit scale) may select
  # another expert on either side.  The prompts are drawn until the oracle's own run stays clear of such ties (gap reported), so that a
  # mismatch below is a defect and not a coin flip.
  rng = np.random.default_rng(10 + B)
  prompts, gaps, drawn = [], [], 0
  while len(prompts) < B and drawn < 40 * B:                        # (every sequence's prompt is drawn on its own: sixteen clear ones in one draw are rare)
    p = [int(t) for t in rng.integers(0, 512, size=12)]; drawn += 1
    o = ollm.Model(SMALL_MOE, host, 128, act_round_f16=False); o.generate(p, 16)
    if o.min_route_gap > 1.5e-3: prompts.append(p); gaps.append(o.min_route_gap)   # (router logits are O(1); fp16 rounding of the activations moves them by a few 1e-4)
  print(f"{drawn} prompts drawn for {B}: smallest router logit gap between the last selected and the first rejected expert {min(gaps):.4f}")
  assert len(prompts) == B
  model = BatchedTransformer(c, sd, B, max_new=32)
  model.expert_path = path
  if path == "grouped" and B > 8:                                   # (the job table of the grouped path holds eight rows per expert)
    with pytest.raises(ValueError, match="batch <= 8"): model.prefill(prompts, False)
    return
  _per_sequence_check(gpu, model, SMALL_MOE, host, prompts, 16, 128)

def test_batched_equals_single_sequence_path(gpu):
  """Sequence b of a batch produces the tokens the batch-1 Transformer produces for the same prompt."""
  from tinygrad_amd.llm import BatchedTransformer, Transformer, TransformerConfig, synth_state_moe
  c = TransformerConfig(max_context=128, **SMALL_MOE)
  sd = synth_state_moe(c, seed=5)
  rng = np.random.default_rng(77)
  prompts = [[int(t) for t in rng.integers(0, 512, size=9)] for _ in range(4)]
  got = list(BatchedTransformer(c, sd, 4, max_new=32).generate(prompts, 10))
  single = Transformer(c, sd, max_new=32)
  for b in range(4): assert [g[b] for g in got] == list(single.generate(prompts[b], 10)), b

GLM_LIKE = dict(num_blocks=3, dim=512, hidden_dim=256, n_heads=8, n_kv_heads=2, norm_eps=1e-5, vocab_size=512, head_dim=64, rope_theta=10000.0,
                num_experts=8, num_experts_per_tok=2, norm_topk_prob=True, expert_gating_func=2, routed_scaling_factor=1.5,
                leading_dense_blocks=1, dense_hidden_dim=768, shared_expert_dim=256, shared_expert_gate=True, expert_bias=True)

@pytest.mark.parametrize("B,gate", [(2, True), (5, True), (4, False)])
def test_batched_glm4moe_like_decode(gpu, B, gate):
  """A leading dense block, sigmoid gating with a selection bias, scaled normalised weights and a (gated or plain) shared expert, at batch 2..5."""
  from tinygrad_amd.llm import BatchedTransformer, TransformerConfig, synth_state_moe
  cfg = dict(GLM_LIKE, shared_expert_gate=gate)
  c = TransformerConfig(max_context=128, **cfg)
  sd = synth_state_moe(c, seed=1010)
  gpu.synchronize()
  host = {k: (b.numpy(), t, shp) for k, (b, t, shp) in sd.items()}
  # prompts clear of selection near-ties, as above.  The ranked quantity is sigmoid(logit) + bias here: a sigmoid passes on at most a quarter of
  # a logit's rounding noise, so the bar is a quarter of the one on router logits.
  bar = 4e-4
  for attempt in range(40):
    rng = np.random.default_rng(20 + B + 100 * attempt)
    prompts = [[int(t) for t in rng.integers(0, 512, size=12)] for _ in range(B)]
    gaps = []
    for p in prompts:
      o = ollm.Model(cfg, host, 128, act_round_f16=False); o.generate(p, 16); gaps.append(o.min_route_gap)
    if min(gaps) > bar: break
  print(f"prompt set {attempt}: smallest biased-score gap {min(gaps):.4f}")
  assert min(gaps) > bar
  model = BatchedTransformer(c, sd, B, max_new=32)
  assert [b["moe"] for b in model.blk] == [False, True, True]
  _per_sequence_check(gpu, model, cfg, host, prompts, 16, 128)
