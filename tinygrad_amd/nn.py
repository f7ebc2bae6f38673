"""QuantLinear: nn.Linear.__call__ (tinygrad/nn/__init__.py:177, `x.linear(self.weight.transpose(), self.bias)`) for a weight
that stays in its packed GGUF block layout.  The weight operand is the raw tensor byte range from the GGUF file buffer
(tinygrad/llm/gguf.py:144-148: rows = out_features, quant blocks along in_features); nothing is repacked or dequantized to memory."""
from __future__ import annotations
import ctypes
import numpy as np
from tinygrad_amd import runtime as rt
from tinygrad_amd.runtime import Buffer, GGML_QUANT

class QuantLinear:
  def __init__(self, blocks: Buffer, ggml_type: int, out_features: int, in_features: int):
    if ggml_type != rt.F16 and ggml_type not in GGML_QUANT: raise ValueError(f"GGML type '{ggml_type}' is not supported!")
    nel, nby = GGML_QUANT.get(ggml_type, (64, 128))                     # dense fp16 rows go in 64-element units
    assert in_features % nel == 0, f"in_features {in_features} must be a multiple of the block size {nel}"
    assert blocks.nbytes >= out_features * (in_features // nel) * nby, "weight buffer too small"
    self.blocks, self.ggml_type, self.out_features, self.in_features = blocks, ggml_type, out_features, in_features

  @property
  def nbytes(self) -> int:
    nel, nby = GGML_QUANT.get(self.ggml_type, (64, 128))
    return self.out_features * (self.in_features // nel) * nby

  def __call__(self, x: Buffer, out: Buffer | None = None, out_dtype=None, stream=None) -> Buffer:
    """x: (..., in_features) float16 or float32 with at most 8 rows (up to 16 for prefill chunks).  Returns (rows, out_features); the caller may pass `out`."""
    assert x.shape[-1] == self.in_features, f"{x.shape} vs in_features {self.in_features}"
    m = int(np.prod(x.shape[:-1], dtype=np.int64)) if len(x.shape) > 1 else 1
    assert 1 <= m <= 128, f"batch of {m} rows is outside the range 1..128"
    if out is None: out = Buffer((*x.shape[:-1], self.out_features), out_dtype or x.dtype)
    assert out.nbytes == m * self.out_features * out.dtype.itemsize
    rt.check(rt.lib().tga_qlinear(self.ggml_type, self.blocks.ptr, x.ptr, rt.dtype_code(x.dtype), out.ptr, rt.dtype_code(out.dtype),
                                  m, self.out_features, self.in_features, stream))
    return out

def qlinear_mixed(layers: list[QuantLinear], x: Buffer, outs: list[Buffer], norm: tuple[Buffer, float], stream=None):
  """Layers of different block types over the same float32 row x with RMSNorm(x) * weight folded in (Q4_K attn_q / attn_k beside a Q6_K attn_v): one launch
  per run of equal types, a single launch for the pairs the two-set kernel serves."""
  nseg, k = len(layers), layers[0].in_features
  assert all(l.in_features == k for l in layers) and x.dtype == np.float32 and len(outs) == nseg
  VP = ctypes.c_void_p * nseg
  rt.check(rt.lib().tga_rmsnorm_qlinear_mixed(norm[0].ptr, norm[1], nseg, (ctypes.c_int32 * nseg)(*[l.ggml_type for l in layers]), VP(*[l.blocks.ptr for l in layers]),
                                              VP(*[o.ptr for o in outs]), (ctypes.c_int64 * nseg)(*[l.out_features for l in layers]), x.ptr, rt.dtype_code(outs[0].dtype), k, stream))
  return outs

def qlinear_multi(layers: list[QuantLinear], x: Buffer, outs: list[Buffer], epilogue: int = 0, resid: list[Buffer] | None = None, stream=None,
                  x_staged: bool = False, stage_out_for: QuantLinear | None = None, norm: tuple[Buffer, float] | None = None,
                  combine: tuple[Buffer, Buffer, int, Buffer] | None = None, touch: tuple | None = None):
  """Several QuantLinear layers over the same activation in one launch (attn_q/k/v, ffn_gate/ffn_up).
  epilogue 0: plain; 1: outs[i] = resid[i] + linear; 2: outs[0] = silu(layers[0](x)) * layers[1](x).
  x_staged: x is already in the staged order of these weights (stage_activation or a staging producer).
  stage_out_for: write the single fp16 output in the staged order of that consumer layer.
  norm = (weight, eps): x is one float32 row and RMSNorm(x) * weight is applied while the kernel stages it; norm = (weight, eps, scratch) for several
  float32 rows (scratch: an fp16 buffer of x's shape that receives the normalised rows when the kernel at hand cannot fold the norm).
  combine = (y, probs, k, x_out) with norm: the row is first completed as x + sum_j probs[j] * y[j] (the MoE weighted sum + residual) and
  the completed row is written to x_out (a buffer other than x).
  touch = (state, cache_k, cache_v, rope table, n_kv_heads, head_dim, max_context) with norm: the launch also touches what the attention launch behind it reads first."""
  nseg = len(layers)
  t, k = layers[0].ggml_type, layers[0].in_features
  assert all(l.ggml_type == t and l.in_features == k for l in layers)
  m = int(np.prod(x.shape[:-1], dtype=np.int64)) if len(x.shape) > 1 else 1
  VP = ctypes.c_void_p * nseg
  w = VP(*[l.blocks.ptr for l in layers])
  y = VP(*[(outs[i].ptr if i < len(outs) else None) for i in range(nseg)])
  n = (ctypes.c_int64 * nseg)(*[l.out_features for l in layers])
  r = VP(*[b.ptr for b in resid]) if resid is not None else None
  ydt = rt.dtype_code(outs[0].dtype)
  so = stage_out_for
  if combine is not None:
    assert norm is not None and m == 1 and x.dtype == np.float32 and not x_staged and epilogue == 0 and so is None and combine[3].ptr != x.ptr
    rt.check(rt.lib().tga_moe_combine_rmsnorm_qlinear_multi(combine[0].ptr, combine[1].ptr, combine[2], x.ptr, combine[3].ptr, norm[0].ptr, norm[1],
                                                            t, nseg, w, y, n, ydt, k, stream))
    return outs
  if norm is not None and len(norm) == 3:                                # rows with a scratch: one launch where the LDS-fed kernel folds the norm in, else norm + linears
    assert x.dtype == np.float32 and not x_staged and so is None and len(norm) == 3, "norm = (weight, eps, fp16 scratch of x's shape) for several rows"
    rt.check(rt.lib().tga_rmsnorm_qlinear_rows(norm[0].ptr, norm[1], t, nseg, w, y, n, x.ptr, norm[2].ptr, ydt, m, k, epilogue, r, stream))
    return outs
  if norm is not None and touch is not None and so is None:              # touch = (state, cache_k, cache_v, rope table, n_kv_heads, head_dim, max_context)
    assert m == 1 and x.dtype == np.float32 and not x_staged
    rt.check(rt.lib().tga_rmsnorm_qlinear_multi_touch(norm[0].ptr, norm[1], t, nseg, w, y, n, x.ptr, ydt, k, epilogue, r, touch[0].ptr, touch[1].ptr, touch[2].ptr, touch[3].ptr,
                                                      touch[4], touch[5], touch[6], stream))
    return outs
  if norm is not None:
    assert m == 1 and x.dtype == np.float32 and not x_staged
    rt.check(rt.lib().tga_rmsnorm_qlinear_multi(norm[0].ptr, norm[1], t, nseg, w, y, n, x.ptr, ydt, k, epilogue, r,
                                                so.ggml_type if so is not None else 0, so.in_features if so is not None else 0, stream))
    return outs
  rt.check(rt.lib().tga_qlinear_multi(t, nseg, w, y, n, x.ptr, rt.F16_STAGED if x_staged else rt.dtype_code(x.dtype), ydt, m, k, epilogue, r,
                                      so.ggml_type if so is not None else 0, so.in_features if so is not None else 0, stream))
  return outs

class ExpertWeights:
  """Like QuantLinear but with a num_experts dimension: weight (num_experts, out_features, in_features) kept in GGUF blocks
  (mirror of ExpertWeights, tinygrad/llm/model.py:21-27).  __call__(sel, x): sel (n_jobs,) int32 device buffer of expert ids,
  x (n_jobs // jobs_per_x_row, in) -> (n_jobs, out)."""
  def __init__(self, blocks: Buffer, ggml_type: int, num_experts: int, out_features: int, in_features: int):
    if ggml_type != rt.F16 and ggml_type not in GGML_QUANT: raise ValueError(f"GGML type '{ggml_type}' is not supported!")
    self.blocks, self.ggml_type, self.num_experts, self.out_features, self.in_features = blocks, ggml_type, num_experts, out_features, in_features

  @property
  def expert_nbytes(self) -> int:
    if self.ggml_type == rt.F16: return 2 * self.out_features * self.in_features
    nel, nby = GGML_QUANT[self.ggml_type]
    return self.out_features * (self.in_features // nel) * nby

  def __call__(self, sel: Buffer, x: Buffer, out: Buffer, jobs_per_x_row: int = 1, up: "ExpertWeights | None" = None, stream=None,
               route: tuple[Buffer, int, bool, float, Buffer] | None = None) -> Buffer:
    """route = (logits, gating, norm_topk_prob, scale, probs_out) with `up`: the jobs are gated inside the launch from the router logits (one row per
    token, jobs_per_x_row = k jobs each); sel and probs_out receive the selection."""
    n_jobs = int(np.prod(sel.shape))
    if route is not None:
      assert up is not None and x.dtype == np.float16 and n_jobs % jobs_per_x_row == 0
      if jobs_per_x_row == n_jobs:
        rt.check(rt.lib().tga_qlinear_experts_routed(self.ggml_type, self.blocks.ptr, up.blocks.ptr, self.num_experts, route[0].ptr, n_jobs, route[1], int(route[2]),
                                                     route[3], sel.ptr, route[4].ptr, x.ptr, out.ptr, rt.dtype_code(out.dtype), self.out_features, self.in_features, stream))
      else:                                                              # several tokens: jobs_per_x_row = k jobs each, gated from their own row of the logits
        rt.check(rt.lib().tga_qlinear_experts_routed_rows(self.ggml_type, self.blocks.ptr, up.blocks.ptr, self.num_experts, route[0].ptr, n_jobs // jobs_per_x_row,
                                                          jobs_per_x_row, route[1], int(route[2]), route[3], sel.ptr, route[4].ptr, x.ptr, out.ptr, rt.dtype_code(out.dtype),
                                                          self.out_features, self.in_features, stream))
      return out
    rt.check(rt.lib().tga_qlinear_experts(self.ggml_type, self.blocks.ptr, up.blocks.ptr if up is not None else None, self.num_experts, sel.ptr, n_jobs,
                                          jobs_per_x_row, x.ptr, rt.dtype_code(x.dtype), out.ptr, rt.dtype_code(out.dtype), self.out_features, self.in_features, stream))
    return out

def moe_gate(logits: Buffer, n_tokens: int, n_experts: int, k: int, sel: Buffer, probs: Buffer, gating: int = 1, norm_topk_prob: bool = False, scale: float = 1.0, stream=None,
             bias: Buffer | None = None):
  """bias: the float32 expert selection bias (`exp_probs_b`, model.py:113): ranks by score + bias, weights from the scores."""
  if bias is not None:
    rt.check(rt.lib().tga_moe_gate_biased(logits.ptr, bias.ptr, n_tokens, n_experts, k, gating, int(norm_topk_prob), scale, sel.ptr, probs.ptr, stream))
  else: rt.check(rt.lib().tga_moe_gate(logits.ptr, n_tokens, n_experts, k, gating, int(norm_topk_prob), scale, sel.ptr, probs.ptr, stream))

def moe_router(x: Buffer, norm_weight: Buffer | None, eps: float, router: QuantLinear, k: int, sel: Buffer, probs: Buffer, logits_ws: Buffer,
               xn_out: Buffer | None = None, gating: int = 1, norm_topk_prob: bool = False, scale: float = 1.0, stream=None):
  """ffn_norm + router logits + gating + top-k of one token in one launch (dense fp16 router weight).  k = 0: logits only (sel / probs None).
  logits_ws: n_experts + 1 float32, zero before the first use (the last word is an arrival counter)."""
  assert router.ggml_type == rt.F16 and logits_ws.nbytes >= 4 * (router.out_features + 1)
  rt.check(rt.lib().tga_moe_router(x.ptr, norm_weight.ptr if norm_weight is not None else None, eps, router.blocks.ptr, router.in_features, router.out_features, k,
                                   gating, int(norm_topk_prob), scale, xn_out.ptr if xn_out is not None else None, logits_ws.ptr,
                                   sel.ptr if sel is not None else None, probs.ptr if probs is not None else None, stream))

def moe_combine(y: Buffer, probs: Buffer, resid: Buffer | None, n_tokens: int, k: int, dim: int, out: Buffer, stream=None):
  rt.check(rt.lib().tga_moe_combine(y.ptr, probs.ptr, resid.ptr if resid is not None else None, n_tokens, k, dim, out.ptr, stream))

def stage_activation(layer: QuantLinear, x: Buffer, out: Buffer | None = None, stream=None) -> Buffer:
  """fp16 copy of one activation row in the order `layer`'s M = 1 GEMV consumes (a permutation of the row)."""
  out = out if out is not None else Buffer((1, layer.in_features), np.float16)
  rt.check(rt.lib().tga_stage_activation(layer.ggml_type, x.ptr, rt.dtype_code(x.dtype), layer.in_features, out.ptr, stream))
  return out

def expert_jobs(sel: Buffer, n_experts: int, table: Buffer, flags: Buffer, stream=None):
  """Groups the (token, slot) jobs of a batch by expert (table: n_experts x 16 int32; flags: one int32 the caller zeroed)."""
  rt.check(rt.lib().tga_expert_jobs(sel.ptr, int(np.prod(sel.shape)), n_experts, table.ptr, flags.ptr, stream))

def experts_grouped(w: ExpertWeights, table: Buffer, n_jobs: int, x: Buffer, out: Buffer, jobs_per_x_row: int = 1, up: ExpertWeights | None = None, stream=None) -> Buffer:
  """ExpertWeights.__call__ for a batch with every selected expert streamed once (tga_qlinear_experts_grouped): x fp16 rows, job j reads row
  j // jobs_per_x_row and writes row j of out (n_jobs, out_features); with `up`, out = silu(gate) * up."""
  assert x.dtype == np.float16 and x.shape[-1] == w.in_features
  rt.check(rt.lib().tga_qlinear_experts_grouped(w.ggml_type, w.blocks.ptr, up.blocks.ptr if up is not None else None, w.num_experts, table.ptr, n_jobs, jobs_per_x_row,
                                                x.ptr, out.ptr, rt.dtype_code(out.dtype), w.out_features, w.in_features, stream))
  return out
