"""numpy restatement of the MXFP8 operand format of the MoE grouped GEMM.  Test infrastructure only.

quantize_mxfp8 / mx_pack / _mx_block_scale: extra/gemm/cdna_asm_gemm.py:149-173 (test twin test/backend/test_asm_gemm.py:278-292).
E4M3 conversion: tinygrad/dtype.py:237-260 (round-to-nearest-even, finite saturation to 448, no infinities, NaN = 0x7f/0xff)."""
import numpy as np

def float_to_e4m3(x: np.ndarray) -> np.ndarray:
  """float -> E4M3 (fn) bits, RNE, saturating: |x| > 464 -> 448 (dtype.py:238-252: ovf_threshold 464, max_norm 0x7E)."""
  x = np.asarray(x, dtype=np.float64)
  sign = (np.signbit(x)).astype(np.uint8) << 7
  a = np.abs(x)
  nan = ~np.isfinite(x)
  a = np.where(nan, 0.0, a)
  with np.errstate(divide="ignore"):
    e = np.floor(np.log2(np.where(a > 0, a, 1.0)))
  e = np.clip(e, -6, 8)
  quantum = np.exp2(e - 3)
  q = np.rint(a / quantum) * quantum                      # RNE on the 3-bit mantissa grid (subnormal grid 2^-9 below 2^-6)
  q = np.where(a > 464.0, 448.0, np.minimum(q, 480.0))
  q = np.where(q > 448.0, 448.0, q)                        # (448, 464] rounds (ties-to-even) down to 448
  with np.errstate(divide="ignore"):
    e2 = np.floor(np.log2(np.where(q > 0, q, 1.0)))
  sub = q < 2.0 ** -6
  expf = np.where(sub, 0, e2 + 7).astype(np.int64)
  mant = np.where(sub, q / 2.0 ** -9, (q / np.exp2(e2) - 1.0) * 8).astype(np.int64)
  bits = (expf << 3 | mant).astype(np.uint8)
  bits = np.where(q == 0, 0, bits).astype(np.uint8)
  return np.where(nan, np.uint8(0x7f), bits) | sign

def e4m3_to_float(b: np.ndarray) -> np.ndarray:
  b = np.asarray(b, dtype=np.uint8)
  s = np.where(b & 0x80, -1.0, 1.0)
  e = ((b >> 3) & 0xF).astype(np.int64); m = (b & 7).astype(np.float64)
  v = np.where(e == 0, m * 2.0 ** -9, (1.0 + m / 8.0) * np.exp2(e - 7.0))
  v = np.where((b & 0x7f) == 0x7f, np.nan, v)
  return (s * v).astype(np.float32)

def quantize_mxfp8(x: np.ndarray):
  """cdna_asm_gemm.py:149-159: per 32 block along the last axis, e8 = clamp(floor(log2(max(amax, 1e-38))) + 127, 0, 254),
  q = e4m3(clamp(x * 2^(127 - e8), +-448)).  Returns (q bits uint8 (.., K), e8 uint8 (.., K/32))."""
  x = np.asarray(x, dtype=np.float32)
  *batch, K = x.shape
  xb = x.reshape(*batch, K // 32, 32)
  amax = np.abs(xb).max(axis=-1)
  e8 = np.clip(np.floor(np.log2(np.maximum(amax, np.float32(1e-38)).astype(np.float32))) + 127, 0, 254).astype(np.uint8)
  qscale = np.exp2(127.0 - e8.astype(np.float32)).astype(np.float32)[..., None]
  xs = np.clip(xb * qscale, -448.0, 448.0)
  return float_to_e4m3(xs).reshape(*batch, K), e8

def silu_mul_quantize_mxfp8(x_w1: np.ndarray, x_w3: np.ndarray):
  """extra/llama_kernels/fused_silu_mul_quantize_mxfp8/__init__.py:33-44: act = w1 * (1 / (1 + exp2(-w1 * log2 e))) * w3 in float32, then
  quantize_mxfp8 of act."""
  w1, w3 = np.asarray(x_w1, dtype=np.float32), np.asarray(x_w3, dtype=np.float32)
  with np.errstate(over="ignore"): sig = (np.float32(1.0) / (np.float32(1.0) + np.exp2(w1 * np.float32(-1.4426950408889634)))).astype(np.float32)
  return quantize_mxfp8((w1 * sig * w3).astype(np.float32))

def transpose_quantize_mxfp8(g: np.ndarray):
  """extra/llama_kernels/transpose_quantize_mxfp8/__init__.py:24-25: "(q, e8, si) == quantize_mxfp8(g.T)" for g (M, N): q (N, M), e8 (N, M/32),
  si = mx_pack(e8) (M/128, N)."""
  q, e8 = quantize_mxfp8(np.ascontiguousarray(np.asarray(g, dtype=np.float32).T))
  return q, e8, (mx_pack(e8) if e8.shape[1] % 4 == 0 else None)

def block_scale(e8: np.ndarray) -> np.ndarray:
  """cdna_asm_gemm.py:165-173: dequant scale 2^(e8-127) broadcast to element shape."""
  return np.repeat(np.exp2(e8.astype(np.float32) - 127.0).astype(np.float32), 32, axis=-1)

def dequant_mxfp8(q: np.ndarray, e8: np.ndarray) -> np.ndarray:
  return e4m3_to_float(q) * block_scale(e8)

def mx_pack(e8: np.ndarray) -> np.ndarray:
  """cdna_asm_gemm.py:161-163: (rows, K/32) u8 -> (K/128, rows) u32, 4 consecutive block scales little-endian, transposed."""
  rows, sk = e8.shape
  return np.ascontiguousarray(np.ascontiguousarray(e8).reshape(rows, sk // 4, 4).view(np.uint32).reshape(rows, sk // 4).T)

def mx_pack_3d(e8: np.ndarray) -> np.ndarray:
  """extra/gemm/moe_gemm.py:87-89: (E, rows, K/32) -> (E, K/128, rows) u32."""
  return np.stack([mx_pack(e) for e in e8])

def to_bf16(x: np.ndarray) -> np.ndarray:
  """float32 -> bfloat16 (RNE) kept as float32 values (tinygrad/dtype.py:224-226)."""
  u = np.asarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
  u = ((u + 0x7FFF + ((u >> 16) & 1)) & 0xFFFF0000).astype(np.uint32)
  return u.view(np.float32)

def tile_experts(expert_off, M: int) -> np.ndarray:
  """Routing.rows_e (extra/gemm/moe_routing.py:98-104) per 256-row tile: expert = #(off[:E] <= 256 t) - 1, i.e. the last expert whose offset
  is <= the tile's first row; the tiles at or beyond off[E] therefore belong to expert E - 1."""
  off = np.asarray(expert_off).reshape(-1)
  E = off.shape[0] - 1
  tr = np.arange(M // 256) * 256
  return ((tr[:, None] >= off[None, :E]).sum(-1) - 1).astype(np.int32)

def grouped_mx_gemm_ref(x_q, x_e8, w_q, w_e8, expert_off):
  """Semantic definition of grouped_mx_gemm (extra/gemm/moe_gemm.py:112-134) through the reference's non-grouped fallback
  matmul_mx (examples/mlperf/models/gpt_oss.py:64-83): bf16(dequant x) @ bf16(dequant w[e])^T accumulated in float, stored as
  bf16, where e is the expert of the row's 256-row tile (tile_experts above; the kernel indexes B by tile, moe_gemm.py:36-48).
  Returned as float32 holding bf16 values."""
  xd = to_bf16(dequant_mxfp8(x_q, x_e8)).astype(np.float64)
  M, N = x_q.shape[0], w_q.shape[1]
  out = np.zeros((M, N), dtype=np.float32)
  te = tile_experts(expert_off, M)
  for e in np.unique(te):
    rows = np.repeat(te == e, 256)
    wd = to_bf16(dequant_mxfp8(w_q[e], w_e8[e])).astype(np.float64)
    out[rows] = to_bf16((xd[rows] @ wd.T).astype(np.float32))
  return out

def add_expert_bias(h_bf16: np.ndarray, bias: np.ndarray, expert_off: np.ndarray) -> np.ndarray:
  """examples/mlperf/models/gpt_oss.py:219-224: h + (onehot(rows_e) @ bias.float()).cast(bf16) as a bf16 tensor add; h holds bf16 values as
  float32.  rows_e gives the tiles at or beyond expert_off[E] to the last expert."""
  out = np.array(h_bf16, dtype=np.float32, copy=True)
  rows_e = np.repeat(tile_experts(expert_off, out.shape[0]), 256)
  return to_bf16(out + to_bf16(bias)[rows_e])

def swiglu_interleaved(h_bf16: np.ndarray, limit: float = 7.0, alpha: float = 1.702) -> np.ndarray:
  """swiglu of examples/mlperf/models/gpt_oss.py:94-98 on a bf16 tensor (values held as float32): glu = h[..., ::2].clamp(max=limit),
  lin = h[..., 1::2].clamp(-limit, limit), (glu * sigmoid(alpha * glu)) * (lin + 1); every elementwise result is a bf16 tensor, so each
  step rounds to bf16 (the sigmoid counted as one step)."""
  h = np.asarray(h_bf16, dtype=np.float32)
  glu, lin = np.minimum(h[..., ::2], np.float32(limit)), np.clip(h[..., 1::2], -np.float32(limit), np.float32(limit))
  sg = to_bf16(np.float32(1.0) / (np.float32(1.0) + np.exp(-to_bf16(np.float32(alpha) * glu))))
  return to_bf16(to_bf16(glu * sg) * to_bf16(lin + np.float32(1.0)))

def matmul_mx(x_bf16: np.ndarray, w_q: np.ndarray, w_e8: np.ndarray) -> np.ndarray:
  """examples/mlperf/models/gpt_oss.py:64-83, the non-ASM branch: quant_dequant_mx(x) @ dequant_weight(w).T -> bf16 (bf16 values as float32)."""
  xq, xe = quantize_mxfp8(x_bf16)
  xd = to_bf16(dequant_mxfp8(xq, xe)).astype(np.float64)
  wd = to_bf16(dequant_mxfp8(w_q, w_e8)).astype(np.float64)
  return to_bf16((xd @ wd.T).astype(np.float32))

def moe_feed_forward_loop(inp_bf16, logits, k, w_gate_up, w_gate_up_e8, b_gate_up, w_down, w_down_e8, b_down, limit: float = 7.0):
  """The reference's per-expert loop, examples/mlperf/models/gpt_oss.py:227-238 (the definition the grouped branch :213-226 must agree with):
  weights = softmax over the logits at or above the k-th largest, out = sum_e bf16(weights[:, e]) * (matmul_mx(swiglu(matmul_mx(inp, gu_e) +
  b_gu[e]), dn_e) + b_dn[e]), every tensor bf16.  inp (T, D) bf16 values; returns (T, D) bf16 values as float32."""
  T, E = logits.shape
  thresh = np.sort(logits, axis=-1)[:, E - k][:, None]
  masked = np.where(logits >= thresh, logits, -np.inf).astype(np.float32)
  ex = np.exp(masked - masked.max(-1, keepdims=True)); wts = (ex / ex.sum(-1, keepdims=True)).astype(np.float32)
  out = None
  for e in range(E):
    gate_up = to_bf16(matmul_mx(inp_bf16, w_gate_up[e], w_gate_up_e8[e]) + to_bf16(b_gate_up[e])[None, :])
    y = to_bf16(matmul_mx(swiglu_interleaved(gate_up, limit), w_down[e], w_down_e8[e]) + to_bf16(b_down[e])[None, :])
    contrib = to_bf16(to_bf16(wts[:, e:e + 1]) * y)
    out = contrib if out is None else to_bf16(out + contrib)
  return out
