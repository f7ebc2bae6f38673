"""MXFP8 MoE grouped-GEMM path behind the reference's names (extra/gemm/moe_routing.py, extra/gemm/moe_gemm.py,
extra/gemm/cdna_asm_gemm.py): route / dispatch / combine, quantize_mxfp8, grouped_mx_gemm.  bf16 and E4M3 tensors are device
Buffers of uint16 / uint8 (numpy has neither type); shapes follow the reference."""
from __future__ import annotations
from dataclasses import dataclass
import numpy as np
from tinygrad_amd import runtime as rt
from tinygrad_amd.runtime import Buffer

BLOCK_ROW = 256

def m_max_for(t_local: int, experts_per_tok: int, n_experts: int) -> int:          # moe_routing.py:89-90
  return (-(-t_local * experts_per_tok // BLOCK_ROW) + n_experts) * BLOCK_ROW

def to_bf16_bits(x: np.ndarray) -> np.ndarray:
  u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
  return (((u + 0x7FFF + ((u >> 16) & 1)) >> 16) & 0xFFFF).astype(np.uint16)

def from_bf16_bits(b: np.ndarray) -> np.ndarray:
  return (np.ascontiguousarray(b).astype(np.uint32) << 16).view(np.float32)

@dataclass
class Routing:
  """moe_routing.py:92-96 (one device group)."""
  weights: Buffer      # (T, k) float32
  dest_row: Buffer     # (T*k,) int32
  off: Buffer          # (E+1,) int32
  m_l: int
  t_local: int
  topi: Buffer         # (T, k) int32
  counts: Buffer       # (E,) int32

def route(logits: Buffer, experts_per_tok: int, n_experts: int, stream=None, out: Routing | None = None) -> Routing:
  """moe_routing.py:109-122.  out: a Routing whose buffers are reused; the call then allocates nothing at all (tga_moe_route_static keeps its
  workspace inside the library), e.g. while a HIP graph is being captured."""
  T, E = logits.shape
  assert E == n_experts
  k = experts_per_tok
  if out is not None:
    assert out.weights.shape == (T, k) and out.off.shape == (E + 1,)
    rt.check(rt.lib().tga_moe_route_static(logits.ptr, T, E, k, out.weights.ptr, out.topi.ptr, out.dest_row.ptr, out.off.ptr, out.counts.ptr, stream))
    return out
  w, topi, dest, off, cnt = Buffer((T, k), np.float32), Buffer((T, k), np.int32), Buffer((T * k,), np.int32), Buffer((E + 1,), np.int32), Buffer((E,), np.int32)
  scratch = Buffer((T * k + ((T * k + 1023) // 1024) * E,), np.int32)
  rt.check(rt.lib().tga_moe_route(logits.ptr, T, E, k, w.ptr, topi.ptr, dest.ptr, off.ptr, cnt.ptr, scratch.ptr, stream))
  r = Routing(w, dest, off, m_max_for(T, k, E), T, topi, cnt)
  r._scratch = scratch                                                            # keep alive until the stream has run
  return r

def dispatch(x: Buffer, r: Routing, stream=None, out: Buffer | None = None) -> Buffer:
  """x (T, D) bf16 bits -> xg (m_l, D) bf16 bits."""
  T, D = x.shape
  k = r.dest_row.shape[0] // T
  xg = out if out is not None else Buffer((r.m_l, D), np.uint16)
  rt.check(rt.lib().tga_moe_dispatch(x.ptr, r.dest_row.ptr, r.off.ptr, r.counts.ptr, T, k, r.off.shape[0] - 1, r.m_l, D, xg.ptr, stream))
  return xg

def combine(y: Buffer, r: Routing, n_tokens: int, experts_per_tok: int, stream=None, out: Buffer | None = None) -> Buffer:
  D = y.shape[-1]
  o = out if out is not None else Buffer((n_tokens, D), np.uint16)
  rt.check(rt.lib().tga_moe_combine_rows(y.ptr, r.dest_row.ptr, r.weights.ptr, n_tokens, experts_per_tok, D, o.ptr, stream))
  return o

def quantize_mxfp8(x: Buffer, stream=None):
  """cdna_asm_gemm.py:149-159: x (rows, K) bf16 bits (uint16) or float32 -> (q uint8 (rows,K), e8 uint8 (rows,K/32), packed uint32 (K/128, rows) or None)."""
  rows, K = x.shape
  q, e8 = Buffer((rows, K), np.uint8), Buffer((rows, K // 32), np.uint8)
  packed = Buffer((K // 128, rows), np.uint32) if K % 128 == 0 else None
  rt.check(rt.lib().tga_quantize_mxfp8(x.ptr, int(x.dtype == np.uint16), rows, K, q.ptr, e8.ptr, packed.ptr if packed is not None else None, stream))
  return q, e8, packed

def fused_silu_mul_quantize_mxfp8(x_w1: Buffer, x_w3: Buffer, stream=None):
  """extra/llama_kernels/fused_silu_mul_quantize_mxfp8/__init__.py:91-104: (rows, K) bf16 bits x 2 -> MXFP8 of silu(x_w1) * x_w3,
  same outputs as quantize_mxfp8 (the SwiGLU product never goes through memory)."""
  assert x_w1.shape == x_w3.shape and x_w1.dtype == np.uint16 and x_w3.dtype == np.uint16, f"{x_w1.shape} != {x_w3.shape}"
  rows, K = x_w1.shape
  q, e8 = Buffer((rows, K), np.uint8), Buffer((rows, K // 32), np.uint8)
  packed = Buffer((K // 128, rows), np.uint32) if K % 128 == 0 else None
  rt.check(rt.lib().tga_silu_mul_quantize_mxfp8(x_w1.ptr, x_w3.ptr, rows, K, q.ptr, e8.ptr, packed.ptr if packed is not None else None, stream))
  return q, e8, packed

def transpose_quantize_mxfp8(g: Buffer, stream=None):
  """extra/llama_kernels/transpose_quantize_mxfp8/__init__.py:24-37: g (M, N) bf16 bits -> (q, e8, si) == quantize_mxfp8(g.T): q uint8 (N, M),
  e8 uint8 (N, M/32), si uint32 (M/128, N) (None when M % 128 != 0); the transposed tensor is never formed."""
  assert len(g.shape) == 2 and g.dtype == np.uint16, f"{g.shape} {g.dtype}"
  M, N = g.shape
  assert M % 32 == 0 and N % 64 == 0, f"M={M} must%32, N={N} must%64"
  q, e8 = Buffer((N, M), np.uint8), Buffer((N, M // 32), np.uint8)
  packed = Buffer((M // 128, N), np.uint32) if M % 128 == 0 else None
  rt.check(rt.lib().tga_transpose_quantize_mxfp8(g.ptr, M, N, q.ptr, e8.ptr, packed.ptr if packed is not None else None, stream))
  return q, e8, packed

def grouped_mx_gemm(x: Buffer | tuple, w: tuple[Buffer, Buffer], expert_off: Buffer, stream=None, out: Buffer | None = None, routed_only: bool = False,
                    counts: Buffer | None = None) -> Buffer:
  """moe_gemm.py:112-134 with pre-quantized weights w = (w_q (E,N,K) e4m3 bits, w_e8 (E,N,K/32)): quantizes x (M,K) bf16 to MXFP8 and
  runs the grouped GEMM; returns (M, N) bf16 bits.  x may also be an already quantized (x_q, x_e8) pair (a producer that quantizes for itself,
  e.g. fused_silu_mul_quantize_mxfp8).  routed_only: skip the tiles at or beyond expert_off[E] (their rows of the result are not written);
  the default writes every tile as the reference does.  counts (with routed_only): the routed rows per expert - padding rows inside an expert's
  range are not multiplied and come out as zeros."""
  w_q, w_e8 = w
  E, N, K2 = w_q.shape
  M, K = x[0].shape if isinstance(x, tuple) else x.shape
  assert K == K2, f"shape mismatch {(M, K)} {w_q.shape}"
  assert M % 256 == 0 and N % 256 == 0 and K % 128 == 0, f"grouped mxfp8 needs M%256,N%256,K%128, got {(M, K)} {w_q.shape}"   # moe_gemm.py:120
  x_q, x_e8, x_si = (x[0], x[1], None) if isinstance(x, tuple) else quantize_mxfp8(x, stream)
  o = out if out is not None else Buffer((M, N), np.uint16)
  if routed_only and counts is not None:
    rt.check(rt.lib().tga_grouped_mxfp8_gemm_counts(o.ptr, x_q.ptr, w_q.ptr, x_e8.ptr, w_e8.ptr, expert_off.ptr, counts.ptr, M, N, K, E, stream))
  elif routed_only: rt.check(rt.lib().tga_grouped_mxfp8_gemm_routed(o.ptr, x_q.ptr, w_q.ptr, x_e8.ptr, w_e8.ptr, expert_off.ptr, M, N, K, E, stream))
  else: rt.check(rt.lib().tga_grouped_mxfp8_gemm(o.ptr, x_q.ptr, w_q.ptr, x_si.ptr if x_si is not None else None, None, x_e8.ptr, w_e8.ptr, expert_off.ptr, M, N, K, E, stream))
  o._keep = (x_q, x_e8, x_si)
  return o

def mx_gemm(x: Buffer, w: tuple[Buffer, Buffer], stream=None, out: Buffer | None = None) -> Buffer:
  """The dense MXFP8 GEMM (hk_mxfp8_gemm, extra/gemm/cdna_asm_gemm.py:91-110): x (M, K) bf16 bits is quantized to MXFP8 and multiplied with
  w = (w_q (N, K) e4m3 bits, w_e8 (N, K/32)) -> (M, N) bf16 bits.  One expert that owns every row: the grouped kernel with E = 1."""
  w_q, w_e8 = w
  (N, K), M = w_q.shape, x.shape[0]
  off = Buffer.from_numpy(np.array([0, M], dtype=np.int32))
  o = grouped_mx_gemm(x, (w_q.view(0, (1, N, K), np.uint8), w_e8.view(0, (1, N, K // 32), np.uint8)), off, stream, out)
  o._keep = (*o._keep, off)
  return o

def add_expert_bias(h: Buffer, bias: Buffer, expert_off: Buffer, stream=None) -> Buffer:
  """`+ (onehot @ bias.float()).cast(bf16)` after a grouped GEMM (examples/mlperf/models/gpt_oss.py:219-224), in place on h (M, N) bf16 bits;
  bias (E, N) float32."""
  M, N = h.shape
  rt.check(rt.lib().tga_add_expert_bias(h.ptr, bias.ptr, expert_off.ptr, M, N, bias.shape[0], stream))
  return h

def swiglu(h: Buffer, limit: float = 7.0, alpha: float = 1.702, stream=None) -> Buffer:
  rows, two_i = h.shape
  y = Buffer((rows, two_i // 2), np.uint16)
  rt.check(rt.lib().tga_swiglu_interleaved(h.ptr, rows, two_i, limit, alpha, y.ptr, stream))
  return y

def moe_feed_forward(inp: Buffer, logits: Buffer, experts_per_tok: int, w_gate_up: tuple[Buffer, Buffer], b_gate_up: Buffer, w_down: tuple[Buffer, Buffer], b_down: Buffer,
                     swiglu_limit: float = 7.0, stream=None, routed_only: bool = True) -> Buffer:
  """The grouped MoE feed-forward of examples/mlperf/models/gpt_oss.py:213-226, from the normed activations on:
    r = route(logits); xg = dispatch(inp, r); h = grouped_mx_gemm(xg, w_gate_up, r.off) + bias_gate_up[rows_e]; y = swiglu(h);
    z = grouped_mx_gemm(y, w_down, r.off) + bias_down[rows_e]; out = combine(z, r)
  inp (T, D) bf16 bits, logits (T, E) float32, w_gate_up = (q (E, 2I, D), e8 (E, 2I, D/32)), b_gate_up (E, 2I) float32, w_down = (q (E, D, I), e8),
  b_down (E, D) float32 -> (T, D) bf16 bits.  D, 2I and I must be multiples of 256 (the reference pads to that, gpt_oss.py:85-92; the
  padding is not built here).  routed_only: the two GEMMs skip the tiles beyond the routed rows, which combine never reads."""
  T, D = inp.shape
  E, N2, _ = w_gate_up[0].shape
  assert D % 256 == 0 and N2 % 256 == 0 and (N2 // 2) % 256 == 0, f"dim {D}, 2*inter {N2} and inter {N2 // 2} must be multiples of 256"
  r = route(logits, experts_per_tok, E, stream)
  xg = dispatch(inp, r, stream)
  cnt = r.counts if routed_only else None                     # padding rows are never gathered by combine: their 16-row groups are not multiplied
  h = add_expert_bias(grouped_mx_gemm(xg, w_gate_up, r.off, stream, routed_only=routed_only, counts=cnt), b_gate_up, r.off, stream)
  y = swiglu(h, swiglu_limit, stream=stream)
  z = add_expert_bias(grouped_mx_gemm(y, w_down, r.off, stream, routed_only=routed_only, counts=cnt), b_down, r.off, stream)
  out = combine(z, r, T, experts_per_tok, stream)
  out._keep = (r, xg, h, y, z)                                                  # alive until the stream has run
  return out
