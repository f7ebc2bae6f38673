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
    if ggml_type not in GGML_QUANT: raise ValueError(f"GGML type '{ggml_type}' is not supported!")
    nel, nby = GGML_QUANT[ggml_type]
    assert in_features % nel == 0, f"in_features {in_features} must be a multiple of the block size {nel}"
    assert blocks.nbytes >= out_features * (in_features // nel) * nby, "weight buffer too small"
    self.blocks, self.ggml_type, self.out_features, self.in_features = blocks, ggml_type, out_features, in_features

  @property
  def nbytes(self) -> int:
    nel, nby = GGML_QUANT[self.ggml_type]
    return self.out_features * (self.in_features // nel) * nby

  def __call__(self, x: Buffer, out: Buffer | None = None, out_dtype=None, stream=None) -> Buffer:
    """x: (..., in_features) float16 or float32 with at most 8 rows.  Returns (rows, out_features); the caller may pass `out`."""
    assert x.shape[-1] == self.in_features, f"{x.shape} vs in_features {self.in_features}"
    m = int(np.prod(x.shape[:-1], dtype=np.int64)) if len(x.shape) > 1 else 1
    assert 1 <= m <= 8, f"batch of {m} rows is outside the decode range 1..8"
    if out is None: out = Buffer((*x.shape[:-1], self.out_features), out_dtype or x.dtype)
    assert out.nbytes == m * self.out_features * out.dtype.itemsize
    rt.check(rt.lib().tga_qlinear(self.ggml_type, self.blocks.ptr, x.ptr, rt.dtype_code(x.dtype), out.ptr, rt.dtype_code(out.dtype),
                                  m, self.out_features, self.in_features, stream))
    return out

def qlinear_multi(layers: list[QuantLinear], x: Buffer, outs: list[Buffer], epilogue: int = 0, resid: list[Buffer] | None = None, stream=None):
  """Several QuantLinear layers over the same activation in one launch (attn_q/k/v, ffn_gate/ffn_up).
  epilogue 0: plain; 1: outs[i] = resid[i] + linear; 2: outs[0] = silu(layers[0](x)) * layers[1](x)."""
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
  rt.check(rt.lib().tga_qlinear_multi(t, nseg, w, y, n, x.ptr, rt.dtype_code(x.dtype), ydt, m, k, epilogue, r, stream))
  return outs
