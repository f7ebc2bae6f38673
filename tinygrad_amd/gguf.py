"""GGUF block dequant on the GPU behind the reference's name and argument meaning.

ggml_data_to_tensor(t, n, ggml_type) mirrors tinygrad/llm/gguf.py:23: `t` is the raw byte buffer (device Buffer of uint8, or a
numpy array that is uploaded), `n` the element count, and the result is a flat float32 device Buffer of n elements, bit-exact
with the reference for Q4_0 (2), Q8_0 (8), Q6_K (14), MXFP4 (39); native float32/float16 (0, 1) are reinterpreted in place.
Unknown types raise ValueError with the reference's message (gguf.py:119)."""
from __future__ import annotations
import numpy as np
from tinygrad_amd import runtime as rt
from tinygrad_amd.runtime import Buffer, GGML_QUANT

def _as_device_bytes(t) -> Buffer:
  if isinstance(t, Buffer): return t
  return Buffer.from_numpy(np.ascontiguousarray(t).view(np.uint8).reshape(-1))

def ggml_data_to_tensor(t, n: int, ggml_type: int, out_dtype=np.float32, stream=None) -> Buffer:
  t = _as_device_bytes(t)
  if ggml_type == rt.F32: return t.view(0, (n,), np.float32)
  if ggml_type == rt.F16: return t.view(0, (n,), np.float16)
  if ggml_type not in GGML_QUANT: raise ValueError(f"GGML type '{ggml_type}' is not supported!")
  nel, nby = GGML_QUANT[ggml_type]
  nfull = (n // nel) * nel                                   # gguf.py:45 uses whole blocks only
  if t.nbytes < (nfull // nel) * nby: raise ValueError(f"buffer of {t.nbytes} bytes holds fewer than {nfull // nel} blocks")
  out = Buffer((nfull,), out_dtype)
  rt.check(rt.lib().tga_dequant(ggml_type, t.ptr, nfull, out.ptr, rt.dtype_code(out_dtype), stream))
  return out
