"""ctypes binding of libtinygrad_amd.so: the only way Python reaches the GPU in this package (no torch, no Triton).

Mirrors the reference's HIP device glue (tinygrad/runtime/ops_hip.py:9-70): a non-zero status becomes RuntimeError with the
library's message, buffers are explicit device allocations owned by the Python side."""
from __future__ import annotations
import ctypes, os, pathlib
import numpy as np

F32, F16, Q4_0, Q8_0, Q4_K, Q5_K, Q6_K, MXFP4 = 0, 1, 2, 8, 12, 13, 14, 39
Q4_1, Q5_0, Q5_1 = 3, 6, 7
IQ4_XS, Q1_0 = 23, 41
IQ3_XXS, IQ3_S, IQ2_S = 18, 21, 22
F16_STAGED = 101          # activation dtype code: fp16 in the staged order of the consuming weight (tga_stage_activation)
# {ggml_type: (elements per block, bytes per block)}: tinygrad/llm/gguf.py:20-21
# (every one of them is read in place by the linear kernels; tga_dequant expands any of them)
GGML_QUANT = {Q4_0: (32, 18), Q4_1: (32, 20), Q5_0: (32, 22), Q5_1: (32, 24), Q8_0: (32, 34), Q4_K: (256, 144), Q5_K: (256, 176), Q6_K: (256, 210), IQ4_XS: (256, 136), MXFP4: (32, 17),
              IQ3_XXS: (256, 98), IQ3_S: (256, 110), IQ2_S: (256, 82), Q1_0: (128, 18)}
_NP_DTYPE = {F32: np.float32, F16: np.float16}

_LIB_PATH = pathlib.Path(os.environ.get("TGA_LIB") or pathlib.Path(__file__).resolve().parent / "libtinygrad_amd.so")   # (TGA_LIB: another build of the same library)
_lib = None
_initialised = False

c_void_pp = ctypes.POINTER(ctypes.c_void_p)

def _declare(lib):
  vp, i, i64, sz = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_size_t
  sig = {
    "tga_init": [i], "tga_device_name": [ctypes.c_char_p, sz], "tga_malloc": [c_void_pp, sz], "tga_free": [vp],
    "tga_memcpy_h2d": [vp, vp, sz], "tga_memcpy_d2h": [vp, vp, sz], "tga_memcpy_d2d": [vp, vp, sz, vp], "tga_memset": [vp, i, sz, vp],
    "tga_sync": [], "tga_stream_create": [c_void_pp], "tga_stream_destroy": [vp], "tga_stream_sync": [vp],
    "tga_event_create": [c_void_pp], "tga_event_destroy": [vp], "tga_event_record": [vp, vp], "tga_event_sync": [vp],
    "tga_event_elapsed_ms": [vp, vp, ctypes.POINTER(ctypes.c_float)],
    "tga_graph_begin": [vp], "tga_graph_end": [vp, c_void_pp], "tga_graph_launch": [vp, vp], "tga_graph_destroy": [vp],
    "tga_cmdlist_end": [vp, c_void_pp], "tga_cmdlist_launch": [vp, vp], "tga_cmdlist_size": [vp], "tga_cmdlist_destroy": [vp],
    "tga_dequant": [i, vp, i64, vp, i, vp],
    "tga_qlinear": [i, vp, vp, i, vp, i, i, i64, i64, vp],
    "tga_qlinear_multi": [i, i, c_void_pp, c_void_pp, ctypes.POINTER(i64), vp, i, i, i, i64, i, c_void_pp, i, i64, vp],
    "tga_rmsnorm_qlinear_multi": [vp, ctypes.c_float, i, i, c_void_pp, c_void_pp, ctypes.POINTER(i64), vp, i, i64, i, c_void_pp, i, i64, vp],
    "tga_rmsnorm_qlinear_mixed": [vp, ctypes.c_float, i, ctypes.POINTER(ctypes.c_int32), c_void_pp, c_void_pp, ctypes.POINTER(i64), vp, i, i64, vp],
    "tga_rmsnorm_qlinear_rows": [vp, ctypes.c_float, i, i, c_void_pp, c_void_pp, ctypes.POINTER(i64), vp, vp, i, i, i64, i, c_void_pp, vp],
    "tga_moe_combine_rmsnorm_qlinear_multi": [vp, vp, i, vp, vp, vp, ctypes.c_float, i, i, c_void_pp, c_void_pp, ctypes.POINTER(i64), i, i64, vp],
    "tga_stage_activation": [i, vp, i, i64, vp, vp],
    "tga_qlinear_experts": [i, vp, vp, i64, vp, i, i, vp, i, vp, i, i64, i64, vp],
    "tga_qlinear_experts_routed": [i, vp, vp, i64, vp, i, i, i, ctypes.c_float, vp, vp, vp, vp, i, i64, i64, vp],
    "tga_qlinear_experts_routed_rows": [i, vp, vp, i64, vp, i, i, i, i, ctypes.c_float, vp, vp, vp, vp, i, i64, i64, vp],
    "tga_moe_gate": [vp, i, i, i, i, i, ctypes.c_float, vp, vp, vp],
    "tga_moe_gate_biased": [vp, vp, i, i, i, i, i, ctypes.c_float, vp, vp, vp],
    "tga_moe_combine": [vp, vp, vp, i, i, i, vp, vp],
    "tga_moe_router_rows": [vp, vp, ctypes.c_float, vp, i, i, i, vp, vp, vp],
    "tga_moe_router": [vp, vp, ctypes.c_float, vp, i, i, i, i, i, ctypes.c_float, vp, vp, vp, vp, vp],
    "tga_quantize_mxfp8": [vp, i, i64, i64, vp, vp, vp, vp],
    "tga_silu_mul_quantize_mxfp8": [vp, vp, i64, i64, vp, vp, vp, vp],
    "tga_transpose_quantize_mxfp8": [vp, i64, i64, vp, vp, vp, vp],
    "tga_moe_route": [vp, i, i, i, vp, vp, vp, vp, vp, vp, vp],
    "tga_moe_route_static": [vp, i, i, i, vp, vp, vp, vp, vp, vp],
    "tga_moe_dispatch": [vp, vp, vp, vp, i, i, i, i64, i, vp, vp],
    "tga_moe_combine_rows": [vp, vp, vp, i, i, i, vp, vp],
    "tga_grouped_mxfp8_gemm": [vp, vp, vp, vp, vp, vp, vp, vp, i64, i64, i64, i, vp],
    "tga_grouped_mxfp8_gemm_routed": [vp, vp, vp, vp, vp, vp, i64, i64, i64, i, vp],
    "tga_grouped_mxfp8_gemm_counts": [vp, vp, vp, vp, vp, vp, vp, i64, i64, i64, i, vp],
    "tga_kernel_symbol": [ctypes.c_char_p, c_void_pp], "tga_launch_kernel": [vp, ctypes.POINTER(ctypes.c_uint32), ctypes.POINTER(ctypes.c_uint32), c_void_pp, vp],
    "tga_swiglu_interleaved": [vp, i64, i, ctypes.c_float, ctypes.c_float, vp, vp],
    "tga_add_expert_bias": [vp, vp, vp, i64, i64, i, vp],
    "tga_embed_row": [vp, i, i, vp, vp, vp],
    "tga_embed_rows": [vp, i, i, vp, i, vp, vp, vp], "tga_rmsnorm_rows": [vp, vp, i, i, ctypes.c_float, vp, vp, i, vp], "tga_silu_mul": [vp, vp, ctypes.c_int64, vp, vp],
    "tga_moe_combine_rmsnorm_rows": [vp, vp, vp, vp, i, i, i, ctypes.c_float, vp, vp, vp],
    "tga_attention_decode_batched": [i, vp, vp, vp, vp, vp, ctypes.c_float, i, vp, vp, vp, vp, i, i, i, i, vp, vp, vp, vp],
    "tga_attention_prefill_chunk": [i, vp, vp, vp, vp, vp, ctypes.c_float, i, vp, vp, vp, vp, i, i, i, i, vp, vp, vp, vp],
    "tga_chunk_advance": [vp, vp, i, vp, i, vp],
    "tga_attention_prefill_chunk_staged": [i, vp, vp, vp, vp, vp, ctypes.c_float, i, vp, vp, vp, vp, i, i, i, i, vp, vp, i, vp],
    "tga_rows_staged_plan": [i, i64, i, ctypes.POINTER(i)],
    "tga_qlinear_rows_deferred": [i, vp, i64, i64, vp, i, vp, ctypes.POINTER(vp), ctypes.POINTER(i), ctypes.POINTER(i), vp],
    "tga_rmsnorm_rows_stage": [vp, vp, i, i, vp, ctypes.c_float, i, i, i, vp, vp, vp],
    "tga_rows_add_partials": [vp, vp, i, i, i, i, vp],
    "tga_argmax_rows_step": [vp, i, i, vp, vp, i, vp, vp, i, vp],
    "tga_expert_jobs": [vp, i, i, vp, vp, vp], "tga_qlinear_experts_grouped": [i, vp, vp, i64, vp, i, i, vp, vp, i, i64, i64, vp],
    "tga_rmsnorm": [vp, vp, i, ctypes.c_float, vp, vp, i, vp],
    "tga_attention_decode": [vp, vp, vp, vp, vp, vp, vp, i, i, i, i, vp, vp, vp, i, vp],
    "tga_attention_decode_normed": [vp, vp, vp, vp, vp, ctypes.c_float, i, vp, vp, vp, vp, i, i, i, i, vp, vp, vp, i, vp],
    "tga_attention_split_plan": [i, vp],
    "tga_rmsnorm_qlinear_multi_touch": [vp, ctypes.c_float, i, i, c_void_pp, c_void_pp, vp, vp, i, i64, i, c_void_pp, vp, vp, vp, vp, i, i, i, vp],
    "tga_attention_decode_split": [vp, vp, vp, vp, vp, vp, vp, i, i, i, i, vp, vp],
    "tga_attention_decode_split_normed": [vp, vp, vp, vp, vp, ctypes.c_float, i, vp, vp, vp, vp, i, i, i, i, vp, vp],
    "tga_attn_merge_qlinear": [i, vp, vp, i64, i64, vp, vp, i, i, vp],
    "tga_argmax_step": [vp, i, vp, vp, vp, vp, vp, i, vp],
    "tga_advance_prompt": [vp, vp, vp],
    "tga_copy_kernel": [vp, vp, ctypes.c_size_t, vp],
    "tga_mfma_peak": [i, i, vp, vp],
    "tga_synth_weights": [i, vp, i64, ctypes.c_uint32, ctypes.c_float, vp],
  }
  for name, args in sig.items():
    fn = getattr(lib, name)
    fn.argtypes, fn.restype = args, ctypes.c_int
  lib.tga_last_error.restype, lib.tga_last_error.argtypes = ctypes.c_char_p, []
  return lib

def load_library() -> ctypes.CDLL:
  """Loads the built library.  Fails loudly when it is missing: there is no CPU fallback."""
  global _lib
  if _lib is None:
    if not _LIB_PATH.exists():
      raise RuntimeError(f"{_LIB_PATH} is missing: build it with `python -m tinygrad_amd.build` (needs hipcc); there is no fallback path")
    _lib = _declare(ctypes.CDLL(str(_LIB_PATH)))
  return _lib

def check(status: int) -> None:
  if status != 0: raise RuntimeError(load_library().tga_last_error().decode())

def init(device: int = 0) -> None:
  global _initialised
  check(load_library().tga_init(device))
  _initialised = True

def lib() -> ctypes.CDLL:
  if not _initialised: init(0)
  return _lib

def device_name() -> str:
  buf = ctypes.create_string_buffer(256)
  check(lib().tga_device_name(buf, 256))
  return buf.value.decode()

def synchronize() -> None: check(lib().tga_sync())

class Buffer:
  """A device allocation plus the (shape, dtype) the host side attaches to it.  dtype is a numpy dtype."""
  def __init__(self, shape, dtype=np.uint8, ptr: int | None = None, owner=None):
    self.shape = tuple(int(s) for s in (shape if isinstance(shape, (tuple, list)) else (shape,)))
    self.dtype = np.dtype(dtype)
    self.nbytes = int(np.prod(self.shape, dtype=np.int64)) * self.dtype.itemsize
    self._owner = owner
    if ptr is None:
      p = ctypes.c_void_p()
      check(lib().tga_malloc(ctypes.byref(p), self.nbytes))
      self.ptr, self._owned = p.value, True
    else: self.ptr, self._owned = ptr, False

  def __del__(self):
    if getattr(self, "_owned", False) and self.ptr and _lib is not None:
      _lib.tga_free(ctypes.c_void_p(self.ptr)); self.ptr = None

  @staticmethod
  def from_numpy(a: np.ndarray) -> "Buffer":
    a = np.ascontiguousarray(a)
    b = Buffer(a.shape, a.dtype)
    if a.nbytes: check(lib().tga_memcpy_h2d(b.ptr, a.ctypes.data, a.nbytes))
    return b

  def copyin(self, a: np.ndarray) -> "Buffer":
    a = np.ascontiguousarray(a)
    assert a.nbytes == self.nbytes, (a.nbytes, self.nbytes)
    if a.nbytes: check(lib().tga_memcpy_h2d(self.ptr, a.ctypes.data, a.nbytes))
    return self

  def numpy(self) -> np.ndarray:
    out = np.empty(self.shape, dtype=self.dtype)
    if self.nbytes: check(lib().tga_memcpy_d2h(out.ctypes.data, self.ptr, self.nbytes))
    return out

  def view(self, byte_offset: int, shape, dtype) -> "Buffer":
    """A non-owning window into this allocation (e.g. one tensor's byte range inside a GGUF file buffer)."""
    v = Buffer(shape, dtype, ptr=self.ptr + byte_offset, owner=self)
    assert byte_offset + v.nbytes <= self.nbytes
    return v

  def zero_(self, stream=None) -> "Buffer":
    if self.nbytes: check(lib().tga_memset(self.ptr, 0, self.nbytes, stream))
    return self

class Stream:
  def __init__(self):
    p = ctypes.c_void_p(); check(lib().tga_stream_create(ctypes.byref(p))); self.handle = p.value
  def synchronize(self): check(lib().tga_stream_sync(self.handle))
  def __del__(self):
    if getattr(self, "handle", None) and _lib is not None: _lib.tga_stream_destroy(ctypes.c_void_p(self.handle)); self.handle = None

class Event:
  def __init__(self):
    p = ctypes.c_void_p(); check(lib().tga_event_create(ctypes.byref(p))); self.handle = p.value
  def record(self, stream=None): check(lib().tga_event_record(self.handle, stream))
  def synchronize(self): check(lib().tga_event_sync(self.handle))
  def elapsed_ms(self, end: "Event") -> float:
    ms = ctypes.c_float(); check(lib().tga_event_elapsed_ms(self.handle, end.handle, ctypes.byref(ms))); return ms.value
  def __del__(self):
    if getattr(self, "handle", None) and _lib is not None: _lib.tga_event_destroy(ctypes.c_void_p(self.handle)); self.handle = None

def _capture_begin(stream: Stream) -> bool:
  """Starts a stream capture with Python's cycle collector held off: a collection in the middle of a capture could free device buffers of dead
  objects (hipFree is not allowed while a capture is open: it invalidates the capture).  Returns whether the collector has to be switched on again."""
  import gc
  was = gc.isenabled()
  gc.collect(); gc.disable()
  try: check(lib().tga_graph_begin(stream.handle))
  except Exception:
    if was: gc.enable()
    raise
  return was

def _capture_done(was_enabled: bool):
  import gc
  if was_enabled: gc.enable()

class Graph:
  """Captured launch sequence replayed per decode step (the reference's TinyJit replay, tinygrad/engine/jit.py:163-198)."""
  def __init__(self, stream: Stream): self.stream, self.handle = stream, None
  def __enter__(self): self._gc = _capture_begin(self.stream); return self
  def __exit__(self, et, ev, tb):
    p = ctypes.c_void_p(); st = lib().tga_graph_end(self.stream.handle, ctypes.byref(p))
    _capture_done(self._gc)
    if et is None: check(st); self.handle = p.value
    return False
  def launch(self): check(lib().tga_graph_launch(self.handle, self.stream.handle))
  def __del__(self):
    if getattr(self, "handle", None) and _lib is not None: _lib.tga_graph_destroy(ctypes.c_void_p(self.handle)); self.handle = None

class CommandList:
  """Graph's interface over tga_cmdlist_*: the captured kernel launches are enqueued one after the other instead of going through hipGraphLaunch."""
  def __init__(self, stream: Stream): self.stream, self.handle = stream, None
  def __enter__(self): self._gc = _capture_begin(self.stream); return self
  def __exit__(self, et, ev, tb):
    p = ctypes.c_void_p(); st = lib().tga_cmdlist_end(self.stream.handle, ctypes.byref(p))
    _capture_done(self._gc)
    if et is None: check(st); self.handle = p.value
    return False
  def launch(self): check(lib().tga_cmdlist_launch(self.handle, self.stream.handle))
  def __len__(self): return lib().tga_cmdlist_size(self.handle)
  def __del__(self):
    if getattr(self, "handle", None) and _lib is not None: _lib.tga_cmdlist_destroy(ctypes.c_void_p(self.handle)); self.handle = None

def dtype_code(dt) -> int:
  dt = np.dtype(dt)
  if dt == np.float32: return F32
  if dt == np.float16: return F16
  raise TypeError(f"unsupported activation dtype {dt}")
