"""ctypes binding of oracle/c/liboracle.so (scalar C restatement; checker + timed CPU baseline).  Test infrastructure only."""
import ctypes, pathlib, subprocess
import numpy as np

_DIR = pathlib.Path(__file__).parent / "c"
_lib = None

def build(force: bool = False) -> pathlib.Path:
  so = _DIR / "liboracle.so"
  if force or not so.exists() or so.stat().st_mtime < (_DIR / "oracle.c").stat().st_mtime:
    subprocess.check_call(["make", "-B", "-C", str(_DIR)], stdout=subprocess.DEVNULL)
  return so

def lib():
  global _lib
  if _lib is None:
    _lib = ctypes.CDLL(str(build()))
    _lib.orc_dequant.argtypes = [ctypes.c_int, ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p, ctypes.c_int]
    _lib.orc_linear.argtypes = [ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int64,
                                ctypes.c_int64, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int]
    _lib.orc_round_f16.argtypes, _lib.orc_round_f16.restype = [ctypes.c_void_p, ctypes.c_int64], None
    _lib.orc_h2f.restype, _lib.orc_h2f.argtypes = ctypes.c_float, [ctypes.c_uint16]
    _lib.orc_f2h.restype, _lib.orc_f2h.argtypes = ctypes.c_uint16, [ctypes.c_float]
  return _lib

_GEOM = {2: (32, 18), 3: (32, 20), 6: (32, 22), 7: (32, 24), 8: (32, 34), 12: (256, 144), 13: (256, 176), 14: (256, 210), 18: (256, 98), 21: (256, 110), 22: (256, 82), 23: (256, 136), 39: (32, 17), 41: (128, 18)}

def dequant(ggml_type: int, blocks: np.ndarray, threads: int = 1) -> np.ndarray:
  nel, nby = _GEOM[ggml_type]
  blocks = np.ascontiguousarray(blocks).view(np.uint8).reshape(-1)
  nb = blocks.size // nby
  out = np.empty(nb * nel, dtype=np.float32)
  rc = lib().orc_dequant(ggml_type, blocks.ctypes.data, nb, out.ctypes.data, threads)
  assert rc == 0, rc
  return out

def linear(ggml_type: int, w: np.ndarray, x: np.ndarray, n: int, k: int, w_round_f16=False, prod_round_f16=False, threads: int = 1) -> np.ndarray:
  """x: (M,K) float32 or float16.  Returns (M,N) float32 accumulators."""
  x = np.ascontiguousarray(x)
  assert x.dtype in (np.float32, np.float16) and x.ndim == 2 and x.shape[1] == k and x.shape[0] <= 8
  w = np.ascontiguousarray(w).view(np.uint8).reshape(-1)
  y = np.empty((x.shape[0], n), dtype=np.float32)
  rc = lib().orc_linear(ggml_type, w.ctypes.data, x.ctypes.data, y.ctypes.data, x.shape[0], n, k,
                        int(x.dtype == np.float16), int(w_round_f16), int(prod_round_f16), threads)
  assert rc == 0, rc
  return y

def round_f16(x: np.ndarray) -> np.ndarray:
  """float32 -> nearest fp16 -> float32 through the conversion orc_linear uses for its weights."""
  y = np.ascontiguousarray(x, dtype=np.float32).copy()
  lib().orc_round_f16(y.ctypes.data, y.size)
  return y

def max_threads() -> int: return lib().orc_max_threads()
