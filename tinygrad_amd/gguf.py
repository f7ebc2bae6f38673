"""GGUF block dequant on the GPU behind the reference's name and argument meaning.

ggml_data_to_tensor(t, n, ggml_type) mirrors tinygrad/llm/gguf.py:23: `t` is the raw byte buffer (device Buffer of uint8, or a
numpy array that is uploaded), `n` the element count, and the result is a flat float32 device Buffer of n elements, bit-exact
with the reference for Q4_0 (2), Q4_1 (3), Q5_0 (6), Q5_1 (7), Q8_0 (8), Q4_K (12), Q5_K (13), Q6_K (14), IQ3_XXS (18), IQ3_S (21), IQ2_S (22), IQ4_XS (23), MXFP4 (39), Q1_0 (41); native float32/float16 (0, 1) and the other native types (int8 24, int16 25, int32 26, int64 27, float64 28; bfloat16 30 as its uint16 bit patterns) are reinterpreted in place.
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
  if ggml_type in _NATIVE_NUMPY:                              # int8 / int16 / int32 / int64 / float64 / bfloat16: the same bytes under their own type (gguf.py:35-36)
    dt = _NATIVE_NUMPY[ggml_type]
    return t.view(0, (n,), dt)                                # bfloat16 (30) has no numpy type: its bit patterns come back as uint16
  if ggml_type not in GGML_QUANT: raise ValueError(f"GGML type '{ggml_type}' is not supported!")
  nel, nby = GGML_QUANT[ggml_type]
  nfull = (n // nel) * nel                                   # gguf.py:45 uses whole blocks only
  if t.nbytes < (nfull // nel) * nby: raise ValueError(f"buffer of {t.nbytes} bytes holds fewer than {nfull // nel} blocks")
  out = Buffer((nfull,), out_dtype)
  rt.check(rt.lib().tga_dequant(ggml_type, t.ptr, nfull, out.ptr, rt.dtype_code(out_dtype), stream))
  return out

# ---------------------------------------------------------------------------------------------------------------------------
# GGUF container (tinygrad/llm/gguf.py:121-176).  Parsing is host-side Python over the file bytes; tensor data is uploaded once
# and every tensor is a window into that device buffer (the kernels read the packed blocks in place).
# ---------------------------------------------------------------------------------------------------------------------------
import io, pathlib, re, struct
from dataclasses import dataclass

_NATIVE_ITEMSIZE = {0: 4, 1: 2, 24: 1, 25: 2, 26: 4, 27: 8, 28: 8, 30: 2}         # gguf.py:16-17
_NATIVE_NUMPY = {24: np.int8, 25: np.int16, 26: np.int32, 27: np.int64, 28: np.float64, 30: np.uint16}
GGUF_F32_LIKE = (0, 30)                                                             # float32, bfloat16

def _rd(fmt, n, r): return struct.unpack("<" + fmt, r.read(n))[0]
def _read_str(r): return str(r.read(_rd("Q", 8, r)), "utf-8")
def _read_arr(r):
  typ, n = _rd("i", 4, r), _rd("Q", 8, r)
  return [_READERS[typ](r) for _ in range(n)]
_READERS = {8: _read_str, 9: _read_arr, **{t: (lambda r, f=f, nb=nb: _rd(f, nb, r)) for t, f, nb in
            [(0, "c", 1), (1, "b", 1), (2, "H", 2), (3, "h", 2), (4, "I", 4), (5, "i", 4), (6, "f", 4), (7, "?", 1), (10, "Q", 8), (11, "q", 8), (12, "d", 8)]}}

@dataclass
class GGUFTensor:
  """One tensor of a GGUF file: raw bytes on the host (numpy view) and, after upload, a device window.  shape is the
  reference's reshape(*reversed(dims)) (gguf.py:148): rows first, quant blocks along the last axis."""
  name: str
  ggml_type: int
  shape: tuple
  data: np.ndarray
  buffer: Buffer | None = None

def tensor_nbytes(ggml_type: int, n: int) -> int:
  if ggml_type in _NATIVE_ITEMSIZE: return _NATIVE_ITEMSIZE[ggml_type] * n
  if ggml_type in GGML_QUANT: nel, nby = GGML_QUANT[ggml_type]; return (n // nel) * nby
  raise ValueError(f"GGML type '{ggml_type}' is not supported!")

def gguf_parse(raw: np.ndarray) -> tuple[dict, dict[str, GGUFTensor]]:
  """_gguf_parse (gguf.py:132-149) over a uint8 array holding one GGUF file."""
  raw = np.ascontiguousarray(raw).view(np.uint8).reshape(-1)
  r = io.BytesIO(raw.data)
  magic, version, n_tensors, n_kv = r.read(4), _rd("i", 4, r), _rd("q", 8, r), _rd("q", 8, r)
  if magic != b"GGUF" or version not in (2, 3): raise ValueError("Invalid GGUF format!")
  kv = {}
  for _ in range(n_kv):
    k, typ = _read_str(r), _rd("i", 4, r)
    kv[k] = _READERS[typ](r)
  infos = [(_read_str(r), tuple(_rd("Q", 8, r) for _ in range(_rd("I", 4, r))), _rd("i", 4, r), _rd("Q", 8, r)) for _ in range(n_tensors)]
  alignment, pos = kv.get("general.alignment", 32), r.tell()
  data_start = (pos + alignment - 1) // alignment * alignment
  tensors = {}
  for name, dims, typ, off in infos:
    n = int(np.prod(dims, dtype=np.int64))
    nb = tensor_nbytes(typ, n)
    tensors[name] = GGUFTensor(name, typ, tuple(reversed(dims)), raw[data_start + off: data_start + off + nb])
  return kv, tensors

_FIRST_SPLIT = re.compile(r"-00001-of-\d{5}\.gguf$")

def _split_paths(path: pathlib.Path, kv: dict) -> list[pathlib.Path]:
  """Every part of a model that llama.cpp's gguf-split wrote as <stem>-00001-of-000NN.gguf ... (the rule of gguf.py:151-155): the part count
  comes from the first part's `split.count`; loading has to start at part 1 because only that one carries the metadata."""
  n_parts = int(kv.get("split.count", 1))
  if n_parts <= 1: return [path]
  this_part = int(kv.get("split.no", 0))
  if this_part != 0: raise ValueError(f"multi-part GGUF must be loaded from the first split, got split.no={this_part}")
  name = str(path)
  hit = _FIRST_SPLIT.search(name)
  if hit is None: raise ValueError(f"first split path must end with -00001-of-NNNNN.gguf: {path}")
  stem = name[:hit.start()]
  return [pathlib.Path(f"{stem}-{part:05d}-of-{n_parts:05d}.gguf") for part in range(1, n_parts + 1)]

def gguf_load(fn, upload: bool = True) -> tuple[dict, dict[str, GGUFTensor]]:
  """gguf_load (gguf.py:157-176): returns (kv_data, {name: GGUFTensor}).  fn: path or uint8 numpy array.  Multi-part splits are
  merged when loaded by path.  With upload=True each file's bytes go to the device once and tensor.buffer is a window into them."""
  def one(raw):
    kv, ts = gguf_parse(raw)
    if upload and ts:
      dev = Buffer.from_numpy(raw)
      base = raw.ctypes.data
      for t in ts.values(): t.buffer = dev.view(t.data.ctypes.data - base, (t.data.size,), np.uint8)
    return kv, ts
  if isinstance(fn, np.ndarray):
    kv, ts = one(np.ascontiguousarray(fn).view(np.uint8).reshape(-1))
    if kv.get("split.count", 1) > 1: raise ValueError("multi-part GGUF requires a path argument (got an array)")
    return kv, ts
  path = pathlib.Path(fn)
  kv, ts = one(np.fromfile(path, dtype=np.uint8))
  for pp in _split_paths(path, kv)[1:]: ts.update(one(np.fromfile(pp, dtype=np.uint8))[1])
  return kv, ts

def gguf_write(path, kvs: list[tuple[str, object]], tensors: list[tuple[str, tuple, int, np.ndarray]], alignment: int = 32) -> bytes:
  """Writes a GGUF v3 file with the byte layout the reference's tests spell out (test/unit/test_gguf.py:118-139):
  header, KV entries (str / uint32 / float32 / list[str]), tensor infos (dims innermost first), padding, data blob.
  tensors: (name, shape rows-first, ggml_type, raw bytes)."""
  buf = bytearray(struct.pack("<4siqq", b"GGUF", 3, len(tensors), len(kvs)))
  def put_str(s): b = s.encode(); return struct.pack("<Q", len(b)) + b
  for k, v in kvs:
    buf += put_str(k)
    if isinstance(v, str): buf += struct.pack("<i", 8) + put_str(v)
    elif isinstance(v, bool): buf += struct.pack("<i?", 7, v)
    elif isinstance(v, int): buf += struct.pack("<iI", 4, v)
    elif isinstance(v, float): buf += struct.pack("<if", 6, v)
    elif isinstance(v, list): buf += struct.pack("<iiQ", 9, 8, len(v)) + b"".join(put_str(s) for s in v)
    else: raise TypeError(f"unsupported KV value {type(v)}")
  off, blobs = 0, []
  for name, shape, typ, data in tensors:
    data = np.ascontiguousarray(data).view(np.uint8).reshape(-1)
    buf += put_str(name) + struct.pack("<I", len(shape))
    for d in reversed(shape): buf += struct.pack("<Q", d)
    buf += struct.pack("<iQ", typ, off)
    pad = (-data.size) % alignment
    blobs.append(data.tobytes() + b"\x00" * pad)
    off += data.size + pad
  buf += b"\x00" * ((-len(buf)) % alignment)
  out = bytes(buf) + b"".join(blobs)
  if path is not None: pathlib.Path(path).write_bytes(out)
  return out
