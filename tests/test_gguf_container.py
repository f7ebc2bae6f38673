"""GGUF container: byte layout of the reference's tests (test/unit/test_gguf.py:118-155, 216-225) parsed on the host (no GPU)."""
import struct, numpy as np, pytest
from tinygrad_amd import gguf as G
from oracle import gguf as ogguf, ggml as og

def _build_gguf(tensors, kvs):
  """Verbatim byte layout of the reference test helper (test/unit/test_gguf.py:118-139), written independently of gguf_write."""
  buf = bytearray(struct.pack("<4siqq", b"GGUF", 3, len(tensors), len(kvs)))
  for k, v in kvs:
    kb = k.encode()
    if isinstance(v, str): buf += struct.pack("<Q", len(kb)) + kb + struct.pack("<i", 8) + struct.pack("<Q", len(v)) + v.encode()
    else: buf += struct.pack("<Q", len(kb)) + kb + struct.pack("<i", 4) + struct.pack("<I", v)
  off = 0
  for name, dims, qtype, data in tensors:
    nb = name.encode()
    buf += struct.pack("<Q", len(nb)) + nb + struct.pack("<I", len(dims))
    for d in reversed(dims): buf += struct.pack("<Q", d)
    buf += struct.pack("<i", qtype) + struct.pack("<Q", off)
    off += len(data)
  buf += b"\x00" * ((32 - len(buf) % 32) % 32)
  for _, _, _, data in tensors: buf += data
  return bytes(buf)

def test_parse_reference_layout_and_multi_part(tmp_path):
  a, b = np.array([1.0, 2.0, 3.0, 4.0], dtype=np.float32), np.array([5.0, 6.0], dtype=np.float32)
  (tmp_path / "test-00001-of-00002.gguf").write_bytes(_build_gguf([("a", (4,), 0, a.tobytes())], [("split.count", 2), ("split.no", 0)]))
  (tmp_path / "test-00002-of-00002.gguf").write_bytes(_build_gguf([("b", (2,), 0, b.tobytes())], [("split.count", 2), ("split.no", 1)]))
  kv, ts = G.gguf_load(tmp_path / "test-00001-of-00002.gguf", upload=False)
  assert kv["split.count"] == 2
  np.testing.assert_array_equal(ts["a"].data.view(np.float32), a); np.testing.assert_array_equal(ts["b"].data.view(np.float32), b)
  (tmp_path / "test-00002-of-00002.gguf").unlink()
  with pytest.raises(FileNotFoundError): G.gguf_load(tmp_path / "test-00001-of-00002.gguf", upload=False)
  with pytest.raises(ValueError): G.gguf_parse(np.frombuffer(b"NOPE" + bytes(28), dtype=np.uint8))

def test_quantized_tensor_slicing_matches_oracle_parse():
  rng = np.random.default_rng(42)
  rows, cols = 64, 256
  blobs = {t: rng.integers(0, 256, size=rows * cols // og.GGML_QUANT[t][0] * og.GGML_QUANT[t][1], dtype=np.uint8) for t in (2, 8, 14, 39)}
  for t in (2, 8): blobs[t].reshape(-1, og.GGML_QUANT[t][1])[:, :2] = np.float16(rng.standard_normal(rows * cols // 32)).view(np.uint8).reshape(-1, 2)
  blobs[14].reshape(-1, 210)[:, 208:] = np.float16(rng.standard_normal(rows * cols // 256)).view(np.uint8).reshape(-1, 2)
  raw = G.gguf_write(None, [("general.architecture", "test"), ("some.count", 7), ("some.scale", 0.5), ("tokenizer.ggml.tokens", ["a", "b", "c"])],
                     [(f"w{t}", (rows, cols), t, blobs[t]) for t in blobs])
  kv, ts = G.gguf_parse(np.frombuffer(raw, dtype=np.uint8))
  okv, osd = ogguf.parse(raw)
  assert kv == okv and kv["tokenizer.ggml.tokens"] == ["a", "b", "c"] and kv["some.count"] == 7
  for t in blobs:
    assert ts[f"w{t}"].shape == (rows, cols) and ts[f"w{t}"].data.tobytes() == blobs[t].tobytes()
    with np.errstate(all="ignore"):
      np.testing.assert_array_equal(og.ggml_data_to_tensor(ts[f"w{t}"].data, rows * cols, t).reshape(rows, cols), osd[f"w{t}"])
  # the writer reproduces the reference helper's bytes for the cases that helper covers
  a = np.arange(8, dtype=np.float32)
  assert G.gguf_write(None, [("split.count", 2), ("x", "y")], [("a", (8,), 0, a)]) == _build_gguf([("a", (8,), 0, a.tobytes())], [("split.count", 2), ("x", "y")])
