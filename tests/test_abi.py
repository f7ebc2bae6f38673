"""The C-ABI library loads and exports every symbol include/tinygrad_amd.h declares (no GPU call is made)."""
import ctypes, pathlib, re
import pytest

ROOT = pathlib.Path(__file__).resolve().parent.parent

def _declared():
  text = (ROOT / "include" / "tinygrad_amd.h").read_text()
  text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
  return sorted(set(re.findall(r"\b(tga_\w+)\s*\(", text)))

def test_header_declares_entry_points():
  names = _declared()
  assert "tga_qlinear" in names and "tga_dequant" in names and "tga_grouped_mxfp8_gemm" in names and len(names) >= 30

def test_library_exports_every_declared_symbol():
  lib_path = ROOT / "tinygrad_amd" / "libtinygrad_amd.so"
  if not lib_path.exists(): pytest.fail(f"{lib_path} is missing: run `python -m tinygrad_amd.build`")
  lib = ctypes.CDLL(str(lib_path))
  missing = [n for n in _declared() if not hasattr(lib, n)]
  assert not missing, f"declared in the header but not exported: {missing}"

def test_python_binding_covers_the_header():
  from tinygrad_amd import runtime as rt
  lib = rt.load_library()
  for n in _declared(): assert getattr(lib, n).restype is not None

def test_missing_library_fails_loudly(monkeypatch, tmp_path):
  from tinygrad_amd import runtime as rt
  monkeypatch.setattr(rt, "_lib", None); monkeypatch.setattr(rt, "_LIB_PATH", tmp_path / "nope.so")
  with pytest.raises(RuntimeError, match="no fallback"): rt.load_library()

def test_host_side_argument_checks_without_gpu():
  from tinygrad_amd import moe
  import numpy as np
  assert moe.m_max_for(4096, 8, 128) == 65536                                     # (ceil(T*k/256) + E) * 256, moe_routing.py:89-90
  b = moe.to_bf16_bits(np.array([1.0, 1.00390625, -2.5, 1.01171875], np.float32))     # 1 + 2^-8 ties to even (1.0); 1 + 3*2^-8 rounds up
  np.testing.assert_array_equal(moe.from_bf16_bits(b), np.array([1.0, 1.0, -2.5, 1.015625], np.float32))
