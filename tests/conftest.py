import os, sys, pathlib
import pytest

ROOT = pathlib.Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path: sys.path.insert(0, str(ROOT))

def golden_kats():
  """The reference tests' known-answer vectors for block dequant (tests/golden/ggml_dequant_kat.json): (name, type, n, block bytes, expected float32)."""
  import json, numpy as np
  g = json.loads((ROOT / "tests" / "golden" / "ggml_dequant_kat.json").read_text())
  return [(k, v["ggml_type"], v["n"], np.array(v["block"], dtype=np.uint8), np.frombuffer(bytes.fromhex(v["expected_f32_hex"]), dtype=np.float32))
          for k, v in g.items() if isinstance(v, dict)]

def pytest_configure(config):
  config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")

def _has_gpu() -> bool:
  return os.path.exists("/dev/kfd")

@pytest.fixture(scope="session")
def gpu():
  """Initialises the HIP library once.  GPU tests fail (not skip) when the library is missing: there is no fallback."""
  from tinygrad_amd import runtime as rt
  rt.init(0)
  return rt

def pytest_collection_modifyitems(config, items):
  if _has_gpu(): return
  skip = pytest.mark.skip(reason="no GPU in this container (/dev/kfd absent)")
  for it in items:
    if "gpu" in it.keywords: it.add_marker(skip)
