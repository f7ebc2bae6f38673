import os, sys, pathlib
import pytest

ROOT = pathlib.Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path: sys.path.insert(0, str(ROOT))

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
