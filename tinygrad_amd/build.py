"""Builds libtinygrad_amd.so (gfx950 code objects + the C-ABI host shim) in-tree with hipcc.  No JIT, no torch."""
import os, pathlib, subprocess, sys
from concurrent.futures import ThreadPoolExecutor

PKG = pathlib.Path(__file__).resolve().parent
CSRC = PKG / "csrc"
LIB = PKG / "libtinygrad_amd.so"
ARCH = "gfx950"
# -packed-fp32-ops off: v_pk_*_f32 forms are not used by this build (scalar float code only)
HIPCC_FLAGS = [f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
               "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option", "-Wno-option-ignored"]

def _hipcc() -> str:
  for c in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
    if c and (pathlib.Path(c).exists() or c == "hipcc"): return c
  raise RuntimeError("hipcc not found")

def sources() -> list[pathlib.Path]: return sorted(CSRC.glob("*.hip"))

def _stale(out: pathlib.Path, deps: list[pathlib.Path]) -> bool:
  return not out.exists() or any(d.stat().st_mtime > out.stat().st_mtime for d in deps)

def build(force: bool = False, verbose: bool = False) -> pathlib.Path:
  """Compile every .hip under csrc/ for gfx950 and link them into one shared library next to this file."""
  objdir = PKG / "build"; objdir.mkdir(exist_ok=True)
  headers = list(CSRC.glob("*.h")) + [PKG.parent / "include" / "tinygrad_amd.h"]
  jobs = []
  for src in sources():
    obj = objdir / (src.stem + ".o")
    if force or _stale(obj, [src] + headers): jobs.append((src, obj))
  def compile_one(job):
    src, obj = job
    cmd = [_hipcc(), *HIPCC_FLAGS, *os.environ.get("TGA_HIPCC_EXTRA", "").split(), "-c", str(src), "-o", str(obj)]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0: raise RuntimeError(f"hipcc failed for {src.name}:\n{r.stderr}")
    if verbose: print(f"compiled {src.name}", file=sys.stderr)
  with ThreadPoolExecutor(max_workers=min(8, max(1, len(jobs)))) as ex: list(ex.map(compile_one, jobs))
  objs = [objdir / (s.stem + ".o") for s in sources()]
  if force or jobs or _stale(LIB, objs):
    r = subprocess.run([_hipcc(), f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", str(LIB), *map(str, objs)], capture_output=True, text=True)
    if r.returncode != 0: raise RuntimeError(f"link failed:\n{r.stderr}")
  return LIB

if __name__ == "__main__":
  print(build(force="--force" in sys.argv, verbose=True))
