"""Guards for the inline-assembly loads of csrc/qgemm_dma.hip (CPU only: the file is compiled to gfx950 assembly and read as text).

The kernel requests activations with `global_load_dwordx4` written as inline assembly and waits for them with a hand-counted `s_waitcnt vmcnt(n)`, so
that weight pieces issued behind them stay in flight.  The compiler takes the destination registers for valid as soon as the request is issued: if it
ever copies or reuses one of them between the request and the wait, the kernel computes with stale data and nothing fails loudly.  These checks read
the generated code in layout order, which is how the requests, the wait and the first use follow each other in every build so far; a failure means
"look at the assembly", not necessarily "wrong code"."""
import os, pathlib, re, subprocess, tempfile
import pytest
from tinygrad_amd import build as tb

SRC = tb.CSRC / "qgemm_dma.hip"

def _regs(line: str) -> set:
  out, code = set(), line.split(";")[0]
  for m in re.finditer(r"\bv\[(\d+):(\d+)\]", code): out.update(range(int(m.group(1)), int(m.group(2)) + 1))
  for m in re.finditer(r"\bv(\d+)\b", code): out.add(int(m.group(1)))
  return out

@pytest.fixture(scope="module")
def kernels():
  try: hipcc = tb._hipcc()
  except RuntimeError: pytest.skip("hipcc not found")
  with tempfile.TemporaryDirectory() as d:
    out = pathlib.Path(d) / "qgemm_dma.s"
    r = subprocess.run([hipcc, *tb.HIPCC_FLAGS, "--cuda-device-only", "-S", str(SRC), "-o", str(out)], capture_output=True, text=True)
    if r.returncode != 0: pytest.fail(f"hipcc -S failed:\n{r.stderr[-2000:]}")
    text = out.read_text()
  ks = {}
  for name in re.findall(r"^(_Z16qgemm_dma_kernelI\w+EEv5QArgsii):", text, re.M):
    ks[name] = text[text.index("\n" + name + ":"):text.index(".set " + name + ".uses_flat_scratch")].split("\n")
  assert len(ks) >= 19, sorted(ks)
  return text, ks

def test_no_scratch(kernels):
  """The register sets that hold requests in flight must be registers: a kernel that spills keeps them in memory."""
  text, ks = kernels
  for name in ks:
    m = re.search(r"\.set " + re.escape(name) + r"\.private_seg_size, (\d+)", text)
    assert m and int(m.group(1)) == 0, (name, m and m.group(1))

def test_prologue_requests_untouched_until_the_wait(kernels):
  """K <= 4096 kernels: every run of activation requests is followed by the hand-written wait before anything else names their registers."""
  _, ks = kernels
  checked = 0
  for name, L in ks.items():
    if not name.endswith("ELb0ELb0EEv5QArgsii"): continue                   # (streamed-activation kernels: next test)
    i = 0
    while i < len(L):
      if "global_load_dwordx4" not in L[i]: i += 1; continue
      S, j, last = set(), i, i
      while j < len(L) and not re.search(r"ds_write_b(128|64)", L[j]):
        m = re.search(r"global_load_dwordx4 v\[(\d+):(\d+)\]", L[j])
        if m: S.update(range(int(m.group(1)), int(m.group(2)) + 1)); last = j
        j += 1
      w = next((k for k in range(last + 1, len(L)) if "s_waitcnt vmcnt" in L[k] and "ASMSTART" in L[k - 1]), None)
      assert w is not None, (name, last)
      for q in range(last + 1, w):
        assert not (_regs(L[q]) & S) or "global_load_dwordx4" in L[q], (name, q + 1, L[q].strip())
      checked += 1; i = j
  assert checked >= 30

def test_streamed_requests_untouched_around_the_loop(kernels):
  """K > 4096 kernels: inside the stage loop the request registers are named only by the LDS writes / conversions that consume them, by code between
  those and the next requests (where they are dead), and by the requests themselves - nothing between the requests and the loop's end."""
  _, ks = kernels
  checked = 0
  for name, L in ks.items():
    if "ELb1ELb0EEv5QArgsii" not in name and "ELb1ELb1EEv5QArgsii" not in name: continue
    S = set()
    for l in L:
      m = re.search(r"global_load_dwordx4 v\[(\d+):(\d+)\]", l)
      if m: S.update(range(int(m.group(1)), int(m.group(2)) + 1))
    hdr = max(i for i, l in enumerate(L) if "Loop Header" in l)
    bars = [i for i, l in enumerate(L) if "s_barrier" in l and i > hdr]
    assert len(bars) >= 2, name                                              # the stage barrier and the one behind the loop
    loop_bar, end_bar = bars[0], bars[-1]
    reqs = [i for i in range(loop_bar, end_bar) if "global_load_dwordx4" in L[i]]
    assert reqs, name
    for q in range(reqs[-1] + 1, end_bar):                                   # requests ... end of the loop body (in layout order)
      assert not (_regs(L[q]) & S), (name, q + 1, L[q].strip())
    first_use = next(i for i in range(hdr, loop_bar) if _regs(L[i]) & S)
    assert any("ASMSTART" in L[k] for k in range(max(hdr, first_use - 12), first_use)), (name, first_use + 1, L[first_use].strip())   # first use sits behind the wait / pin
    checked += 1
  assert checked == 4
