"""Guards for the inline-assembly loads of csrc/qgemm_dma.hip and csrc/qgemm_wp.hip (CPU only: the files are compiled to gfx950 assembly and read as text).

The kernel requests activations with `global_load_dwordx4` written as inline assembly and waits for them with a hand-counted `s_waitcnt vmcnt(n)`, so
that weight pieces issued behind them stay in flight.  The compiler takes the destination registers for valid as soon as the request is issued: if it
ever copies or reuses one of them between the request and the wait, the kernel computes with stale data and nothing fails loudly.  These checks read
the generated code in layout order, which is how the requests, the wait and the first use follow each other in every build so far; a failure means
"look at the assembly", not necessarily "wrong code"."""
import os, pathlib, re, subprocess, tempfile
import pytest
from tinygrad_amd import build as tb

SOURCES = {"qgemm_dma.hip": (r"^(_Z16qgemm_dma_kernelI\w+EEv5QArgsii):", 19), "qgemm_wp.hip": (r"^(_Z15qgemm_wp_kernelI\w+EEv5QArgsii):", 12)}

def _regs(line: str) -> set:
  out, code = set(), line.split(";")[0]
  for m in re.finditer(r"\bv\[(\d+):(\d+)\]", code): out.update(range(int(m.group(1)), int(m.group(2)) + 1))
  for m in re.finditer(r"\bv(\d+)\b", code): out.add(int(m.group(1)))
  return out

@pytest.fixture(scope="module", params=sorted(SOURCES))
def kernels(request):
  try: hipcc = tb._hipcc()
  except RuntimeError: pytest.skip("hipcc not found")
  pattern, at_least = SOURCES[request.param]
  with tempfile.TemporaryDirectory() as d:
    out = pathlib.Path(d) / (request.param + ".s")
    r = subprocess.run([hipcc, *tb.HIPCC_FLAGS, "--cuda-device-only", "-S", str(tb.CSRC / request.param), "-o", str(out)], capture_output=True, text=True)
    if r.returncode != 0: pytest.fail(f"hipcc -S failed:\n{r.stderr[-2000:]}")
    text = out.read_text()
  ks = {}
  for name in re.findall(pattern, text, re.M):
    ks[name] = text[text.index("\n" + name + ":"):text.index(".set " + name + ".uses_flat_scratch")].split("\n")
  assert len(ks) >= at_least, sorted(ks)
  return text, ks

def test_no_scratch(kernels):
  """The register sets that hold requests in flight must be registers: a kernel that spills keeps them in memory."""
  text, ks = kernels
  for name in ks:
    m = re.search(r"\.set " + re.escape(name) + r"\.private_seg_size, (\d+)", text)
    assert m and int(m.group(1)) == 0, (name, m and m.group(1))

def _touches_in_flight(L):
  """Forward data flow over the kernel's basic blocks: a request (`global_load_dwordx4 v[a:b]`, only written as inline assembly in this file) puts its destination
  registers in flight; the source passes them through an asm statement marked "; landed" right behind the hand-counted wait, which lands them all (the wait itself is a
  switch over immediates that the compiler lowers to a tree of branches with paths no run takes, so it cannot serve as the landing point of a path-insensitive
  analysis); an instruction that names a register in flight - other than a request that overwrites it - is a finding.  Returns the findings as (line number, text)."""
  ins = []                                                                     # (line index, text) of instructions; labels -> index of the next instruction
  labels = {}
  in_asm, has_marks = False, any(l.strip().startswith(";;#ASMSTART") for l in L)   # (hand-made listings carry no ASMSTART / ASMEND: every request counts there)
  for i, l in enumerate(L):
    m = re.match(r"(\.LBB\d+_\d+):", l)
    if m: labels[m.group(1)] = len(ins); continue
    if l.strip().startswith(";;#ASMSTART"): in_asm = True; continue
    if l.strip().startswith(";;#ASMEND"): in_asm = False; continue
    if l.strip() == "; landed": ins.append((i, "; landed")); continue
    t = l.split(";")[0].strip()
    if not l.startswith("\t") or not t or t.startswith("."): continue
    # a 16-byte load that the compiler wrote (it places that load's wait itself) is an ordinary instruction here, not a request
    if has_marks and not in_asm and t.startswith("global_load_dwordx4"): t = "compiler_" + t
    ins.append((i, t))
  n = len(ins)
  succ = [[] for _ in range(n)]
  for k, (_, t) in enumerate(ins):
    op = t.split()[0]
    if op == "s_endpgm": continue
    if op == "s_branch": succ[k].append(labels[t.split()[1]]); continue
    if op.startswith("s_cbranch"): succ[k].append(labels[t.split()[1]])
    if k + 1 < n: succ[k].append(k + 1)
  state = [None] * n                                                           # registers in flight BEFORE instruction k
  state[0] = frozenset()
  work, found = [0], {}
  while work:
    k = work.pop()
    cur, (li, t) = state[k], ins[k]
    m = re.match(r"global_load_dwordx4 v\[(\d+):(\d+)\]", t)
    if m: out = cur | frozenset(range(int(m.group(1)), int(m.group(2)) + 1))   # (its address registers are read at issue: not a use of data in flight)
    elif t == "; landed": out = frozenset()
    else:
      if _regs(t) & cur: found[li + 1] = t
      out = cur
    for j in succ[k]:
      new = out if state[j] is None else state[j] | out
      if new != state[j]: state[j] = new; work.append(j)
  return sorted(found.items())

def test_requests_in_flight_are_not_touched(kernels):
  """Every kernel of the file, K <= 4096 (requests in the prologue) and K > 4096 (one request site in the stage loop, waited for in the next pass)."""
  _, ks = kernels
  for name, L in ks.items():
    assert any("global_load_dwordx4" in l for l in L), name
    bad = _touches_in_flight(L)
    assert not bad, (name, bad[:5])

def test_the_check_itself():
  """The data-flow check on hand-made listings: a copy of a register in flight is found on a straight path, around a loop's back edge and behind a branch; uses behind
  the landing mark and reuse of the request's address registers are not."""
  ok = ["\tglobal_load_dwordx4 v[4:7], v[4:5], off", "\ts_cbranch_scc1 .LBB0_2", "\tv_mov_b32_e32 v9, v1", ".LBB0_2:", "\ts_waitcnt vmcnt(0)", "\t; landed", "\tv_mov_b32_e32 v8, v5", "\ts_endpgm"]
  assert _touches_in_flight(ok) == []
  straight = ["\tglobal_load_dwordx4 v[4:7], v[2:3], off", "\tv_mov_b32_e32 v8, v5", "\t; landed", "\ts_endpgm"]
  assert [t for _, t in _touches_in_flight(straight)] == ["v_mov_b32_e32 v8, v5"]
  branch = ["\tglobal_load_dwordx4 v[4:7], v[2:3], off", "\ts_cbranch_scc1 .LBB0_2", "\t; landed", "\ts_branch .LBB0_3", ".LBB0_2:", "\tv_add_u32_e32 v6, v1, v2", "\t; landed", ".LBB0_3:", "\ts_endpgm"]
  assert [t for _, t in _touches_in_flight(branch)] == ["v_add_u32_e32 v6, v1, v2"]
  loop = [".LBB0_1:", "\tv_mov_b32_e32 v9, v4", "\t; landed", "\tds_write_b128 v1, v[4:7]", "\tglobal_load_dwordx4 v[4:7], v[2:3], off", "\ts_cbranch_scc1 .LBB0_1", "\t; landed", "\ts_endpgm"]
  assert [t for _, t in _touches_in_flight(loop)] == ["v_mov_b32_e32 v9, v4"]

def test_wave_private_loop_keeps_its_ring_in_flight(kernels):
  """qgemm_wp.hip counts its direct-to-LDS pieces by hand; a compiler-placed `s_waitcnt vmcnt(0)` inside the row-group loop (it puts one in front of an LDS atomic
  builtin, for instance, because it cannot tell the counters from the rings) would empty the ring once per group.  Inside the loop of the SwiGLU
  instantiations every vector-memory wait must be one of the source's own (between ASMSTART / ASMEND); the others also hold the residual load of the
  summing wave, which the compiler waits for."""
  _, ks = kernels
  names = [n for n in ks if "qgemm_wp_kernel" in n]
  if not names: pytest.skip("not the wave-private source")
  checked = 0
  for name in names:
    m = re.match(r"_Z15qgemm_wp_kernelILi\d+ELb([01])ELb([01])E", name)
    if m.group(2) == "0": continue                                           # (plain, residual, q / k / v)
    L = ks[name]
    start = max(i for i, l in enumerate(L) if "This Loop Header: Depth=1" in l)
    inside_asm, bad = False, []
    for i in range(start, len(L)):
      t = L[i].strip()
      if t.startswith(";;#ASMSTART"): inside_asm = True
      elif t.startswith(";;#ASMEND"): inside_asm = False
      elif t.startswith("s_waitcnt") and "vmcnt" in t and not inside_asm and i < len(L) - 6: bad.append((i, t))
    assert not bad, (name, bad)
    checked += 1
  assert checked >= 4
