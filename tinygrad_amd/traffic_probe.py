"""Workload for the HBM-traffic counter runs (rocprofv3 --pmc FETCH_SIZE, then --pmc WRITE_SIZE): one 1 GiB plain copy kernel
(the yardstick: it must read 1 GiB and write 1 GiB) followed by a few eager decode steps of the benchmark model at context ~1024.

    rocprofv3 --pmc FETCH_SIZE --output-format csv -d out -o t -- python3 tinygrad_amd/traffic_probe.py [--fused]

Default: the decode steps take the per-op launch path (the kernels the benchmark runs); --fused: the one-launch block kernel."""
import os, sys
sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
import numpy as np
from tinygrad_amd import runtime as rt
from tinygrad_amd.llm import Transformer, TransformerConfig, synth_state, LLAMA3_8B

def main():
  rt.init(0)
  n = 1 << 30
  a, b = rt.Buffer((n,), np.uint8).zero_(), rt.Buffer((n,), np.uint8)
  rt.check(rt.lib().tga_copy_kernel(b.ptr, a.ptr, n, None)); rt.synchronize()
  c = TransformerConfig(max_context=1088, **LLAMA3_8B)
  # the 1023 prompt steps always go through the one-launch block kernel (three dispatches per token: a counter run intercepts every
  # dispatch); the four decode steps that are measured take the per-op launches unless --fused is given
  model = Transformer(c, synth_state(c, seed=1003), max_new=16, fused=True)
  rng = np.random.default_rng(1003)
  model.prefill([int(t) for t in rng.integers(0, c.vocab_size, size=1024)], False)
  model.check_fused()
  if "--fused" not in sys.argv: model.layer_table = None
  for _ in range(4): model.decode_step(False)
  model.check_fused()
  print("probe done")

if __name__ == "__main__":
  main()
