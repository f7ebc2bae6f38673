"""GPU block dequant vs the oracle: bit-exact (the bar for ggml_data_to_tensor, tinygrad/llm/gguf.py:23-119)."""
import numpy as np, pytest
from oracle import ggml as og
from tinygrad_amd import synth
from tinygrad_amd.runtime import GGML_QUANT

pytestmark = pytest.mark.gpu
TYPES = [2, 3, 6, 7, 8, 12, 13, 14, 18, 21, 22, 23, 39, 41]

def _gpu_dequant(gpu, data, n, t, dtype=np.float32):
  from tinygrad_amd.gguf import ggml_data_to_tensor
  return ggml_data_to_tensor(data, n, t, out_dtype=dtype).numpy()

from conftest import golden_kats

@pytest.mark.parametrize("name,t,n,block,exp", golden_kats(), ids=[k[0] for k in golden_kats()])
def test_golden_fixture_vectors(gpu, name, t, n, block, exp):
  """The committed fixture of the reference tests' vectors through the device kernel, bit for bit."""
  assert _gpu_dequant(gpu, block, n, t).tobytes() == exp.tobytes()

def test_q8_0_reference_kat(gpu):
  # test/unit/test_gguf.py:36-40
  block = np.frombuffer(np.float16(2.0).tobytes() + np.arange(1, 33, dtype=np.int8).tobytes(), dtype=np.uint8).copy()
  np.testing.assert_array_equal(_gpu_dequant(gpu, block, 32, 8), np.arange(1, 33, dtype=np.float32) * 2.0)

def test_mxfp4_reference_kats(gpu):
  # test/unit/test_gguf.py:42-48
  block = np.array([0x80] + list(range(16)), dtype=np.uint8)
  exp = np.array([0., 1., 2., 3., 4., 6., 8., 12., -0., -1., -2., -3., -4., -6., -8., -12.] + [0.] * 16, dtype=np.float32)
  out = _gpu_dequant(gpu, block, 32, 39)
  assert out.tobytes() == exp.tobytes()          # includes the sign of -0.0
  # test/unit/test_gguf.py:89-105 (a real GLM-4.7-Flash block)
  block = np.array([0x7a, 0x29, 0xab, 0x61, 0x10, 0x21, 0x02, 0x4a, 0x15, 0xca, 0x05, 0x01, 0x9b, 0x39, 0x0b, 0x0b, 0x1c], dtype=np.uint8)
  exp = np.array([-0.015625, -0.046875, 0.015625, 0.0, 0.015625, 0.03125, -0.03125, 0.09375, -0.03125, 0.09375, 0.015625, -0.046875,
                  -0.015625, -0.046875, -0.046875, -0.0625, 0.03125, -0.03125, 0.125, 0.015625, 0.03125, 0.0, 0.0625, 0.015625,
                  -0.0625, 0.0, 0.0, -0.015625, 0.046875, 0.0, 0.0, 0.015625], dtype=np.float32)
  np.testing.assert_array_equal(_gpu_dequant(gpu, block, 32, 39), exp)

@pytest.mark.parametrize("t", TYPES)
def test_random_blocks_bit_exact(gpu, t):
  rng = np.random.default_rng(100 + t)
  nel, nby = GGML_QUANT[t]
  nb = 4096 + 37
  data = rng.integers(0, 256, size=(nb, nby), dtype=np.uint8)       # every byte random: includes NaN/Inf/subnormal fp16 scales
  if t == 39: data[:8, 0] = [0, 1, 2, 3, 254, 255, 127, 128]       # E8M0 corner cases incl. the two fp32-subnormal scales
  with np.errstate(all="ignore"): ref = og.ggml_data_to_tensor(data, nb * nel, t)
  out = _gpu_dequant(gpu, data, nb * nel, t)
  same = (out.view(np.uint32) == ref.view(np.uint32)) | (np.isnan(out) & np.isnan(ref))
  assert same.all(), f"type {t}: {np.count_nonzero(~same)} of {same.size} elements differ"

@pytest.mark.parametrize("t", TYPES)
def test_model_path_fp16_cast(gpu, t):
  """TGA_F16 output == RNE fp16 cast of the float32 dequant (the HALF=1 cast at tinygrad/llm/model.py:376)."""
  rng = np.random.default_rng(200 + t)
  data = synth.random_blocks(rng, t, 64, 1024)
  ref = og.ggml_data_to_tensor(data, 64 * 1024, t).astype(np.float16)
  out = _gpu_dequant(gpu, data, 64 * 1024, t, np.float16)
  assert out.tobytes() == ref.tobytes()

def test_empty_and_unknown_type(gpu):
  from tinygrad_amd.gguf import ggml_data_to_tensor
  assert ggml_data_to_tensor(np.zeros(0, dtype=np.uint8), 0, 2).numpy().size == 0
  with pytest.raises(ValueError): ggml_data_to_tensor(np.zeros(512, dtype=np.uint8), 256, 1337)   # test/unit/test_gguf.py:114-116

def test_lm_head_sized_q6_k(gpu):
  """A full-size slice property: dequant of the first and last 64 rows of a 128256x4096 Q6_K tensor addressed inside one big buffer."""
  rng = np.random.default_rng(7)
  rows, k = 2048, 4096
  data = synth.random_blocks(rng, 14, rows, k)
  out = _gpu_dequant(gpu, data, rows * k, 14)
  ref = og.ggml_data_to_tensor(data, rows * k, 14)
  assert out.tobytes() == ref.tobytes()

def test_synth_q4_k_writer_produces_valid_blocks(gpu):
  """tga_synth_weights(Q4_K): the blocks decode (oracle) to within one quantization step of U(-amp, amp) values: max |w| <= amp * (1 + 1/15)
  and the values are spread (not a constant), i.e. a valid block stream of the right magnitude."""
  n, amp = 256 * 64, 0.02
  buf = gpu.Buffer((n // 256 * 144,), np.uint8)
  gpu.check(gpu.lib().tga_synth_weights(12, buf.ptr, n, 77, amp, None))
  w = og.ggml_data_to_tensor(buf.numpy(), n, 12)
  assert np.isfinite(w).all() and np.abs(w).max() <= amp * 1.1 and w.std() > amp * 0.4
  assert _gpu_dequant(gpu, buf.numpy(), n, 12).tobytes() == w.tobytes()
