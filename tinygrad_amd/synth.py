"""Seeded synthetic inputs for the benchmark configurations (random packed blocks with valid fp16 scales).
Pure numpy; generators draw from numpy.random.default_rng(seed) so tests, bench and the CPU baseline see identical bytes."""
from __future__ import annotations
import numpy as np
from tinygrad_amd.runtime import GGML_QUANT, Q4_0, Q4_1, Q5_0, Q5_1, Q8_0, Q4_K, Q5_K, Q6_K, MXFP4

SEEDS = {1: 1001, 2: 1002, 3: 1003, 4: 1004, 5: 1005}

def _scales(rng, nblocks: int, sigma: float = 0.003) -> np.ndarray:
  """fp16 d = |N(0,1)| * sigma as two little-endian bytes per block."""
  return np.float16(np.abs(rng.standard_normal(nblocks)) * sigma).view(np.uint8).reshape(nblocks, 2)

def random_blocks(rng, ggml_type: int, n: int, k: int, sigma: float = 0.003, mx_exp=(119, 124)) -> np.ndarray:
  """(n, k) weight as raw GGUF block bytes: payload bytes uniform in 0..255 (nibbles uniform 0..15), scales valid.
  Q8_0 quants avoid -128 (uniform in [-127, 127]); Q6_K sub-scales are int8 uniform in [-128, 127]; Q4_1 / Q5_1 get a valid d and m, Q5_0 a valid d; Q4_K / Q5_K get valid d and dmin, their packed 6-bit scales and mins are uniform;
  MXFP4 exponent bytes are uniform in [mx_exp[0], mx_exp[1])."""
  nel, nby = GGML_QUANT[ggml_type]
  assert k % nel == 0
  nb = n * (k // nel)
  b = rng.integers(0, 256, size=(nb, nby), dtype=np.uint8)
  if ggml_type in (Q4_0, Q5_0, 18, 21, 22, 23, 41): b[:, :2] = _scales(rng, nb, sigma)   # (18 / 21 / 22 = IQ3_XXS / IQ3_S / IQ2_S, 23 = IQ4_XS, 41 = Q1_0)
  elif ggml_type in (Q4_1, Q5_1):                                       # d > 0 and a signed fp16 minimum of the same magnitude as the weights
    b[:, :2] = _scales(rng, nb, sigma)
    b[:, 2:4] = np.float16(rng.standard_normal(nb) * sigma * 4).view(np.uint8).reshape(nb, 2)
  elif ggml_type == Q8_0:
    b[:, :2] = _scales(rng, nb, sigma)
    b[:, 2:] = rng.integers(-127, 128, size=(nb, 32), dtype=np.int8).view(np.uint8)
  elif ggml_type == Q6_K: b[:, 208:210] = _scales(rng, nb, sigma)
  elif ggml_type in (Q4_K, Q5_K): b[:, 0:2] = _scales(rng, nb, sigma / 8); b[:, 2:4] = _scales(rng, nb, sigma / 8)   # d and dmin; 6-bit scales / mins stay random
  elif ggml_type == MXFP4: b[:, 0] = rng.integers(mx_exp[0], mx_exp[1], size=nb, dtype=np.uint8)
  return b.reshape(-1)

def activations(rng, m: int, k: int, dtype=np.float16) -> np.ndarray:
  return rng.standard_normal((m, k)).astype(np.float32).astype(dtype)

def config1(seed: int = SEEDS[1]):
  """Single Q4_0 dequant-GEMV: W 4096x4096 (d = |N(0,1)|*0.003, nibbles uniform), x fp16 [1,4096] ~ N(0,1)."""
  rng = np.random.default_rng(seed)
  return random_blocks(rng, Q4_0, 4096, 4096), activations(rng, 1, 4096), (4096, 4096)
