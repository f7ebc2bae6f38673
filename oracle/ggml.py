"""numpy restatement of ggml_data_to_tensor (tinygrad/llm/gguf.py:23-119) for the block layouts on the path (Q4_0, Q8_0, Q6_K,
MXFP4, the Q4_K / Q5_K superblocks most GGUF model files are made of, and the older Q4_1 / Q5_0 / Q5_1 blocks),
plus the ggml reference quantizers used only to build synthetic models.  Test infrastructure only."""
import numpy as np

Q4_0, Q8_0, Q4_K, Q5_K, Q6_K, MXFP4, F32, F16 = 2, 8, 12, 13, 14, 39, 0, 1
Q4_1, Q5_0, Q5_1 = 3, 6, 7
IQ4_XS, Q1_0 = 23, 41
IQ3_XXS, IQ3_S, IQ2_S = 18, 21, 22
# {ggml_type: (elements per block, bytes per block)}  tinygrad/llm/gguf.py:20-21
GGML_QUANT = {Q4_0: (32, 18), Q4_1: (32, 20), Q5_0: (32, 22), Q5_1: (32, 24), Q8_0: (32, 34), Q4_K: (256, 144), Q5_K: (256, 176), Q6_K: (256, 210), MXFP4: (32, 17), IQ4_XS: (256, 136), Q1_0: (128, 18),
              IQ3_XXS: (256, 98), IQ3_S: (256, 110), IQ2_S: (256, 82)}
# tinygrad/llm/gguf.py:108-110 (== 2 * E2M1 values; ggml_common.py:218 kvalues_mxfp4)
FP4_LUT = np.array([0.0, 1.0, 2.0, 3.0, 4.0, 6.0, 8.0, 12.0, -0.0, -1.0, -2.0, -3.0, -4.0, -6.0, -8.0, -12.0], dtype=np.float32)

def q_to_uint8(t: np.ndarray, b: int) -> np.ndarray:
  """gguf.py:38-41: unpack 8//b b-bit fields per byte, FIELD-MAJOR over the last axis
  (all field-0 values of the row first, then all field-1 values, ...)."""
  shifts = np.arange(8 // b, dtype=np.uint8) * b
  fields = (t[..., None] >> shifts) & (0xff >> (8 - b))          # (..., nbytes, 8//b)
  return np.swapaxes(fields, -1, -2).reshape(*t.shape[:-1], -1)   # (..., 8//b * nbytes)

def _blocks(data: np.ndarray, n: int, ggml_type: int) -> np.ndarray:
  nel, nby = GGML_QUANT[ggml_type]
  data = np.ascontiguousarray(data).view(np.uint8).reshape(-1)
  return data[:(n // nel) * nby].reshape(-1, nby)                  # gguf.py:45

def _f16(b: np.ndarray) -> np.ndarray: return np.ascontiguousarray(b).view(np.float16).astype(np.float32)

def dequant_q4_0(blocks: np.ndarray) -> np.ndarray:
  """gguf.py:46  (q_to_uint8(qs,4).bitcast(int8) - 8) * float32(fp16 d)"""
  return (q_to_uint8(blocks[:, 2:], 4).view(np.int8) - np.int8(8)).astype(np.float32) * _f16(blocks[:, :2])

def dequant_q4_1(blocks: np.ndarray) -> np.ndarray:
  """gguf.py:47-49  block = fp16 d, fp16 m, 16 nibble bytes: q * d + m"""
  d, m = _f16(blocks[:, 0:2]), _f16(blocks[:, 2:4])
  return q_to_uint8(blocks[:, 4:], 4).astype(np.float32) * d + m

def _dequant_q5(blocks: np.ndarray, one: bool) -> np.ndarray:
  """gguf.py:50-55  Q5_0 (22 B: d, qh[4], qs[16]) / Q5_1 (24 B: d, m, qh[4], qs[16]): q = nibble + 16 * (bit e of the 32-bit qh),
  value = q * d + (m for Q5_1, -16 * d for Q5_0)."""
  d = _f16(blocks[:, :2]); off = 4 if one else 2
  qh = np.swapaxes(q_to_uint8(blocks[:, off:off + 4], 1).reshape(-1, 8, 4), -1, -2).reshape(-1, 32)
  q = (q_to_uint8(blocks[:, off + 4:], 4) + qh * np.uint8(16)).astype(np.float32)
  return q * d + (_f16(blocks[:, 2:4]) if one else np.float32(-16) * d)

def dequant_q5_0(blocks: np.ndarray) -> np.ndarray: return _dequant_q5(blocks, False)
def dequant_q5_1(blocks: np.ndarray) -> np.ndarray: return _dequant_q5(blocks, True)

def dequant_q8_0(blocks: np.ndarray) -> np.ndarray:
  """gguf.py:56  float32(fp16 d) * int8 qs"""
  return _f16(blocks[:, :2]) * np.ascontiguousarray(blocks[:, 2:]).view(np.int8).astype(np.float32)

def dequant_q6_k(blocks: np.ndarray) -> np.ndarray:
  """gguf.py:68-72  d * (int8(xl | xh) - 32) * scales, in that association order"""
  nb = blocks.shape[0]
  xl = q_to_uint8(blocks[:, :128].reshape(nb, 2, 64), 4)
  xh = q_to_uint8(blocks[:, 128:192].reshape(nb, 2, 32), 2) << 4
  scales = np.repeat(np.ascontiguousarray(blocks[:, 192:208]).view(np.int8), 16, axis=1).astype(np.float32)
  d = _f16(blocks[:, 208:210])
  q = ((xl | xh).view(np.int8) - np.int8(32)).reshape(nb, 256).astype(np.float32)
  return (d * q) * scales

def _dequant_q45_k(blocks: np.ndarray, five: bool) -> np.ndarray:
  """gguf.py:57-67  Q4_K (144 B: d, dmin, scales[12], qs[128]) / Q5_K (176 B: d, dmin, scales[12], qh[32], qs[128]):
  (d * sc) * q - dmin * mn per 32-element sub-block, 6-bit sc / mn unpacked from the 12 scale bytes."""
  nb = blocks.shape[0]
  d, dmin = _f16(blocks[:, 0:2])[:, :, None], _f16(blocks[:, 2:4])[:, :, None]
  s = blocks[:, 4:16]
  sc = np.concatenate([s[:, 0:4] & 63, (s[:, 8:12] & 0xF) | ((s[:, 0:4] >> 6) << 4)], axis=-1).astype(np.float32)[:, :, None]
  mn = np.concatenate([s[:, 4:8] & 63, (s[:, 8:12] >> 4) | ((s[:, 4:8] >> 6) << 4)], axis=-1).astype(np.float32)[:, :, None]
  off = 48 if five else 16
  qs = blocks[:, off:off + 128].reshape(nb, 4, 32)
  q = np.stack([qs & 0xF, qs >> 4], axis=2).reshape(nb, 8, 32)          # sub-blocks 2p (low nibbles), 2p+1 (high nibbles)
  if five: q = q + q_to_uint8(blocks[:, 16:48], 1).reshape(nb, 8, 32) * np.uint8(16)
  return ((d * sc) * q.astype(np.float32) - dmin * mn).reshape(nb, 256)

def dequant_q4_k(blocks: np.ndarray) -> np.ndarray: return _dequant_q45_k(blocks, False)
def dequant_q5_k(blocks: np.ndarray) -> np.ndarray: return _dequant_q45_k(blocks, True)

def dequant_mxfp4(blocks: np.ndarray) -> np.ndarray:
  """gguf.py:105-114  d = bitcast_f32((e-1)<<23) (e>=2), 2^-127 (e==1), 2^-128 (e==0); value = LUT[code] * d"""
  e = blocks[:, 0].astype(np.uint32)
  small = np.array([0x00200000, 0x00400000], dtype=np.uint32)[np.clip(e, 0, 1)]
  d = np.where(e < 2, small, (e - 1) * np.uint32(0x00800000)).astype(np.uint32).view(np.float32)[:, None]
  return FP4_LUT[q_to_uint8(blocks[:, 1:17], 4)] * d

# ggml's kvalues_iq4nl (ggml-common.h; the reference reads it from its generated ggml_common module, gguf.py:98)
KVALUES_IQ4NL = np.array([-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113], dtype=np.float32)

def dequant_iq4_xs(blocks: np.ndarray) -> np.ndarray:
  """gguf.py:96-104  136 B: d, scales_h (u16), scales_l[4], qs[128]; eight sub-blocks of 32: scale = int8(nibble ib of scales_l |
  (2 bits ib of scales_h) << 4) - 32; value = d * scale * lut[nibble], low nibbles = elements 0..15, high = 16..31 of the sub-block."""
  nb = blocks.shape[0]
  d = _f16(blocks[:, :2]).reshape(nb, 1, 1)
  sl = blocks[:, 4:8]
  scales_l = np.stack([sl & 0xF, sl >> 4], axis=2).reshape(nb, 8)
  sh = np.ascontiguousarray(blocks[:, 2:4]).view(np.uint16).reshape(nb, 1)
  scales_h = ((sh >> (np.arange(8, dtype=np.uint16) * 2)[None, :]) & 3).astype(np.uint8)
  scales = ((scales_l | (scales_h << 4)).view(np.int8).astype(np.int32) - 32).astype(np.float32).reshape(nb, 8, 1)
  qs = blocks[:, 8:].reshape(nb, 8, 16)
  q = np.concatenate([qs & 0xF, qs >> 4], axis=2)
  return ((d * scales) * KVALUES_IQ4NL[q]).reshape(nb, 256)

def dequant_q1_0(blocks: np.ndarray) -> np.ndarray:
  """gguf.py:115-118  18 B: fp16 d, 128 sign bits (element e = bit e % 8 of byte e // 8): d * (2 bit - 1).  The reference's result is
  float16 (+-d); it is returned here as the same values in float32."""
  bits = np.swapaxes(q_to_uint8(blocks[:, 2:], 1).reshape(-1, 8, 16), -1, -2).reshape(-1, 128).view(np.int8)
  return _f16(blocks[:, :2]) * (bits.astype(np.float32) * 2 - 1)

def _sign_pm1(sign_bytes: np.ndarray) -> np.ndarray:
  """bit k of byte b -> element 8 b + k: +1.0 where the bit is clear, -1.0 where it is set (gguf.py:79, 86, 92)."""
  return np.where(q_to_uint8(sign_bytes.reshape(-1, sign_bytes.shape[-1], 1), 1).reshape(sign_bytes.shape[0], -1) == 0, np.float32(1), np.float32(-1))

def dequant_iq3_xxs(blocks: np.ndarray) -> np.ndarray:
  """gguf.py:73-81  98 B: d, 64 codebook indices (4 values each), 8 uint32 words; word ib of sub-block ib (32 values): bits 28..31 =
  scale s, four 7-bit sign indices at bits 0, 7, 14, 21 (one per 8 values; the 8th sign bit makes the parity even).
  value = d * (s + 0.5) * 0.5 * grid * sign."""
  from oracle.iq_grids import grid
  nb = blocks.shape[0]
  d = _f16(blocks[:, :2]).reshape(nb, 1, 1, 1)
  words = np.ascontiguousarray(blocks[:, 66:98]).view(np.uint32).reshape(nb, 8)
  db = d * ((words >> 28).astype(np.float32) + np.float32(0.5)).reshape(nb, 8, 1, 1) * np.float32(0.5)
  sign_idx = ((words[:, :, None] >> np.array([0, 7, 14, 21], dtype=np.uint32)) & 0x7F).reshape(nb, 32)
  even_signs = np.array([i | (0x80 if bin(i).count("1") % 2 else 0) for i in range(128)], dtype=np.uint8)
  signs = _sign_pm1(even_signs[sign_idx]).reshape(nb, 8, 4, 8)
  g = grid("iq3xxs")[blocks[:, 2:66]].reshape(nb, 8, 4, 8)
  return (db * g * signs).reshape(nb, 256)

def dequant_iq3_s(blocks: np.ndarray) -> np.ndarray:
  """gguf.py:82-88  110 B: d, qs[64] (low 8 index bits), qh[8] (bit i % 8 of qh[i // 8] = 9th bit of index i), signs[32], scales[4]
  (nibble ib of sub-block ib).  value = d * (1 + 2 nibble) * grid[index] * sign."""
  from oracle.iq_grids import grid
  nb = blocks.shape[0]
  d = _f16(blocks[:, :2]).reshape(nb, 1, 1, 1)
  scales = (1 + 2 * q_to_uint8(blocks[:, 106:110].reshape(nb, 4, 1), 4).reshape(nb, 8)).astype(np.float32).reshape(nb, 8, 1, 1)
  qh = q_to_uint8(blocks[:, 66:74].reshape(nb, 8, 1), 1).reshape(nb, 64).astype(np.uint16)
  signs = _sign_pm1(blocks[:, 74:106]).reshape(nb, 8, 4, 8)
  q = blocks[:, 2:66].astype(np.uint16) + (qh << 8)
  return (d * scales * grid("iq3s")[q].reshape(nb, 8, 4, 8) * signs).reshape(nb, 256)

def dequant_iq2_s(blocks: np.ndarray) -> np.ndarray:
  """gguf.py:89-95  82 B: d, qs[32] (low 8 index bits), signs[32], qh[8] (2-bit field i % 4 of qh[i // 4] = index bits 8..9), scales[8]
  (nibble g of the g-th run of 16 values).  value = d * (nibble + 0.5) * 0.25 * grid[index] * sign, 8 values per index."""
  from oracle.iq_grids import grid
  nb = blocks.shape[0]
  d = _f16(blocks[:, :2]).reshape(nb, 1, 1, 1)
  db = d * (q_to_uint8(blocks[:, 74:82].reshape(nb, 8, 1), 4).reshape(nb, 16).astype(np.float32) + np.float32(0.5)).reshape(nb, 16, 1, 1) * np.float32(0.25)
  signs = _sign_pm1(blocks[:, 34:66]).reshape(nb, 16, 2, 8)
  qh = q_to_uint8(blocks[:, 66:74].reshape(nb, 8, 1), 2).reshape(nb, 32).astype(np.uint16)
  q = blocks[:, 2:34].astype(np.uint16) + (qh << 8)
  return (db * grid("iq2s")[q].reshape(nb, 16, 2, 8) * signs).reshape(nb, 256)

_DEQ = {IQ3_XXS: dequant_iq3_xxs, IQ3_S: dequant_iq3_s, IQ2_S: dequant_iq2_s, IQ4_XS: dequant_iq4_xs, Q1_0: dequant_q1_0, Q4_0: dequant_q4_0, Q4_1: dequant_q4_1, Q5_0: dequant_q5_0, Q5_1: dequant_q5_1, Q8_0: dequant_q8_0, Q4_K: dequant_q4_k, Q5_K: dequant_q5_k, Q6_K: dequant_q6_k, MXFP4: dequant_mxfp4}

def ggml_data_to_tensor(data: np.ndarray, n: int, ggml_type: int) -> np.ndarray:
  """gguf.py:23-119 restricted to the types on the path; returns flat float32 of n elements."""
  if ggml_type == F32: return np.ascontiguousarray(data).view(np.uint8)[:4 * n].view(np.float32).copy()
  if ggml_type == F16: return np.ascontiguousarray(data).view(np.uint8)[:2 * n].view(np.float16).copy()
  if ggml_type not in _DEQ: raise ValueError(f"GGML type '{ggml_type}' is not supported!")   # gguf.py:119
  return _DEQ[ggml_type](_blocks(data, n, ggml_type)).reshape(-1)[:n]

def row_bytes(ggml_type: int, k: int) -> int:
  nel, nby = GGML_QUANT[ggml_type]
  assert k % nel == 0
  return k // nel * nby

# ---------------------------------------------------------------------------------------------------------------
# Quantizers.  The reference has none (weights arrive quantized inside GGUF files); these restate ggml's published
# reference quantizers (ggml-quants.c quantize_row_q4_0_ref / q8_0_ref / q6_K_ref is NOT restated: Q6_K synthetic
# weights use the simpler rule documented below) and exist only to build synthetic models.
# ---------------------------------------------------------------------------------------------------------------
def quantize_q4_0(w: np.ndarray) -> np.ndarray:
  """ggml rule: per 32 block, max = signed value of largest magnitude, d = max / -8, id = 1/d (0 if d == 0),
  q = min(15, int8(x*id + 8.5)); byte j = q[j] | q[j+16] << 4; d stored as fp16."""
  x = np.ascontiguousarray(w, dtype=np.float32).reshape(-1, 32)
  idx = np.argmax(np.abs(x), axis=1)
  mx = x[np.arange(x.shape[0]), idx]
  d = mx / np.float32(-8.0)
  with np.errstate(divide="ignore"): idv = np.where(d != 0, np.float32(1.0) / d, np.float32(0)).astype(np.float32)
  q = np.minimum(15, (x * idv[:, None] + np.float32(8.5)).astype(np.int8)).astype(np.uint8)
  out = np.empty((x.shape[0], 18), dtype=np.uint8)
  out[:, :2] = d.astype(np.float16).view(np.uint8).reshape(-1, 2)
  out[:, 2:] = q[:, :16] | (q[:, 16:] << 4)
  return out.reshape(-1)

def _pack_q5_bits(q: np.ndarray) -> np.ndarray:
  """fifth bits of the 32 quants of each block as the little-endian 32-bit qh (bit e = element e), 4 bytes per block"""
  bits = ((q >> 4) & 1).astype(np.uint32) << np.arange(32, dtype=np.uint32)[None, :]
  return np.bitwise_or.reduce(bits, axis=1).astype("<u4").view(np.uint8).reshape(-1, 4)

def quantize_q4_1(w: np.ndarray) -> np.ndarray:
  """ggml rule (quantize_row_q4_1_ref): d = (max - min) / 15, m = min, q = min(15, int((x - min) / d + 0.5)); d, m stored as fp16."""
  x = np.ascontiguousarray(w, dtype=np.float32).reshape(-1, 32)
  mn, mx = x.min(axis=1), x.max(axis=1)
  d = (mx - mn) / np.float32(15)
  with np.errstate(divide="ignore"): idv = np.where(d != 0, np.float32(1.0) / d, np.float32(0)).astype(np.float32)
  q = np.minimum(15, ((x - mn[:, None]) * idv[:, None] + np.float32(0.5)).astype(np.int32)).astype(np.uint8)
  out = np.empty((x.shape[0], 20), dtype=np.uint8)
  out[:, 0:2] = d.astype(np.float16).view(np.uint8).reshape(-1, 2); out[:, 2:4] = mn.astype(np.float16).view(np.uint8).reshape(-1, 2)
  out[:, 4:] = q[:, :16] | (q[:, 16:] << 4)
  return out.reshape(-1)

def quantize_q5_0(w: np.ndarray) -> np.ndarray:
  """ggml rule (quantize_row_q5_0_ref): max = signed value of largest magnitude, d = max / -16, q = min(31, int8(x / d + 16.5));
  nibbles in qs (element j low, j + 16 high), fifth bits in qh."""
  x = np.ascontiguousarray(w, dtype=np.float32).reshape(-1, 32)
  mx = x[np.arange(x.shape[0]), np.argmax(np.abs(x), axis=1)]
  d = mx / np.float32(-16.0)
  with np.errstate(divide="ignore"): idv = np.where(d != 0, np.float32(1.0) / d, np.float32(0)).astype(np.float32)
  q = np.minimum(31, (x * idv[:, None] + np.float32(16.5)).astype(np.int8)).astype(np.uint8)
  out = np.empty((x.shape[0], 22), dtype=np.uint8)
  out[:, 0:2] = d.astype(np.float16).view(np.uint8).reshape(-1, 2)
  out[:, 2:6] = _pack_q5_bits(q)
  out[:, 6:] = (q[:, :16] & 0xF) | ((q[:, 16:] & 0xF) << 4)
  return out.reshape(-1)

def quantize_q5_1(w: np.ndarray) -> np.ndarray:
  """ggml rule (quantize_row_q5_1_ref): d = (max - min) / 31, m = min, q = uint8((x - min) / d + 0.5)."""
  x = np.ascontiguousarray(w, dtype=np.float32).reshape(-1, 32)
  mn, mx = x.min(axis=1), x.max(axis=1)
  d = (mx - mn) / np.float32(31)
  with np.errstate(divide="ignore"): idv = np.where(d != 0, np.float32(1.0) / d, np.float32(0)).astype(np.float32)
  q = np.minimum(31, ((x - mn[:, None]) * idv[:, None] + np.float32(0.5)).astype(np.int32)).astype(np.uint8)
  out = np.empty((x.shape[0], 24), dtype=np.uint8)
  out[:, 0:2] = d.astype(np.float16).view(np.uint8).reshape(-1, 2); out[:, 2:4] = mn.astype(np.float16).view(np.uint8).reshape(-1, 2)
  out[:, 4:8] = _pack_q5_bits(q)
  out[:, 8:] = (q[:, :16] & 0xF) | ((q[:, 16:] & 0xF) << 4)
  return out.reshape(-1)

def quantize_q8_0(w: np.ndarray) -> np.ndarray:
  """ggml rule: d = amax / 127, q = round(x / d) (round half away from zero, as roundf)."""
  x = np.ascontiguousarray(w, dtype=np.float32).reshape(-1, 32)
  d = np.abs(x).max(axis=1) / np.float32(127.0)
  with np.errstate(divide="ignore"): idv = np.where(d != 0, np.float32(1.0) / d, np.float32(0)).astype(np.float32)
  v = x * idv[:, None]
  q = (np.sign(v) * np.floor(np.abs(v) + np.float32(0.5))).astype(np.int8)
  out = np.empty((x.shape[0], 34), dtype=np.uint8)
  out[:, :2] = d.astype(np.float16).view(np.uint8).reshape(-1, 2)
  out[:, 2:] = q.view(np.uint8)
  return out.reshape(-1)

def quantize_q6_k(w: np.ndarray) -> np.ndarray:
  """Simple absmax rule (NOT ggml's iterative make_qx_quants search): per 16-group scale s_g = amax_g / 31,
  d = max_g |s_g| / 127, sc_g = round(s_g / d) in int8, q = clamp(round(x / (d*sc_g)), -32, 31) + 32.
  The byte packing is exactly the layout dequant_q6_k / gguf.py:68-72 decodes."""
  x = np.ascontiguousarray(w, dtype=np.float32).reshape(-1, 16, 16)
  nb = x.shape[0]
  s = np.abs(x).max(axis=2) / np.float32(31.0)
  d = (s.max(axis=1) / np.float32(127.0)).astype(np.float16).astype(np.float32)
  with np.errstate(divide="ignore", invalid="ignore"):
    sc = np.where(d[:, None] > 0, np.rint(s / d[:, None]), 0).clip(-128, 127).astype(np.int8)
    eff = d[:, None] * sc.astype(np.float32)
    q = np.where(eff[:, :, None] != 0, np.rint(x / eff[:, :, None]), 0).clip(-32, 31).astype(np.int8)
  u = (q.reshape(nb, 256).astype(np.int16) + 32).astype(np.uint8)               # 0..63
  lo, hi = (u & 0xF).reshape(nb, 2, 4, 32), (u >> 4).reshape(nb, 2, 4, 32)       # [half][32-group j][l]
  out = np.empty((nb, 210), dtype=np.uint8)
  ql = np.empty((nb, 2, 64), dtype=np.uint8)
  ql[:, :, :32] = lo[:, :, 0] | (lo[:, :, 2] << 4)
  ql[:, :, 32:] = lo[:, :, 1] | (lo[:, :, 3] << 4)
  out[:, :128] = ql.reshape(nb, 128)
  out[:, 128:192] = (hi[:, :, 0] | (hi[:, :, 1] << 2) | (hi[:, :, 2] << 4) | (hi[:, :, 3] << 6)).reshape(nb, 64)
  out[:, 192:208] = sc.view(np.uint8)
  out[:, 208:210] = d.astype(np.float16).view(np.uint8).reshape(-1, 2)
  return out.reshape(-1)

def _quantize_q45_k(w: np.ndarray, five: bool) -> np.ndarray:
  """Simple min/max rule (NOT ggml's iterative make_qkx2_quants search): per 32-weight sub-block min m = max(0, -min x),
  scale s = (max x + m) / qmax; superblock d = max s / 63, dmin = max m / 63 (fp16); 6-bit sc = round(s / d), mn = round(m / dmin);
  q = clamp(round((x + dmin mn) / (d sc)), 0, qmax).  The byte packing is exactly the layout dequant_q4_k / dequant_q5_k decode."""
  qmax = 31 if five else 15
  x = np.ascontiguousarray(w, dtype=np.float32).reshape(-1, 8, 32)
  nb = x.shape[0]
  m = np.maximum(0, -x.min(axis=2)); s = (x.max(axis=2) + m) / np.float32(qmax)
  d = (s.max(axis=1) / np.float32(63)).astype(np.float16).astype(np.float32); dmin = (m.max(axis=1) / np.float32(63)).astype(np.float16).astype(np.float32)
  with np.errstate(divide="ignore", invalid="ignore"):
    sc = np.where(d[:, None] > 0, np.rint(s / d[:, None]), 0).clip(0, 63).astype(np.uint8)
    mn = np.where(dmin[:, None] > 0, np.rint(m / dmin[:, None]), 0).clip(0, 63).astype(np.uint8)
    eff = d[:, None] * sc.astype(np.float32)
    q = np.where(eff[:, :, None] > 0, np.rint((x + (dmin[:, None] * mn.astype(np.float32))[:, :, None]) / eff[:, :, None]), 0).clip(0, qmax).astype(np.uint8)
  out = np.zeros((nb, 176 if five else 144), dtype=np.uint8)
  out[:, 0:2] = d.astype(np.float16).view(np.uint8).reshape(-1, 2); out[:, 2:4] = dmin.astype(np.float16).view(np.uint8).reshape(-1, 2)
  sb = out[:, 4:16]                                                              # inverse of get_scale_min_k4
  sb[:, 0:4] = (sc[:, 0:4] & 63) | ((sc[:, 4:8] >> 4) << 6)
  sb[:, 4:8] = (mn[:, 0:4] & 63) | ((mn[:, 4:8] >> 4) << 6)
  sb[:, 8:12] = (sc[:, 4:8] & 0xF) | ((mn[:, 4:8] & 0xF) << 4)
  off = 48 if five else 16
  out[:, off:off + 128] = ((q[:, 0::2] & 0xF) | ((q[:, 1::2] & 0xF) << 4)).reshape(nb, 128)
  if five: out[:, 16:48] = np.bitwise_or.reduce(((q >> 4) & 1) << np.arange(8, dtype=np.uint8)[None, :, None], axis=1)
  return out.reshape(-1)

def quantize_iq4_xs(w: np.ndarray) -> np.ndarray:
  """Simple rule (NOT ggml's search): per 32-weight sub-block s = amax / 127, superblock d = max s / 31 (fp16), 6-bit field ls = 32 + round(s / d)
  (positive scales only), code = index of the kvalues_iq4nl entry nearest to x / (d (ls - 32)).  Packing as dequant_iq4_xs decodes."""
  x = np.ascontiguousarray(w, dtype=np.float32).reshape(-1, 8, 32)
  nb = x.shape[0]
  sb = np.abs(x).max(axis=2) / np.float32(127)
  d = (sb.max(axis=1) / np.float32(31)).astype(np.float16).astype(np.float32)
  with np.errstate(divide="ignore", invalid="ignore"):
    ls = np.where(d[:, None] > 0, np.rint(sb / d[:, None]), 0).clip(0, 31).astype(np.uint8) + np.uint8(32)
    eff = d[:, None] * (ls.astype(np.float32) - 32)
    t = np.where(eff[:, :, None] > 0, x / eff[:, :, None], 0)
  code = np.abs(t[..., None] - KVALUES_IQ4NL[None, None, None, :]).argmin(-1).astype(np.uint8)
  out = np.zeros((nb, 136), dtype=np.uint8)
  out[:, 0:2] = d.astype(np.float16).view(np.uint8).reshape(-1, 2)
  sh = np.zeros(nb, dtype=np.uint16)
  for ib in range(8): sh |= ((ls[:, ib] >> 4).astype(np.uint16) << np.uint16(2 * ib))
  out[:, 2:4] = sh.view(np.uint8).reshape(-1, 2)
  out[:, 4:8] = (ls[:, 0::2] & 0xF) | ((ls[:, 1::2] & 0xF) << 4)
  out[:, 8:] = (code[:, :, :16] | (code[:, :, 16:] << 4)).reshape(nb, 128)
  return out.reshape(-1)

def quantize_q1_0(w: np.ndarray) -> np.ndarray:
  """d = mean |x| over the 128-weight block (fp16), bit = x >= 0.  Packing as dequant_q1_0 decodes."""
  x = np.ascontiguousarray(w, dtype=np.float32).reshape(-1, 128)
  out = np.zeros((x.shape[0], 18), dtype=np.uint8)
  out[:, 0:2] = np.abs(x).mean(axis=1).astype(np.float16).view(np.uint8).reshape(-1, 2)
  out[:, 2:] = np.packbits((x >= 0).astype(np.uint8).reshape(-1, 16, 8), axis=2, bitorder="little").reshape(-1, 16)
  return out.reshape(-1)

def _nearest_entry(mag: np.ndarray, table: np.ndarray) -> np.ndarray:
  """index of the codebook entry (rows of `table`) nearest in L2 to every row of `mag`."""
  return (np.float32(-2) * (mag @ table.T) + (table * table).sum(1)[None, :]).argmin(1)

def _d_and_steps(amax_run: np.ndarray, top: float, step_of_d, n_steps: int = 16):
  """block scale d (fp16) and per-run integer step so that step_of_d(step) * d * top covers the run's largest magnitude."""
  eff = amax_run / np.float32(top)
  d = (eff.max(axis=1, keepdims=True) / np.float32(step_of_d(n_steps - 1))).astype(np.float16).astype(np.float32)
  safe = np.where(d > 0, d, np.float32(1))
  steps = np.arange(n_steps, dtype=np.float32)
  step = np.abs(eff[..., None] / safe[..., None] - step_of_d(steps)[None, None, :]).argmin(-1)
  return d, step.astype(np.uint8), safe * step_of_d(step.astype(np.float32))

def quantize_iq3_xxs(w: np.ndarray) -> np.ndarray:
  """Simple IQ3_XXS writer for synthetic models (not ggml's search): per 32 weights the 4-bit step nearest to max|x| / 62, per 4 weights the
  nearest codebook entry; where a run of eight has an odd number of negative weights the smallest one loses its sign (the format stores
  seven sign bits and fixes the eighth by parity).  Packing as dequant_iq3_xxs decodes."""
  from oracle.iq_grids import grid
  x = np.ascontiguousarray(w, dtype=np.float32).reshape(-1, 8, 32); nb = x.shape[0]
  d, s, db = _d_and_steps(np.abs(x).max(-1), 62, lambda t: (t + np.float32(0.5)) * np.float32(0.5))
  idx = _nearest_entry((np.abs(x) / db[..., None]).reshape(-1, 4), grid("iq3xxs")).reshape(nb, 64)
  neg = (x < 0).reshape(nb, 32, 8)
  odd = neg.sum(-1) % 2 == 1
  flip = np.abs(x).reshape(nb, 32, 8).argmin(-1)
  neg[odd, flip[odd]] ^= True
  s7 = (neg[:, :, :7] * (1 << np.arange(7))).sum(-1).astype(np.uint32).reshape(nb, 8, 4)
  words = (s.astype(np.uint32) << 28) | (s7 << (7 * np.arange(4, dtype=np.uint32))).sum(-1).astype(np.uint32)
  out = np.zeros((nb, 98), dtype=np.uint8)
  out[:, 0:2] = d.astype(np.float16).view(np.uint8).reshape(-1, 2)
  out[:, 2:66] = idx.astype(np.uint8)
  out[:, 66:98] = np.ascontiguousarray(words.astype("<u4")).view(np.uint8).reshape(nb, 32)
  return out.reshape(-1)

def quantize_iq3_s(w: np.ndarray) -> np.ndarray:
  """Simple IQ3_S writer (not ggml's search): per 32 weights the odd multiplier 1 + 2 nibble nearest to max|x| / 15 / d, per 4 weights the nearest of
  the 512 codebook entries, one sign bit per weight.  Packing as dequant_iq3_s decodes."""
  from oracle.iq_grids import grid
  x = np.ascontiguousarray(w, dtype=np.float32).reshape(-1, 8, 32); nb = x.shape[0]
  d, nib, dl = _d_and_steps(np.abs(x).max(-1), 15, lambda t: 1 + 2 * t)
  idx = _nearest_entry((np.abs(x) / dl[..., None]).reshape(-1, 4), grid("iq3s")).reshape(nb, 64)
  out = np.zeros((nb, 110), dtype=np.uint8)
  out[:, 0:2] = d.astype(np.float16).view(np.uint8).reshape(-1, 2)
  out[:, 2:66] = (idx & 255).astype(np.uint8)
  out[:, 66:74] = np.packbits((idx >> 8).astype(np.uint8).reshape(nb, 8, 8), axis=2, bitorder="little").reshape(nb, 8)
  out[:, 74:106] = np.packbits((x < 0).astype(np.uint8).reshape(nb, 32, 8), axis=2, bitorder="little").reshape(nb, 32)
  out[:, 106:110] = nib[:, 0::2] | (nib[:, 1::2] << 4)
  return out.reshape(-1)

def quantize_iq2_s(w: np.ndarray) -> np.ndarray:
  """Simple IQ2_S writer (not ggml's search): per 16 weights the nibble whose (nibble + 0.5) / 4 is nearest to max|x| / 43 / d, per 8 weights the nearest
  of the 1024 codebook entries, one sign bit per weight.  Packing as dequant_iq2_s decodes."""
  from oracle.iq_grids import grid
  x = np.ascontiguousarray(w, dtype=np.float32).reshape(-1, 16, 16); nb = x.shape[0]
  d, nib, dl = _d_and_steps(np.abs(x).max(-1), 43, lambda t: (t + np.float32(0.5)) * np.float32(0.25))
  idx = _nearest_entry((np.abs(x) / dl[..., None]).reshape(-1, 8), grid("iq2s")).reshape(nb, 32)
  out = np.zeros((nb, 82), dtype=np.uint8)
  out[:, 0:2] = d.astype(np.float16).view(np.uint8).reshape(-1, 2)
  out[:, 2:34] = (idx & 255).astype(np.uint8)
  out[:, 34:66] = np.packbits((x < 0).astype(np.uint8).reshape(nb, 32, 8), axis=2, bitorder="little").reshape(nb, 32)
  hi = (idx >> 8).astype(np.uint8).reshape(nb, 8, 4)
  out[:, 66:74] = hi[:, :, 0] | (hi[:, :, 1] << 2) | (hi[:, :, 2] << 4) | (hi[:, :, 3] << 6)
  out[:, 74:82] = nib[:, 0::2] | (nib[:, 1::2] << 4)
  return out.reshape(-1)

def quantize_q4_k(w: np.ndarray) -> np.ndarray: return _quantize_q45_k(w, False)
def quantize_q5_k(w: np.ndarray) -> np.ndarray: return _quantize_q45_k(w, True)
