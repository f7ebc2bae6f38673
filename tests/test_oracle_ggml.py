"""Pins the oracle's block dequant (no GPU): the reference's own known-answer vectors, the independent scalar C restatement of
the published ggml loops, brute force on the bit layout, and closed forms."""
import numpy as np, pytest
from oracle import ggml as og, cref

from conftest import golden_kats

@pytest.mark.parametrize("name,t,n,block,exp", golden_kats(), ids=[k[0] for k in golden_kats()])
def test_golden_fixture_vectors(name, t, n, block, exp):
  """The committed fixture of the reference tests' vectors, bit for bit (incl. the sign of -0.0)."""
  assert og.ggml_data_to_tensor(block, n, t).tobytes() == exp.tobytes()

def test_q8_0_reference_kat():
  # test/unit/test_gguf.py:36-40
  block = np.frombuffer(np.float16(2.0).tobytes() + np.arange(1, 33, dtype=np.int8).tobytes(), dtype=np.uint8).copy()
  np.testing.assert_array_equal(og.ggml_data_to_tensor(block, 32, 8), np.arange(1, 33, dtype=np.float32) * 2.0)

def test_mxfp4_reference_kat_hardcoded():
  # test/unit/test_gguf.py:42-48: pins low-nibbles-first order, scale 2^(E-128) and the doubled table
  block = np.array([0x80] + list(range(16)), dtype=np.uint8)
  exp = np.array([0., 1., 2., 3., 4., 6., 8., 12., -0., -1., -2., -3., -4., -6., -8., -12.] + [0.] * 16, dtype=np.float32)
  np.testing.assert_array_equal(og.ggml_data_to_tensor(block, 32, 39), exp)

def test_mxfp4_reference_closed_form_seed42():
  # test/unit/test_gguf.py:65-87: independent E2M1 x E8M0 formula incl. E < 2 subnormal scales
  def decode(code, E):
    sign = -1.0 if (code & 0b1000) else 1.0
    exp, mant = (code >> 1) & 0b11, code & 0b1
    val = 2 * ((1.0 + 0.5 * mant) * np.exp2(exp - 1) if exp else 0.5 * mant)
    return sign * val * (np.exp2(E - 128) if E >= 2 else np.exp2(-127 if E == 1 else -128))
  blocks, expected = [], []
  rng = np.random.default_rng(42)
  for _ in range(4):
    E = rng.integers(0, 256)
    codes = rng.integers(0, 16, size=32, dtype=np.uint8)
    blocks.append(np.array([E] + [(lo & 0xF) | ((hi & 0xF) << 4) for lo, hi in zip(codes[:16], codes[16:])], dtype=np.uint8))
    expected.extend(decode(int(c), int(E)) for c in codes)
  with np.errstate(over="ignore"):
    out = og.ggml_data_to_tensor(np.concatenate(blocks), len(expected), 39)
    np.testing.assert_array_equal(out, np.array(expected, dtype=np.float32))
  for E in (0, 1, 2):                                        # the two fp32-subnormal scales explicitly
    b = np.array([E] + [0x21] * 16, dtype=np.uint8)
    np.testing.assert_array_equal(og.ggml_data_to_tensor(b, 32, 39), np.array([decode(1, E)] * 16 + [decode(2, E)] * 16, dtype=np.float32))

def test_mxfp4_reference_real_block():
  # test/unit/test_gguf.py:89-105 (first block of GLM-4.7-Flash blk.0.attn_k_b.weight)
  block = np.array([0x7a, 0x29, 0xab, 0x61, 0x10, 0x21, 0x02, 0x4a, 0x15, 0xca, 0x05, 0x01, 0x9b, 0x39, 0x0b, 0x0b, 0x1c], dtype=np.uint8)
  exp = np.array([-0.015625, -0.046875, 0.015625, 0.0, 0.015625, 0.03125, -0.03125, 0.09375, -0.03125, 0.09375, 0.015625, -0.046875,
                  -0.015625, -0.046875, -0.046875, -0.0625, 0.03125, -0.03125, 0.125, 0.015625, 0.03125, 0.0, 0.0625, 0.015625,
                  -0.0625, 0.0, 0.0, -0.015625, 0.046875, 0.0, 0.0, 0.015625], dtype=np.float32)
  np.testing.assert_array_equal(og.ggml_data_to_tensor(block, 32, 39), exp)

def test_q4_0_brute_force_layout():
  """Every nibble position: w[j] = (low nibble of qs[j]) - 8, w[j+16] = (high nibble of qs[j]) - 8, times d (ggml_common.py:21)."""
  for j in range(16):
    for nib, hi in ((0x0, False), (0xF, False), (0x5, True), (0xF, True)):
      b = np.zeros(18, dtype=np.uint8); b[:2] = np.frombuffer(np.float16(0.5).tobytes(), np.uint8)
      b[2:] = 0x88                                            # all weights 0
      b[2 + j] = (0x80 | nib) if not hi else (0x08 | (nib << 4))
      exp = np.zeros(32, dtype=np.float32); exp[j + (16 if hi else 0)] = (nib - 8) * 0.5
      np.testing.assert_array_equal(og.ggml_data_to_tensor(b, 32, 2), exp)

def test_q6_k_brute_force_layout():
  """One weight at a time: ggml's dequantize_row_q6_K index map (ql/qh/scale position of element e)."""
  for e in [0, 1, 15, 16, 31, 32, 63, 64, 95, 96, 127, 128, 129, 160, 200, 255]:
    b = np.zeros(210, dtype=np.uint8)
    b[208:210] = np.frombuffer(np.float16(1.0).tobytes(), np.uint8)
    b[192:208] = 1                                            # all sub-scales 1
    # all quants = 32 (-> 0): low nibble 0, high bits 2
    b[:128] = 0x00; b[128:192] = 0xAA
    half, j, l = e >> 7, (e >> 5) & 3, e & 31
    q = 63                                                    # -> +31
    qi = 64 * half + (32 if j & 1 else 0) + l
    b[qi] = (int(b[qi]) & (0x0F if j & 2 else 0xF0)) | ((q & 0xF) << (4 if j & 2 else 0))
    hi_i = 128 + 32 * half + l
    b[hi_i] = (int(b[hi_i]) & (0xFF ^ (3 << (2 * j)))) | ((q >> 4) << (2 * j))
    b[192 + e // 16] = 0xFD                                   # int8 -3
    exp = np.zeros(256, dtype=np.float32); exp[e] = 31 * -3.0
    out = og.ggml_data_to_tensor(b, 256, 14)
    np.testing.assert_array_equal(out, exp, err_msg=f"element {e}")

@pytest.mark.parametrize("t", [2, 3, 6, 7, 8, 12, 13, 14, 18, 21, 22, 23, 39, 41])
def test_numpy_restatement_equals_scalar_c_loops(t):
  """Vectorised restatement of tinygrad/llm/gguf.py (field-major q_to_uint8) == independent scalar loops of the published ggml
  routines, bit for bit, on fully random bytes (NaN/Inf/subnormal scales included)."""
  rng = np.random.default_rng(t)
  nel, nby = og.GGML_QUANT[t]
  data = rng.integers(0, 256, size=(2048, nby), dtype=np.uint8)
  if t == 39: data[:6, 0] = [0, 1, 2, 254, 255, 127]
  with np.errstate(all="ignore"): a = og.ggml_data_to_tensor(data, 2048 * nel, t)
  c = cref.dequant(t, data)
  same = (a.view(np.uint32) == c.view(np.uint32)) | (np.isnan(a) & np.isnan(c))
  assert same.all()

@pytest.mark.parametrize("t", [12, 13])
def test_q4_k_q5_k_brute_force_layout(t):
  """One weight at a time against ggml's dequantize_row_q4_K / q5_K index map: element e of a superblock sits in sub-block e // 32
  (6-bit scale / min from get_scale_min_k4), nibble (e // 32) & 1 of qs[32 * (e // 64) + e % 32], fifth bit = bit e // 32 of qh[e % 32]."""
  nby = og.GGML_QUANT[t][1]; qs_off = 48 if t == 13 else 16
  def put_scale(b, sb, sc, mn):                                 # inverse of get_scale_min_k4
    s = b[4:16]
    if sb < 4: s[sb] = (int(s[sb]) & 0xC0) | sc; s[sb + 4] = (int(s[sb + 4]) & 0xC0) | mn
    else:
      s[sb + 4] = (sc & 0xF) | ((mn & 0xF) << 4)
      s[sb - 4] = (int(s[sb - 4]) & 0x3F) | ((sc >> 4) << 6); s[sb] = (int(s[sb]) & 0x3F) | ((mn >> 4) << 6)
  for e in [0, 1, 31, 32, 33, 63, 64, 100, 127, 128, 160, 191, 192, 223, 224, 255]:
    b = np.zeros(nby, dtype=np.uint8)
    b[0:2] = np.frombuffer(np.float16(0.5).tobytes(), np.uint8); b[2:4] = np.frombuffer(np.float16(0.25).tobytes(), np.uint8)
    sb = e // 32
    put_scale(b, sb, 37, 51)                                    # both above 15: exercises the split high bits
    q = 29 if t == 13 else 13
    byte = qs_off + 32 * (e // 64) + e % 32
    b[byte] = (q & 0xF) << (4 if sb & 1 else 0)
    if t == 13 and q >> 4: b[16 + e % 32] = 1 << sb
    exp = np.zeros(256, dtype=np.float32)
    exp[32 * sb:32 * sb + 32] = -0.25 * 51                      # the sub-block's min applies to all its 32 weights
    exp[e] = (0.5 * 37) * q - 0.25 * 51
    np.testing.assert_array_equal(og.ggml_data_to_tensor(b, 256, t), exp, err_msg=f"element {e}")
    np.testing.assert_array_equal(cref.dequant(t, b[None]).reshape(-1), exp, err_msg=f"element {e} (C)")

@pytest.mark.parametrize("t", [3, 6, 7])
def test_q4_1_q5_0_q5_1_brute_force_layout(t):
  """One weight at a time against ggml's block_q4_1 / block_q5_0 / block_q5_1 (dequantize_row_q4_1 / q5_0 / q5_1): element j < 16 is
  the low nibble of qs[j], element j + 16 the high nibble; the fifth bit of element e is bit e of the little-endian 32-bit qh; the
  value is q * d + m (Q4_1, Q5_1) or (q - 16) * d (Q5_0)."""
  nby = og.GGML_QUANT[t][1]
  qh_off = {3: None, 6: 2, 7: 4}[t]; qs_off = {3: 4, 6: 6, 7: 8}[t]
  d, m = 0.5, -3.25
  for e in range(32):
    for q in ((1, 15) if t == 3 else (1, 15, 16, 31)):
      b = np.zeros(nby, dtype=np.uint8)
      b[0:2] = np.frombuffer(np.float16(d).tobytes(), np.uint8)
      if t != 6: b[2:4] = np.frombuffer(np.float16(m).tobytes(), np.uint8)
      b[qs_off + e % 16] = (q & 0xF) << (4 if e >= 16 else 0)
      if q >> 4: b[qh_off + e // 8] = 1 << (e % 8)
      base = -16 * d if t == 6 else m                              # what a zero quant decodes to
      exp = np.full(32, base, dtype=np.float32); exp[e] = q * d + base
      np.testing.assert_array_equal(og.ggml_data_to_tensor(b, 32, t), exp, err_msg=f"element {e} q {q}")
      np.testing.assert_array_equal(cref.dequant(t, b[None]).reshape(-1), exp, err_msg=f"element {e} q {q} (C)")

def test_q5_0_equals_q4_0_when_fifth_bits_mirror_the_sign():
  """Q5_0 with q5 = 2 * q4 (fifth bit = top bit of the nibble, low bit 0) and half the scale decodes to the Q4_0 values:
  (2 q - 16) * (d / 2) = (q - 8) * d - ties the new decoder to the Q4_0 one the reference's own tests pin."""
  rng = np.random.default_rng(5)
  q4 = rng.integers(0, 16, size=(64, 32)).astype(np.uint8)
  d = np.float16(rng.uniform(0.01, 2.0, 64))
  b4 = np.zeros((64, 18), np.uint8); b4[:, :2] = d.view(np.uint8).reshape(-1, 2); b4[:, 2:] = q4[:, :16] | (q4[:, 16:] << 4)
  q5 = q4 * 2
  b5 = np.zeros((64, 22), np.uint8); b5[:, :2] = (d / np.float16(2)).astype(np.float16).view(np.uint8).reshape(-1, 2)
  b5[:, 2:6] = og._pack_q5_bits(q5); b5[:, 6:] = (q5[:, :16] & 0xF) | ((q5[:, 16:] & 0xF) << 4)
  np.testing.assert_array_equal(og.ggml_data_to_tensor(b5, 64 * 32, 6), og.ggml_data_to_tensor(b4, 64 * 32, 2))

def test_iq4_xs_brute_force_layout():
  """One weight at a time against ggml's block_iq4_xs (dequantize_row_iq4_xs): sub-block ib = e // 32 has the 6-bit scale
  (nibble ib of scales_l) | (bits 2 ib, 2 ib + 1 of scales_h) << 4, minus 32; element j < 16 of it is the low nibble of qs[16 ib + j],
  element j + 16 the high nibble; the nibble indexes kvalues_iq4nl."""
  kv = [-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113]
  for e in [0, 1, 15, 16, 31, 32, 47, 48, 100, 127, 128, 200, 255]:
    for code, ls in ((0, 45), (15, 3), (9, 63)):
      b = np.zeros(136, dtype=np.uint8)
      b[0:2] = np.frombuffer(np.float16(0.25).tobytes(), np.uint8)
      ib, l = e // 32, e % 32
      b[8:] = 0x88                                              # every nibble 8 -> kvalues[8] = 1
      sl = np.zeros(8, np.uint8) + (32 & 0xF); shh = 0
      for k in range(8): shh |= (32 >> 4) << (2 * k)             # all scales 32 -> (32 - 32) = 0: other sub-blocks decode to 0
      sl[ib] = ls & 0xF; shh = (shh & ~(3 << (2 * ib))) | ((ls >> 4) << (2 * ib))
      b[4:8] = sl[0::2] | (sl[1::2] << 4)
      b[2:4] = np.frombuffer(np.uint16(shh).tobytes(), np.uint8)
      byte = 8 + 16 * ib + l % 16
      b[byte] = (0x80 | code) if l < 16 else (0x08 | (code << 4))
      exp = np.zeros(256, dtype=np.float32)
      exp[32 * ib:32 * ib + 32] = 0.25 * (ls - 32) * 1.0          # nibble 8 everywhere else in the sub-block
      exp[e] = 0.25 * (ls - 32) * kv[code]
      np.testing.assert_array_equal(og.ggml_data_to_tensor(b, 256, 23), exp, err_msg=f"element {e}")
      np.testing.assert_array_equal(cref.dequant(23, b[None]).reshape(-1), exp, err_msg=f"element {e} (C)")

def test_codebooks_are_the_published_tables():
  """The three codebooks, expanded as _ggml_iq_grid does (gguf.py:11-13: value i = byte i of the packed word), hash to the SHA-256 of the
  tables the format publishes (ggml-common.h iq3xxs_grid / iq3s_grid / iq2s_grid = tinygrad/runtime/autogen/ggml_common.py:214-216), taken
  from that text; a few entries are also spelled out (little-endian bytes of the published words 0x0c140c14, 0x3e341c04, 0x05090507,
  0x0f0f0101, 0x0819081919191919, 0x192b080819191908)."""
  import hashlib
  from oracle.iq_grids import grid_u8
  want = {"iq3xxs": ((256, 4), "46e35f5a997efdee6c99ce57854c8a0d4f0ff8ca57e5e8a60c0793ea580acf5d"),
          "iq3s": ((512, 4), "bd1af4945a1717c65610b0284e4628b9a1ba3b306fae3a06f6e5f597356e349f"),
          "iq2s": ((1024, 8), "e1aa1473412b0552c2174c30ef22ab4073f6a181b85a17056e8249bd2932fd88")}
  for name, (shape, digest) in want.items():
    g = grid_u8(name)
    assert g.shape == shape and g.dtype == np.uint8
    assert hashlib.sha256(g.tobytes()).hexdigest() == digest, name
    words = sum(g[:, i].astype(np.uint64) << np.uint64(8 * i) for i in range(shape[1]))
    assert (words[1:] > words[:-1]).all(), name                     # the published tables are sorted as integers
  assert grid_u8("iq3xxs")[77].tolist() == [0x14, 0x0c, 0x14, 0x0c] and grid_u8("iq3xxs")[255].tolist() == [0x04, 0x1c, 0x34, 0x3e]
  assert grid_u8("iq3s")[256].tolist() == [7, 5, 9, 5] and grid_u8("iq3s")[511].tolist() == [1, 1, 15, 15]
  assert grid_u8("iq2s")[256].tolist() == [0x19, 0x19, 0x19, 0x19, 0x19, 0x08, 0x19, 0x08] and grid_u8("iq2s")[770].tolist() == [0x08, 0x19, 0x19, 0x19, 0x08, 0x08, 0x2b, 0x19]

_D = np.frombuffer(np.float16(0.25).tobytes(), np.uint8)

def test_iq3_xxs_brute_force_layout():
  """One weight at a time against ggml's block_iq3_xxs (dequantize_row_iq3_xxs): sub-block ib = e // 32 reads word ib at byte 66 + 4 ib: bits
  28..31 scale s (db = d (s + 0.5) / 2), bits 7 l..7 l + 6 the sign index of its l-th run of eight (the eighth sign bit = odd parity of the
  seven); index byte 2 + e // 4 selects four values."""
  entry = {5: [62, 12, 4, 4], 77: [20, 12, 20, 12], 255: [4, 28, 52, 62]}
  for e in [0, 3, 4, 7, 8, 31, 32, 45, 100, 127, 128, 199, 254, 255]:
    for idx, s in ((5, 5), (77, 15), (255, 1)):
      b = np.zeros(98, dtype=np.uint8); b[0:2] = _D
      ib, l, k = e // 32, (e % 32) // 8, e % 8
      s7 = (1 << k) if k < 7 else 1                              # odd parity: element 7 of the run flips as well
      b[66 + 4 * ib:70 + 4 * ib] = np.frombuffer(np.uint32((s << 28) | (s7 << (7 * l))).tobytes(), np.uint8)
      b[2 + e // 4] = idx
      exp = np.full(256, 0.25 * 0.5 * 0.5 * 4, dtype=np.float32)
      db = 0.25 * (s + 0.5) * 0.5
      exp[32 * ib:32 * ib + 32] = db * 4
      exp[4 * (e // 4):4 * (e // 4) + 4] = [db * v for v in entry[idx]]
      run = 32 * ib + 8 * l
      for kk in ({k, 7} if k < 7 else {0, 7}): exp[run + kk] = -exp[run + kk]
      np.testing.assert_array_equal(og.ggml_data_to_tensor(b, 256, 18), exp, err_msg=f"element {e}")
      np.testing.assert_array_equal(cref.dequant(18, b[None]).reshape(-1), exp, err_msg=f"element {e} (C)")

def test_iq3_s_brute_force_layout():
  """block_iq3_s (dequantize_row_iq3_s): 9-bit index i = e // 4 = qs[i] | bit i % 8 of qh[i // 8] << 8 (qs at byte 2, qh at 66); sign of element e = bit
  e % 8 of byte 74 + e // 8; scale of sub-block ib = 1 + 2 * nibble ib of the four bytes at 106."""
  entry = {3: [11, 1, 1, 1], 256: [7, 5, 9, 5], 300: [3, 5, 3, 7], 511: [1, 1, 15, 15]}
  for e in [0, 3, 4, 7, 8, 31, 32, 45, 100, 127, 128, 199, 254, 255]:
    for idx, nib in ((3, 6), (256, 15), (300, 1), (511, 9)):
      b = np.zeros(110, dtype=np.uint8); b[0:2] = _D
      ib, i = e // 32, e // 4
      b[106 + ib // 2] = nib << (4 * (ib % 2))
      b[2 + i] = idx & 255; b[66 + i // 8] = (idx >> 8) << (i % 8)
      b[74 + e // 8] = 1 << (e % 8)
      exp = np.full(256, 0.25, dtype=np.float32)                 # entry 0 = (1, 1, 1, 1), scale 1
      dl = 0.25 * (1 + 2 * nib)
      exp[32 * ib:32 * ib + 32] = dl
      exp[4 * i:4 * i + 4] = [dl * v for v in entry[idx]]
      exp[e] = -exp[e]
      np.testing.assert_array_equal(og.ggml_data_to_tensor(b, 256, 21), exp, err_msg=f"element {e}")
      np.testing.assert_array_equal(cref.dequant(21, b[None]).reshape(-1), exp, err_msg=f"element {e} (C)")

def test_iq2_s_brute_force_layout():
  """block_iq2_s (dequantize_row_iq2_s): 10-bit index i = e // 8 = qs[i] | 2-bit field i % 4 of qh[i // 4] << 8 (qs at byte 2, qh at 66), eight values per
  index; sign of element e = bit e % 8 of byte 34 + i; the g-th run of 16 has db = d (nibble g + 0.5) / 4, nibbles in the eight bytes at 74."""
  entry = {2: [25, 25, 8, 8, 8, 8, 8, 8], 255: [43, 8, 25, 25, 25, 8, 25, 8], 513: [25, 8, 8, 25, 25, 8, 8, 25], 770: [8, 25, 25, 25, 8, 8, 43, 25], 1023: [43] * 8}
  for e in [0, 7, 8, 15, 16, 31, 32, 45, 100, 127, 128, 199, 248, 255]:
    for idx, nib in ((2, 7), (255, 15), (513, 1), (770, 4), (1023, 10)):
      b = np.zeros(82, dtype=np.uint8); b[0:2] = _D
      g, i = e // 16, e // 8
      b[74 + g // 2] = nib << (4 * (g % 2))
      b[2 + i] = idx & 255; b[66 + i // 4] = (idx >> 8) << (2 * (i % 4))
      b[34 + i] = 1 << (e % 8)
      exp = np.full(256, 0.25 * 0.5 * 0.25 * 8, dtype=np.float32)   # entry 0 = eight 8s, nibble 0
      dl = 0.25 * (nib + 0.5) * 0.25
      exp[16 * g:16 * g + 16] = dl * 8
      exp[8 * i:8 * i + 8] = [dl * v for v in entry[idx]]
      exp[e] = -exp[e]
      np.testing.assert_array_equal(og.ggml_data_to_tensor(b, 256, 22), exp, err_msg=f"element {e}")
      np.testing.assert_array_equal(cref.dequant(22, b[None]).reshape(-1), exp, err_msg=f"element {e} (C)")

def test_q1_0_brute_force_layout():
  """Q1_0: element e is bit e % 8 of byte 2 + e // 8; set bit -> +d, clear bit -> -d."""
  for e in [0, 1, 7, 8, 9, 63, 64, 100, 127]:
    b = np.zeros(18, dtype=np.uint8); b[0:2] = np.frombuffer(np.float16(1.5).tobytes(), np.uint8)
    b[2 + e // 8] = 1 << (e % 8)
    exp = np.full(128, -1.5, dtype=np.float32); exp[e] = 1.5
    np.testing.assert_array_equal(og.ggml_data_to_tensor(b, 128, 41), exp)
    np.testing.assert_array_equal(cref.dequant(41, b[None]).reshape(-1), exp)

def test_q6_k_association_order_is_exact():
  """(d*q)*sc == d*(sc*q) == (d*sc)*q in float32: 11 + 6 + 8 significant bits fit in 24."""
  rng = np.random.default_rng(3)
  d = np.float16(rng.standard_normal(4096)).astype(np.float32); q = rng.integers(-32, 32, 4096).astype(np.float32); sc = rng.integers(-128, 128, 4096).astype(np.float32)
  np.testing.assert_array_equal((d * q) * sc, (d * sc) * q)

def test_quantizers_round_trip():
  rng = np.random.default_rng(0)
  w = rng.standard_normal(256 * 64).astype(np.float32)
  for t, qf, tol in ((2, og.quantize_q4_0, 1 / 7.0), (8, og.quantize_q8_0, 1 / 127.0), (14, og.quantize_q6_k, 1 / 30.0), (12, og.quantize_q4_k, 1 / 6.0), (13, og.quantize_q5_k, 1 / 13.0),
                      (3, og.quantize_q4_1, 1 / 7.0), (6, og.quantize_q5_0, 1 / 15.0), (7, og.quantize_q5_1, 1 / 15.0), (23, og.quantize_iq4_xs, 1 / 7.0)):
    dq = og.ggml_data_to_tensor(qf(w), w.size, t)
    nel = {14: 16, 23: 32}.get(t, og.GGML_QUANT[t][0])
    amax = np.abs(w.reshape(-1, nel)).max(1, keepdims=True)
    assert (np.abs(dq.reshape(-1, nel) - w.reshape(-1, nel)) <= tol * amax + 1e-6).all(), t
  # the codebook types: a vector codebook bounds no single weight's error; the decoded weights must follow the originals closely
  for t, qf, corr in ((18, og.quantize_iq3_xxs, 0.97), (21, og.quantize_iq3_s, 0.98), (22, og.quantize_iq2_s, 0.95)):
    dq = og.ggml_data_to_tensor(qf(w), w.size, t)
    assert np.corrcoef(dq, w)[0, 1] > corr and (np.sign(dq) == np.sign(w)).mean() > 0.93, t

def test_unknown_type_raises():
  with pytest.raises(ValueError): og.ggml_data_to_tensor(np.zeros(512, np.uint8), 256, 1337)   # test/unit/test_gguf.py:114-116

def test_fp16_conversions_exhaustive():
  L = cref.lib()
  f = np.arange(65536, dtype=np.uint16).view(np.float16).astype(np.float32)
  for h in range(0, 65536, 3):
    v = np.float32(L.orc_h2f(h))
    assert v.tobytes() == f[h].tobytes() or (np.isnan(v) and np.isnan(f[h]))
  rng = np.random.default_rng(5)
  xs = (rng.standard_normal(5000) * np.float32(10.0) ** rng.integers(-9, 6, 5000)).astype(np.float32)
  with np.errstate(over="ignore"): exp = xs.astype(np.float16).view(np.uint16)
  assert all(L.orc_f2h(float(v)) == int(e) for v, e in zip(xs, exp))

def test_c_vector_f16_rounding_equals_the_bit_level_conversion():
  """orc_linear rounds its dequantized weights to fp16 with the CPU's conversion instructions; the bit-level f2h / h2f of the same file (checked against numpy
  above) must give the same float for normals, subnormals, ties, overflow and signed zeros."""
  rng = np.random.default_rng(11)
  xs = np.concatenate([rng.standard_normal(4096).astype(np.float32) * s for s in (1e-8, 1e-5, 1e-3, 1.0, 300.0, 7e4)] +
                      [np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, -65520.0, 2.0 ** -24, 2.0 ** -25, 1.5 * 2.0 ** -25, 2.0 ** -14, 1.0 + 2.0 ** -11, 1.0 + 3 * 2.0 ** -11, 5.9604645e-08], np.float32)])
  got = cref.round_f16(xs)
  with np.errstate(over="ignore"): want = xs.astype(np.float16).astype(np.float32)
  assert got.tobytes() == want.tobytes()
  L = cref.lib()
  sw = np.array([L.orc_h2f(L.orc_f2h(float(v))) for v in xs[-64:]], np.float32)
  assert sw.tobytes() == got[-64:].tobytes()
