// Bit-exact block decode of ggml_data_to_tensor (tinygrad/llm/gguf.py:23-119): 4 consecutive elements of one block at a time.
// Float contraction is off inside every get4: each product must round exactly like the reference's separate multiplies.
#pragma once
#include "common.h"
#include "iq_grids.h"

// 4 consecutive dequantized values starting at element e0 (a multiple of 4) of block `b`.
template <int T> struct Deq;

template <> struct Deq<GGML_Q4_0> {
  static constexpr int NEL = 32, NBY = 18;
  static __device__ __forceinline__ void get4(const uint8_t* b, int e0, float* o) {
#pragma clang fp contract(off)
    const float d = h2f_bits(ld2(b));
    const int sh = (e0 >= 16) ? 4 : 0; const uint8_t* q = b + 2 + (e0 & 15);
#pragma unroll
    for (int i = 0; i < 4; i++) o[i] = (float)((int)((q[i] >> sh) & 0xF) - 8) * d;
  }
};
// Q4_1 (20 B: d, m, qs[16]), tinygrad/llm/gguf.py:47-49: q * d + m
template <> struct Deq<GGML_Q4_1> {
  static constexpr int NEL = 32, NBY = 20;
  static __device__ __forceinline__ void get4(const uint8_t* b, int e0, float* o) {
#pragma clang fp contract(off)
    const float d = h2f_bits(ld2(b)), m = h2f_bits(ld2(b + 2));
    const int sh = (e0 >= 16) ? 4 : 0; const uint8_t* q = b + 4 + (e0 & 15);
#pragma unroll
    for (int i = 0; i < 4; i++) o[i] = (float)((q[i] >> sh) & 0xF) * d + m;
  }
};
// Q5_0 (22 B: d, qh[4], qs[16]) and Q5_1 (24 B: d, m, qh[4], qs[16]), tinygrad/llm/gguf.py:50-55: q = nibble + 16 * bit e of the
// 32-bit qh; q * d + (m for Q5_1, -16 * d for Q5_0)
template <bool ONE> struct DeqQ5 {
  static constexpr int NEL = 32, NBY = ONE ? 24 : 22;
  static __device__ __forceinline__ void get4(const uint8_t* b, int e0, float* o) {
#pragma clang fp contract(off)
    const float d = h2f_bits(ld2(b)), off = ONE ? h2f_bits(ld2(b + 2)) : -16.0f * d;
    const uint8_t* p = b + (ONE ? 4 : 2);
    const uint32_t qh = (uint32_t)ld2(p) | ((uint32_t)ld2(p + 2) << 16);
    const int sh = (e0 >= 16) ? 4 : 0; const uint8_t* q = p + 4 + (e0 & 15);
#pragma unroll
    for (int i = 0; i < 4; i++) o[i] = (float)(((q[i] >> sh) & 0xF) | (((qh >> (e0 + i)) & 1u) << 4)) * d + off;
  }
};
template <> struct Deq<GGML_Q5_0> : DeqQ5<false> {};
template <> struct Deq<GGML_Q5_1> : DeqQ5<true> {};
template <> struct Deq<GGML_Q8_0> {
  static constexpr int NEL = 32, NBY = 34;
  static __device__ __forceinline__ void get4(const uint8_t* b, int e0, float* o) {
#pragma clang fp contract(off)
    const float d = h2f_bits(ld2(b));
#pragma unroll
    for (int i = 0; i < 4; i++) o[i] = d * (float)(int8_t)b[2 + e0 + i];
  }
};
template <> struct Deq<GGML_Q6_K> {
  static constexpr int NEL = 256, NBY = 210;
  static __device__ __forceinline__ void get4(const uint8_t* b, int e0, float* o) {
#pragma clang fp contract(off)
    const float d = h2f_bits(ld2(b + 208));
    const int half = e0 >> 7, r = e0 & 127, j = r >> 5, l = r & 31;      // element = 128*half + 32*j + l
    const uint8_t* ql = b + 64 * half + ((j & 1) ? 32 : 0) + l;
    const uint8_t* qh = b + 128 + 32 * half + l;
    const float sc = (float)(int8_t)b[192 + (e0 >> 4)];
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const int lo = (j & 2) ? (ql[i] >> 4) : (ql[i] & 0xF);
      const int q = (int)(int8_t)(lo | (((qh[i] >> (2 * j)) & 3) << 4)) - 32;
      o[i] = (d * (float)q) * sc;                                        // reference association: (d * q) * scale
    }
  }
};
// Q4_K (144 B: d, dmin, scales[12], qs[128]) and Q5_K (176 B: ... qh[32], qs[128]), tinygrad/llm/gguf.py:57-67: sub-block sb = e / 32
// has a 6-bit scale and min packed in the 12 scale bytes; value = (d * sc) * q - dmin * mn with q = nibble (sb & 1) of
// qs[32 * (sb / 2) + e % 32] (+ 16 * bit sb of qh[e % 32] for Q5_K).
template <bool FIVE> struct DeqK45 {
  static constexpr int NEL = 256, NBY = FIVE ? 176 : 144;
  static __device__ __forceinline__ void get4(const uint8_t* b, int e0, float* o) {
#pragma clang fp contract(off)
    const float d = h2f_bits(ld2(b)), dmin = h2f_bits(ld2(b + 2));
    const int sb = e0 >> 5, l = e0 & 31;
    const uint8_t* s = b + 4;
    int sc, mn;
    if (sb < 4) { sc = s[sb] & 63; mn = s[sb + 4] & 63; }
    else { sc = (s[sb + 4] & 0xF) | ((s[sb - 4] >> 6) << 4); mn = (s[sb + 4] >> 4) | ((s[sb] >> 6) << 4); }
    const float d1 = d * (float)sc, m1 = dmin * (float)mn;
    const uint8_t* q = b + (FIVE ? 48 : 16) + 32 * (sb >> 1) + l;
#pragma unroll
    for (int i = 0; i < 4; i++) {
      int v = (sb & 1) ? (q[i] >> 4) : (q[i] & 0xF);
      if (FIVE) v += ((b[16 + l + i] >> sb) & 1) << 4;
      o[i] = d1 * (float)v - m1;
    }
  }
};
template <> struct Deq<GGML_Q4_K> : DeqK45<false> {};
template <> struct Deq<GGML_Q5_K> : DeqK45<true> {};
// IQ4_XS (136 B: d, scales_h u16, scales_l[4], qs[128]), tinygrad/llm/gguf.py:96-104: eight sub-blocks of 32; 6-bit scale ls =
// nibble ib of scales_l | 2 bits of scales_h << 4; value = (d * (ls - 32)) * kvalues_iq4nl[nibble]; qs[16 ib + j] holds elements j (low
// nibble) and j + 16 (high nibble) of sub-block ib.
__device__ __forceinline__ float iq4nl_value(uint32_t code) {
  // ggml's kvalues_iq4nl, packed four int8 per dword
  const uint32_t t[4] = {0xBFAD9881u, 0xF6EADDCFu, 0x26190D01u, 0x71594535u};   // -127 -104 -83 -65 | -49 -35 -22 -10 | 1 13 25 38 | 53 69 89 113
  return (float)(int)(int8_t)(t[code >> 2] >> (8 * (code & 3)));
}
template <> struct Deq<GGML_IQ4_XS> {
  static constexpr int NEL = 256, NBY = 136;
  static __device__ __forceinline__ void get4(const uint8_t* b, int e0, float* o) {
#pragma clang fp contract(off)
    const float d = h2f_bits(ld2(b));
    const uint32_t sh = ld2(b + 2);
    const int ib = e0 >> 5, l = e0 & 31;
    const int ls = (int)(((b[4 + (ib >> 1)] >> (4 * (ib & 1))) & 0xF) | (((sh >> (2 * ib)) & 3) << 4));
    const float dl = d * (float)(ls - 32);
    const int hi = (l >= 16) ? 4 : 0; const uint8_t* q = b + 8 + 16 * ib + (l & 15);
#pragma unroll
    for (int i = 0; i < 4; i++) o[i] = dl * iq4nl_value((q[i] >> hi) & 0xF);
  }
};
// The codebook types (tinygrad/llm/gguf.py:73-95).  A codebook entry is kept as its digits over the codebook's alphabet (iq_grids.h); sign bit k
// of a sign byte negates value k of its run of eight.
__device__ __forceinline__ float pm1(uint32_t bits, int k) { return ((bits >> k) & 1u) ? -1.0f : 1.0f; }
// IQ3_XXS (98 B: d, qs[64], 8 uint32 words), gguf.py:73-81: word ib of sub-block ib holds the scale s in bits 28..31 and four 7-bit sign indices
// (an eighth bit makes each sign byte's parity even); value = ((d * (s + 0.5)) * 0.5) * grid * sign, 4 values per index byte.
template <> struct Deq<GGML_IQ3_XXS> {
  static constexpr int NEL = 256, NBY = 98;
  static __device__ __forceinline__ void get4(const uint8_t* b, int e0, float* o) {
#pragma clang fp contract(off)
    const float d = h2f_bits(ld2(b));
    const int ib = e0 >> 5, l = (e0 >> 3) & 3;
    const uint8_t* w = b + 66 + 4 * ib;
    const uint32_t aux = (uint32_t)ld2(w) | ((uint32_t)ld2(w + 2) << 16);
    const float db = d * ((float)(aux >> 28) + 0.5f) * 0.5f;
    const uint32_t s7 = (aux >> (7 * l)) & 127u, signs = (s7 | ((__builtin_popcount(s7) & 1u) << 7)) >> (e0 & 4);
    const uint32_t code = IQ3XXS_CODE[b[2 + (e0 >> 2)]];
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const uint32_t dg = (code >> (3 * i)) & 7u;
      o[i] = db * (float)(dg == 7u ? 62u : 4u + 8u * dg) * pm1(signs, i);
    }
  }
};
// IQ3_S (110 B: d, qs[64], qh[8], signs[32], scales[4]), gguf.py:82-88: index i = qs[i] | bit i % 8 of qh[i / 8] << 8;
// value = ((d * (1 + 2 nibble ib)) * grid) * sign
template <> struct Deq<GGML_IQ3_S> {
  static constexpr int NEL = 256, NBY = 110;
  static __device__ __forceinline__ void get4(const uint8_t* b, int e0, float* o) {
#pragma clang fp contract(off)
    const float d = h2f_bits(ld2(b));
    const int ib = e0 >> 5, i = e0 >> 2;
    const float dl = d * (float)(1 + 2 * (int)((b[106 + (ib >> 1)] >> (4 * (ib & 1))) & 0xF));
    const uint32_t code = IQ3S_CODE[(uint32_t)b[2 + i] | ((((uint32_t)b[66 + (i >> 3)] >> (i & 7)) & 1u) << 8)];
    const uint32_t signs = (uint32_t)b[74 + (e0 >> 3)] >> (e0 & 4);
#pragma unroll
    for (int k = 0; k < 4; k++) o[k] = dl * (float)(1u + 2u * ((code >> (3 * k)) & 7u)) * pm1(signs, k);
  }
};
// IQ2_S (82 B: d, qs[32], signs[32], qh[8], scales[8]), gguf.py:89-95: index i = qs[i] | 2-bit field i % 4 of qh[i / 4] << 8, 8 values per index;
// value = (((d * (nibble g + 0.5)) * 0.25) * grid) * sign, g = the run of 16 values
template <> struct Deq<GGML_IQ2_S> {
  static constexpr int NEL = 256, NBY = 82;
  static __device__ __forceinline__ void get4(const uint8_t* b, int e0, float* o) {
#pragma clang fp contract(off)
    const float d = h2f_bits(ld2(b));
    const int g = e0 >> 4, i = e0 >> 3;
    const float dl = d * ((float)((b[74 + (g >> 1)] >> (4 * (g & 1))) & 0xF) + 0.5f) * 0.25f;
    uint32_t code = IQ2S_CODE[(uint32_t)b[2 + i] | ((((uint32_t)b[66 + (i >> 2)] >> (2 * (i & 3))) & 3u) << 8)];
    if (e0 & 4) code /= 81u;                                   // skip the first four base-3 digits
    const uint32_t signs = (uint32_t)b[34 + i] >> (e0 & 4);
#pragma unroll
    for (int k = 0; k < 4; k++) {
      const uint32_t t = code % 3u; code /= 3u;
      o[k] = dl * (float)(8u + 17u * t + (t >> 1)) * pm1(signs, k);   // {8, 25, 43}
    }
  }
};
// Q1_0 (18 B: d, 128 sign bits), tinygrad/llm/gguf.py:115-118: value = d * (2 bit - 1), element e = bit e % 8 of byte e / 8
template <> struct Deq<GGML_Q1_0> {
  static constexpr int NEL = 128, NBY = 18;
  static __device__ __forceinline__ void get4(const uint8_t* b, int e0, float* o) {
#pragma clang fp contract(off)
    const float d = h2f_bits(ld2(b));
    const uint32_t bits = b[2 + (e0 >> 3)] >> (e0 & 7);
#pragma unroll
    for (int i = 0; i < 4; i++) o[i] = d * (float)((int)((bits >> i) & 1u) * 2 - 1);
  }
};
template <> struct Deq<GGML_MXFP4> {
  static constexpr int NEL = 32, NBY = 17;
  static __device__ __forceinline__ void get4(const uint8_t* b, int e0, float* o) {
#pragma clang fp contract(off)
    const uint32_t e = b[0];
    const float d = __builtin_bit_cast(float, e < 2 ? (0x00200000u << e) : ((e - 1) << 23));   // 2^(e-128)
    const int sh = (e0 >= 16) ? 4 : 0; const uint8_t* q = b + 1 + (e0 & 15);
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const uint32_t c = (q[i] >> sh) & 0xF, mag = c & 7;
      // doubled E2M1 table {0,1,2,3,4,6,8,12}; bit 3 is the sign (code 8 is -0.0 in the reference's float LUT)
      const float v = (float)(mag < 4 ? mag : (mag < 6 ? 2 * mag - 4 : 4 * mag - 16));
      o[i] = __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, v) | ((c & 8) << 28)) * d;
    }
  }
};

