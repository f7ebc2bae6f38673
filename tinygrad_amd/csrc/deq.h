// Bit-exact block decode of ggml_data_to_tensor (tinygrad/llm/gguf.py:23-119): 4 consecutive elements of one block at a time.
// Float contraction is off inside every get4: each product must round exactly like the reference's separate multiplies.
#pragma once
#include "common.h"

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

