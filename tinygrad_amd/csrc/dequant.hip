// Block dequant kernels: bit-exact restatement of ggml_data_to_tensor (tinygrad/llm/gguf.py:23-119) for Q4_0 (:46), Q8_0 (:56),
// Q4_K / Q5_K (:57-67), Q6_K (:68-72) and MXFP4 (:105-114).  One thread produces 4 consecutive output elements (one 16-byte or 8-byte store), so
// stores are fully coalesced; the packed bytes are re-read through L1/L2 (this kernel is a load-time / test utility, the
// decode path never materialises weights).
// Float contraction is off for this file: every product below must round exactly like the reference's separate multiplies.
#include "common.h"
#include "host.h"

#pragma clang fp contract(off)

// 4 consecutive dequantized values starting at element e0 (a multiple of 4) of block `b`.
template <int T> struct Deq;

template <> struct Deq<GGML_Q4_0> {
  static constexpr int NEL = 32, NBY = 18;
  static __device__ __forceinline__ void get4(const uint8_t* b, int e0, float* o) {
    const float d = h2f_bits(ld2(b));
    const int sh = (e0 >= 16) ? 4 : 0; const uint8_t* q = b + 2 + (e0 & 15);
#pragma unroll
    for (int i = 0; i < 4; i++) o[i] = (float)((int)((q[i] >> sh) & 0xF) - 8) * d;
  }
};
template <> struct Deq<GGML_Q8_0> {
  static constexpr int NEL = 32, NBY = 34;
  static __device__ __forceinline__ void get4(const uint8_t* b, int e0, float* o) {
    const float d = h2f_bits(ld2(b));
#pragma unroll
    for (int i = 0; i < 4; i++) o[i] = d * (float)(int8_t)b[2 + e0 + i];
  }
};
template <> struct Deq<GGML_Q6_K> {
  static constexpr int NEL = 256, NBY = 210;
  static __device__ __forceinline__ void get4(const uint8_t* b, int e0, float* o) {
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

template <int T, bool F16>
__global__ __launch_bounds__(256) void dequant_kernel(const uint8_t* __restrict__ blocks, void* __restrict__ out, int64_t n4) {
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n4; i += (int64_t)gridDim.x * 256) {
    const int64_t e = i * 4, blk = e / Deq<T>::NEL; const int e0 = (int)(e % Deq<T>::NEL);
    float o[4];
    Deq<T>::get4(blocks + blk * Deq<T>::NBY, e0, o);
    if (F16) {
      // keep the float32 result opaque: folding the multiply into v_fma_mixlo_f16 (product + 0) would turn -0.0 into +0.0
#pragma unroll
      for (int q = 0; q < 4; q++) asm volatile("" : "+v"(o[q]));
      u32x2 v = {f2h_bits(o[0]) | (f2h_bits(o[1]) << 16), f2h_bits(o[2]) | (f2h_bits(o[3]) << 16)};
      ((u32x2*)out)[i] = v;
    } else {
      f32x4 v = {o[0], o[1], o[2], o[3]};
      ((f32x4*)out)[i] = v;
    }
  }
}

template <int T> static int launch_dequant(const void* blocks, int64_t n, void* out, int out_dtype, hipStream_t s) {
  TGA_REQUIRE(n % Deq<T>::NEL == 0, "tga_dequant: n=%lld is not a multiple of the block size %d", (long long)n, Deq<T>::NEL);
  if (n == 0) return 0;
  const int64_t n4 = n / 4;
  const int grid = (int)((n4 + 255) / 256 < 65536 ? (n4 + 255) / 256 : 65536);
  if (out_dtype == TGA_F32) dequant_kernel<T, false><<<grid, 256, 0, s>>>((const uint8_t*)blocks, out, n4);
  else dequant_kernel<T, true><<<grid, 256, 0, s>>>((const uint8_t*)blocks, out, n4);
  TGA_LAUNCH_CHECK();
  return 0;
}

extern "C" int tga_dequant(int ggml_type, const void* blocks, int64_t n, void* out, int out_dtype, void* stream) {
  TGA_REQUIRE(out_dtype == TGA_F32 || out_dtype == TGA_F16, "tga_dequant: out_dtype must be TGA_F32 or TGA_F16");
  TGA_REQUIRE(n >= 0 && (n == 0 || (blocks && out)), "tga_dequant: null pointer");
  hipStream_t s = (hipStream_t)stream;
  switch (ggml_type) {
    case GGML_Q4_0: return launch_dequant<GGML_Q4_0>(blocks, n, out, out_dtype, s);
    case GGML_Q8_0: return launch_dequant<GGML_Q8_0>(blocks, n, out, out_dtype, s);
    case GGML_Q4_K: return launch_dequant<GGML_Q4_K>(blocks, n, out, out_dtype, s);
    case GGML_Q5_K: return launch_dequant<GGML_Q5_K>(blocks, n, out, out_dtype, s);
    case GGML_Q6_K: return launch_dequant<GGML_Q6_K>(blocks, n, out, out_dtype, s);
    case GGML_MXFP4: return launch_dequant<GGML_MXFP4>(blocks, n, out, out_dtype, s);
  }
  return tga_set_error("GGML type '%d' is not supported!", ggml_type);   // message of tinygrad/llm/gguf.py:119
}
