// Shared device helpers for the gfx950 (CDNA4, wave64) kernels.  No CUDA-compat paths: this code only targets gfx950.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

#define TGA_WAVE 64

// ggml type ids (tinygrad/llm/gguf.py:20-21 keys)
enum { GGML_F32 = 0, GGML_F16 = 1, GGML_Q4_0 = 2, GGML_Q4_1 = 3, GGML_Q5_0 = 6, GGML_Q5_1 = 7, GGML_Q8_0 = 8, GGML_Q4_K = 12, GGML_Q5_K = 13, GGML_Q6_K = 14, GGML_IQ3_XXS = 18, GGML_IQ3_S = 21, GGML_IQ2_S = 22, GGML_IQ4_XS = 23, GGML_MXFP4 = 39, GGML_Q1_0 = 41 };

// weights per block of a ggml block type (the (elements, bytes) table of tinygrad/llm/gguf.py:20-21); 0: not a block type
static inline int tga_block_weights(int t) {
  switch (t) {
    case GGML_Q4_0: case GGML_Q4_1: case GGML_Q5_0: case GGML_Q5_1: case GGML_Q8_0: case GGML_MXFP4: return 32;
    case GGML_Q4_K: case GGML_Q5_K: case GGML_Q6_K: case GGML_IQ3_XXS: case GGML_IQ3_S: case GGML_IQ2_S: case GGML_IQ4_XS: return 256;
    case GGML_Q1_0: return 128;
    case GGML_F16: case GGML_F32: return 1;
  }
  return 0;
}

__device__ __forceinline__ half2_t as_h2(uint32_t u) { return __builtin_bit_cast(half2_t, u); }
__device__ __forceinline__ uint32_t as_u32(half2_t h) { return __builtin_bit_cast(uint32_t, h); }
__device__ __forceinline__ float h2f_bits(uint32_t h16) { return (float)__builtin_bit_cast(_Float16, (uint16_t)h16); }
__device__ __forceinline__ uint32_t f2h_bits(float f) { return (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)f); }
// v_dot2_f32_f16: a.x*b.x + a.y*b.y + c with a float32 accumulator
__device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float c) { return __builtin_amdgcn_fdot2(as_h2(a), as_h2(b), c, false); }
// (a & b) | c in one VALU op (v_and_or_b32)
__device__ __forceinline__ uint32_t and_or(uint32_t a, uint32_t b, uint32_t c) { return (a & b) | c; }

// loads from addresses that are only byte/2-byte aligned: gfx950 under HSA runs global memory in unaligned-access mode, and
// the compiler turns these into single global_load_dwordx4 / dwordx2 / ushort instructions.
__device__ __forceinline__ u32x4 ld16(const uint8_t* p) { u32x4 v; __builtin_memcpy(&v, p, 16); return v; }
__device__ __forceinline__ uint32_t ld4(const uint8_t* p) { uint32_t v; __builtin_memcpy(&v, p, 4); return v; }
__device__ __forceinline__ uint32_t ld2(const uint8_t* p) { uint16_t v; __builtin_memcpy(&v, p, 2); return v; }

template <int CTRL, int ROW_MASK = 0xF>
__device__ __forceinline__ float dpp_add(float v) {
  // lanes whose row is masked out (or whose source is invalid) receive 0 and keep v
  int r = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, ROW_MASK, 0xF, false);
  return v + __builtin_bit_cast(float, r);
}
// Sum over the 64 lanes of a wave with DPP only (no LDS).  Result valid in lane 63.
__device__ __forceinline__ float wave_sum_lane63(float v) {
  v = dpp_add<0xB1>(v);        // quad_perm [1,0,3,2]
  v = dpp_add<0x4E>(v);        // quad_perm [2,3,0,1]
  v = dpp_add<0x141>(v);       // row_half_mirror
  v = dpp_add<0x140>(v);       // row_mirror: every lane of a 16-lane row holds the row sum
  v = dpp_add<0x142, 0xA>(v);  // row_bcast15 into rows 1,3
  v = dpp_add<0x143, 0xC>(v);  // row_bcast31 into rows 2,3
  return v;
}
// Sums over lanes 0-31 and over lanes 32-63 separately.  Results valid in lanes 31 and 63.
__device__ __forceinline__ float half_sum_lane31(float v) {
  v = dpp_add<0xB1>(v);
  v = dpp_add<0x4E>(v);
  v = dpp_add<0x141>(v);
  v = dpp_add<0x140>(v);
  v = dpp_add<0x142, 0xA>(v);  // row_bcast15 into rows 1,3: lane 31 = rows 0+1, lane 63 = rows 2+3
  return v;
}
__device__ __forceinline__ float wave_sum(float v) {
  v = wave_sum_lane63(v);
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}
