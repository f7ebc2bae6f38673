// The codebook and 1-bit GGUF block types as GEMV / GEMM weight formats (included by qfmt.h): IQ3_XXS (tinygrad/llm/gguf.py:73-81), IQ3_S (:82-88),
// IQ2_S (:89-95) and Q1_0 (:115-118), read in place.
//
// A unit is 64 consecutive weights (a quarter of a 256-weight superblock, half of a Q1_0 block).  The codebooks live in LDS, one copy per workgroup, written
// by Fmt::consts() at the start of a kernel (every thread of the workgroup calls it before any of them leaves): a grid entry is kept as the fp16 values it
// stands for (4 values = 8 bytes for the 3-bit types, 8 values = 16 bytes for IQ2_S), so a lane fetches an entry with one ds_read.  LDS reads count on a
// counter of their own, so the lookups of one step do not wait for the weight loads of the next (a table in global memory would: a wave's loads return in
// the order they were asked for).  Grid values are positive, so a sign is an OR into bit 15 / 31 of a dword of two fp16 values: a sign byte s becomes
// t = s | s << 15, and (t << 15 - 2p) & 0x80008000 carries bits 2p and 2p + 1 of s to the sign bits of pair p - two VALU operations per pair, no table
// (sign patterns read from LDS, 16 bytes per sign byte, made the kernels wait on bank conflicts of the random reads: 14336 x 4096 IQ3_XXS 10.7 us).
// The decoded unit is 32 dwords of signed fp16 pairs in the natural order of the weights.  The grids are constants of the file format, kept as digit codes in
// iq_grids.h; block scales are applied per accumulator group by finish(), or folded into the fp16 weights by to_f16() for the matrix-core kernels.
#pragma once
#include "iq_grids.h"

typedef u32x4 u32x4_a2 __attribute__((aligned(2)));
typedef u32x2 u32x2_a2 __attribute__((aligned(2)));
__device__ __forceinline__ u32x4 ld16_a2(const uint8_t* p) { return *(const TGA_GLOBAL u32x4_a2*)p; }
__device__ __forceinline__ u32x2 ld8_a2(const uint8_t* p) { return *(const TGA_GLOBAL u32x2_a2*)p; }
__device__ __forceinline__ uint32_t ld2_g(const uint8_t* p) { return *(const TGA_GLOBAL uint16_t*)p; }

__device__ __forceinline__ uint32_t cb_h2(float lo, float hi) { return f2h_bits(lo) | (f2h_bits(hi) << 16); }
// the signs of eight weights (bit k of the byte s negates weight k) onto four dwords of positive fp16 pairs
__device__ __forceinline__ void cb_signs(uint32_t s, uint32_t& w0, uint32_t& w1, uint32_t& w2, uint32_t& w3) {
  const uint32_t t = (s << 15) | s;
  w0 = and_or(t << 15, 0x80008000u, w0); w1 = and_or(t << 13, 0x80008000u, w1); w2 = and_or(t << 11, 0x80008000u, w2); w3 = and_or(t << 9, 0x80008000u, w3);
}
__device__ __forceinline__ u32x2* cb_grid_iq3xxs() { __shared__ u32x2 t[256]; return t; }
__device__ __forceinline__ u32x2* cb_grid_iq3s() { __shared__ u32x2 t[512]; return t; }
__device__ __forceinline__ u32x4* cb_grid_iq2s() { __shared__ u32x4 t[1024]; return t; }

// (TAB: bytes of LDS a workgroup's tables take, beside what the kernel itself declares; fmt_tab<F>() is 0 for the formats that have none)
// what the four formats share: 64 consecutive weights per unit, activations staged in their natural order, no bias correction
struct FmtCbBase {
  static constexpr int UW = 64, XV = 8, NKC = 1;
  static __device__ __forceinline__ int unit_of(int e) { return e >> 6; }
  static __device__ __forceinline__ int pair_of(int e) { return (e & 63) >> 1; }
  static __device__ __forceinline__ int xoff(int u, int k) { return 64 * u + 2 * k; }
  static __device__ __forceinline__ int spos(int e, int nu) { return ((((e >> 3) & 7) * nu + (e >> 6)) << 3) | (e & 7); }
  template <int NG>
  static __device__ __forceinline__ void stage_n(const uint32_t* nx, u32x4* xv, float* c) {
#pragma unroll
    for (int v = 0; v < 8; v++) { xv[v].x = nx[4 * v]; xv[v].y = nx[4 * v + 1]; xv[v].z = nx[4 * v + 2]; xv[v].w = nx[4 * v + 3]; }
#pragma unroll
    for (int g = 0; g < NG; g++) c[g] = 0.f;
  }
  // fp16 weights = pattern * scale, one rounding; NG accumulator groups of 32 / NG dwords, their float32 scales behind the 32 pattern dwords
  template <int NG>
  static __device__ __forceinline__ void scale_n(uint32_t* wv) {
#pragma unroll
    for (int g = 0; g < NG; g++) {
      const float s = __builtin_bit_cast(float, wv[32 + g]);
#pragma unroll
      for (int i = 0; i < 32 / NG; i++) wv[(32 / NG) * g + i] = h2_unbias_scale_f32(wv[(32 / NG) * g + i], s, 0.f);
    }
  }
};

// ------------------------------------------------------------------------------------------------ IQ3_XXS (gguf.py:73-81)
// 98 bytes: fp16 d, qs[64] (one grid index per 4 weights), 8 words; word ib of sub-block ib (32 weights) holds the 4-bit scale s in bits 28..31 and four 7-bit sign
// indices; w = ((d (s + 0.5)) 0.5) grid sign.  Unit p: qs[16 p .. 16 p + 15], words 2 p and 2 p + 1; accumulator group g = sub-block 2 p + g.
template <> struct Fmt<GGML_IQ3_XXS> : FmtCbBase {
  static constexpr int UPB = 4, BW = 256, BB = 98, NG = 2, NWV = 34, TAB = 256 * 8;
  struct Raw { u32x4 q; u32x2 aux; uint32_t d; };
  static __device__ __forceinline__ Raw load(const uint8_t* row, int u) {
    const uint8_t* b = row + (size_t)BB * (u >> 2); const int p = u & 3;
    Raw r; r.d = ld2_g(b); r.q = ld16_a2(b + 2 + 16 * p); r.aux = ld8_a2(b + 66 + 8 * p); return r;
  }
  static __device__ __forceinline__ void consts(uint32_t* kc) {
    u32x2* g = cb_grid_iq3xxs();
    for (int i = threadIdx.x; i < 256; i += blockDim.x) {
      const uint32_t code = IQ3XXS_CODE[i];
      float v[4];
#pragma unroll
      for (int k = 0; k < 4; k++) { const uint32_t dg = (code >> (3 * k)) & 7u; v[k] = (float)(dg == 7u ? 62u : 4u + 8u * dg); }
      u32x2 e; e.x = cb_h2(v[0], v[1]); e.y = cb_h2(v[2], v[3]); g[i] = e;
    }
    __syncthreads();
    kc[0] = 0;
  }
  static __device__ __forceinline__ void decode(const Raw& r, uint32_t* wv, const uint32_t*) {
    const u32x2* grid = cb_grid_iq3xxs();
#pragma unroll
    for (int g = 0; g < 2; g++) {
      const uint32_t aux = g ? r.aux.y : r.aux.x;
#pragma unroll
      for (int l = 0; l < 4; l++) {
        const uint32_t qw = r.q[2 * g + (l >> 1)] >> (16 * (l & 1));
        const u32x2 g0 = grid[qw & 0xFFu], g1 = grid[(qw >> 8) & 0xFFu];
        const uint32_t s7 = (aux >> (7 * l)) & 127u;                       // seven stored bits; the eighth makes the number of set bits even
        uint32_t* o = wv + 16 * g + 4 * l;
        o[0] = g0.x; o[1] = g0.y; o[2] = g1.x; o[3] = g1.y;
        cb_signs(s7 | (((uint32_t)__builtin_popcount(s7) & 1u) << 7), o[0], o[1], o[2], o[3]);
      }
      wv[32 + g] = __builtin_bit_cast(uint32_t, h2f_bits(r.d) * ((float)(aux >> 28) + 0.5f) * 0.5f);
    }
  }
  static __device__ __forceinline__ void stage(const uint32_t* nx, u32x4* xv, float* c) { stage_n<NG>(nx, xv, c); }
  static __device__ __forceinline__ float finish(const Raw&, const uint32_t* wv, const float* a, const float*) {
    return __builtin_bit_cast(float, wv[32]) * a[0] + __builtin_bit_cast(float, wv[33]) * a[1];
  }
  static __device__ __forceinline__ void to_f16(const Raw&, uint32_t* wv) { scale_n<NG>(wv); }
  static __device__ __forceinline__ void cfromx(const u32x4*, float* c) { c[0] = 0.f; c[1] = 0.f; }
};

// ------------------------------------------------------------------------------------------------ IQ3_S (gguf.py:82-88)
// 110 bytes: fp16 d, qs[64], qh[8], signs[32], scales[4]; grid index i = qs[i] | bit i % 8 of qh[i / 8] << 8 (4 weights per index), sign byte per 8 weights,
// w = (d (1 + 2 nibble ib)) grid sign per sub-block ib of 32.  Unit p: qs[16 p ..], qh[2 p], qh[2 p + 1], signs[8 p ..], scales[p].
template <> struct Fmt<GGML_IQ3_S> : FmtCbBase {
  static constexpr int UPB = 4, BW = 256, BB = 110, NG = 2, NWV = 34, TAB = 512 * 8;
  struct Raw { u32x4 q; u32x2 sg; uint32_t qh, sc, d; };
  static __device__ __forceinline__ Raw load(const uint8_t* row, int u) {
    const uint8_t* b = row + (size_t)BB * (u >> 2); const int p = u & 3;
    Raw r; r.d = ld2_g(b); r.q = ld16_a2(b + 2 + 16 * p); r.qh = ld2_g(b + 66 + 2 * p); r.sg = ld8_a2(b + 74 + 8 * p);
    r.sc = ld2_g(b + 106 + (p & 2)) >> (8 * (p & 1));
    return r;
  }
  static __device__ __forceinline__ void consts(uint32_t* kc) {
    u32x2* g = cb_grid_iq3s();
    for (int i = threadIdx.x; i < 512; i += blockDim.x) {
      const uint32_t code = IQ3S_CODE[i];
      float v[4];
#pragma unroll
      for (int k = 0; k < 4; k++) v[k] = (float)(1u + 2u * ((code >> (3 * k)) & 7u));
      u32x2 e; e.x = cb_h2(v[0], v[1]); e.y = cb_h2(v[2], v[3]); g[i] = e;
    }
    __syncthreads();
    kc[0] = 0;
  }
  static __device__ __forceinline__ void decode(const Raw& r, uint32_t* wv, const uint32_t*) {
    const u32x2* grid = cb_grid_iq3s();
#pragma unroll
    for (int g = 0; g < 2; g++) {
      const uint32_t sw = g ? r.sg.y : r.sg.x, qh = r.qh >> (8 * g);
#pragma unroll
      for (int l = 0; l < 4; l++) {
        const uint32_t qw = r.q[2 * g + (l >> 1)] >> (16 * (l & 1));
        const u32x2 g0 = grid[(qw & 0xFFu) | (((qh >> (2 * l)) & 1u) << 8)], g1 = grid[((qw >> 8) & 0xFFu) | (((qh >> (2 * l + 1)) & 1u) << 8)];
        uint32_t* o = wv + 16 * g + 4 * l;
        o[0] = g0.x; o[1] = g0.y; o[2] = g1.x; o[3] = g1.y;
        cb_signs((sw >> (8 * l)) & 0xFFu, o[0], o[1], o[2], o[3]);
      }
      wv[32 + g] = __builtin_bit_cast(uint32_t, h2f_bits(r.d) * (float)(1 + 2 * (int)((r.sc >> (4 * g)) & 0xFu)));
    }
  }
  static __device__ __forceinline__ void stage(const uint32_t* nx, u32x4* xv, float* c) { stage_n<NG>(nx, xv, c); }
  static __device__ __forceinline__ float finish(const Raw&, const uint32_t* wv, const float* a, const float*) {
    return __builtin_bit_cast(float, wv[32]) * a[0] + __builtin_bit_cast(float, wv[33]) * a[1];
  }
  static __device__ __forceinline__ void to_f16(const Raw&, uint32_t* wv) { scale_n<NG>(wv); }
  static __device__ __forceinline__ void cfromx(const u32x4*, float* c) { c[0] = 0.f; c[1] = 0.f; }
};

// ------------------------------------------------------------------------------------------------ IQ2_S (gguf.py:89-95)
// 82 bytes: fp16 d, qs[32], signs[32], qh[8], scales[8]; grid index i = qs[i] | 2-bit field i % 4 of qh[i / 4] << 8 (8 weights per index), sign byte per 8
// weights, w = (((d (nibble g + 0.5)) 0.25) grid) sign per run g of 16.  Unit p: qs[8 p ..], signs[8 p ..], qh[2 p], qh[2 p + 1], scales[2 p], scales[2 p + 1];
// four accumulator groups of 16 weights.
template <> struct Fmt<GGML_IQ2_S> : FmtCbBase {
  static constexpr int UPB = 4, BW = 256, BB = 82, NG = 4, NWV = 36, TAB = 1024 * 16;
  struct Raw { u32x2 q, sg; uint32_t qh, sc, d; };
  static __device__ __forceinline__ Raw load(const uint8_t* row, int u) {
    const uint8_t* b = row + (size_t)BB * (u >> 2); const int p = u & 3;
    Raw r; r.d = ld2_g(b); r.q = ld8_a2(b + 2 + 8 * p); r.sg = ld8_a2(b + 34 + 8 * p); r.qh = ld2_g(b + 66 + 2 * p); r.sc = ld2_g(b + 74 + 2 * p);
    return r;
  }
  static __device__ __forceinline__ void consts(uint32_t* kc) {
    u32x4* g = cb_grid_iq2s();
    for (int i = threadIdx.x; i < 1024; i += blockDim.x) {
      uint32_t code = IQ2S_CODE[i];
      float v[8];
#pragma unroll
      for (int k = 0; k < 8; k++) { const uint32_t t = code % 3u; code /= 3u; v[k] = (float)(8u + 17u * t + (t >> 1)); }   // {8, 25, 43}
      u32x4 e; e.x = cb_h2(v[0], v[1]); e.y = cb_h2(v[2], v[3]); e.z = cb_h2(v[4], v[5]); e.w = cb_h2(v[6], v[7]); g[i] = e;
    }
    __syncthreads();
    kc[0] = 0;
  }
  static __device__ __forceinline__ void decode(const Raw& r, uint32_t* wv, const uint32_t*) {
    const u32x4* grid = cb_grid_iq2s();
#pragma unroll
    for (int j = 0; j < 8; j++) {
      const uint32_t qb = ((j < 4 ? r.q.x : r.q.y) >> (8 * (j & 3))) & 0xFFu, sb = ((j < 4 ? r.sg.x : r.sg.y) >> (8 * (j & 3))) & 0xFFu;
      const u32x4 e = grid[qb | (((r.qh >> (2 * j)) & 3u) << 8)];
      wv[4 * j + 0] = e.x; wv[4 * j + 1] = e.y; wv[4 * j + 2] = e.z; wv[4 * j + 3] = e.w;
      cb_signs(sb, wv[4 * j + 0], wv[4 * j + 1], wv[4 * j + 2], wv[4 * j + 3]);
    }
#pragma unroll
    for (int g = 0; g < 4; g++) wv[32 + g] = __builtin_bit_cast(uint32_t, h2f_bits(r.d) * ((float)((r.sc >> (4 * g)) & 0xFu) + 0.5f) * 0.25f);
  }
  static __device__ __forceinline__ void stage(const uint32_t* nx, u32x4* xv, float* c) { stage_n<NG>(nx, xv, c); }
  static __device__ __forceinline__ float finish(const Raw&, const uint32_t* wv, const float* a, const float*) {
    return __builtin_bit_cast(float, wv[32]) * a[0] + __builtin_bit_cast(float, wv[33]) * a[1] + __builtin_bit_cast(float, wv[34]) * a[2] + __builtin_bit_cast(float, wv[35]) * a[3];
  }
  static __device__ __forceinline__ void to_f16(const Raw&, uint32_t* wv) { scale_n<NG>(wv); }
  static __device__ __forceinline__ void cfromx(const u32x4*, float* c) { c[0] = 0.f; c[1] = 0.f; c[2] = 0.f; c[3] = 0.f; }
};

// ------------------------------------------------------------------------------------------------ Q1_0 (gguf.py:115-118)
// 18 bytes per 128 weights: fp16 d, 128 bits; w = d (2 bit - 1), weight e = bit e % 8 of byte e / 8.  Unit h of a block: d and bytes 8 h .. 8 h + 7.  A byte's
// eight weights are fp16 1.0 with the sign bit taken from the inverted bit: no table at all.
template <> struct Fmt<GGML_Q1_0> : FmtCbBase {
  static constexpr int UPB = 2, BW = 128, BB = 18, NG = 1, NWV = 33;
  struct Raw { u32x2 q; uint32_t d; };
  static __device__ __forceinline__ Raw load(const uint8_t* row, int u) {
    const uint8_t* b = row + (size_t)BB * (u >> 1);
    Raw r; r.d = ld2_g(b); r.q = ld8_a2(b + 2 + 8 * (u & 1)); return r;
  }
  static __device__ __forceinline__ void consts(uint32_t* kc) { kc[0] = vgpr_const(0x3C003C00u); }
  static __device__ __forceinline__ void decode(const Raw& r, uint32_t* wv, const uint32_t* kc) {
#pragma unroll
    for (int j = 0; j < 8; j++) {
      wv[4 * j + 0] = kc[0]; wv[4 * j + 1] = kc[0]; wv[4 * j + 2] = kc[0]; wv[4 * j + 3] = kc[0];
      cb_signs((~((j < 4 ? r.q.x : r.q.y) >> (8 * (j & 3)))) & 0xFFu, wv[4 * j + 0], wv[4 * j + 1], wv[4 * j + 2], wv[4 * j + 3]);     // a clear bit is -1
    }
    wv[32] = __builtin_bit_cast(uint32_t, h2f_bits(r.d));
  }
  static __device__ __forceinline__ void stage(const uint32_t* nx, u32x4* xv, float* c) { stage_n<NG>(nx, xv, c); }
  static __device__ __forceinline__ float finish(const Raw&, const uint32_t* wv, const float* a, const float*) { return __builtin_bit_cast(float, wv[32]) * a[0]; }
  static __device__ __forceinline__ void to_f16(const Raw&, uint32_t* wv) { scale_n<NG>(wv); }
  static __device__ __forceinline__ void cfromx(const u32x4*, float* c) { c[0] = 0.f; }
};
