// GGUF block formats as seen by the dequant-GEMV kernels: unit geometry, loads, in-register decode, activation staging.
#pragma once
#include "common.h"
#include "host.h"

#define QG_THREADS 256
#define QG_WAVES 4
#define QG_MAX_SEG 3

struct QArgs {
  const uint8_t* w[QG_MAX_SEG];
  void* y[QG_MAX_SEG];
  const float* resid[QG_MAX_SEG];
  long long n[QG_MAX_SEG];
  const void* x;
  long long ntot;       // rows over all segments (epilogue 2: rows of one segment)
  long long row_bytes;  // bytes per weight row
  int nseg, x_f32, y_f32, epilogue;
  int K, nu;            // units per row
  int chunk_u, nchunks; // units per LDS chunk
  // job indirection (MoE expert GEMVs): blockIdx.y = job; expert = sel[job]; weights shifted by expert * estride bytes;
  // activation row = job / xdiv; outputs shifted by job * ystride elements.  sel == nullptr: a single job.
  int* sel; long long estride, ystride; int xdiv, xdiv_jobs;   // xdiv_jobs: number of jobs (grid.y)
  // x_staged: x already holds fp16 activations in the consumer format's staged order (Fmt::spos).
  // y_stage_fmt / y_stage_nu: when y_stage_fmt != 0 the fp16 outputs are written in the staged order of THAT consumer format.
  int x_staged, y_stage_fmt, y_stage_nu;
  // attn_S > 0 (M = 1 fast path, residual epilogue): x holds float32 split partials of the attention, per head (K >> attn_hd_log2 heads) [attn_S][head_dim]
  // weighted V sums followed by 16 floats holding the splits' (max, sum) pairs; the row is their merge, sum_s e_s o_s / sum_s e_s l_s with e_s = exp(m_s - max m), rounded to fp16
  // (the two fields sit where the struct had padding: qgemv1_two_kernel counts on the size of two of these)
  int attn_S;
  // norm_w != nullptr (M = 1 fast path, fp32 x): the activation row is RMS-normalised while it is staged,
  // x * rsqrt(mean(x^2) + norm_eps) * norm_w (nn.RMSNorm, tinygrad/nn/__init__.py:296-304), then rounded to fp16.
  const float* norm_w; float norm_eps; int attn_hd_log2;
  // comb_y != nullptr (with norm_w): the activation row is first completed as x + sum_j comb_p[j] * comb_y[j] over comb_k rows of K values
  // (the weighted sum over the selected experts' outputs plus the block residual, tinygrad/llm/model.py:130, 150); the completed row is
  // also written to comb_x_out (a different buffer: every workgroup reads x) by the first workgroup.
  const float* comb_y; const float* comb_p; int comb_k; float* comb_x_out;
  // route_logits != nullptr (expert gate/up jobs of one token): the kernel gates for itself - scores, pairwise top-k and weights of
  // the route_k experts from the router logits (tinygrad/llm/model.py:112-128) - instead of reading sel; job j takes the j-th selected
  // expert, and the first workgroup writes the selection and the weights to sel / route_probs_out for the launches that follow.
  const float* route_logits; int route_E, route_k, route_gating, route_norm_topk; float route_scale; float* route_probs_out;
  // M = 1 fast path: row groups per team and the remainder (the first team_rem teams take one more), so that the kernel divides nothing
  int team_base, team_rem;
  int team_skew, team_first;   // the first team_first teams own team_skew row groups more than that, the others as many fewer (0: no skew)
  int team_stride;             // > 0: team t owns row groups t, t + team_stride, ... of the one matrix instead of a contiguous range
  // touch_pos != nullptr (prologue 1, the q / k / v launch): every lane reads one dword of one 128-byte line of what the attention launch behind this one
  // will ask for - the cached K / V rows below *touch_pos of the kv heads whose attention workgroups run on this workgroup's XCD, and the rotation row of
  // that position - so that those lines wait in that XCD's L2 (caches [touch_n_kv][touch_max_ctx] rows of touch_row_bytes; nothing depends on it)
  const int* touch_pos; const uint8_t* touch_k; const uint8_t* touch_v; const uint8_t* touch_rope;
  int touch_n_kv, touch_max_ctx, touch_row_bytes, touch_rope_row_bytes;
};

// staged position of element e for a consumer of format `fmt` (row length K = UW * nu)
__device__ __forceinline__ int staged_pos(int fmt, int e, int nu);

__device__ __forceinline__ uint32_t pack_even(uint32_t a, uint32_t b) { return (a & 0xFFFFu) | (b << 16); }        // (a.lo, b.lo)
__device__ __forceinline__ uint32_t pack_odd(uint32_t a, uint32_t b) { return (a >> 16) | (b & 0xFFFF0000u); }     // (a.hi, b.hi)

template <int T> struct Fmt;
// bytes of LDS that a format's lookup tables take in every workgroup (the codebook types, qfmt_cb.h); 0 for the others
template <class F, class = void> struct FmtTab { static constexpr int value = 0; };
template <class F> struct FmtTab<F, decltype((void)F::TAB)> { static constexpr int value = F::TAB; };
template <class F> constexpr int fmt_tab() { return FmtTab<F>::value; }

// Decoded weights still carry their exponent-bias and integer offsets (1024 + q etc.) and no block scale.  to_f16 turns a decoded
// unit into the true weights as fp16 pairs, (pattern - bias) * scale: the subtraction is exact in fp16 (small integers), the
// product rounds once to fp16 - the same rounding as the reference's fp16 weight cast (tinygrad/llm/model.py:376).  Used by the
// MFMA small-batch kernel, where one decode serves all activation rows and the block scale cannot be applied after the MFMA.
__device__ __forceinline__ uint32_t h2_unbias_scale(uint32_t pattern, float bias, half2_t scale) {
  const half2_t b = {(_Float16)bias, (_Float16)bias};
  return as_u32((as_h2(pattern) - b) * scale);
}
// the same with a float32 scale: pattern * s - bias * s evaluated in float32 and rounded to fp16 once (v_fma_mix), for scales that are
// themselves products (Q6_K: d * sub-scale) and would otherwise be rounded twice
__device__ __forceinline__ uint32_t h2_unbias_scale_f32(uint32_t pattern, float scale, float neg_bias_scale) {
  const half2_t p = as_h2(pattern);
  half2_t o = {(_Float16)((float)p.x * scale + neg_bias_scale), (_Float16)((float)p.y * scale + neg_bias_scale)};
  return as_u32(o);
}
__device__ __forceinline__ half2_t h2_splat_bits(uint32_t h16) { const _Float16 v = __builtin_bit_cast(_Float16, (uint16_t)h16); half2_t r = {v, v}; return r; }
__device__ __forceinline__ half2_t h2_splat_f(float f) { const _Float16 v = (_Float16)f; half2_t r = {v, v}; return r; }


// A constant the compiler must keep in a VGPR: VOP3 forms such as v_and_or_b32 / v_perm_b32 accept a single scalar
// operand and no literal on this ISA, so (x & MASK) | BIAS only becomes one instruction when BIAS already lives in a VGPR.
__device__ __forceinline__ uint32_t vgpr_const(uint32_t c) { asm("" : "+v"(c)); return c; }

// ------------------------------------------------------------------------------------------------ Q4_0 (gguf.py:46)
template <> struct Fmt<GGML_Q4_0> {
  static constexpr int UW = 32, UPB = 1, BW = 32, BB = 18;   // weights per unit, units per block, block weights / bytes
  static __device__ __forceinline__ int unit_of(int e) { return e / UW; }
  static __device__ __forceinline__ int pair_of(int e) { return (e % UW) >> 1; }
  static constexpr int XV = 4, NG = 1, NWV = 16;
  struct Raw { u32x4 q; uint32_t d; };
  static __device__ __forceinline__ Raw load(const uint8_t* row, int u) {
    const uint8_t* p = row + 18 * u; Raw r; r.d = ld2(p); r.q = ld16(p + 2); return r;
  }
  // element index (within the row) of natural pair k (elements 2k, 2k+1) of unit u
  static __device__ __forceinline__ int xoff(int u, int k) { return 32 * u + 2 * k; }
  // wv[4t+c] multiplies x pair xs[t][c].  low nibble -> 1024+n (0x6400), high nibble in place -> 64+n (0x5400)
  static constexpr int NKC = 2;
  static __device__ __forceinline__ void consts(uint32_t* kc) { kc[0] = vgpr_const(0x64006400u); kc[1] = vgpr_const(0x54005400u); }
  static __device__ __forceinline__ void decode(const Raw& r, uint32_t* wv, const uint32_t* kc) {
#pragma unroll
    for (int t = 0; t < 4; t++) {
      const uint32_t w = r.q[t], w8 = w >> 8;
      wv[4 * t + 0] = and_or(w, 0x000F000Fu, kc[0]);    // weights 4t, 4t+2
      wv[4 * t + 1] = and_or(w, 0x00F000F0u, kc[1]);    // weights 4t+16, 4t+18
      wv[4 * t + 2] = and_or(w8, 0x000F000Fu, kc[0]);   // weights 4t+1, 4t+3
      wv[4 * t + 3] = and_or(w8, 0x00F000F0u, kc[1]);   // weights 4t+17, 4t+19
    }
  }
  static __device__ __forceinline__ void stage(const uint32_t* nx, u32x4* xv, float* c) {
#pragma unroll
    for (int t = 0; t < 4; t++) {
      xv[t].x = pack_even(nx[2 * t], nx[2 * t + 1]);       xv[t].y = pack_even(nx[2 * t + 8], nx[2 * t + 9]);
      xv[t].z = pack_odd(nx[2 * t], nx[2 * t + 1]);        xv[t].w = pack_odd(nx[2 * t + 8], nx[2 * t + 9]);
    }
    float lo = 0.f, hi = 0.f;
#pragma unroll
    for (int k = 0; k < 8; k++) { lo = dot2(nx[k], 0x64086408u, lo); hi = dot2(nx[k + 8], 0x54805480u, hi); }   // 1032, 72
    c[0] = -(lo + hi);
  }
  static __device__ __forceinline__ float finish(const Raw& r, const uint32_t*, const float* a, const float*) { return h2f_bits(r.d) * a[0]; }
};

// ------------------------------------------------------------------------------------------------ Q8_0 (gguf.py:56)
template <> struct Fmt<GGML_Q8_0> {
  static constexpr int UW = 32, UPB = 1, BW = 32, BB = 34;
  static __device__ __forceinline__ int unit_of(int e) { return e / UW; }
  static __device__ __forceinline__ int pair_of(int e) { return (e % UW) >> 1; }
  static constexpr int XV = 4, NG = 1, NWV = 16;
  struct Raw { u32x4 q0, q1; uint32_t d; };
  static __device__ __forceinline__ Raw load(const uint8_t* row, int u) {
    const uint8_t* p = row + 34 * u; Raw r; r.d = ld2(p); r.q0 = ld16(p + 2); r.q1 = ld16(p + 18); return r;
  }
  static __device__ __forceinline__ int xoff(int u, int k) { return 32 * u + 2 * k; }
  // int8 q -> byte q^0x80 = q+128 placed under exponent byte 0x64: fp16 value 1024 + 128 + q
  static constexpr int NKC = 1;
  static __device__ __forceinline__ void consts(uint32_t* kc) { kc[0] = vgpr_const(0x64646464u); }
  static __device__ __forceinline__ void decode(const Raw& r, uint32_t* wv, const uint32_t* kc) {
#pragma unroll
    for (int t = 0; t < 8; t++) {
      const uint32_t u = (t < 4 ? r.q0[t] : r.q1[t - 4]) ^ 0x80808080u;
      wv[2 * t + 0] = __builtin_amdgcn_perm(kc[0], u, 0x04010400u);   // bytes (u0,0x64,u1,0x64): weights 4t, 4t+1
      wv[2 * t + 1] = __builtin_amdgcn_perm(kc[0], u, 0x04030402u);   // weights 4t+2, 4t+3
    }
  }
  static __device__ __forceinline__ void stage(const uint32_t* nx, u32x4* xv, float* c) {
    float s = 0.f;
#pragma unroll
    for (int t = 0; t < 4; t++) { xv[t].x = nx[4 * t]; xv[t].y = nx[4 * t + 1]; xv[t].z = nx[4 * t + 2]; xv[t].w = nx[4 * t + 3]; }
#pragma unroll
    for (int k = 0; k < 16; k++) s = dot2(nx[k], 0x64806480u, s);   // 1152
    c[0] = -s;
  }
  static __device__ __forceinline__ float finish(const Raw& r, const uint32_t*, const float* a, const float*) { return h2f_bits(r.d) * a[0]; }
};


enum { F_Q4_0P = 1002, F_Q8_0P = 1008 };   // block-pair formats (4-byte aligned 36 / 68 byte units)

// Weight bytes always live in global memory: the loads name that address space, so that pointers which reach a kernel through
// a table in memory (and carry no address space of their own) still become global_load instead of FLAT instructions.
#define TGA_GLOBAL __attribute__((address_space(1)))
typedef u32x4 u32x4_a4 __attribute__((aligned(4)));
__device__ __forceinline__ u32x4 ld16_a4(const uint8_t* p) { return *(const TGA_GLOBAL u32x4_a4*)p; }   // 4-byte aligned 16-byte load
__device__ __forceinline__ uint32_t ld4_a4(const uint8_t* p) { return *(const TGA_GLOBAL uint32_t*)p; }
__device__ __forceinline__ u32x4 gld16(const void* p) { return *(const TGA_GLOBAL u32x4*)p; }            // 16-byte aligned
__device__ __forceinline__ f32x4 gld16f(const void* p) { return *(const TGA_GLOBAL f32x4*)p; }
// 16 bytes at a 2-byte aligned address: the five enclosing aligned dwords, funnel-shifted by 0 or 16 bits per lane
__device__ __forceinline__ u32x4 ld16_a2(const uint8_t* p, uint32_t& tail_dword, uint32_t& sh) {
  const uintptr_t a = (uintptr_t)p; sh = (uint32_t)(a & 2) * 8;
  const uint8_t* q = (const uint8_t*)(a & ~(uintptr_t)3);
  const u32x4 v = ld16_a4(q); const uint32_t e = ld4_a4(q + 16);
  tail_dword = e;
  u32x4 r = {__builtin_amdgcn_alignbit(v.y, v.x, sh), __builtin_amdgcn_alignbit(v.z, v.y, sh),
             __builtin_amdgcn_alignbit(v.w, v.z, sh), __builtin_amdgcn_alignbit(e, v.w, sh)};
  return r;
}

// ------------------------------------------------------------------------------------------------ Q4_0 block pair
// unit u = blocks 2u, 2u+1 of the row = 9 dwords D0..D8 at a 4-byte aligned address:
//   D0 = d0 | q0[0..1] << 16,  D1..D3 = q0[2..13],  D4 = q0[14..15] | d1 << 16,  D5..D8 = q1[0..15].
// Quant dwords: Q0 = (D0 >> 16) | (D4 << 16) = bytes q0[0], q0[1], q0[14], q0[15];  Q1..Q3 = D1..D3;  Q4..Q7 = D5..D8.
// The byte order inside Q0..Q3 differs from the block order; the activations are staged in the matching order instead.
template <> struct Fmt<F_Q4_0P> {
  static constexpr int UW = 64, UPB = 1, BW = 64, BB = 36;
  static __device__ __forceinline__ int unit_of(int e) { return e / UW; }
  static __device__ __forceinline__ int pair_of(int e) { return (e % UW) >> 1; }
  static constexpr int XV = 8, NG = 2, NWV = 32;
  struct Raw { u32x4 a, b; uint32_t c; };
  static __device__ __forceinline__ Raw load(const uint8_t* row, int u) {
    const uint8_t* p = row + 36 * u; Raw r; r.a = ld16_a4(p); r.b = ld16_a4(p + 16); r.c = ld4_a4(p + 32); return r;
  }
  static __device__ __forceinline__ int xoff(int u, int k) { return 64 * u + 2 * k; }
  static constexpr int NKC = 2;
  static __device__ __forceinline__ void consts(uint32_t* kc) { kc[0] = vgpr_const(0x64006400u); kc[1] = vgpr_const(0x54005400u); }
  static __device__ __forceinline__ void decode(const Raw& r, uint32_t* wv, const uint32_t* kc) {
    const uint32_t q[8] = {__builtin_amdgcn_alignbit(r.b.x, r.a.x, 16), r.a.y, r.a.z, r.a.w, r.b.y, r.b.z, r.b.w, r.c};
#pragma unroll
    for (int i = 0; i < 8; i++) {
      const uint32_t w = q[i], w8 = w >> 8;
      wv[4 * i + 0] = and_or(w, 0x000F000Fu, kc[0]);    // low nibbles of bytes 0, 2
      wv[4 * i + 1] = and_or(w, 0x00F000F0u, kc[1]);    // high nibbles of bytes 0, 2 (weights +16)
      wv[4 * i + 2] = and_or(w8, 0x000F000Fu, kc[0]);   // low nibbles of bytes 1, 3
      wv[4 * i + 3] = and_or(w8, 0x00F000F0u, kc[1]);   // high nibbles of bytes 1, 3
    }
  }
  // nx[k] = (x[2k], x[2k+1]) of the unit's 64 activations.  Quant dword i holds bytes (b0, b0+1, b2, b2+1) of its block with
  // (b0, b2)/2 = (0,7), (1,2), (3,4), (5,6) for block 0 and (2t, 2t+1) for block 1.
  static __device__ __forceinline__ void stage(const uint32_t* nx, u32x4* xv, float* c) {
    constexpr int P0[8] = {0, 1, 3, 5, 16, 18, 20, 22}, P2[8] = {7, 2, 4, 6, 17, 19, 21, 23};
#pragma unroll
    for (int i = 0; i < 8; i++) {
      xv[i].x = pack_even(nx[P0[i]], nx[P2[i]]);     xv[i].y = pack_even(nx[P0[i] + 8], nx[P2[i] + 8]);
      xv[i].z = pack_odd(nx[P0[i]], nx[P2[i]]);      xv[i].w = pack_odd(nx[P0[i] + 8], nx[P2[i] + 8]);
    }
#pragma unroll
    for (int j = 0; j < 2; j++) {
      float lo = 0.f, hi = 0.f;
#pragma unroll
      for (int k = 0; k < 8; k++) { lo = dot2(nx[16 * j + k], 0x64086408u, lo); hi = dot2(nx[16 * j + k + 8], 0x54805480u, hi); }   // 1032, 72
      c[j] = -(lo + hi);
    }
  }
  static __device__ __forceinline__ float finish(const Raw& r, const uint32_t*, const float* a, const float*) {
    return h2f_bits(r.a.x & 0xFFFFu) * a[0] + h2f_bits(r.b.x >> 16) * a[1];
  }
  static __device__ __forceinline__ void to_f16(const Raw& r, uint32_t* wv) {
    const half2_t d0 = h2_splat_bits(r.a.x & 0xFFFFu), d1 = h2_splat_bits(r.b.x >> 16);
#pragma unroll
    for (int i = 0; i < 8; i++) {
      const half2_t d = i < 4 ? d0 : d1;
      wv[4 * i + 0] = h2_unbias_scale(wv[4 * i + 0], 1032.f, d); wv[4 * i + 1] = h2_unbias_scale(wv[4 * i + 1], 72.f, d);
      wv[4 * i + 2] = h2_unbias_scale(wv[4 * i + 2], 1032.f, d); wv[4 * i + 3] = h2_unbias_scale(wv[4 * i + 3], 72.f, d);
    }
  }
  // halfword index of row element e inside the staged activation buffer ([XV][nu] vectors of 4 fp16 pairs)
  static __device__ __forceinline__ int spos(int e, int nu) {
    const int u = e >> 6, w = e & 63, blk = w >> 5, b = w & 31, hi = b >> 4, q = b & 15;
    int i, p;
    if (blk) { i = 4 + (q >> 2); p = q & 3; }
    else if (q < 2) { i = 0; p = q; }
    else if (q >= 14) { i = 0; p = q - 12; }
    else { i = 1 + ((q - 2) >> 2); p = (q - 2) & 3; }
    return ((i * nu + u) * 4 + (p & 1) * 2 + hi) * 2 + (p >> 1);
  }
  // the accumulator start values recomputed from staged vectors (x,z: low-nibble weights, bias 1032; y,w: high-nibble, bias 72)
  static __device__ __forceinline__ void cfromx(const u32x4* xv, float* c) {
#pragma unroll
    for (int j = 0; j < 2; j++) {
      float lo = 0.f, hi = 0.f;
#pragma unroll
      for (int i = 4 * j; i < 4 * j + 4; i++) { lo = dot2(xv[i].x, 0x64086408u, lo); lo = dot2(xv[i].z, 0x64086408u, lo); hi = dot2(xv[i].y, 0x54805480u, hi); hi = dot2(xv[i].w, 0x54805480u, hi); }
      c[j] = -(lo + hi);
    }
  }
};

// ------------------------------------------------------------------------------------------------ Q8_0 block pair
// unit u = 17 dwords D0..D16:  D0 = d0 | q0[0..1] << 16,  D1..D7 = q0[2..29],  D8 = q0[30..31] | d1 << 16,  D9..D16 = q1[0..31].
// Quant dwords: Q0 = (D0 >> 16) | (D8 << 16) = q0[0], q0[1], q0[30], q0[31];  Q1..Q7 = D1..D7;  Q8..Q15 = D9..D16.
template <> struct Fmt<F_Q8_0P> {
  static constexpr int UW = 64, UPB = 1, BW = 64, BB = 68;
  static __device__ __forceinline__ int unit_of(int e) { return e / UW; }
  static __device__ __forceinline__ int pair_of(int e) { return (e % UW) >> 1; }
  static constexpr int XV = 8, NG = 2, NWV = 32;
  struct Raw { u32x4 a, b, c, d; uint32_t e; };
  static __device__ __forceinline__ Raw load(const uint8_t* row, int u) {
    const uint8_t* p = row + 68 * u; Raw r; r.a = ld16_a4(p); r.b = ld16_a4(p + 16); r.c = ld16_a4(p + 32); r.d = ld16_a4(p + 48); r.e = ld4_a4(p + 64); return r;
  }
  static __device__ __forceinline__ int xoff(int u, int k) { return 64 * u + 2 * k; }
  static constexpr int NKC = 1;
  static __device__ __forceinline__ void consts(uint32_t* kc) { kc[0] = vgpr_const(0x64646464u); }
  static __device__ __forceinline__ void decode(const Raw& r, uint32_t* wv, const uint32_t* kc) {
    const uint32_t q[16] = {__builtin_amdgcn_alignbit(r.c.x, r.a.x, 16), r.a.y, r.a.z, r.a.w, r.b.x, r.b.y, r.b.z, r.b.w,
                            r.c.y, r.c.z, r.c.w, r.d.x, r.d.y, r.d.z, r.d.w, r.e};
#pragma unroll
    for (int i = 0; i < 16; i++) {
      const uint32_t u = q[i] ^ 0x80808080u;
      wv[2 * i + 0] = __builtin_amdgcn_perm(kc[0], u, 0x04010400u);   // bytes 0, 1 -> fp16 1152 + q
      wv[2 * i + 1] = __builtin_amdgcn_perm(kc[0], u, 0x04030402u);   // bytes 2, 3
    }
  }
  // pairs in decode order: block 0: N0, N15, N1, N2, ..., N14;  block 1: natural
  static __device__ __forceinline__ void stage(const uint32_t* nx, u32x4* xv, float* c) {
    constexpr int ORD[16] = {0, 15, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14};
#pragma unroll
    for (int v = 0; v < 4; v++) { xv[v].x = nx[ORD[4 * v]]; xv[v].y = nx[ORD[4 * v + 1]]; xv[v].z = nx[ORD[4 * v + 2]]; xv[v].w = nx[ORD[4 * v + 3]]; }
#pragma unroll
    for (int v = 4; v < 8; v++) { xv[v].x = nx[4 * v]; xv[v].y = nx[4 * v + 1]; xv[v].z = nx[4 * v + 2]; xv[v].w = nx[4 * v + 3]; }
#pragma unroll
    for (int j = 0; j < 2; j++) {
      float t = 0.f;
#pragma unroll
      for (int k = 0; k < 16; k++) t = dot2(nx[16 * j + k], 0x64806480u, t);   // 1152
      c[j] = -t;
    }
  }
  static __device__ __forceinline__ float finish(const Raw& r, const uint32_t*, const float* a, const float*) {
    return h2f_bits(r.a.x & 0xFFFFu) * a[0] + h2f_bits(r.c.x >> 16) * a[1];
  }
  static __device__ __forceinline__ void to_f16(const Raw& r, uint32_t* wv) {
    const half2_t d0 = h2_splat_bits(r.a.x & 0xFFFFu), d1 = h2_splat_bits(r.c.x >> 16);
#pragma unroll
    for (int i = 0; i < 32; i++) wv[i] = h2_unbias_scale(wv[i], 1152.f, i < 16 ? d0 : d1);
  }
  static __device__ __forceinline__ int spos(int e, int nu) {
    const int u = e >> 6, w = e & 63, blk = w >> 5, b = w & 31, n = b >> 1;
    const int s = blk ? 16 + n : (n == 0 ? 0 : (n == 15 ? 1 : n + 1));
    return (((s >> 2) * nu + u) * 4 + (s & 3)) * 2 + (b & 1);
  }
  static __device__ __forceinline__ void cfromx(const u32x4* xv, float* c) {
#pragma unroll
    for (int j = 0; j < 2; j++) {
      float t = 0.f;
#pragma unroll
      for (int i = 4 * j; i < 4 * j + 4; i++) { t = dot2(xv[i].x, 0x64806480u, t); t = dot2(xv[i].y, 0x64806480u, t); t = dot2(xv[i].z, 0x64806480u, t); t = dot2(xv[i].w, 0x64806480u, t); }
      c[j] = -t;
    }
  }
};


// ------------------------------------------------------------------------------------------------ F16 (dense fp16 rows, gguf.py:35-36)
// unit = 64 consecutive fp16 weights (128 bytes); no decode: the weight dwords are the fp16 pairs.
template <> struct Fmt<GGML_F16> {
  // A unit is 64 weights, but NOT 64 consecutive ones: the row is cut into 16-byte pieces (8 weights) and unit u owns pieces
  // u, u + nu, ..., u + 7 nu (nu = units per row), so that load instruction j of a wave covers pieces j*nu .. j*nu + 63, one
  // contiguous span (a lane stride of 128 bytes would touch 64 cache lines per instruction).  The fast M = 1 kernel uses
  // load_nu / unit_of_nu / pair_of_nu; the staged order of a row is therefore the natural order.
  static constexpr int UW = 64, UPB = 1, BW = 64, BB = 128;
  static __device__ __forceinline__ int unit_of(int e) { return e / UW; }
  static __device__ __forceinline__ int pair_of(int e) { return (e % UW) >> 1; }
  static __device__ __forceinline__ int unit_of_nu(int e, int nu) { return (e >> 3) % nu; }
  static __device__ __forceinline__ int pair_of_nu(int e, int nu) { return ((e >> 3) / nu) * 4 + ((e & 7) >> 1); }
  static constexpr int XV = 8, NG = 1, NWV = 32;
  struct Raw { u32x4 q[8]; };
  static __device__ __forceinline__ Raw load(const uint8_t* row, int u) {
    const uint8_t* p = row + 128 * u; Raw r;
#pragma unroll
    for (int i = 0; i < 8; i++) r.q[i] = ld16_a4(p + 16 * i);
    return r;
  }
  static __device__ __forceinline__ Raw load_nu(const uint8_t* row, int u, int nu) {
    const uint8_t* p = row + 16 * u; Raw r;
#pragma unroll
    for (int i = 0; i < 8; i++) r.q[i] = ld16_a4(p + (size_t)16 * nu * i);
    return r;
  }
  static __device__ __forceinline__ int xoff(int u, int k) { return 64 * u + 2 * k; }
  static constexpr int NKC = 1;
  static __device__ __forceinline__ void consts(uint32_t* kc) { kc[0] = 0; }
  static __device__ __forceinline__ void decode(const Raw& r, uint32_t* wv, const uint32_t*) {
#pragma unroll
    for (int i = 0; i < 8; i++) { wv[4 * i] = r.q[i].x; wv[4 * i + 1] = r.q[i].y; wv[4 * i + 2] = r.q[i].z; wv[4 * i + 3] = r.q[i].w; }
  }
  static __device__ __forceinline__ void stage(const uint32_t* nx, u32x4* xv, float* c) {
#pragma unroll
    for (int v = 0; v < 8; v++) { xv[v].x = nx[4 * v]; xv[v].y = nx[4 * v + 1]; xv[v].z = nx[4 * v + 2]; xv[v].w = nx[4 * v + 3]; }
    c[0] = 0.f;
  }
  static __device__ __forceinline__ float finish(const Raw&, const uint32_t*, const float* a, const float*) { return a[0]; }
  static __device__ __forceinline__ void to_f16(const Raw&, uint32_t*) {}      // already the fp16 weights
  static __device__ __forceinline__ int spos(int e, int nu) { return e; }
  static __device__ __forceinline__ void cfromx(const u32x4*, float* c) { c[0] = 0.f; }
};

// ------------------------------------------------------------------------------------------------ MXFP4 (gguf.py:105-114)
template <> struct Fmt<GGML_MXFP4> {
  static constexpr int UW = 32, UPB = 1, BW = 32, BB = 17;
  static __device__ __forceinline__ int unit_of(int e) { return e / UW; }
  static __device__ __forceinline__ int pair_of(int e) { return (e % UW) >> 1; }
  static constexpr int XV = 4, NG = 1, NWV = 16;
  struct Raw { u32x4 q; uint32_t e; };
  static __device__ __forceinline__ Raw load(const uint8_t* row, int u) {
    // the 17-byte block starts at any byte offset o of an aligned dword: load the five enclosing dwords and shift
    const uintptr_t a = (uintptr_t)(row + 17 * u); const uint32_t o = (uint32_t)(a & 3);
    const uint8_t* q = (const uint8_t*)(a & ~(uintptr_t)3);
    const u32x4 v = ld16_a4(q); const uint32_t t = ld4_a4(q + 16);
    const uint32_t sh = 8 * (o + 1);   // 8..32
    Raw r; r.e = (v.x >> (8 * o)) & 0xFFu;
    r.q.x = (uint32_t)((((uint64_t)v.y << 32) | v.x) >> sh); r.q.y = (uint32_t)((((uint64_t)v.z << 32) | v.y) >> sh);
    r.q.z = (uint32_t)((((uint64_t)v.w << 32) | v.z) >> sh); r.q.w = (uint32_t)((((uint64_t)t << 32) | v.w) >> sh);
    return r;
  }
  static __device__ __forceinline__ int xoff(int u, int k) { return 32 * u + 2 * k; }
  // hardware E2M1 -> fp16 (true values 0..6); byte s of dword t holds weights 4t+s (low nibble) and 4t+s+16 (high nibble)
  static constexpr int NKC = 1;
  static __device__ __forceinline__ void consts(uint32_t* kc) { kc[0] = 0; }
  static __device__ __forceinline__ void decode(const Raw& r, uint32_t* wv, const uint32_t*) {
#pragma unroll
    for (int t = 0; t < 4; t++) {
      wv[4 * t + 0] = as_u32(__builtin_amdgcn_cvt_scalef32_pk_f16_fp4(r.q[t], 1.0f, 0));
      wv[4 * t + 1] = as_u32(__builtin_amdgcn_cvt_scalef32_pk_f16_fp4(r.q[t], 1.0f, 1));
      wv[4 * t + 2] = as_u32(__builtin_amdgcn_cvt_scalef32_pk_f16_fp4(r.q[t], 1.0f, 2));
      wv[4 * t + 3] = as_u32(__builtin_amdgcn_cvt_scalef32_pk_f16_fp4(r.q[t], 1.0f, 3));
    }
  }
  static __device__ __forceinline__ void stage(const uint32_t* nx, u32x4* xv, float* c) {
#pragma unroll
    for (int t = 0; t < 4; t++) {   // pairs (x[j], x[j+16]), j = 4t..4t+3
      xv[t].x = pack_even(nx[2 * t], nx[2 * t + 8]);         xv[t].y = pack_odd(nx[2 * t], nx[2 * t + 8]);
      xv[t].z = pack_even(nx[2 * t + 1], nx[2 * t + 9]);     xv[t].w = pack_odd(nx[2 * t + 1], nx[2 * t + 9]);
    }
    c[0] = 0.f;
  }
  // reference value = (2 * e2m1) * 2^(e-128) = e2m1 * 2^(e-127); e = 0 is the fp32 subnormal 2^-127
  static __device__ __forceinline__ float finish(const Raw& r, const uint32_t*, const float* a, const float*) {
    return __builtin_bit_cast(float, r.e ? (r.e << 23) : 0x00400000u) * a[0];
  }
  // true weights e2m1 * 2^(e-127) as fp16 (exact unless the scale leaves the fp16 range, where the reference's fp16 weight cast saturates too)
  static __device__ __forceinline__ void to_f16(const Raw& r, uint32_t* wv) {
    const float sc = __builtin_bit_cast(float, r.e ? (r.e << 23) : 0x00400000u);
#pragma unroll
    for (int t = 0; t < 4; t++) {
      wv[4 * t + 0] = as_u32(__builtin_amdgcn_cvt_scalef32_pk_f16_fp4(r.q[t], sc, 0));
      wv[4 * t + 1] = as_u32(__builtin_amdgcn_cvt_scalef32_pk_f16_fp4(r.q[t], sc, 1));
      wv[4 * t + 2] = as_u32(__builtin_amdgcn_cvt_scalef32_pk_f16_fp4(r.q[t], sc, 2));
      wv[4 * t + 3] = as_u32(__builtin_amdgcn_cvt_scalef32_pk_f16_fp4(r.q[t], sc, 3));
    }
  }
  static __device__ __forceinline__ int spos(int e, int nu) { const int u = e >> 5, b = e & 31, q = b & 15; return (((q >> 2) * nu + u) * 4 + (q & 3)) * 2 + (b >> 4); }
  static __device__ __forceinline__ void cfromx(const u32x4*, float* c) { c[0] = 0.f; }
};

// ------------------------------------------------------------------------------------------------ Q6_K (gguf.py:68-72)
// unit u of a row: superblock u>>2, half h=(u>>1)&1, sixteen-run g=u&1.  Its 64 weights are, for j = 0..3 and i = 0..15,
// element 256*sb + 128*h + 32*j + 16*g + i, decoded from ql[64h+16g+i] (j even) / ql[64h+32+16g+i] (j odd), low nibble for
// j < 2 and high nibble for j >= 2, and bits 2j..2j+1 of qh[32h+16g+i]; all sixteen share scale sc[8h + 2j + g].
template <> struct Fmt<GGML_Q6_K> {
  static constexpr int UW = 64, UPB = 4, BW = 256, BB = 210;
  static __device__ __forceinline__ int unit_of(int e) { return ((e >> 8) << 2) + (((e >> 7) & 1) << 1) + ((e >> 4) & 1); }
  static __device__ __forceinline__ int pair_of(int e) { return (((e >> 5) & 3) << 3) + ((e & 15) >> 1); }
  static constexpr int XV = 8, NG = 4, NWV = 32;
  struct Raw { u32x4 a, b, h; uint32_t sc0, sc1, d; };
  static __device__ __forceinline__ Raw load(const uint8_t* row, int u) {
    // superblocks are 2-byte aligned: every piece is loaded as its enclosing aligned dwords and funnel-shifted per lane
    const uint8_t* p = row + 210 * (u >> 2); const int h = (u >> 1) & 1, g = u & 1;
    uint32_t tail, sh;
    Raw r; r.a = ld16_a2(p + 64 * h + 16 * g, tail, sh); r.b = ld16_a2(p + 64 * h + 32 + 16 * g, tail, sh); r.h = ld16_a2(p + 128 + 32 * h + 16 * g, tail, sh);
    const u32x4 sc = ld16_a2(p + 192, tail, sh);                         // sc[0..15]; tail dword holds d (bytes 208, 209)
    r.sc0 = h ? sc.z : sc.x; r.sc1 = h ? sc.w : sc.y;
    r.d = (uint32_t)g | (__builtin_amdgcn_alignbit(0u, tail, sh) << 16);
    return r;
  }
  static __device__ __forceinline__ int xoff(int u, int k) {   // k = 0..31: natural pair k of the unit's 64 x values (j = k/8)
    return 256 * (u >> 2) + 128 * ((u >> 1) & 1) + 32 * (k >> 3) + 16 * (u & 1) + 2 * (k & 7);
  }
  // wv[8j + 2t + {0,1}] = even / odd pairs of dword t of group j; value 1024 + 6-bit q
  static constexpr int NKC = 1;
  static __device__ __forceinline__ void consts(uint32_t* kc) { kc[0] = vgpr_const(0x64006400u); }
  static __device__ __forceinline__ void decode(const Raw& r, uint32_t* wv, const uint32_t* kc) {
    const uint32_t K64 = kc[0];
#pragma unroll
    for (int t = 0; t < 4; t++) {
      const uint32_t A = r.a[t], B = r.b[t], H = r.h[t];
      wv[0 + 2 * t]      = and_or(H << 4, 0x00300030u, and_or(A, 0x000F000Fu, K64));
      wv[0 + 2 * t + 1]  = and_or(H >> 4, 0x00300030u, and_or(A >> 8, 0x000F000Fu, K64));
      wv[8 + 2 * t]      = and_or(H << 2, 0x00300030u, and_or(B, 0x000F000Fu, K64));
      wv[8 + 2 * t + 1]  = and_or(H >> 6, 0x00300030u, and_or(B >> 8, 0x000F000Fu, K64));
      wv[16 + 2 * t]     = and_or(H, 0x00300030u, and_or(A >> 4, 0x000F000Fu, K64));
      wv[16 + 2 * t + 1] = and_or(H >> 8, 0x00300030u, and_or(A >> 12, 0x000F000Fu, K64));
      wv[24 + 2 * t]     = and_or(H >> 2, 0x00300030u, and_or(B >> 4, 0x000F000Fu, K64));
      wv[24 + 2 * t + 1] = and_or(H >> 10, 0x00300030u, and_or(B >> 12, 0x000F000Fu, K64));
    }
  }
  // xv[2j + t/2] = {E(t), O(t), E(t+1), O(t+1)} (t even), E/O = even/odd element pairs of dword t of group j
  static __device__ __forceinline__ void stage(const uint32_t* nx, u32x4* xv, float* c) {
#pragma unroll
    for (int j = 0; j < 4; j++) {
      const uint32_t* n = nx + 8 * j;
      xv[2 * j].x = pack_even(n[0], n[1]); xv[2 * j].y = pack_odd(n[0], n[1]); xv[2 * j].z = pack_even(n[2], n[3]); xv[2 * j].w = pack_odd(n[2], n[3]);
      xv[2 * j + 1].x = pack_even(n[4], n[5]); xv[2 * j + 1].y = pack_odd(n[4], n[5]); xv[2 * j + 1].z = pack_even(n[6], n[7]); xv[2 * j + 1].w = pack_odd(n[6], n[7]);
      float s = 0.f;
#pragma unroll
      for (int k = 0; k < 8; k++) s = dot2(n[k], 0x64206420u, s);   // 1056 = 1024 + 32
      c[j] = -s;
    }
  }
  static __device__ __forceinline__ float finish(const Raw& r, const uint32_t*, const float* a, const float*) {
    const int g8 = (r.d & 1) * 8;   // scales 8h + 2j + g live in bytes g, g+2 of sc0 (j = 0, 1) and sc1 (j = 2, 3)
    const float s0 = (float)(int)(int8_t)(r.sc0 >> g8), s1 = (float)(int)(int8_t)(r.sc0 >> (16 + g8));
    const float s2 = (float)(int)(int8_t)(r.sc1 >> g8), s3 = (float)(int)(int8_t)(r.sc1 >> (16 + g8));
    return h2f_bits(r.d >> 16) * (s0 * a[0] + s1 * a[1] + s2 * a[2] + s3 * a[3]);
  }
  static __device__ __forceinline__ void to_f16(const Raw& r, uint32_t* wv) {
    const int g8 = (r.d & 1) * 8;
    const float d = h2f_bits(r.d >> 16);
    const float s[4] = {d * (float)(int)(int8_t)(r.sc0 >> g8), d * (float)(int)(int8_t)(r.sc0 >> (16 + g8)),
                        d * (float)(int)(int8_t)(r.sc1 >> g8), d * (float)(int)(int8_t)(r.sc1 >> (16 + g8))};
#pragma unroll
    for (int i = 0; i < 32; i++) wv[i] = h2_unbias_scale_f32(wv[i], s[i >> 3], -1056.f * s[i >> 3]);
  }
  static __device__ __forceinline__ int spos(int e, int nu) {
    const int u = unit_of(e), j = (e >> 5) & 3, i = e & 15, td = i >> 2, p = i & 3;
    return (((2 * j + (td >> 1)) * nu + u) * 4 + (td & 1) * 2 + (p & 1)) * 2 + (p >> 1);
  }
  static __device__ __forceinline__ void cfromx(const u32x4* xv, float* c) {
#pragma unroll
    for (int j = 0; j < 4; j++) {
      float t = 0.f;
#pragma unroll
      for (int i = 2 * j; i < 2 * j + 2; i++) { t = dot2(xv[i].x, 0x64206420u, t); t = dot2(xv[i].y, 0x64206420u, t); t = dot2(xv[i].z, 0x64206420u, t); t = dot2(xv[i].w, 0x64206420u, t); }
      c[j] = -t;
    }
  }
};


__device__ __forceinline__ float silu_f(float v) { return v / (1.0f + __expf(-v)); }

// ------------------------------------------------------------------------------------------------ Q4_K / Q5_K (gguf.py:57-67)
// Superblock of 256 weights: fp16 d, dmin, 12 bytes of packed 6-bit (scale, min) for 8 sub-blocks of 32, [Q5_K: qh[32]], qs[128].
// qs[32p + i] holds weight i of sub-block 2p (low nibble) and of sub-block 2p + 1 (high nibble); Q5_K adds 16 * bit sb of qh[i].
// A unit is one such pair of sub-blocks (64 consecutive weights, 32 bytes of qs); accumulator group 0 is the low-nibble sub-block
// (decoded as 1024 + q), group 1 the high-nibble one (64 + q, nibble left in place).  w = (d sc) q - dmin mn, so the unit's
// contribution is d (sc0 S0 + sc1 S1) - dmin (mn0 X0 + mn1 X1) with S = sum q x and X = sum x; X comes out of the bias
// corrections the lane already holds (c0 = -1024 X0, c1 = -64 X1).  Blocks are multiples of 16 bytes: all loads are aligned.
template <bool FIVE> struct RawK45;
template <> struct RawK45<false> { u32x4 q0, q1, hdr; uint32_t p; };
template <> struct RawK45<true> { u32x4 q0, q1, hdr, h0, h1; uint32_t p; };
template <bool FIVE> struct FmtK45 {
  static constexpr int UW = 64, UPB = 4, BW = 256, BB = FIVE ? 176 : 144, QS = FIVE ? 48 : 16;
  static __device__ __forceinline__ int unit_of(int e) { return e >> 6; }
  static __device__ __forceinline__ int pair_of(int e) { return (e & 63) >> 1; }
  static constexpr int XV = 8, NG = 2, NWV = 36;
  typedef RawK45<FIVE> Raw;
  static __device__ __forceinline__ Raw load(const uint8_t* row, int u) {
    const uint8_t* b = row + (size_t)BB * (u >> 2); const int p = u & 3;
    Raw r; r.hdr = ld16_a4(b); r.q0 = ld16_a4(b + QS + 32 * p); r.q1 = ld16_a4(b + QS + 32 * p + 16);
    if constexpr (FIVE) { r.h0 = ld16_a4(b + 16); r.h1 = ld16_a4(b + 32); }
    r.p = (uint32_t)p;
    return r;
  }
  static __device__ __forceinline__ int xoff(int u, int k) { return 64 * u + 2 * k; }
  static constexpr int NKC = 2;
  static __device__ __forceinline__ void consts(uint32_t* kc) { kc[0] = vgpr_const(0x64006400u); kc[1] = vgpr_const(0x54005400u); }
  // wv[16g + 2t + o] = weights (4t + o, 4t + o + 2) of group g (t = dword of the 32 qs bytes, o = odd byte)
  static __device__ __forceinline__ void decode(const Raw& r, uint32_t* wv, const uint32_t* kc) {
#pragma unroll
    for (int t = 0; t < 8; t++) {
      const uint32_t w = t < 4 ? r.q0[t & 3] : r.q1[t & 3], w8 = w >> 8;
      uint32_t le = and_or(w, 0x000F000Fu, kc[0]), lo = and_or(w8, 0x000F000Fu, kc[0]);
      uint32_t he = and_or(w, 0x00F000F0u, kc[1]), ho = and_or(w8, 0x00F000F0u, kc[1]);
      if constexpr (FIVE) {
        const uint32_t H = (t < 4 ? r.h0[t & 3] : r.h1[t & 3]) >> (2 * r.p);   // bit 0 / 1 of every byte: fifth bit of sub-block 2p / 2p + 1
        le = and_or(H << 4, 0x00100010u, le); lo = and_or(H >> 4, 0x00100010u, lo);
        he = and_or(H << 7, 0x01000100u, he); ho = and_or(H >> 1, 0x01000100u, ho);
      }
      wv[2 * t] = le; wv[2 * t + 1] = lo; wv[16 + 2 * t] = he; wv[16 + 2 * t + 1] = ho;
    }
    // get_scale_min_k4 for sub-blocks 2p, 2p + 1: byte index i = 2 (p & 1) (+1) of scales[0..3] / [4..7] / [8..11]; branch-free blend
    const uint32_t sh = 16 * (r.p & 1), hm = 0u - (r.p >> 1);                 // hm = all ones for sub-blocks 4..7
    const uint32_t y0 = (r.hdr.y >> sh) & 0xFF, y1 = (r.hdr.y >> (sh + 8)) & 0xFF, z0 = (r.hdr.z >> sh) & 0xFF, z1 = (r.hdr.z >> (sh + 8)) & 0xFF;
    const uint32_t w0 = (r.hdr.w >> sh) & 0xFF, w1 = (r.hdr.w >> (sh + 8)) & 0xFF;
    const uint32_t sc0 = ((y0 & 63) & ~hm) | (((w0 & 0xF) | ((y0 >> 6) << 4)) & hm), sc1 = ((y1 & 63) & ~hm) | (((w1 & 0xF) | ((y1 >> 6) << 4)) & hm);
    const uint32_t mn0 = ((z0 & 63) & ~hm) | (((w0 >> 4) | ((z0 >> 6) << 4)) & hm), mn1 = ((z1 & 63) & ~hm) | (((w1 >> 4) | ((z1 >> 6) << 4)) & hm);
    const float d = h2f_bits(r.hdr.x & 0xFFFF), dmin = h2f_bits(r.hdr.x >> 16);
    wv[32] = __builtin_bit_cast(uint32_t, d * (float)sc0); wv[33] = __builtin_bit_cast(uint32_t, d * (float)sc1);
    wv[34] = __builtin_bit_cast(uint32_t, dmin * (float)mn0 * (1.0f / 1024.0f)); wv[35] = __builtin_bit_cast(uint32_t, dmin * (float)mn1 * (1.0f / 64.0f));
  }
  // nx[k] = natural pair k of the unit's 64 activations; xv[4g + v] = {E, O, E', O'} of dwords 2v, 2v + 1 of group g
  static __device__ __forceinline__ void stage(const uint32_t* nx, u32x4* xv, float* c) {
#pragma unroll
    for (int g = 0; g < 2; g++) {
      const uint32_t* n = nx + 16 * g;
#pragma unroll
      for (int v = 0; v < 4; v++) {
        xv[4 * g + v].x = pack_even(n[4 * v], n[4 * v + 1]); xv[4 * g + v].y = pack_odd(n[4 * v], n[4 * v + 1]);
        xv[4 * g + v].z = pack_even(n[4 * v + 2], n[4 * v + 3]); xv[4 * g + v].w = pack_odd(n[4 * v + 2], n[4 * v + 3]);
      }
      float s = 0.f;
#pragma unroll
      for (int k = 0; k < 16; k++) s = dot2(n[k], g ? 0x54005400u : 0x64006400u, s);
      c[g] = -s;
    }
  }
  // decode() leaves the unit's four scale factors behind the weights: wv[32..35] = d sc0, d sc1, dmin mn0 / 1024, dmin mn1 / 64
  // (extracted once per unit, not once per activation row)
  static __device__ __forceinline__ float finish(const Raw&, const uint32_t* wv, const float* a, const float* c) {
    return __builtin_bit_cast(float, wv[32]) * a[0] + __builtin_bit_cast(float, wv[33]) * a[1]
         + __builtin_bit_cast(float, wv[34]) * c[0] + __builtin_bit_cast(float, wv[35]) * c[1];
  }
  // true weights (d sc) q - dmin mn as fp16, one rounding: group 0 patterns are 1024 + q, group 1 patterns 64 + q
  static __device__ __forceinline__ void to_f16(const Raw&, uint32_t* wv) {
    const float s0 = __builtin_bit_cast(float, wv[32]), s1 = __builtin_bit_cast(float, wv[33]);
    const float c0 = -1024.f * s0 - 1024.f * __builtin_bit_cast(float, wv[34]), c1 = -64.f * s1 - 64.f * __builtin_bit_cast(float, wv[35]);
#pragma unroll
    for (int i = 0; i < 16; i++) { wv[i] = h2_unbias_scale_f32(wv[i], s0, c0); wv[16 + i] = h2_unbias_scale_f32(wv[16 + i], s1, c1); }
  }
  static __device__ __forceinline__ int spos(int e, int nu) {
    const int u = e >> 6, g = (e >> 5) & 1, r = e & 31, wi = 2 * (r >> 2) + (r & 1);
    return (((4 * g + (wi >> 2)) * nu + u) * 4 + (wi & 3)) * 2 + ((r >> 1) & 1);
  }
  static __device__ __forceinline__ void cfromx(const u32x4* xv, float* c) {
#pragma unroll
    for (int g = 0; g < 2; g++) {
      const uint32_t k = g ? 0x54005400u : 0x64006400u;
      float t = 0.f;
#pragma unroll
      for (int i = 4 * g; i < 4 * g + 4; i++) { t = dot2(xv[i].x, k, t); t = dot2(xv[i].y, k, t); t = dot2(xv[i].z, k, t); t = dot2(xv[i].w, k, t); }
      c[g] = -t;
    }
  }
};
template <> struct Fmt<GGML_Q4_K> : FmtK45<false> {};
template <> struct Fmt<GGML_Q5_K> : FmtK45<true> {};

// ------------------------------------------------------------------------------------------------ IQ4_XS (gguf.py:96-104)
// Superblock of 256 weights, 136 bytes: fp16 d, uint16 scales_h, scales_l[4], qs[128].  Sub-block s (32 weights) = qs[16 s .. 16 s + 15], weight j the low
// nibble of byte j, weight j + 16 the high nibble (the Q4_0 order); its 6-bit scale is ls = (nibble s of scales_l | bits 2 s, 2 s + 1 of scales_h << 4) - 32;
// w = d ls kvalues_iq4nl[code], a 16-entry table of int8 values.  A unit is a pair of sub-blocks (64 consecutive weights, 32 bytes of qs at an 8-byte
// aligned offset), accumulator group g = sub-block 2 p + g.  The table lives in four registers as bytes value + 128: two v_perm_b32 look four codes up in
// either half of it, a third picks per byte by the code's top bit, a fourth pairs the bytes with an 0x64 exponent byte, so that a weight decodes to the
// fp16 pattern 1024 + 128 + value (bias 1152, removed through the accumulator's start value like every other format's).
template <> struct Fmt<GGML_IQ4_XS> {
  static constexpr int UW = 64, UPB = 4, BW = 256, BB = 136;
  static __device__ __forceinline__ int unit_of(int e) { return e >> 6; }
  static __device__ __forceinline__ int pair_of(int e) { return (e & 63) >> 1; }
  static constexpr int XV = 8, NG = 2, NWV = 34;
  struct Raw { u32x4 q0, q1; uint32_t h0, h1, p; };
  static __device__ __forceinline__ Raw load(const uint8_t* row, int u) {
    const uint8_t* b = row + (size_t)BB * (u >> 2); const int p = u & 3;
    Raw r; r.h0 = ld4_a4(b); r.h1 = ld4_a4(b + 4); r.q0 = ld16_a4(b + 8 + 32 * p); r.q1 = ld16_a4(b + 24 + 32 * p); r.p = (uint32_t)p;
    return r;
  }
  static __device__ __forceinline__ int xoff(int u, int k) { return 64 * u + 2 * k; }
  static constexpr int NKC = 5;
  // kvalues_iq4nl + 128 = 1, 24, 45, 63 | 79, 93, 106, 118 | 129, 141, 153, 166 | 181, 197, 217, 241
  static __device__ __forceinline__ void consts(uint32_t* kc) {
    kc[0] = vgpr_const(0x3F2D1801u); kc[1] = vgpr_const(0x766A5D4Fu); kc[2] = vgpr_const(0xA6998D81u); kc[3] = vgpr_const(0xF1D9C5B5u); kc[4] = vgpr_const(0x64646464u);
  }
  // the table bytes of four codes (bits 0..3 of every byte of `codes`; the upper nibbles are ignored)
  static __device__ __forceinline__ uint32_t lut4(uint32_t codes, const uint32_t* kc) {
    const uint32_t sel = codes & 0x07070707u;
    const uint32_t lo = __builtin_amdgcn_perm(kc[1], kc[0], sel), hi = __builtin_amdgcn_perm(kc[3], kc[2], sel);
    return __builtin_amdgcn_perm(hi, lo, and_or(codes >> 1, 0x04040404u, 0x03020100u));      // byte i from lo (selector i) or from hi (4 + i) by the code's bit 3
  }
  // wv[4 (4 g + t) + {0, 1, 2, 3}] = weights (4t, 4t+1), (4t+2, 4t+3), (16+4t, 16+4t+1), (16+4t+2, 16+4t+3) of sub-block 2 p + g (t = dword of its 16 bytes)
  static __device__ __forceinline__ void decode(const Raw& r, uint32_t* wv, const uint32_t* kc) {
#pragma unroll
    for (int i = 0; i < 8; i++) {
      const uint32_t w = i < 4 ? r.q0[i & 3] : r.q1[i & 3];
      const uint32_t l = lut4(w, kc), h = lut4(w >> 4, kc);
      wv[4 * i + 0] = __builtin_amdgcn_perm(kc[4], l, 0x04010400u); wv[4 * i + 1] = __builtin_amdgcn_perm(kc[4], l, 0x04030402u);
      wv[4 * i + 2] = __builtin_amdgcn_perm(kc[4], h, 0x04010400u); wv[4 * i + 3] = __builtin_amdgcn_perm(kc[4], h, 0x04030402u);
    }
    const uint32_t lb = (r.h1 >> (8 * r.p)) & 0xFF, hs = (r.h0 >> (16 + 4 * r.p)) & 0xF;
    const int ls0 = (int)((lb & 0xF) | ((hs & 3) << 4)) - 32, ls1 = (int)((lb >> 4) | ((hs >> 2) << 4)) - 32;
    const float d = h2f_bits(r.h0 & 0xFFFF);
    wv[32] = __builtin_bit_cast(uint32_t, d * (float)ls0); wv[33] = __builtin_bit_cast(uint32_t, d * (float)ls1);
  }
  // nx[k] = natural pair k of the unit's 64 activations; xv[4 g + t] = pairs 2t, 2t + 1, 8 + 2t, 8 + 2t + 1 of sub-block g
  static __device__ __forceinline__ void stage(const uint32_t* nx, u32x4* xv, float* c) {
#pragma unroll
    for (int g = 0; g < 2; g++) {
      const uint32_t* n = nx + 16 * g;
#pragma unroll
      for (int t = 0; t < 4; t++) { xv[4 * g + t].x = n[2 * t]; xv[4 * g + t].y = n[2 * t + 1]; xv[4 * g + t].z = n[8 + 2 * t]; xv[4 * g + t].w = n[8 + 2 * t + 1]; }
      float s = 0.f;
#pragma unroll
      for (int k = 0; k < 16; k++) s = dot2(n[k], 0x64806480u, s);        // 1152
      c[g] = -s;
    }
  }
  static __device__ __forceinline__ float finish(const Raw&, const uint32_t* wv, const float* a, const float*) {
    return __builtin_bit_cast(float, wv[32]) * a[0] + __builtin_bit_cast(float, wv[33]) * a[1];
  }
  static __device__ __forceinline__ void to_f16(const Raw&, uint32_t* wv) {
    const float s0 = __builtin_bit_cast(float, wv[32]), s1 = __builtin_bit_cast(float, wv[33]);
#pragma unroll
    for (int i = 0; i < 16; i++) { wv[i] = h2_unbias_scale_f32(wv[i], s0, -1152.f * s0); wv[16 + i] = h2_unbias_scale_f32(wv[16 + i], s1, -1152.f * s1); }
  }
  static __device__ __forceinline__ int spos(int e, int nu) {
    const int u = e >> 6, g = (e >> 5) & 1, r = e & 31, hi = r >> 4, q = r & 15, t = q >> 2, k = q & 3;
    return (((4 * g + t) * nu + u) * 4 + hi * 2 + (k >> 1)) * 2 + (k & 1);
  }
  static __device__ __forceinline__ void cfromx(const u32x4* xv, float* c) {
#pragma unroll
    for (int g = 0; g < 2; g++) {
      float t = 0.f;
#pragma unroll
      for (int i = 4 * g; i < 4 * g + 4; i++) { t = dot2(xv[i].x, 0x64806480u, t); t = dot2(xv[i].y, 0x64806480u, t); t = dot2(xv[i].z, 0x64806480u, t); t = dot2(xv[i].w, 0x64806480u, t); }
      c[g] = -t;
    }
  }
};

// ------------------------------------------------------------------------------------------------ Q4_1 / Q5_0 / Q5_1 (gguf.py:47-55)
// Blocks of 32 weights: fp16 d, [fp16 m], [qh: the 32 fifth bits, little endian], qs[16]; weight j is the low nibble of qs[j],
// weight j + 16 the high nibble (+ 16 * bit of qh).  w = q d + m (Q4_1, Q5_1) or (q - 16) d (Q5_0).
// A unit is a PAIR of blocks (64 weights; 40 / 44 / 48 bytes, 4-byte aligned) with four accumulator groups: (block, nibble half).
// Low nibbles decode as 1024 + q, high nibbles stay in place as 64 + q; the fifth bit lands on mantissa bit 4 / bit 8.  The unit's
// contribution is d_j (S_lo + S_hi) + off_j X_j per block with S = sum q x, X = sum x and off = m or -16 d; X comes out of the bias
// corrections the lane already holds (c_lo = -1024 X_lo, c_hi = -64 X_hi).
// Q5_0 blocks are 22 bytes: block 0's qs starts at byte 6 of the unit, so its first quant dword is assembled from the halves around
// it and holds bytes (0, 1, 14, 15) of qs; the activations are staged in the matching order (as for the Q4_0 block pair).
typedef u32x2 u32x2_a4 __attribute__((aligned(4)));
__device__ __forceinline__ u32x2 ld8_a4(const uint8_t* p) { return *(const TGA_GLOBAL u32x2_a4*)p; }
template <int KIND> struct FmtL {     // KIND 0: Q4_1, 1: Q5_0, 2: Q5_1
  static constexpr bool FIVE = KIND != 0;
  static constexpr int UW = 64, UPB = 1, BW = 64, BB = KIND == 0 ? 40 : KIND == 1 ? 44 : 48, ND = BB / 4;
  static __device__ __forceinline__ int unit_of(int e) { return e >> 6; }
  static __device__ __forceinline__ int pair_of(int e) { return (e & 63) >> 1; }
  static constexpr int XV = 8, NG = 4, NWV = 36;
  struct Raw { u32x4 a, b; uint32_t t[ND - 8]; };
  static __device__ __forceinline__ Raw load(const uint8_t* row, int u) {
    const uint8_t* p = row + BB * u; Raw r; r.a = ld16_a4(p); r.b = ld16_a4(p + 16);
    if constexpr (KIND == 2) { const u32x4 v = ld16_a4(p + 32); r.t[0] = v.x; r.t[1] = v.y; r.t[2] = v.z; r.t[3] = v.w; }
    else { const u32x2 v = ld8_a4(p + 32); r.t[0] = v.x; r.t[1] = v.y; if constexpr (KIND == 1) r.t[2] = ld4_a4(p + 40); }
    return r;
  }
  static __device__ __forceinline__ int xoff(int u, int k) { return 64 * u + 2 * k; }
  static constexpr int NKC = 2;
  static __device__ __forceinline__ void consts(uint32_t* kc) { kc[0] = vgpr_const(0x64006400u); kc[1] = vgpr_const(0x54005400u); }
  // block 0 of a Q5_0 pair: quant dword i holds bytes (b0, b0 + 1, b2, b2 + 1) with (b0, b2) / 2 = (0, 7), (1, 2), (3, 4), (5, 6)
  static __device__ __forceinline__ constexpr bool odd_block(int j) { return KIND == 1 && j == 0; }
  // wv[8 (2j + hi) + 2i + o]: block j, nibble half hi, quant dword i, o = odd bytes of the dword
  static __device__ __forceinline__ void decode(const Raw& r, uint32_t* wv, const uint32_t* kc) {
    const uint32_t D[12] = {r.a.x, r.a.y, r.a.z, r.a.w, r.b.x, r.b.y, r.b.z, r.b.w, r.t[0], r.t[1], ND > 10 ? r.t[ND > 10 ? 2 : 0] : 0u, ND > 11 ? r.t[ND > 11 ? 3 : 0] : 0u};
    uint32_t Q[2][4], qh[2] = {0u, 0u}, hdr[2];
    if constexpr (KIND == 0) { hdr[0] = D[0]; hdr[1] = D[5]; for (int i = 0; i < 4; i++) { Q[0][i] = D[1 + i]; Q[1][i] = D[6 + i]; } }
    else if constexpr (KIND == 2) { hdr[0] = D[0]; hdr[1] = D[6]; qh[0] = D[1]; qh[1] = D[7]; for (int i = 0; i < 4; i++) { Q[0][i] = D[2 + i]; Q[1][i] = D[8 + i]; } }
    else {
      hdr[0] = D[0] & 0xFFFFu; hdr[1] = D[5] >> 16; qh[0] = __builtin_amdgcn_alignbit(D[1], D[0], 16); qh[1] = D[6];
      Q[0][0] = __builtin_amdgcn_alignbit(D[5], D[1], 16); Q[0][1] = D[2]; Q[0][2] = D[3]; Q[0][3] = D[4];
      for (int i = 0; i < 4; i++) Q[1][i] = D[7 + i];
    }
#pragma unroll
    for (int j = 0; j < 2; j++) {
#pragma unroll
      for (int i = 0; i < 4; i++) {
        const uint32_t w = Q[j][i], w8 = w >> 8;
        uint32_t le = and_or(w, 0x000F000Fu, kc[0]), lo = and_or(w8, 0x000F000Fu, kc[0]);
        uint32_t he = and_or(w, 0x00F000F0u, kc[1]), ho = and_or(w8, 0x00F000F0u, kc[1]);
        if constexpr (FIVE) {
          // fifth bits of the dword's four bytes: t for the low-nibble weights (elements b0..b3), u for the high-nibble ones (16 + b)
          uint32_t t, u;
          if (odd_block(j)) {
            if (i == 0) { t = (qh[j] & 3u) | ((qh[j] >> 12) & 0xCu); u = ((qh[j] >> 16) & 3u) | ((qh[j] >> 28) & 0xCu); }
            else { t = (qh[j] >> (4 * i - 2)) & 0xFu; u = (qh[j] >> (4 * i + 14)) & 0xFu; }
          } else { t = (qh[j] >> (4 * i)) & 0xFu; u = (qh[j] >> (4 * i + 16)) & 0xFu; }
          const uint32_t X = t | (t << 14), Y = u | (u << 14);   // bits 0, 1 and 16, 17: bytes 0, 1 and 2, 3
          le = and_or(X << 4, 0x00100010u, le); lo = and_or(X << 3, 0x00100010u, lo);
          he = and_or(Y << 8, 0x01000100u, he); ho = and_or(Y << 7, 0x01000100u, ho);
        }
        wv[16 * j + 2 * i] = le; wv[16 * j + 2 * i + 1] = lo; wv[16 * j + 8 + 2 * i] = he; wv[16 * j + 8 + 2 * i + 1] = ho;
      }
    }
    // scale slots: d0, d1, and off_j * (-1 / 64) with off = m (Q4_1, Q5_1) or -16 d (Q5_0)
#pragma unroll
    for (int j = 0; j < 2; j++) {
      const float d = h2f_bits(hdr[j] & 0xFFFFu);
      wv[32 + j] = __builtin_bit_cast(uint32_t, d);
      wv[34 + j] = __builtin_bit_cast(uint32_t, KIND == 1 ? d * 0.25f : h2f_bits(hdr[j] >> 16) * (-1.0f / 64.0f));
    }
  }
  // nx[k] = natural pair k of the unit's 64 activations
  static __device__ __forceinline__ void stage(const uint32_t* nx, u32x4* xv, float* c) {
    constexpr int P0[4] = {0, 1, 3, 5}, P2[4] = {7, 2, 4, 6};
#pragma unroll
    for (int g = 0; g < 4; g++) {
      const uint32_t* n = nx + 8 * g;
      const int j = g >> 1;
#pragma unroll
      for (int v = 0; v < 2; v++) {
        const int a0 = odd_block(j) ? P0[2 * v] : 4 * v, a2 = odd_block(j) ? P2[2 * v] : 4 * v + 1;
        const int b0 = odd_block(j) ? P0[2 * v + 1] : 4 * v + 2, b2 = odd_block(j) ? P2[2 * v + 1] : 4 * v + 3;
        xv[2 * g + v].x = pack_even(n[a0], n[a2]); xv[2 * g + v].y = pack_odd(n[a0], n[a2]);
        xv[2 * g + v].z = pack_even(n[b0], n[b2]); xv[2 * g + v].w = pack_odd(n[b0], n[b2]);
      }
      float s = 0.f;
#pragma unroll
      for (int k = 0; k < 8; k++) s = dot2(n[k], (g & 1) ? 0x54005400u : 0x64006400u, s);
      c[g] = -s;
    }
  }
  static __device__ __forceinline__ float finish(const Raw&, const uint32_t* wv, const float* a, const float* c) {
    return __builtin_bit_cast(float, wv[32]) * (a[0] + a[1]) + __builtin_bit_cast(float, wv[33]) * (a[2] + a[3])
         + __builtin_bit_cast(float, wv[34]) * (c[0] * 0.0625f + c[1]) + __builtin_bit_cast(float, wv[35]) * (c[2] * 0.0625f + c[3]);
  }
  // true weights q d + off as fp16, one rounding
  static __device__ __forceinline__ void to_f16(const Raw&, uint32_t* wv) {
#pragma unroll
    for (int j = 0; j < 2; j++) {
      const float s = __builtin_bit_cast(float, wv[32 + j]), off = __builtin_bit_cast(float, wv[34 + j]) * -64.0f;
      const float c_lo = off - 1024.f * s, c_hi = off - 64.f * s;
#pragma unroll
      for (int i = 0; i < 8; i++) { wv[16 * j + i] = h2_unbias_scale_f32(wv[16 * j + i], s, c_lo); wv[16 * j + 8 + i] = h2_unbias_scale_f32(wv[16 * j + 8 + i], s, c_hi); }
    }
  }
  static __device__ __forceinline__ int spos(int e, int nu) {
    const int u = e >> 6, w = e & 63, j = w >> 5, b = w & 31, hi = b >> 4, q = b & 15, g = 2 * j + hi;
    int i, p;
    if (odd_block(j)) {
      if (q < 2) { i = 0; p = q; } else if (q >= 14) { i = 0; p = q - 12; } else { i = 1 + ((q - 2) >> 2); p = (q - 2) & 3; }
    } else { i = q >> 2; p = q & 3; }
    return (((2 * g + (i >> 1)) * nu + u) * 4 + (i & 1) * 2 + (p & 1)) * 2 + (p >> 1);
  }
  static __device__ __forceinline__ void cfromx(const u32x4* xv, float* c) {
#pragma unroll
    for (int g = 0; g < 4; g++) {
      const uint32_t k = (g & 1) ? 0x54005400u : 0x64006400u;
      float t = 0.f;
#pragma unroll
      for (int i = 2 * g; i < 2 * g + 2; i++) { t = dot2(xv[i].x, k, t); t = dot2(xv[i].y, k, t); t = dot2(xv[i].z, k, t); t = dot2(xv[i].w, k, t); }
      c[g] = -t;
    }
  }
};
template <> struct Fmt<GGML_Q4_1> : FmtL<0> {};
template <> struct Fmt<GGML_Q5_0> : FmtL<1> {};
template <> struct Fmt<GGML_Q5_1> : FmtL<2> {};

#include "qfmt_cb.h"     // IQ3_XXS, IQ3_S, IQ2_S, Q1_0: codebooks and sign patterns in LDS

// unit_dot with the unit's activations already in registers (M = 1)
template <int T>
__device__ __forceinline__ void unit_dot_reg(const typename Fmt<T>::Raw& raw, const u32x4* xv, const float* cv, float& acc, const uint32_t* kc) {
  using F = Fmt<T>;
  uint32_t wv[F::NWV];
  F::decode(raw, wv, kc);
  constexpr int VPG = F::XV / F::NG;
  float g[F::NG];
#pragma unroll
  for (int j = 0; j < F::NG; j++) {
    float t = cv[j];
#pragma unroll
    for (int v = 0; v < VPG; v++) {
      const u32x4 x = xv[j * VPG + v];
      const int wi = 4 * (j * VPG + v);
      t = dot2(wv[wi + 0], x.x, t); t = dot2(wv[wi + 1], x.y, t); t = dot2(wv[wi + 2], x.z, t); t = dot2(wv[wi + 3], x.w, t);
    }
    g[j] = t;
  }
  acc += F::finish(raw, wv, g, cv);
}

// the same for MR activation rows: one decode, MR sets of dot products
template <int T, int MR>
__device__ __forceinline__ void unit_dot_reg_m(const typename Fmt<T>::Raw& raw, const u32x4 (*xv)[Fmt<T>::XV], const float (*cv)[Fmt<T>::NG], float* acc, const uint32_t* kc) {
  using F = Fmt<T>;
  uint32_t wv[F::NWV];
  F::decode(raw, wv, kc);
  constexpr int VPG = F::XV / F::NG;
#pragma unroll
  for (int m = 0; m < MR; m++) {
    float g[F::NG];
#pragma unroll
    for (int j = 0; j < F::NG; j++) {
      float t = cv[m][j];
#pragma unroll
      for (int v = 0; v < VPG; v++) {
        const u32x4 x = xv[m][j * VPG + v];
        const int wi = 4 * (j * VPG + v);
        t = dot2(wv[wi + 0], x.x, t); t = dot2(wv[wi + 1], x.y, t); t = dot2(wv[wi + 2], x.z, t); t = dot2(wv[wi + 3], x.w, t);
      }
      g[j] = t;
    }
    acc[m] += F::finish(raw, wv, g, cv[m]);
  }
}

// M = 1 stores.  EPI 0: plain, EPI 1: + residual, EPI 2: silu(gate) * up into output row `row` of segment 0.
template <int EPI>
__device__ __forceinline__ void store_one(const QArgs& a, int seg, long long row, float v, long long yofs = 0) {
  if constexpr (EPI == 1) v += a.resid[seg][yofs + row];
  if (a.y_f32) ((float*)a.y[seg])[yofs + row] = v;
  else ((_Float16*)a.y[seg])[yofs + row] = (_Float16)v;        // (the staged output order exists for the SwiGLU epilogue only: store_swiglu)
}
__device__ __forceinline__ void store_swiglu(const QArgs& a, long long row, float gate, float up, long long yofs = 0) {
  const float o = silu_f(gate) * up;
  if (a.y_f32) ((float*)a.y[0])[yofs + row] = o;
  else ((_Float16*)a.y[0])[yofs + (a.y_stage_fmt ? staged_pos(a.y_stage_fmt, (int)row, a.y_stage_nu) : row)] = (_Float16)o;
}


__device__ __forceinline__ int staged_pos(int fmt, int e, int nu) {
  switch (fmt) {
    case F_Q4_0P: return Fmt<F_Q4_0P>::spos(e, nu);
    case F_Q8_0P: return Fmt<F_Q8_0P>::spos(e, nu);
    case GGML_Q6_K: return Fmt<GGML_Q6_K>::spos(e, nu);
    case GGML_Q4_K: return Fmt<GGML_Q4_K>::spos(e, nu);
    case GGML_Q5_K: return Fmt<GGML_Q5_K>::spos(e, nu);
    case GGML_Q4_1: return Fmt<GGML_Q4_1>::spos(e, nu);
    case GGML_Q5_0: return Fmt<GGML_Q5_0>::spos(e, nu);
    case GGML_Q5_1: return Fmt<GGML_Q5_1>::spos(e, nu);
    case GGML_IQ4_XS: return Fmt<GGML_IQ4_XS>::spos(e, nu);
    case GGML_IQ3_XXS: case GGML_IQ3_S: case GGML_IQ2_S: case GGML_Q1_0: return FmtCbBase::spos(e, nu);
    case GGML_MXFP4: return Fmt<GGML_MXFP4>::spos(e, nu);
    case GGML_F16: return Fmt<GGML_F16>::spos(e, nu);
  }
  return e;
}

// Halfword index of element e of activation row m in the layout the 17 .. 128 row GEMM (qgemm64.hip) multiplies from, for a consumer of format fmt (units of 64
// values) and ncg column groups: per step of four units [vector][column group][unit][column] 16-byte pieces (the formats' staged vectors, Fmt::stage).  The staged
// position inside a superblock's four units does not depend on the row length, so it is taken for a row of four units (no division by the unit count).
__device__ __forceinline__ size_t rows_staged_pos(int fmt, int e, int m, int ncg) {
  int u, i, h;
  if (fmt == GGML_F16) { u = e >> 6; i = (e >> 3) & 7; h = e & 7; }                      // (fp16 weights: the vectors are the unit's values in order)
  else { const int full = staged_pos(fmt, e & 255, 4); h = full & 7; const int t = full >> 3; i = t >> 2; u = ((e >> 8) << 2) | (t & 3); }
  return ((size_t)(u >> 2) * (8 * ncg * 64) + (i * ncg + (m >> 4)) * 64 + (u & 3) * 16 + (m & 15)) * 8 + h;
}

// ------------------------------------------------------------------------------------------------ activation staging (M rows, LDS)
// LDS layout for units [u0, u0+cu): xs[(m*XV + t) * cu + (u-u0)] (u32x4), then cs[(m*NG + j) * cu + (u-u0)] (float)
// one staging item = one unit of one activation row: stage_fetch reads its K values (as fp16 pairs), stage_put writes its vectors to LDS
template <int T>
__device__ __forceinline__ void stage_fetch(const QArgs& a, int m, int u, uint32_t* nx) {
  using F = Fmt<T>;
  constexpr int NP = F::UW / 2;
  // four consecutive pairs (8 activations) of a unit are contiguous in every format: 16-byte (fp16) / 2 x 16-byte (fp32) loads
  if (a.x_f32) {
    const float* x = (const float*)a.x + (long long)m * a.K;
#pragma unroll
    for (int k = 0; k < NP; k += 4) {
      const f32x4 lo = *(const f32x4*)(x + F::xoff(u, k)), hi = *(const f32x4*)(x + F::xoff(u, k) + 4);
      nx[k] = f2h_bits(lo.x) | (f2h_bits(lo.y) << 16); nx[k + 1] = f2h_bits(lo.z) | (f2h_bits(lo.w) << 16);
      nx[k + 2] = f2h_bits(hi.x) | (f2h_bits(hi.y) << 16); nx[k + 3] = f2h_bits(hi.z) | (f2h_bits(hi.w) << 16);
    }
  } else {
    const uint16_t* x = (const uint16_t*)a.x + (long long)m * a.K;
#pragma unroll
    for (int k = 0; k < NP; k += 4) { const u32x4 v = *(const u32x4*)(x + F::xoff(u, k)); nx[k] = v.x; nx[k + 1] = v.y; nx[k + 2] = v.z; nx[k + 3] = v.w; }
  }
}
template <int T>
__device__ __forceinline__ void stage_put(const uint32_t* nx, u32x4* xs, float* cs, int m, int ul, int cu) {
  using F = Fmt<T>;
  u32x4 xv[F::XV]; float c[F::NG];
  F::stage(nx, xv, c);
#pragma unroll
  for (int t = 0; t < F::XV; t++) xs[(m * F::XV + t) * cu + ul] = xv[t];
#pragma unroll
  for (int j = 0; j < F::NG; j++) cs[(m * F::NG + j) * cu + ul] = c[j];
}
template <int T, int M, int NT = QG_THREADS>
__device__ __forceinline__ void stage_chunk(const QArgs& a, u32x4* xs, float* cs, int u0, int cu, int first = -1) {
  using F = Fmt<T>;
  for (int i = first < 0 ? (int)threadIdx.x : first; i < M * cu; i += NT) {
    const int m = i / cu, ul = i - m * cu;
    uint32_t nx[F::UW / 2];
    stage_fetch<T>(a, m, u0 + ul, nx);
    stage_put<T>(nx, xs, cs, m, ul, cu);
  }
}

