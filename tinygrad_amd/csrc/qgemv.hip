// Fused GGUF block dequant + GEMV / small-batch GEMM (1 <= M <= 8) for gfx950.
//
// Replaces the kernel(s) tinygrad schedules for  x.linear(W.T)  (tinygrad/nn/__init__.py:177, tinygrad/mixin/op.py:367-392)
// when W is the lazy ggml_data_to_tensor expression over raw GGUF bytes (tinygrad/llm/gguf.py:46,56,68-72,105-114).
//
// Design (bandwidth-bound, no MFMA):
//  * a "unit" is the slice of one weight row a lane owns per step: one 32-weight block (Q4_0 18 B, Q8_0 34 B, MXFP4 17 B) or a
//    quarter of a Q6_K superblock (64 weights).  Lane l of a wave takes unit l, l+64, ... of a row, so a wave's loads cover a
//    contiguous span of the row; each lane issues 128-bit loads straight from the packed GGUF bytes (no repacking).
//  * nibbles / bytes are turned into fp16 with biased-exponent tricks in registers (v_and_or_b32, v_perm_b32,
//    v_cvt_scalef32_pk_f16_fp4) and multiplied with v_dot2_f32_f16 (two fp16 products, float32 accumulate).  The integer offset
//    (-8, -32, +128 bias, plus the 1024/64 exponent bias) is removed with a per-unit correction  c = -bias * sum(x)  that is
//    computed once per workgroup when the activations are staged, and used as the accumulator's start value.
//  * activations (fp16, or fp32 rounded to fp16) are staged once per workgroup into LDS in the pair order the decode
//    produces, [vector t][unit] so that every ds_read_b128 is conflict-free.
//  * a wave owns whole rows: K is reduced inside the lane, then across the wave with DPP adds (no LDS, no atomics).
//  * when M*K activations do not fit LDS the kernel walks K in chunks with one row group per wave (accumulators stay in
//    registers across chunks).
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
};

__device__ __forceinline__ uint32_t pack_even(uint32_t a, uint32_t b) { return (a & 0xFFFFu) | (b << 16); }        // (a.lo, b.lo)
__device__ __forceinline__ uint32_t pack_odd(uint32_t a, uint32_t b) { return (a >> 16) | (b & 0xFFFF0000u); }     // (a.hi, b.hi)

template <int T> struct Fmt;

// ------------------------------------------------------------------------------------------------ Q4_0 (gguf.py:46)
template <> struct Fmt<GGML_Q4_0> {
  static constexpr int UW = 32, UPB = 1, BW = 32, BB = 18;   // weights per unit, units per block, block weights / bytes
  static constexpr int XV = 4, NG = 1, NWV = 16;
  struct Raw { u32x4 q; uint32_t d; };
  static __device__ __forceinline__ Raw load(const uint8_t* row, int u) {
    const uint8_t* p = row + 18 * u; Raw r; r.d = ld2(p); r.q = ld16(p + 2); return r;
  }
  // element index (within the row) of natural pair k (elements 2k, 2k+1) of unit u
  static __device__ __forceinline__ int xoff(int u, int k) { return 32 * u + 2 * k; }
  // wv[4t+c] multiplies x pair xs[t][c].  low nibble -> 1024+n (0x6400), high nibble in place -> 64+n (0x5400)
  static __device__ __forceinline__ void decode(const Raw& r, uint32_t* wv) {
#pragma unroll
    for (int t = 0; t < 4; t++) {
      const uint32_t w = r.q[t], w8 = w >> 8;
      wv[4 * t + 0] = and_or(w, 0x000F000Fu, 0x64006400u);    // weights 4t, 4t+2
      wv[4 * t + 1] = and_or(w, 0x00F000F0u, 0x54005400u);    // weights 4t+16, 4t+18
      wv[4 * t + 2] = and_or(w8, 0x000F000Fu, 0x64006400u);   // weights 4t+1, 4t+3
      wv[4 * t + 3] = and_or(w8, 0x00F000F0u, 0x54005400u);   // weights 4t+17, 4t+19
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
  static __device__ __forceinline__ float finish(const Raw& r, const float* a) { return h2f_bits(r.d) * a[0]; }
};

// ------------------------------------------------------------------------------------------------ Q8_0 (gguf.py:56)
template <> struct Fmt<GGML_Q8_0> {
  static constexpr int UW = 32, UPB = 1, BW = 32, BB = 34;
  static constexpr int XV = 4, NG = 1, NWV = 16;
  struct Raw { u32x4 q0, q1; uint32_t d; };
  static __device__ __forceinline__ Raw load(const uint8_t* row, int u) {
    const uint8_t* p = row + 34 * u; Raw r; r.d = ld2(p); r.q0 = ld16(p + 2); r.q1 = ld16(p + 18); return r;
  }
  static __device__ __forceinline__ int xoff(int u, int k) { return 32 * u + 2 * k; }
  // int8 q -> byte q^0x80 = q+128 placed under exponent byte 0x64: fp16 value 1024 + 128 + q
  static __device__ __forceinline__ void decode(const Raw& r, uint32_t* wv) {
#pragma unroll
    for (int t = 0; t < 8; t++) {
      const uint32_t u = (t < 4 ? r.q0[t] : r.q1[t - 4]) ^ 0x80808080u;
      wv[2 * t + 0] = __builtin_amdgcn_perm(0x64646464u, u, 0x04010400u);   // bytes (u0,0x64,u1,0x64): weights 4t, 4t+1
      wv[2 * t + 1] = __builtin_amdgcn_perm(0x64646464u, u, 0x04030402u);   // weights 4t+2, 4t+3
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
  static __device__ __forceinline__ float finish(const Raw& r, const float* a) { return h2f_bits(r.d) * a[0]; }
};

// ------------------------------------------------------------------------------------------------ MXFP4 (gguf.py:105-114)
template <> struct Fmt<GGML_MXFP4> {
  static constexpr int UW = 32, UPB = 1, BW = 32, BB = 17;
  static constexpr int XV = 4, NG = 1, NWV = 16;
  struct Raw { u32x4 q; uint32_t e; };
  static __device__ __forceinline__ Raw load(const uint8_t* row, int u) {
    const uint8_t* p = row + 17 * u; Raw r; r.e = p[0]; r.q = ld16(p + 1); return r;
  }
  static __device__ __forceinline__ int xoff(int u, int k) { return 32 * u + 2 * k; }
  // hardware E2M1 -> fp16 (true values 0..6); byte s of dword t holds weights 4t+s (low nibble) and 4t+s+16 (high nibble)
  static __device__ __forceinline__ void decode(const Raw& r, uint32_t* wv) {
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
  static __device__ __forceinline__ float finish(const Raw& r, const float* a) {
    return __builtin_bit_cast(float, r.e ? (r.e << 23) : 0x00400000u) * a[0];
  }
};

// ------------------------------------------------------------------------------------------------ Q6_K (gguf.py:68-72)
// unit u of a row: superblock u>>2, half h=(u>>1)&1, sixteen-run g=u&1.  Its 64 weights are, for j = 0..3 and i = 0..15,
// element 256*sb + 128*h + 32*j + 16*g + i, decoded from ql[64h+16g+i] (j even) / ql[64h+32+16g+i] (j odd), low nibble for
// j < 2 and high nibble for j >= 2, and bits 2j..2j+1 of qh[32h+16g+i]; all sixteen share scale sc[8h + 2j + g].
template <> struct Fmt<GGML_Q6_K> {
  static constexpr int UW = 64, UPB = 4, BW = 256, BB = 210;
  static constexpr int XV = 8, NG = 4, NWV = 32;
  struct Raw { u32x4 a, b, h; uint32_t sc0, sc1, d; };
  static __device__ __forceinline__ Raw load(const uint8_t* row, int u) {
    const uint8_t* p = row + 210 * (u >> 2); const int h = (u >> 1) & 1, g = u & 1;
    Raw r; r.a = ld16(p + 64 * h + 16 * g); r.b = ld16(p + 64 * h + 32 + 16 * g); r.h = ld16(p + 128 + 32 * h + 16 * g);
    r.sc0 = ld4(p + 192 + 8 * h); r.sc1 = ld4(p + 196 + 8 * h); r.d = (uint32_t)g | (ld2(p + 208) << 16);
    return r;
  }
  static __device__ __forceinline__ int xoff(int u, int k) {   // k = 0..31: natural pair k of the unit's 64 x values (j = k/8)
    return 256 * (u >> 2) + 128 * ((u >> 1) & 1) + 32 * (k >> 3) + 16 * (u & 1) + 2 * (k & 7);
  }
  // wv[8j + 2t + {0,1}] = even / odd pairs of dword t of group j; value 1024 + 6-bit q
  static __device__ __forceinline__ void decode(const Raw& r, uint32_t* wv) {
#pragma unroll
    for (int t = 0; t < 4; t++) {
      const uint32_t A = r.a[t], B = r.b[t], H = r.h[t];
      wv[0 + 2 * t]      = and_or(H << 4, 0x00300030u, and_or(A, 0x000F000Fu, 0x64006400u));
      wv[0 + 2 * t + 1]  = and_or(H >> 4, 0x00300030u, and_or(A >> 8, 0x000F000Fu, 0x64006400u));
      wv[8 + 2 * t]      = and_or(H << 2, 0x00300030u, and_or(B, 0x000F000Fu, 0x64006400u));
      wv[8 + 2 * t + 1]  = and_or(H >> 6, 0x00300030u, and_or(B >> 8, 0x000F000Fu, 0x64006400u));
      wv[16 + 2 * t]     = and_or(H, 0x00300030u, and_or(A >> 4, 0x000F000Fu, 0x64006400u));
      wv[16 + 2 * t + 1] = and_or(H >> 8, 0x00300030u, and_or(A >> 12, 0x000F000Fu, 0x64006400u));
      wv[24 + 2 * t]     = and_or(H >> 2, 0x00300030u, and_or(B >> 4, 0x000F000Fu, 0x64006400u));
      wv[24 + 2 * t + 1] = and_or(H >> 10, 0x00300030u, and_or(B >> 12, 0x000F000Fu, 0x64006400u));
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
  static __device__ __forceinline__ float finish(const Raw& r, const float* a) {
    const int g8 = (r.d & 1) * 8;   // scales 8h + 2j + g live in bytes g, g+2 of sc0 (j = 0, 1) and sc1 (j = 2, 3)
    const float s0 = (float)(int)(int8_t)(r.sc0 >> g8), s1 = (float)(int)(int8_t)(r.sc0 >> (16 + g8));
    const float s2 = (float)(int)(int8_t)(r.sc1 >> g8), s3 = (float)(int)(int8_t)(r.sc1 >> (16 + g8));
    return h2f_bits(r.d >> 16) * (s0 * a[0] + s1 * a[1] + s2 * a[2] + s3 * a[3]);
  }
};

// ------------------------------------------------------------------------------------------------ kernel
// LDS layout for units [u0, u0+cu): xs[(m*XV + t) * cu + (u-u0)] (u32x4), then cs[(m*NG + j) * cu + (u-u0)] (float)
template <int T, int M>
__device__ __forceinline__ void stage_chunk(const QArgs& a, u32x4* xs, float* cs, int u0, int cu) {
  using F = Fmt<T>;
  constexpr int NP = F::UW / 2;
  for (int i = threadIdx.x; i < M * cu; i += QG_THREADS) {
    const int m = i / cu, ul = i - m * cu, u = u0 + ul;
    uint32_t nx[NP];
    if (a.x_f32) {
      const float* x = (const float*)a.x + (long long)m * a.K;
#pragma unroll
      for (int k = 0; k < NP; k++) { const float2 v = *(const float2*)(x + F::xoff(u, k)); nx[k] = f2h_bits(v.x) | (f2h_bits(v.y) << 16); }
    } else {
      const uint16_t* x = (const uint16_t*)a.x + (long long)m * a.K;
#pragma unroll
      for (int k = 0; k < NP; k++) nx[k] = *(const uint32_t*)(x + F::xoff(u, k));
    }
    u32x4 xv[F::XV]; float c[F::NG];
    F::stage(nx, xv, c);
#pragma unroll
    for (int t = 0; t < F::XV; t++) xs[(m * F::XV + t) * cu + ul] = xv[t];
#pragma unroll
    for (int j = 0; j < F::NG; j++) cs[(m * F::NG + j) * cu + ul] = c[j];
  }
}

template <int T, int M>
__device__ __forceinline__ void unit_dot(const typename Fmt<T>::Raw& raw, const u32x4* xs, const float* cs, int cu, int ul, float* acc) {
  using F = Fmt<T>;
  uint32_t wv[F::NWV];
  F::decode(raw, wv);
  constexpr int VPG = F::XV / F::NG;   // x vectors per accumulator group
#pragma unroll
  for (int m = 0; m < M; m++) {
    float g[F::NG];
#pragma unroll
    for (int j = 0; j < F::NG; j++) {
      float s = cs[(m * F::NG + j) * cu + ul];
#pragma unroll
      for (int v = 0; v < VPG; v++) {
        const u32x4 xv = xs[(m * F::XV + j * VPG + v) * cu + ul];
        const int wi = 4 * (j * VPG + v);
        s = dot2(wv[wi + 0], xv.x, s); s = dot2(wv[wi + 1], xv.y, s); s = dot2(wv[wi + 2], xv.z, s); s = dot2(wv[wi + 3], xv.w, s);
      }
      g[j] = s;
    }
    acc[m] += F::finish(raw, g);
  }
}

__device__ __forceinline__ float silu_f(float v) { return v / (1.0f + __expf(-v)); }

// row r (0..R-1) of row group rg -> segment and local row.  epilogue 2 pairs gate row rg with up row rg.
template <int R>
__device__ __forceinline__ void map_row(const QArgs& a, long long rg, int r, int& seg, long long& lr, bool& valid) {
  if (a.epilogue == 2) { seg = r; lr = rg; valid = true; return; }
  long long row = rg * R + r;
  valid = row < a.ntot;
  if (!valid) row = a.ntot - 1;
  seg = 0;
  if (a.nseg > 1 && row >= a.n[0]) { row -= a.n[0]; seg = 1; if (a.nseg > 2 && row >= a.n[1]) { row -= a.n[1]; seg = 2; } }
  lr = row;
}

template <int T, int M, int R>
__device__ __forceinline__ void store_rows(const QArgs& a, long long rg, float (&acc)[R][M]) {
  const int lane = threadIdx.x & 63;
#pragma unroll
  for (int r = 0; r < R; r++)
#pragma unroll
    for (int m = 0; m < M; m++) acc[r][m] = wave_sum_lane63(acc[r][m]);
  if (lane != 63) return;
  if (a.epilogue == 2) {
    if constexpr (R == 2) {
#pragma unroll
      for (int m = 0; m < M; m++) {
        const float v = silu_f(acc[0][m]) * acc[1][m];
        if (a.y_f32) ((float*)a.y[0])[(long long)m * a.n[0] + rg] = v; else ((_Float16*)a.y[0])[(long long)m * a.n[0] + rg] = (_Float16)v;
      }
    }
    return;
  }
#pragma unroll
  for (int r = 0; r < R; r++) {
    int seg; long long lr; bool valid;
    map_row<R>(a, rg, r, seg, lr, valid);
    if (!valid) continue;
#pragma unroll
    for (int m = 0; m < M; m++) {
      const long long o = (long long)m * a.n[seg] + lr;
      float v = acc[r][m];
      if (a.epilogue == 1) v += a.resid[seg][o];
      if (a.y_f32) ((float*)a.y[seg])[o] = v; else ((_Float16*)a.y[seg])[o] = (_Float16)v;
    }
  }
}

template <int T, int M, int R>
__global__ __launch_bounds__(QG_THREADS) void qgemv_kernel(const QArgs a) {
  using F = Fmt<T>;
  extern __shared__ u32x4 lds[];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const long long gw = (long long)blockIdx.x * QG_WAVES + wave, nw = (long long)gridDim.x * QG_WAVES;
  const long long ngroups = (a.epilogue == 2) ? a.ntot : (a.ntot + R - 1) / R;

  if (a.nchunks == 1) {
    const int cu = a.nu;
    u32x4* xs = lds; float* cs = (float*)(lds + M * F::XV * cu);
    stage_chunk<T, M>(a, xs, cs, 0, cu);
    __syncthreads();
    for (long long rg = gw; rg < ngroups; rg += nw) {
      const uint8_t* rp[R];
#pragma unroll
      for (int r = 0; r < R; r++) { int seg; long long lr; bool valid; map_row<R>(a, rg, r, seg, lr, valid); rp[r] = a.w[seg] + lr * a.row_bytes; }
      float acc[R][M];
#pragma unroll
      for (int r = 0; r < R; r++)
#pragma unroll
        for (int m = 0; m < M; m++) acc[r][m] = 0.f;
      for (int u = lane; u < cu; u += 64) {
        typename F::Raw raw[R];
#pragma unroll
        for (int r = 0; r < R; r++) raw[r] = F::load(rp[r], u);
#pragma unroll
        for (int r = 0; r < R; r++) unit_dot<T, M>(raw[r], xs, cs, cu, u, acc[r]);
      }
      store_rows<T, M, R>(a, rg, acc);
    }
  } else {
    // K walked in LDS-sized chunks; one row group per wave (the host sizes the grid so that gw covers every group)
    const long long rg = gw;
    const bool active = rg < ngroups;
    const uint8_t* rp[R];
#pragma unroll
    for (int r = 0; r < R; r++) { int seg; long long lr; bool valid; map_row<R>(a, active ? rg : 0, r, seg, lr, valid); rp[r] = a.w[seg] + lr * a.row_bytes; }
    float acc[R][M];
#pragma unroll
    for (int r = 0; r < R; r++)
#pragma unroll
      for (int m = 0; m < M; m++) acc[r][m] = 0.f;
    for (int ch = 0; ch < a.nchunks; ch++) {
      const int u0 = ch * a.chunk_u, cu = min(a.chunk_u, a.nu - u0);
      u32x4* xs = lds; float* cs = (float*)(lds + M * F::XV * cu);
      __syncthreads();
      stage_chunk<T, M>(a, xs, cs, u0, cu);
      __syncthreads();
      if (active) {
        for (int ul = lane; ul < cu; ul += 64) {
          typename F::Raw raw[R];
#pragma unroll
          for (int r = 0; r < R; r++) raw[r] = F::load(rp[r], u0 + ul);
#pragma unroll
          for (int r = 0; r < R; r++) unit_dot<T, M>(raw[r], xs, cs, cu, ul, acc[r]);
        }
      }
    }
    if (active) store_rows<T, M, R>(a, rg, acc);
  }
}

// ------------------------------------------------------------------------------------------------ host side
static int g_cu_count = 0;
static int cu_count() {
  if (!g_cu_count) { int dev = 0; hipDeviceProp_t p; if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&p, dev) == hipSuccess) g_cu_count = p.multiProcessorCount; else g_cu_count = 256; }
  return g_cu_count;
}

#define QG_LDS_BUDGET (144 * 1024)

template <int T, int M, int R>
static int launch_qgemv(QArgs a, hipStream_t s) {
  using F = Fmt<T>;
  const int per_unit = M * (16 * F::XV + 4 * F::NG);
  a.nu = a.K / F::UW;
  a.row_bytes = (long long)(a.K / F::BW) * F::BB;
  const long long ngroups = (a.epilogue == 2) ? a.ntot : (a.ntot + R - 1) / R;
  long long grid; size_t lds;
  if ((long long)per_unit * a.nu <= QG_LDS_BUDGET) {
    a.nchunks = 1; a.chunk_u = a.nu;
    lds = (size_t)per_unit * a.nu;
    // resident workgroups per CU by LDS (160 KB), capped at 4 (16 waves); never more workgroups than row groups need
    int per_cu = (int)((160 * 1024) / (lds + 256)); if (per_cu > 4) per_cu = 4; if (per_cu < 1) per_cu = 1;
    grid = (long long)cu_count() * per_cu;
    const long long need = (ngroups + QG_WAVES - 1) / QG_WAVES;
    if (grid > need) grid = need;
  } else {
    int cu = QG_LDS_BUDGET / 2 / per_unit;                 // two workgroups per CU
    cu -= cu % (64 * F::UPB); if (cu < 64 * F::UPB) cu = 64 * F::UPB;
    TGA_REQUIRE((long long)cu * per_unit <= QG_LDS_BUDGET, "tga_qlinear: activations of one K chunk do not fit LDS");
    a.chunk_u = cu; a.nchunks = (a.nu + cu - 1) / cu;
    lds = (size_t)per_unit * cu;
    grid = (ngroups + QG_WAVES - 1) / QG_WAVES;
  }
  if (grid < 1) grid = 1;
  auto kern = qgemv_kernel<T, M, R>;
  if (lds > 48 * 1024) {
    static size_t configured = 0;   // per instantiation
    if (lds > configured) { TGA_HIP(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, QG_LDS_BUDGET)); configured = QG_LDS_BUDGET; }
  }
  kern<<<dim3((unsigned)grid), dim3(QG_THREADS), lds, s>>>(a);
  TGA_LAUNCH_CHECK();
  return 0;
}

template <int T, int M>
static int launch_qgemv_r(const QArgs& a, hipStream_t s) {
  // SwiGLU pairs gate/up rows: exactly two rows per group.  Otherwise two rows per wave step as well (more loads in flight
  // per lane); a single row per group when there are too few rows to fill the chip.
  if (a.epilogue == 2) return launch_qgemv<T, M, 2>(a, s);
  if (a.ntot < (long long)cu_count() * QG_WAVES * 2) return launch_qgemv<T, M, 1>(a, s);
  return launch_qgemv<T, M, 2>(a, s);
}

template <int T>
static int launch_qgemv_m(const QArgs& a, int M, hipStream_t s) {
  switch (M) {
    case 1: return launch_qgemv_r<T, 1>(a, s);
    case 2: return launch_qgemv_r<T, 2>(a, s);
    case 3: return launch_qgemv_r<T, 3>(a, s);
    case 4: return launch_qgemv_r<T, 4>(a, s);
    case 5: return launch_qgemv_r<T, 5>(a, s);
    case 6: return launch_qgemv_r<T, 6>(a, s);
    case 7: return launch_qgemv_r<T, 7>(a, s);
    case 8: return launch_qgemv_r<T, 8>(a, s);
  }
  return tga_set_error("tga_qlinear: M=%d out of range 1..8", M);
}

extern "C" int tga_qlinear_multi(int ggml_type, int nseg, const void* const* w, void* const* y, const int64_t* n,
                                 const void* x, int x_dtype, int y_dtype, int M, int64_t K,
                                 int epilogue, const void* const* resid, void* stream) {
  TGA_REQUIRE(nseg >= 1 && nseg <= QG_MAX_SEG, "tga_qlinear_multi: nseg=%d out of range 1..%d", nseg, QG_MAX_SEG);
  TGA_REQUIRE(M >= 1 && M <= 8, "tga_qlinear: M=%d out of range 1..8", M);
  TGA_REQUIRE(x_dtype == TGA_F16 || x_dtype == TGA_F32, "tga_qlinear: x_dtype must be TGA_F16 or TGA_F32");
  TGA_REQUIRE(y_dtype == TGA_F16 || y_dtype == TGA_F32, "tga_qlinear: y_dtype must be TGA_F16 or TGA_F32");
  TGA_REQUIRE(epilogue >= 0 && epilogue <= 2, "tga_qlinear: epilogue=%d unknown", epilogue);
  TGA_REQUIRE(epilogue != 1 || (y_dtype == TGA_F32 && resid), "tga_qlinear: the residual epilogue needs float32 y and resid pointers");
  TGA_REQUIRE(epilogue != 2 || (nseg == 2 && n[0] == n[1]), "tga_qlinear: the SwiGLU epilogue needs two segments of equal rows");
  int bw;
  switch (ggml_type) { case GGML_Q4_0: case GGML_Q8_0: case GGML_MXFP4: bw = 32; break; case GGML_Q6_K: bw = 256; break;
    default: return tga_set_error("GGML type '%d' is not supported!", ggml_type); }
  TGA_REQUIRE(K > 0 && K % bw == 0 && K <= (1 << 24), "tga_qlinear: K=%lld must be a positive multiple of %d", (long long)K, bw);
  TGA_REQUIRE(x, "tga_qlinear: null x");
  QArgs a = {};
  a.nseg = nseg; a.x = x; a.x_f32 = x_dtype == TGA_F32; a.y_f32 = y_dtype == TGA_F32; a.epilogue = epilogue; a.K = (int)K;
  long long ntot = 0;
  for (int i = 0; i < nseg; i++) {
    TGA_REQUIRE(n[i] > 0 && w[i] && (y[i] || (epilogue == 2 && i == 1)), "tga_qlinear: segment %d has a null pointer or no rows", i);
    TGA_REQUIRE(ggml_type == GGML_MXFP4 || ((uintptr_t)w[i] & 1) == 0, "tga_qlinear: weight pointer of segment %d must be 2-byte aligned", i);
    a.w[i] = (const uint8_t*)w[i]; a.y[i] = y[i]; a.n[i] = n[i]; a.resid[i] = epilogue == 1 ? (const float*)resid[i] : nullptr;
    TGA_REQUIRE(epilogue != 1 || a.resid[i], "tga_qlinear: null resid for segment %d", i);
    ntot += n[i];
  }
  a.ntot = (epilogue == 2) ? n[0] : ntot;
  hipStream_t s = (hipStream_t)stream;
  switch (ggml_type) {
    case GGML_Q4_0: return launch_qgemv_m<GGML_Q4_0>(a, M, s);
    case GGML_Q8_0: return launch_qgemv_m<GGML_Q8_0>(a, M, s);
    case GGML_Q6_K: return launch_qgemv_m<GGML_Q6_K>(a, M, s);
    case GGML_MXFP4: return launch_qgemv_m<GGML_MXFP4>(a, M, s);
  }
  return 1;
}

extern "C" int tga_qlinear(int ggml_type, const void* w, const void* x, int x_dtype, void* y, int y_dtype,
                           int M, int64_t N, int64_t K, void* stream) {
  const void* ws[1] = {w}; void* ys[1] = {y}; int64_t ns[1] = {N};
  return tga_qlinear_multi(ggml_type, 1, ws, ys, ns, x, x_dtype, y_dtype, M, K, 0, nullptr, stream);
}
