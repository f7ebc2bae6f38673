// Decode-step neighbours of the quantized linears (batch 1): embedding row dequant, RMSNorm, RoPE + KV append + GQA attention
// (flash-decoding over 64-position splits), split combine, argmax / token bookkeeping.
// They restate, for one token, what tinygrad/llm/model.py:167-204 (_attention), :144-151 (block), :358-364 (forward) compute.
// The position and token live in device memory so that one captured launch sequence can be replayed for every token
// (the reference binds symbolic start_pos into a replayed JIT graph: tinygrad/llm/model.py:464-484).
#include <type_traits>
#include <stdlib.h>
#include <string.h>
#include "qfmt.h"
#include "decode.h"
#include "coherent.h"
#include "deq.h"

// ---------------------------------------------------------------------------------------------- embedding (one row of any table type)
// token_embd(tokens).float() for one token: tinygrad/llm/model.py:359.  The table stays in GGUF blocks; only the row is dequantized
// (bit-exact block decode shared with tga_dequant, then rounded to fp16: the reference casts the table to fp16 like every weight, model.py:376).
template <int T>
__device__ __forceinline__ void embed_row_blocks(const uint8_t* __restrict__ table, int dim, int tok, float* __restrict__ out) {
  const uint8_t* row = table + (size_t)tok * (dim / Deq<T>::NEL) * Deq<T>::NBY;
  for (int e = threadIdx.x * 4; e < dim; e += 1024) {
    float o[4];
    Deq<T>::get4(row + (size_t)(e / Deq<T>::NEL) * Deq<T>::NBY, e % Deq<T>::NEL, o);
    out[e] = (float)(_Float16)o[0]; out[e + 1] = (float)(_Float16)o[1]; out[e + 2] = (float)(_Float16)o[2]; out[e + 3] = (float)(_Float16)o[3];
  }
}
__global__ __launch_bounds__(256) void embed_row_kernel(const uint8_t* __restrict__ table, int ggml_type, int dim, DecodeState* st, float* __restrict__ out,
                                                        const int* __restrict__ tokens) {
  int tok = tokens ? tokens[blockIdx.x] : st->token;     // batched decode: one workgroup per sequence, its token from the list
  out += (size_t)blockIdx.x * dim;
  if (tok < 0 || (st->vocab > 0 && tok >= st->vocab)) {         // a token id outside the table (e.g. argmax over NaN logits): row 0 is read instead, the host sees the flag
    if (threadIdx.x == 0) atomicOr(&st->error, 1);
    tok = 0;
  }
  switch (ggml_type) {
    case GGML_Q4_0: embed_row_blocks<GGML_Q4_0>(table, dim, tok, out); break;
    case GGML_Q8_0: embed_row_blocks<GGML_Q8_0>(table, dim, tok, out); break;
    case GGML_Q4_K: embed_row_blocks<GGML_Q4_K>(table, dim, tok, out); break;
    case GGML_Q5_K: embed_row_blocks<GGML_Q5_K>(table, dim, tok, out); break;
    case GGML_Q4_1: embed_row_blocks<GGML_Q4_1>(table, dim, tok, out); break;
    case GGML_Q5_0: embed_row_blocks<GGML_Q5_0>(table, dim, tok, out); break;
    case GGML_Q5_1: embed_row_blocks<GGML_Q5_1>(table, dim, tok, out); break;
    case GGML_Q6_K: embed_row_blocks<GGML_Q6_K>(table, dim, tok, out); break;
    case GGML_IQ4_XS: embed_row_blocks<GGML_IQ4_XS>(table, dim, tok, out); break;
    case GGML_IQ3_XXS: embed_row_blocks<GGML_IQ3_XXS>(table, dim, tok, out); break;
    case GGML_IQ3_S: embed_row_blocks<GGML_IQ3_S>(table, dim, tok, out); break;
    case GGML_IQ2_S: embed_row_blocks<GGML_IQ2_S>(table, dim, tok, out); break;
    case GGML_Q1_0: embed_row_blocks<GGML_Q1_0>(table, dim, tok, out); break;
    case GGML_MXFP4: embed_row_blocks<GGML_MXFP4>(table, dim, tok, out); break;
    case GGML_F16: { const uint16_t* row = (const uint16_t*)table + (size_t)tok * dim; for (int e = threadIdx.x; e < dim; e += 256) out[e] = h2f_bits(row[e]); break; }
    default: { const float* row = (const float*)table + (size_t)tok * dim; for (int e = threadIdx.x; e < dim; e += 256) out[e] = (float)(_Float16)row[e]; }
  }
}

// ---------------------------------------------------------------------------------------------- RMSNorm
// nn.RMSNorm (tinygrad/nn/__init__.py:296-304): x * rsqrt(mean(x^2) + eps), then * weight.  Output fp16 (the activation the
// dequant-GEMV multiplies) and optionally fp32.
// COMB: the row is first completed in place as x + sum_j probs[row, j] * y[row, j, :] (the weighted sum over the selected experts' outputs plus the block
// residual, tinygrad/llm/model.py:130, 150) - the same expression, in the same order, as moe_combine_kernel - and the norm is taken of the completed row.
template <bool COMB>
__global__ __launch_bounds__(1024) void rmsnorm_kernel(const float* x, const float* __restrict__ w, int dim, float eps,
                                                       _Float16* __restrict__ out16, float* __restrict__ out32, int stage_fmt, int stage_nu,
                                                       float* x_rw, const float* __restrict__ y, const float* __restrict__ probs, int k) {
  __shared__ float red[16];
  const int row = blockIdx.x;                           // one workgroup per row
  x += (size_t)row * dim;
  if (out16) out16 += (size_t)row * dim;
  if (out32) out32 += (size_t)row * dim;
  auto value = [&](int e) {                             // element e of the (completed) row; COMB: also written back (read again below only by the thread that wrote it)
    float a = x[e];
    if constexpr (COMB) {
      for (int j0 = 0; j0 < k; j0 += 8) {               // eight experts' values requested together, added in order
        float yy[8], pp[8];
#pragma unroll
        for (int i = 0; i < 8; i++) { const int j = j0 + i < k ? j0 + i : k - 1; pp[i] = probs[(size_t)row * k + j]; yy[i] = y[((size_t)row * k + j) * dim + e]; }
#pragma unroll
        for (int i = 0; i < 8; i++) if (j0 + i < k) a += pp[i] * yy[i];
      }
      x_rw[(size_t)row * dim + e] = a;
    }
    return a;
  };
  // two elements per thread and loop pass are requested together and kept for the second pass (rows up to 2048 values never reload)
  float s = 0.f, v0 = 0.f, v1 = 0.f, w0 = 0.f, w1 = 0.f;
  const int e0 = threadIdx.x, e1 = threadIdx.x + 1024;
  if (e0 < dim) { v0 = value(e0); w0 = w[e0]; }
  if (e1 < dim) { v1 = value(e1); w1 = w[e1]; }
  s = v0 * v0 + v1 * v1;
  for (int b = threadIdx.x + 2048; b < dim; b += 4096) {
    float t[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
      if constexpr (COMB) t[j] = b + 1024 * j < dim ? value(b + 1024 * j) : 0.f;      // (an element is completed exactly once)
      else t[j] = value(b + 1024 * j < dim ? b + 1024 * j : dim - 1);
    }
#pragma unroll
    for (int j = 0; j < 4; j++) if (b + 1024 * j < dim) s += t[j] * t[j];
  }
  s = wave_sum(s);
  const int wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  if ((threadIdx.x & 63) == 0) red[wave] = s;
  __syncthreads();
  float tot = 0.f;
  for (int i = 0; i < nw; i++) tot += red[i];
  const float scale = 1.0f / sqrtf(tot / (float)dim + eps);
  auto emit = [&](int e, float v) {
    if (out16) out16[stage_fmt ? staged_pos(stage_fmt, e, stage_nu) : e] = (_Float16)v;
    if (out32) out32[e] = v;
  };
  if (e0 < dim) emit(e0, (v0 * scale) * w0);
  if (e1 < dim) emit(e1, (v1 * scale) * w1);
  for (int b = threadIdx.x + 2048; b < dim; b += 4096) {
    float t[4], u[4];
#pragma unroll
    for (int j = 0; j < 4; j++) { const int e = b + 1024 * j < dim ? b + 1024 * j : dim - 1; t[j] = x[e]; u[j] = w[e]; }
#pragma unroll
    for (int j = 0; j < 4; j++) if (b + 1024 * j < dim) emit(b + 1024 * j, (t[j] * scale) * u[j]);
  }
}

// ---------------------------------------------------------------------------------------------- RoPE + KV append + attention
// One workgroup per (kv head, 64-position split).  q, k are rotated with the half-split rule of apply_rope
// (tinygrad/llm/model.py:29-33) using the caller's freqs_cis table [max_ctx][hd] = cos half | sin half (precompute_freqs_cis,
// model.py:16-19); the split that contains `pos` writes the rotated k and v into the fp16 cache.  With q_norm / k_norm the
// full-width RMSNorm of model.py:169 (attn_q_norm / attn_k_norm over all heads at once) is applied to q and k first.
// Softmax partials per split (max, sum, weighted V) go to `part`; attn_merge_kernel, the next launch, merges them per query head.
struct AttnArgs {
  const float* q; const float* k; const float* v;     // this token's projections: [n_heads*hd], [n_kv*hd], [n_kv*hd]
  _Float16* cache_k; _Float16* cache_v;                // [n_kv][max_ctx][hd]
  float* part;                                         // [n_heads][nsplit][hd + 2]
  DecodeState* st;
  int n_heads, n_kv, hd, max_ctx, nsplit;
  const float* rope;                                   // [max_ctx][hd]: cos(pos * f_i) for i < hd/2, then sin(pos * f_i)
  float scale;
  _Float16* out16; float* out32;                       // attention output [n_heads*hd]
  int stage_fmt, stage_nu;                             // != 0: out16 in the staged order of the consuming linear
  int stage_rows_ncg;                                  // != 0 (rows of a prefill step): out16 is ONE buffer for all rows, in the layout the 17 .. 128 row GEMM multiplies from (rows_staged_pos)
  const float* q_norm; const float* k_norm; float norm_eps;   // optional RMSNorm weights: over the whole q / k vectors, or
  int norm_per_head;                                           // per head (weights of head_dim values shared by all heads)
  // batched decode (sequences in lockstep at one position): sequence z = blockIdx.z (split launch) / blockIdx.y (merge launch) uses the
  // operands shifted by z times these element strides; all zero for a single sequence
  long long q_bs, kv_bs, cache_bs, part_bs, out_bs;
  // chunked prefill (rows z = 0, 1, ... are consecutive positions of ONE sequence: cache_bs = 0, row z sits at position st->pos + z pos_step):
  // chunk 1 = the launch that only rotates and appends every row's key / value, chunk 2 = the launch that attends from the cache alone
  // (the rows of the chunk were appended by the launch before; a row sees the positions up to its own).  0: decode.
  int chunk, pos_step;
  int split_shift;                                     // log2 of the positions per split partial that the merge launch sums (6: splits of 64; the matrix-core chunk launch may cover several tiles per partial)
};
__device__ __forceinline__ AttnArgs attn_args_of_sequence(AttnArgs a, int z) {
  a.q += z * a.q_bs; a.k += z * a.kv_bs; a.v += z * a.kv_bs; a.cache_k += z * a.cache_bs; a.cache_v += z * a.cache_bs; a.part += z * a.part_bs;
  if (a.out16) a.out16 += z * a.out_bs;
  if (a.out32) a.out32 += z * a.out_bs;
  return a;
}

// One rotated pair of apply_rope (tinygrad/llm/model.py:29-33): (x1 c - x2 s, x2 c + x1 s).  Written as one rounded product and one fused multiply-add, so
// that every kernel that rotates (the two attention kernels, decode and prefill) produces the same bits whatever the compiler would contract on its own.
__device__ __forceinline__ float rope_lo(float x1, float x2, float c, float s) { return __builtin_fmaf(x1, c, -(x2 * s)); }
__device__ __forceinline__ float rope_hi(float x1, float x2, float c, float s) { return __builtin_fmaf(x2, c, x1 * s); }

__device__ __forceinline__ u32x4 pack8_f16(const float* c) {
  u32x4 r = {f2h_bits(c[0]) | (f2h_bits(c[1]) << 16), f2h_bits(c[2]) | (f2h_bits(c[3]) << 16),
             f2h_bits(c[4]) | (f2h_bits(c[5]) << 16), f2h_bits(c[6]) | (f2h_bits(c[7]) << 16)};
  return r;
}
// sum over the HD8 (8, 16 or 32) consecutive lanes that hold one row; every lane of the run gets the sum
template <int HD8>
__device__ __forceinline__ float run_sum(float v) {
  v = dpp_add<0xB1>(v); v = dpp_add<0x4E>(v); v = dpp_add<0x141>(v);
  if constexpr (HD8 >= 16) v = dpp_add<0x140>(v);
  if constexpr (HD8 == 32) v += __shfl_xor(v, 16, 64);
  return v;
}
// sums of squares of two float vectors (lengths % 4 == 0, 16-byte aligned) over the whole workgroup of 256 threads; red: 8 floats
// of LDS.  The loads of four loop iterations of both vectors go out as one batch.
__device__ __forceinline__ void block_sumsq2(const float* q, int nq, const float* k, int nk, float* red, float& sq, float& sk) {
  float s0 = 0.f, s1 = 0.f;
  const int n4q = nq >> 2, n4k = nk >> 2, nmax = n4q > n4k ? n4q : n4k;
  for (int b = threadIdx.x; b < nmax; b += 1024) {
    f32x4 vq[4], vk[4];
#pragma unroll
    for (int t = 0; t < 4; t++) { const int i = b + 256 * t; vq[t] = ((const f32x4*)q)[i < n4q ? i : n4q - 1]; vk[t] = ((const f32x4*)k)[i < n4k ? i : n4k - 1]; }
#pragma unroll
    for (int t = 0; t < 4; t++) {
      const int i = b + 256 * t;
      if (i < n4q) s0 += vq[t].x * vq[t].x + vq[t].y * vq[t].y + vq[t].z * vq[t].z + vq[t].w * vq[t].w;
      if (i < n4k) s1 += vk[t].x * vk[t].x + vk[t].y * vk[t].y + vk[t].z * vk[t].z + vk[t].w * vk[t].w;
    }
  }
  s0 = wave_sum(s0); s1 = wave_sum(s1);
  if ((threadIdx.x & 63) == 0) { red[threadIdx.x >> 6] = s0; red[4 + (threadIdx.x >> 6)] = s1; }
  __syncthreads();
  sq = red[0] + red[1] + red[2] + red[3]; sk = red[4] + red[5] + red[6] + red[7];
}

// HD8 = head_dim / 8 (16-byte pieces per row).  The four waves split the 64 positions (16 each) and every wave serves all
// query heads of the group.  A wave's K and V tiles are 16 rows in one shared register layout: load instruction i covers rows
// i*RPI + lane / HD8 (RPI = 64 / HD8) and lane % HD8 picks the 16-byte piece, so a lane only needs the 8 query values of its
// piece.  Scores: 8 FMAs per instruction, then a DPP sum over the HD8 lanes of a row.  Each run of HD8 lanes keeps its own
// softmax partial (its rows only); the partials meet in LDS and leave as one partial per (head, split) with plain stores: the
// merge over splits is a launch of its own (attn_merge_kernel).
//
// The kernel is a chain of latencies, not of bytes, so its loads are arranged as ONE round trip: everything that does not depend
// on the position (this token's q / k / v rows and norm weights, then the cached K / V tiles with rows clamped to the cache, not to
// the position) is requested first, in straight-line code and small loads first (loads return in issue order); the position is a
// scalar load in flight meanwhile, and only the rotation row waits for it.  NORM selects the q/k RMSNorm at compile time so that no
// load sits behind a branch (a join makes the compiler wait for every outstanding load):
//   0 none, 1 over the whole q and k vectors of at most 4096 values each (read in one batch), 2 per head, 3 over whole vectors of any length
template <int HD8, int NORM>
__global__ __launch_bounds__(256) void attn_decode_kernel(const AttnArgs args) {
  const AttnArgs a = attn_args_of_sequence(args, blockIdx.z);   // field reads become kernel-argument loads in the entry block
  const int zrow = blockIdx.z * a.pos_step;
  constexpr int HD = HD8 * 8, RPI = 64 / HD8, NVI = 16 / RPI, NGRP = 4 * RPI, CSTR = HD + 4;
  constexpr int QPL = (HD / 2 + 63) / 64;               // query pairs per lane
  const int kvh = blockIdx.x, split = blockIdx.y;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int half = HD >> 1, group = a.n_heads / a.n_kv;
  __shared__ float qs[4][HD];                           // rotated queries of the 4 heads in flight
  __shared__ float ks[HD], vs[HD];                      // rotated key / value of this token
  __shared__ float comb[4 * NGRP * CSTR];               // [head in flight][run]: o[HD], m, l
  __shared__ float red[8];
  const int vr = lane / HD8, vp = lane % HD8;
  const int p0 = split * 64 + wave * 16;                // first position of this wave
  // ---- loads that do not depend on the position
  const int ki = tid < half ? tid : half - 1;           // thread t rotates pair t of the key and copies element t of the value (head_dim <= 256)
  const int vi = tid < HD ? tid : HD - 1;
  const float kx1 = a.k[kvh * HD + ki], kx2 = a.k[kvh * HD + half + ki];
  const float vx = a.v[kvh * HD + vi];
  const int head0 = kvh * group + (wave < group ? wave : 0);   // the head whose query this wave rotates in the first pass
  float qx1[QPL], qx2[QPL];
#pragma unroll
  for (int j = 0; j < QPL; j++) {
    const int i = lane + 64 * j < half ? lane + 64 * j : half - 1;
    qx1[j] = a.q[head0 * HD + i]; qx2[j] = a.q[head0 * HD + half + i];
  }
  float kw1 = 1.f, kw2 = 1.f, qw1[QPL], qw2[QPL];
  if constexpr (NORM != 0) {                            // weight index = position in the whole vector, or inside the head for the per-head norm
    const int kb = NORM == 2 ? 0 : kvh * HD, qb = NORM == 2 ? 0 : head0 * HD;
    kw1 = a.k_norm[kb + ki]; kw2 = a.k_norm[kb + half + ki];
#pragma unroll
    for (int j = 0; j < QPL; j++) {
      const int i = lane + 64 * j < half ? lane + 64 * j : half - 1;
      qw1[j] = a.q_norm[qb + i]; qw2[j] = a.q_norm[qb + half + i];
    }
  }
  f32x4 nq4[4], nk4[4];
  if constexpr (NORM == 1) {                            // the whole q and k vectors for the sums of squares: four 16-byte pieces per thread each
    const int n4q = (a.n_heads * HD) >> 2, n4k = (a.n_kv * HD) >> 2;
#pragma unroll
    for (int t = 0; t < 4; t++) {
      const int i = tid + 256 * t;
      nq4[t] = ((const f32x4*)a.q)[i < n4q ? i : n4q - 1]; nk4[t] = ((const f32x4*)a.k)[i < n4k ? i : n4k - 1];
    }
  }
  u32x4 kt[NVI], vt[NVI];
  {
    const _Float16* kbase = a.cache_k + (size_t)kvh * a.max_ctx * HD + vp * 8;
    const _Float16* vbase = a.cache_v + (size_t)kvh * a.max_ctx * HD + vp * 8;
#pragma unroll
    for (int i = 0; i < NVI; i++) {
      const int r = p0 + i * RPI + vr, rc = r < a.max_ctx ? r : a.max_ctx - 1;   // rows from the position on are replaced or masked below
      kt[i] = *(const u32x4*)(kbase + (size_t)rc * HD);
      vt[i] = *(const u32x4*)(vbase + (size_t)rc * HD);
    }
  }
  // ---- the position, and the one load that needs it
  const int pos = a.st->pos + zrow;
  if (pos >= a.max_ctx || pos < 0) {                    // no cache row and no rotation row for this position: nothing is read or written, the host sees the flag
    if (kvh == 0 && split == 0 && tid == 0) atomicOr(&a.st->error, 2);
    return;
  }
  if (split * 64 > pos) return;                         // nothing cached in this split yet
  const float kc = a.rope[(size_t)pos * HD + ki], ksn = a.rope[(size_t)pos * HD + half + ki];
  float qc[QPL], qsn[QPL];
#pragma unroll
  for (int j = 0; j < QPL; j++) {
    const int i = lane + 64 * j < half ? lane + 64 * j : half - 1;
    qc[j] = a.rope[(size_t)pos * HD + i]; qsn[j] = a.rope[(size_t)pos * HD + half + i];
  }
  // ---- norms
  float qscale = 1.f, kscale = 1.f;
  if constexpr (NORM == 1) {
    const int n4q = (a.n_heads * HD) >> 2, n4k = (a.n_kv * HD) >> 2;
    float s0 = 0.f, s1 = 0.f;
#pragma unroll
    for (int t = 0; t < 4; t++) {
      const int i = tid + 256 * t;
      const f32x4 x = nq4[t], y = nk4[t];
      s0 += i < n4q ? x.x * x.x + x.y * x.y + x.z * x.z + x.w * x.w : 0.f;
      s1 += i < n4k ? y.x * y.x + y.y * y.y + y.z * y.z + y.w * y.w : 0.f;
    }
    s0 = wave_sum(s0); s1 = wave_sum(s1);
    if (lane == 0) { red[wave] = s0; red[4 + wave] = s1; }
    __syncthreads();
    qscale = 1.0f / sqrtf((red[0] + red[1] + red[2] + red[3]) / (float)(a.n_heads * HD) + a.norm_eps);
    kscale = 1.0f / sqrtf((red[4] + red[5] + red[6] + red[7]) / (float)(a.n_kv * HD) + a.norm_eps);
  } else if constexpr (NORM == 3) {
    float sq, sk;
    block_sumsq2(a.q, a.n_heads * HD, a.k, a.n_kv * HD, red, sq, sk);
    qscale = 1.0f / sqrtf(sq / (float)(a.n_heads * HD) + a.norm_eps);
    kscale = 1.0f / sqrtf(sk / (float)(a.n_kv * HD) + a.norm_eps);
  } else if constexpr (NORM == 2) {                     // the key of this kv head over the workgroup, the wave's query inside the wave
    float sk = tid < half ? kx1 * kx1 + kx2 * kx2 : 0.f, sq = 0.f;
#pragma unroll
    for (int j = 0; j < QPL; j++) sq += lane + 64 * j < half ? qx1[j] * qx1[j] + qx2[j] * qx2[j] : 0.f;
    sk = wave_sum(sk); sq = wave_sum(sq);
    if (lane == 0) red[wave] = sk;
    __syncthreads();
    kscale = 1.0f / sqrtf((red[0] + red[1] + red[2] + red[3]) / (float)HD + a.norm_eps);
    qscale = 1.0f / sqrtf(sq / (float)HD + a.norm_eps);
  }
  // normalised values for the later head passes (weights re-read there)
  auto qval = [&](int i) { return NORM != 0 ? (a.q[i] * qscale) * a.q_norm[NORM == 2 ? i % HD : i] : a.q[i]; };
  if (tid < half) {
    const float x1 = NORM != 0 ? (kx1 * kscale) * kw1 : kx1, x2 = NORM != 0 ? (kx2 * kscale) * kw2 : kx2;
    ks[tid] = rope_lo(x1, x2, kc, ksn); ks[half + tid] = rope_hi(x1, x2, kc, ksn);
  }
  if (tid < HD) vs[tid] = vx;
  if (wave < group) {                                   // first pass: wave w rotates the query of head w
#pragma unroll
    for (int j = 0; j < QPL; j++) {
      const int i = lane + 64 * j;
      const float x1 = NORM != 0 ? (qx1[j] * qscale) * qw1[j] : qx1[j], x2 = NORM != 0 ? (qx2[j] * qscale) * qw2[j] : qx2[j];
      if (i < half) { qs[wave][i] = rope_lo(x1, x2, qc[j], qsn[j]); qs[wave][half + i] = rope_hi(x1, x2, qc[j], qsn[j]); }
    }
  }
  __syncthreads();
  if (a.chunk == 1 || (a.chunk == 0 && (pos >> 6) == split)) {   // owner split appends this token to the cache (chunked prefill: the append launch, one workgroup per row and kv head)
    for (int i = tid; i < HD; i += 256) {
      a.cache_k[((size_t)kvh * a.max_ctx + pos) * HD + i] = (_Float16)ks[i];
      a.cache_v[((size_t)kvh * a.max_ctx + pos) * HD + i] = (_Float16)vs[i];
    }
  }
  if (a.chunk == 1) return;
  if (a.chunk == 0) {                                   // (chunked prefill reads this row's key / value, like those of the rows before it, from the cache)
    const u32x4 kcur = pack8_f16(ks + vp * 8), vcur = pack8_f16(vs + vp * 8);   // rounded to fp16 exactly like the cached copy
#pragma unroll
    for (int i = 0; i < NVI; i++) if (p0 + i * RPI + vr >= pos) { kt[i] = kcur; vt[i] = vcur; }
  }
  for (int h0 = 0; h0 < group; h0 += 4) {
    if (h0 > 0) {                                       // later passes (more than four query heads per kv head): rotate the next four
      if (h0 + wave < group) {
        const int head = kvh * group + h0 + wave;
        if constexpr (NORM == 2) {
          float sq = 0.f;
          for (int i = lane; i < HD; i += 64) { const float v = a.q[head * HD + i]; sq += v * v; }
          qscale = 1.0f / sqrtf(wave_sum(sq) / (float)HD + a.norm_eps);
        }
        for (int i = lane; i < half; i += 64) {
          const float c = a.rope[(size_t)pos * HD + i], sn = a.rope[(size_t)pos * HD + half + i];
          const float x1 = qval(head * HD + i), x2 = qval(head * HD + half + i);
          qs[wave][i] = rope_lo(x1, x2, c, sn); qs[wave][half + i] = rope_hi(x1, x2, c, sn);
        }
      }
      __syncthreads();
    }
#pragma unroll
    for (int hh = 0; hh < 4; hh++) {
      if (h0 + hh < group) {
        float qq[8];
#pragma unroll
        for (int j = 0; j < 8; j++) qq[j] = qs[hh][vp * 8 + j];
        float sc[NVI];
        float m = -INFINITY;
#pragma unroll
        for (int i = 0; i < NVI; i++) {
          const u32x4 kk = kt[i];
          const half2_t k0 = as_h2(kk.x), k1 = as_h2(kk.y), k2 = as_h2(kk.z), k3 = as_h2(kk.w);
          float t = qq[0] * (float)k0.x; t += qq[1] * (float)k0.y; t += qq[2] * (float)k1.x; t += qq[3] * (float)k1.y;
          t += qq[4] * (float)k2.x; t += qq[5] * (float)k2.y; t += qq[6] * (float)k3.x; t += qq[7] * (float)k3.y;
          t = run_sum<HD8>(t);
          sc[i] = (p0 + i * RPI + vr <= pos) ? t * a.scale : -INFINITY;
          m = fmaxf(m, sc[i]);
        }
        // softmax partial of this lane run (rows i * RPI + vr of the wave): no cross-lane traffic, the fold below sums the runs
        float l = 0.f;
        f32x4 o0 = {0.f, 0.f, 0.f, 0.f}, o1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int i = 0; i < NVI; i++) {
          const float pj = (p0 + i * RPI + vr <= pos) ? __expf(sc[i] - m) : 0.f;
          l += pj;
          const u32x4 vv = vt[i];
          const half2_t v0 = as_h2(vv.x), v1 = as_h2(vv.y), v2 = as_h2(vv.z), v3 = as_h2(vv.w);
          o0.x += pj * (float)v0.x; o0.y += pj * (float)v0.y; o0.z += pj * (float)v1.x; o0.w += pj * (float)v1.y;
          o1.x += pj * (float)v2.x; o1.y += pj * (float)v2.y; o1.z += pj * (float)v3.x; o1.w += pj * (float)v3.y;
        }
        float* cw = comb + (size_t)(hh * NGRP + wave * RPI + vr) * CSTR;
        *(f32x4*)(cw + vp * 8) = o0; *(f32x4*)(cw + vp * 8 + 4) = o1;
        if (vp == 0) { cw[HD] = m; cw[HD + 1] = l; }
      }
    }
    __syncthreads();
    if (h0 + wave < group) {                            // wave w folds the row-run partials of head h0 + w into the split partial
      const int head = kvh * group + h0 + wave;
      const float* cb = comb + (size_t)wave * NGRP * CSTR;
      float m = -INFINITY;                              // the first run of wave 0 always holds a valid position: m is finite
#pragma unroll
      for (int g = 0; g < NGRP; g++) m = fmaxf(m, cb[g * CSTR + HD]);
      float l = 0.f, od[HD / 64];
#pragma unroll
      for (int j = 0; j < HD / 64; j++) od[j] = 0.f;
#pragma unroll
      for (int g = 0; g < NGRP; g++) {
        const float mg = cb[g * CSTR + HD];
        const float wg = mg == -INFINITY ? 0.f : __expf(mg - m);   // a run without valid rows contributes nothing
        l += wg * cb[g * CSTR + HD + 1];
#pragma unroll
        for (int j = 0; j < HD / 64; j++) od[j] += wg * cb[g * CSTR + lane + 64 * j];
      }
      float* po = a.part + ((size_t)head * a.nsplit + split) * (HD + 2);
#pragma unroll
      for (int j = 0; j < HD / 64; j++) po[lane + 64 * j] = od[j];
      if (lane == 0) { po[HD] = m; po[HD + 1] = l; }
    }
    __syncthreads();
  }
}

// Chunked prefill, the attending launch on the matrix cores (chunk rows z = 0, 1, ... are consecutive positions of one sequence; the launch before has rotated
// and appended every row's key / value).  Workgroup = (kv head, split of 64 TS cached positions walked in tiles of 64, tile of 16 chunk rows): the per-row workgroups of
// attn_decode_kernel read every 32 KB K / V tile once per row and query-head group - 64 rows x 8 kv heads x 16 splits = 268 MB of L2 reads per layer at a
// context of 1024 - here a tile is read once per sixteen rows.  Wave w serves query head w of the group (w + 4, ... for larger groups):
//   S^T = K Q^T   v_mfma_f32_16x16x32_f16, A = lane (g, r): 8 values 32 j + 8 g .. of cached key 16 t + r (16-byte loads straight from the cache), B = lane (g, c):
//                 the same 8 values of chunk row c's rotated query as TWO fp16 operands (the rounded value and what the rounding left over, so the scores see the
//                 float32 query: rounding it alone put the result at 1.0e-3 of the float32 attention on random rows); D = lane (g, c): keys 16 t + 4 g + i of row c
//   softmax partial of the split per chunk row: the 16 scores of a lane, then the four lanes of a row (m, l: float32; a row sees the positions up to its own)
//   O^T = V^T P^T A = lane (g, r): V of 8 keys for dimension 16 h + r, B = lane (g, c): exp(s - m) of the SAME 8 keys for row c, rounded to fp16 - the eight
//                 keys a lane holds after the first product (tiles 2 u and 2 u + 1, rows 4 g + i) are taken as they are, and the V tile is written to LDS
//                 transposed with its keys in that order, so that the A operand is one 16-byte LDS read
// The partial (float32 weighted V sums, max, sum) goes where attn_decode_kernel writes it; attn_merge_kernel finishes.  Deviation from the float32 products of
// the per-row kernel: the probabilities are rounded to fp16 (2^-11 relative, fp32 accumulation).
// TS consecutive 64-key tiles per workgroup (one split partial of 64 TS positions): the rotated queries are formed once and the softmax partial runs over
// the tiles with a running maximum (the sums and the weighted V sums are rescaled when it grows), so TS times fewer partials are written here and read by the merge
// launch, and the queries are read and rotated TS times less often.  HPW: query heads per wave (the group has at most 4 HPW heads).
template <int HD8, int TS, int HPW>
__global__ __launch_bounds__(256) void attn_chunk_mfma_kernel(const AttnArgs a, const int rows) {
  typedef _Float16 v8f16 __attribute__((ext_vector_type(8)));
  typedef float v4f32 __attribute__((ext_vector_type(4)));
  constexpr int HD = HD8 * 8, NJ = HD / 32, NH = HD / 16, half = HD / 2;
  constexpr int VP = 64 + 8;                            // halfwords per transposed V row (64 keys + 16 bytes: rows 16 bytes apart in the banks)
  __shared__ __attribute__((aligned(16))) uint16_t vts[HD * VP];
  const int kvh = blockIdx.x, split = blockIdx.y, rz = blockIdx.z;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, g = lane >> 4, c = lane & 15;
  const int group = a.n_heads / a.n_kv;
  const int row = 16 * rz + c < rows ? 16 * rz + c : rows - 1;             // this lane's chunk row (a tile that the chunk ends in repeats the last row, stored by nobody)
  const bool row_ok = 16 * rz + c < rows;
  // ---- loads that do not depend on the position: the V tile (lane = key, pieces 4 wave .. 4 wave + 3 of HD8) and the K operands of the first tile
  u32x4 vv[HD8 / 4];
  u32x4 kt[4][NJ];
  auto load_tile = [&](int key0) __attribute__((always_inline)) {
    {
      const int kr = key0 + lane < a.max_ctx ? key0 + lane : a.max_ctx - 1;
      const _Float16* vb = a.cache_v + ((size_t)kvh * a.max_ctx + kr) * HD;
#pragma unroll
      for (int i = 0; i < HD8 / 4; i++) vv[i] = *(const u32x4*)(vb + 8 * ((HD8 / 4) * wave + i));
    }
#pragma unroll
    for (int t = 0; t < 4; t++) {
      const int kr = key0 + 16 * t + c < a.max_ctx ? key0 + 16 * t + c : a.max_ctx - 1;   // (rows beyond the cache are masked below: they lie beyond every position)
      const _Float16* kb = a.cache_k + ((size_t)kvh * a.max_ctx + kr) * HD + 8 * g;
#pragma unroll
      for (int j = 0; j < NJ; j++) kt[t][j] = *(const u32x4*)(kb + 32 * j);
    }
  };
  const int key_first = split * 64 * TS;
  load_tile(key_first);
  const int pos0 = a.st->pos;
  const int last = pos0 + (16 * rz + 15 < rows ? 16 * rz + 15 : rows - 1);   // the last position of this row tile
  if (pos0 < 0 || last >= a.max_ctx) return;             // (refused by the appending launch: state.error)
  if (key_first > last) return;                          // nothing of this split is visible to the tile
  const int pos = pos0 + row;
  // ---- the rotated queries of this wave's heads (row, head): the lane's values 32 j + 8 g + e; the partner of a low value is the value half further, in the same
  // lane (j + NJ / 2); as TWO fp16 operands, the rounded value and what the rounding left over, so that the scores see the float32 queries
  u32x4 qb[HPW][NJ], qr[HPW][NJ];
  auto form_queries = [&]() __attribute__((always_inline)) {
#pragma unroll
  for (int hw = 0; hw < HPW; hw++) {
    const int hh = wave + 4 * hw < group ? wave + 4 * hw : group - 1;
    const int head = kvh * group + hh;
    const float* qrow = a.q + (size_t)row * a.q_bs + (size_t)head * HD;
    const float* rr = a.rope + (size_t)pos * HD;
#pragma unroll
    for (int j = 0; j < NJ / 2; j++) {
      float lo[8], hi[8];
#pragma unroll
      for (int e4 = 0; e4 < 8; e4 += 4) {
        const int i = 32 * j + 8 * g + e4;
        const f32x4 x1 = *(const f32x4*)(qrow + i), x2 = *(const f32x4*)(qrow + half + i), cs = *(const f32x4*)(rr + i), sn = *(const f32x4*)(rr + half + i);
        lo[e4] = rope_lo(x1.x, x2.x, cs.x, sn.x); lo[e4 + 1] = rope_lo(x1.y, x2.y, cs.y, sn.y); lo[e4 + 2] = rope_lo(x1.z, x2.z, cs.z, sn.z); lo[e4 + 3] = rope_lo(x1.w, x2.w, cs.w, sn.w);
        hi[e4] = rope_hi(x1.x, x2.x, cs.x, sn.x); hi[e4 + 1] = rope_hi(x1.y, x2.y, cs.y, sn.y); hi[e4 + 2] = rope_hi(x1.z, x2.z, cs.z, sn.z); hi[e4 + 3] = rope_hi(x1.w, x2.w, cs.w, sn.w);
      }
      qb[hw][j] = pack8_f16(lo); qb[hw][j + NJ / 2] = pack8_f16(hi);
      float lr[8], hr[8];
#pragma unroll
      for (int e = 0; e < 8; e++) { lr[e] = lo[e] - (float)(_Float16)lo[e]; hr[e] = hi[e] - (float)(_Float16)hi[e]; }
      qr[hw][j] = pack8_f16(lr); qr[hw][j + NJ / 2] = pack8_f16(hr);
    }
  }
  };
  float M[HPW], L[HPW];
  v4f32 O[HPW][NH];
#pragma unroll
  for (int hw = 0; hw < HPW; hw++) {
    M[hw] = -INFINITY; L[hw] = 0.f;
#pragma unroll
    for (int h = 0; h < NH; h++) O[hw][h] = v4f32{0.f, 0.f, 0.f, 0.f};
  }
#pragma unroll
  for (int tt = 0; tt < TS; tt++) {
    const int key0 = key_first + 64 * tt;
    if (key0 > last) break;                              // (the same for the whole workgroup)
    const bool final = tt + 1 == TS || key0 + 64 > last;  // the last tile of this split that the row tile sees: its weighted sums go straight to the partial
    if (tt > 0) { __syncthreads(); load_tile(key0); }    // every wave is done with the V tile in LDS before it is replaced
    // ---- the V tile transposed: key j of the tile goes to slot 32 (j / 32) + 8 ((j % 16) / 4) + 4 ((j % 32) / 16) + j % 4 of every dimension's row
    {
      const int j = lane, slot = (j & 32) + 8 * ((j & 15) >> 2) + 4 * ((j >> 4) & 1) + (j & 3);
#pragma unroll
      for (int i = 0; i < HD8 / 4; i++) {
        const int d0 = 8 * ((HD8 / 4) * wave + i);
        const uint32_t w[4] = {vv[i].x, vv[i].y, vv[i].z, vv[i].w};
#pragma unroll
        for (int e = 0; e < 8; e++) vts[(d0 + e) * VP + slot] = (uint16_t)(w[e >> 1] >> (16 * (e & 1)));
      }
    }
    __syncthreads();
    if (tt == 0) form_queries();                        // (behind the first tile's V transposition: the query and rotation rows arrive while it runs)
#pragma unroll
    for (int hw = 0; hw < HPW; hw++) {
      if (wave + 4 * hw >= group) break;
      // scores of the 64 keys x 16 rows
      v4f32 sc[4];
#pragma unroll
      for (int t = 0; t < 4; t++) {
        sc[t] = v4f32{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < NJ; j++) {
          sc[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8f16, kt[t][j]), __builtin_bit_cast(v8f16, qr[hw][j]), sc[t], 0, 0, 0);
          sc[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8f16, kt[t][j]), __builtin_bit_cast(v8f16, qb[hw][j]), sc[t], 0, 0, 0);
        }
      }
      float m = -INFINITY;
#pragma unroll
      for (int t = 0; t < 4; t++) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
          const float sv = key0 + 16 * t + 4 * g + i <= pos ? sc[t][i] * a.scale : -INFINITY;
          sc[t][i] = sv; m = fmaxf(m, sv);
        }
      }
      m = fmaxf(m, __shfl_xor(m, 16, 64)); m = fmaxf(m, __shfl_xor(m, 32, 64));
      const float mn = fmaxf(M[hw], m);                  // the running maximum of the row (still -inf: the row lies before everything seen so far)
      const bool seen = mn != -INFINITY;
      const float alpha = M[hw] != -INFINITY ? __expf(M[hw] - mn) : 0.f;
      float l = 0.f;
      float pr[4][4];
#pragma unroll
      for (int t = 0; t < 4; t++) {
#pragma unroll
        for (int i = 0; i < 4; i++) { const float pj = seen ? __expf(sc[t][i] - mn) : 0.f; pr[t][i] = pj; l += pj; }
      }
      l += __shfl_xor(l, 16, 64); l += __shfl_xor(l, 32, 64);
      L[hw] = L[hw] * alpha + l; M[hw] = mn;
      u32x4 pb[2];
#pragma unroll
      for (int u = 0; u < 2; u++) {
        const float e8[8] = {pr[2 * u][0], pr[2 * u][1], pr[2 * u][2], pr[2 * u][3], pr[2 * u + 1][0], pr[2 * u + 1][1], pr[2 * u + 1][2], pr[2 * u + 1][3]};
        pb[u] = pack8_f16(e8);
      }
      // weighted V sums: dimension tile h, lane (g, c) ends with dimensions 16 h + 4 g + i of row c
      float* po = a.part + (size_t)row * a.part_bs + ((size_t)(kvh * group + wave + 4 * hw) * a.nsplit + split) * (HD + 2);
#pragma unroll
      for (int h = 0; h < NH; h++) {
        v4f32 o = tt == 0 ? v4f32{0.f, 0.f, 0.f, 0.f} : O[hw][h] * alpha;   // (the first tile starts the sums: nothing to rescale)
#pragma unroll
        for (int u = 0; u < 2; u++) {
          const u32x4 va = *(const u32x4*)(vts + (16 * h + c) * VP + 32 * u + 8 * g);
          o = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8f16, va), __builtin_bit_cast(v8f16, pb[u]), o, 0, 0, 0);
        }
        if (final) { if (row_ok && seen) { float* pd = po + 16 * h + 4 * g; pd[0] = o[0]; pd[1] = o[1]; pd[2] = o[2]; pd[3] = o[3]; } }   // (the stores leave while the next products run)
        else O[hw][h] = o;
      }
      if (final && row_ok && seen && g == 0) { po[HD] = M[hw]; po[HD + 1] = L[hw]; }
    }
    if (final) break;
  }
}

// The attention of one token as ONE launch whose consumer merges (tga_attn_merge_qlinear): workgroup = (query head, split of SP = 16 NW IT positions), NW waves
// of 16 rows per tile, IT tiles per wave, every cached row of the split requested up front (rows clamped to the cache, not to the position), at most six splits.
// The flattened workgroup index is kv head + n_kv (head in group + group * split): with n_kv a multiple of 8 all readers of a kv head's rows run on one XCD.
// A split that starts beyond the position writes an empty partial (max -inf, sum 0).  Partials per head: [n_splits][head_dim] weighted V sums, then the
// (max, sum) pairs of the splits in 16 floats.
// NORM: q and k pass through an RMSNorm before the rotation (nn.RMSNorm, tinygrad/nn/__init__.py:296-304): 1 = over the whole q / k rows with weights of that
// length (model.py:169), 2 = per head with head_dim weights (model.py:180); the workgroup sums the squares for itself.
template <int HD8, int IT, int NW, int NORM>
__global__ __launch_bounds__(NW * 64) void attn_split1_kernel(const AttnArgs a) {
  constexpr int HD = HD8 * 8, RPI = 64 / HD8, NVI = 16 / RPI, NGRP = NW * RPI, CSTR = HD + 4, SP = 16 * NW * IT;
  const int group = a.n_heads / a.n_kv;
  const int kvh = blockIdx.x % a.n_kv, rest = blockIdx.x / a.n_kv, hh = rest % group, split = rest / group, head = kvh * group + hh;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, half = HD >> 1;
  __shared__ float qs[HD], ks[HD], vs[HD];
  __shared__ float comb[NGRP * CSTR];                   // [run]: o[HD], m, l
  const int vr = lane / HD8, vp = lane % HD8;
  const int p0 = split * SP + wave * 16;                // first position of this wave's first tile; tile t starts 16 NW t further
  // ---- loads that do not depend on the position
  const int ki = tid < half ? tid : half - 1, vi = tid < HD ? tid : HD - 1;
  const float kx1 = a.k[kvh * HD + ki], kx2 = a.k[kvh * HD + half + ki], vx = a.v[kvh * HD + vi];
  const float qx1 = a.q[head * HD + ki], qx2 = a.q[head * HD + half + ki];
  float kw1 = 1.f, kw2 = 1.f, qw1 = 1.f, qw2 = 1.f, ssq = 0.f, ssk = 0.f;   // norm weights of this thread's pairs; its share of the sums of squares
  if constexpr (NORM != 0) {
    const int kb = NORM == 2 ? 0 : kvh * HD, qb = NORM == 2 ? 0 : head * HD;
    kw1 = a.k_norm[kb + ki]; kw2 = a.k_norm[kb + half + ki]; qw1 = a.q_norm[qb + ki]; qw2 = a.q_norm[qb + half + ki];
    if constexpr (NORM == 2) { if (tid < half) { ssq = qx1 * qx1 + qx2 * qx2; ssk = kx1 * kx1 + kx2 * kx2; } }
    else {
      const int n4q = (a.n_heads * HD) >> 2, n4k = (a.n_kv * HD) >> 2, nmax = n4q > n4k ? n4q : n4k;
      for (int i = tid; i < nmax; i += NW * 64) {
        const f32x4 x = ((const f32x4*)a.q)[i < n4q ? i : n4q - 1], y = ((const f32x4*)a.k)[i < n4k ? i : n4k - 1];
        if (i < n4q) ssq += x.x * x.x + x.y * x.y + x.z * x.z + x.w * x.w;
        if (i < n4k) ssk += y.x * y.x + y.y * y.y + y.z * y.z + y.w * y.w;
      }
    }
  }
  u32x4 kt[IT][NVI], vt[IT][NVI];
  {
    const _Float16* kbase = a.cache_k + (size_t)kvh * a.max_ctx * HD + vp * 8;
    const _Float16* vbase = a.cache_v + (size_t)kvh * a.max_ctx * HD + vp * 8;
#pragma unroll
    for (int t = 0; t < IT; t++) {
#pragma unroll
      for (int i = 0; i < NVI; i++) {
        const int r = p0 + t * 16 * NW + i * RPI + vr, rc = r < a.max_ctx ? r : a.max_ctx - 1;
        kt[t][i] = *(const u32x4*)(kbase + (size_t)rc * HD);
        vt[t][i] = *(const u32x4*)(vbase + (size_t)rc * HD);
      }
    }
  }
  const int pos = a.st->pos;
  if (pos >= a.max_ctx || pos < 0) {                    // no cache row and no rotation row for this position: nothing is written, the host sees the flag
    if (blockIdx.x == 0 && tid == 0) atomicOr(&a.st->error, 2);
    return;
  }
  float* ph_ = a.part + (size_t)head * (a.nsplit * HD + 16);
  float* po = ph_ + (size_t)split * HD;                    // this split's weighted V sums
  float* pml = ph_ + (size_t)a.nsplit * HD + 2 * split;    // and its (max, sum)
  if (split * SP > pos) {                               // nothing cached in this split yet
    if (tid < HD) po[tid] = 0.f;
    if (tid == 0) { pml[0] = -INFINITY; pml[1] = 0.f; }
    return;
  }
  const float rc_ = a.rope[(size_t)pos * HD + ki], rs_ = a.rope[(size_t)pos * HD + half + ki];
  float qscale = 1.f, kscale = 1.f;
  if constexpr (NORM != 0) {
    __shared__ float red[2][NW];
    ssq = wave_sum(ssq); ssk = wave_sum(ssk);
    if (lane == 0) { red[0][wave] = ssq; red[1][wave] = ssk; }
    __syncthreads();
    float sq = 0.f, sk = 0.f;
#pragma unroll
    for (int w = 0; w < NW; w++) { sq += red[0][w]; sk += red[1][w]; }
    qscale = 1.0f / sqrtf(sq / (float)(NORM == 2 ? HD : a.n_heads * HD) + a.norm_eps);
    kscale = 1.0f / sqrtf(sk / (float)(NORM == 2 ? HD : a.n_kv * HD) + a.norm_eps);
  }
  if (tid < half) {
    const float k1 = NORM != 0 ? (kx1 * kscale) * kw1 : kx1, k2 = NORM != 0 ? (kx2 * kscale) * kw2 : kx2;
    const float q1 = NORM != 0 ? (qx1 * qscale) * qw1 : qx1, q2 = NORM != 0 ? (qx2 * qscale) * qw2 : qx2;
    ks[tid] = rope_lo(k1, k2, rc_, rs_); ks[half + tid] = rope_hi(k1, k2, rc_, rs_);
    qs[tid] = rope_lo(q1, q2, rc_, rs_); qs[half + tid] = rope_hi(q1, q2, rc_, rs_);
  }
  if (tid < HD) vs[tid] = vx;
  __syncthreads();
  if (hh == 0 && pos / SP == split && tid < HD) {       // one workgroup per kv head appends this token to the cache
    a.cache_k[((size_t)kvh * a.max_ctx + pos) * HD + tid] = (_Float16)ks[tid];
    a.cache_v[((size_t)kvh * a.max_ctx + pos) * HD + tid] = (_Float16)vs[tid];
  }
  const u32x4 kcur = pack8_f16(ks + vp * 8), vcur = pack8_f16(vs + vp * 8);   // rounded to fp16 exactly like the cached copy
  float qq[8];
#pragma unroll
  for (int j = 0; j < 8; j++) qq[j] = qs[vp * 8 + j];
  float sc[IT][NVI];
  float m = -INFINITY;
#pragma unroll
  for (int t = 0; t < IT; t++) {
#pragma unroll
    for (int i = 0; i < NVI; i++) {
      const int r = p0 + t * 16 * NW + i * RPI + vr;
      const u32x4 kk = r >= pos ? kcur : kt[t][i];
      const half2_t k0 = as_h2(kk.x), k1 = as_h2(kk.y), k2 = as_h2(kk.z), k3 = as_h2(kk.w);
      float s = qq[0] * (float)k0.x; s += qq[1] * (float)k0.y; s += qq[2] * (float)k1.x; s += qq[3] * (float)k1.y;
      s += qq[4] * (float)k2.x; s += qq[5] * (float)k2.y; s += qq[6] * (float)k3.x; s += qq[7] * (float)k3.y;
      s = run_sum<HD8>(s);
      sc[t][i] = r <= pos ? s * a.scale : -INFINITY;
      m = fmaxf(m, sc[t][i]);
    }
  }
  // softmax partial of this lane run (its rows of every tile): no cross-lane traffic, the fold below sums the runs
  float l = 0.f;
  f32x4 o0 = {0.f, 0.f, 0.f, 0.f}, o1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int t = 0; t < IT; t++) {
#pragma unroll
    for (int i = 0; i < NVI; i++) {
      const int r = p0 + t * 16 * NW + i * RPI + vr;
      const float pj = r <= pos ? __expf(sc[t][i] - m) : 0.f;
      l += pj;
      const u32x4 vv = r >= pos ? vcur : vt[t][i];
      const half2_t v0 = as_h2(vv.x), v1 = as_h2(vv.y), v2 = as_h2(vv.z), v3 = as_h2(vv.w);
      o0.x += pj * (float)v0.x; o0.y += pj * (float)v0.y; o0.z += pj * (float)v1.x; o0.w += pj * (float)v1.y;
      o1.x += pj * (float)v2.x; o1.y += pj * (float)v2.y; o1.z += pj * (float)v3.x; o1.w += pj * (float)v3.y;
    }
  }
  float* cw = comb + (size_t)(wave * RPI + vr) * CSTR;
  *(f32x4*)(cw + vp * 8) = o0; *(f32x4*)(cw + vp * 8 + 4) = o1;
  if (vp == 0) { cw[HD] = m; cw[HD + 1] = l; }
  __syncthreads();
  // fold of the row-run partials into the split partial: the run maximum by every thread, then thread (part, d) sums every NP-th run of dimension d
  // and the NP parts meet in LDS (the q / k / v rows, no longer needed)
  constexpr int NP = NW * 64 / HD, GP = NGRP / NP;
  static_assert(NGRP % NP == 0 && NP >= 1 && NP <= 16, "fold layout");
  __shared__ float fold_o[NP][HD], fold_l[NP];
  float mm = -INFINITY;                                 // the first run of wave 0 always holds a valid position: mm is finite
#pragma unroll
  for (int g = 0; g < NGRP; g++) mm = fmaxf(mm, comb[g * CSTR + HD]);
  {
    const int part = tid / HD, d = tid % HD;
    float ll = 0.f, od = 0.f;
#pragma unroll
    for (int j = 0; j < GP; j++) {
      const int g = part + NP * j;
      const float mg = comb[g * CSTR + HD];
      const float wg = mg == -INFINITY ? 0.f : __expf(mg - mm);   // a run without valid rows contributes nothing
      ll += wg * comb[g * CSTR + HD + 1];
      od += wg * comb[g * CSTR + d];
    }
    fold_o[part][d] = od;
    if (d == 0) fold_l[part] = ll;
  }
  __syncthreads();
  if (tid < HD) {
    float od = 0.f, ll = 0.f;
#pragma unroll
    for (int q = 0; q < NP; q++) { od += fold_o[q][tid]; ll += fold_l[q]; }
    po[tid] = od;
    if (tid == 0) { pml[0] = mm; pml[1] = ll; }
  }
}

// Second launch: one workgroup of HD threads per query head combines that head's split partials (max, sum, weighted V).  A kernel
// boundary orders the partials; it costs less than publishing them inside one launch (write-through stores, completion wait, arrival
// counter, cache-bypassing reads: four dependent memory round trips on the critical path of the last workgroup to arrive).
template <int HD>
__global__ __launch_bounds__(HD) void attn_merge_kernel(const AttnArgs args) {
  const AttnArgs a = attn_args_of_sequence(args, blockIdx.y);   // field reads become kernel-argument loads in the entry block
  constexpr int FB = 24, NB = 16;                       // splits read ahead of the position (contexts up to 1536 in one round trip), later batches
  const int head = blockIdx.x, d = threadIdx.x;
  __shared__ float sw[1024];                            // exp(m_s - m) per split
  __shared__ float red[2 * (HD / 64)];
  const int nsp = a.nsplit;
  const float* ph = a.part + (size_t)head * nsp * (HD + 2);
  // position-independent loads first (splits that were never written are masked below): thread d takes (m, l) of split d, and every
  // thread the first FB partial outputs of its dimension
  const int spc = d < nsp ? d : nsp - 1;
  const float mv = ph[(size_t)spc * (HD + 2) + HD], lv = ph[(size_t)spc * (HD + 2) + HD + 1];
  float v[FB];
#pragma unroll
  for (int j = 0; j < FB; j++) v[j] = ph[(size_t)(j < nsp ? j : nsp - 1) * (HD + 2) + d];
  const int pos = a.st->pos + blockIdx.y * a.pos_step, ns = (pos >> a.split_shift) + 1;
  if (pos >= a.max_ctx || pos < 0) return;              // refused by the split launch (state.error): the output row keeps its contents
  float m = -INFINITY, l = 0.f;
  if (nsp <= HD) {
    m = wave_max(d < ns ? mv : -INFINITY);
    if constexpr (HD > 64) {
      if ((d & 63) == 0) red[d >> 6] = m;
      __syncthreads();
      m = red[0];
#pragma unroll
      for (int i = 1; i < HD / 64; i++) m = fmaxf(m, red[i]);
    }
    const float e = d < ns ? __expf(mv - m) : 0.f;
    if (d < ns) sw[d] = e;
    l = d < ns ? lv * e : 0.f;
  } else {                                              // more splits than threads: thread t takes splits t, t + HD, ...
    for (int sp = d; sp < ns; sp += HD) m = fmaxf(m, ph[(size_t)sp * (HD + 2) + HD]);
    m = wave_max(m);
    if constexpr (HD > 64) {
      if ((d & 63) == 0) red[d >> 6] = m;
      __syncthreads();
      m = red[0];
#pragma unroll
      for (int i = 1; i < HD / 64; i++) m = fmaxf(m, red[i]);
    }
    for (int sp = d; sp < ns; sp += HD) { const float e = __expf(ph[(size_t)sp * (HD + 2) + HD] - m); sw[sp] = e; l += ph[(size_t)sp * (HD + 2) + HD + 1] * e; }
  }
  l = wave_sum(l);
  if constexpr (HD > 64) {
    if ((d & 63) == 0) red[HD / 64 + (d >> 6)] = l;
    __syncthreads();
    l = 0.f;
#pragma unroll
    for (int i = 0; i < HD / 64; i++) l += red[HD / 64 + i];
  } else __syncthreads();
  float o = 0.f;
#pragma unroll
  for (int j = 0; j < FB; j++) o += j < ns ? v[j] * sw[j] : 0.f;
  for (int s0 = FB; s0 < ns; s0 += NB) {
    float w[NB];
#pragma unroll
    for (int j = 0; j < NB; j++) w[j] = ph[(size_t)min(s0 + j, ns - 1) * (HD + 2) + d];
#pragma unroll
    for (int j = 0; j < NB; j++) o += s0 + j < ns ? w[j] * sw[s0 + j] : 0.f;
  }
  o *= 1.0f / l;
  const int e = head * HD + d;
  if (a.stage_rows_ncg) args.out16[rows_staged_pos(a.stage_fmt, e, blockIdx.y, a.stage_rows_ncg)] = (_Float16)o;
  else if (a.out16) a.out16[a.stage_fmt ? staged_pos(a.stage_fmt, e, a.stage_nu) : e] = (_Float16)o;
  if (a.out32) a.out32[e] = o;
}

// ---------------------------------------------------------------------------------------------- argmax + token bookkeeping
// argmax(-1) with the reference's tie rule: the first index of the maximum (tinygrad/mixin/op.py:866-891).
__global__ __launch_bounds__(256) void argmax_partial_kernel(const float* __restrict__ logits, int n, float* __restrict__ pv, int* __restrict__ pi) {
  float best = -INFINITY; int bi = 0;                   // (no finite or -inf maximum at all, i.e. NaN logits: index 0, never an index outside the row)
  for (int i = blockIdx.x * 256 + threadIdx.x; i < n; i += gridDim.x * 256) {
    const float v = logits[i];
    if (v > best || (v == best && i < bi)) { best = v; bi = i; }
  }
  __shared__ float sv[256]; __shared__ int si[256];
  sv[threadIdx.x] = best; si[threadIdx.x] = bi;
  __syncthreads();
  for (int o = 128; o > 0; o >>= 1) {
    if (threadIdx.x < o) {
      const float v = sv[threadIdx.x + o]; const int i = si[threadIdx.x + o];
      if (v > sv[threadIdx.x] || (v == sv[threadIdx.x] && i < si[threadIdx.x])) { sv[threadIdx.x] = v; si[threadIdx.x] = i; }
    }
    __syncthreads();
  }
  if (threadIdx.x == 0) { pv[blockIdx.x] = sv[0]; pi[blockIdx.x] = si[0]; }
}
// Final reduce and the loop bookkeeping of Transformer.generate (tinygrad/llm/model.py:475-484) kept on the device: while
// prompt tokens remain the next input is prompt[pos + 1]; afterwards the argmax token is appended to out_tokens and fed back.
__global__ __launch_bounds__(256) void argmax_final_kernel(const float* __restrict__ pv, const int* __restrict__ pi, int np, DecodeState* st,
                                                           const int* __restrict__ prompt, int* __restrict__ out_tokens, int max_tokens) {
  __shared__ float sv[256]; __shared__ int si[256];
  float best = -INFINITY; int bi = 0;
  for (int i = threadIdx.x; i < np; i += 256) {
    const float v = pv[i]; const int ix = pi[i];
    if (v > best || (v == best && ix < bi)) { best = v; bi = ix; }
  }
  sv[threadIdx.x] = best; si[threadIdx.x] = bi;
  __syncthreads();
  for (int o = 128; o > 0; o >>= 1) {
    if (threadIdx.x < o) {
      const float v = sv[threadIdx.x + o]; const int i = si[threadIdx.x + o];
      if (v > sv[threadIdx.x] || (v == sv[threadIdx.x] && i < si[threadIdx.x])) { sv[threadIdx.x] = v; si[threadIdx.x] = i; }
    }
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    const int next = st->pos + 1;
    if (next < st->n_prompt) st->token = prompt[next];
    else {
      const int tok = si[0];
      if (out_tokens && st->step < max_tokens) out_tokens[st->step] = tok;
      st->token = tok; st->step += 1;
    }
    st->pos = next;
  }
}
// Prompt step without sampling (no lm-head was run): feed prompt[pos + 1] and advance.
__global__ void advance_prompt_kernel(DecodeState* st, const int* __restrict__ prompt) {
  const int next = st->pos + 1;
  if (next < st->n_prompt) st->token = prompt[next];
  st->pos = next;
}

// Batched decode (sequences in lockstep): workgroup b takes sequence b.  While prompt tokens remain the next input of sequence b is
// prompts[b][pos + 1]; afterwards the first index of the row maximum (logits == nullptr: a prompt step that ran no lm-head) is stored at
// out_tokens[step][b] and fed back.  The shared position advances in a launch of its own (advance_batch_kernel), after every row has read it.
__global__ __launch_bounds__(1024) void argmax_rows_kernel(const float* __restrict__ logits, int n, const DecodeState* st, const int* __restrict__ prompts, int prompt_stride,
                                                           int* __restrict__ tokens, int* __restrict__ out_tokens, int max_steps, int batch) {
  const int b = blockIdx.x, next = st->pos + 1;
  if (next < st->n_prompt || !logits) { if (threadIdx.x == 0 && next < st->n_prompt) tokens[b] = prompts[(size_t)b * prompt_stride + next]; return; }
  const float* row = logits + (size_t)b * n;
  float best = -INFINITY; int bi = 0;
  // a thread meets its indices in increasing order: the first of equal values stays.  Aligned rows are read as 16-byte pieces, eight requests at a time
  // (one workgroup per row: what bounds the launch is the number of dependent round trips, 125 of them with one value per request)
  int i0 = 0;
  if (((uintptr_t)row & 15) == 0) {
    const int n4 = n >> 2;
    const float4* r4 = (const float4*)row;
    int q = threadIdx.x;
    for (; q + 7 * 1024 < n4; q += 8 * 1024) {
      float4 v[8];
#pragma unroll
      for (int u = 0; u < 8; u++) v[u] = r4[q + u * 1024];
#pragma unroll
      for (int u = 0; u < 8; u++) {
        const int i = 4 * (q + u * 1024);
        if (v[u].x > best) { best = v[u].x; bi = i; }
        if (v[u].y > best) { best = v[u].y; bi = i + 1; }
        if (v[u].z > best) { best = v[u].z; bi = i + 2; }
        if (v[u].w > best) { best = v[u].w; bi = i + 3; }
      }
    }
    for (; q < n4; q += 1024) {
      const float4 v = r4[q]; const int i = 4 * q;
      if (v.x > best) { best = v.x; bi = i; }
      if (v.y > best) { best = v.y; bi = i + 1; }
      if (v.z > best) { best = v.z; bi = i + 2; }
      if (v.w > best) { best = v.w; bi = i + 3; }
    }
    i0 = 4 * n4;
  }
  for (int i = i0 + threadIdx.x; i < n; i += 1024) { const float v = row[i]; if (v > best) { best = v; bi = i; } }
  __shared__ float sv[1024]; __shared__ int si[1024];
  sv[threadIdx.x] = best; si[threadIdx.x] = bi;
  __syncthreads();
  for (int o = 512; o > 0; o >>= 1) {
    if (threadIdx.x < o) {
      const float v = sv[threadIdx.x + o]; const int i = si[threadIdx.x + o];
      if (v > sv[threadIdx.x] || (v == sv[threadIdx.x] && i < si[threadIdx.x])) { sv[threadIdx.x] = v; si[threadIdx.x] = i; }
    }
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    tokens[b] = si[0];
    if (out_tokens && st->step < max_steps) out_tokens[(size_t)st->step * batch + b] = si[0];
  }
}
__global__ void advance_batch_kernel(DecodeState* st, int had_logits) {
  const int next = st->pos + 1;
  if (next >= st->n_prompt && had_logits) st->step += 1;
  st->pos = next;
}

// chunked prefill: the next `rows` prompt tokens become the input rows, the position moves on by `rows` (positions past the prompt table read its last entry)
__global__ void chunk_advance_kernel(DecodeState* st, const int* __restrict__ prompt, int rows, int* __restrict__ tokens, int max_ctx) {
  const int np = st->pos + rows;
  __syncthreads();
  if ((int)threadIdx.x < rows) { const int i = np + (int)threadIdx.x; tokens[threadIdx.x] = prompt[i < max_ctx ? (i < 0 ? 0 : i) : max_ctx - 1]; }
  if (threadIdx.x == 0) st->pos = np;
}

// silu(gate) * up over n float32 values, rounded to fp16 (the feed-forward's activation, tinygrad/llm/model.py:137, where ffn_gate and ffn_up are of different
// block types and run as two launches instead of one with the SwiGLU epilogue)
__global__ __launch_bounds__(256) void silu_mul_kernel(const float* __restrict__ gate, const float* __restrict__ up, int n, _Float16* __restrict__ out) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i < n) out[i] = (_Float16)(silu_f(gate[i]) * up[i]);
}

// ---------------------------------------------------------------------------------------------- C-ABI
extern "C" {

int tga_embed_row(const void* table, int ggml_type, int dim, const void* state, float* out, void* stream) {
  TGA_REQUIRE(table && state && out, "tga_embed_row: null pointer");
  int blk = 0;
  switch (ggml_type) { case GGML_Q4_0: case GGML_Q8_0: case GGML_MXFP4: case GGML_Q4_1: case GGML_Q5_0: case GGML_Q5_1: blk = 32; break; case GGML_Q4_K: case GGML_Q5_K: case GGML_Q6_K: case GGML_IQ4_XS: case GGML_IQ3_XXS: case GGML_IQ3_S: case GGML_IQ2_S: blk = 256; break;
    case GGML_Q1_0: blk = 128; break; case GGML_F16: case GGML_F32: blk = 1; break; default: return tga_set_error("tga_embed_row: unsupported table type %d", ggml_type); }
  TGA_REQUIRE(dim > 0 && dim % blk == 0 && dim % 4 == 0, "tga_embed_row: dim=%d must be a positive multiple of 4 and of the table's block size %d", dim, blk);
  embed_row_kernel<<<1, 256, 0, (hipStream_t)stream>>>((const uint8_t*)table, ggml_type, dim, (DecodeState*)state, out, nullptr);
  TGA_LAUNCH_CHECK();
  return 0;
}

int tga_embed_rows(const void* table, int ggml_type, int dim, const int32_t* tokens, int n_rows, void* state, float* out, void* stream) {
  TGA_REQUIRE(table && state && out && tokens && n_rows >= 1, "tga_embed_rows: null pointer or no rows");
  int blk = 0;
  switch (ggml_type) { case GGML_Q4_0: case GGML_Q8_0: case GGML_MXFP4: case GGML_Q4_1: case GGML_Q5_0: case GGML_Q5_1: blk = 32; break; case GGML_Q4_K: case GGML_Q5_K: case GGML_Q6_K: case GGML_IQ4_XS: case GGML_IQ3_XXS: case GGML_IQ3_S: case GGML_IQ2_S: blk = 256; break;
    case GGML_Q1_0: blk = 128; break; case GGML_F16: case GGML_F32: blk = 1; break; default: return tga_set_error("tga_embed_rows: unsupported table type %d", ggml_type); }
  TGA_REQUIRE(dim > 0 && dim % blk == 0 && dim % 4 == 0, "tga_embed_rows: dim=%d must be a positive multiple of 4 and of the table's block size %d", dim, blk);
  embed_row_kernel<<<n_rows, 256, 0, (hipStream_t)stream>>>((const uint8_t*)table, ggml_type, dim, (DecodeState*)state, out, tokens);
  TGA_LAUNCH_CHECK();
  return 0;
}

// staged layout lookup shared with the GEMV host side (qgemv.hip)
static int decode_staged_fmt(int ggml_type, long long K, int* nu) {
  int fmt = -1, uw = 64;
  switch (ggml_type) {
    case GGML_Q4_0: fmt = F_Q4_0P; break; case GGML_Q8_0: fmt = F_Q8_0P; break; case GGML_Q6_K: fmt = GGML_Q6_K; break;
    case GGML_Q4_K: fmt = GGML_Q4_K; break; case GGML_Q5_K: fmt = GGML_Q5_K; break;
    case GGML_Q4_1: fmt = GGML_Q4_1; break; case GGML_Q5_0: fmt = GGML_Q5_0; break; case GGML_Q5_1: fmt = GGML_Q5_1; break; case GGML_IQ4_XS: fmt = GGML_IQ4_XS; break;
    case GGML_IQ3_XXS: case GGML_IQ3_S: case GGML_IQ2_S: case GGML_Q1_0: fmt = ggml_type; break;
    case GGML_F16: fmt = GGML_F16; break; case GGML_MXFP4: fmt = GGML_MXFP4; uw = 32; break;
  }
  if (fmt < 0 || K <= 0 || K % tga_block_weights(ggml_type) != 0 || K % 64 != 0) return -1;
  *nu = (int)(K / uw);
  return fmt;
}

int tga_rmsnorm_rows(const float* x, const float* weight, int rows, int dim, float eps, void* out_f16, float* out_f32, int stage_type, void* stream) {
  TGA_REQUIRE(x && weight && (out_f16 || out_f32), "tga_rmsnorm: null pointer");
  TGA_REQUIRE(dim > 0 && rows >= 1, "tga_rmsnorm: rows=%d dim=%d", rows, dim);
  int sfmt = 0, snu = 0;
  if (stage_type) { sfmt = decode_staged_fmt(stage_type, dim, &snu); TGA_REQUIRE(sfmt >= 0, "tga_rmsnorm: no staged layout for type %d with K=%d", stage_type, dim); }
  rmsnorm_kernel<false><<<rows, 1024, 0, (hipStream_t)stream>>>(x, weight, dim, eps, (_Float16*)out_f16, out_f32, sfmt, snu, nullptr, nullptr, nullptr, 0);
  TGA_LAUNCH_CHECK();
  return 0;
}
int tga_moe_combine_rmsnorm_rows(const float* y, const float* probs, float* x, const float* weight, int rows, int k, int dim, float eps, void* out_f16, float* out_f32,
                                 void* stream) {
  TGA_REQUIRE(y && probs && x && weight && (out_f16 || out_f32), "tga_moe_combine_rmsnorm_rows: null pointer");
  TGA_REQUIRE(dim > 0 && rows >= 1 && k >= 1, "tga_moe_combine_rmsnorm_rows: rows=%d k=%d dim=%d", rows, k, dim);
  rmsnorm_kernel<true><<<rows, 1024, 0, (hipStream_t)stream>>>(x, weight, dim, eps, (_Float16*)out_f16, out_f32, 0, 0, x, y, probs, k);
  TGA_LAUNCH_CHECK();
  return 0;
}
int tga_silu_mul(const float* gate, const float* up, int64_t n, void* out_f16, void* stream) {
  TGA_REQUIRE(gate && up && out_f16 && n > 0 && n < (1ll << 31), "tga_silu_mul: null pointer or bad length");
  silu_mul_kernel<<<(unsigned)((n + 255) / 256), 256, 0, (hipStream_t)stream>>>(gate, up, (int)n, (_Float16*)out_f16);
  TGA_LAUNCH_CHECK();
  return 0;
}
int tga_rmsnorm(const float* x, const float* weight, int dim, float eps, void* out_f16, float* out_f32, int stage_type, void* stream) {
  return tga_rmsnorm_rows(x, weight, 1, dim, eps, out_f16, out_f32, stage_type, stream);
}

static int attention_launch(int chunk, int batch, const float* q, const float* k, const float* v, const float* q_norm_weight, const float* k_norm_weight, float norm_eps,
                            int norm_per_head, void* cache_k, void* cache_v, float* partials, const void* state,
                            int n_heads, int n_kv_heads, int head_dim, int max_ctx, const float* rope_table, void* out_f16, float* out_f32, int stage_type, void* stream) {
  TGA_REQUIRE(batch >= 1 && batch <= 65535, "tga_attention_decode: batch=%d", batch);
  TGA_REQUIRE(q && k && v && cache_k && cache_v && partials && state && rope_table && (out_f16 || out_f32), "tga_attention_decode: null pointer");
  TGA_REQUIRE(n_kv_heads > 0 && n_heads % n_kv_heads == 0, "tga_attention_decode: n_heads=%d must be a multiple of n_kv_heads=%d", n_heads, n_kv_heads);
  TGA_REQUIRE(head_dim == 64 || head_dim == 128 || head_dim == 256, "tga_attention_decode: head_dim=%d must be 64, 128 or 256", head_dim);
  TGA_REQUIRE(max_ctx > 0 && (n_heads / n_kv_heads) * ((max_ctx + 63) / 64) <= 1024, "tga_attention_decode: max_ctx=%d too long for the merge table ((n_heads/n_kv_heads) * ceil(max_ctx/64) <= 1024)", max_ctx);
  TGA_REQUIRE((q_norm_weight == nullptr) == (k_norm_weight == nullptr), "tga_attention_decode: q and k norm weights come together");
  TGA_REQUIRE(!q_norm_weight || ((((uintptr_t)q | (uintptr_t)k) & 15) == 0), "tga_attention_decode: q and k must be 16-byte aligned for the fused norm");
  AttnArgs a;
  a.q = q; a.k = k; a.v = v; a.cache_k = (_Float16*)cache_k; a.cache_v = (_Float16*)cache_v; a.part = partials; a.st = (DecodeState*)state;
  a.n_heads = n_heads; a.n_kv = n_kv_heads; a.hd = head_dim; a.max_ctx = max_ctx; a.nsplit = (max_ctx + 63) / 64;
  a.rope = rope_table; a.scale = 1.0f / sqrtf((float)head_dim);
  a.out16 = (_Float16*)out_f16; a.out32 = out_f32;
  a.stage_fmt = 0; a.stage_nu = 0; a.stage_rows_ncg = 0;
  a.q_norm = q_norm_weight; a.k_norm = k_norm_weight; a.norm_eps = norm_eps; a.norm_per_head = norm_per_head;
  a.q_bs = (long long)n_heads * head_dim; a.kv_bs = (long long)n_kv_heads * head_dim; a.cache_bs = (long long)n_kv_heads * max_ctx * head_dim;
  a.part_bs = (long long)n_heads * a.nsplit * (head_dim + 2); a.out_bs = (long long)n_heads * head_dim;
  a.chunk = 0; a.pos_step = 0; a.split_shift = 6;
  if (chunk) { a.cache_bs = 0; a.pos_step = 1; }
  if (stage_type) { a.stage_fmt = decode_staged_fmt(stage_type, (long long)n_heads * head_dim, &a.stage_nu); TGA_REQUIRE(a.stage_fmt >= 0, "tga_attention_decode: no staged layout for type %d", stage_type); }
  if (stage_type && chunk) {                            // the rows of a prefill step for the 17 .. 128 row GEMM
    TGA_REQUIRE(out_f16 && batch >= 17 && batch <= 128 && ((long long)n_heads * head_dim) % 256 == 0 && stage_type != GGML_MXFP4 && stage_type != GGML_Q4_1 && stage_type != GGML_Q5_0 && stage_type != GGML_Q5_1,
                "tga_attention_prefill_chunk: rows in the multiplying layout need 17..128 rows, n_heads * head_dim a multiple of 256 and a block type the prefill kernel takes");
    a.stage_rows_ncg = batch <= 32 ? 2 : batch <= 64 ? 4 : 8;
  }
  dim3 grid(n_kv_heads, a.nsplit, batch);
  hipStream_t s = (hipStream_t)stream;
  const int norm = !q_norm_weight ? 0 : norm_per_head ? 2 : ((long long)n_heads * head_dim <= 4096 && (long long)n_kv_heads * head_dim <= 4096) ? 1 : 3;
#define TGA_ATTN_LAUNCH(HD8) do { \
    if (norm == 0) attn_decode_kernel<HD8, 0><<<grid, 256, 0, s>>>(a); else if (norm == 1) attn_decode_kernel<HD8, 1><<<grid, 256, 0, s>>>(a); \
    else if (norm == 2) attn_decode_kernel<HD8, 2><<<grid, 256, 0, s>>>(a); else attn_decode_kernel<HD8, 3><<<grid, 256, 0, s>>>(a); } while (0)
  static const bool chunk_mfma_off = getenv("TGA_ATTN_CHUNK") && !strcmp(getenv("TGA_ATTN_CHUNK"), "rows");
  const bool chunk_mfma = chunk && batch > 8 && norm == 0 && (head_dim == 64 || head_dim == 128) && n_heads / n_kv_heads <= 8 && !chunk_mfma_off;   // chunks of more than eight rows attend on the matrix cores
  for (int pass = chunk ? 1 : 0; pass <= (chunk ? 2 : 0); pass++) {   // chunked prefill: append every row, then attend from the cache
    a.chunk = pass;
    if (pass == 2 && chunk_mfma) {
      // TS tiles of 64 keys per split partial: fewer and larger partials for the merge launch (its arguments follow)
      static const int env_ts = getenv("TGA_ATTN_CHUNK_TILES") ? atoi(getenv("TGA_ATTN_CHUNK_TILES")) : 0;
      const int group = n_heads / n_kv_heads;
      const int ts = env_ts == 1 ? 1 : 2;                                  // (four tiles per partial leave a context of 1024 with one workgroup per CU: 21 us against 17)
      a.split_shift = ts == 2 ? 7 : 6;
      a.nsplit = (a.nsplit + ts - 1) / ts;
      a.part_bs = (long long)n_heads * a.nsplit * (head_dim + 2);
      const dim3 cgrid(n_kv_heads, a.nsplit, (batch + 15) / 16);
#define TGA_CHUNK_T(HD8, TS) do { if (group <= 4) attn_chunk_mfma_kernel<HD8, TS, 1><<<cgrid, 256, 0, s>>>(a, batch); else attn_chunk_mfma_kernel<HD8, TS, 2><<<cgrid, 256, 0, s>>>(a, batch); } while (0)
#define TGA_CHUNK(HD8) do { if (ts == 2) TGA_CHUNK_T(HD8, 2); else TGA_CHUNK_T(HD8, 1); } while (0)
      if (head_dim == 64) TGA_CHUNK(8); else TGA_CHUNK(16);
#undef TGA_CHUNK
#undef TGA_CHUNK_T
      TGA_LAUNCH_CHECK();
      break;
    }
    grid = dim3(n_kv_heads, pass == 1 ? 1 : a.nsplit, batch);
    if (head_dim == 64) TGA_ATTN_LAUNCH(8);
    else if (head_dim == 128) TGA_ATTN_LAUNCH(16);
    else TGA_ATTN_LAUNCH(32);
    TGA_LAUNCH_CHECK();
  }
#undef TGA_ATTN_LAUNCH
  const dim3 mgrid(n_heads, batch);
  if (head_dim == 64) attn_merge_kernel<64><<<mgrid, 64, 0, s>>>(a);
  else if (head_dim == 128) attn_merge_kernel<128><<<mgrid, 128, 0, s>>>(a);
  else attn_merge_kernel<256><<<mgrid, 256, 0, s>>>(a);
  TGA_LAUNCH_CHECK();
  return 0;
}

int tga_attention_decode_normed(const float* q, const float* k, const float* v, const float* q_norm_weight, const float* k_norm_weight, float norm_eps,
                                int norm_per_head, void* cache_k, void* cache_v, float* partials, const void* state,
                                int n_heads, int n_kv_heads, int head_dim, int max_ctx, const float* rope_table, void* out_f16, float* out_f32, int stage_type, void* stream) {
  return attention_launch(0, 1, q, k, v, q_norm_weight, k_norm_weight, norm_eps, norm_per_head, cache_k, cache_v, partials, state, n_heads, n_kv_heads, head_dim, max_ctx,
                          rope_table, out_f16, out_f32, stage_type, stream);
}

// Tiles per wave (1..4) and number of splits (at most six) of the one-launch attention for a cache of max_ctx positions, nw waves per workgroup; 0: too long
static int attn_split1_waves() { static const int nw = getenv("TGA_ATTN_WAVES") ? atoi(getenv("TGA_ATTN_WAVES")) : 8; return nw == 4 || nw == 16 ? nw : 8; }
static int attn_split1_tiles(int max_ctx, int* n_splits) {
  static const int forced = getenv("TGA_ATTN_TILES") ? atoi(getenv("TGA_ATTN_TILES")) : 0;
  const int rows = 16 * attn_split1_waves();
  for (int it = 1; it <= 4; it++) { const int s = (max_ctx + rows * it - 1) / (rows * it); if (s <= 6 && (!forced || it == forced || it == 4)) { *n_splits = s; return it; } }
  *n_splits = 0; return 0;
}
int tga_attention_split_plan(int max_ctx, int* n_splits) {
  TGA_REQUIRE(n_splits && max_ctx > 0, "tga_attention_split_plan: null pointer or max_ctx=%d", max_ctx);
  attn_split1_tiles(max_ctx, n_splits);
  return 0;
}
static int attention_decode_split(const float* q, const float* k, const float* v, const float* q_norm_weight, const float* k_norm_weight, float norm_eps, int norm_per_head,
                                  void* cache_k, void* cache_v, float* partials, const void* state,
                                  int n_heads, int n_kv_heads, int head_dim, int max_ctx, const float* rope_table, void* stream) {
  TGA_REQUIRE(q && k && v && cache_k && cache_v && partials && state && rope_table, "tga_attention_decode_split: null pointer");
  TGA_REQUIRE(!q_norm_weight == !k_norm_weight, "tga_attention_decode_split: q and k norm weights come together");
  TGA_REQUIRE(!q_norm_weight || ((((uintptr_t)q | (uintptr_t)k) & 15) == 0), "tga_attention_decode_split: normed q and k rows must be 16-byte aligned");
  TGA_REQUIRE(n_kv_heads > 0 && n_heads % n_kv_heads == 0, "tga_attention_decode_split: n_heads=%d must be a multiple of n_kv_heads=%d", n_heads, n_kv_heads);
  TGA_REQUIRE(head_dim == 64 || head_dim == 128 || head_dim == 256, "tga_attention_decode_split: head_dim=%d must be 64, 128 or 256", head_dim);
  TGA_REQUIRE(((uintptr_t)partials & 15) == 0, "tga_attention_decode_split: partials must be 16-byte aligned");
  int ns = 0; const int it = max_ctx > 0 ? attn_split1_tiles(max_ctx, &ns) : 0;
  TGA_REQUIRE(it > 0, "tga_attention_decode_split: max_ctx=%d outside 1..2048 (tga_attention_split_plan reports 0 splits)", max_ctx);
  AttnArgs a = {};
  a.q = q; a.k = k; a.v = v; a.cache_k = (_Float16*)cache_k; a.cache_v = (_Float16*)cache_v; a.part = partials; a.st = (DecodeState*)state;
  a.n_heads = n_heads; a.n_kv = n_kv_heads; a.hd = head_dim; a.max_ctx = max_ctx; a.nsplit = ns; a.split_shift = 6;
  a.rope = rope_table; a.scale = 1.0f / sqrtf((float)head_dim);
  a.q_norm = q_norm_weight; a.k_norm = k_norm_weight; a.norm_eps = norm_eps;
  const int norm = q_norm_weight ? (norm_per_head ? 2 : 1) : 0;
  const unsigned grid = (unsigned)(n_heads * ns);
  hipStream_t s = (hipStream_t)stream;
#define TGA_SPLIT1_N(HD8, IT, NW) do { if (norm == 0) attn_split1_kernel<HD8, IT, NW, 0><<<grid, NW * 64, 0, s>>>(a); else if (norm == 1) attn_split1_kernel<HD8, IT, NW, 1><<<grid, NW * 64, 0, s>>>(a); \
    else attn_split1_kernel<HD8, IT, NW, 2><<<grid, NW * 64, 0, s>>>(a); } while (0)
#define TGA_SPLIT1_W(HD8, NW) do { if (it == 1) TGA_SPLIT1_N(HD8, 1, NW); else if (it == 2) TGA_SPLIT1_N(HD8, 2, NW); else if (it == 3) TGA_SPLIT1_N(HD8, 3, NW); else TGA_SPLIT1_N(HD8, 4, NW); } while (0)
#define TGA_SPLIT1(HD8) do { const int nw = attn_split1_waves(); if (nw == 4) TGA_SPLIT1_W(HD8, 4); else if (nw == 16) TGA_SPLIT1_W(HD8, 16); else TGA_SPLIT1_W(HD8, 8); } while (0)
  if (head_dim == 64) TGA_SPLIT1(8); else if (head_dim == 128) TGA_SPLIT1(16); else TGA_SPLIT1(32);
#undef TGA_SPLIT1_N
#undef TGA_SPLIT1_W
#undef TGA_SPLIT1
  TGA_LAUNCH_CHECK();
  return 0;
}
int tga_attention_decode_split(const float* q, const float* k, const float* v, void* cache_k, void* cache_v, float* partials, const void* state,
                               int n_heads, int n_kv_heads, int head_dim, int max_ctx, const float* rope_table, void* stream) {
  return attention_decode_split(q, k, v, nullptr, nullptr, 0.f, 0, cache_k, cache_v, partials, state, n_heads, n_kv_heads, head_dim, max_ctx, rope_table, stream);
}
int tga_attention_decode_split_normed(const float* q, const float* k, const float* v, const float* q_norm_weight, const float* k_norm_weight, float norm_eps, int norm_per_head,
                                      void* cache_k, void* cache_v, float* partials, const void* state,
                                      int n_heads, int n_kv_heads, int head_dim, int max_ctx, const float* rope_table, void* stream) {
  return attention_decode_split(q, k, v, q_norm_weight, k_norm_weight, norm_eps, norm_per_head, cache_k, cache_v, partials, state, n_heads, n_kv_heads, head_dim, max_ctx, rope_table, stream);
}

int tga_attention_decode_batched(int batch, const float* q, const float* k, const float* v, const float* q_norm_weight, const float* k_norm_weight, float norm_eps,
                                 int norm_per_head, void* cache_k, void* cache_v, float* partials, const void* state,
                                 int n_heads, int n_kv_heads, int head_dim, int max_ctx, const float* rope_table, void* out_f16, float* out_f32, void* stream) {
  return attention_launch(0, batch, q, k, v, q_norm_weight, k_norm_weight, norm_eps, norm_per_head, cache_k, cache_v, partials, state, n_heads, n_kv_heads, head_dim, max_ctx,
                          rope_table, out_f16, out_f32, 0, stream);
}

int tga_attention_prefill_chunk(int rows, const float* q, const float* k, const float* v, const float* q_norm_weight, const float* k_norm_weight, float norm_eps,
                                int norm_per_head, void* cache_k, void* cache_v, float* partials, const void* state,
                                int n_heads, int n_kv_heads, int head_dim, int max_ctx, const float* rope_table, void* out_f16, float* out_f32, void* stream) {
  TGA_REQUIRE(rows >= 1 && rows <= 128, "tga_attention_prefill_chunk: rows=%d", rows);
  return attention_launch(1, rows, q, k, v, q_norm_weight, k_norm_weight, norm_eps, norm_per_head, cache_k, cache_v, partials, state, n_heads, n_kv_heads, head_dim, max_ctx,
                          rope_table, out_f16, out_f32, 0, stream);
}

int tga_attention_prefill_chunk_staged(int rows, const float* q, const float* k, const float* v, const float* q_norm_weight, const float* k_norm_weight, float norm_eps,
                                       int norm_per_head, void* cache_k, void* cache_v, float* partials, const void* state,
                                       int n_heads, int n_kv_heads, int head_dim, int max_ctx, const float* rope_table, void* out_rows_staged, int consumer_type, void* stream) {
  TGA_REQUIRE(rows >= 17 && rows <= 128 && consumer_type != 0, "tga_attention_prefill_chunk_staged: rows=%d (17..128), consumer type %d", rows, consumer_type);
  return attention_launch(1, rows, q, k, v, q_norm_weight, k_norm_weight, norm_eps, norm_per_head, cache_k, cache_v, partials, state, n_heads, n_kv_heads, head_dim, max_ctx,
                          rope_table, out_rows_staged, nullptr, consumer_type, stream);
}

int tga_chunk_advance(void* state, const int32_t* prompt, int rows, int32_t* tokens, int max_ctx, void* stream) {
  TGA_REQUIRE(state && prompt && tokens && rows >= 1 && rows <= 128 && max_ctx >= 1, "tga_chunk_advance: null pointer or rows=%d outside 1..128", rows);
  chunk_advance_kernel<<<1, 128, 0, (hipStream_t)stream>>>((DecodeState*)state, prompt, rows, tokens, max_ctx);
  TGA_LAUNCH_CHECK();
  return 0;
}

int tga_attention_decode(const float* q, const float* k, const float* v, void* cache_k, void* cache_v, float* partials, const void* state,
                         int n_heads, int n_kv_heads, int head_dim, int max_ctx, const float* rope_table, void* out_f16, float* out_f32, int stage_type, void* stream) {
  return tga_attention_decode_normed(q, k, v, nullptr, nullptr, 0.f, 0, cache_k, cache_v, partials, state, n_heads, n_kv_heads, head_dim, max_ctx, rope_table,
                                     out_f16, out_f32, stage_type, stream);
}

int tga_argmax_step(const float* logits, int n, float* scratch_v, int* scratch_i, void* state, const int* prompt, int* out_tokens, int max_tokens, void* stream) {
  TGA_REQUIRE(logits && scratch_v && scratch_i && state && prompt, "tga_argmax_step: null pointer");
  TGA_REQUIRE(n > 0, "tga_argmax_step: n=%d", n);
  const int np = 256;
  argmax_partial_kernel<<<np, 256, 0, (hipStream_t)stream>>>(logits, n, scratch_v, scratch_i);
  TGA_LAUNCH_CHECK();
  argmax_final_kernel<<<1, 256, 0, (hipStream_t)stream>>>(scratch_v, scratch_i, np, (DecodeState*)state, prompt, out_tokens, max_tokens);
  TGA_LAUNCH_CHECK();
  return 0;
}

int tga_argmax_rows_step(const float* logits, int batch, int n, void* state, const int32_t* prompts, int prompt_stride, int32_t* tokens, int32_t* out_tokens,
                         int max_steps, void* stream) {
  TGA_REQUIRE(state && prompts && tokens && batch >= 1 && (!logits || n > 0), "tga_argmax_rows_step: null pointer or empty rows");
  argmax_rows_kernel<<<batch, 1024, 0, (hipStream_t)stream>>>(logits, n, (const DecodeState*)state, prompts, prompt_stride, tokens, out_tokens, max_steps, batch);
  TGA_LAUNCH_CHECK();
  advance_batch_kernel<<<1, 1, 0, (hipStream_t)stream>>>((DecodeState*)state, logits != nullptr);
  TGA_LAUNCH_CHECK();
  return 0;
}

int tga_advance_prompt(void* state, const int* prompt, void* stream) {
  TGA_REQUIRE(state && prompt, "tga_advance_prompt: null pointer");
  advance_prompt_kernel<<<1, 1, 0, (hipStream_t)stream>>>((DecodeState*)state, prompt);
  TGA_LAUNCH_CHECK();
  return 0;
}

}  // extern "C"
