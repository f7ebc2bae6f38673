// Decode-step neighbours of the quantized linears (batch 1): embedding row dequant, RMSNorm, RoPE + KV append + GQA attention
// (flash-decoding over 64-position splits), split combine, argmax / token bookkeeping.
// They restate, for one token, what tinygrad/llm/model.py:167-204 (_attention), :144-151 (block), :358-364 (forward) compute.
// The position and token live in device memory so that one captured launch sequence can be replayed for every token
// (the reference binds symbolic start_pos into a replayed JIT graph: tinygrad/llm/model.py:464-484).
#include "qfmt.h"
#include "decode.h"

// ---------------------------------------------------------------------------------------------- embedding (Q4_0 / F16 / F32 row)
// token_embd(tokens).float() for one token: tinygrad/llm/model.py:359.  The table stays in GGUF blocks; only the row is dequantized.
__global__ __launch_bounds__(256) void embed_row_kernel(const uint8_t* __restrict__ table, int ggml_type, int dim, const DecodeState* st, float* __restrict__ out) {
  const int tok = st->token;
  if (ggml_type == GGML_Q4_0) {
    const uint8_t* row = table + (size_t)tok * (dim / 32) * 18;
    for (int e = threadIdx.x; e < dim; e += 256) {
      const uint8_t* b = row + (e >> 5) * 18; const int j = e & 31;
      const float d = h2f_bits(ld2(b));
      const int q = (j < 16) ? (b[2 + j] & 0xF) : (b[2 + j - 16] >> 4);
      out[e] = (float)(q - 8) * d;
    }
  } else if (ggml_type == GGML_Q8_0) {
    const uint8_t* row = table + (size_t)tok * (dim / 32) * 34;
    for (int e = threadIdx.x; e < dim; e += 256) {
      const uint8_t* b = row + (e >> 5) * 34;
      out[e] = h2f_bits(ld2(b)) * (float)(int8_t)b[2 + (e & 31)];
    }
  } else if (ggml_type == GGML_F16) {
    const uint16_t* row = (const uint16_t*)table + (size_t)tok * dim;
    for (int e = threadIdx.x; e < dim; e += 256) out[e] = h2f_bits(row[e]);
  } else {
    const float* row = (const float*)table + (size_t)tok * dim;
    for (int e = threadIdx.x; e < dim; e += 256) out[e] = row[e];
  }
}

// ---------------------------------------------------------------------------------------------- RMSNorm
// nn.RMSNorm (tinygrad/nn/__init__.py:296-304): x * rsqrt(mean(x^2) + eps), then * weight.  Output fp16 (the activation the
// dequant-GEMV multiplies) and optionally fp32.
__global__ __launch_bounds__(1024) void rmsnorm_kernel(const float* __restrict__ x, const float* __restrict__ w, int dim, float eps,
                                                       _Float16* __restrict__ out16, float* __restrict__ out32, int stage_fmt, int stage_nu) {
  __shared__ float red[16];
  float s = 0.f;
  for (int e = threadIdx.x; e < dim; e += blockDim.x) { const float v = x[e]; s += v * v; }
  s = wave_sum(s);
  const int wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  if ((threadIdx.x & 63) == 0) red[wave] = s;
  __syncthreads();
  float tot = 0.f;
  for (int i = 0; i < nw; i++) tot += red[i];
  const float scale = 1.0f / sqrtf(tot / (float)dim + eps);
  for (int e = threadIdx.x; e < dim; e += blockDim.x) {
    const float v = (x[e] * scale) * w[e];
    if (out16) out16[stage_fmt ? staged_pos(stage_fmt, e, stage_nu) : e] = (_Float16)v;
    if (out32) out32[e] = v;
  }
}

// ---------------------------------------------------------------------------------------------- RoPE + KV append + attention
// One workgroup per (kv head, 64-position split); wave w of the workgroup serves query head kvh * group + w (group <= 4 waves
// per pass).  q, k are rotated with the half-split rule of apply_rope (tinygrad/llm/model.py:29-33) using the caller's
// freqs_cis table [max_ctx][hd] = cos half | sin half (precompute_freqs_cis, model.py:16-19); the split that contains `pos` writes the rotated k and v into the fp16 cache.
// Scores: lane <-> position, softmax partials per split (max, sum, weighted V) go to `part` for the combine kernel.
struct AttnArgs {
  const float* q; const float* k; const float* v;     // this token's projections: [n_heads*hd], [n_kv*hd], [n_kv*hd]
  _Float16* cache_k; _Float16* cache_v;                // [n_kv][max_ctx][hd]
  float* part;                                         // [n_heads][nsplit][hd + 2], then n_kv int32 arrival counters (zero between launches)
  const DecodeState* st;
  int n_heads, n_kv, hd, max_ctx, nsplit;
  const float* rope;                                   // [max_ctx][hd]: cos(pos * f_i) for i < hd/2, then sin(pos * f_i)
  float scale;
  _Float16* out16; float* out32;                       // attention output [n_heads*hd]
  int stage_fmt, stage_nu;                             // != 0: out16 in the staged order of the consuming linear
};

// 8 fp16 values (one 16-byte piece) of row `p` of a cache plane; the row of the token being processed comes from LDS (fp32
// values rounded to fp16 exactly like the copy that goes into the cache)
__device__ __forceinline__ u32x4 kv_piece(const _Float16* plane_row0, int hd, int p, int pos, int piece, const float* cur) {
  if (p == pos) {
    const float* c = cur + piece * 8;
    u32x4 r = {f2h_bits(c[0]) | (f2h_bits(c[1]) << 16), f2h_bits(c[2]) | (f2h_bits(c[3]) << 16),
               f2h_bits(c[4]) | (f2h_bits(c[5]) << 16), f2h_bits(c[6]) | (f2h_bits(c[7]) << 16)};
    return r;
  }
  return *(const u32x4*)(plane_row0 + (size_t)p * hd + piece * 8);
}

// HD8 = head_dim / 8 (16-byte pieces per row).  Workgroup = (kv head, 64-position split), wave w serves query heads w, w+4, ...
// of the group.  K: lane <-> position (whole row in registers).  V: RPI = 64 / HD8 rows per load instruction, lane = (row-in-
// instruction, piece); both tiles are requested before any arithmetic so their latencies overlap.
// The last workgroup of a kv head to finish (device-scope arrival counter) merges that head group's split partials.
template <int HD8>
__global__ __launch_bounds__(256) void attn_decode_kernel(const AttnArgs a) {
  constexpr int HD = HD8 * 8, RPI = 64 / HD8, NVI = 64 / RPI;   // rows per V instruction, V instructions per 64 rows
  const int kvh = blockIdx.x, split = blockIdx.y;
  const int pos = a.st->pos;
  const int p0 = split * 64;
  if (p0 > pos) return;                                 // nothing cached in this split yet
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int half = HD >> 1, group = a.n_heads / a.n_kv;
  __shared__ float qs[4][HD];                           // rotated queries of the 4 heads in flight
  __shared__ float ks[HD], vs[HD];                      // rotated key / value of this token
  __shared__ int last_flag;
  for (int i = threadIdx.x; i < half; i += 256) {
    const float c = a.rope[(size_t)pos * HD + i], s = a.rope[(size_t)pos * HD + half + i];
    const float x1 = a.k[kvh * HD + i], x2 = a.k[kvh * HD + half + i];
    ks[i] = x1 * c - x2 * s; ks[half + i] = x2 * c + x1 * s;
  }
  for (int i = threadIdx.x; i < HD; i += 256) vs[i] = a.v[kvh * HD + i];
  __syncthreads();
  const _Float16* krow0 = a.cache_k + (size_t)kvh * a.max_ctx * HD;
  const _Float16* vrow0 = a.cache_v + (size_t)kvh * a.max_ctx * HD;
  if ((pos >> 6) == split) {                            // owner split appends this token to the cache
    for (int i = threadIdx.x; i < HD; i += 256) {
      a.cache_k[((size_t)kvh * a.max_ctx + pos) * HD + i] = (_Float16)ks[i];
      a.cache_v[((size_t)kvh * a.max_ctx + pos) * HD + i] = (_Float16)vs[i];
    }
  }
  // K tile: lane <-> position p0 + lane;  V tile: instruction i covers rows p0 + i*RPI + lane / HD8, piece lane % HD8
  const int p = p0 + lane;
  const bool pvalid = p <= pos;
  const int pc = pvalid ? p : pos;                      // clamp to a valid row, result masked
  u32x4 kt[HD8], vt[NVI];
#pragma unroll
  for (int i = 0; i < HD8; i++) kt[i] = kv_piece(krow0, HD, pc, pos, i, ks);
  const int vr = lane / HD8, vp = lane % HD8;
#pragma unroll
  for (int i = 0; i < NVI; i++) { const int r = p0 + i * RPI + vr; vt[i] = kv_piece(vrow0, HD, r <= pos ? r : pos, pos, vp, vs); }

  for (int h0 = 0; h0 < group; h0 += 4) {
    const int gh = h0 + wave;
    const bool hvalid = gh < group;
    const int head = kvh * group + gh;
    if (hvalid) {
      for (int i = lane; i < half; i += 64) {
        const float c = a.rope[(size_t)pos * HD + i], s = a.rope[(size_t)pos * HD + half + i];
        const float x1 = a.q[head * HD + i], x2 = a.q[head * HD + half + i];
        qs[wave][i] = x1 * c - x2 * s; qs[wave][half + i] = x2 * c + x1 * s;
      }
    }
    __syncthreads();
    if (hvalid) {
      float acc = 0.f;
#pragma unroll
      for (int i = 0; i < HD8; i++) {
        const float* qq = &qs[wave][i * 8];
        const u32x4 kk = kt[i];
        acc += qq[0] * h2f_bits(kk.x & 0xFFFF) + qq[1] * h2f_bits(kk.x >> 16) + qq[2] * h2f_bits(kk.y & 0xFFFF) + qq[3] * h2f_bits(kk.y >> 16)
             + qq[4] * h2f_bits(kk.z & 0xFFFF) + qq[5] * h2f_bits(kk.z >> 16) + qq[6] * h2f_bits(kk.w & 0xFFFF) + qq[7] * h2f_bits(kk.w >> 16);
      }
      const float sc = pvalid ? acc * a.scale : -INFINITY;
      const float m = wave_max(sc);
      const float e = pvalid ? __expf(sc - m) : 0.f;
      const float l = wave_sum(e);
      float o[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int i = 0; i < NVI; i++) {
        const float pj = __shfl(e, i * RPI + vr, 64);          // weight of the row this lane holds in instruction i (0 beyond pos)
        const u32x4 vv = vt[i];
        o[0] += pj * h2f_bits(vv.x & 0xFFFF); o[1] += pj * h2f_bits(vv.x >> 16); o[2] += pj * h2f_bits(vv.y & 0xFFFF); o[3] += pj * h2f_bits(vv.y >> 16);
        o[4] += pj * h2f_bits(vv.z & 0xFFFF); o[5] += pj * h2f_bits(vv.z >> 16); o[6] += pj * h2f_bits(vv.w & 0xFFFF); o[7] += pj * h2f_bits(vv.w >> 16);
      }
      // sum the RPI lane groups that hold the same piece
#pragma unroll
      for (int off = HD8; off < 64; off <<= 1)
#pragma unroll
        for (int j = 0; j < 8; j++) o[j] += __shfl_xor(o[j], off, 64);
      float* po = a.part + ((size_t)head * a.nsplit + split) * (HD + 2);
      if (lane < HD8) {
#pragma unroll
        for (int j = 0; j < 8; j++) po[lane * 8 + j] = o[j];
      }
      if (lane == 0) { po[HD] = m; po[HD + 1] = l; }
    }
    __syncthreads();
  }
  // ---- merge: the last split of this kv head to arrive combines all its heads' partials ----
  int* counters = (int*)(a.part + (size_t)a.n_heads * a.nsplit * (HD + 2));
  const int ns = (pos >> 6) + 1;
  __threadfence();
  __syncthreads();
  if (threadIdx.x == 0) {
    const int prev = __hip_atomic_fetch_add(&counters[kvh], 1, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
    last_flag = (prev == ns - 1);
    if (prev == ns - 1) __hip_atomic_store(&counters[kvh], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // ready for the next launch
  }
  __syncthreads();
  if (!last_flag) return;
  __threadfence();
  // softmax weights of every (head, split) first (parallel loads), then the weighted sum with 8 partial rows in flight per thread
  __shared__ float sw[2048];                            // exp(m_s - m) / l per (head in group, split); host guarantees group * nsplit <= 2048
  for (int idx = threadIdx.x; idx < group * ns; idx += 256) {
    const int gh = idx / ns, sp = idx - gh * ns;
    const float* ph = a.part + ((size_t)(kvh * group + gh) * a.nsplit + sp) * (HD + 2);
    sw[gh * a.nsplit + sp] = __builtin_nontemporal_load(&ph[HD]);
    sw[1024 + gh * a.nsplit + sp] = __builtin_nontemporal_load(&ph[HD + 1]);
  }
  __syncthreads();
  for (int gh = wave; gh < group; gh += 4) {            // one wave per head: m, l, then normalised weights in place
    float m = -INFINITY;
    for (int sp = lane; sp < ns; sp += 64) m = fmaxf(m, sw[gh * a.nsplit + sp]);
    m = wave_max(m);
    float l = 0.f;
    for (int sp = lane; sp < ns; sp += 64) l += sw[1024 + gh * a.nsplit + sp] * __expf(sw[gh * a.nsplit + sp] - m);
    l = wave_sum(l);
    for (int sp = lane; sp < ns; sp += 64) sw[gh * a.nsplit + sp] = __expf(sw[gh * a.nsplit + sp] - m) / l;
  }
  __syncthreads();
  for (int idx = threadIdx.x; idx < group * HD; idx += 256) {
    const int gh = idx / HD, d = idx - gh * HD, head = kvh * group + gh;
    const float* ph = a.part + (size_t)head * a.nsplit * (HD + 2) + d;
    float o = 0.f;
    for (int s0 = 0; s0 < ns; s0 += 8) {
      float v[8];
#pragma unroll
      for (int j = 0; j < 8; j++) v[j] = __builtin_nontemporal_load(&ph[(size_t)min(s0 + j, ns - 1) * (HD + 2)]);
#pragma unroll
      for (int j = 0; j < 8; j++) if (s0 + j < ns) o += v[j] * sw[gh * a.nsplit + s0 + j];
    }
    if (a.out16) a.out16[a.stage_fmt ? staged_pos(a.stage_fmt, head * HD + d, a.stage_nu) : head * HD + d] = (_Float16)o;
    if (a.out32) a.out32[head * HD + d] = o;
  }
}

// ---------------------------------------------------------------------------------------------- argmax + token bookkeeping
// argmax(-1) with the reference's tie rule: the first index of the maximum (tinygrad/mixin/op.py:866-891).
__global__ __launch_bounds__(256) void argmax_partial_kernel(const float* __restrict__ logits, int n, float* __restrict__ pv, int* __restrict__ pi) {
  float best = -INFINITY; int bi = 0x7fffffff;
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
  float best = -INFINITY; int bi = 0x7fffffff;
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

// ---------------------------------------------------------------------------------------------- C-ABI
extern "C" {

int tga_embed_row(const void* table, int ggml_type, int dim, const void* state, float* out, void* stream) {
  TGA_REQUIRE(table && state && out, "tga_embed_row: null pointer");
  TGA_REQUIRE(ggml_type == GGML_Q4_0 || ggml_type == GGML_Q8_0 || ggml_type == GGML_F16 || ggml_type == GGML_F32, "tga_embed_row: unsupported table type %d", ggml_type);
  TGA_REQUIRE(dim > 0 && dim % 32 == 0, "tga_embed_row: dim=%d must be a positive multiple of 32", dim);
  embed_row_kernel<<<1, 256, 0, (hipStream_t)stream>>>((const uint8_t*)table, ggml_type, dim, (const DecodeState*)state, out);
  TGA_LAUNCH_CHECK();
  return 0;
}

// staged layout lookup shared with the GEMV host side (qgemv.hip)
static int decode_staged_fmt(int ggml_type, long long K, int* nu) {
  int fmt = -1, uw = 64;
  switch (ggml_type) {
    case GGML_Q4_0: fmt = F_Q4_0P; break; case GGML_Q8_0: fmt = F_Q8_0P; break; case GGML_Q6_K: fmt = GGML_Q6_K; break;
    case GGML_F16: fmt = GGML_F16; break; case GGML_MXFP4: fmt = GGML_MXFP4; uw = 32; break;
  }
  if (fmt < 0 || K <= 0 || K % (ggml_type == GGML_Q6_K ? 256 : 64) != 0) return -1;
  *nu = (int)(K / uw);
  return fmt;
}

int tga_rmsnorm(const float* x, const float* weight, int dim, float eps, void* out_f16, float* out_f32, int stage_type, void* stream) {
  TGA_REQUIRE(x && weight && (out_f16 || out_f32), "tga_rmsnorm: null pointer");
  TGA_REQUIRE(dim > 0, "tga_rmsnorm: dim=%d", dim);
  int sfmt = 0, snu = 0;
  if (stage_type) { sfmt = decode_staged_fmt(stage_type, dim, &snu); TGA_REQUIRE(sfmt >= 0, "tga_rmsnorm: no staged layout for type %d with K=%d", stage_type, dim); }
  rmsnorm_kernel<<<1, 1024, 0, (hipStream_t)stream>>>(x, weight, dim, eps, (_Float16*)out_f16, out_f32, sfmt, snu);
  TGA_LAUNCH_CHECK();
  return 0;
}

int tga_attention_decode(const float* q, const float* k, const float* v, void* cache_k, void* cache_v, float* partials, const void* state,
                         int n_heads, int n_kv_heads, int head_dim, int max_ctx, const float* rope_table, void* out_f16, float* out_f32, int stage_type, void* stream) {
  TGA_REQUIRE(q && k && v && cache_k && cache_v && partials && state && rope_table && (out_f16 || out_f32), "tga_attention_decode: null pointer");
  TGA_REQUIRE(n_kv_heads > 0 && n_heads % n_kv_heads == 0, "tga_attention_decode: n_heads=%d must be a multiple of n_kv_heads=%d", n_heads, n_kv_heads);
  TGA_REQUIRE(head_dim == 64 || head_dim == 128 || head_dim == 256, "tga_attention_decode: head_dim=%d must be 64, 128 or 256", head_dim);
  TGA_REQUIRE(max_ctx > 0 && (n_heads / n_kv_heads) * ((max_ctx + 63) / 64) <= 1024, "tga_attention_decode: max_ctx=%d too long for the merge table ((n_heads/n_kv_heads) * ceil(max_ctx/64) <= 1024)", max_ctx);
  AttnArgs a;
  a.q = q; a.k = k; a.v = v; a.cache_k = (_Float16*)cache_k; a.cache_v = (_Float16*)cache_v; a.part = partials; a.st = (const DecodeState*)state;
  a.n_heads = n_heads; a.n_kv = n_kv_heads; a.hd = head_dim; a.max_ctx = max_ctx; a.nsplit = (max_ctx + 63) / 64;
  a.rope = rope_table; a.scale = 1.0f / sqrtf((float)head_dim);
  a.out16 = (_Float16*)out_f16; a.out32 = out_f32;
  a.stage_fmt = 0; a.stage_nu = 0;
  if (stage_type) { a.stage_fmt = decode_staged_fmt(stage_type, (long long)n_heads * head_dim, &a.stage_nu); TGA_REQUIRE(a.stage_fmt >= 0, "tga_attention_decode: no staged layout for type %d", stage_type); }
  const dim3 grid(n_kv_heads, a.nsplit);
  hipStream_t s = (hipStream_t)stream;
  if (head_dim == 64) attn_decode_kernel<8><<<grid, 256, 0, s>>>(a);
  else if (head_dim == 128) attn_decode_kernel<16><<<grid, 256, 0, s>>>(a);
  else attn_decode_kernel<32><<<grid, 256, 0, s>>>(a);
  TGA_LAUNCH_CHECK();
  return 0;
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

int tga_advance_prompt(void* state, const int* prompt, void* stream) {
  TGA_REQUIRE(state && prompt, "tga_advance_prompt: null pointer");
  advance_prompt_kernel<<<1, 1, 0, (hipStream_t)stream>>>((DecodeState*)state, prompt);
  TGA_LAUNCH_CHECK();
  return 0;
}

}  // extern "C"
