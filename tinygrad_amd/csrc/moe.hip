// MoE routing pieces of the decode path (tinygrad/llm/model.py:110-135): expert gating + pairwise top-k, and the weighted
// sum over the selected experts' outputs.
#include "coherent.h"
#include "moe_gate.h"

// One workgroup (64 threads) per token.
__global__ __launch_bounds__(64) void moe_gate_kernel(const float* __restrict__ logits, const float* __restrict__ bias, int n_experts, int k, int gating, int norm_topk,
                                                      float scale, int* __restrict__ sel, float* __restrict__ probs) {
  extern __shared__ float sc[];                         // n_experts scores (+ n_experts biased scores when there is a selection bias)
  __shared__ float tmp[192];
  const int t = blockIdx.x;
  gate_topk_wave(logits + (size_t)t * n_experts, n_experts, k, gating, norm_topk, scale, sel + (size_t)t * k, probs + (size_t)t * k, sc, tmp, threadIdx.x,
                 bias, sc + n_experts);
}

// Router of one token in one launch (tinygrad/llm/model.py:112-121 with the block's ffn_norm, :150): h = RMSNorm(x) * weight rounded
// to fp16 (also written to xn_out for the expert GEMVs that follow), logits = h @ Wr^T for a dense fp16 router weight (n_experts,
// dim), then gating + top-k as above.  Workgroup b (4 waves) takes rows 4b .. 4b+3, one per wave, and normalises the row for
// itself (the row is a few KB); the last workgroup to publish its logits (arrival counter behind them) does the gating.
#define ROUTER_THREADS 256
#define ROUTER_XP 2       // 8-value pieces of the activation row per thread kept in registers (rows up to 4096 values)
#define ROUTER_PF 4       // 16-byte weight pieces per lane requested before the norm (rows up to 2048 values are fully in flight)
__global__ __launch_bounds__(ROUTER_THREADS) void moe_router_kernel(const float* __restrict__ x, const float* __restrict__ norm_w, float eps, const _Float16* __restrict__ wr,
                                                                    int dim, int n_experts, int k, int gating, int norm_topk, float scale,
                                                                    _Float16* __restrict__ xn_out, float* logits_ws, int* __restrict__ sel, float* __restrict__ probs) {
  extern __shared__ float dyn[];                        // logits[n_experts] | scores[n_experts] | fp16 row [dim]
  float* lg = dyn; float* sc = dyn + n_experts;
  _Float16* xn = (_Float16*)(dyn + 2 * n_experts);
  __shared__ float red[ROUTER_THREADS / 64];
  __shared__ float tmp[192];
  __shared__ int last_flag;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  // blockIdx.y: the token (logits-only launches over several rows: tga_moe_router_rows)
  x += (size_t)blockIdx.y * dim; logits_ws += (size_t)blockIdx.y * n_experts;
  if (xn_out) xn_out += (size_t)blockIdx.y * dim;
  const int row = blockIdx.x * 4 + wave, rowc = row < n_experts ? row : n_experts - 1;
  const int np = dim / 8;                               // 16-byte pieces per row
  const _Float16* wrow = wr + (size_t)rowc * dim;
  u32x4 wv[ROUTER_PF];
#pragma unroll
  for (int j = 0; j < ROUTER_PF; j++) { const int p = lane + 64 * j; wv[j] = *(const u32x4*)(wrow + 8 * (p < np ? p : np - 1)); }
  // the row (and the norm weight) in 8-value pieces: the first ROUTER_XP pieces of a thread are requested in one batch and stay in
  // registers for both passes (a load per loop iteration would be a memory round trip per iteration)
  f32x4 xa[ROUTER_XP][2], wa[ROUTER_XP][2];
#pragma unroll
  for (int j = 0; j < ROUTER_XP; j++) {
    const int p = tid + ROUTER_THREADS * j, pc = p < np ? p : np - 1;
    xa[j][0] = ((const f32x4*)x)[2 * pc]; xa[j][1] = ((const f32x4*)x)[2 * pc + 1];
    if (norm_w) { wa[j][0] = ((const f32x4*)norm_w)[2 * pc]; wa[j][1] = ((const f32x4*)norm_w)[2 * pc + 1]; }
  }
  float s = 0.f;
#pragma unroll
  for (int j = 0; j < ROUTER_XP; j++) {
    if (tid + ROUTER_THREADS * j < np) {
#pragma unroll
      for (int h = 0; h < 2; h++) s += xa[j][h].x * xa[j][h].x + xa[j][h].y * xa[j][h].y + xa[j][h].z * xa[j][h].z + xa[j][h].w * xa[j][h].w;
    }
  }
  for (int e = 8 * ROUTER_THREADS * ROUTER_XP + tid; e < dim; e += ROUTER_THREADS) { const float v = x[e]; s += v * v; }
  s = wave_sum(s);
  if (lane == 0) red[wave] = s;
  __syncthreads();
  const float nscale = norm_w ? 1.0f / sqrtf((red[0] + red[1] + red[2] + red[3]) / (float)dim + eps) : 1.f;
#pragma unroll
  for (int j = 0; j < ROUTER_XP; j++) {
    const int p = tid + ROUTER_THREADS * j;
    if (p < np) {
      float v[8] = {xa[j][0].x, xa[j][0].y, xa[j][0].z, xa[j][0].w, xa[j][1].x, xa[j][1].y, xa[j][1].z, xa[j][1].w};
      if (norm_w) {
        const float w[8] = {wa[j][0].x, wa[j][0].y, wa[j][0].z, wa[j][0].w, wa[j][1].x, wa[j][1].y, wa[j][1].z, wa[j][1].w};
#pragma unroll
        for (int i = 0; i < 8; i++) v[i] = (v[i] * nscale) * w[i];
      }
      const u32x4 h = {f2h_bits(v[0]) | (f2h_bits(v[1]) << 16), f2h_bits(v[2]) | (f2h_bits(v[3]) << 16),
                       f2h_bits(v[4]) | (f2h_bits(v[5]) << 16), f2h_bits(v[6]) | (f2h_bits(v[7]) << 16)};
      *(u32x4*)(xn + 8 * p) = h;
      if (xn_out && blockIdx.x == 0) *(u32x4*)(xn_out + 8 * p) = h;
    }
  }
  for (int e = 8 * ROUTER_THREADS * ROUTER_XP + tid; e < dim; e += ROUTER_THREADS) {
    const _Float16 h = (_Float16)(norm_w ? (x[e] * nscale) * norm_w[e] : x[e]);
    xn[e] = h;
    if (xn_out && blockIdx.x == 0) xn_out[e] = h;
  }
  __syncthreads();
  float acc = 0.f;
#pragma unroll
  for (int j = 0; j < ROUTER_PF; j++) {
    const int p = lane + 64 * j;
    if (p < np) { const u32x4 xv = *(const u32x4*)(xn + 8 * p); acc = dot2(wv[j].w, xv.w, dot2(wv[j].z, xv.z, dot2(wv[j].y, xv.y, dot2(wv[j].x, xv.x, acc)))); }
  }
  for (int p = lane + 64 * ROUTER_PF; p < np; p += 64) {
    const u32x4 xv = *(const u32x4*)(xn + 8 * p), w4 = *(const u32x4*)(wrow + 8 * p);
    acc = dot2(w4.w, xv.w, dot2(w4.z, xv.z, dot2(w4.y, xv.y, dot2(w4.x, xv.x, acc))));
  }
  acc = wave_sum(acc);
  if (k == 0) {                                         // logits only: the consumer (a later launch) gates for itself
    if (lane == 0 && row < n_experts) logits_ws[row] = acc;
    return;
  }
  if (lane == 0 && row < n_experts) cst(&logits_ws[row], acc);
  stores_done();
  __syncthreads();
  int* counter = (int*)(logits_ws + n_experts);
  if (tid == 0) {
    const int prev = __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    last_flag = (prev == (int)gridDim.x - 1);
    if (prev == (int)gridDim.x - 1) __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // ready for the next launch
  }
  __syncthreads();
  if (!last_flag) return;
  for (int i = tid; i < n_experts; i += ROUTER_THREADS) lg[i] = cld(&logits_ws[i]);
  __syncthreads();
  if (wave == 0) gate_topk_wave(lg, n_experts, k, gating, norm_topk, scale, sel, probs, sc, tmp, lane);
}

// out[t, :] = resid[t, :] + sum_s probs[t, s] * y[t, s, :]     ((x_down * probs).sum(axis=2), model.py:130, plus the block residual :150)
__global__ __launch_bounds__(256) void moe_combine_kernel(const float* __restrict__ y, const float* __restrict__ probs, const float* __restrict__ resid,
                                                          int k, int dim, float* __restrict__ out) {
  const int t = blockIdx.y;
  const int d = blockIdx.x * 256 + threadIdx.x;
  if (d >= dim) return;
  float acc = resid ? resid[(size_t)t * dim + d] : 0.f;
  for (int s = 0; s < k; s++) acc += probs[(size_t)t * k + s] * y[((size_t)t * k + s) * dim + d];
  out[(size_t)t * dim + d] = acc;
}

extern "C" {

int tga_moe_gate(const float* logits, int n_tokens, int n_experts, int k, int gating, int norm_topk_prob, float scale,
                 int32_t* sel, float* probs, void* stream) {
  TGA_REQUIRE(logits && sel && probs, "tga_moe_gate: null pointer");
  TGA_REQUIRE(n_tokens >= 1 && n_experts >= 1 && n_experts <= 4096 && k >= 1 && k <= 64 && k <= n_experts, "tga_moe_gate: bad geometry (k <= 64, n_experts <= 4096)");
  TGA_REQUIRE(gating >= 1 && gating <= 4, "tga_moe_gate: unknown ExpertGating %d", gating);
  moe_gate_kernel<<<n_tokens, 64, n_experts * sizeof(float), (hipStream_t)stream>>>(logits, nullptr, n_experts, k, gating, norm_topk_prob, scale, sel, probs);
  TGA_LAUNCH_CHECK();
  return 0;
}

int tga_moe_gate_biased(const float* logits, const float* selection_bias, int n_tokens, int n_experts, int k, int gating, int norm_topk_prob, float scale,
                        int32_t* sel, float* probs, void* stream) {
  TGA_REQUIRE(logits && selection_bias && sel && probs, "tga_moe_gate_biased: null pointer");
  TGA_REQUIRE(n_tokens >= 1 && n_experts >= 1 && n_experts <= 4096 && k >= 1 && k <= 64 && k <= n_experts, "tga_moe_gate_biased: bad geometry (k <= 64, n_experts <= 4096)");
  TGA_REQUIRE(gating >= 1 && gating <= 4, "tga_moe_gate_biased: unknown ExpertGating %d", gating);
  moe_gate_kernel<<<n_tokens, 64, 2 * n_experts * sizeof(float), (hipStream_t)stream>>>(logits, selection_bias, n_experts, k, gating, norm_topk_prob, scale, sel, probs);
  TGA_LAUNCH_CHECK();
  return 0;
}

int tga_moe_router(const float* x, const float* norm_weight, float norm_eps, const void* router_w_f16, int dim, int n_experts, int k,
                   int gating, int norm_topk_prob, float scale, void* xn_out_f16, float* logits_ws, int32_t* sel, float* probs, void* stream) {
  TGA_REQUIRE(x && router_w_f16 && logits_ws && (k == 0 || (sel && probs)), "tga_moe_router: null pointer");
  TGA_REQUIRE(dim >= 8 && dim % 8 == 0 && dim <= 16384 && ((uintptr_t)router_w_f16 & 15) == 0, "tga_moe_router: dim=%d must be a multiple of 8, at most 16384, with a 16-byte aligned weight", dim);
  TGA_REQUIRE((((uintptr_t)x | (uintptr_t)norm_weight | (uintptr_t)xn_out_f16) & 15) == 0, "tga_moe_router: x, norm_weight and xn_out must be 16-byte aligned");
  TGA_REQUIRE(n_experts >= 1 && n_experts <= 1024 && k >= 0 && k <= 64 && k <= n_experts, "tga_moe_router: bad geometry (k <= 64, n_experts <= 1024)");
  TGA_REQUIRE(gating >= 1 && gating <= 4, "tga_moe_router: unknown ExpertGating %d", gating);
  moe_router_kernel<<<(n_experts + 3) / 4, ROUTER_THREADS, 2 * n_experts * sizeof(float) + (size_t)dim * 2, (hipStream_t)stream>>>(
      x, norm_weight, norm_eps, (const _Float16*)router_w_f16, dim, n_experts, k, gating, norm_topk_prob, scale, (_Float16*)xn_out_f16, logits_ws, sel, probs);
  TGA_LAUNCH_CHECK();
  return 0;
}

int tga_moe_router_rows(const float* x, const float* norm_weight, float norm_eps, const void* router_w_f16, int rows, int dim, int n_experts,
                        void* xn_out_f16, float* logits, void* stream) {
  TGA_REQUIRE(x && router_w_f16 && logits, "tga_moe_router_rows: null pointer");
  TGA_REQUIRE(rows >= 1 && rows <= 65535 && dim >= 8 && dim % 8 == 0 && dim <= 16384 && ((uintptr_t)router_w_f16 & 15) == 0,
              "tga_moe_router_rows: rows=%d, dim=%d must be a multiple of 8, at most 16384, with a 16-byte aligned weight", rows, dim);
  TGA_REQUIRE((((uintptr_t)x | (uintptr_t)norm_weight | (uintptr_t)xn_out_f16) & 15) == 0, "tga_moe_router_rows: x, norm_weight and xn_out must be 16-byte aligned");
  TGA_REQUIRE(n_experts >= 1 && n_experts <= 1024, "tga_moe_router_rows: n_experts <= 1024");
  moe_router_kernel<<<dim3((n_experts + 3) / 4, rows), ROUTER_THREADS, 2 * n_experts * sizeof(float) + (size_t)dim * 2, (hipStream_t)stream>>>(
      x, norm_weight, norm_eps, (const _Float16*)router_w_f16, dim, n_experts, 0, 1, 0, 1.f, (_Float16*)xn_out_f16, logits, nullptr, nullptr);
  TGA_LAUNCH_CHECK();
  return 0;
}

int tga_moe_combine(const float* y, const float* probs, const float* resid, int n_tokens, int k, int dim, float* out, void* stream) {
  TGA_REQUIRE(y && probs && out, "tga_moe_combine: null pointer");
  TGA_REQUIRE(n_tokens >= 1 && k >= 1 && dim >= 1, "tga_moe_combine: bad geometry");
  moe_combine_kernel<<<dim3((dim + 255) / 256, n_tokens), 256, 0, (hipStream_t)stream>>>(y, probs, resid, k, dim, out);
  TGA_LAUNCH_CHECK();
  return 0;
}

}  // extern "C"
