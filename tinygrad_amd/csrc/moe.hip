// MoE routing pieces of the decode path (tinygrad/llm/model.py:110-135): expert gating + pairwise top-k, and the weighted
// sum over the selected experts' outputs.
#include "common.h"
#include "host.h"

// One workgroup (64 threads) per token.  scores per ExpertGating (model.py:9-13, 116-121): 1 SOFTMAX, 2 SIGMOID,
// 3 SOFTMAX_WEIGHT (softmax over the selected logits), 4 SQRT_SOFTPLUS.  Top-k by pairwise rank exactly as pairwise_topk
// (model.py:35-41): rank_i = #{j: s_i > s_j or (s_i == s_j and i < j)}; the k highest ranks are emitted in ASCENDING rank
// order (the largest last), so among equal scores the lower index ranks higher.
__global__ __launch_bounds__(64) void moe_gate_kernel(const float* __restrict__ logits, int n_experts, int k, int gating, int norm_topk,
                                                      float scale, int* __restrict__ sel, float* __restrict__ probs) {
  extern __shared__ float sc[];                         // n_experts scores
  const int t = blockIdx.x, lane = threadIdx.x;
  const float* lg = logits + (size_t)t * n_experts;
  if (gating == 1 && norm_topk) { gating = 3; norm_topk = 0; }   // model.py:116-117 fast path (no selection bias)
  float mx = -INFINITY;
  for (int i = lane; i < n_experts; i += 64) mx = fmaxf(mx, lg[i]);
  mx = wave_max(mx);
  float sum = 0.f;
  if (gating == 1) { for (int i = lane; i < n_experts; i += 64) sum += expf(lg[i] - mx); sum = wave_sum(sum); }
  for (int i = lane; i < n_experts; i += 64) {
    const float v = lg[i];
    float s;
    if (gating == 3) s = v;
    else if (gating == 1) s = expf(v - mx) * (1.0f / sum);
    else if (gating == 2) s = 1.0f / (1.0f + expf(-v));
    else s = sqrtf(log1pf(expf(v)));
    sc[i] = s;
  }
  __syncthreads();
  __shared__ int s_sel[64]; __shared__ float s_p[64];
  for (int i = lane; i < n_experts; i += 64) {
    const float si = sc[i];
    int rank = 0;
    for (int j = 0; j < n_experts; j++) { const float sj = sc[j]; rank += (si > sj) || (si == sj && i < j); }
    const int slot = rank - (n_experts - k);
    if (slot >= 0) { s_sel[slot] = i; s_p[slot] = si; }
  }
  __syncthreads();
  __shared__ float s_q[64];
  float p = lane < k ? s_p[lane] : 0.f;
  if (gating == 3 && lane < k) {                          // softmax over the selected logits
    float m2 = -INFINITY; for (int j = 0; j < k; j++) m2 = fmaxf(m2, s_p[j]);
    float z = 0.f; for (int j = 0; j < k; j++) z += expf(s_p[j] - m2);
    p = expf(p - m2) * (1.0f / z);
  }
  s_q[lane] = p;
  __syncthreads();
  if (lane < k) {
    if (norm_topk) { float z = 0.f; for (int j = 0; j < k; j++) z += s_q[j]; p = p / z; }
    sel[(size_t)t * k + lane] = s_sel[lane];
    probs[(size_t)t * k + lane] = p * scale;
  }
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
  moe_gate_kernel<<<n_tokens, 64, n_experts * sizeof(float), (hipStream_t)stream>>>(logits, n_experts, k, gating, norm_topk_prob, scale, sel, probs);
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
