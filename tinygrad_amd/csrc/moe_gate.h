// Expert gating + pairwise top-k of one token on one wave (tinygrad/llm/model.py:35-41, 110-121); shared by the MoE kernels and the
// expert GEMV that routes for itself.
#pragma once
#include "common.h"

// scores per ExpertGating (model.py:9-13, 116-121): 1 SOFTMAX, 2 SIGMOID, 3 SOFTMAX_WEIGHT (softmax over the selected logits),
// 4 SQRT_SOFTPLUS.  Top-k by pairwise rank exactly as pairwise_topk (model.py:35-41): rank_i = #{j: s_i > s_j or (s_i == s_j and
// i < j)}; the k highest ranks are emitted in ASCENDING rank order (the largest last), so among equal scores the lower index
// ranks higher.  Runs on ONE wave (lane = threadIdx.x & 63 of the calling wave); lg may live in LDS or global memory, sc is
// n_experts floats of LDS, tmp 192 floats of LDS.  The caller separates the call from earlier LDS writes with a barrier.
// bias (optional, n_experts floats): the expert selection bias of model.py:113, 123 - experts are ranked by score + bias, the weights are
// gathered from the unbiased scores; scb is then n_experts more floats of LDS for the biased scores (without a bias pass scb = sc).
__device__ __forceinline__ void gate_topk_wave(const float* lg, int n_experts, int k, int gating, int norm_topk, float scale,
                                               int* __restrict__ sel, float* __restrict__ probs, float* sc, float* tmp, int lane,
                                               const float* bias = nullptr, float* scb = nullptr) {
  int* s_sel = (int*)tmp; float* s_p = tmp + 64; float* s_q = tmp + 128;
  if (!bias) scb = sc;
  if (gating == 1 && norm_topk && !bias) { gating = 3; norm_topk = 0; }   // model.py:116-117 fast path (only without a selection bias)
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
    if (bias) scb[i] = s + bias[i];
  }
  s_sel[lane] = 0; s_p[lane] = 0.f;                       // a slot no rank lands in (NaN scores compare false with everything) selects expert 0, like the reference's zero-filled scatter
  __builtin_amdgcn_wave_barrier(); __builtin_amdgcn_s_waitcnt(0xc07f);   // this wave's LDS writes are visible to its own lanes
  for (int i = lane; i < n_experts; i += 64) {
    const float si = scb[i];
    int rank = 0;
    for (int j = 0; j < n_experts; j++) { const float sj = scb[j]; rank += (si > sj) || (si == sj && i < j); }
    const int slot = rank - (n_experts - k);
    if (slot >= 0) { s_sel[slot] = i; s_p[slot] = sc[i]; }
  }
  __builtin_amdgcn_wave_barrier(); __builtin_amdgcn_s_waitcnt(0xc07f);
  float p = lane < k ? s_p[lane] : 0.f;
  if (gating == 3 && lane < k) {                          // softmax over the selected logits
    float m2 = -INFINITY; for (int j = 0; j < k; j++) m2 = fmaxf(m2, s_p[j]);
    float z = 0.f; for (int j = 0; j < k; j++) z += expf(s_p[j] - m2);
    p = expf(p - m2) * (1.0f / z);
  }
  s_q[lane] = p;
  __builtin_amdgcn_wave_barrier(); __builtin_amdgcn_s_waitcnt(0xc07f);
  if (lane < k) {
    if (norm_topk) { float z = 0.f; for (int j = 0; j < k; j++) z += s_q[j]; p = p / z; }
    sel[lane] = s_sel[lane];
    probs[lane] = p * scale;
  }
}

