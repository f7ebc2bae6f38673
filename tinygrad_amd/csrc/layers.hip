// All transformer blocks of one batch-1 decode step in ONE persistent launch (dense llama-family blocks, Q4_0 / Q8_0 linears).
// Restates tinygrad/llm/model.py:144-204 (TransformerBlock: attn_norm -> q/k/v -> RoPE + KV append + attention -> attn_output +
// residual -> ffn_norm -> silu(gate) * up -> down + residual) for one token, like the per-op kernels in decode.hip / qgemv1.hip,
// but without a launch per op: the grid is sized to be fully resident (2 workgroups per CU) and walks the five phases of every
// block separated by a device-wide barrier.  What that buys at batch 1, where every op is a few microseconds:
//   * no launch gap / ramp-up / drain per op (a decode step was ~225 launches);
//   * RMSNorm is folded into the activation staging of the consuming GEMV (each workgroup normalises its own copy);
//   * the first weight rows (and the K/V tiles) of the NEXT phase are requested before the barrier wait, so the barrier and the
//     activation staging that follows overlap with HBM latency.
// Barrier: arrival counters in device memory that only grow during a launch and are zeroed by the last workgroup to leave.  The wait is bounded: after spin_limit polls the workgroup records an error and
// leaves the kernel, so a launch that was not fully resident (or shares the device with another such launch) ends instead of
// hanging; the counters then stay dirty and the caller has to zero them.
#include "qfmt.h"
#include "decode.h"
#include "coherent.h"

struct LayerPtrs {     // one record per block, in device memory (11 pointers)
  const uint8_t *wq, *wk, *wv, *wo, *wg, *wu, *wd;
  const float *attn_norm, *ffn_norm;
  _Float16 *cache_k, *cache_v;
};

struct LayersArgs {
  const LayerPtrs* layers; int n_layers;
  float* x;                       // residual stream, fp32 [dim] (in/out)
  float* qkv;                     // fp32 [n_heads*hd | n_kv*hd | n_kv*hd]
  _Float16* attn;                 // fp16 [n_heads*hd], natural order
  _Float16* act;                  // fp16 [hidden], natural order
  float* part;                    // attention split partials [n_heads][nsplit][hd + 2] + n_kv int32 arrival counters
  const DecodeState* st;
  const float* rope;              // [max_ctx][hd]
  unsigned* sync;                 // 320 uint32: [0] groups arrived, [1] workgroups done, [2] error flag, [32 * (1 + g)] arrivals of group g
  int dim, hidden, n_heads, n_kv, hd, max_ctx, nsplit;
  float eps, scale;
  unsigned spin_limit;
  unsigned long long* trace;      // optional: a few workgroups record the 100 MHz wall clock at every phase boundary
};

#define LY_THREADS 256

// A per-phase copy of a lane-dependent value the optimiser cannot hoist out of the block loop (hoisted address arithmetic of
// all five phases would otherwise stay live across the whole kernel and spill).
__device__ __forceinline__ int opaque_i(int v) { asm volatile("" : "+v"(v)); return v; }

// ------------------------------------------------------------------------------------------------ device-wide barrier
// Two levels: workgroup w counts itself into group w % 8 (own counter, own cache line: on this part consecutive workgroups go to
// the 8 XCDs round-robin, so a group's arrivals come from one XCD), the last of a group counts the group into the top counter,
// and everyone polls the top counter.  One flat counter costs ~8 us per barrier at 512 workgroups (same-address device-scope
// atomics serialise), this layout ~2.5 us.
#define LY_GROUPS 8
struct GridSync {
  unsigned* top; unsigned* grp;                                         // sync[0]; sync[32 * (1 + g)]
  unsigned* done;                                                       // sync[1]
  unsigned top_target, grp_target, grp_size, nwg, limit;
  int* ok_flag;                                                         // LDS
  __device__ __forceinline__ void init(unsigned* c, unsigned g, unsigned lim, int* f) {
    const unsigned me = blockIdx.x % LY_GROUPS;
    top = c; done = c + 1; grp = c + 32 * (1 + me); nwg = g; limit = lim; ok_flag = f;
    grp_size = g / LY_GROUPS + (me < g % LY_GROUPS ? 1u : 0u);
    top_target = 0; grp_target = 0;
  }
  // count this workgroup in (its stores have reached memory)
  __device__ __forceinline__ void arrive() {
    stores_done();
    __syncthreads();
    grp_target += grp_size; top_target += (nwg < LY_GROUPS ? nwg : LY_GROUPS);
    if (threadIdx.x == 0) {
      const unsigned prev = __hip_atomic_fetch_add(grp, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (prev + 1 == grp_target) __hip_atomic_fetch_add(top, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
  // returns false when the bounded wait ran out (every thread of the workgroup sees the same value)
  __device__ __forceinline__ bool wait() {
    if (threadIdx.x == 0) {
      unsigned spins = 0; int ok = 1;
      while (__hip_atomic_load(top, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < top_target) {
        __builtin_amdgcn_s_sleep(1);
        if (++spins > limit) { ok = 0; break; }
      }
      *ok_flag = ok;
    }
    __syncthreads();
    return *ok_flag != 0;
  }
  // end of the launch: the last workgroup to get here zeroes the counters for the next launch (a workgroup that is still
  // polling the last barrier has not been here yet, so the reset cannot overtake it)
  __device__ __forceinline__ void finish() {
    if (threadIdx.x == 0) {
      const unsigned d = __hip_atomic_fetch_add(done, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (d == nwg - 1) {
        __hip_atomic_store(top, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(done, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        for (int g = 0; g < LY_GROUPS; g++) __hip_atomic_store(top + 32 * (1 + g), 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
  }
};

// ------------------------------------------------------------------------------------------------ GEMV phase pieces
// A phase multiplies `ngroups` row groups (R rows each) by one activation row held in registers (lane <-> unit).  WK = 1: a wave
// is a team and owns whole rows; WK = 4: the workgroup is a team, wave w owns units 64w..64w+63 and partial sums meet in LDS.
// Each team owns a contiguous range of groups and keeps D groups of raw weight bytes in flight.  store(group, sums, owner) is
// called by every lane of the wave that holds the sums; only the owner lane writes.
template <int T, int R, int D, class PF>
__device__ __forceinline__ void gemv_prefetch(typename Fmt<T>::Raw (&buf)[D * R], int g0, int g1, int uc, PF ptr) {
#pragma unroll
  for (int d = 0; d < D; d++) {
    int g = g0 + d; g = g < g1 ? g : g1 - 1; g = g < 0 ? 0 : g;          // clamped to a valid group: loads are unconditional
#pragma unroll
    for (int r = 0; r < R; r++) buf[d * R + r] = Fmt<T>::load(ptr(g, r), uc);
  }
}

template <int T, int WK, int R, int D, class PF, class SF>
__device__ __forceinline__ void gemv_run(typename Fmt<T>::Raw (&buf)[D * R], int g0, int g1, int uc, bool uvalid, const u32x4* xv, const float* cv,
                                         const uint32_t* kc, PF ptr, SF store, float (*part)[4][2], int lane, int wave) {
  static_assert(R <= 2, "two partial-sum slots per wave");
  int parity = 0;
  for (int g = g0; g < g1; g += D) {
#pragma unroll
    for (int d = 0; d < D; d++) {
      const int gg = g + d;
      if (gg < g1) {
        float acc[R];
#pragma unroll
        for (int r = 0; r < R; r++) {
          acc[r] = 0.f;
          unit_dot_reg<T>(buf[d * R + r], xv, cv, acc[r], kc);
          acc[r] = wave_sum_lane63(uvalid ? acc[r] : 0.f);
        }
        if constexpr (WK > 1) {
          if (lane == 63) {
#pragma unroll
            for (int r = 0; r < R; r++) part[parity][wave][r] = acc[r];
          }
          __syncthreads();
          if (wave == 0) {
            float t = 0.f;
            if (lane < R) {
#pragma unroll
              for (int j = 0; j < WK; j++) t += part[parity][j][lane];
            }
            float o[R];
#pragma unroll
            for (int r = 0; r < R; r++) o[r] = __shfl(t, r, 64);
            store(gg, o, lane == 0);
          }
          parity ^= 1;
        } else {
          store(gg, acc, lane == 63);
        }
      }
      int gn = gg + D; gn = gn < g1 ? gn : g1 - 1;                       // refill (clamped past the end)
#pragma unroll
      for (int r = 0; r < R; r++) buf[d * R + r] = Fmt<T>::load(ptr(gn, r), uc);
    }
  }
}

// Residual rows of a team (two per group, contiguous): lane j fetches x[2 g0 + j] once at the start of the phase, so the GEMV loop
// holds no load whose result it must wait for (a wait there would also wait for every weight row in flight).
__device__ __forceinline__ float resid_load(const float* x, int g0, int g1, int dim, int lane) {
  int i = 2 * g0 + (lane < 2 * (g1 - g0) ? lane : 0);
  return cld(&x[i < dim ? i : dim - 1]);
}
__device__ __forceinline__ void resid_store(float* x, int g, int g0, int g1, float resid, const float* v, bool own) {
  float r0, r1;
  if (2 * (g1 - g0) <= 64) { r0 = __shfl(resid, 2 * (g - g0), 64); r1 = __shfl(resid, 2 * (g - g0) + 1, 64); }
  else { r0 = cld(&x[2 * g]); r1 = cld(&x[2 * g + 1]); }
  if (own) { cst(&x[2 * g], r0 + v[0]); cst(&x[2 * g + 1], r1 + v[1]); }
}

// contiguous share of `n` groups for team `t` of `nt`
__device__ __forceinline__ void team_range(int n, int t, int nt, int& g0, int& g1) {
  g0 = (int)(((unsigned)n * (unsigned)t) / (unsigned)nt); g1 = (int)(((unsigned)n * (unsigned)(t + 1)) / (unsigned)nt);   // n * nt < 2^32 (host-checked)
}

// ---- activation staging: global (natural order) -> LDS (padded unit stride) -> this lane's unit -> staged registers ----
template <int T>
__device__ __forceinline__ void stage_read(const uint32_t* xl, int uc, u32x4* xv, float* cv) {
  using F = Fmt<T>; constexpr int NP = F::UW / 2, US = NP + 4;
  uint32_t nx[NP];
#pragma unroll
  for (int k = 0; k < NP; k += 4) { const u32x4 v = *(const u32x4*)(xl + uc * US + k); nx[k] = v.x; nx[k + 1] = v.y; nx[k + 2] = v.z; nx[k + 3] = v.w; }
  F::stage(nx, xv, cv);
}
__device__ __forceinline__ u32x4 pack8(const f32x4 lo, const f32x4 hi) {
  u32x4 v = {f2h_bits(lo.x) | (f2h_bits(lo.y) << 16), f2h_bits(lo.z) | (f2h_bits(lo.w) << 16),
             f2h_bits(hi.x) | (f2h_bits(hi.y) << 16), f2h_bits(hi.z) | (f2h_bits(hi.w) << 16)};
  return v;
}
// fp16 source, no norm.  NIT = pieces per thread (K <= 2048 * NIT): all loads go out before the first LDS write.
template <int T, int NIT>
__device__ __forceinline__ void stage_f16(int tid, const _Float16* src, int K, int uc, uint32_t* xl, u32x4* xv, float* cv) {
  using F = Fmt<T>; constexpr int US = F::UW / 2 + 4;
  const int nq = K >> 3;
  u32x4 v[NIT];
#pragma unroll
  for (int j = 0; j < NIT; j++) { const int i = tid + LY_THREADS * j; v[j] = cld16((const u32x4*)src + (i < nq ? i : nq - 1)); }
#pragma unroll
  for (int j = 0; j < NIT; j++) { const int i = tid + LY_THREADS * j; if (i < nq) *(u32x4*)(xl + F::unit_of(8 * i) * US + F::pair_of(8 * i)) = v[j]; }
  __syncthreads();
  stage_read<T>(xl, uc, xv, cv);
}
// fp32 source with RMSNorm folded in: nn.RMSNorm (tinygrad/nn/__init__.py:296-304), (x * rsqrt(mean(x^2) + eps)) * weight -> fp16
template <int T, bool SMALLK>
__device__ __forceinline__ void stage_norm(int tid, const float* x, const float* nw, float eps, int K, int uc, uint32_t* xl, float* red, u32x4* xv, float* cv) {
  using F = Fmt<T>; constexpr int US = F::UW / 2 + 4;
  const int nq = K >> 3, lane = tid & 63, wave = tid >> 6;
  const f32x4* xr = (const f32x4*)x; const f32x4* wr = (const f32x4*)nw;
  auto X = [&](int i) { return cld16f(xr + i); };
  auto W = [&](int i) { return gld16f(wr + i); };
  float ss = 0.f;
  auto sq = [](const f32x4 v) { return v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w; };
  auto finish_scale = [&](float s) {
    s = wave_sum(s);
    if (lane == 0) red[wave] = s;
    __syncthreads();
    const float tot = (red[0] + red[1]) + (red[2] + red[3]);
    return 1.0f / sqrtf(tot / (float)K + eps);
  };
  auto put = [&](int i, const f32x4 a0, const f32x4 a1, const f32x4 w0, const f32x4 w1, float sc) {
    const f32x4 lo = {(a0.x * sc) * w0.x, (a0.y * sc) * w0.y, (a0.z * sc) * w0.z, (a0.w * sc) * w0.w};
    const f32x4 hi = {(a1.x * sc) * w1.x, (a1.y * sc) * w1.y, (a1.z * sc) * w1.z, (a1.w * sc) * w1.w};
    *(u32x4*)(xl + F::unit_of(8 * i) * US + F::pair_of(8 * i)) = pack8(lo, hi);
  };
  if constexpr (SMALLK) {                                                // K <= 4096: two 8-element pieces per thread stay in registers
    f32x4 a[2][2], w[2][2];
#pragma unroll
    for (int j = 0; j < 2; j++) {
      const int i = tid + LY_THREADS * j, ic = i < nq ? i : nq - 1;
      a[j][0] = X(2 * ic); a[j][1] = X(2 * ic + 1); w[j][0] = W(2 * ic); w[j][1] = W(2 * ic + 1);
    }
#pragma unroll
    for (int j = 0; j < 2; j++) if (tid + LY_THREADS * j < nq) ss += sq(a[j][0]) + sq(a[j][1]);
    const float sc = finish_scale(ss);
#pragma unroll
    for (int j = 0; j < 2; j++) if (tid + LY_THREADS * j < nq) put(tid + LY_THREADS * j, a[j][0], a[j][1], w[j][0], w[j][1], sc);
  } else {
    for (int i = tid; i < nq; i += LY_THREADS) ss += sq(X(2 * i)) + sq(X(2 * i + 1));
    const float sc = finish_scale(ss);
    for (int i = tid; i < nq; i += LY_THREADS) put(i, X(2 * i), X(2 * i + 1), W(2 * i), W(2 * i + 1), sc);
  }
  __syncthreads();
  stage_read<T>(xl, uc, xv, cv);
}

// ------------------------------------------------------------------------------------------------ attention pieces
// (kv head, 64-position split) tasks as in attn_decode_kernel (decode.hip), with the split's positions divided over the four
// waves (16 each) and every wave serving all query heads of the group: a wave's K and V tiles are 16 rows (HD8 / 4 load
// instructions each: instruction i covers rows i*RPI + lane / HD8, RPI = 64 / HD8, and lane % HD8 picks the 16-byte piece), so
// a lane only ever needs the 8 query values of ITS piece.  Scores: 8 FMAs per instruction, then a DPP sum over the HD8 lanes
// of a row.  Each run of HD8 lanes keeps its own softmax partial (its rows only); the partials meet in LDS and leave as one
// partial per (head, split).
// The tiles of a workgroup's first task are requested before the barrier that publishes q/k/v; the row of the current token
// (and the clamped rows behind it) is patched in from LDS afterwards.
#define LY_ATTN_LDS_FLOATS(HD) (6 * (HD) + 16 * (512 / (HD)) * ((HD) + 4) + 2048)
template <int HD8>
__device__ __forceinline__ void attn_load_tiles(const LayersArgs& a, const LayerPtrs& L, int kvh, int split, int pos, int tid, u32x4* kt, u32x4* vt) {
  constexpr int HD = HD8 * 8, RPI = 64 / HD8, NVI = 16 / RPI;
  const int lane = tid & 63, wave = tid >> 6;
  const int vr = lane / HD8, vp = lane % HD8;
  const _Float16* kbase = L.cache_k + (size_t)kvh * a.max_ctx * HD + vp * 8;
  const _Float16* vbase = L.cache_v + (size_t)kvh * a.max_ctx * HD + vp * 8;
#pragma unroll
  for (int i = 0; i < NVI; i++) {
    const int r = split * 64 + wave * 16 + i * RPI + vr, rc = r < pos ? r : pos;
    kt[i] = gld16(kbase + (size_t)rc * HD);
    vt[i] = gld16(vbase + (size_t)rc * HD);
  }
}
__device__ __forceinline__ u32x4 pack8_lds(const float* c) {
  u32x4 r = {f2h_bits(c[0]) | (f2h_bits(c[1]) << 16), f2h_bits(c[2]) | (f2h_bits(c[3]) << 16),
             f2h_bits(c[4]) | (f2h_bits(c[5]) << 16), f2h_bits(c[6]) | (f2h_bits(c[7]) << 16)};
  return r;
}
// sum over the HD8 (8 or 16) consecutive lanes that hold one row; every lane of the run gets the sum
template <int HD8>
__device__ __forceinline__ float row_sum(float v) {
  v = dpp_add<0xB1>(v); v = dpp_add<0x4E>(v); v = dpp_add<0x141>(v);
  if constexpr (HD8 == 16) v = dpp_add<0x140>(v);
  return v;
}

template <int HD8>
__device__ __forceinline__ void attn_task(const LayersArgs& a, const LayerPtrs& L, int kvh, int split, int pos, int tid, u32x4* kt, u32x4* vt, float* lds, int* last_flag) {
  constexpr int HD = HD8 * 8, RPI = 64 / HD8, NVI = 16 / RPI;
  const int lane = tid & 63, wave = tid >> 6;
  const int half = HD >> 1, group = a.n_heads / a.n_kv;
  float (*qs)[HD] = (float (*)[HD])lds;                 // rotated queries of the 4 heads in flight
  float* ks = lds + 4 * HD; float* vs = ks + HD;        // rotated key / value of this token
  constexpr int NGRP = 4 * RPI, CSTR = HD + 4;          // row runs per workgroup (wave, lane / HD8); floats per partial (16-byte multiple)
  float* comb = vs + HD;                                // [head in flight][run]: o[HD], m, l
  float* sw = comb + 4 * NGRP * CSTR;                   // [2048] merge weights
  const float* q = a.qkv; const float* k = a.qkv + a.n_heads * HD; const float* v = k + a.n_kv * HD;
  const int p0 = split * 64 + wave * 16;                // first position of this wave
  // the query of the first head pass is requested together with k and v (one round trip instead of two); half <= 64 lanes
  const int qi = lane < half ? lane : half - 1, qh = kvh * group + (wave < group ? wave : 0);
  const float qx1 = cld(&q[qh * HD + qi]), qx2 = cld(&q[qh * HD + half + qi]);
  const float qc = a.rope[(size_t)pos * HD + qi], qsn = a.rope[(size_t)pos * HD + half + qi];
  for (int i = tid; i < half; i += LY_THREADS) {
    const float c = a.rope[(size_t)pos * HD + i], s = a.rope[(size_t)pos * HD + half + i];
    const float x1 = cld(&k[kvh * HD + i]), x2 = cld(&k[kvh * HD + half + i]);
    ks[i] = x1 * c - x2 * s; ks[half + i] = x2 * c + x1 * s;
  }
  for (int i = tid; i < HD; i += LY_THREADS) vs[i] = cld(&v[kvh * HD + i]);
  __syncthreads();
  if ((pos >> 6) == split) {                            // owner split appends this token to the cache
    for (int i = tid; i < HD; i += LY_THREADS) {
      L.cache_k[((size_t)kvh * a.max_ctx + pos) * HD + i] = (_Float16)ks[i];
      L.cache_v[((size_t)kvh * a.max_ctx + pos) * HD + i] = (_Float16)vs[i];
    }
  }
  const int vr = lane / HD8, vp = lane % HD8;
  {
    const u32x4 kcur = pack8_lds(ks + vp * 8), vcur = pack8_lds(vs + vp * 8);
#pragma unroll
    for (int i = 0; i < NVI; i++) if (p0 + i * RPI + vr >= pos) { kt[i] = kcur; vt[i] = vcur; }
  }
  for (int h0 = 0; h0 < group; h0 += 4) {
    if (h0 == 0) {
      if (wave < group && lane < half) { qs[wave][lane] = qx1 * qc - qx2 * qsn; qs[wave][half + lane] = qx2 * qc + qx1 * qsn; }
    } else if (h0 + wave < group) {                     // wave w rotates the query of head h0 + w
      const int head = kvh * group + h0 + wave;
      for (int i = lane; i < half; i += 64) {
        const float c = a.rope[(size_t)pos * HD + i], s = a.rope[(size_t)pos * HD + half + i];
        const float x1 = cld(&q[head * HD + i]), x2 = cld(&q[head * HD + half + i]);
        qs[wave][i] = x1 * c - x2 * s; qs[wave][half + i] = x2 * c + x1 * s;
      }
    }
    __syncthreads();
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
          t = row_sum<HD8>(t);
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
        const float wg = __expf(cb[g * CSTR + HD] - m);
        l += wg * cb[g * CSTR + HD + 1];
#pragma unroll
        for (int j = 0; j < HD / 64; j++) od[j] += wg * cb[g * CSTR + lane + 64 * j];
      }
      float* po = a.part + ((size_t)head * a.nsplit + split) * (HD + 2);
#pragma unroll
      for (int j = 0; j < HD / 64; j++) cst(&po[lane + 64 * j], od[j]);
      if (lane == 0) { cst(&po[HD], m); cst(&po[HD + 1], l); }
    }
    __syncthreads();
  }
  // ---- merge: the last split of this kv head to arrive combines its heads' partials ----
  int* counters = (int*)(a.part + (size_t)a.n_heads * a.nsplit * (HD + 2));
  const int ns = (pos >> 6) + 1;
  stores_done();
  __syncthreads();
  if (tid == 0) {
    const int prev = __hip_atomic_fetch_add(&counters[kvh], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    *last_flag = (prev == ns - 1);
    if (prev == ns - 1) __hip_atomic_store(&counters[kvh], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  __syncthreads();
  if (*last_flag) {
    // All loads of the merge go out in one batch: (m, l) of every (head, split), then the first 2 x 16 partial values of this
    // thread's outputs, and only then are the softmax weights formed (loads return in issue order).
    constexpr int SC = 16;                              // splits in flight per output
    const int nml = group * ns, nout = group * HD;
    const int e0 = tid < nml ? tid : nml - 1;
    const int e0h = e0 / ns, e0s = e0 - e0h * ns;
    const float* ph0 = a.part + ((size_t)(kvh * group + e0h) * a.nsplit + e0s) * (HD + 2);
    const float mv = cld(&ph0[HD]), lv = cld(&ph0[HD + 1]);
    float vv[2][SC];
    auto load_chunk = [&](int ib, int sb) {
#pragma unroll
      for (int k = 0; k < 2; k++) {
        const int c = ib + LY_THREADS * k < nout ? ib + LY_THREADS * k : nout - 1;
        const int gh = c / HD, d = c - gh * HD;
        const float* p = a.part + (size_t)(kvh * group + gh) * a.nsplit * (HD + 2) + d;
#pragma unroll
        for (int j = 0; j < SC; j++) vv[k][j] = cld(&p[(size_t)min(sb + j, ns - 1) * (HD + 2)]);
      }
    };
    load_chunk(tid, 0);
    if (tid < nml) { sw[e0h * a.nsplit + e0s] = mv; sw[1024 + e0h * a.nsplit + e0s] = lv; }
    for (int idx = tid + LY_THREADS; idx < nml; idx += LY_THREADS) {
      const int gh = idx / ns, sp = idx - gh * ns;
      const float* ph = a.part + ((size_t)(kvh * group + gh) * a.nsplit + sp) * (HD + 2);
      sw[gh * a.nsplit + sp] = cld(&ph[HD]);
      sw[1024 + gh * a.nsplit + sp] = cld(&ph[HD + 1]);
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
    for (int ib = tid; ib < nout; ib += 2 * LY_THREADS) {
      float o[2] = {0.f, 0.f};
      for (int sb = 0; sb < ns; sb += SC) {
        if (ib != tid || sb != 0) load_chunk(ib, sb);
#pragma unroll
        for (int k = 0; k < 2; k++) {
          const int c = ib + LY_THREADS * k < nout ? ib + LY_THREADS * k : nout - 1;
          const float* wrow = sw + (c / HD) * a.nsplit + sb;
#pragma unroll
          for (int j = 0; j < SC; j++) if (sb + j < ns) o[k] += vv[k][j] * wrow[j];
        }
      }
#pragma unroll
      for (int k = 0; k < 2; k++) if (ib + LY_THREADS * k < nout) cst_h(&a.attn[kvh * group * HD + ib + LY_THREADS * k], o[k]);
    }
  }
  __syncthreads();                                      // LDS is reused by the next task / phase
}

// ------------------------------------------------------------------------------------------------ the kernel
__device__ __forceinline__ LayerPtrs load_layer(const LayerPtrs* table, int l) { return table[l]; }

// T: block-pair weight format of every linear; WKD / WKH: waves that split K for K = dim / K = hidden (1 or 4); HD8 = head_dim / 8.
template <int T, int WKD, int WKH, int HD8>
__global__ __launch_bounds__(LY_THREADS, 2) void decode_layers_kernel(const LayersArgs a) {
  using F = Fmt<T>;
  typedef typename F::Raw Raw;
  constexpr int HD = HD8 * 8, RPI = 64 / HD8, NVI = 16 / RPI;
  extern __shared__ uint32_t dyn[];                     // activation staging (nu * (UW/2 + 4) dwords) | attention arrays
  __shared__ float red[4];
  __shared__ float part[2][4][2];
  __shared__ int flag_sync, flag_last;
  const int lane0 = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int G = gridDim.x;
  const int pos = a.st->pos;
  const int nq = a.n_heads * HD, nkv = a.n_kv * HD;
  const int nu_d = a.dim / F::UW, nu_h = a.hidden / F::UW;
  const unsigned rb_d = (unsigned)(a.dim / F::BW) * F::BB, rb_h = (unsigned)(a.hidden / F::BW) * F::BB;
  // teams for K = dim / K = hidden
  const int team_d = (WKD == 1) ? blockIdx.x * 4 + wave : blockIdx.x, nteam_d = (WKD == 1) ? G * 4 : G;
  const int team_h = (WKH == 1) ? blockIdx.x * 4 + wave : blockIdx.x, nteam_h = (WKH == 1) ? G * 4 : G;
  uint32_t kc[F::NKC];
  F::consts(kc);

  GridSync gs;
  gs.init(a.sync, (unsigned)G, a.spin_limit, &flag_sync);
  int tr_i = 0;
#define LY_TRACE() do { if (a.trace && threadIdx.x == 0) { if (blockIdx.x % 73 == 0) a.trace[(blockIdx.x / 73) * 11 * a.n_layers + tr_i] = wall_clock64(); } tr_i++; } while (0)
#define LY_WAIT() do { if (!gs.wait()) { if (threadIdx.x == 0) a.sync[2] = 1u; return; } } while (0)

  // row ranges (identical for every block)
  int ga0, ga1, gc0, gc1, gd0, gd1, ge0, ge1;
  team_range(nq + 2 * nkv, team_d, nteam_d, ga0, ga1);   // q/k/v: one row per group
  team_range(a.dim / 2, team_d, nteam_d, gc0, gc1);      // attn_output: two rows per group
  team_range(a.hidden, team_d, nteam_d, gd0, gd1);       // gate/up: group = one (gate row, up row) pair
  team_range(a.dim / 2, team_h, nteam_h, ge0, ge1);      // down: two rows per group
  const int ns = (pos >> 6) + 1, ntasks = a.n_kv * ns;

  constexpr int NB = 4, NB2 = NB / 2;                   // weight rows in flight per wave (six measured no faster)
  Raw buf[NB];
  u32x4 xv[F::XV]; float cv[F::NG];
  // this lane's unit (clamped) for K = dim / K = hidden, from a per-phase opaque lane id
  auto unit_d = [&](int lane, bool& valid) { const int u = (WKD == 1) ? lane : wave * 64 + lane; valid = u < nu_d; return valid ? u : nu_d - 1; };
  auto unit_h = [&](int lane, bool& valid) { const int u = (WKH == 1) ? lane : wave * 64 + lane; valid = u < nu_h; return valid ? u : nu_h - 1; };
  {
    const LayerPtrs L0 = load_layer(a.layers, 0);
    bool uv; const int uc = unit_d(lane0, uv);
    auto ptrA = [&](int g, int) { return g < nq ? L0.wq + (size_t)((unsigned)g * rb_d) : (g < nq + nkv ? L0.wk + (size_t)((unsigned)(g - nq) * rb_d) : L0.wv + (size_t)((unsigned)(g - nq - nkv) * rb_d)); };
    gemv_prefetch<T, 1, NB>(buf, ga0, ga1, uc, ptrA);
  }
  for (int l = 0; l < a.n_layers; l++) {
    const LayerPtrs L = load_layer(a.layers, l);
    // ---------------- phase A: q/k/v = W_qkv * attn_norm(x) ----------------
    {
      const int tid = opaque_i(threadIdx.x), lane = tid & 63; bool uv; const int uc = unit_d(lane, uv);
      auto ptrA = [&](int g, int) { return g < nq ? L.wq + (size_t)((unsigned)g * rb_d) : (g < nq + nkv ? L.wk + (size_t)((unsigned)(g - nq) * rb_d) : L.wv + (size_t)((unsigned)(g - nq - nkv) * rb_d)); };
      stage_norm<T, WKD == 1>(tid, a.x, L.attn_norm, a.eps, a.dim, uc, dyn, red, xv, cv);
      LY_TRACE();
      gemv_run<T, WKD, 1, NB>(buf, ga0, ga1, uc, uv, xv, cv, kc, ptrA, [&](int g, const float* v, bool own) { if (own) cst(&a.qkv[g], v[0]); }, part, lane, wave);
      LY_TRACE();
    }
    gs.arrive();
    // ---------------- phase B: RoPE + KV append + attention ----------------
    {
      const int tid = opaque_i(threadIdx.x), lane = tid & 63;
      u32x4 kt[NVI], vt[NVI];
      int task = blockIdx.x;
      if (task < ntasks) attn_load_tiles<HD8>(a, L, task % a.n_kv, task / a.n_kv, pos, tid, kt, vt);
      LY_WAIT();
      LY_TRACE();
      bool first = true;
      for (; task < ntasks; task += G) {
        if (!first) attn_load_tiles<HD8>(a, L, task % a.n_kv, task / a.n_kv, pos, tid, kt, vt);
        attn_task<HD8>(a, L, task % a.n_kv, task / a.n_kv, pos, tid, kt, vt, (float*)dyn, &flag_last);
        first = false;
      }
      LY_TRACE();
    }
    gs.arrive();
    // ---------------- phase C: x += W_o * attn ----------------
    {
      const int tid = opaque_i(threadIdx.x), lane = tid & 63; bool uv; const int uc = unit_d(lane, uv);
      auto ptrC = [&](int g, int r) { return L.wo + (size_t)((unsigned)(2 * g + r) * rb_d); };
      gemv_prefetch<T, 2, NB2>(buf, gc0, gc1, uc, ptrC);
      LY_WAIT();
      LY_TRACE();
      const float resid = resid_load(a.x, gc0, gc1, a.dim, lane);
      stage_f16<T, WKD == 1 ? 2 : 8>(tid, a.attn, a.dim, uc, dyn, xv, cv);
      gemv_run<T, WKD, 2, NB2>(buf, gc0, gc1, uc, uv, xv, cv, kc, ptrC,
                             [&](int g, const float* v, bool own) { resid_store(a.x, g, gc0, gc1, resid, v, own); }, part, lane, wave);
      LY_TRACE();
    }
    gs.arrive();
    // ---------------- phase D: act = silu(W_gate * n) * (W_up * n), n = ffn_norm(x) ----------------
    {
      const int tid = opaque_i(threadIdx.x), lane = tid & 63; bool uv; const int uc = unit_d(lane, uv);
      auto ptrD = [&](int g, int r) { return (r ? L.wu : L.wg) + (size_t)((unsigned)g * rb_d); };
      gemv_prefetch<T, 2, NB2>(buf, gd0, gd1, uc, ptrD);
      LY_WAIT();
      LY_TRACE();
      stage_norm<T, WKD == 1>(tid, a.x, L.ffn_norm, a.eps, a.dim, uc, dyn, red, xv, cv);
      gemv_run<T, WKD, 2, NB2>(buf, gd0, gd1, uc, uv, xv, cv, kc, ptrD,
                             [&](int g, const float* v, bool own) { if (own) cst_h(&a.act[g], silu_f(v[0]) * v[1]); }, part, lane, wave);
      LY_TRACE();
    }
    gs.arrive();
    // ---------------- phase E: x += W_down * act ----------------
    {
      const int tid = opaque_i(threadIdx.x), lane = tid & 63; bool uv; const int uc = unit_h(lane, uv);
      auto ptrE = [&](int g, int r) { return L.wd + (size_t)((unsigned)(2 * g + r) * rb_h); };
      gemv_prefetch<T, 2, NB2>(buf, ge0, ge1, uc, ptrE);
      LY_WAIT();
      LY_TRACE();
      const float resid = resid_load(a.x, ge0, ge1, a.dim, lane);
      stage_f16<T, WKH == 1 ? 2 : 8>(tid, a.act, a.hidden, uc, dyn, xv, cv);
      gemv_run<T, WKH, 2, NB2>(buf, ge0, ge1, uc, uv, xv, cv, kc, ptrE,
                             [&](int g, const float* v, bool own) { resid_store(a.x, g, ge0, ge1, resid, v, own); }, part, lane, wave);
      LY_TRACE();
    }
    if (l + 1 < a.n_layers) {
      gs.arrive();
      const int lane = opaque_i(lane0); bool uv; const int uc = unit_d(lane, uv);
      const LayerPtrs Ln = load_layer(a.layers, l + 1);
      auto ptrA = [&](int g, int) { return g < nq ? Ln.wq + (size_t)((unsigned)g * rb_d) : (g < nq + nkv ? Ln.wk + (size_t)((unsigned)(g - nq) * rb_d) : Ln.wv + (size_t)((unsigned)(g - nq - nkv) * rb_d)); };
      gemv_prefetch<T, 1, NB>(buf, ga0, ga1, uc, ptrA);
      LY_WAIT();
    }
    LY_TRACE();
  }
  gs.finish();
#undef LY_WAIT
#undef LY_TRACE
}

// ------------------------------------------------------------------------------------------------ host side
template <int T, int WKD, int WKH, int HD8>
static int launch_layers(const LayersArgs& a, size_t lds, hipStream_t s) {
  auto kern = decode_layers_kernel<T, WKD, WKH, HD8>;
  static int grid = 0;
  if (!grid) {
    int dev = 0, per_cu = 0; hipDeviceProp_t p;
    TGA_HIP(hipGetDevice(&dev));
    TGA_HIP(hipGetDeviceProperties(&p, dev));
    TGA_HIP(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, 64 * 1024));
    TGA_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kern, LY_THREADS, 64 * 1024));
    TGA_REQUIRE(per_cu >= 1, "tga_decode_layers: the kernel does not fit on a CU");
    grid = p.multiProcessorCount * (per_cu >= 2 ? 2 : 1);              // every workgroup resident at once
  }
  kern<<<grid, LY_THREADS, lds, s>>>(a);
  TGA_LAUNCH_CHECK();
  return 0;
}

template <int T, int HD8>
static int launch_layers_w(const LayersArgs& a, size_t lds, hipStream_t s) {
  const int nu_d = a.dim / 64, nu_h = a.hidden / 64;
  if (nu_d <= 64) return nu_h <= 64 ? launch_layers<T, 1, 1, HD8>(a, lds, s) : launch_layers<T, 1, 4, HD8>(a, lds, s);
  return nu_h <= 64 ? launch_layers<T, 4, 1, HD8>(a, lds, s) : launch_layers<T, 4, 4, HD8>(a, lds, s);
}

static unsigned long long* g_layers_trace = nullptr;
// Profiling aid: a device buffer of at least 8 * 11 * n_layers uint64 that workgroups 0, 73, 146, ... (at most 8) of later
// tga_decode_layers launches fill with 100 MHz wall-clock stamps, [workgroup / 73][block][11]: [stage A done, A done, B start, B done, C start, C done, D start, D done, E start, E done,
// next block ready].  NULL switches it off.
extern "C" int tga_decode_layers_trace(void* buf) { g_layers_trace = (unsigned long long*)buf; return 0; }

extern "C" int tga_decode_layers(const void* layer_table, int n_layers, int weight_type, float* x, float* qkv, void* attn_f16, void* act_f16,
                                 float* partials, const void* state, const float* rope_table, void* sync, int dim, int hidden, int n_heads,
                                 int n_kv_heads, int head_dim, int max_ctx, float eps, void* stream) {
  TGA_REQUIRE(layer_table && x && qkv && attn_f16 && act_f16 && partials && state && rope_table && sync, "tga_decode_layers: null pointer");
  TGA_REQUIRE(weight_type == GGML_Q4_0 || weight_type == GGML_Q8_0, "tga_decode_layers: weight type %d is not built (Q4_0, Q8_0)", weight_type);
  TGA_REQUIRE(n_layers >= 1, "tga_decode_layers: n_layers=%d", n_layers);
  TGA_REQUIRE(head_dim == 64 || head_dim == 128, "tga_decode_layers: head_dim=%d must be 64 or 128", head_dim);
  TGA_REQUIRE(n_kv_heads > 0 && n_heads % n_kv_heads == 0, "tga_decode_layers: n_heads=%d must be a multiple of n_kv_heads=%d", n_heads, n_kv_heads);
  TGA_REQUIRE(n_heads * head_dim == dim, "tga_decode_layers: n_heads * head_dim = %d must equal dim = %d", n_heads * head_dim, dim);
  TGA_REQUIRE(dim % 64 == 0 && hidden % 64 == 0 && dim >= 64 && hidden >= 64, "tga_decode_layers: dim=%d and hidden=%d must be multiples of 64", dim, hidden);
  TGA_REQUIRE(dim <= 16384 && hidden <= 16384, "tga_decode_layers: dim=%d / hidden=%d above 16384", dim, hidden);
  TGA_REQUIRE(max_ctx > 0 && (n_heads / n_kv_heads) * ((max_ctx + 63) / 64) <= 1024, "tga_decode_layers: max_ctx=%d too long for the merge table", max_ctx);
  TGA_REQUIRE((((uintptr_t)x | (uintptr_t)qkv | (uintptr_t)attn_f16 | (uintptr_t)act_f16) & 15) == 0, "tga_decode_layers: activation buffers must be 16-byte aligned");
  LayersArgs a;
  a.layers = (const LayerPtrs*)layer_table; a.n_layers = n_layers;
  a.x = x; a.qkv = qkv; a.attn = (_Float16*)attn_f16; a.act = (_Float16*)act_f16; a.part = partials;
  a.st = (const DecodeState*)state; a.rope = rope_table; a.sync = (unsigned*)sync;
  a.dim = dim; a.hidden = hidden; a.n_heads = n_heads; a.n_kv = n_kv_heads; a.hd = head_dim; a.max_ctx = max_ctx; a.nsplit = (max_ctx + 63) / 64;
  a.eps = eps; a.scale = 1.0f / sqrtf((float)head_dim);
  a.trace = g_layers_trace;
  a.spin_limit = 1u << 20;                                             // polls before a barrier wait gives up (seconds)
  const int numax = (dim > hidden ? dim : hidden) / 64;
  const long long rb_max = (long long)numax * (weight_type == GGML_Q4_0 ? 36 : 68);
  size_t lds = (size_t)numax * 36 * 4;
  const size_t attn_lds = (size_t)LY_ATTN_LDS_FLOATS(head_dim) * 4;
  if (lds < attn_lds) lds = attn_lds;
  TGA_REQUIRE((long long)(dim > hidden ? dim : hidden) * 4 * 1024 < (1ll << 32) && (long long)hidden * rb_max < (1ll << 32), "tga_decode_layers: shape too large for 32-bit row arithmetic");
  TGA_REQUIRE(lds <= 64 * 1024, "tga_decode_layers: staging needs %zu bytes of LDS", lds);
  hipStream_t s = (hipStream_t)stream;
  if (weight_type == GGML_Q4_0) return head_dim == 128 ? launch_layers_w<F_Q4_0P, 16>(a, lds, s) : launch_layers_w<F_Q4_0P, 8>(a, lds, s);
  return head_dim == 128 ? launch_layers_w<F_Q8_0P, 16>(a, lds, s) : launch_layers_w<F_Q8_0P, 8>(a, lds, s);
}
