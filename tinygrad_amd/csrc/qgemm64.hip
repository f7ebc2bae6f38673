// Prefill GEMM over GGUF blocks: 17 .. 128 activation rows (the positions of one prefill step, tinygrad/llm/model.py:464, 476-481: a T > 1 call of the same
// linears, x.linear(W.T) over the lazily dequantized weight, tinygrad/nn/__init__.py:177, tinygrad/mixin/op.py:367-392) in ONE pass over the weights.
// The small-batch kernels multiply sixteen rows per pass (the sixteen columns of one MFMA tile), so a step of 64 positions decoded every weight four times;
// here a unit is decoded once into fp16 weights (the reference's own fp16 weight cast, model.py:376) and multiplied with two, four or eight column groups of
// sixteen rows (up to 128 positions per pass: at 64 the pass is bound by how the weights stream, at 128 by the LDS reads of the B operands).
//
// Up to three launches per call, all on the caller's stream:
//  1. q64_stage_kernel: the activations - up to 128 rows x K, fp16 or float32 - are permuted ONCE into the formats' staged order (Fmt::stage), laid out per step
//     of 256 values of K as [vector][column group][unit][column] 16-byte pieces: exactly the bytes the multiplying workgroups want in LDS, rows at and beyond M
//     as zeros.  (When every workgroup staged for itself, each of its 256 threads fetched one 128-byte line in eight instructions that touch 64 lines each:
//     the texture path, not the matrix cores, set the pace - gate/up of the 8B shapes 54 us, of which 20 us were that fetch.)
//  2. qgemm64_kernel: a workgroup is four waves and owns 64 weight rows (SwiGLU pair: 32 gate rows and the same 32 up rows), wave w rows 16 w .. 16 w + 15, over
//     a contiguous range of steps.  As in qgemm.hip lane 16 g + r loads unit 4 s + g of weight row r straight from global memory (a ring of three steps in
//     flight), decodes it and supplies the A operands of eight v_mfma_f32_16x16x32_f16 per column group; the B operand of lane 16 g + c is the matching vector
//     of activation row c of that column group, read from LDS.  The staged activations of a step are a straight copy, 1 KB per wave instruction: requested
//     while the step before is multiplied, written to the other of two LDS stages behind it, one barrier per step.  (Direct-to-LDS loads for this copy,
//     three stages deep, made the compiler drain every outstanding load - the weight ring included - at each use of a weight register: ordinary loads
//     keep its counting exact.)
//     Matrices of few rows (4096: 64 row tiles for 256 CUs) split K over gridDim.y workgroups per row tile, which write float32 partial tiles.
//  3. q64_reduce_kernel (only when K was split): y = [residual +] the partials summed in the order of K - the same sum whichever workgroup finished first.
// Without a split the multiplying kernel stores for itself: plain, + residual (in place allowed: every element is read and written by one lane), or
// silu(gate) * up, for which a lane's gate rows and the matching up rows sit 32 lanes apart.
//
// The staged activations (at most 8 MB) and the partial tiles (at most 32 MB) live in a workspace that tga_init allocates once per device: Q64_SLOTS slots, a
// stream keeps the slot it was given first (launches of one stream are ordered, so they may share one), a call on a further stream gets none and is told to
// run blocks of sixteen rows instead.
#include "qfmt.h"
#include <mutex>

typedef _Float16 v8f16 __attribute__((ext_vector_type(8)));
typedef float v4f32 __attribute__((ext_vector_type(4)));

#define Q64_MAX_K 32768
#define Q64_COLS 128                  // activation rows of a call at most = columns of a partial tile's split
#define Q64_XS_BYTES ((size_t)Q64_COLS * Q64_MAX_K * 2)
#define Q64_PART_BYTES ((size_t)32 << 20)
#define Q64_SLOTS 4
#define Q64_MAX_DEVICES 64
#ifndef Q64_RING
#define Q64_RING 3
#endif

// Options of a call (qgemv.hip fills them): prestaged - the activations already lie in the multiplying layout, in the workspace (xs_ext == nullptr) or in the caller's
// buffer xs_ext; defer (residual epilogue, one matrix) - when K is split, the partial tiles are left for the caller's next launch to sum (q64_norm_stage_kernel,
// tga_rows_add_partials) and part / ks / np say where they are; ks = 0 on return: nothing is pending, y is complete.
struct Q64Opt { bool prestaged; const void* xs_ext; bool defer; float* part; int ks, np; };

struct Q64X {
  u32x4* xs;            // staged activations: [step][8 vectors][NCG column groups][4 units][16 columns] pieces
  float* part;          // (K split) partial tiles [split][Q64_COLS columns][np rows]
  int ks, np;
};

template <int T_, int NCG>
__global__ __launch_bounds__(256) void q64_stage_kernel(const QArgs args, const int M, u32x4* __restrict__ xs) {
  using F = Fmt<T_>;
  const int tid = threadIdx.x, scol = (tid & 63) + 64 * blockIdx.y, sug = tid >> 6, s = blockIdx.x;      // this thread's item: activation row scol, unit 4 s + sug
  if (scol >= 16 * NCG) return;
  uint32_t nx[F::UW / 2];
  stage_fetch<T_>(args, scol < M ? scol : 0, 4 * s + sug, nx);
  u32x4 xv[F::XV]; float cs[F::NG];
  F::stage(nx, xv, cs);
  u32x4* dst = xs + (size_t)s * (F::XV * NCG * 64) + (scol >> 4) * 64 + sug * 16 + (scol & 15);
#pragma unroll
  for (int v = 0; v < F::XV; v++) dst[v * NCG * 64] = scol < M ? xv[v] : u32x4{0u, 0u, 0u, 0u};
}

// The RMSNorm in front of a linear (attn_norm -> q / k / v, ffn_norm -> gate / up; nn.RMSNorm, tinygrad/nn/__init__.py:296-304) and q64_stage_kernel in one launch: one
// workgroup per row sums the squares of the float32 row, writes (x rsqrt(mean x^2 + eps)) w rounded to fp16 - rmsnorm_kernel's expression - to xn_out and to LDS, and
// its threads then stage the row's units from LDS.  Workgroups at and beyond M fill their rows of the staged buffer with zeros.
// part != nullptr: the row is first completed in place as x + the sum of the partial tiles a deferred linear left (ks splits of [64][np] float32, in the order of K:
// what q64_reduce_kernel would have written).
template <int T_, int NCG>
__global__ __launch_bounds__(1024) void q64_norm_stage_kernel(float* __restrict__ x, const float* __restrict__ w, const int K, const float eps,
                                                             _Float16* __restrict__ xn_out, u32x4* __restrict__ xs, const int M,
                                                             const float* __restrict__ part, const int ks, const int np) {
  using F = Fmt<T_>;
  extern __shared__ u32x4 lds[];                          // the normalised fp16 row
  __shared__ float red[16];
  const int m = blockIdx.x, tid = threadIdx.x, nu = K >> 6, nth = blockDim.x;      // 256 or 1024 threads: with one 16-byte piece of the row per thread the partial tiles of all splits are requested in one round trip
  auto dst_of = [&](int u) { return xs + (size_t)(u >> 2) * (F::XV * NCG * 64) + (m >> 4) * 64 + (u & 3) * 16 + (m & 15); };
  if (m >= M) {
    for (int u = tid; u < nu; u += nth) {
      u32x4* dst = dst_of(u);
#pragma unroll
      for (int v = 0; v < F::XV; v++) dst[v * NCG * 64] = u32x4{0u, 0u, 0u, 0u};
    }
    return;
  }
  f32x4* xr = (f32x4*)(x + (size_t)m * K);
  const f32x4* wr = (const f32x4*)w;
  const int n4 = K >> 2;
  float s = 0.f;
  for (int i = tid; i < n4; i += nth) {
    f32x4 v = xr[i];
    if (part) {                                           // (the same thread reads this piece again below: its own store, in program order)
      for (int k0 = 0; k0 < ks; k0 += 8) {                // eight splits requested together, added in the order of K
        f32x4 t[8];
#pragma unroll
        for (int k = 0; k < 8; k++) t[k] = *(const f32x4*)(part + ((size_t)(k0 + k < ks ? k0 + k : ks - 1) * Q64_COLS + m) * np + 4 * i);
#pragma unroll
        for (int k = 0; k < 8; k++) if (k0 + k < ks) { v.x += t[k].x; v.y += t[k].y; v.z += t[k].z; v.w += t[k].w; }
      }
      xr[i] = v;
    }
    s += v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w;
  }
  s = wave_sum(s);
  if ((tid & 63) == 0) red[tid >> 6] = s;
  __syncthreads();
  float tot = 0.f;
  for (int j = 0; j < (nth >> 6); j++) tot += red[j];
  const float scale = 1.0f / sqrtf(tot / (float)K + eps);
  uint32_t* row32 = (uint32_t*)lds;
  uint32_t* out32 = (uint32_t*)(xn_out + (size_t)m * K);
  for (int i = tid; i < n4; i += nth) {
    const f32x4 v = xr[i], g = wr[i];
    const uint32_t lo = f2h_bits((v.x * scale) * g.x) | (f2h_bits((v.y * scale) * g.y) << 16), hi = f2h_bits((v.z * scale) * g.z) | (f2h_bits((v.w * scale) * g.w) << 16);
    row32[2 * i] = lo; row32[2 * i + 1] = hi;
    if (xn_out) { out32[2 * i] = lo; out32[2 * i + 1] = hi; }
  }
  __syncthreads();
  QArgs q = {};
  q.x = (const void*)lds; q.x_f32 = 0; q.K = K;
  for (int u = tid; u < nu; u += nth) {
    uint32_t nx[F::UW / 2];
    stage_fetch<T_>(q, 0, u, nx);
    u32x4 xv[F::XV]; float cs[F::NG];
    F::stage(nx, xv, cs);
    u32x4* dst = dst_of(u);
#pragma unroll
    for (int v = 0; v < F::XV; v++) dst[v * NCG * 64] = xv[v];
  }
}

template <int T_, bool MS, bool SW, int NCG, int NT>
__global__ __launch_bounds__(512) void qgemm64_kernel(const QArgs args, const int M, const Q64X ex) {
  const QArgs a = args;
  using F = Fmt<T_>;
  typedef typename F::Raw Raw;
  static_assert(F::UW == 64 && F::XV == 8, "units of 64 weights in eight vectors");
  static_assert(!(MS && SW), "the SwiGLU pair is not combined with the q / k / v walk");
  constexpr int SP = F::XV * NCG * 64;                    // 16-byte pieces of one stage
  constexpr int NI = SP / 256;                            // pieces per thread and stage (4, 8 or 16)
  extern __shared__ u32x4 lds[];                          // two stages of SP pieces
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 15, g = lane >> 4;
  uint32_t kc[F::NKC];
  F::consts(kc);
  const int nsteps = a.nu >> 2;                           // (the launch has checked: whole steps)
  const int ky = blockIdx.y, s0 = (int)((long long)ky * nsteps / ex.ks), n = (int)((long long)(ky + 1) * nsteps / ex.ks) - s0;   // this workgroup's steps
  constexpr int WR = SW ? 8 : 16;                         // output rows of one weight tile
  // The NT weight tiles of this wave, 16 weight rows each (SwiGLU: 8 gate rows and the same 8 up rows).  A tile lies in one segment (q / k / v: every segment a
  // multiple of 16 rows); rows at and beyond the segment's end repeat its last one.
  long long grow0[NT], row0[NT], nrows[NT]; int sg[NT]; bool has_rows[NT]; const uint8_t* rowp[NT];
#pragma unroll
  for (int t = 0; t < NT; t++) {
    grow0[t] = (((long long)blockIdx.x * 4 + wave) * NT + t) * WR;     // first output row of the tile (over all segments)
    row0[t] = grow0[t];
    const uint8_t* wb = a.w[0]; nrows[t] = a.n[0]; sg[t] = 0;
    if constexpr (MS) {
      if (row0[t] >= a.n[0]) {
        row0[t] -= a.n[0]; sg[t] = 1; wb = a.w[1]; nrows[t] = a.n[1];
        if (a.nseg > 2 && row0[t] >= a.n[1]) { row0[t] -= a.n[1]; sg[t] = 2; wb = a.w[2]; nrows[t] = a.n[2]; }
      }
    }
    has_rows[t] = row0[t] < nrows[t];
    long long wrow = row0[t] + (SW ? (r & 7) : r); wrow = wrow < nrows[t] ? wrow : nrows[t] - 1; wrow = wrow < 0 ? 0 : wrow;
    rowp[t] = ((SW && r >= 8) ? a.w[1] : wb) + wrow * a.row_bytes;
  }

  // Waves 4 .. 7 stage: wave 4 + w copies pieces 64 (NI w + j) + lane, j < NI, of every stage - 1 KB per instruction - two steps ahead of its use, through two
  // register sets in turn.  They issue nothing else, so these loads (L2 hits) never queue behind a weight load from HBM: loads return in the order of issue,
  // and a copy requested by the multiplying waves themselves arrived no earlier than the weights requested a step before it.
  if (wave >= 4) {
    const int sw = wave - 4;
    u32x4 xa[NI], xb[NI];
    auto fetch = [&](int i, u32x4 (&xr)[NI]) __attribute__((always_inline)) {
      const u32x4* src = ex.xs + (size_t)(s0 + (i < n ? i : n - 1)) * SP + sw * NI * 64 + lane;   // (past the end: the last stage again, never written to LDS)
#pragma unroll
      for (int j = 0; j < NI; j++) xr[j] = src[j * 64];
    };
    auto put = [&](int st, const u32x4 (&xr)[NI]) __attribute__((always_inline)) {
      u32x4* dst = lds + st * SP + sw * NI * 64 + lane;
#pragma unroll
      for (int j = 0; j < NI; j++) dst[j * 64] = xr[j];
    };
    fetch(0, xa); fetch(1, xb);
    put(0, xa);
    fetch(2, xa);
    __syncthreads();
    int i = 0;                                            // step i: stage i + 1 goes to LDS (requested two steps ago), stage i + 3 is requested
    for (; i + 2 <= n; i += 2) {
      put((i + 1) & 1, xb); fetch(i + 3, xb); __syncthreads();
      put(i & 1, xa); fetch(i + 4, xa); __syncthreads();
    }
    if (i < n) { put((i + 1) & 1, xb); __syncthreads(); }
    return;
  }
  constexpr int RD = Q64_RING;                            // weight steps in flight, the one being multiplied included
  Raw wq[RD][NT];
#pragma unroll
  for (int k = 0; k < RD - 1; k++)
#pragma unroll
    for (int t = 0; t < NT; t++) wq[k][t] = F::load(rowp[t], 4 * (s0 + (k < n ? k : n - 1)) + g);
  __syncthreads();
  v4f32 acc[NT][NCG];
#pragma unroll
  for (int t = 0; t < NT; t++)
#pragma unroll
    for (int cg = 0; cg < NCG; cg++) acc[t][cg] = v4f32{0.f, 0.f, 0.f, 0.f};
  auto compute = [&](const Raw (&buf)[NT], int slot) __attribute__((always_inline)) {
    uint32_t wv[NT][F::NWV];
#pragma unroll
    for (int t = 0; t < NT; t++) { F::decode(buf[t], wv[t], kc); F::to_f16(buf[t], wv[t]); }
    const u32x4* src = lds + slot * SP + lane;
    u32x4 bv[2][NCG];                                     // a B operand is read once and meets the NT weight tiles; the operands of vector v + 1 are requested before
#pragma unroll                                            // vector v is multiplied (left to itself the compiler waits for every pair of reads right behind them)
    for (int cg = 0; cg < NCG; cg++) bv[0][cg] = src[cg * 64];
#pragma unroll
    for (int v = 0; v < F::XV; v++) {
      if (v + 1 < F::XV) {
#pragma unroll
        for (int cg = 0; cg < NCG; cg++) bv[(v + 1) & 1][cg] = src[((v + 1) * NCG + cg) * 64];
      }
#pragma unroll
      for (int t = 0; t < NT; t++) {
        const u32x4 av = {wv[t][4 * v], wv[t][4 * v + 1], wv[t][4 * v + 2], wv[t][4 * v + 3]};
#pragma unroll
        for (int cg = 0; cg < NCG; cg++)
          acc[t][cg] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8f16, av), __builtin_bit_cast(v8f16, bv[v & 1][cg]), acc[t][cg], 0, 0, 0);
      }
    }
  };
  auto step = [&](const Raw (&cur)[NT], Raw (&nxt2)[NT], int i) __attribute__((always_inline)) {
    const int i2 = i + RD - 1 < n ? i + RD - 1 : n - 1;
#pragma unroll
    for (int t = 0; t < NT; t++) nxt2[t] = F::load(rowp[t], 4 * (s0 + i2) + g);
    compute(cur, i & 1);
    __syncthreads();
  };
  int i = 0;
  for (; i + RD <= n; i += RD) {
#pragma unroll
    for (int k = 0; k < RD; k++) step(wq[k], wq[(k + RD - 1) % RD], i + k);
  }
#pragma unroll
  for (int k = 0; k < RD - 1; k++) if (i < n) { step(wq[k], wq[(k + RD - 1) % RD], i); i++; }

  // ---- epilogue: lane (g, c) holds, per tile and column group, activation row 16 cg + c x weight rows 4 g .. 4 g + 3 of the tile
  const int c = r;
  if constexpr (SW && NT == 2) {
    // silu(gate) * up in the layout the consuming linear multiplies from: the workgroup's 64 output rows are one unit of that linear's K, so the unit's eight
    // vectors for every column are assembled in LDS (the stages are free now; the staging waves have left) and leave as 16-byte pieces, 256-byte runs per (vector,
    // column group).  (As 2-byte stores straight from the accumulators the launch took 40.5 instead of 32 us.)  Not for a Q6_K consumer, whose units are not 64
    // consecutive values: its rows take the general path below.
    if (a.y_stage_fmt && a.y_stage_fmt != GGML_Q6_K) {
      uint16_t* tile = (uint16_t*)lds;                    // [vector][column group][column] pieces of eight halves
#pragma unroll
      for (int t = 0; t < NT; t++) {
#pragma unroll
        for (int cg = 0; cg < NCG; cg++) {
          float up[4];
#pragma unroll
          for (int k = 0; k < 4; k++) up[k] = __shfl_down(acc[t][cg][k], 32, 64);
          if (g < 2) {
#pragma unroll
            for (int k = 0; k < 4; k++) {
              const int lrow = (wave * NT + t) * 8 + 4 * g + k;                  // row inside the unit
              const int hw = a.y_stage_fmt == GGML_F16 ? lrow : staged_pos(a.y_stage_fmt, lrow, 1);     // vector hw / 8, half hw % 8
              const _Float16 hv = 16 * cg + c < M ? (_Float16)(silu_f(acc[t][cg][k]) * up[k]) : (_Float16)0.f;
              tile[(((hw >> 3) * NCG + cg) * 16 + c) * 8 + (hw & 7)] = __builtin_bit_cast(uint16_t, hv);
            }
          }
        }
      }
      asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");            // (the four multiplying waves: the others have ended)
      const long long u = blockIdx.x;                     // the consumer's unit
      u32x4* dst = (u32x4*)a.y[0] + (size_t)(u >> 2) * (F::XV * NCG * 64) + (u & 3) * 16;
      for (int p = tid; p < F::XV * NCG * 16; p += 256) dst[(p >> 4) * 64 + (p & 15)] = lds[p];
      return;
    }
  }
#pragma unroll
  for (int t = 0; t < NT; t++) {
    if (ex.ks > 1) {                                      // partial tile: [split][column][padded row], every lane stores its four rows
#pragma unroll
      for (int cg = 0; cg < NCG; cg++)
        *(v4f32*)(ex.part + ((size_t)ky * Q64_COLS + 16 * cg + c) * ex.np + grow0[t] + 4 * g) = acc[t][cg];
      continue;
    }
    if (!has_rows[t]) continue;
    if constexpr (SW) {
#pragma unroll
      for (int cg = 0; cg < NCG; cg++) {
        float up[4];
#pragma unroll
        for (int k = 0; k < 4; k++) up[k] = __shfl_down(acc[t][cg][k], 32, 64);
        const int col = 16 * cg + c;
        if (a.y_stage_fmt) {                              // fp16 rows in the layout the consuming linear multiplies from (its K = these rows); rows at and beyond M as zeros
          if (g < 2) {
#pragma unroll
            for (int k = 0; k < 4; k++) {
              const long long row = row0[t] + 4 * g + k;
              if (row < nrows[t]) ((_Float16*)a.y[0])[rows_staged_pos(a.y_stage_fmt, (int)row, col, NCG)] = col < M ? (_Float16)(silu_f(acc[t][cg][k]) * up[k]) : (_Float16)0.f;
            }
          }
        } else if (g < 2 && col < M) {
#pragma unroll
          for (int k = 0; k < 4; k++) {
            const long long row = row0[t] + 4 * g + k;
            if (row < nrows[t]) {
              const float v = silu_f(acc[t][cg][k]) * up[k];
              const long long o = (long long)col * nrows[t] + row;
              if (a.y_f32) ((float*)a.y[0])[o] = v; else ((_Float16*)a.y[0])[o] = (_Float16)v;
            }
          }
        }
      }
    } else {
      void* yb = !MS ? a.y[0] : sg[t] == 0 ? a.y[0] : sg[t] == 1 ? a.y[1] : a.y[2];
      const float* rb = a.epilogue == 1 ? (!MS ? a.resid[0] : sg[t] == 0 ? a.resid[0] : sg[t] == 1 ? a.resid[1] : a.resid[2]) : nullptr;
#pragma unroll
      for (int cg = 0; cg < NCG; cg++) {
        const int col = 16 * cg + c;
        if (col < M) {
#pragma unroll
          for (int k = 0; k < 4; k++) {
            const long long row = row0[t] + 4 * g + k;
            if (row < nrows[t]) {
              const long long o = (long long)col * nrows[t] + row;
              float v = acc[t][cg][k];
              if (rb) v += rb[o];
              if (a.y_f32) ((float*)yb)[o] = v; else ((_Float16*)yb)[o] = (_Float16)v;
            }
          }
        }
      }
    }
  }
}

// y = [residual +] sum over the splits, in the order of K.  One thread per (activation row, four consecutive padded weight rows).
__global__ __launch_bounds__(256) void q64_reduce_kernel(const QArgs a, const int M, const float* __restrict__ part, const int ks, const int np) {
  const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
  const int q = np >> 2;
  const int m = (int)(idx / q); long long row = 4 * (idx - (long long)m * q);
  if (m >= M) return;
  v4f32 v = *(const v4f32*)(part + (size_t)m * np + row);
  for (int k0 = 1; k0 < ks; k0 += 8) {                   // eight splits requested together (one round trip), added in the order of K
    v4f32 t[8];
#pragma unroll
    for (int k = 0; k < 8; k++) t[k] = *(const v4f32*)(part + ((size_t)(k0 + k < ks ? k0 + k : ks - 1) * Q64_COLS + m) * np + row);
#pragma unroll
    for (int k = 0; k < 8; k++) if (k0 + k < ks) v += t[k];
  }
  int sg = 0; long long nrows = a.n[0];
  if (a.nseg > 1 && row >= a.n[0]) { row -= a.n[0]; sg = 1; nrows = a.n[1]; if (a.nseg > 2 && row >= a.n[1]) { row -= a.n[1]; sg = 2; nrows = a.n[2]; } }
  void* yb = sg == 0 ? a.y[0] : sg == 1 ? a.y[1] : a.y[2];
  const float* rb = a.epilogue == 1 ? (sg == 0 ? a.resid[0] : sg == 1 ? a.resid[1] : a.resid[2]) : nullptr;
#pragma unroll
  for (int k = 0; k < 4; k++) {
    if (row + k < nrows) {
      const long long o = (long long)m * nrows + row + k;
      float t = v[k];
      if (rb) t += rb[o];
      if (a.y_f32) ((float*)yb)[o] = t; else ((_Float16*)yb)[o] = (_Float16)t;
    }
  }
}

// ---------------------------------------------------------------------------------------------------------------- workspace
static uint8_t* g_q64_ws[Q64_MAX_DEVICES];                 // device d: Q64_SLOTS x (staged activations, partial tiles), allocated by tga_qgemm64_setup(d)
static hipStream_t g_q64_owner[Q64_MAX_DEVICES][Q64_SLOTS];
static bool g_q64_taken[Q64_MAX_DEVICES][Q64_SLOTS];
static std::mutex g_q64_mu;

int tga_qgemm64_setup(int device) {                         // called by tga_init after hipSetDevice(device)
  TGA_REQUIRE(device >= 0 && device < Q64_MAX_DEVICES, "tga_init: device %d is beyond the %d devices the prefill workspace table covers", device, Q64_MAX_DEVICES);
  std::lock_guard<std::mutex> lk(g_q64_mu);
  if (g_q64_ws[device]) return 0;
  void* p = nullptr;
  TGA_HIP(hipMalloc(&p, Q64_SLOTS * (Q64_XS_BYTES + Q64_PART_BYTES)));
  g_q64_ws[device] = (uint8_t*)p;
  return 0;
}

static uint8_t* q64_slot(hipStream_t s) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= Q64_MAX_DEVICES) return nullptr;
  std::lock_guard<std::mutex> lk(g_q64_mu);
  if (!g_q64_ws[dev]) return nullptr;
  int free_slot = -1;
  for (int i = 0; i < Q64_SLOTS; i++) {
    if (g_q64_taken[dev][i] && g_q64_owner[dev][i] == s) return g_q64_ws[dev] + (size_t)i * (Q64_XS_BYTES + Q64_PART_BYTES);
    if (!g_q64_taken[dev][i] && free_slot < 0) free_slot = i;
  }
  if (free_slot < 0) return nullptr;
  g_q64_taken[dev][free_slot] = true; g_q64_owner[dev][free_slot] = s;
  return g_q64_ws[dev] + (size_t)free_slot * (Q64_XS_BYTES + Q64_PART_BYTES);
}

// The stream is about to be destroyed (tga_stream_destroy, which has waited for its work): the slot it holds, on whichever device, is free again.
void tga_qgemm64_release(hipStream_t s) {
  std::lock_guard<std::mutex> lk(g_q64_mu);
  for (int d = 0; d < Q64_MAX_DEVICES; d++)
    for (int i = 0; i < Q64_SLOTS; i++)
      if (g_q64_taken[d][i] && g_q64_owner[d][i] == s) g_q64_taken[d][i] = false;
}

static int q64_split(bool sw, long long tiles, int nsteps, int ncg) {   // workgroups per row tile: about 512 workgroups (256 with eight column groups: one per CU) of at least four steps, partial tiles within the workspace
  static const int env_ks = getenv("TGA_Q64_KS") ? atoi(getenv("TGA_Q64_KS")) : 0;
  int ks = 1;
  if (!sw && tiles < 192) {
    ks = (int)(((ncg == 8 ? 256 : 512) + tiles / 2) / tiles);
    if (ks > nsteps / 4) ks = nsteps / 4;
  }
  if (env_ks >= 1 && !sw) ks = env_ks < nsteps ? env_ks : nsteps;
  if (ks < 1) ks = 1;
  return ks;
}

template <int T, bool MS, bool SW, int NCG, int NT>
static int launch_q64_v(const QArgs& a, int M, uint8_t* ws, Q64Opt& o, hipStream_t s) {
  using F = Fmt<T>;
  auto kern = qgemm64_kernel<T, MS, SW, NCG, NT>;
  constexpr size_t stage_bytes = (size_t)F::XV * NCG * 64 * 16;
  static const hipError_t configured = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)(2 * stage_bytes));
  TGA_HIP(configured);
  const int nsteps = a.nu >> 2;
  const long long tiles = (a.ntot + 64 * NT / (SW ? 2 : 1) - 1) / (64 * NT / (SW ? 2 : 1));   // workgroups over the rows: 64 NT weight rows each (SwiGLU: half of them gate rows)
  Q64X ex;
  ex.xs = o.xs_ext ? (u32x4*)o.xs_ext : (u32x4*)ws; ex.part = ws ? (float*)(ws + Q64_XS_BYTES) : nullptr; ex.np = (int)(tiles * 64 * NT);
  // K split: row tiles alone leave most of the 256 CUs idle when the matrix has few rows (not without a workspace slot for the partial tiles)
  int ks = ws ? q64_split(SW, tiles, nsteps, NCG) : 1;
  while (ks > 1 && (size_t)ks * Q64_COLS * ex.np * 4 > Q64_PART_BYTES) ks--;
  ex.ks = ks;
  if (!o.prestaged) {
    q64_stage_kernel<T, NCG><<<dim3((unsigned)nsteps, NCG > 4 ? 2 : 1), dim3(256), 0, s>>>(a, M, ex.xs);
    TGA_LAUNCH_CHECK();
  }
  kern<<<dim3((unsigned)tiles, (unsigned)ks), dim3(512), 2 * stage_bytes, s>>>(a, M, ex);
  TGA_LAUNCH_CHECK();
  o.ks = 0;
  if (ks > 1 && o.defer) { o.part = ex.part; o.ks = ks; o.np = ex.np; }
  else if (ks > 1) {
    const long long items = (long long)M * (ex.np / 4);
    q64_reduce_kernel<<<dim3((unsigned)((items + 255) / 256)), dim3(256), 0, s>>>(a, M, ex.part, ks, ex.np);
    TGA_LAUNCH_CHECK();
  }
  return 0;
}

template <int T, bool MS, bool SW, int NCG>
static int launch_q64_t(const QArgs& a, int M, uint8_t* ws, Q64Opt& o, hipStream_t s) {
  using F = Fmt<T>;
  // Two weight tiles per wave halve the activation bytes that reach a CU (global -> LDS -> operand) per weight; taken when the row tiles of 128, split over K,
  // still fill the chip.  (fp16 weights: a unit is 128 bytes per lane, a ring of three steps for two tiles does not fit the registers.)
  static const int env_nt = getenv("TGA_Q64_NT") ? atoi(getenv("TGA_Q64_NT")) : 0;
  const int nsteps = a.nu >> 2;
  const long long rows_wg2 = SW ? 64 : 128, tiles2 = (a.ntot + rows_wg2 - 1) / rows_wg2;
  bool two = sizeof(typename F::Raw) <= 64 && (NCG == 8 || tiles2 * q64_split(SW, tiles2, nsteps, NCG) >= 224);      // (eight column groups: the LDS reads of the B operands set the pace, and a B operand meets both tiles)
  if (env_nt == 1) two = false; else if (env_nt == 2) two = sizeof(typename F::Raw) <= 64;
  if constexpr (sizeof(typename F::Raw) <= 64) { if (two) return launch_q64_v<T, MS, SW, NCG, 2>(a, M, ws, o, s); }
  return launch_q64_v<T, MS, SW, NCG, 1>(a, M, ws, o, s);
}

template <int T>
static int launch_q64(QArgs a, int M, uint8_t* ws, Q64Opt& o, hipStream_t s) {
  using F = Fmt<T>;
  if constexpr (F::UW != 64 || F::XV != 8) return -1;
  else {
    a.nu = a.K / F::UW;
    a.row_bytes = (long long)(a.K / F::BW) * F::BB;
    // two column groups instead of four: half the MFMAs and half the staged bytes.  (One group, for up to sixteen rows, was measured and dropped: the kernel
    // streams weights at about 2.5 TB/s - Q8_0 14336 x 4096 at M = 8 24.6 us, the Q6_K lm-head 211 us - where the LDS-fed small-batch kernels take 18.4 / 134.)
    // Eight groups (65 .. 128 rows): a pass over the weights costs what it costs at 64 rows - the weight stream, not the matrix cores, sets its pace.
    const int ncg = M <= 32 ? 2 : M <= 64 ? 4 : 8;
    if (a.epilogue == 2) return ncg == 2 ? launch_q64_t<T, false, true, 2>(a, M, ws, o, s) : ncg == 4 ? launch_q64_t<T, false, true, 4>(a, M, ws, o, s) : launch_q64_t<T, false, true, 8>(a, M, ws, o, s);
    if (a.nseg > 1) return ncg == 2 ? launch_q64_t<T, true, false, 2>(a, M, ws, o, s) : ncg == 4 ? launch_q64_t<T, true, false, 4>(a, M, ws, o, s) : launch_q64_t<T, true, false, 8>(a, M, ws, o, s);
    return ncg == 2 ? launch_q64_t<T, false, false, 2>(a, M, ws, o, s) : ncg == 4 ? launch_q64_t<T, false, false, 4>(a, M, ws, o, s) : launch_q64_t<T, false, false, 8>(a, M, ws, o, s);
  }
}

// Whether the call is inside this kernel's range: 17 .. 128 rows of fp16 or float32 activations, K a multiple of 256 up to Q64_MAX_K, one to three matrices
// (several: each a multiple of 16 rows) with the plain or residual epilogue, or the SwiGLU pair, in one of the formats with units of 64 weights.
static bool q64_in_range(int fmt, const QArgs& a, int M) {
  if (M < 17 || M > Q64_COLS || a.K % 256 != 0 || a.K > Q64_MAX_K || a.nseg < 1 || a.nseg > 3 || a.epilogue > 2 || a.sel || a.x_staged || (a.y_stage_fmt && a.epilogue != 2) || a.norm_w || a.comb_y) return false;
  if (a.nseg > 1 && a.epilogue != 2) for (int i = 0; i < a.nseg; i++) if (a.n[i] % 16 != 0) return false;
  if (((uintptr_t)a.x & 15) != 0) return false;
  if (a.y_stage_fmt && (a.y_f32 || a.y_stage_nu != (int)(a.n[0] / 64) || a.n[0] % 256 != 0)) return false;   // (staged SwiGLU rows: the consumer's K is this N)
  switch (fmt) { case F_Q4_0P: case F_Q8_0P: case GGML_Q6_K: case GGML_Q4_K: case GGML_Q5_K: case GGML_IQ4_XS: case GGML_F16: return true; }
  return false;
}

// For a producer that writes the activations in the multiplying layout itself (rows_staged_pos in qfmt.h, ncg column groups): where to, or nullptr when the call
// is outside the kernel's range or the stream holds no workspace slot.  The call that follows passes prestaged = true.
void* tga_qgemm64_staging(int fmt, const QArgs& a, int M, hipStream_t s, int* ncg) {
  if (!q64_in_range(fmt, a, M)) return nullptr;
  *ncg = M <= 32 ? 2 : M <= 64 ? 4 : 8;
  return q64_slot(s);
}

template <int T>
static int launch_norm_stage(float* x, const float* w, int K, float eps, void* xn_out, void* staged, int M, int ncg, const float* part, int ks, int np, hipStream_t s) {
  using F = Fmt<T>;
  if constexpr (F::UW != 64 || F::XV != 8) return -1;
  else {
    static const hipError_t c2 = hipFuncSetAttribute((const void*)q64_norm_stage_kernel<T, 2>, hipFuncAttributeMaxDynamicSharedMemorySize, 65536);
    static const hipError_t c4 = hipFuncSetAttribute((const void*)q64_norm_stage_kernel<T, 4>, hipFuncAttributeMaxDynamicSharedMemorySize, 65536);
    static const hipError_t c8 = hipFuncSetAttribute((const void*)q64_norm_stage_kernel<T, 8>, hipFuncAttributeMaxDynamicSharedMemorySize, 65536);
    TGA_HIP(c2); TGA_HIP(c4); TGA_HIP(c8);
    static const int env_nth = getenv("TGA_NS_THREADS") ? atoi(getenv("TGA_NS_THREADS")) : 0;
    const int nth = env_nth == 256 || env_nth == 1024 ? env_nth : (K >= 4096 ? 1024 : 256);
    if (ncg == 2) q64_norm_stage_kernel<T, 2><<<dim3(32), dim3(nth), (size_t)K * 2, s>>>(x, w, K, eps, (_Float16*)xn_out, (u32x4*)staged, M, part, ks, np);
    else if (ncg == 4) q64_norm_stage_kernel<T, 4><<<dim3(64), dim3(nth), (size_t)K * 2, s>>>(x, w, K, eps, (_Float16*)xn_out, (u32x4*)staged, M, part, ks, np);
    else q64_norm_stage_kernel<T, 8><<<dim3(128), dim3(nth), (size_t)K * 2, s>>>(x, w, K, eps, (_Float16*)xn_out, (u32x4*)staged, M, part, ks, np);
    TGA_LAUNCH_CHECK();
    return 0;
  }
}
// RMSNorm of M float32 rows of K values (K a multiple of 256 up to Q64_MAX_K, x and w 16-byte aligned) into xn_out (fp16 rows; may be null) and into `staged`, the
// buffer of a consumer of format fmt in the multiplying layout (tga_qgemm64_staging's, or the caller's).  part != nullptr: the rows are first completed in place with
// the partial tiles of a deferred linear (ks splits, row pitch np).  -1: outside the range.
int tga_qgemm64_norm_stage(int fmt, float* x, const float* w, int K, float eps, void* xn_out, void* staged, int M, int ncg, const float* part, int ks, int np, hipStream_t s) {
  if ((((uintptr_t)x | (uintptr_t)w | (uintptr_t)xn_out | (uintptr_t)staged | (uintptr_t)part) & 15) != 0 || K % 256 != 0 || K > Q64_MAX_K || M < 1 || M > 16 * ncg || (ncg != 2 && ncg != 4 && ncg != 8)) return -1;
  if (part && (ks < 1 || np < K || np % 4 != 0)) return -1;
  switch (fmt) {
    case F_Q4_0P: return launch_norm_stage<F_Q4_0P>(x, w, K, eps, xn_out, staged, M, ncg, part, ks, np, s);
    case F_Q8_0P: return launch_norm_stage<F_Q8_0P>(x, w, K, eps, xn_out, staged, M, ncg, part, ks, np, s);
    case GGML_Q6_K: return launch_norm_stage<GGML_Q6_K>(x, w, K, eps, xn_out, staged, M, ncg, part, ks, np, s);
    case GGML_Q4_K: return launch_norm_stage<GGML_Q4_K>(x, w, K, eps, xn_out, staged, M, ncg, part, ks, np, s);
    case GGML_Q5_K: return launch_norm_stage<GGML_Q5_K>(x, w, K, eps, xn_out, staged, M, ncg, part, ks, np, s);
    case GGML_IQ4_XS: return launch_norm_stage<GGML_IQ4_XS>(x, w, K, eps, xn_out, staged, M, ncg, part, ks, np, s);
    case GGML_F16: return launch_norm_stage<GGML_F16>(x, w, K, eps, xn_out, staged, M, ncg, part, ks, np, s);
  }
  return -1;
}

// Returns -1 when the call is outside this kernel's range or no workspace slot is left for the stream where one is needed (the caller then runs blocks of
// sixteen rows): activations staged here need the slot; activations staged by the caller (o.xs_ext) run without one, with K unsplit.
int tga_qgemm64_dispatch(int fmt, const QArgs& a, int M, Q64Opt& o, hipStream_t s) {
  if (!q64_in_range(fmt, a, M)) return -1;
  uint8_t* ws = q64_slot(s);
  if (!ws && !(o.prestaged && o.xs_ext)) return -1;
  if (o.defer && (a.epilogue != 1 || a.nseg != 1)) return -1;
  switch (fmt) {
    case F_Q4_0P: return launch_q64<F_Q4_0P>(a, M, ws, o, s);
    case F_Q8_0P: return launch_q64<F_Q8_0P>(a, M, ws, o, s);
    case GGML_Q6_K: return launch_q64<GGML_Q6_K>(a, M, ws, o, s);
    case GGML_Q4_K: return launch_q64<GGML_Q4_K>(a, M, ws, o, s);
    case GGML_Q5_K: return launch_q64<GGML_Q5_K>(a, M, ws, o, s);
    case GGML_IQ4_XS: return launch_q64<GGML_IQ4_XS>(a, M, ws, o, s);
    case GGML_F16: return launch_q64<GGML_F16>(a, M, ws, o, s);
  }
  return -1;
}

// x[m, :] += sum over the splits of the partial tiles a deferred call left (tga_qgemm64_dispatch with o.defer), in the order of K: rows x dim float32, in place
int tga_qgemm64_add_partials(float* x, const float* part, int ks, int np, int rows, int dim, hipStream_t s) {
  QArgs a = {};
  a.nseg = 1; a.n[0] = dim; a.ntot = dim; a.y[0] = x; a.resid[0] = x; a.y_f32 = 1; a.epilogue = 1;
  const long long items = (long long)rows * (np / 4);
  q64_reduce_kernel<<<dim3((unsigned)((items + 255) / 256)), dim3(256), 0, s>>>(a, rows, part, ks, np);
  TGA_LAUNCH_CHECK();
  return 0;
}
