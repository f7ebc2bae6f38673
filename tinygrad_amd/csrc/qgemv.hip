// Fused GGUF block dequant + GEMV / small-batch GEMM (1 <= M <= 8; 9 .. 16 rows for the chunked prefill, see qlinear_multi_impl) for gfx950.
//
// Replaces the kernel(s) tinygrad schedules for  x.linear(W.T)  (tinygrad/nn/__init__.py:177, tinygrad/mixin/op.py:367-392)
// when W is the lazy ggml_data_to_tensor expression over raw GGUF bytes (tinygrad/llm/gguf.py:46,56,68-72,105-114).
//
// Design (bandwidth-bound, no MFMA):
//  * a "unit" is the slice of one weight row a lane owns per step: a PAIR of 32-weight blocks for Q4_0 (36 B) and Q8_0 (68 B),
//    one MXFP4 block (17 B), or a quarter of a Q6_K superblock (64 weights).  Lane l of a wave takes unit l, l+64, ... of a row,
//    so a wave's loads cover a contiguous span of the row; each lane issues 128-bit loads straight from the packed GGUF
//    bytes (no repacking).  Measured on MI355X, dwordx4 loads that are only 2-byte aligned run ~25 % slower than 4-byte
//    aligned ones, so every hot load is 4-byte aligned: block pairs start on 4-byte boundaries, and the 17/210-byte layouts load
//    the enclosing aligned dwords and realign in registers (v_alignbit_b32 / 64-bit shift).  An aligned dword that holds at
//    least one byte of the tensor never leaves that byte's page, so the realigned loads cannot fault past the buffer.
//    Shapes whose rows are not pair-aligned (odd K/32, or a 2-byte aligned base) take a single-block fallback format.
//  * nibbles / bytes are turned into fp16 with biased-exponent tricks in registers (v_and_or_b32, v_perm_b32,
//    v_cvt_scalef32_pk_f16_fp4) and multiplied with v_dot2_f32_f16 (two fp16 products, float32 accumulate).  The integer offset
//    (-8, -32, +128 bias, plus the 1024/64 exponent bias) is removed with a per-unit correction  c = -bias * sum(x)  that is
//    computed once per workgroup when the activations are staged, and used as the accumulator's start value.
//  * activations (fp16, or fp32 rounded to fp16) are staged once per workgroup into LDS in the pair order the decode
//    produces, [vector t][unit] so that every ds_read_b128 is conflict-free.
//  * a wave owns whole rows: K is reduced inside the lane, then across the wave with DPP adds (no LDS, no atomics).
//  * when M*K activations do not fit LDS the kernel walks K in chunks with one row group per wave (accumulators stay in
//    registers across chunks).
#include "qfmt.h"

// ------------------------------------------------------------------------------------------------ kernel
template <int T, int M>
__device__ __forceinline__ void unit_dot(const typename Fmt<T>::Raw& raw, const u32x4* xs, const float* cs, int cu, int ul, float* acc, const uint32_t* kc) {
  using F = Fmt<T>;
  uint32_t wv[F::NWV];
  F::decode(raw, wv, kc);
  constexpr int VPG = F::XV / F::NG;   // x vectors per accumulator group
#pragma unroll
  for (int m = 0; m < M; m++) {
    float g[F::NG], cc[F::NG];
#pragma unroll
    for (int j = 0; j < F::NG; j++) {
      float s = cs[(m * F::NG + j) * cu + ul];
      cc[j] = s;
#pragma unroll
      for (int v = 0; v < VPG; v++) {
        const u32x4 xv = xs[(m * F::XV + j * VPG + v) * cu + ul];
        const int wi = 4 * (j * VPG + v);
        s = dot2(wv[wi + 0], xv.x, s); s = dot2(wv[wi + 1], xv.y, s); s = dot2(wv[wi + 2], xv.z, s); s = dot2(wv[wi + 3], xv.w, s);
      }
      g[j] = s;
    }
    acc[m] += F::finish(raw, wv, g, cc);
  }
}

// R rows of one unit against the M staged activation rows: the R weight slices are decoded first, then each activation's
// vectors are read from LDS ONCE and used for all R rows (the LDS traffic per weight byte falls with R; at M = 8 it is what
// bounds the kernel).
template <int T, int M, int R>
__device__ __forceinline__ void unit_dot_rows(const typename Fmt<T>::Raw* raw, const u32x4* xs, const float* cs, int cu, int ul, float (&acc)[R][M], const uint32_t* kc) {
  using F = Fmt<T>;
  uint32_t wv[R][F::NWV];
#pragma unroll
  for (int r = 0; r < R; r++) F::decode(raw[r], wv[r], kc);
  constexpr int VPG = F::XV / F::NG;   // x vectors per accumulator group
#pragma unroll
  for (int m = 0; m < M; m++) {
    float g[R][F::NG], cc[F::NG];
#pragma unroll
    for (int j = 0; j < F::NG; j++) {
      const float c0 = cs[(m * F::NG + j) * cu + ul];
      cc[j] = c0;
      float s[R];
#pragma unroll
      for (int r = 0; r < R; r++) s[r] = c0;
#pragma unroll
      for (int v = 0; v < VPG; v++) {
        const u32x4 xv = xs[(m * F::XV + j * VPG + v) * cu + ul];
        const int wi = 4 * (j * VPG + v);
#pragma unroll
        for (int r = 0; r < R; r++) {
          s[r] = dot2(wv[r][wi + 0], xv.x, s[r]); s[r] = dot2(wv[r][wi + 1], xv.y, s[r]); s[r] = dot2(wv[r][wi + 2], xv.z, s[r]); s[r] = dot2(wv[r][wi + 3], xv.w, s[r]);
        }
      }
#pragma unroll
      for (int r = 0; r < R; r++) g[r][j] = s[r];
    }
#pragma unroll
    for (int r = 0; r < R; r++) acc[r][m] += F::finish(raw[r], wv[r], g[r], cc);
    // one activation row's vectors live at a time: without this the scheduler hoists the LDS reads of all M rows (M x 32 VGPRs)
    if constexpr (M * R > 4) __builtin_amdgcn_sched_barrier(0);
  }
}

// Reduce R x M partial sums across the wave and let lane 63 write rows row0 .. row0+R-1 of segment `seg` (rows >= row_end are
// skipped; ld = rows of the segment = leading dimension of y).  Epilogue 2 (SwiGLU) treats the two accumulator rows as
// (gate, up) of output row row0.
template <int M, int R>
__device__ __forceinline__ void store_rows(const QArgs& a, int seg, long long row0, long long row_end, long long ld, float (&acc)[R][M]) {
#pragma unroll
  for (int r = 0; r < R; r++)
#pragma unroll
    for (int m = 0; m < M; m++) acc[r][m] = wave_sum_lane63(acc[r][m]);
  if ((threadIdx.x & 63) != 63) return;
  if (a.epilogue == 2) {
    if constexpr (R == 2) {
#pragma unroll
      for (int m = 0; m < M; m++) {
        const float v = silu_f(acc[0][m]) * acc[1][m];
        const long long o = (long long)m * ld + row0;
        if (a.y_f32) ((float*)a.y[0])[o] = v; else ((_Float16*)a.y[0])[o] = (_Float16)v;
      }
    }
    return;
  }
#pragma unroll
  for (int r = 0; r < R; r++) {
    if (row0 + r >= row_end) continue;
#pragma unroll
    for (int m = 0; m < M; m++) {
      const long long o = (long long)m * ld + row0 + r;
      float v = acc[r][m];
      if (a.epilogue == 1) v += a.resid[seg][o];
      if (a.y_f32) ((float*)a.y[seg])[o] = v; else ((_Float16*)a.y[seg])[o] = (_Float16)v;
    }
  }
}

// The wave's slice [lo, hi) of a segment's rows (SwiGLU: of the paired gate/up rows), walked as a software pipeline over
// "steps" (R rows x one 64-unit slice of K): the loads of step s+1 are in flight while step s is multiplied.
// PRIMED: the first step's loads were already issued into b0 before the activations were staged.
template <int T, int M, int R>
struct RowWalker {
  using F = Fmt<T>;
  typedef typename F::Raw Raw;
  const QArgs& a; const u32x4* xs; const float* cs; const uint32_t* kc;
  int cu, iters, lane;
  // load stream
  const uint8_t* base[R]; long long l_row, hi; int l_it;
  __device__ __forceinline__ void issue(Raw* buf) {
    const int u = l_it * 64 + lane;
    if (u < cu) {
#pragma unroll
      for (int r = 0; r < R; r++) {
        long long row = (a.epilogue == 2) ? l_row : l_row + r;
        if (row > hi - 1) row = hi - 1;                      // ragged last group: reload a valid row, the result is dropped
        buf[r] = F::load(base[(a.epilogue == 2) ? r : 0] + row * a.row_bytes, u);
      }
    }
    if (++l_it == iters) { l_it = 0; l_row += (a.epilogue == 2) ? 1 : R; }
  }
};

template <int T, int M, int R>
__global__ __launch_bounds__(QG_THREADS) void qgemv_kernel(const QArgs a) {
  using F = Fmt<T>;
  typedef typename F::Raw Raw;
  extern __shared__ u32x4 lds[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);   // wave-uniform: row pointers stay in SGPRs
  const long long gw = (long long)blockIdx.x * QG_WAVES + wave, nw = (long long)gridDim.x * QG_WAVES;
  const int RS = (a.epilogue == 2) ? 1 : R;                            // output rows per row group
  const long long ngroups = (a.ntot + RS - 1) / RS;
  uint32_t kc[F::NKC];
  F::consts(kc);
  float acc[R][M];
#pragma unroll
  for (int r = 0; r < R; r++)
#pragma unroll
    for (int m = 0; m < M; m++) acc[r][m] = 0.f;

  if (a.nchunks == 1) {
    // contiguous share of the row groups for this wave: groups [g0, g1), sizes differing by at most one
    const long long gbase = ngroups / nw, grem = ngroups % nw;
    const long long g0 = gw * gbase + (gw < grem ? gw : grem), g1 = g0 + gbase + (gw < grem ? 1 : 0);
    const long long row_lo = g0 * RS, row_hi = g1 * RS < a.ntot ? g1 * RS : a.ntot;
    const int cu = a.nu, iters = (cu + 63) >> 6;
    u32x4* xs = lds; float* cs = (float*)(lds + M * F::XV * cu);
    RowWalker<T, M, R> wk{a, xs, cs, kc, cu, iters, lane};
    Raw b0[R], b1[R];
    bool staged = false;
    long long seg_start = 0;
    const int nseg = (a.epilogue == 2) ? 1 : a.nseg;
    for (int seg = 0; seg < nseg; seg++) {
      const long long seg_rows = a.n[seg];
      // this wave's rows inside the segment, as local row indices [lo, hi)
      long long lo = row_lo - seg_start, hi = row_hi - seg_start;
      if (lo < 0) lo = 0;
      if (hi > seg_rows) hi = seg_rows;
      seg_start += seg_rows;
      const long long nrg = hi > lo ? (hi - lo + RS - 1) / RS : 0, nsteps = nrg * iters;
      wk.base[0] = a.w[seg]; if constexpr (R > 1) { if (a.epilogue == 2) wk.base[1] = a.w[1]; }
      wk.l_row = lo; wk.hi = hi; wk.l_it = 0;
      if (nsteps) wk.issue(b0);
      if (!staged) { stage_chunk<T, M>(a, xs, cs, 0, cu); __syncthreads(); staged = true; }
      long long c_row = lo; int c_it = 0;
      auto compute = [&](const Raw* buf) {
        const int u = c_it * 64 + lane;
        if (u < cu) unit_dot_rows<T, M, R>(buf, xs, cs, cu, u, acc, kc);
        if (++c_it == iters) {
          store_rows<M, R>(a, seg, c_row, hi, seg_rows, acc);
#pragma unroll
          for (int r = 0; r < R; r++)
#pragma unroll
            for (int m = 0; m < M; m++) acc[r][m] = 0.f;
          c_it = 0; c_row += RS;
        }
      };
      for (long long s = 0; s < nsteps; s += 2) {
        if (s + 1 < nsteps) wk.issue(b1);
        compute(b0);
        if (s + 1 < nsteps) {
          if (s + 2 < nsteps) wk.issue(b0);
          compute(b1);
        }
      }
    }
    if (!staged) { stage_chunk<T, M>(a, xs, cs, 0, cu); __syncthreads(); }   // keep the barrier count uniform across waves
  } else {
    // K walked in LDS-sized chunks; one row group per wave (the host sizes the grid so that gw covers every group)
    const bool active = gw < ngroups;
    // locate the group's segment and local row (rows of a group never straddle a segment: host enforces R == 1 or nseg == 1)
    long long row = (active ? gw : 0) * RS; int seg = 0;
    if (a.epilogue != 2) while (seg + 1 < a.nseg && row >= a.n[seg]) { row -= a.n[seg]; seg++; }
    const long long seg_rows = a.n[seg];
    const uint8_t* rp[R];
#pragma unroll
    for (int r = 0; r < R; r++) {
      long long rr = (a.epilogue == 2) ? row : (row + r < seg_rows ? row + r : seg_rows - 1);
      rp[r] = a.w[(a.epilogue == 2) ? r : seg] + rr * a.row_bytes;
    }
    for (int ch = 0; ch < a.nchunks; ch++) {
      const int u0 = ch * a.chunk_u, cu = min(a.chunk_u, a.nu - u0);
      u32x4* xs = lds; float* cs = (float*)(lds + M * F::XV * cu);
      __syncthreads();
      stage_chunk<T, M>(a, xs, cs, u0, cu);
      __syncthreads();
      if (active) {
        for (int ul = lane; ul < cu; ul += 64) {
          Raw raw[R];
#pragma unroll
          for (int r = 0; r < R; r++) raw[r] = F::load(rp[r], u0 + ul);
          unit_dot_rows<T, M, R>(raw, xs, cs, cu, ul, acc, kc);
        }
      }
    }
    if (active) store_rows<M, R>(a, seg, row, seg_rows, seg_rows, acc);
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
  constexpr int BUDGET = QG_LDS_BUDGET - fmt_tab<F>();      // (a format's tables share the CU's LDS with the staged activations)
  if ((long long)per_unit * a.nu <= BUDGET) {
    a.nchunks = 1; a.chunk_u = a.nu;
    lds = (size_t)per_unit * a.nu;
    // resident workgroups per CU by LDS (160 KB), capped at 4 (16 waves); never more workgroups than row groups need
    int per_cu = (int)((160 * 1024) / (lds + 256)); if (per_cu > 4) per_cu = 4; if (per_cu < 1) per_cu = 1;
    grid = (long long)cu_count() * per_cu;
    const long long need = (ngroups + QG_WAVES - 1) / QG_WAVES;
    if (grid > need) grid = need;
  } else {
    int cu = (QG_LDS_BUDGET / 2 - fmt_tab<F>()) / per_unit;   // two workgroups per CU
    cu -= cu % 64; if (cu < 64) cu = 64;                   // whole waves of units (64 is a multiple of every format's units per block)
    TGA_REQUIRE((long long)cu * per_unit <= BUDGET, "tga_qlinear: activations of one K chunk do not fit LDS");
    a.chunk_u = cu; a.nchunks = (a.nu + cu - 1) / cu;
    lds = (size_t)per_unit * cu;
    grid = (ngroups + QG_WAVES - 1) / QG_WAVES;
  }
  if (grid < 1) grid = 1;
  auto kern = qgemv_kernel<T, M, R>;
  if (lds > 48 * 1024) {
    static const hipError_t configured = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, BUDGET);   // once per instantiation, thread-safe
    TGA_HIP(configured);
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
  const bool chunked = (long long)M * (16 * Fmt<T>::XV + 4 * Fmt<T>::NG) * (a.K / Fmt<T>::UW) > QG_LDS_BUDGET - fmt_tab<Fmt<T>>();
  // (chunked K with several segments needs one row per group: a group must not straddle a segment)
  if ((chunked && a.nseg > 1) || a.ntot < (long long)cu_count() * QG_WAVES * 2) return launch_qgemv<T, M, 1>(a, s);
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

int tga_qgemv1_dispatch(int fmt, const QArgs& a, hipStream_t s);   // qgemv1.hip
int tga_qgemm_mfma_dispatch(int fmt, const QArgs& a, int M, hipStream_t s);   // qgemm.hip
int tga_qgemm_dma_dispatch(int fmt, const QArgs& a, int M, hipStream_t s);    // qgemm_dma.hip
int tga_qgemm_wp_checked_dispatch(int fmt, const QArgs& a, int M, hipStream_t s);   // qgemm_dma.hip / qgemm_wp.hip
int tga_qgemv1_multi_dispatch(int fmt, const QArgs& a, int M, hipStream_t s); // qgemv1_multi.hip
struct Q64Opt { bool prestaged; const void* xs_ext; bool defer; float* part; int ks, np; };   // qgemm64.hip
int tga_qgemm64_dispatch(int fmt, const QArgs& a, int M, Q64Opt& o, hipStream_t s);            // qgemm64.hip
int tga_qgemm64_add_partials(float* x, const float* part, int ks, int np, int rows, int dim, hipStream_t s);   // qgemm64.hip
void* tga_qgemm64_staging(int fmt, const QArgs& a, int M, hipStream_t s, int* ncg);              // qgemm64.hip
int tga_qgemm64_norm_stage(int fmt, float* x, const float* w, int K, float eps, void* xn_out, void* staged, int M, int ncg, const float* part, int ks, int np, hipStream_t s);   // qgemm64.hip

// internal format id and unit count of the staged activation layout a weight of (ggml_type, K) consumes; fmt < 0: none
static int staged_fmt(int ggml_type, long long K, int* nu) {
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

__global__ __launch_bounds__(256) void stage_activation_kernel(const void* __restrict__ x, int x_f32, int K, int fmt, int nu, _Float16* __restrict__ out) {
  for (int e = blockIdx.x * 256 + threadIdx.x; e < K; e += gridDim.x * 256) {
    const _Float16 v = x_f32 ? (_Float16)((const float*)x)[e] : ((const _Float16*)x)[e];
    out[staged_pos(fmt, e, nu)] = v;
  }
}

// fp16 copy of one activation row in the order the M = 1 GEMV of a (ggml_type, K) weight consumes (a permutation of the row)
extern "C" int tga_stage_activation(int ggml_type, const void* x, int x_dtype, int64_t K, void* out_f16, void* stream) {
  TGA_REQUIRE(x && out_f16, "tga_stage_activation: null pointer");
  TGA_REQUIRE(x_dtype == TGA_F16 || x_dtype == TGA_F32, "tga_stage_activation: x_dtype must be TGA_F16 or TGA_F32");
  int nu; const int fmt = staged_fmt(ggml_type, K, &nu);
  TGA_REQUIRE(fmt >= 0, "tga_stage_activation: no staged layout for type %d with K=%lld", ggml_type, (long long)K);
  stage_activation_kernel<<<(unsigned)((K + 255) / 256), 256, 0, (hipStream_t)stream>>>(x, x_dtype == TGA_F32, (int)K, fmt, nu, (_Float16*)out_f16);
  TGA_LAUNCH_CHECK();
  return 0;
}

struct CombineIn { const float* y; const float* p; int k; float* x_out; };
// n_splits > 0: x holds the split partials of the attention (tga_attention_decode_split), merged while the row is staged.  touch_pos: the launch also touches
// the cache rows and the rotation row that the attention launch behind it will read (QArgs::touch_*)
struct AttnIn { int n_splits, head_dim; const int* touch_pos; const void* k; const void* v; const void* rope; int n_kv, max_ctx; };
static int qlinear_multi_impl(const CombineIn* comb, const AttnIn* attn, const float* norm_w, float norm_eps, int ggml_type, int nseg, const void* const* w, void* const* y, const int64_t* n,
                              const void* x, int x_dtype, int y_dtype, int M, int64_t K,
                              int epilogue, const void* const* resid, int y_stage_type, int64_t y_stage_K, void* stream);
// the prefill kernel's format for a weight of this type with rows of K values, -1: none (block pairs need an even number of blocks; K in steps of 256)
static int q64_fmt_of(int ggml_type, int64_t K) {
  if (K <= 0 || K % 256 != 0) return -1;
  switch (ggml_type) {
    case GGML_Q4_0: return F_Q4_0P; case GGML_Q8_0: return F_Q8_0P;
    case GGML_Q6_K: case GGML_Q4_K: case GGML_Q5_K: case GGML_IQ4_XS: case GGML_F16: return ggml_type;
  }
  return -1;
}
// the arguments of the 17 .. 128 row GEMM (qgemm64.hip) for a call whose pointers and epilogue have been checked; false: a format or alignment it does not take
static bool q64_args(int ggml_type, int nseg, const void* const* w, void* const* y, const int64_t* n, const void* x, int x_dtype, int y_dtype, int64_t K,
                     int epilogue, const void* const* resid, QArgs& q, int& fmt64) {
  bool pair64 = K > 0 && (K / 32) % 2 == 0;
  for (int i = 0; i < nseg; i++) pair64 = pair64 && ((uintptr_t)w[i] & 3) == 0;
  fmt64 = ggml_type == GGML_Q4_0 ? (pair64 ? F_Q4_0P : -1) : ggml_type == GGML_Q8_0 ? (pair64 ? F_Q8_0P : -1) : ggml_type;
  if (fmt64 < 0 || !pair64) return false;
  q = QArgs{};
  q.nseg = nseg; q.x = x; q.x_f32 = x_dtype == TGA_F32; q.y_f32 = y_dtype == TGA_F32; q.epilogue = epilogue; q.K = (int)K;
  long long nt = 0;
  for (int i = 0; i < nseg; i++) { q.w[i] = (const uint8_t*)w[i]; q.y[i] = y[i]; q.n[i] = n[i]; q.resid[i] = epilogue == 1 ? (const float*)resid[i] : nullptr; nt += n[i]; }
  q.ntot = epilogue == 2 ? n[0] : nt;
  return true;
}
// M rows as calls of at most `block` rows ((M, n) outputs and (M, K) activations: row blocks are contiguous)
static int qlinear_row_blocks(int block, int ggml_type, int nseg, const void* const* w, void* const* y, const int64_t* n, const void* x, int x_dtype, int y_dtype, int M, int64_t K,
                              int epilogue, const void* const* resid, void* stream) {
  const size_t xs = x_dtype == TGA_F32 ? 4 : 2, ys = y_dtype == TGA_F32 ? 4 : 2;
  for (int m0 = 0; m0 < M; m0 += block) {
    const void* wv[QG_MAX_SEG]; void* yv[QG_MAX_SEG]; const void* rv[QG_MAX_SEG];
    for (int i = 0; i < nseg; i++) {
      wv[i] = w[i];
      yv[i] = y[i] ? (char*)y[i] + (size_t)m0 * n[i] * ys : nullptr;
      rv[i] = (epilogue == 1) ? (const char*)resid[i] + (size_t)m0 * n[i] * 4 : nullptr;
    }
    const int rc = qlinear_multi_impl(nullptr, nullptr, nullptr, 0.f, ggml_type, nseg, wv, yv, n, (const char*)x + (size_t)m0 * K * xs, x_dtype, y_dtype, M - m0 < block ? M - m0 : block, K,
                                      epilogue, epilogue == 1 ? rv : nullptr, 0, 0, stream);
    if (rc) return rc;
  }
  return 0;
}
static int qlinear_multi_impl(const CombineIn* comb, const AttnIn* attn, const float* norm_w, float norm_eps, int ggml_type, int nseg, const void* const* w, void* const* y, const int64_t* n,
                              const void* x, int x_dtype, int y_dtype, int M, int64_t K,
                              int epilogue, const void* const* resid, int y_stage_type, int64_t y_stage_K, void* stream) {
  TGA_REQUIRE(nseg >= 1 && nseg <= QG_MAX_SEG, "tga_qlinear_multi: nseg=%d out of range 1..%d", nseg, QG_MAX_SEG);
  TGA_REQUIRE(M >= 1 && M <= 128, "tga_qlinear: M=%d out of range 1..128", M);
  // 17 .. 128 rows (prefill steps): one pass over the weights on the prefill kernel where it applies (qgemm64.hip), else blocks of sixteen rows (every block
  // after the first finds the weights in the Infinity Cache)
  if (M > 16) {
    // x_dtype TGA_F16_STAGED: x holds the rows in the layout the prefill kernel multiplies from (written by tga_rmsnorm_rows_stage, by a SwiGLU launch with
    // y_stage_type, or by tga_attention_prefill_chunk_staged); y_stage_type (SwiGLU): the fp16 rows are written in that layout for a consumer of that type
    const bool xst = x_dtype == TGA_F16_STAGED;
    TGA_REQUIRE(!comb && !norm_w && (x_dtype == TGA_F16 || x_dtype == TGA_F32 || xst) && x && (epilogue != 1 || resid) && epilogue >= 0 && epilogue <= 2,
                "tga_qlinear: more than 16 rows only for fp16 / float32 activations (plain, or in the multiplying layout)");
    TGA_REQUIRE(!y_stage_type || (epilogue == 2 && y_dtype == TGA_F16 && y_stage_K == n[0]), "tga_qlinear: rows in a consumer's layout only from the SwiGLU epilogue, fp16, with y_stage_K = its rows");
    TGA_REQUIRE(y_dtype == TGA_F16 || y_dtype == TGA_F32, "tga_qlinear: y_dtype must be TGA_F16 or TGA_F32");
    TGA_REQUIRE(epilogue != 1 || y_dtype == TGA_F32, "tga_qlinear: the residual epilogue needs float32 y");
    TGA_REQUIRE(epilogue != 2 || (nseg == 2 && n[0] == n[1]), "tga_qlinear: the SwiGLU epilogue needs two segments of equal rows");
    for (int i = 0; i < nseg; i++) TGA_REQUIRE(n[i] > 0 && w[i] && (y[i] || (epilogue == 2 && i == 1)) && (epilogue != 1 || resid[i]), "tga_qlinear: segment %d has a null pointer or no rows", i);
    QArgs q; int fmt64;
    if (q64_args(ggml_type, nseg, w, y, n, x, xst ? TGA_F16 : x_dtype, y_dtype, K, epilogue, resid, q, fmt64)) {
      bool ok = true;
      if (y_stage_type) { q.y_stage_fmt = q64_fmt_of(y_stage_type, y_stage_K); q.y_stage_nu = (int)(y_stage_K / 64); ok = q.y_stage_fmt >= 0; }
      if (ok) {
        Q64Opt o = {xst, xst ? x : nullptr, false, nullptr, 0, 0};
        const int rc = tga_qgemm64_dispatch(fmt64, q, M, o, (hipStream_t)stream);
        if (rc >= 0) return rc;
      }
    }
    TGA_REQUIRE(!xst && !y_stage_type, "tga_qlinear: rows in the multiplying layout are outside the prefill kernel's range here (tga_rows_staged_plan says which linears take them)");
    return qlinear_row_blocks(16, ggml_type, nseg, w, y, n, x, x_dtype, y_dtype, M, K, epilogue, resid, stream);
  }
  TGA_REQUIRE(x_dtype == TGA_F16 || x_dtype == TGA_F32 || x_dtype == TGA_F16_STAGED, "tga_qlinear: x_dtype must be TGA_F16, TGA_F32 or TGA_F16_STAGED");
  TGA_REQUIRE(y_dtype == TGA_F16 || y_dtype == TGA_F32, "tga_qlinear: y_dtype must be TGA_F16 or TGA_F32");
  TGA_REQUIRE(epilogue >= 0 && epilogue <= 2, "tga_qlinear: epilogue=%d unknown", epilogue);
  TGA_REQUIRE(x_dtype != TGA_F16_STAGED || M == 1, "tga_qlinear: staged activations are an M = 1 format");
  TGA_REQUIRE(epilogue != 1 || (y_dtype == TGA_F32 && resid), "tga_qlinear: the residual epilogue needs float32 y and resid pointers");
  TGA_REQUIRE(epilogue != 2 || (nseg == 2 && n[0] == n[1]), "tga_qlinear: the SwiGLU epilogue needs two segments of equal rows");
  int bw;
  switch (ggml_type) { case GGML_Q4_0: case GGML_Q8_0: case GGML_MXFP4: bw = 32; break; case GGML_Q6_K: case GGML_Q4_K: case GGML_Q5_K: case GGML_IQ4_XS: case GGML_IQ3_XXS: case GGML_IQ3_S: case GGML_IQ2_S: bw = 256; break; case GGML_F16: bw = 64; break;
    case GGML_Q4_1: case GGML_Q5_0: case GGML_Q5_1: bw = 64; break;      // served as block pairs
    case GGML_Q1_0: bw = 128; break;
    default: return tga_set_error("GGML type '%d' is not supported!", ggml_type); }
  const bool align4 = ggml_type == GGML_Q4_K || ggml_type == GGML_Q5_K || ggml_type == GGML_Q4_1 || ggml_type == GGML_Q5_0 || ggml_type == GGML_Q5_1 || ggml_type == GGML_IQ4_XS;
  TGA_REQUIRE(K > 0 && K % bw == 0 && K <= (1 << 24), "tga_qlinear: K=%lld must be a positive multiple of %d", (long long)K, bw);
  TGA_REQUIRE(x, "tga_qlinear: null x");
  QArgs a = {};
  a.nseg = nseg; a.x = x; a.x_staged = x_dtype == TGA_F16_STAGED; a.x_f32 = x_dtype == TGA_F32; a.y_f32 = y_dtype == TGA_F32; a.epilogue = epilogue; a.K = (int)K;
  long long ntot = 0;
  for (int i = 0; i < nseg; i++) {
    TGA_REQUIRE(n[i] > 0 && w[i] && (y[i] || (epilogue == 2 && i == 1)), "tga_qlinear: segment %d has a null pointer or no rows", i);
    TGA_REQUIRE(ggml_type == GGML_MXFP4 || ((uintptr_t)w[i] & 1) == 0, "tga_qlinear: weight pointer of segment %d must be 2-byte aligned", i);
    TGA_REQUIRE(!align4 || ((uintptr_t)w[i] & 3) == 0, "tga_qlinear: Q4_K / Q5_K / Q4_1 / Q5_0 / Q5_1 / IQ4_XS weights of segment %d must be 4-byte aligned", i);
    a.w[i] = (const uint8_t*)w[i]; a.y[i] = y[i]; a.n[i] = n[i]; a.resid[i] = epilogue == 1 ? (const float*)resid[i] : nullptr;
    TGA_REQUIRE(epilogue != 1 || a.resid[i], "tga_qlinear: null resid for segment %d", i);
    ntot += n[i];
  }
  a.ntot = (epilogue == 2) ? n[0] : ntot;
  if (y_stage_type) {
    TGA_REQUIRE(M == 1 && y_dtype == TGA_F16 && epilogue == 2, "tga_qlinear: staged output needs M = 1, fp16 y and the SwiGLU epilogue");
    TGA_REQUIRE(y_stage_K == a.ntot, "tga_qlinear: staged output length %lld must equal the output rows %lld", (long long)y_stage_K, (long long)a.ntot);
    a.y_stage_fmt = staged_fmt(y_stage_type, y_stage_K, &a.y_stage_nu);
    TGA_REQUIRE(a.y_stage_fmt >= 0, "tga_qlinear: no staged layout for consumer type %d with K=%lld", y_stage_type, (long long)y_stage_K);
  }
  if (norm_w) {
    TGA_REQUIRE((M == 1 || !comb) && x_dtype == TGA_F32 && ((uintptr_t)norm_w & 15) == 0, "tga_rmsnorm_qlinear: needs float32 x and a 16-byte aligned norm weight (M = 1 with the expert sum)");
    a.norm_w = norm_w; a.norm_eps = norm_eps;
  }
  if (comb) {
    TGA_REQUIRE(norm_w && comb->y && comb->p && comb->x_out && comb->k >= 1 && comb->k <= 8 && epilogue == 0, "tga_moe_combine_rmsnorm_qlinear_multi: needs the norm, 1..8 summands and the plain epilogue");
    TGA_REQUIRE(((((uintptr_t)comb->y | (uintptr_t)comb->x_out | (uintptr_t)x) & 15) == 0) && K % 8 == 0, "tga_moe_combine_rmsnorm_qlinear_multi: rows must be 16-byte aligned");
    a.comb_y = comb->y; a.comb_p = comb->p; a.comb_k = comb->k; a.comb_x_out = comb->x_out;
  }
  hipStream_t s = (hipStream_t)stream;
  // block-pair units need an even number of blocks per row and 4-byte aligned rows
  bool pair = (K / 32) % 2 == 0;
  for (int i = 0; i < nseg; i++) pair = pair && ((uintptr_t)w[i] & 3) == 0;
  if (attn && attn->touch_pos) {
    TGA_REQUIRE(M == 1 && norm_w && attn->k && attn->v && attn->rope && attn->n_kv > 0 && attn->max_ctx > 0 && (attn->head_dim == 64 || attn->head_dim == 128 || attn->head_dim == 256),
                "tga_rmsnorm_qlinear_multi_touch: null pointer or bad cache shape");
    if (attn->n_kv % 8 == 0) {                                    // (else the attention workgroups of a kv head do not share an XCD: nothing to aim at)
      a.touch_pos = attn->touch_pos; a.touch_k = (const uint8_t*)attn->k; a.touch_v = (const uint8_t*)attn->v; a.touch_rope = (const uint8_t*)attn->rope;
      a.touch_n_kv = attn->n_kv; a.touch_max_ctx = attn->max_ctx; a.touch_row_bytes = attn->head_dim * 2; a.touch_rope_row_bytes = attn->head_dim * 4;
    }
  }
  if (attn && attn->n_splits > 0) {
    const int hd = attn->head_dim;
    TGA_REQUIRE(M == 1 && nseg == 1 && epilogue == 1 && x_dtype == TGA_F32 && !norm_w && !comb && !y_stage_type, "tga_attn_merge_qlinear: one matrix, one row, residual epilogue");
    TGA_REQUIRE((hd == 64 || hd == 128 || hd == 256) && K % hd == 0 && attn->n_splits >= 1 && attn->n_splits <= 6 && ((uintptr_t)x & 15) == 0,
                "tga_attn_merge_qlinear: head_dim=%d n_splits=%d (1..6 splits, 16-byte aligned partials)", hd, attn->n_splits);
    a.attn_S = attn->n_splits; a.attn_hd_log2 = hd == 64 ? 6 : hd == 128 ? 7 : 8;
    const int fmt = ggml_type == GGML_Q4_0 ? (pair ? F_Q4_0P : -1) : ggml_type == GGML_Q8_0 ? (pair ? F_Q8_0P : -1) : ggml_type;
    const int rc = fmt >= 0 ? tga_qgemv1_dispatch(fmt, a, s) : -1;
    if (rc < 0) return tga_set_error("tga_attn_merge_qlinear: needs the M = 1 fast path with rows of at most 64 units (K <= 4096) and 4-byte aligned weights");
    return rc;
  }
  if (M == 1) {
    const int fmt = ggml_type == GGML_Q4_0 ? (pair ? F_Q4_0P : -1) : ggml_type == GGML_Q8_0 ? (pair ? F_Q8_0P : -1) : ggml_type;
    if (fmt >= 0) { const int rc = tga_qgemv1_dispatch(fmt, a, s); if (rc >= 0) return rc; }
  }
  if (M >= 2 && norm_w) {                                         // several rows with the norm folded in: the LDS-fed kernel or nothing (-2: the caller norms first)
    const int fmt = ggml_type == GGML_Q4_0 ? (pair ? F_Q4_0P : -1) : ggml_type == GGML_Q8_0 ? (pair ? F_Q8_0P : -1) : ggml_type;
    if (fmt >= 0) { const int rc = tga_qgemm_dma_dispatch(fmt, a, M, s); if (rc >= 0) return rc; }
    return -2;
  }
  if (M == 2 && !comb) {
    // two rows: the single-row kernel's walk (Q4_0 / Q8_0 pairs, Q6_K) from 2^25 weights on, below that the LDS-fed matrix-core kernel where it applies
    // (Q4_0 4096 x 4096: 7.4 us against 9.1 us on the LDS-staged dot2 kernel, which takes the rest)
    const int fmt = ggml_type == GGML_Q4_0 ? (pair ? F_Q4_0P : -1) : ggml_type == GGML_Q8_0 ? (pair ? F_Q8_0P : -1) : ggml_type == GGML_Q6_K ? GGML_Q6_K : -1;
    if (fmt == F_Q8_0P && a.K > 4096) { const int rc = tga_qgemm_dma_dispatch(fmt, a, M, s); if (rc >= 0) return rc; }   // (Q8_0 4096 x 14336: streamed activations 17.3 us, the walk 18.7)
    if (fmt == F_Q8_0P && a.K <= 4096) { const int rc = tga_qgemm_wp_checked_dispatch(fmt, a, M, s); if (rc >= 0) return rc; }   // (Q8_0 14336 x 4096: wave-private rings 15.8 us, the walk 17.0)
    if (ggml_type == GGML_F16) { const int rc = tga_qgemm_wp_checked_dispatch(GGML_F16, a, M, s); if (rc >= 0) return rc; }          // (fp16 50304 x 2048 lm-head: 41 us against 55 on the LDS-staged kernel)
    if (fmt >= 0) { const int rc = tga_qgemv1_multi_dispatch(fmt, a, M, s); if (rc >= 0) return rc; }
    const int fmt2 = ggml_type == GGML_Q4_0 ? (pair ? F_Q4_0P : -1) : ggml_type == GGML_Q8_0 ? (pair ? F_Q8_0P : -1) : ggml_type;
    if (fmt2 >= 0 && a.ntot * (long long)a.K < (1ll << 25)) { const int rc = tga_qgemm_dma_dispatch(fmt2, a, M, s); if (rc >= 0) return rc; }
  }
  if (M >= 3) {                                                   // matrix-core small-batch kernels: weights through LDS where that kernel applies, else through registers
    const int fmt = ggml_type == GGML_Q4_0 ? (pair ? F_Q4_0P : -1) : ggml_type == GGML_Q8_0 ? (pair ? F_Q8_0P : -1) : ggml_type;
    if (fmt >= 0) { const int rc = tga_qgemm_dma_dispatch(fmt, a, M, s); if (rc >= 0) return rc; }
    if (fmt >= 0) { const int rc = tga_qgemm_mfma_dispatch(fmt, a, M, s); if (rc >= 0) return rc; }
  }
  if (M > 8) {                                                    // 9..16 rows outside the LDS-fed kernel's range: two calls of at most eight rows
    TGA_REQUIRE(!comb && !norm_w && !a.x_staged && !a.y_stage_fmt, "tga_qlinear: more than 8 rows only for plain activations");
    return qlinear_row_blocks(8, ggml_type, nseg, w, y, n, x, x_dtype, y_dtype, M, K, epilogue, resid, stream);
  }
  TGA_REQUIRE(!comb, "tga_moe_combine_rmsnorm_qlinear_multi: needs the M = 1 fast path with K <= 2048");
  TGA_REQUIRE(!norm_w, "tga_rmsnorm_qlinear: the fused norm needs the M = 1 fast path (K %% 64 == 0, 4-byte aligned weights, 16-byte aligned x, K <= 65536)");
  TGA_REQUIRE(!a.x_staged && !a.y_stage_fmt, "tga_qlinear: staged activations need the M = 1 fast path (K %% 64 == 0, 4-byte aligned weights, K <= 65536)");
  switch (ggml_type) {
    case GGML_Q4_0: return pair ? launch_qgemv_m<F_Q4_0P>(a, M, s) : launch_qgemv_m<GGML_Q4_0>(a, M, s);
    case GGML_Q8_0: return pair ? launch_qgemv_m<F_Q8_0P>(a, M, s) : launch_qgemv_m<GGML_Q8_0>(a, M, s);
    case GGML_Q6_K: return launch_qgemv_m<GGML_Q6_K>(a, M, s);
    case GGML_Q4_K: return launch_qgemv_m<GGML_Q4_K>(a, M, s);
    case GGML_Q5_K: return launch_qgemv_m<GGML_Q5_K>(a, M, s);
    case GGML_Q4_1: return launch_qgemv_m<GGML_Q4_1>(a, M, s);
    case GGML_Q5_0: return launch_qgemv_m<GGML_Q5_0>(a, M, s);
    case GGML_Q5_1: return launch_qgemv_m<GGML_Q5_1>(a, M, s);
    case GGML_IQ4_XS: return launch_qgemv_m<GGML_IQ4_XS>(a, M, s);
    case GGML_IQ3_XXS: return launch_qgemv_m<GGML_IQ3_XXS>(a, M, s);
    case GGML_IQ3_S: return launch_qgemv_m<GGML_IQ3_S>(a, M, s);
    case GGML_IQ2_S: return launch_qgemv_m<GGML_IQ2_S>(a, M, s);
    case GGML_Q1_0: return launch_qgemv_m<GGML_Q1_0>(a, M, s);
    case GGML_MXFP4: return launch_qgemv_m<GGML_MXFP4>(a, M, s);
    case GGML_F16: return launch_qgemv_m<GGML_F16>(a, M, s);
  }
  return tga_set_error("tga_qlinear: no kernel for type %d with this shape (K=%lld)", ggml_type, (long long)K);
}

// attn_output + residual of one token whose activation row is still in split partials (model.py:198 after :194-197): the merge over the splits
// (max, sum, weighted V, division) happens while the row is staged, so the attention needs no merge launch
extern "C" int tga_attn_merge_qlinear(int ggml_type, const void* w, float* y, int64_t N, int64_t K, const float* resid, const float* partials, int n_splits, int head_dim, void* stream) {
  TGA_REQUIRE(w && y && resid && partials, "tga_attn_merge_qlinear: null pointer");
  const AttnIn in = {n_splits, head_dim, nullptr, nullptr, nullptr, nullptr, 0, 0};
  const void* wv[1] = {w}; void* yv[1] = {y}; const void* rv[1] = {resid}; const int64_t nv[1] = {N};
  return qlinear_multi_impl(nullptr, &in, nullptr, 0.f, ggml_type, 1, wv, yv, nv, partials, TGA_F32, TGA_F32, 1, K, 1, rv, 0, 0, stream);
}

extern "C" int tga_qlinear_multi(int ggml_type, int nseg, const void* const* w, void* const* y, const int64_t* n,
                                 const void* x, int x_dtype, int y_dtype, int M, int64_t K,
                                 int epilogue, const void* const* resid, int y_stage_type, int64_t y_stage_K, void* stream) {
  return qlinear_multi_impl(nullptr, nullptr, nullptr, 0.f, ggml_type, nseg, w, y, n, x, x_dtype, y_dtype, M, K, epilogue, resid, y_stage_type, y_stage_K, stream);
}

// RMSNorm (nn.RMSNorm, tinygrad/nn/__init__.py:296-304) of the float32 activation row folded into the M = 1 linear that consumes it
// (attn_norm -> attn_q/k/v, ffn_norm -> ffn_gate/up, output_norm -> output: tinygrad/llm/model.py:149-150, 362): no normalised copy
// of the row goes through memory.
extern "C" int tga_rmsnorm_qlinear_multi(const float* norm_weight, float norm_eps, int ggml_type, int nseg, const void* const* w, void* const* y, const int64_t* n,
                                         const void* x, int y_dtype, int64_t K, int epilogue, const void* const* resid,
                                         int y_stage_type, int64_t y_stage_K, void* stream) {
  TGA_REQUIRE(norm_weight, "tga_rmsnorm_qlinear_multi: null norm weight");
  return qlinear_multi_impl(nullptr, nullptr, norm_weight, norm_eps, ggml_type, nseg, w, y, n, x, TGA_F32, y_dtype, 1, K, epilogue, resid, y_stage_type, y_stage_K, stream);
}

// tga_rmsnorm_qlinear_multi for the q / k / v launch of a decode step: its lanes also read one dword each of the lines that the attention launch behind it
// will ask for first (cached K / V rows below state.pos, the rotation row of that position), on the XCD that will ask
extern "C" int tga_rmsnorm_qlinear_multi_touch(const float* norm_weight, float norm_eps, int ggml_type, int nseg, const void* const* w, void* const* y, const int64_t* n,
                                               const void* x, int y_dtype, int64_t K, int epilogue, const void* const* resid,
                                               const void* state, const void* cache_k, const void* cache_v, const void* rope_table, int n_kv_heads, int head_dim, int max_ctx,
                                               void* stream) {
  TGA_REQUIRE(norm_weight && state, "tga_rmsnorm_qlinear_multi_touch: null norm weight or state");
  const AttnIn in = {0, head_dim, (const int*)state, cache_k, cache_v, rope_table, n_kv_heads, max_ctx};
  return qlinear_multi_impl(nullptr, &in, norm_weight, norm_eps, ggml_type, nseg, w, y, n, x, TGA_F32, y_dtype, 1, K, epilogue, resid, 0, 0, stream);
}

// tga_rmsnorm_qlinear_multi (plain epilogue) for matrices of different block types over the same row: runs of equal types are one launch each, and the two
// runs of a Q4_K_M / Q5_K_M block (Q4_K or Q5_K attn_q / attn_k, Q6_K attn_v) share a launch where the single-row kernel's two-set variant applies.
int tga_qgemv1_two_dispatch(int fmt_a, int fmt_b, const QArgs& a, const QArgs& b, hipStream_t s);   // qgemv1_two.hip
extern "C" int tga_rmsnorm_qlinear_mixed(const float* norm_weight, float norm_eps, int nseg, const int32_t* ggml_types, const void* const* w, void* const* y, const int64_t* n,
                                         const float* x, int y_dtype, int64_t K, void* stream) {
  TGA_REQUIRE(norm_weight && ggml_types && w && y && n && x, "tga_rmsnorm_qlinear_mixed: null pointer");
  TGA_REQUIRE(nseg >= 1 && nseg <= QG_MAX_SEG, "tga_rmsnorm_qlinear_mixed: nseg=%d out of range 1..%d", nseg, QG_MAX_SEG);
  TGA_REQUIRE(y_dtype == TGA_F16 || y_dtype == TGA_F32, "tga_rmsnorm_qlinear_mixed: y_dtype must be TGA_F16 or TGA_F32");
  int cut = 1;                                                    // end of the first run
  while (cut < nseg && ggml_types[cut] == ggml_types[0]) cut++;
  bool two_runs = cut < nseg;
  for (int i = cut + 1; i < nseg; i++) two_runs = two_runs && ggml_types[i] == ggml_types[cut];
  if (two_runs && K > 0 && K <= 4096 && (((uintptr_t)norm_weight | (uintptr_t)x) & 15) == 0) {
    QArgs q[2] = {};
    bool ok = true;
    for (int r = 0; r < 2; r++) {
      QArgs& a = q[r];
      const int i0 = r ? cut : 0, i1 = r ? nseg : cut;
      a.nseg = i1 - i0; a.x = x; a.x_f32 = 1; a.y_f32 = y_dtype == TGA_F32; a.K = (int)K; a.norm_w = norm_weight; a.norm_eps = norm_eps;
      for (int i = i0; i < i1; i++) {
        ok = ok && n[i] > 0 && w[i] && y[i] && ((uintptr_t)w[i] & 3) == 0;
        a.w[i - i0] = (const uint8_t*)w[i]; a.y[i - i0] = y[i]; a.n[i - i0] = n[i]; a.ntot += n[i];
      }
    }
    if (ok) { const int rc = tga_qgemv1_two_dispatch(ggml_types[0], ggml_types[cut], q[0], q[1], (hipStream_t)stream); if (rc >= 0) return rc; }
  }
  for (int i0 = 0; i0 < nseg;) {                                  // one launch per run (the checks of tga_rmsnorm_qlinear_multi apply to each)
    int i1 = i0 + 1;
    while (i1 < nseg && ggml_types[i1] == ggml_types[i0]) i1++;
    const int rc = qlinear_multi_impl(nullptr, nullptr, norm_weight, norm_eps, ggml_types[i0], i1 - i0, w + i0, y + i0, n + i0, x, TGA_F32, y_dtype, 1, K, 0, nullptr, 0, 0, stream);
    if (rc) return rc;
    i0 = i1;
  }
  return 0;
}

// tga_rmsnorm_rows followed by tga_qlinear_multi for M rows: one launch where the LDS-fed small-batch kernel folds the norm into its prologue (Q4_0 / Q8_0 / Q6_K,
// 2 <= M <= 8, K <= 4096), otherwise the norm into xn_scratch (M, K) fp16 and the linears on that.
extern "C" int tga_rmsnorm_qlinear_rows(const float* norm_weight, float norm_eps, int ggml_type, int nseg, const void* const* w, void* const* y, const int64_t* n,
                                        const float* x, void* xn_scratch_f16, int y_dtype, int M, int64_t K, int epilogue, const void* const* resid, void* stream) {
  TGA_REQUIRE(norm_weight && x && xn_scratch_f16, "tga_rmsnorm_qlinear_rows: null pointer");
  TGA_REQUIRE(M >= 1 && M <= 128 && K > 0 && K <= (1 << 24), "tga_rmsnorm_qlinear_rows: M=%d (1..128), K=%lld", M, (long long)K);
  // up to eight rows: beyond, what every workgroup reads and normalises again (M float32 rows) costs more than the norm's own launch (8B-arch prefill in
  // chunks of sixteen: 208 ms folded against 195 ms; chunks of eight 320 against 328, of four 562 against 610)
  if (M >= 2 && M <= 8 && ((uintptr_t)norm_weight & 15) == 0) {
    const int rc = qlinear_multi_impl(nullptr, nullptr, norm_weight, norm_eps, ggml_type, nseg, w, y, n, x, TGA_F32, y_dtype, M, K, epilogue, resid, 0, 0, stream);
    if (rc != -2) return rc;
  }
  if (M > 16 && nseg >= 1 && nseg <= QG_MAX_SEG && w && y && n && (y_dtype == TGA_F16 || y_dtype == TGA_F32) && epilogue >= 0 && epilogue <= 2 && (epilogue != 1 || (resid && y_dtype == TGA_F32)) &&
      (epilogue != 2 || (nseg == 2 && n[0] == n[1]))) {
    // 17 .. 128 rows on the prefill kernel: the norm's launch writes the rows in the layout that kernel multiplies from as well (no staging launch)
    bool ok = true;
    for (int i = 0; i < nseg; i++) ok = ok && n[i] > 0 && w[i] && (y[i] || (epilogue == 2 && i == 1)) && (epilogue != 1 || resid[i]);
    QArgs q; int fmt64, ncg = 0;
    if (ok && q64_args(ggml_type, nseg, w, y, n, xn_scratch_f16, TGA_F16, y_dtype, K, epilogue, resid, q, fmt64)) {
      void* staged = tga_qgemm64_staging(fmt64, q, M, (hipStream_t)stream, &ncg);
      if (staged) {
        const int rn = tga_qgemm64_norm_stage(fmt64, const_cast<float*>(x), norm_weight, (int)K, norm_eps, xn_scratch_f16, staged, M, ncg, nullptr, 0, 0, (hipStream_t)stream);
        if (rn > 0) return rn;
        if (rn == 0) {
          Q64Opt o = {true, nullptr, false, nullptr, 0, 0};
          const int rc = tga_qgemm64_dispatch(fmt64, q, M, o, (hipStream_t)stream);
          if (rc >= 0) return rc;                                 // (cannot be refused here: the same checks have passed above)
        }
      }
    }
  }
  const int rc = tga_rmsnorm_rows(x, norm_weight, M, (int)K, norm_eps, xn_scratch_f16, nullptr, 0, stream);
  if (rc) return rc;
  return qlinear_multi_impl(nullptr, nullptr, nullptr, 0.f, ggml_type, nseg, w, y, n, xn_scratch_f16, TGA_F16, y_dtype, M, K, epilogue, resid, 0, 0, stream);
}

// ---- a prefill step of 17 .. 128 rows with the rows handed from launch to launch in the layout the prefill kernel multiplies from, and the split-K sums of the
// residual linears completed by the norm launch behind them (llm.BatchedTransformer's step for chunks of more than sixteen positions)

// Whether a linear of this type with rows of K values takes M activation rows in the multiplying layout: *ncg = column groups of sixteen rows (2 or 4; the buffer holds
// 16 ncg x K fp16 values), 0 = no.
extern "C" int tga_rows_staged_plan(int ggml_type, int64_t K, int M, int* ncg) {
  TGA_REQUIRE(ncg, "tga_rows_staged_plan: null pointer");
  *ncg = (M >= 17 && M <= 128 && K <= 32768 && q64_fmt_of(ggml_type, K) >= 0) ? (M <= 32 ? 2 : M <= 64 ? 4 : 8) : 0;
  return 0;
}

// y = y + x W^T for one matrix (attn_output, ffn_down: the residual adds of model.py:149-150) over rows in the multiplying layout.  When the kernel splits K, the sum over
// the splits is NOT taken: *partials / *ks / *np describe the partial tiles (in the stream's workspace, valid until the next call of 17 .. 128 rows on this stream) and y is
// untouched - tga_rmsnorm_rows_stage (or tga_rows_add_partials) completes it.  *ks = 0: nothing is pending, y is complete.
extern "C" int tga_qlinear_rows_deferred(int ggml_type, const void* w, int64_t N, int64_t K, const void* x_staged, int M, float* y, const float** partials, int* ks, int* np, void* stream) {
  TGA_REQUIRE(w && x_staged && y && partials && ks && np && N > 0, "tga_qlinear_rows_deferred: null pointer or no rows");
  const void* wv[1] = {w}; void* yv[1] = {y}; const void* rv[1] = {y}; const int64_t nv[1] = {N};
  QArgs q; int fmt64;
  TGA_REQUIRE(q64_args(ggml_type, 1, wv, yv, nv, x_staged, TGA_F16, TGA_F32, K, 1, rv, q, fmt64), "tga_qlinear_rows_deferred: type %d with K=%lld is outside the prefill kernel's range", ggml_type, (long long)K);
  Q64Opt o = {true, x_staged, true, nullptr, 0, 0};
  const int rc = tga_qgemm64_dispatch(fmt64, q, M, o, (hipStream_t)stream);
  TGA_REQUIRE(rc >= 0, "tga_qlinear_rows_deferred: M=%d, N=%lld, K=%lld outside the prefill kernel's range", M, (long long)N, (long long)K);
  *partials = o.part; *ks = o.ks; *np = o.np;
  return rc;
}

// RMSNorm of `rows` float32 rows (nn.RMSNorm, tinygrad/nn/__init__.py:296-304) written as fp16 in the multiplying layout of a consumer of consumer_type (and, when
// xn_out is given, as plain fp16 rows).  partials != NULL: every row is first completed in place with the partial tiles a tga_qlinear_rows_deferred call left.
extern "C" int tga_rmsnorm_rows_stage(float* x, const float* partials, int ks, int np, const float* weight, float eps, int rows, int dim, int consumer_type, void* xn_out_f16, void* staged_out, void* stream) {
  TGA_REQUIRE(x && weight && staged_out && rows >= 17 && rows <= 128, "tga_rmsnorm_rows_stage: null pointer or rows=%d outside 17..128", rows);
  const int fmt = q64_fmt_of(consumer_type, dim);
  TGA_REQUIRE(fmt >= 0, "tga_rmsnorm_rows_stage: no multiplying layout for type %d with K=%d", consumer_type, dim);
  const int rc = tga_qgemm64_norm_stage(fmt, x, weight, dim, eps, xn_out_f16, staged_out, rows, rows <= 32 ? 2 : rows <= 64 ? 4 : 8, partials, ks, np, (hipStream_t)stream);
  TGA_REQUIRE(rc >= 0, "tga_rmsnorm_rows_stage: pointers must be 16-byte aligned, dim a multiple of 256 up to 32768");
  return rc;
}

// x += the sum of the partial tiles a tga_qlinear_rows_deferred call left (what its own reduce launch would have done): rows x dim float32
extern "C" int tga_rows_add_partials(float* x, const float* partials, int ks, int np, int rows, int dim, void* stream) {
  TGA_REQUIRE(x && partials && ks >= 1 && np >= dim && np % 4 == 0 && rows >= 1 && rows <= 128 && dim > 0, "tga_rows_add_partials: null pointer or ks=%d np=%d rows=%d dim=%d", ks, np, rows, dim);
  return tga_qgemm64_add_partials(x, partials, ks, np, rows, dim, (hipStream_t)stream);
}

// The MoE weighted sum and block residual (x += sum_j probs[j] * y[j], tinygrad/llm/model.py:130, 150) folded into the launch that
// consumes the completed row: tga_rmsnorm_qlinear_multi on x_in + sum_j probs[j] * y[j], with the completed row written to x_out (by
// one workgroup) for the residual adds that follow.  x_out must not be x_in: every workgroup reads x_in while one writes x_out.
// y: (k, K) float32 rows, probs: k float32, k <= 8, K <= 2048.
extern "C" int tga_moe_combine_rmsnorm_qlinear_multi(const float* y_experts, const float* probs, int k, const float* x_in, float* x_out,
                                                     const float* norm_weight, float norm_eps, int ggml_type, int nseg, const void* const* w, void* const* y,
                                                     const int64_t* n, int y_dtype, int64_t K, void* stream) {
  TGA_REQUIRE(norm_weight && y_experts && probs && x_in && x_out && x_in != x_out, "tga_moe_combine_rmsnorm_qlinear_multi: null pointer, or x_out aliases x_in");
  const CombineIn c = {y_experts, probs, k, x_out};
  return qlinear_multi_impl(&c, nullptr, norm_weight, norm_eps, ggml_type, nseg, w, y, n, x_in, TGA_F32, y_dtype, 1, K, 0, nullptr, 0, 0, stream);
}

extern "C" int tga_qlinear(int ggml_type, const void* w, const void* x, int x_dtype, void* y, int y_dtype,
                           int M, int64_t N, int64_t K, void* stream) {
  const void* ws[1] = {w}; void* ys[1] = {y}; int64_t ns[1] = {N};
  return tga_qlinear_multi(ggml_type, 1, ws, ys, ns, x, x_dtype, y_dtype, M, K, 0, nullptr, 0, 0, stream);
}

// ExpertWeights.__call__ (tinygrad/llm/model.py:21-27): per (token, slot) job j, y[j] = x[j / jobs_per_x_row] @ W[sel[j]]^T over a
// stacked (n_experts, N, K) weight; with w_up the output is silu(x Wgate[e]^T) * (x Wup[e]^T) (model.py:129).  Only the
// selected experts' bytes are read (the indexed load the reference's codegen produces from weight[sel]).
struct RouteIn { const float* logits; int k, gating, norm_topk; float scale; float* probs_out; };
static int qlinear_experts_impl(const RouteIn* route, int ggml_type, const void* w, const void* w_up, int64_t n_experts, int32_t* sel, int n_jobs,
                                int jobs_per_x_row, const void* x, int x_dtype, void* y, int y_dtype, int64_t N, int64_t K, void* stream) {
  TGA_REQUIRE(w && sel && x && y, "tga_qlinear_experts: null pointer");
  TGA_REQUIRE(n_jobs >= 1 && n_jobs <= 65535 && jobs_per_x_row >= 1 && n_experts >= 1, "tga_qlinear_experts: bad job geometry");
  TGA_REQUIRE(x_dtype == TGA_F16 || x_dtype == TGA_F32, "tga_qlinear_experts: x_dtype must be TGA_F16 or TGA_F32");
  TGA_REQUIRE(y_dtype == TGA_F16 || y_dtype == TGA_F32, "tga_qlinear_experts: y_dtype must be TGA_F16 or TGA_F32");
  int bw, bb;
  switch (ggml_type) { case GGML_Q4_0: bw = 32; bb = 18; break; case GGML_Q8_0: bw = 32; bb = 34; break; case GGML_MXFP4: bw = 32; bb = 17; break;
    case GGML_Q6_K: bw = 256; bb = 210; break; case GGML_Q4_K: bw = 256; bb = 144; break; case GGML_Q5_K: bw = 256; bb = 176; break;
    case GGML_F16: bw = 64; bb = 128; break;
    case GGML_Q4_1: bw = 64; bb = 40; break; case GGML_Q5_0: bw = 64; bb = 44; break; case GGML_Q5_1: bw = 64; bb = 48; break;   // block pairs
    case GGML_IQ4_XS: bw = 256; bb = 136; break; case GGML_IQ3_XXS: bw = 256; bb = 98; break; case GGML_IQ3_S: bw = 256; bb = 110; break; case GGML_IQ2_S: bw = 256; bb = 82; break;
    case GGML_Q1_0: bw = 128; bb = 18; break;
    default: return tga_set_error("GGML type '%d' is not supported!", ggml_type); }
  TGA_REQUIRE(K > 0 && K % bw == 0 && N > 0, "tga_qlinear_experts: K=%lld must be a positive multiple of %d", (long long)K, bw);
  TGA_REQUIRE((ggml_type != GGML_Q4_K && ggml_type != GGML_Q5_K && ggml_type != GGML_Q4_1 && ggml_type != GGML_Q5_0 && ggml_type != GGML_Q5_1 && ggml_type != GGML_IQ4_XS) || ((((uintptr_t)w | (uintptr_t)w_up) & 3) == 0),
              "tga_qlinear_experts: Q4_K / Q5_K / Q4_1 / Q5_0 / Q5_1 / IQ4_XS weights must be 4-byte aligned");
  QArgs a = {};
  a.nseg = w_up ? 2 : 1; a.x = x; a.x_f32 = x_dtype == TGA_F32; a.y_f32 = y_dtype == TGA_F32; a.epilogue = w_up ? 2 : 0; a.K = (int)K;
  a.w[0] = (const uint8_t*)w; a.w[1] = (const uint8_t*)w_up; a.y[0] = y; a.n[0] = N; a.n[1] = N; a.ntot = N;
  a.sel = sel; a.estride = (long long)N * (K / bw) * bb; a.ystride = N; a.xdiv = jobs_per_x_row; a.xdiv_jobs = n_jobs;
  if (route) {
    a.route_logits = route->logits; a.route_E = (int)n_experts; a.route_k = route->k; a.route_gating = route->gating; a.route_norm_topk = route->norm_topk;
    a.route_scale = route->scale; a.route_probs_out = route->probs_out;
  }
  const bool pair = (K / 32) % 2 == 0 && ((uintptr_t)w & 3) == 0 && (!w_up || ((uintptr_t)w_up & 3) == 0) && a.estride % 4 == 0;
  const int fmt = ggml_type == GGML_Q4_0 ? (pair ? F_Q4_0P : -1) : ggml_type == GGML_Q8_0 ? (pair ? F_Q8_0P : -1) : ggml_type;
  TGA_REQUIRE(fmt >= 0, "tga_qlinear_experts: Q4_0/Q8_0 expert weights need K %% 64 == 0 and 4-byte aligned experts");
  const int rc = tga_qgemv1_dispatch(fmt, a, (hipStream_t)stream);
  TGA_REQUIRE(rc >= 0, "tga_qlinear_experts: shape K=%lld outside the expert GEMV path", (long long)K);
  return rc;
}

extern "C" int tga_qlinear_experts(int ggml_type, const void* w, const void* w_up, int64_t n_experts, const int32_t* sel, int n_jobs,
                                   int jobs_per_x_row, const void* x, int x_dtype, void* y, int y_dtype, int64_t N, int64_t K, void* stream) {
  return qlinear_experts_impl(nullptr, ggml_type, w, w_up, n_experts, (int32_t*)sel, n_jobs, jobs_per_x_row, x, x_dtype, y, y_dtype, N, K, stream);
}

// The expert gate/up jobs of ONE token with the gating inside the launch: every workgroup computes the scores, the pairwise top-k and
// the weights from the router logits (tinygrad/llm/model.py:112-128) for itself, job j multiplies the j-th selected expert, and the
// selection / weights are written to sel_out / probs_out (k entries) for the launches that follow (expert down, weighted sum).
// y[j] = silu(x Wgate[e_j]^T) * (x Wup[e_j]^T), x one fp16 row of at most 4096 values.
extern "C" int tga_qlinear_experts_routed(int ggml_type, const void* w_gate, const void* w_up, int64_t n_experts, const float* logits, int k,
                                          int gating, int norm_topk_prob, float scale, int32_t* sel_out, float* probs_out,
                                          const void* x_f16, void* y, int y_dtype, int64_t N, int64_t K, void* stream) {
  TGA_REQUIRE(logits && sel_out && probs_out && w_up, "tga_qlinear_experts_routed: null pointer");
  TGA_REQUIRE(n_experts >= 1 && n_experts <= 1024 && k >= 1 && k <= 64 && k <= n_experts, "tga_qlinear_experts_routed: bad geometry (k <= 64, n_experts <= 1024)");
  TGA_REQUIRE(gating >= 1 && gating <= 4, "tga_qlinear_experts_routed: unknown ExpertGating %d", gating);
  const RouteIn r = {logits, k, gating, norm_topk_prob, scale, probs_out};
  return qlinear_experts_impl(&r, ggml_type, w_gate, w_up, n_experts, sel_out, k, k, x_f16, TGA_F16, y, y_dtype, N, K, stream);
}

// The same for n_tokens tokens in one launch (ExpertWeights.__call__ over a (B, T, k) selection, model.py:21-27): jobs t k .. t k + k - 1 are token t's,
// gated from row t of the logits; x (n_tokens, K) fp16, y (n_tokens k, N), sel_out / probs_out (n_tokens, k).
extern "C" int tga_qlinear_experts_routed_rows(int ggml_type, const void* w_gate, const void* w_up, int64_t n_experts, const float* logits, int n_tokens, int k,
                                               int gating, int norm_topk_prob, float scale, int32_t* sel_out, float* probs_out,
                                               const void* x_f16, void* y, int y_dtype, int64_t N, int64_t K, void* stream) {
  TGA_REQUIRE(logits && sel_out && probs_out && w_up, "tga_qlinear_experts_routed_rows: null pointer");
  TGA_REQUIRE(n_tokens >= 1 && n_experts >= 1 && n_experts <= 1024 && k >= 1 && k <= 64 && k <= n_experts, "tga_qlinear_experts_routed_rows: bad geometry (k <= 64, n_experts <= 1024)");
  TGA_REQUIRE((long long)n_tokens * k <= 65535, "tga_qlinear_experts_routed_rows: %d x %d jobs exceed one launch", n_tokens, k);
  TGA_REQUIRE(gating >= 1 && gating <= 4, "tga_qlinear_experts_routed_rows: unknown ExpertGating %d", gating);
  const RouteIn r = {logits, k, gating, norm_topk_prob, scale, probs_out};
  return qlinear_experts_impl(&r, ggml_type, w_gate, w_up, n_experts, sel_out, n_tokens * k, k, x_f16, TGA_F16, y, y_dtype, N, K, stream);
}
