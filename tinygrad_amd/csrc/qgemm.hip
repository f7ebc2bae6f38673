// Small-batch GEMM over GGUF blocks on the matrix cores (3 <= M <= 8 activation rows), for the same call sites as qgemv.hip
// (x.linear(W.T) over a lazily dequantized weight: tinygrad/nn/__init__.py:177, tinygrad/mixin/op.py:367-392).
//
// The dot2 kernel decodes a weight once per TWO activation rows and multiplies on the VALU, so from M = 4 on it is bound by
// VALU issue, not by HBM.  Here a unit is decoded ONCE into true fp16 weights ((pattern - bias) * block scale, one fp16 rounding -
// the rounding of the reference's fp16 weight cast, tinygrad/llm/model.py:376) and v_mfma_f32_16x16x32_f16 multiplies it with all
// activation rows at once (M padded to 16 columns): the VALU work per weight byte no longer depends on M.
//
// Mapping: a wave owns 16 weight rows at a time.  Lane l = 16 g + r loads unit 4 s + g of row r (step s): the four lane groups
// cover four consecutive units of each row.  A unit's XV vectors of 8 fp16 are the A operands of XV MFMAs; the B operand of lane
// 16 g + c is activation row c's vector of the SAME unit (zero for c >= M), read from the LDS staging that qgemv.hip uses
// ([row][vector][unit]).  Both operands of a lane group name the same 8 k-values element by element, which is all the MFMA needs.
// The four waves of a workgroup take the steps of a row group round-robin (a split of K) and their 16 x 16 partial results meet
// in LDS.  K is walked in LDS-sized chunks when M * K does not fit.  Q4_0 / Q8_0 with K <= 4096 take qgemm_dma.hip instead (weights
// through LDS in contiguous pieces).  An eight-wave variant with one workgroup per CU (activations staged once per CU) was measured and
// dropped: faster on Q8_0 14336 x 4096 (19.5 against 24.6 us at M = 4), slower on the Q6_K lm-head (160 against 148 us at M = 8) and on
// 2048-wide fp16 linears, and the shapes it won on are the ones the LDS-fed kernel now serves.
#include "qfmt.h"

typedef _Float16 v8f16 __attribute__((ext_vector_type(8)));
typedef float v4f32 __attribute__((ext_vector_type(4)));

#define QM_LDS_BUDGET (72 * 1024)     // activations of one chunk when two workgroups share a CU
#define QM_LDS_CU (160 * 1024)        // LDS of one CU

template <int T_, int M, int NW, bool MS>
__global__ __launch_bounds__(NW * 64) void qgemm_mfma_kernel(const QArgs args) {
  const QArgs a = args;                                  // field reads become kernel-argument loads in the entry block
  constexpr int T = T_;
  using F = Fmt<T>;
  typedef typename F::Raw Raw;
  extern __shared__ u32x4 lds[];
  __shared__ float part[2][NW][16][9];                   // [parity][wave][weight row][activation row]
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int r = lane & 15, g = lane >> 4;
  uint32_t kc[F::NKC];
  F::consts(kc);
  const long long ngroups = (a.ntot + 15) / 16;
  // Several weight matrices in one launch (q / k / v): rows run over the segments in order, every segment a multiple of 16 rows (checked by the
  // dispatch), so a 16-row group lies inside one segment.  first row of a group -> segment, first row inside the segment
  // MS (several matrices) is a template parameter and every per-segment field is picked with selects: an index that is only known at run
  // time would put the argument arrays into memory, and the loads that fetch them back sit in front of every weight load.
  auto seg_of = [&](long long row0, int& sg, long long& local0) {
    sg = 0; local0 = row0;
    if constexpr (MS) { if (local0 >= a.n[0]) { local0 -= a.n[0]; sg = 1; if (a.nseg > 2 && local0 >= a.n[1]) { local0 -= a.n[1]; sg = 2; } } }
  };
  auto rows_of = [&](int sg) -> long long { return !MS ? a.n[0] : sg == 0 ? a.n[0] : sg == 1 ? a.n[1] : a.n[2]; };
  auto w_of = [&](int sg) -> const uint8_t* { return !MS ? a.w[0] : sg == 0 ? a.w[0] : sg == 1 ? a.w[1] : a.w[2]; };
  auto store_tile = [&](long long row0, int p) {                    // 256 threads = 16 weight rows x 16 activation rows
    int sg; long long l0; seg_of(row0, sg, l0);
    const int t = threadIdx.x, wr = (t >> 4) & 15, c = t & 15;
    const long long nrows = rows_of(sg);
    if (t < 256 && c < M && l0 + wr < nrows) {
      float v = 0.f;
#pragma unroll
      for (int w = 0; w < NW; w++) v += part[p][w][wr][c];
      const long long o = (long long)c * nrows + l0 + wr;
      if (a.epilogue == 1) v += (!MS ? a.resid[0] : sg == 0 ? a.resid[0] : sg == 1 ? a.resid[1] : a.resid[2])[o];      // y = resid + x W^T (may be in place: each element is read and written by one thread)
      void* yb = !MS ? a.y[0] : sg == 0 ? a.y[0] : sg == 1 ? a.y[1] : a.y[2];
      if (a.y_f32) ((float*)yb)[o] = v; else ((_Float16*)yb)[o] = (_Float16)v;
    }
  };
  if (a.nchunks == 1) {
    // ---- the whole K in LDS, staged once per workgroup: the workgroup walks its row groups, the NW waves split K (wave w takes steps
    // w, w + NW, ... of every group), and each wave runs one software pipeline over ALL its (row group, step) pairs.  Every load is
    // unconditional and in straight-line code (pairs past the end reload the last one; a step that does not exist for this wave multiplies
    // zeros), so the compiler's s_waitcnt placement keeps the ring in flight across row groups and across the one barrier per group in
    // which the waves' partial tiles meet (two LDS slots in turn, so a wave may run one group ahead).
    const int cu = a.nu, nsteps = (cu + 3) >> 2, spw = (nsteps + NW - 1) / NW;   // steps per wave and row group, the same for all waves
    const long long G = ((long long)blockIdx.x < ngroups) ? (ngroups - blockIdx.x + gridDim.x - 1) / gridDim.x : 0;
    const long long T = G * spw;
    u32x4* xs = lds;
    const bool ragged = (cu & 3) != 0 || (nsteps % NW) != 0;
    constexpr int D = 3;                                              // ring of loads
    Raw b[D];
    long long lj = 0; int li = 0;                                       // load stream: row group index (of this workgroup), step index
    auto issue = [&](Raw& buf) {
      const long long grp = (long long)blockIdx.x + lj * gridDim.x;
      int sg; long long l0; seg_of(grp * 16, sg, l0);
      const long long row = l0 + r, nr = rows_of(sg), rowc = row < nr ? row : nr - 1;
      const uint8_t* wb = w_of(sg);
      const int ul = 4 * (wave + NW * li) + g;
      buf = F::load(wb + rowc * a.row_bytes, ul < cu ? ul : cu - 1);
      const bool more = lj * spw + li + 1 < T;                          // past the end: stay on the last step
      li = more ? (li + 1 == spw ? 0 : li + 1) : li;
      lj = more && li == 0 ? lj + 1 : lj;
    };
    if (T > 0) {
      // the activations of this thread's first staging item are requested FIRST (loads return in issue order: behind the weights they would
      // arrive last), the weights second; the staging arithmetic runs while the weights are in flight
      float* cs = (float*)(lds + M * F::XV * cu);
      const int nitems = M * cu, it0 = (int)threadIdx.x < nitems ? (int)threadIdx.x : nitems - 1;
      const int m0 = it0 / cu, ul0 = it0 - m0 * cu;
      uint32_t nx0[F::UW / 2];
      stage_fetch<T_>(a, m0, ul0, nx0);
#pragma unroll
      for (int d = 0; d < D - 1; d++) issue(b[d]);
      if ((int)threadIdx.x < nitems) stage_put<T_>(nx0, xs, cs, m0, ul0, cu);
      stage_chunk<T_, M, NW * 64>(a, xs, cs, 0, cu, threadIdx.x + NW * 64);      // (more items than threads: K > 4096 or so)
      __syncthreads();
      v4f32 acc0 = {0.f, 0.f, 0.f, 0.f}, acc1 = {0.f, 0.f, 0.f, 0.f};   // two chains: an MFMA does not wait for the one just issued
      long long cj = 0; int ci = 0, par = 0;                            // compute stream
      auto compute = [&](const Raw& buf) {
        const int ul = 4 * (wave + NW * ci) + g;
        uint32_t wv[F::NWV];
        F::decode(buf, wv, kc);
        F::to_f16(buf, wv);
        const bool uval = ul < cu;
        const int ulc = uval ? ul : cu - 1;
        u32x4 bv[F::XV];
#pragma unroll
        for (int v = 0; v < F::XV; v++) { bv[v] = u32x4{0u, 0u, 0u, 0u}; if (r < M) bv[v] = xs[(r * F::XV + v) * cu + ulc]; }
#pragma unroll
        for (int v = 0; v < F::XV; v++) {
          u32x4 av = {wv[4 * v], wv[4 * v + 1], wv[4 * v + 2], wv[4 * v + 3]};
          if (ragged && !uval) av = u32x4{0u, 0u, 0u, 0u};
          if (v & 1) acc1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8f16, av), __builtin_bit_cast(v8f16, bv[v]), acc1, 0, 0, 0);
          else acc0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8f16, av), __builtin_bit_cast(v8f16, bv[v]), acc0, 0, 0, 0);
        }
        if (++ci == spw) {                                              // row group complete: the waves' partial tiles meet in LDS
          const long long row0 = ((long long)blockIdx.x + cj * gridDim.x) * 16;
#pragma unroll
          for (int i = 0; i < 4; i++) if (r < 9) part[par][wave][4 * g + i][r] = acc0[i] + acc1[i];
          __syncthreads();
          store_tile(row0, par);
          par ^= 1;
          acc0 = v4f32{0.f, 0.f, 0.f, 0.f}; acc1 = v4f32{0.f, 0.f, 0.f, 0.f};
          ci = 0; cj++;
        }
      };
      long long t = 0;
      for (; t + D <= T; t += D) {
#pragma unroll
        for (int d = 0; d < D; d++) { issue(b[(d + D - 1) % D]); compute(b[d]); }
      }
#pragma unroll
      for (int d = 0; d < D - 1; d++) if (t + d < T) compute(b[d]);
    }
    return;
  }
  if constexpr (NW == 4)                                              // K in LDS-sized chunks: four waves, one row group at a time
  for (long long grp = blockIdx.x; grp < ngroups; grp += gridDim.x) {
    const long long row0 = grp * 16;
    int sg0; long long l00; seg_of(row0, sg0, l00);
    const long long myrow = l00 + r < rows_of(sg0) ? l00 + r : rows_of(sg0) - 1;   // ragged last group: reload a valid row, results dropped
    const uint8_t* rowp = w_of(sg0) + myrow * a.row_bytes;
    v4f32 acc = {0.f, 0.f, 0.f, 0.f};
    for (int ch = 0; ch < a.nchunks; ch++) {
      const int u0 = ch * a.chunk_u, cu = min(a.chunk_u, a.nu - u0);
      u32x4* xs = lds; float* cs = (float*)(lds + M * F::XV * cu);
      const int nsteps = (cu + 3) >> 2;                                 // steps of 4 units in this chunk; wave w takes s = w, w + 4, ...
      Raw b0, b1;
      auto issue = [&](Raw& buf, int s) { const int ul = 4 * s + g; buf = F::load(rowp, u0 + (ul < cu ? ul : cu - 1)); };
      if (wave < nsteps) issue(b0, wave);                               // first loads ahead of the staging
      if (a.nchunks > 1 || grp == (long long)blockIdx.x) {              // a single chunk is staged once per workgroup
        __syncthreads();
        stage_chunk<T, M, NW * 64>(a, xs, cs, u0, cu);
        __syncthreads();
      }
      const bool ragged = (cu & 3) != 0;
      auto compute = [&](const Raw& buf, int s) {
        const int ul = 4 * s + g;
        uint32_t wv[F::NWV];
        F::decode(buf, wv, kc);
        F::to_f16(buf, wv);
        const bool uval = ul < cu;
        const int ulc = uval ? ul : cu - 1;
#pragma unroll
        for (int v = 0; v < F::XV; v++) {
          u32x4 av = {wv[4 * v], wv[4 * v + 1], wv[4 * v + 2], wv[4 * v + 3]};
          if (ragged && !uval) av = u32x4{0u, 0u, 0u, 0u};      // (whole steps only when the chunk is a multiple of 4 units)
          u32x4 bv = {0u, 0u, 0u, 0u};
          if (r < M) bv = xs[(r * F::XV + v) * cu + ulc];
          acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8f16, av), __builtin_bit_cast(v8f16, bv), acc, 0, 0, 0);
        }
      };
      for (int s = wave; s < nsteps; s += 8) {
        if (s + 4 < nsteps) issue(b1, s + 4);
        compute(b0, s);
        if (s + 4 < nsteps) {
          if (s + 8 < nsteps) issue(b0, s + 8);
          compute(b1, s + 4);
        }
      }
    }
    // D: lane (g, c) holds weight rows 4 g + i (i = 0..3) for activation row c
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; i++) if (r < 9) part[0][wave][4 * g + i][r] = acc[i];
    __syncthreads();
    store_tile(row0, 0);
  }
}

static int qm_cu_count() {
  static int n = 0;
  if (!n) { int dev = 0; hipDeviceProp_t p; n = (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&p, dev) == hipSuccess) ? p.multiProcessorCount : 256; }
  return n;
}

template <int T, int M, int NW, bool MS>
static int launch_qgemm_ms(const QArgs& a, long long grid, size_t lds, hipStream_t s) {
  auto kern = qgemm_mfma_kernel<T, M, NW, MS>;
  // dynamic LDS up to what the CU holds beside the kernel's static arrays; set once per instantiation (thread-safe)
  static const hipError_t configured = [&]() {
    hipFuncAttributes fa;
    hipError_t e = hipFuncGetAttributes(&fa, (const void*)kern);
    if (e != hipSuccess) return e;
    return hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)(QM_LDS_CU - fa.sharedSizeBytes));
  }();
  TGA_HIP(configured);
  kern<<<dim3((unsigned)grid), dim3(NW * 64), lds, s>>>(a);
  TGA_LAUNCH_CHECK();
  return 0;
}

template <int T, int M, int NW>
static int launch_qgemm_nw(const QArgs& a, long long grid, size_t lds, hipStream_t s) {
  return a.nseg > 1 ? launch_qgemm_ms<T, M, NW, true>(a, grid, lds, s) : launch_qgemm_ms<T, M, NW, false>(a, grid, lds, s);
}

template <int T, int M>
static int launch_qgemm(QArgs a, hipStream_t s) {
  using F = Fmt<T>;
  const int per_unit = M * (16 * F::XV + 4 * F::NG);
  a.nu = a.K / F::UW;
  a.row_bytes = (long long)(a.K / F::BW) * F::BB;
  const long long ngroups = (a.ntot + 15) / 16;
  const int cus = qm_cu_count();
  // LDS budget for one chunk of activations: two workgroups per CU, or the whole CU when there is at most one row group per CU anyway
  const int budget = (ngroups <= cus ? 2 * QM_LDS_BUDGET : QM_LDS_BUDGET) - fmt_tab<F>();
  int cu = budget / per_unit; cu -= cu % 16; if (cu < 16) cu = 16;
  if (cu >= a.nu) { a.chunk_u = a.nu; a.nchunks = 1; } else { a.nchunks = (a.nu + cu - 1) / cu; a.chunk_u = ((a.nu + a.nchunks - 1) / a.nchunks + 15) / 16 * 16; }
  const size_t lds = (size_t)per_unit * a.chunk_u;
  // single chunk: the activations are staged once per workgroup, so no more workgroups than stay resident (by LDS, at most 8 per
  // CU); chunked K: every row group restages each chunk, one group per workgroup
  int resident = (int)(QM_LDS_CU / (lds + 6 * 1024 + fmt_tab<F>())); resident = resident < 1 ? 1 : resident > 8 ? 8 : resident;
  long long grid = ngroups;
  const long long cap = (long long)cus * (a.nchunks == 1 ? resident : 8);
  if (grid > cap) grid = cap;
  return launch_qgemm_nw<T, M, 4>(a, grid, lds, s);
}

template <int T>
static int launch_qgemm_m(const QArgs& a, int M, hipStream_t s) {
  switch (M) {
    case 3: return launch_qgemm<T, 3>(a, s);
    case 4: return launch_qgemm<T, 4>(a, s);
    case 5: return launch_qgemm<T, 5>(a, s);
    case 6: return launch_qgemm<T, 6>(a, s);
    case 7: return launch_qgemm<T, 7>(a, s);
    case 8: return launch_qgemm<T, 8>(a, s);
  }
  return -1;
}

// Returns -1 when the call is outside this kernel's range (the caller then takes the dot2 kernel): linears (plain or with the residual / bias
// row added) over one to three
// matrices (q / k / v in one launch; with several, each a multiple of 16 rows) of the block-pair / superblock formats with 3 <= M <= 8.
int tga_qgemm_mfma_dispatch(int fmt, const QArgs& a, int M, hipStream_t s) {
  if (M < 3 || M > 8 || a.nseg < 1 || a.nseg > 3 || a.epilogue > 1 || a.sel || a.x_staged || a.y_stage_fmt || a.norm_w) return -1;
  if (a.nseg > 1) for (int i = 0; i < a.nseg; i++) if (a.n[i] % 16 != 0) return -1;      // several matrices: every 16-row group inside one of them
  if (((uintptr_t)a.x & 15) != 0) return -1;
  switch (fmt) {
    case F_Q4_0P: return launch_qgemm_m<F_Q4_0P>(a, M, s);
    case F_Q8_0P: return launch_qgemm_m<F_Q8_0P>(a, M, s);
    case GGML_Q6_K: return launch_qgemm_m<GGML_Q6_K>(a, M, s);
    case GGML_Q4_K: return launch_qgemm_m<GGML_Q4_K>(a, M, s);
    case GGML_Q5_K: return launch_qgemm_m<GGML_Q5_K>(a, M, s);
    case GGML_Q4_1: return launch_qgemm_m<GGML_Q4_1>(a, M, s);
    case GGML_Q5_0: return launch_qgemm_m<GGML_Q5_0>(a, M, s);
    case GGML_Q5_1: return launch_qgemm_m<GGML_Q5_1>(a, M, s);
    case GGML_IQ4_XS: return launch_qgemm_m<GGML_IQ4_XS>(a, M, s);
    case GGML_IQ3_XXS: return launch_qgemm_m<GGML_IQ3_XXS>(a, M, s);
    case GGML_IQ3_S: return launch_qgemm_m<GGML_IQ3_S>(a, M, s);
    case GGML_IQ2_S: return launch_qgemm_m<GGML_IQ2_S>(a, M, s);
    case GGML_Q1_0: return launch_qgemm_m<GGML_Q1_0>(a, M, s);
    case GGML_F16: return launch_qgemm_m<GGML_F16>(a, M, s);
    case GGML_MXFP4: return launch_qgemm_m<GGML_MXFP4>(a, M, s);
  }
  return -1;
}
