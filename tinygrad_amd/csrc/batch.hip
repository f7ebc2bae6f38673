// Pieces of the batched decode step (2..8 sequences in lockstep on this path) that have no batch-1 twin: the expert GEMMs of a MoE block with the
// (token, slot) jobs grouped by expert, so that an expert selected by several tokens is streamed once (ExpertWeights.__call__ over a
// (B, T, k) selection, tinygrad/llm/model.py:21-27, 110-135; the reference's indexed load reads every selected expert once per job).
//
// expert_jobs_kernel turns the selection sel[n_jobs] into a table per expert: how many jobs picked it (at most 8: the experts of one token are
// distinct and there are at most 8 tokens) and which.  qexperts_mfma_kernel then runs one small-batch GEMM per expert that has jobs, on the
// matrix cores like qgemm.hip: a unit of the expert's weight is decoded once into true fp16 weights and v_mfma_f32_16x16x32_f16 multiplies
// it with the activation rows of all its jobs at once (rows gathered into LDS in the staged order, padded to 16 columns); with a second
// weight stack the epilogue is silu(gate) * up (model.py:129).  Workgroup (bx, e): expert e, row groups bx, bx + gridDim.x, ...
#include "qfmt.h"

typedef _Float16 v8f16 __attribute__((ext_vector_type(8)));
typedef float v4f32 __attribute__((ext_vector_type(4)));

#define EJ_STRIDE 16           // int32 words per expert in the job table: [0] number of jobs, [1..8] job indices
#define EXP_THREADS 256
#define EXP_MAX_ROWS 8

__global__ __launch_bounds__(256) void expert_jobs_kernel(const int* __restrict__ sel, int n_jobs, int n_experts, int* __restrict__ table, int* __restrict__ overflow) {
  extern __shared__ int cnt[];
  for (int e = threadIdx.x; e < n_experts; e += 256) cnt[e] = 0;
  __syncthreads();
  for (int j = threadIdx.x; j < n_jobs; j += 256) {
    const int e = sel[j];
    if ((unsigned)e >= (unsigned)n_experts) { atomicOr(overflow, 2); continue; }      // an expert id outside the stack: the job is dropped, the host sees the flag
    const int p = atomicAdd(&cnt[e], 1);
    if (p < EXP_MAX_ROWS) table[e * EJ_STRIDE + 1 + p] = j; else atomicOr(overflow, 1);
  }
  __syncthreads();
  for (int e = threadIdx.x; e < n_experts; e += 256) table[e * EJ_STRIDE] = cnt[e] < EXP_MAX_ROWS ? cnt[e] : EXP_MAX_ROWS;
}

struct ExpArgs {
  const uint8_t* w; const uint8_t* w_up; long long estride;     // (E, N, K) stacks in GGUF blocks, bytes per expert
  const int* table;                                             // expert_jobs_kernel's output
  const uint16_t* x; int xdiv;                                  // fp16 activation rows; job j reads row j / xdiv
  void* y; int y_f32;                                           // (n_jobs, N): job j writes row j
  long long N; int K, nu; long long row_bytes;
};

template <int T_, bool TWO>
__global__ __launch_bounds__(EXP_THREADS) void qexperts_mfma_kernel(const ExpArgs args) {
  const ExpArgs a = args;
  constexpr int T = T_;
  using F = Fmt<T>;
  typedef typename F::Raw Raw;
  constexpr int NP = F::UW / 2;
  extern __shared__ u32x4 xs[];                                  // [(row * XV + vector) * nu + unit]
  __shared__ float part[TWO ? 2 : 1][4][16][17];
  __shared__ int jobs[EXP_MAX_ROWS];
  const int e = blockIdx.y;
  const int count = a.table[e * EJ_STRIDE];
  const long long ngroups = (a.N + 15) / 16;
  if (count == 0 || (long long)blockIdx.x >= ngroups) return;     // (uniform over the workgroup)
  if (threadIdx.x < EXP_MAX_ROWS) jobs[threadIdx.x] = threadIdx.x < count ? a.table[e * EJ_STRIDE + 1 + threadIdx.x] : 0;
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int r = lane & 15, g = lane >> 4;
  uint32_t kc[F::NKC];
  F::consts(kc);
  const int cu = a.nu, nsteps = (cu + 3) >> 2, spw = (nsteps + 3) >> 2;   // steps of four units per wave and row group
  const long long G = (ngroups - blockIdx.x + gridDim.x - 1) / gridDim.x;
  const long long TT = G * spw;
  const bool ragged = (cu & 3) != 0 || (nsteps & 3) != 0;
  const uint8_t* wg = a.w + (long long)e * a.estride;
  const uint8_t* wu = TWO ? a.w_up + (long long)e * a.estride : nullptr;
  Raw b[3], bu[TWO ? 3 : 1];
  long long lj = 0; int li = 0;                                   // load stream: row group index (of this workgroup), step index
  auto issue = [&](int slot) {                                     // every load unconditional: rows and units clamped, steps past the end reload the last one
    const long long grp = (long long)blockIdx.x + lj * gridDim.x;
    const long long row = grp * 16 + r, rowc = row < a.N ? row : a.N - 1;
    const int ul = 4 * (wave + 4 * li) + g, ulc = ul < cu ? ul : cu - 1;
    b[slot] = F::load(wg + rowc * a.row_bytes, ulc);
    if constexpr (TWO) bu[slot] = F::load(wu + rowc * a.row_bytes, ulc);
    const bool more = lj * spw + li + 1 < TT;
    li = more ? (li + 1 == spw ? 0 : li + 1) : li;
    lj = more && li == 0 ? lj + 1 : lj;
  };
  issue(0);
  __syncthreads();                                                 // the job list
  for (int i = threadIdx.x; i < EXP_MAX_ROWS * cu; i += EXP_THREADS) {   // the activation rows of this expert's jobs, gathered, in staged order; rows beyond `count` are zero
    const int m = i / cu, ul = i - m * cu;
    u32x4 xv[F::XV];
    if (m < count) {
      const uint16_t* x = a.x + (long long)(jobs[m] / a.xdiv) * a.K;
      uint32_t nx[NP];
#pragma unroll
      for (int k = 0; k < NP; k += 4) { const u32x4 v = *(const u32x4*)(x + F::xoff(ul, k)); nx[k] = v.x; nx[k + 1] = v.y; nx[k + 2] = v.z; nx[k + 3] = v.w; }
      float c[F::NG];
      F::stage(nx, xv, c);
    } else {
#pragma unroll
      for (int t = 0; t < F::XV; t++) xv[t] = u32x4{0u, 0u, 0u, 0u};
    }
#pragma unroll
    for (int t = 0; t < F::XV; t++) xs[(m * F::XV + t) * cu + ul] = xv[t];
  }
  __syncthreads();
  issue(1);
  v4f32 acc = {0.f, 0.f, 0.f, 0.f}, accu = {0.f, 0.f, 0.f, 0.f};
  long long cj = 0; int ci = 0;                                    // compute stream
  auto mma = [&](const Raw& buf, v4f32& dst, int ulc, bool uval) {
    uint32_t wv[F::NWV];
    F::decode(buf, wv, kc);
    F::to_f16(buf, wv);
#pragma unroll
    for (int v = 0; v < F::XV; v++) {
      u32x4 av = {wv[4 * v], wv[4 * v + 1], wv[4 * v + 2], wv[4 * v + 3]};
      if (ragged && !uval) av = u32x4{0u, 0u, 0u, 0u};
      u32x4 bv = {0u, 0u, 0u, 0u};
      if (r < EXP_MAX_ROWS) bv = xs[(r * F::XV + v) * cu + ulc];
      dst = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8f16, av), __builtin_bit_cast(v8f16, bv), dst, 0, 0, 0);
    }
  };
  auto compute = [&](int slot) {
    const int ul = 4 * (wave + 4 * ci) + g;
    const bool uval = ul < cu;
    const int ulc = uval ? ul : cu - 1;
    mma(b[slot], acc, ulc, uval);
    if constexpr (TWO) mma(bu[slot], accu, ulc, uval);
    if (++ci == spw) {                                              // row group complete: the four waves' partial tiles meet in LDS
      const long long row0 = ((long long)blockIdx.x + cj * gridDim.x) * 16;
#pragma unroll
      for (int i = 0; i < 4; i++) { part[0][wave][4 * g + i][r] = acc[i]; if constexpr (TWO) part[1][wave][4 * g + i][r] = accu[i]; }
      __syncthreads();
      {
        const int t = threadIdx.x, wr = t >> 4, c = t & 15;          // 256 threads = 16 weight rows x 16 activation columns
        if (c < count && row0 + wr < a.N) {
          float v = part[0][0][wr][c] + part[0][1][wr][c] + part[0][2][wr][c] + part[0][3][wr][c];
          if constexpr (TWO) v = silu_f(v) * (part[1][0][wr][c] + part[1][1][wr][c] + part[1][2][wr][c] + part[1][3][wr][c]);
          const long long o = (long long)jobs[c] * a.N + row0 + wr;
          if (a.y_f32) ((float*)a.y)[o] = v; else ((_Float16*)a.y)[o] = (_Float16)v;
        }
      }
      __syncthreads();
      acc = v4f32{0.f, 0.f, 0.f, 0.f}; accu = v4f32{0.f, 0.f, 0.f, 0.f};
      ci = 0; cj++;
    }
  };
  long long t = 0;
  for (; t + 3 <= TT; t += 3) {
    issue(2); compute(0);
    issue(0); compute(1);
    issue(1); compute(2);
  }
  if (t < TT) compute(0);
  if (t + 1 < TT) compute(1);
}

static int exp_cu_count() {
  static int n = 0;
  if (!n) { int dev = 0; hipDeviceProp_t p; n = (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&p, dev) == hipSuccess) ? p.multiProcessorCount : 256; }
  return n;
}

template <int T, bool TWO>
static int launch_qexperts(ExpArgs a, int n_experts, int n_jobs, int xdiv_hint, hipStream_t s) {
  using F = Fmt<T>;
  a.nu = a.K / F::UW;
  a.row_bytes = (long long)(a.K / F::BW) * F::BB;
  const size_t lds = (size_t)EXP_MAX_ROWS * F::XV * a.nu * 16;
  TGA_REQUIRE(lds <= 144 * 1024 - fmt_tab<F>(), "tga_qlinear_experts_grouped: K=%d does not fit the activation staging (%zu bytes of LDS)", a.K, lds);
  const long long ngroups = (a.N + 15) / 16;
  // About two workgroups per CU over the experts that have jobs.  How many do is only known on the device; the launch is sized for the number
  // expected when the tokens pick independently (n_jobs = B k jobs over E experts, each token k distinct ones): E (1 - (1 - k / E)^B) with
  // k = jobs_per_x_row for the gate/up launch; the down launch (one job per row) is told the same k through xdiv_hint.
  const int kk = xdiv_hint > 0 ? xdiv_hint : 1, nb = (n_jobs + kk - 1) / kk;
  double miss = 1.0; for (int t = 0; t < nb; t++) miss *= 1.0 - (double)(kk < n_experts ? kk : n_experts) / (double)n_experts;
  double distinct = (double)n_experts * (1.0 - miss); if (distinct < 1.0) distinct = 1.0; if (distinct > n_jobs) distinct = n_jobs;
  // (measured on the OLMoE-arch batched step, B = 8: 1 / 2 / 3 / 4 workgroups per CU = 3196 / 3699 / 3755 / 3812 tok/s; 32 KB of staged rows per workgroup)
  const int wg_per_cu = 4;
  long long gx = (long long)((double)wg_per_cu * exp_cu_count() / distinct + 0.5);
  if (gx > ngroups) gx = ngroups;
  if (gx < 1) gx = 1;
  auto kern = qexperts_mfma_kernel<T, TWO>;
  if (lds > 48 * 1024) {
    static const hipError_t configured = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, 144 * 1024 - fmt_tab<F>());   // once per instantiation, thread-safe
    TGA_HIP(configured);
  }
  kern<<<dim3((unsigned)gx, (unsigned)n_experts), dim3(EXP_THREADS), lds, s>>>(a);
  TGA_LAUNCH_CHECK();
  return 0;
}

template <int T>
static int launch_qexperts_t(const ExpArgs& a, int n_experts, int n_jobs, int xdiv_hint, hipStream_t s) {
  return a.w_up ? launch_qexperts<T, true>(a, n_experts, n_jobs, xdiv_hint, s) : launch_qexperts<T, false>(a, n_experts, n_jobs, xdiv_hint, s);
}

extern "C" {

int tga_expert_jobs(const int32_t* sel, int n_jobs, int n_experts, int32_t* table, int32_t* flags, void* stream) {
  TGA_REQUIRE(sel && table && flags, "tga_expert_jobs: null pointer");
  TGA_REQUIRE(n_jobs >= 1 && n_experts >= 1 && n_experts <= 8192, "tga_expert_jobs: bad geometry (n_experts <= 8192)");
  expert_jobs_kernel<<<1, 256, n_experts * sizeof(int), (hipStream_t)stream>>>(sel, n_jobs, n_experts, table, flags);
  TGA_LAUNCH_CHECK();
  return 0;
}

int tga_qlinear_experts_grouped(int ggml_type, const void* w, const void* w_up, int64_t n_experts, const int32_t* table, int n_jobs, int jobs_per_x_row,
                                const void* x_f16, void* y, int y_dtype, int64_t N, int64_t K, void* stream) {
  TGA_REQUIRE(w && table && x_f16 && y, "tga_qlinear_experts_grouped: null pointer");
  TGA_REQUIRE(n_jobs >= 1 && jobs_per_x_row >= 1 && n_experts >= 1 && n_experts <= 65535, "tga_qlinear_experts_grouped: bad job geometry");
  TGA_REQUIRE(y_dtype == TGA_F16 || y_dtype == TGA_F32, "tga_qlinear_experts_grouped: y_dtype must be TGA_F16 or TGA_F32");
  TGA_REQUIRE(((uintptr_t)x_f16 & 15) == 0 && K % 8 == 0, "tga_qlinear_experts_grouped: activation rows must be 16-byte aligned");
  int bw, bb;
  switch (ggml_type) { case GGML_Q4_0: bw = 64; bb = 36; break; case GGML_Q8_0: bw = 64; bb = 68; break; case GGML_MXFP4: bw = 32; bb = 17; break;   // Q4_0 / Q8_0 as block pairs
    case GGML_Q6_K: bw = 256; bb = 210; break; case GGML_Q4_K: bw = 256; bb = 144; break; case GGML_Q5_K: bw = 256; bb = 176; break;
    case GGML_F16: bw = 64; bb = 128; break;
    case GGML_Q4_1: bw = 64; bb = 40; break; case GGML_Q5_0: bw = 64; bb = 44; break; case GGML_Q5_1: bw = 64; bb = 48; break;
    case GGML_IQ4_XS: bw = 256; bb = 136; break; case GGML_IQ3_XXS: bw = 256; bb = 98; break; case GGML_IQ3_S: bw = 256; bb = 110; break; case GGML_IQ2_S: bw = 256; bb = 82; break;
    case GGML_Q1_0: bw = 128; bb = 18; break;
    default: return tga_set_error("GGML type '%d' is not supported!", ggml_type); }
  TGA_REQUIRE(K > 0 && K % bw == 0 && N > 0, "tga_qlinear_experts_grouped: K=%lld must be a positive multiple of %d", (long long)K, bw);
  ExpArgs a = {};
  a.w = (const uint8_t*)w; a.w_up = (const uint8_t*)w_up; a.estride = (long long)N * (K / bw) * bb; a.table = table;
  a.x = (const uint16_t*)x_f16; a.xdiv = jobs_per_x_row; a.y = y; a.y_f32 = y_dtype == TGA_F32; a.N = N; a.K = (int)K;
  const bool align2 = ggml_type == GGML_IQ3_XXS || ggml_type == GGML_IQ3_S || ggml_type == GGML_IQ2_S || ggml_type == GGML_Q1_0;      // (blocks of 98 / 110 / 82 / 18 bytes, read with 2-byte aligned loads)
  TGA_REQUIRE(ggml_type == GGML_MXFP4 || ((((uintptr_t)w | (uintptr_t)w_up) & (align2 ? 1 : 3)) == 0 && a.estride % (align2 ? 2 : 4) == 0), "tga_qlinear_experts_grouped: expert weights must be 4-byte aligned (2-byte for IQ3 / IQ2 / Q1_0)");
  hipStream_t s = (hipStream_t)stream;
  const int E = (int)n_experts;
  const int k_hint = jobs_per_x_row > 1 ? jobs_per_x_row : 8;       // the down launch has one job per activation row: assume eight experts per token
  switch (ggml_type) {
    case GGML_Q4_0: return launch_qexperts_t<F_Q4_0P>(a, E, n_jobs, k_hint, s);
    case GGML_Q8_0: return launch_qexperts_t<F_Q8_0P>(a, E, n_jobs, k_hint, s);
    case GGML_MXFP4: return launch_qexperts_t<GGML_MXFP4>(a, E, n_jobs, k_hint, s);
    case GGML_Q6_K: return launch_qexperts_t<GGML_Q6_K>(a, E, n_jobs, k_hint, s);
    case GGML_Q4_K: return launch_qexperts_t<GGML_Q4_K>(a, E, n_jobs, k_hint, s);
    case GGML_Q5_K: return launch_qexperts_t<GGML_Q5_K>(a, E, n_jobs, k_hint, s);
    case GGML_Q4_1: return launch_qexperts_t<GGML_Q4_1>(a, E, n_jobs, k_hint, s);
    case GGML_Q5_0: return launch_qexperts_t<GGML_Q5_0>(a, E, n_jobs, k_hint, s);
    case GGML_Q5_1: return launch_qexperts_t<GGML_Q5_1>(a, E, n_jobs, k_hint, s);
    case GGML_F16: return launch_qexperts_t<GGML_F16>(a, E, n_jobs, k_hint, s);
    case GGML_IQ4_XS: return launch_qexperts_t<GGML_IQ4_XS>(a, E, n_jobs, k_hint, s);
    case GGML_IQ3_XXS: return launch_qexperts_t<GGML_IQ3_XXS>(a, E, n_jobs, k_hint, s);
    case GGML_IQ3_S: return launch_qexperts_t<GGML_IQ3_S>(a, E, n_jobs, k_hint, s);
    case GGML_IQ2_S: return launch_qexperts_t<GGML_IQ2_S>(a, E, n_jobs, k_hint, s);
    case GGML_Q1_0: return launch_qexperts_t<GGML_Q1_0>(a, E, n_jobs, k_hint, s);
  }
  return tga_set_error("tga_qlinear_experts_grouped: no kernel for type %d", ggml_type);
}

}  // extern "C"
