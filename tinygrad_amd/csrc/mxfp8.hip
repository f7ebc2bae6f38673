// MXFP8 MoE prefill path (benchmark configuration 5): E4M3 quantisation with E8M0 per-32 block scales, token-sorted expert grouping
// (route / dispatch / combine) and the grouped GEMM on CDNA4 scaled MFMA.
// Reference: extra/gemm/cdna_asm_gemm.py:149-173 (quantize_mxfp8, mx_pack), extra/gemm/moe_routing.py:89-131 (route, dispatch,
// combine), extra/gemm/moe_gemm.py:112-134 (grouped_mx_gemm; its HIP kernel source is absent from the reference tree).
#include "common.h"
#include "host.h"
#include <string.h>

typedef int v8i32 __attribute__((ext_vector_type(8)));
typedef float v4f32 __attribute__((ext_vector_type(4)));

#define MX_BLOCK_ROW 256

__device__ __forceinline__ float bf16_to_f(uint16_t b) { return __builtin_bit_cast(float, (uint32_t)b << 16); }
__device__ __forceinline__ uint16_t f_to_bf16(float f) {   // round to nearest even (tinygrad/dtype.py:224-226)
  uint32_t u = __builtin_bit_cast(uint32_t, f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);
  return (uint16_t)((u + 0x7FFFu + ((u >> 16) & 1)) >> 16);
}
// float -> E4M3 (fn) bits, RNE, finite saturation (tinygrad/dtype.py:237-260); |x| is already clamped to 448 by the caller
__device__ __forceinline__ uint32_t f_to_e4m3(float x) {
  const uint32_t u = __builtin_bit_cast(uint32_t, x), sign = (u >> 24) & 0x80;
  const float a = fabsf(x);
  if (!(a == a)) return sign | 0x7f;
  if (a >= 464.0f) return sign | 0x7e;
  if (a < 0.0009765625f) return sign;                       // <= 2^-10 (half the smallest subnormal) rounds to zero (ties to even)
  int e; (void)frexpf(a, &e); e -= 1;                       // a = m * 2^e, 1 <= m < 2
  if (e < -6) e = -6;
  const float q = rintf(ldexpf(a, 3 - e));                  // mantissa grid: 8..16 (normal) or 0..8 (subnormal)
  float v = ldexpf(q, e - 3);
  if (v > 448.0f) v = 448.0f;
  int e2; const float m2 = frexpf(v, &e2); e2 -= 1;
  if (v < 0.015625f) return sign | (uint32_t)(v * 512.0f);  // subnormal: v / 2^-9
  return sign | ((uint32_t)(e2 + 7) << 3) | (uint32_t)((m2 * 2.0f - 1.0f) * 8.0f);
}

// ------------------------------------------------------------------------------------------------ quantize_mxfp8
// One thread per 32-element block: amax, e8 = clamp(floor(log2(max(amax, 1e-38))) + 127, 0, 254), q = e4m3(clamp(x * 2^(127-e8), +-448)).
// Also writes the packed scales of mx_pack: packed[k/128][row] = 4 consecutive e8 bytes (little-endian).
// One 32-element block: e8 = clamp(floor(log2(max(amax, 1e-38))) + 127, 0, 254); out = 32 E4M3 bytes of clamp(v * 2^(127 - e8), +-448).
__device__ __forceinline__ int mx_quant32(const float* v, uint32_t* out) {
  float amax = 0.f;
#pragma unroll
  for (int i = 0; i < 32; i++) amax = fmaxf(amax, fabsf(v[i]));
  int ex; (void)frexpf(amax, &ex);                         // floor(log2(a)) = ex - 1
  // below the smallest normal float the reference's max(amax, 1e-38) floor gives floor(log2) = -127 -> e8 = 0
  int e = amax < 1.17549435e-38f ? 0 : ex - 1 + 127; e = e < 0 ? 0 : (e > 254 ? 254 : e);
  const float qs = __builtin_bit_cast(float, (uint32_t)(254 - e) << 23);   // 2^(127 - e), exact for e in 0..253; e = 254 -> 2^-127 below
  const float scale = (e == 254) ? __builtin_bit_cast(float, 0x00400000u) : qs;
#pragma unroll
  for (int i = 0; i < 8; i++) {
    uint32_t w = 0;
#pragma unroll
    for (int j = 0; j < 4; j++) { float s = v[4 * i + j] * scale; s = fminf(fmaxf(s, -448.0f), 448.0f); w |= f_to_e4m3(s) << (8 * j); }
    out[i] = w;
  }
  return e;
}
// MODE 0: x float32; 1: x bf16; 2: fused SwiGLU producer, value = w1 * sigmoid(w1) * w3 in float32 from two bf16 tensors x (= x_w1)
// and x2 (= x_w3), sigmoid as 1 / (1 + exp2(-w1 * log2(e)))  (extra/llama_kernels/fused_silu_mul_quantize_mxfp8/__init__.py:33-36)
template <int MODE>
__global__ __launch_bounds__(256) void quantize_mxfp8_kernel(const void* __restrict__ x, const void* __restrict__ x2, long long rows, int K, uint8_t* __restrict__ q,
                                                             uint8_t* __restrict__ e8, uint8_t* __restrict__ packed) {
  const long long nb = rows * (K / 32);
  for (long long b = (long long)blockIdx.x * 256 + threadIdx.x; b < nb; b += (long long)gridDim.x * 256) {
    const long long row = b / (K / 32); const int kb = (int)(b % (K / 32));
    float v[32];
    auto load_bf16 = [&](const void* src, float* o) {
      const u32x4* p = (const u32x4*)((const uint16_t*)src + row * K + kb * 32);
#pragma unroll
      for (int i = 0; i < 4; i++) { const u32x4 w = p[i];
        o[8*i] = bf16_to_f(w.x & 0xFFFF); o[8*i+1] = bf16_to_f(w.x >> 16); o[8*i+2] = bf16_to_f(w.y & 0xFFFF); o[8*i+3] = bf16_to_f(w.y >> 16);
        o[8*i+4] = bf16_to_f(w.z & 0xFFFF); o[8*i+5] = bf16_to_f(w.z >> 16); o[8*i+6] = bf16_to_f(w.w & 0xFFFF); o[8*i+7] = bf16_to_f(w.w >> 16); }
    };
    if constexpr (MODE == 1) load_bf16(x, v);
    else if constexpr (MODE == 2) {
      float u[32];
      load_bf16(x, v); load_bf16(x2, u);
#pragma unroll
      for (int i = 0; i < 32; i++) { const float sig = 1.0f / (1.0f + exp2f(v[i] * -1.4426950408889634f)); v[i] = v[i] * sig * u[i]; }
    } else {
      const f32x4* p = (const f32x4*)((const float*)x + row * K + kb * 32);
#pragma unroll
      for (int i = 0; i < 8; i++) { const f32x4 w = p[i]; v[4*i] = w.x; v[4*i+1] = w.y; v[4*i+2] = w.z; v[4*i+3] = w.w; }
    }
    uint32_t out[8];
    const int e = mx_quant32(v, out);
    u32x4* qo = (u32x4*)(q + row * K + kb * 32);
    qo[0] = u32x4{out[0], out[1], out[2], out[3]}; qo[1] = u32x4{out[4], out[5], out[6], out[7]};
    e8[row * (K / 32) + kb] = (uint8_t)e;
    if (packed) packed[((long long)(kb >> 2) * rows + row) * 4 + (kb & 3)] = (uint8_t)e;
  }
}

// transpose_quantize_mxfp8 (extra/llama_kernels/transpose_quantize_mxfp8/__init__.py:24-37) == quantize_mxfp8(g.T) without the transposed
// tensor: g (M, N) bf16 -> q (N, M), e8 (N, M / 32), packed (M / 128, N).  One workgroup takes 128 rows x 64 columns of g through LDS
// (row-wise 16-byte loads, column-wise reads), thread (column c, 32-row run r) quantizes one block, and the four runs of a column fill one
// 128-byte line of q.
__global__ __launch_bounds__(256) void transpose_quantize_mxfp8_kernel(const uint16_t* __restrict__ g, int M, int N, uint8_t* __restrict__ q,
                                                                       uint8_t* __restrict__ e8, uint8_t* __restrict__ packed) {
  __shared__ uint16_t tile[128][64 + 8];                    // 144-byte rows: 16-byte aligned, column reads of a wave hit 32 different banks
  const int n0 = blockIdx.x * 64, m0 = blockIdx.y * 128, t = threadIdx.x;
#pragma unroll
  for (int p = 0; p < 4; p++) {
    const int r = p * 32 + (t >> 3), c8 = (t & 7) * 8;
    u32x4 w = {0, 0, 0, 0};
    if (m0 + r < M) w = *(const u32x4*)(g + (size_t)(m0 + r) * N + n0 + c8);
    *(u32x4*)&tile[r][c8] = w;
  }
  __syncthreads();
  const int c = t & 63, run = t >> 6;
  if (m0 + run * 32 >= M) return;
  float v[32];
#pragma unroll
  for (int i = 0; i < 32; i++) v[i] = bf16_to_f(tile[run * 32 + i][c]);
  uint32_t out[8];
  const int e = mx_quant32(v, out);
  const int kb = (m0 >> 5) + run;
  u32x4* qo = (u32x4*)(q + (size_t)(n0 + c) * M + m0 + run * 32);
  qo[0] = u32x4{out[0], out[1], out[2], out[3]}; qo[1] = u32x4{out[4], out[5], out[6], out[7]};
  e8[(size_t)(n0 + c) * (M / 32) + kb] = (uint8_t)e;
  if (packed) packed[((size_t)(kb >> 2) * N + n0 + c) * 4 + (kb & 3)] = (uint8_t)e;
}

// ------------------------------------------------------------------------------------------------ route
// (1) top-k + softmax per token: one wave per token.  Tensor.topk order: descending value, the lower index first among equals.
__global__ __launch_bounds__(64) void route_topk_kernel(const float* __restrict__ logits, int E, int k, int* __restrict__ topi, float* __restrict__ weights) {
  const int t = blockIdx.x, lane = threadIdx.x;
  extern __shared__ float sl[];
  for (int i = lane; i < E; i += 64) sl[i] = logits[(size_t)t * E + i];
  __syncthreads();
  __shared__ float tv[64]; __shared__ int ti[64];
  for (int s = 0; s < k; s++) {
    float best = -INFINITY; int bi = 0x7fffffff;
    for (int i = lane; i < E; i += 64) { const float v = sl[i]; if (v > best || (v == best && i < bi)) { best = v; bi = i; } }
    for (int o = 32; o > 0; o >>= 1) {
      const float ov = __shfl_xor(best, o, 64); const int oi = __shfl_xor(bi, o, 64);
      if (ov > best || (ov == best && oi < bi)) { best = ov; bi = oi; }
    }
    if (lane == 0) { tv[s] = best; ti[s] = bi; sl[bi] = -INFINITY; }
    __syncthreads();
  }
  if (lane < k) {
    const float m = tv[0];
    float z = 0.f; for (int j = 0; j < k; j++) z += expf(tv[j] - m);
    weights[(size_t)t * k + lane] = expf(tv[lane] - m) * (1.0f / z);
    topi[(size_t)t * k + lane] = ti[lane];
  }
}
// (2) per 1024-assignment chunk: stable rank of every assignment among those of the same expert inside the chunk + per-expert counts
__global__ __launch_bounds__(256) void route_rank_kernel(const int* __restrict__ topi, int n_assign, int E, int* __restrict__ local_rank, int* __restrict__ chunk_cnt) {
  __shared__ int ids[1024]; __shared__ int rk[1024];
  const int c0 = blockIdx.x * 1024, n = min(1024, n_assign - c0);
  for (int i = threadIdx.x; i < n; i += 256) ids[i] = topi[c0 + i];
  __syncthreads();
  for (int e = threadIdx.x; e < E; e += 256) {
    int cnt = 0;
    for (int j = 0; j < n; j++) if (ids[j] == e) rk[j] = cnt++;
    chunk_cnt[(size_t)blockIdx.x * E + e] = cnt;
  }
  __syncthreads();
  for (int i = threadIdx.x; i < n; i += 256) local_rank[c0 + i] = rk[i];
}
// (3) per expert: total count, pad to 256, offsets (exclusive scan over experts) and per-chunk bases (exclusive scan over chunks)
__global__ __launch_bounds__(256) void route_offsets_kernel(int* __restrict__ chunk_cnt, int nchunks, int E, int* __restrict__ off, int* __restrict__ counts) {
  extern __shared__ int tot[];
  for (int e = threadIdx.x; e < E; e += 256) {
    int run = 0;
    for (int c = 0; c < nchunks; c++) { const int v = chunk_cnt[(size_t)c * E + e]; chunk_cnt[(size_t)c * E + e] = run; run += v; }
    tot[e] = run; counts[e] = run;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int o = 0; off[0] = 0;
    for (int e = 0; e < E; e++) { o += (tot[e] + MX_BLOCK_ROW - 1) / MX_BLOCK_ROW * MX_BLOCK_ROW; off[e + 1] = o; }
  }
}
// (4) dest_row[j] = off[e_j] + base[chunk(j)][e_j] + local_rank[j]
__global__ __launch_bounds__(256) void route_dest_kernel(const int* __restrict__ topi, const int* __restrict__ local_rank, const int* __restrict__ chunk_base,
                                                         const int* __restrict__ off, int n_assign, int E, int* __restrict__ dest_row) {
  const int j = blockIdx.x * 256 + threadIdx.x;
  if (j >= n_assign) return;
  const int e = topi[j];
  dest_row[j] = off[e] + chunk_base[(size_t)(j >> 10) * E + e] + local_rank[j];
}

// ------------------------------------------------------------------------------------------------ dispatch / combine
// xg[dest_row[j], :] = x[j / k, :]; padding rows (between an expert's count and its 256-padded end, and after off[E]) are zeroed.
__global__ __launch_bounds__(256) void dispatch_kernel(const uint16_t* __restrict__ x, const int* __restrict__ dest_row, int k, int D, uint16_t* __restrict__ xg) {
  const int j = blockIdx.x;
  const u32x4* src = (const u32x4*)(x + (size_t)(j / k) * D);
  u32x4* dst = (u32x4*)(xg + (size_t)dest_row[j] * D);
  for (int i = threadIdx.x; i < D / 8; i += 256) dst[i] = src[i];
}
__global__ __launch_bounds__(256) void dispatch_zero_pad_kernel(const int* __restrict__ off, const int* __restrict__ counts, int E, int m_l, int D, uint16_t* __restrict__ xg) {
  // blockIdx.x = padded row index within the whole buffer; each block decides whether its row is padding
  const int row = blockIdx.x;
  int e = 0;
  if (row >= off[E]) e = -1;
  else { int lo = 0, hi = E; while (hi - lo > 1) { const int mid = (lo + hi) >> 1; if (off[mid] <= row) lo = mid; else hi = mid; } e = lo; }
  if (e >= 0 && row < off[e] + counts[e]) return;
  u32x4* dst = (u32x4*)(xg + (size_t)row * D);
  for (int i = threadIdx.x; i < D / 8; i += 256) dst[i] = u32x4{0, 0, 0, 0};
}
// out[t, :] = sum_s bf16(weights[t, s]) * z[dest_row[t*k + s], :]: bf16 products, float32 accumulation, bf16 result
__global__ __launch_bounds__(256) void combine_kernel(const uint16_t* __restrict__ z, const int* __restrict__ dest_row, const float* __restrict__ weights,
                                                      int k, int D, uint16_t* __restrict__ out) {
  const int t = blockIdx.x;
  for (int d = threadIdx.x; d < D; d += 256) {
    float acc = 0.f;
    for (int s = 0; s < k; s++) {
      const float w = bf16_to_f(f_to_bf16(weights[(size_t)t * k + s]));
      acc += bf16_to_f(f_to_bf16(bf16_to_f(z[(size_t)dest_row[(size_t)t * k + s] * D + d]) * w));
    }
    out[(size_t)t * D + d] = f_to_bf16(acc);
  }
}

// ------------------------------------------------------------------------------------------------ grouped MXFP8 GEMM
// C[r, :] = deq(A[r, :]) . deq(B[e(r)])^T, float32 accumulate, bf16 store; e(r) = expert owning the 256-row tile of r
// (Routing.rows_e, moe_routing.py:98-104: the last expert whose offset is <= the tile's first row, so the tiles at or beyond
// expert_off[E] belong to expert E - 1).  A (M, K) e4m3 row-major; B (E, N, K) e4m3; scales E8M0 per 32 along K.
// Operand layout of v_mfma_scale_f32_16x16x128_f8f6f4 as measured on MI355X: lane l = 16 g + r supplies row (A) / column (B) r; its 32
// operand bytes are K = 16 g + 0..15 followed by K = 64 + 16 g + 0..15 of the 128-wide K step; byte 0 of its scale register (op_sel 0)
// is the E8M0 scale of the 32-block K = 32 g .. 32 g + 31 of row / column r (so a lane's scale does NOT belong to the lane's
// own bytes); the 16 x 16 result has column l % 16 and rows 4 * (l / 16) + 0..3 in the lane's 4 accumulator registers.
struct GemmArgs {
  uint16_t* C; const uint8_t* A; const uint8_t* B; const uint8_t* a_e8; const uint8_t* b_e8; const int* off;
  int M, N, K, E;
  int routed_only;          // != 0: tiles at or beyond expert_off[E] are skipped (their rows of C keep their contents)
  const int* counts;        // optional: routed rows per expert; rows of an expert's range at or beyond its count are padding - not multiplied, written as zeros
};

// ---- LDS-tiled variant: 256 x 256 output tile per workgroup, 8 waves as 2 (M) x 4 (N), each 128 x 64 = 8 x 4 MFMAs per K step of
// 128, two LDS stages of 64 KB (two waves per SIMD: one multiplies while the other waits on LDS).  A 16-row x 128-byte operand
// sub-tile lives in LDS in the order the MFMA consumes it: plane p (the lane's first / second 16 bytes), slot 16g + r <- row r,
// bytes [64p + 16g, 64p + 16g + 16), with the slot's low three bits XORed by (g + 4p): the 8 threads that copy one row's 128
// bytes then hit 8 different 16-byte bank groups, and so do the 8 consecutive lanes of every ds_read_b128.  While step s is
// multiplied, the global loads of step s + 1 (8 x 16 bytes + one scale dword per thread) are in flight (a scheduling barrier
// keeps them ahead of the MFMAs); they are written to the other stage after the MFMAs, one workgroup barrier per step.
// Operands are swapped in the MFMA (weights as A, activations as B), so a lane ends up with four consecutive output columns
// of one row: 8-byte bf16 stores.
#define GG_TILE 256
#define GG_THREADS 512
#define GG_STAGE_BYTES (2 * GG_TILE * 128 + 2 * GG_TILE * 4)   // operand tiles + one scale dword per row
__device__ __forceinline__ int gg_slot_off(int R, int c) {       // byte offset inside a 256-row operand region of (row R, 16-byte chunk c)
  const int sub = R >> 4, r = R & 15, p = c >> 2, g = c & 3;
  return sub * 2048 + p * 1024 + ((16 * g + (r ^ (g + 4 * p))) << 4);
}

// Which tile workgroup b computes.  Consecutive workgroups go to different XCDs (the dispatcher deals them round-robin), so XCD x = b % 8
// gets a contiguous run of the routed tiles: the N tiles of one row block (which share the activation tile) and the row blocks of one
// expert (which share the weight tile) meet in one L2.  The routed tiles (rows below expert_off[E]) are shared evenly; the workgroups an
// XCD has left take the tiles beyond, in order.  A bijection from [0, gridDim.x) onto the (M / 256) (N / 256) tiles for any grid size.
__device__ __forceinline__ int gg_tile_of_workgroup(int b, int nwg, int nact, bool& routed) {
  const int x = b & 7, j = b >> 3;
  const int cnt_a = nact / 8 + (x < nact % 8), start_a = x * (nact / 8) + min(x, nact % 8);
  routed = j < cnt_a;
  if (routed) return start_a + j;
  const int start_g = x * (nwg / 8) + min(x, nwg % 8);
  return nact + (start_g - start_a) + (j - cnt_a);
}

// A workgroup walks the tiles b, b + gridDim.x, ... of the map above (the C-ABI launch starts one workgroup per CU; a launch with one
// workgroup per tile, as a PROGRAM bound through Tensor.custom_kernel makes, runs the same code with one trip).  Measured per tile with
// wall-clock stamps before this loop existed (config 5 gate/up, 16 K steps): 3.6 us until the first stage is in LDS, 36.5 us in the K loop,
// 6.2 us in the epilogue (manual bf16 rounding, 8-byte stores in 32-byte runs) and 1.1-1.8 us until the CU has its next workgroup.  Here
//   * the landing registers, which the last K step used to fill with a reload that was dropped, receive the FIRST step of the workgroup's next
//     tile, so the next tile starts with its operands already in LDS;
//   * the expert offsets sit in LDS (one read of the table per workgroup, binary search without memory round trips);
//   * the epilogue rounds with v_cvt_pk_bf16_f32 and turns the accumulators through the idle LDS stage (wave-private 32-row slabs), so that a
//     store instruction writes eight whole 128-byte row segments.
#define GG_OFF_MAX 4096                                           // expert offsets 0 .. E kept in LDS when E < GG_OFF_MAX
#define GG_EPI_PITCH 144                                          // bytes per 64-column bf16 row in the epilogue slab (128 + 16: conflict-free 8-byte writes)
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {          // round to nearest even (tinygrad/dtype.py:224-226); one v_cvt_pk_bf16_f32
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2_t{lo, hi}, bf16x2_t));
}
struct GGCur { const uint8_t* A; const uint8_t* B; const uint8_t* sc; int row0, tn, valid; };   // valid: rows of the tile that are not padding   // scalar (wave-uniform) state of one tile

__device__ __forceinline__ void grouped_mxfp8_gemm_tile(const GemmArgs& g, uint8_t* smem, int* s_off) {
  const int tiles_n = g.N / GG_TILE, tiles_total = (g.M / GG_TILE) * tiles_n;
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 2, wn = wave & 3;
  const int r16 = lane & 15, kg = lane >> 4;
  const int KB = g.K / 32, nsteps = g.K / 128;
  const bool off_in_lds = g.E < GG_OFF_MAX;
  if (off_in_lds) for (int i = tid; i <= g.E; i += GG_THREADS) s_off[i] = g.off[i];
  const int off_end = min(max(g.off[g.E], 0), g.M);             // an offset table that overruns the matrix is clamped to it
  const int nact = (off_end / GG_TILE) * tiles_n;              // routed row blocks x column blocks
  __syncthreads();
  // first virtual workgroup index >= b (in steps of the grid size) that has a tile to compute, or -1
  auto find_tile = [&](int b, int& tile) {
    for (; b < tiles_total; b += (int)gridDim.x) {
      bool routed;
      const int t = gg_tile_of_workgroup(b, tiles_total, nact, routed);
      if (t < tiles_total && (routed || !g.routed_only)) { tile = t; return b; }
    }
    return -1;
  };
  auto setup = [&](int tile, GGCur& c) {
    const int tm = tile / tiles_n;
    c.tn = tile % tiles_n; c.row0 = tm * GG_TILE;
    int lo = 0, hi = g.E;                                       // the last expert whose offset is <= the tile's first row
    while (hi - lo > 1) {
      const int mid = (lo + hi) >> 1;
      const int v = off_in_lds ? __builtin_amdgcn_readfirstlane(s_off[mid]) : g.off[mid];
      if (v <= c.row0) lo = mid; else hi = mid;
    }
    c.valid = GG_TILE;
    if (g.counts && c.row0 < off_end) {                         // (tiles beyond the routed range have no count: all of their rows are multiplied)
      const int first = off_in_lds ? __builtin_amdgcn_readfirstlane(s_off[lo]) : g.off[lo];
      c.valid = min(max(first + g.counts[lo] - c.row0, 0), GG_TILE);
    }
    const size_t wrow = (size_t)lo * g.N + (size_t)c.tn * GG_TILE;
    c.A = g.A + (size_t)c.row0 * g.K;
    c.B = g.B + wrow * g.K;
    // scale dwords (the four E8M0 bytes of K blocks 4s .. 4s+3 of one row) travel through LDS too: thread t < 256 copies activation
    // row t's, thread t >= 256 weight row t - 256's; lane (g, r) of sub-tile i then takes byte g of row 16 i + r
    c.sc = wave < 4 ? g.a_e8 + (size_t)c.row0 * KB : g.b_e8 + wrow * KB;
  };
  // this thread's 4 + 4 chunks per step: rows cpy_r + 64 j, 16-byte piece cpy_c (a 32-bit offset from the tile's scalar base)
  const int cpy_c = tid & 7, cpy_r = tid >> 3;
  int cpy_off[4];
#pragma unroll
  for (int j = 0; j < 4; j++) cpy_off[j] = gg_slot_off(cpy_r + 64 * j, cpy_c);
  const uint32_t cpy_voff = (uint32_t)cpy_r * (uint32_t)g.K + (uint32_t)cpy_c * 16u;
  const uint32_t sc_voff = (uint32_t)(tid & (GG_TILE - 1)) * (uint32_t)KB;
  const size_t rows64 = (size_t)64 * g.K;
  // fragment read offsets of this lane inside a sub-tile (plane 0 / plane 1)
  const int f0 = ((16 * kg + (r16 ^ kg)) << 4), f1 = 1024 + ((16 * kg + (r16 ^ (kg + 4))) << 4);

  u32x4 stg_a[4], stg_b[4]; uint32_t stg_sc;
  // one of the nine loads of a step: 2 j = activation rows cpy_r + 64 j, 2 j + 1 = weight rows, 8 = the scale dword
  auto load_piece = [&](const GGCur& c, int s, int which) {
    const size_t ks = (size_t)s * 128;
    if (which == 8) stg_sc = *(const uint32_t*)(c.sc + 4 * s + sc_voff);
    else if (which & 1) stg_b[which >> 1] = *(const u32x4*)(c.B + ks + (which >> 1) * rows64 + cpy_voff);
    else stg_a[which >> 1] = *(const u32x4*)(c.A + ks + (which >> 1) * rows64 + cpy_voff);
  };
  auto load_step = [&](const GGCur& c, int s) {
#pragma unroll
    for (int w = 0; w < 9; w++) load_piece(c, s, w);
  };
  auto store_piece = [&](int stage, int which) {
    uint8_t* base = smem + stage * GG_STAGE_BYTES;
    if (which == 8) ((uint32_t*)(base + 2 * GG_TILE * 128))[tid] = stg_sc;
    else if (which & 1) *(u32x4*)(base + GG_TILE * 128 + cpy_off[which >> 1]) = stg_b[which >> 1];
    else *(u32x4*)(base + cpy_off[which >> 1]) = stg_a[which >> 1];
  };
  auto store_step = [&](int stage) {
#pragma unroll
    for (int w = 0; w < 9; w++) store_piece(stage, w);
  };

  int tile;
  int b = find_tile((int)blockIdx.x, tile);
  if (b < 0) return;
  GGCur cur;
  setup(tile, cur);
  load_step(cur, 0);
  store_step(0);
  __syncthreads();
  int par = 0;                                                   // LDS stage of the current tile's step 0
  while (true) {
    int tile_n;
    const int bn = find_tile(b + (int)gridDim.x, tile_n);
    GGCur nxt = cur;
    if (bn >= 0) setup(tile_n, nxt);
    const int nxt_step = bn >= 0 ? 0 : nsteps - 1;             // no further tile: the last step reloads itself (dropped)

    v4f32 acc[8][4];                                            // [m sub-tile][n sub-tile]
#pragma unroll
    for (int i = 0; i < 8; i++)
#pragma unroll
      for (int j = 0; j < 4; j++) acc[i][j] = v4f32{0.f, 0.f, 0.f, 0.f};

    // 16-row sub-tiles of this wave that hold routed rows (8 without counts); the others keep their zero accumulators
    const int nsub = min(max((cur.valid - wm * 128 + 15) >> 4, 0), 8);
    for (int s = 0; s < nsteps; s++) {
      const bool lastk = s + 1 == nsteps;
      GGCur src = cur;
      if (lastk) src = nxt;
      // The loads of the next step (of this tile, or the first step of the next tile) are issued one per sub-tile, between the MFMA groups: a
      // CU takes 24-38 cycles to accept a 64 x 16-byte load, so the 72 loads of a step issued together held the last wave back by 1.1 us
      // before it could start multiplying (measured with wall-clock stamps per phase), and the barrier passed that on to every wave.
      const int ls = lastk ? nxt_step : s + 1;
      load_piece(src, ls, 8);
      const uint8_t* base = smem + ((par + s) & 1) * GG_STAGE_BYTES;
      const uint8_t* As = base + wm * 8 * 2048;
      const uint8_t* Bs = base + GG_TILE * 128 + wn * 4 * 2048;
      const uint32_t* sA = (const uint32_t*)(base + 2 * GG_TILE * 128) + wm * 128 + r16;
      const uint32_t* sB = (const uint32_t*)(base + 2 * GG_TILE * 128) + GG_TILE + wn * 64 + r16;
      v8i32 bf[4]; int sb[4];
      if (nsub > 0)
#pragma unroll
      for (int j = 0; j < 4; j++) {
        const u32x4 y0 = *(const u32x4*)(Bs + j * 2048 + f0), y1 = *(const u32x4*)(Bs + j * 2048 + f1);
        bf[j] = v8i32{(int)y0.x, (int)y0.y, (int)y0.z, (int)y0.w, (int)y1.x, (int)y1.y, (int)y1.z, (int)y1.w};
        sb[j] = (int)(sB[16 * j] >> (8 * kg));
      }
      // the activation fragment of sub-tile i + 1 is requested before the MFMAs of sub-tile i are issued: they run while it arrives
      auto frag = [&](int i, v8i32& af, int& sa) {
        const u32x4 x0 = *(const u32x4*)(As + i * 2048 + f0), x1 = *(const u32x4*)(As + i * 2048 + f1);
        af = v8i32{(int)x0.x, (int)x0.y, (int)x0.z, (int)x0.w, (int)x1.x, (int)x1.y, (int)x1.z, (int)x1.w};
        sa = (int)sA[16 * i];
      };
      v8i32 af[2]; int sa[2];
      if (nsub > 0) frag(0, af[0], sa[0]);
#pragma unroll
      for (int i = 0; i < 8; i++) {
        if (i + 1 < nsub) frag(i + 1, af[(i + 1) & 1], sa[(i + 1) & 1]);
        if (i < 4) { load_piece(src, ls, 2 * i); load_piece(src, ls, 2 * i + 1); }
        __builtin_amdgcn_sched_barrier(0);
        if (i < nsub) {                                         // (a branch around LDS reads and MFMAs only: the global loads stay unconditional)
          const int sai = sa[i & 1] >> (8 * kg);
#pragma unroll
          for (int j = 0; j < 4; j++)
            acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(bf[j], af[i & 1], acc[i][j], 0, 0, 0, sb[j], 0, sai);
        }
        __builtin_amdgcn_sched_barrier(0);
        // the other stage was last read one step ago: the landed pieces go there while the second half of the MFMAs runs
        if (i >= 4) { store_piece((par + s + 1) & 1, 2 * (i - 4)); store_piece((par + s + 1) & 1, 2 * (i - 4) + 1); __builtin_amdgcn_sched_barrier(0); }
      }
      __builtin_amdgcn_sched_barrier(0);
      store_piece((par + s + 1) & 1, 8);
      __syncthreads();
    }
    // ---- epilogue.  The stage the last step was read from is idle now (the other one already holds the next tile's first step).  A lane holds
    // output row (activation row) r16 of m sub-tile i, columns 4 kg .. 4 kg + 3 of n sub-tile j; 32 rows at a time go through the wave's slab.
    {
      uint8_t* slab = smem + ((par + nsteps - 1) & 1) * GG_STAGE_BYTES + wave * (32 * GG_EPI_PITCH);
      uint16_t* cw = g.C + (size_t)(cur.row0 + wm * 128) * g.N + (size_t)cur.tn * GG_TILE + wn * 64;
      const int rrow = lane >> 3, rc = lane & 7;
#pragma unroll
      for (int q = 0; q < 4; q++) {
#pragma unroll
        for (int ii = 0; ii < 2; ii++)
#pragma unroll
          for (int j = 0; j < 4; j++) {
            const v4f32 v = acc[2 * q + ii][j];
            *(u32x2*)(slab + (16 * ii + r16) * GG_EPI_PITCH + 32 * j + 8 * kg) = u32x2{pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
          }
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");    // LDS operations of a wave execute in order: ordering for the compiler only
        u32x4 o[4];
#pragma unroll
        for (int p2 = 0; p2 < 4; p2++) o[p2] = *(const u32x4*)(slab + (rrow + 8 * p2) * GG_EPI_PITCH + 16 * rc);
#pragma unroll
        for (int p2 = 0; p2 < 4; p2++) *(u32x4*)(cw + (size_t)(32 * q + rrow + 8 * p2) * g.N + 8 * rc) = o[p2];
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
      }
    }
    if (bn < 0) break;
    __syncthreads();                                             // the slabs are free before any wave's next step writes that stage
    par = (par + nsteps) & 1; cur = nxt; b = bn;
  }
}

// C-ABI launch: arguments in one by-value record.
__global__ __launch_bounds__(GG_THREADS) void grouped_mxfp8_gemm_lds_kernel(const GemmArgs g) {
  __shared__ __attribute__((aligned(16))) uint8_t smem[2 * GG_STAGE_BYTES];   // [stage][A 32 KB | B 32 KB | 512 scale dwords]
  __shared__ int s_off[GG_OFF_MAX];
  grouped_mxfp8_gemm_tile(g, smem, s_off);
}

// The same kernel with the argument list a pre-compiled PROGRAM bound through Tensor.custom_kernel hands over: one pointer per buffer in
// the order of the sink's sources (extra/gemm/moe_gemm.py:36-48: C, A, B, x_si, w_si, x_e8, w_e8, expert_off), then the scalar
// variables (tinygrad/uop/ops.py:1194-1198).  Launch: 512 threads x (M / 256) (N / 256) workgroups, no dynamic LDS (the reference's HIP
// runtime passes 0 shared bytes, tinygrad/runtime/ops_hip.py:44-47), so the two 66 KB stages are static.  x_si / w_si are not read.
extern "C" __global__ __launch_bounds__(GG_THREADS) void tga_grouped_mxfp8_gemm_kernel(uint16_t* C, const uint8_t* A, const uint8_t* B, const uint32_t* x_si,
                                                                                        const uint32_t* w_si, const uint8_t* x_e8, const uint8_t* w_e8,
                                                                                        const int* expert_off, int M, int N, int K, int E) {
  __shared__ __attribute__((aligned(16))) uint8_t smem[2 * GG_STAGE_BYTES];
  __shared__ int s_off[GG_OFF_MAX];
  (void)x_si; (void)w_si;
  GemmArgs g; g.C = C; g.A = A; g.B = B; g.a_e8 = x_e8; g.b_e8 = w_e8; g.off = expert_off; g.M = M; g.N = N; g.K = K; g.E = E; g.routed_only = 0; g.counts = nullptr;
  grouped_mxfp8_gemm_tile(g, smem, s_off);
}

// clamped, interleaved SwiGLU between the two grouped GEMMs (examples/mlperf/models/gpt_oss.py:94-98): bf16 in/out
__global__ __launch_bounds__(256) void swiglu_interleaved_kernel(const uint16_t* __restrict__ h, long long rows, int two_inter, float limit, float alpha, uint16_t* __restrict__ y) {
  const int inter = two_inter / 2;
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < rows * inter; i += (long long)gridDim.x * 256) {
    const long long r = i / inter; const int c = (int)(i % inter);
    float glu = bf16_to_f(h[r * two_inter + 2 * c]), lin = bf16_to_f(h[r * two_inter + 2 * c + 1]);
    glu = fminf(glu, limit); lin = fminf(fmaxf(lin, -limit), limit);
    // bf16 elementwise chain like the reference's bf16 tensors: each op rounds to bf16
    const float sg = bf16_to_f(f_to_bf16(1.0f / (1.0f + expf(-bf16_to_f(f_to_bf16(alpha * glu))))));
    const float a = bf16_to_f(f_to_bf16(glu * sg)), b = bf16_to_f(f_to_bf16(lin + 1.0f));
    y[r * inter + c] = f_to_bf16(a * b);
  }
}

// h[r, :] += bias[e(r), :] for the rows of every expert (examples/mlperf/models/gpt_oss.py:219-224: `+ (onehot @ bias.float()).cast(bf16)`
// after each grouped GEMM): the bias row is cast to bf16 first and the sum of the two bf16 values is rounded to bf16, as the reference's
// bf16 tensor add does.  Rows are located by 256-row tile (Routing.rows_e, moe_routing.py:98-104: the last expert whose offset is <= the tile's
// first row, so the tiles at or beyond off[E] get the last expert's bias).
__global__ __launch_bounds__(256) void add_expert_bias_kernel(uint16_t* __restrict__ h, const float* __restrict__ bias, const int* __restrict__ off, int n_experts, int N) {
  const int tile = blockIdx.y, row0 = tile * 256;
  int lo = 0, hi = n_experts;
  while (hi - lo > 1) { const int mid = (lo + hi) >> 1; if (off[mid] <= row0) lo = mid; else hi = mid; }
  const float* b = bias + (size_t)lo * N;
  for (int c = blockIdx.x * 256 + threadIdx.x; c < N; c += gridDim.x * 256) {
    const float bv = bf16_to_f(f_to_bf16(b[c]));
    for (int r = 0; r < 256; r++) { uint16_t* p = h + (size_t)(row0 + r) * N + c; *p = f_to_bf16(bf16_to_f(*p) + bv); }
  }
}

extern "C" {

int tga_quantize_mxfp8(const void* x, int x_is_bf16, int64_t rows, int64_t K, void* q, void* e8, void* packed, void* stream) {
  TGA_REQUIRE(x && q && e8, "tga_quantize_mxfp8: null pointer");
  TGA_REQUIRE(rows >= 0 && K > 0 && K % 32 == 0, "tga_quantize_mxfp8: K=%lld must be a positive multiple of 32", (long long)K);
  TGA_REQUIRE(!packed || K % 128 == 0, "tga_quantize_mxfp8: packed scales need K %% 128 == 0");
  if (rows == 0) return 0;
  const long long nb = rows * (K / 32);
  const int grid = (int)((nb + 255) / 256 < 65536 ? (nb + 255) / 256 : 65536);
  if (x_is_bf16) quantize_mxfp8_kernel<1><<<grid, 256, 0, (hipStream_t)stream>>>(x, nullptr, rows, (int)K, (uint8_t*)q, (uint8_t*)e8, (uint8_t*)packed);
  else quantize_mxfp8_kernel<0><<<grid, 256, 0, (hipStream_t)stream>>>(x, nullptr, rows, (int)K, (uint8_t*)q, (uint8_t*)e8, (uint8_t*)packed);
  TGA_LAUNCH_CHECK();
  return 0;
}

int tga_silu_mul_quantize_mxfp8(const void* x_w1_bf16, const void* x_w3_bf16, int64_t rows, int64_t K, void* q, void* e8, void* packed, void* stream) {
  TGA_REQUIRE(x_w1_bf16 && x_w3_bf16 && q && e8, "tga_silu_mul_quantize_mxfp8: null pointer");
  TGA_REQUIRE(rows >= 0 && K > 0 && K % 32 == 0, "tga_silu_mul_quantize_mxfp8: K=%lld must be a positive multiple of 32", (long long)K);
  TGA_REQUIRE(!packed || K % 128 == 0, "tga_silu_mul_quantize_mxfp8: packed scales need K %% 128 == 0");
  if (rows == 0) return 0;
  const long long nb = rows * (K / 32);
  const int grid = (int)((nb + 255) / 256 < 65536 ? (nb + 255) / 256 : 65536);
  quantize_mxfp8_kernel<2><<<grid, 256, 0, (hipStream_t)stream>>>(x_w1_bf16, x_w3_bf16, rows, (int)K, (uint8_t*)q, (uint8_t*)e8, (uint8_t*)packed);
  TGA_LAUNCH_CHECK();
  return 0;
}

int tga_transpose_quantize_mxfp8(const void* g_bf16, int64_t M, int64_t N, void* q, void* e8, void* packed, void* stream) {
  TGA_REQUIRE(g_bf16 && q && e8, "tga_transpose_quantize_mxfp8: null pointer");
  TGA_REQUIRE(M > 0 && N > 0 && M % 32 == 0 && N % 64 == 0, "tga_transpose_quantize_mxfp8: M=%lld must be a multiple of 32 and N=%lld of 64", (long long)M, (long long)N);
  TGA_REQUIRE(!packed || M % 128 == 0, "tga_transpose_quantize_mxfp8: packed scales need M %% 128 == 0");
  TGA_REQUIRE(M < (1ll << 31) && N < (1ll << 31) && (M + 127) / 128 <= 65535, "tga_transpose_quantize_mxfp8: matrix too large");
  transpose_quantize_mxfp8_kernel<<<dim3((unsigned)(N / 64), (unsigned)((M + 127) / 128)), 256, 0, (hipStream_t)stream>>>((const uint16_t*)g_bf16, (int)M, (int)N, (uint8_t*)q, (uint8_t*)e8,
                                                                                                                        (uint8_t*)packed);
  TGA_LAUNCH_CHECK();
  return 0;
}

static int moe_route_launch(const char* who, const float* logits, int n_tokens, int n_experts, int k, float* weights, int32_t* topi, int32_t* dest_row, int32_t* off,
                            int32_t* counts, int32_t* scratch, hipStream_t s) {
  TGA_REQUIRE(logits && weights && topi && dest_row && off && counts && scratch, "%s: null pointer", who);
  TGA_REQUIRE(n_tokens >= 1 && n_experts >= 1 && n_experts <= 8192 && k >= 1 && k <= 64 && k <= n_experts, "%s: bad geometry", who);
  const int n_assign = n_tokens * k, nchunks = (n_assign + 1023) / 1024;
  int* local_rank = scratch; int* chunk_cnt = scratch + n_assign;          // both are written in full before they are read: nothing has to start at zero
  route_topk_kernel<<<n_tokens, 64, n_experts * sizeof(float), s>>>(logits, n_experts, k, topi, weights);
  TGA_LAUNCH_CHECK();
  route_rank_kernel<<<nchunks, 256, 0, s>>>(topi, n_assign, n_experts, local_rank, chunk_cnt);
  TGA_LAUNCH_CHECK();
  route_offsets_kernel<<<1, 256, n_experts * sizeof(int), s>>>(chunk_cnt, nchunks, n_experts, off, counts);
  TGA_LAUNCH_CHECK();
  route_dest_kernel<<<(n_assign + 255) / 256, 256, 0, s>>>(topi, local_rank, chunk_cnt, off, n_assign, n_experts, dest_row);
  TGA_LAUNCH_CHECK();
  return 0;
}

int tga_moe_route(const float* logits, int n_tokens, int n_experts, int k, float* weights, int32_t* topi, int32_t* dest_row, int32_t* off,
                  int32_t* counts, int32_t* scratch, void* stream) {
  return moe_route_launch("tga_moe_route", logits, n_tokens, n_experts, k, weights, topi, dest_row, off, counts, scratch, (hipStream_t)stream);
}

// ---- tga_moe_route for callers that cannot allocate: its workspace (the per-assignment ranks and the per-chunk expert counts) is this
// file-scope device array instead of a caller buffer.  Every GPU the library runs on holds its own copy of the array at its own address
// until the process ends; `scratch` itself is only the host-side stand-in of the symbol, so the device address is looked up once per
// device (tga_init, with that device current) and everything below uses that pointer.
#define ROUTE_STATIC_WORDS (2 * 65536)                       // int32: n_tokens * k + ceil(n_tokens * k / 1024) * n_experts must fit (512 KiB)
#define ROUTE_MAX_DEVICES 64
static __device__ __align__(256) int32_t scratch[ROUTE_STATIC_WORDS];
static int32_t* g_route_scratch[ROUTE_MAX_DEVICES];          // device address of `scratch` on device d, filled by tga_route_scratch_setup(d)

int tga_route_scratch_setup(int device) {                    // called by tga_init after hipSetDevice(device)
  TGA_REQUIRE(device >= 0 && device < ROUTE_MAX_DEVICES, "tga_init: device %d is beyond the %d devices the static workspace table covers", device, ROUTE_MAX_DEVICES);
  if (g_route_scratch[device]) return 0;
  int32_t* p = nullptr;
  TGA_HIP(hipGetSymbolAddress((void**)&p, HIP_SYMBOL(scratch)));
  g_route_scratch[device] = p;
  return 0;
}

int tga_moe_route_static(const float* logits, int n_tokens, int n_experts, int k, float* weights, int32_t* topi, int32_t* dest_row, int32_t* off,
                         int32_t* counts, void* stream) {
  int dev = -1;
  TGA_HIP(hipGetDevice(&dev));
  TGA_REQUIRE(dev >= 0 && dev < ROUTE_MAX_DEVICES && g_route_scratch[dev], "tga_moe_route_static: tga_init has not run on device %d", dev);
  TGA_REQUIRE(n_tokens >= 1 && k >= 1 && n_experts >= 1 && (long long)n_tokens * k <= 65536, "tga_moe_route_static: n_tokens * k = %lld exceeds the static workspace (65536 assignments)", (long long)n_tokens * k);
  const long long words = (long long)n_tokens * k + (((long long)n_tokens * k + 1023) / 1024) * n_experts;
  TGA_REQUIRE(words <= ROUTE_STATIC_WORDS, "tga_moe_route_static: %lld workspace words needed, the static workspace holds %d (n_tokens * k + ceil(n_tokens * k / 1024) * n_experts)", words, ROUTE_STATIC_WORDS);
  return moe_route_launch("tga_moe_route_static", logits, n_tokens, n_experts, k, weights, topi, dest_row, off, counts, g_route_scratch[dev], (hipStream_t)stream);
}

int tga_moe_dispatch(const void* x_bf16, const int32_t* dest_row, const int32_t* off, const int32_t* counts, int n_tokens, int k, int n_experts,
                     int64_t m_l, int D, void* xg_bf16, void* stream) {
  TGA_REQUIRE(x_bf16 && dest_row && off && counts && xg_bf16, "tga_moe_dispatch: null pointer");
  TGA_REQUIRE(D > 0 && D % 8 == 0 && m_l > 0 && m_l % MX_BLOCK_ROW == 0, "tga_moe_dispatch: D %% 8 and m_l %% 256 must be 0");
  hipStream_t s = (hipStream_t)stream;
  dispatch_zero_pad_kernel<<<(unsigned)m_l, 256, 0, s>>>(off, counts, n_experts, (int)m_l, D, (uint16_t*)xg_bf16);
  TGA_LAUNCH_CHECK();
  dispatch_kernel<<<n_tokens * k, 256, 0, s>>>((const uint16_t*)x_bf16, dest_row, k, D, (uint16_t*)xg_bf16);
  TGA_LAUNCH_CHECK();
  return 0;
}

int tga_moe_combine_rows(const void* z_bf16, const int32_t* dest_row, const float* weights, int n_tokens, int k, int D, void* out_bf16, void* stream) {
  TGA_REQUIRE(z_bf16 && dest_row && weights && out_bf16, "tga_moe_combine_rows: null pointer");
  combine_kernel<<<n_tokens, 256, 0, (hipStream_t)stream>>>((const uint16_t*)z_bf16, dest_row, weights, k, D, (uint16_t*)out_bf16);
  TGA_LAUNCH_CHECK();
  return 0;
}

static int grouped_mxfp8_gemm_launch(void* C, const void* A, const void* B, const void* x_e8, const void* w_e8, const int32_t* expert_off,
                                     int64_t M, int64_t N, int64_t K, int n_experts, int routed_only, const int32_t* counts, void* stream) {
  TGA_REQUIRE(C && A && B && x_e8 && w_e8 && expert_off, "tga_grouped_mxfp8_gemm: null pointer");
  // the reference's precondition (extra/gemm/moe_gemm.py:120)
  TGA_REQUIRE(M % 256 == 0 && N % 256 == 0 && K % 128 == 0, "grouped mxfp8 needs M%%256,N%%256,K%%128, got (%lld, %lld) (%d, %lld, %lld)",
              (long long)M, (long long)K, n_experts, (long long)N, (long long)K);
  TGA_REQUIRE(M > 0 && N > 0 && K > 0 && n_experts >= 1 && (M / GG_TILE) * (N / GG_TILE) < (1ll << 31) && M < (1ll << 31) && N < (1ll << 31) && K < (1ll << 31),
              "tga_grouped_mxfp8_gemm: empty or oversized problem (%lld, %lld, %lld), %d experts", (long long)M, (long long)N, (long long)K, n_experts);
  GemmArgs g; g.C = (uint16_t*)C; g.A = (const uint8_t*)A; g.B = (const uint8_t*)B; g.a_e8 = (const uint8_t*)x_e8; g.b_e8 = (const uint8_t*)w_e8;
  g.off = expert_off; g.M = (int)M; g.N = (int)N; g.K = (int)K; g.E = n_experts; g.routed_only = routed_only; g.counts = counts;
  // one workgroup per CU (its 148 KB of LDS fill the CU anyway); each walks its share of the tiles
  static const int n_cu = [] { int dev = 0, n = 0; return (hipGetDevice(&dev) == hipSuccess && hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0) ? n : 256; }();
  const long long tiles = (M / GG_TILE) * (N / GG_TILE);
  grouped_mxfp8_gemm_lds_kernel<<<(unsigned)(tiles < n_cu ? tiles : n_cu), GG_THREADS, 0, (hipStream_t)stream>>>(g);
  TGA_LAUNCH_CHECK();
  return 0;
}

int tga_grouped_mxfp8_gemm(void* C, const void* A, const void* B, const void* x_si, const void* w_si, const void* x_e8, const void* w_e8,
                           const int32_t* expert_off, int64_t M, int64_t N, int64_t K, int n_experts, void* stream) {
  (void)x_si; (void)w_si;   // the packed (K/128, rows) scale copies the reference's kernel reads are accepted but not needed here
  return grouped_mxfp8_gemm_launch(C, A, B, x_e8, w_e8, expert_off, M, N, K, n_experts, 0, nullptr, stream);
}

int tga_grouped_mxfp8_gemm_routed(void* C, const void* A, const void* B, const void* x_e8, const void* w_e8, const int32_t* expert_off,
                                  int64_t M, int64_t N, int64_t K, int n_experts, void* stream) {
  return grouped_mxfp8_gemm_launch(C, A, B, x_e8, w_e8, expert_off, M, N, K, n_experts, 1, nullptr, stream);
}

int tga_grouped_mxfp8_gemm_counts(void* C, const void* A, const void* B, const void* x_e8, const void* w_e8, const int32_t* expert_off, const int32_t* counts,
                                  int64_t M, int64_t N, int64_t K, int n_experts, void* stream) {
  TGA_REQUIRE(counts, "tga_grouped_mxfp8_gemm_counts: null counts");
  return grouped_mxfp8_gemm_launch(C, A, B, x_e8, w_e8, expert_off, M, N, K, n_experts, 1, counts, stream);
}

int tga_kernel_symbol(const char* name, const void** host_function) {
  TGA_REQUIRE(name && host_function, "tga_kernel_symbol: null pointer");
  if (strcmp(name, "tga_grouped_mxfp8_gemm_kernel") == 0) { *host_function = (const void*)tga_grouped_mxfp8_gemm_kernel; return 0; }
  return tga_set_error("tga_kernel_symbol: no kernel named '%s'", name);
}

int tga_add_expert_bias(void* h_bf16, const float* bias, const int32_t* expert_off, int64_t M, int64_t N, int n_experts, void* stream) {
  TGA_REQUIRE(h_bf16 && bias && expert_off, "tga_add_expert_bias: null pointer");
  TGA_REQUIRE(M >= 0 && M % 256 == 0 && N > 0 && n_experts >= 1, "tga_add_expert_bias: M=%lld must be a multiple of 256", (long long)M);
  if (M == 0) return 0;
  const int gx = (int)((N + 255) / 256 < 64 ? (N + 255) / 256 : 64);
  add_expert_bias_kernel<<<dim3(gx, (unsigned)(M / 256)), 256, 0, (hipStream_t)stream>>>((uint16_t*)h_bf16, bias, expert_off, n_experts, (int)N);
  TGA_LAUNCH_CHECK();
  return 0;
}

int tga_swiglu_interleaved(const void* h_bf16, int64_t rows, int two_inter, float limit, float alpha, void* y_bf16, void* stream) {
  TGA_REQUIRE(h_bf16 && y_bf16 && two_inter > 0 && two_inter % 2 == 0, "tga_swiglu_interleaved: bad argument");
  if (rows == 0) return 0;
  const long long n = rows * (two_inter / 2);
  const int grid = (int)((n + 255) / 256 < 65536 ? (n + 255) / 256 : 65536);
  swiglu_interleaved_kernel<<<grid, 256, 0, (hipStream_t)stream>>>((const uint16_t*)h_bf16, rows, two_inter, limit, alpha, (uint16_t*)y_bf16);
  TGA_LAUNCH_CHECK();
  return 0;
}

}  // extern "C"
