// Small-batch GEMM over Q4_0 / Q8_0 / Q4_1 / Q5_0 / Q5_1 block pairs, Q4_K / Q5_K superblocks (K = 2048 or 4096) and fp16 weights (K = 2048), 2 <= M <= 16 activation rows, with the weights streamed into LDS by direct-to-LDS loads into rings
// that belong to ONE WAVE each: the same call sites and arithmetic as qgemm_dma.hip (x.linear(W.T) over a lazily dequantized weight: tinygrad/nn/__init__.py:177,
// tinygrad/mixin/op.py:367-392; a unit is decoded once into fp16 weights - the reference's fp16 weight cast, tinygrad/llm/model.py:376 - and
// v_mfma_f32_16x16x32_f16 multiplies it with all activation rows), without a workgroup barrier in the loop.
//
// Why.  In qgemm_dma.hip the eight waves of a workgroup request a stage's pieces together and meet at one barrier per stage, so all of them wait, read LDS, decode
// and multiply in the same phase at the same time: a stage costs the sum of its phases.  Here wave w of the workgroup owns units [w UPW, (w + 1) UPW) of every row
// (UPW = 4 or 8: an eighth of K), i.e. bytes [w S, (w + 1) S) of each of the 16 rows of a row group (S = 144 .. 544); it requests them itself (16-byte
// pieces, 64 per instruction), waits for them with its own counter, reads them back in the MFMA operand layout and requests the next group into the freed ring
// position - nobody else touches its ring, so no barrier orders it, and the waves of a CU drift into different phases by themselves.  Measured: bare streaming of
// that pattern (requests and LDS reads only) moves 14336 x 4096 of Q4_0 / Q8_0 bytes in 7.2 / 12.2 us; the kernel at eight rows: Q8_0 16.0 us where the barrier
// kernel takes 18.4 (4096 x 4096: 7.6 against 9.05), Q4_0 13.4 against 13.3 (6.55 against 7.2), the K-quants and 5-bit pairs 3 - 20 % less on 4096 x 4096 and
// -8 .. +4 % on 14336 x 4096.  Replayed batched decode of 8B-architecture models, B = 4 / 8 / 16: Q8_0 -5 / -6 % per step, Q4_0 -2 / -1.2 / -0.6 %, the Q4_K_M mix
// -1.1 / -0.9 / -2 %; OLMoE-architecture (fp16 dense weights) +4 / +3 / +1.5 % tokens per second.  Per-wave clock stamps put what is left in the decode's VALU work
// (the 4- to 6-bit formats: 2.3 operations per weight) and a 1.7 - 3 us prologue (the second wave of a SIMD forms its activation operands behind the first).
// The eight partial 16 x 16 tiles of a row group meet in LDS once per group: every wave stores its tile and counts itself in with an LDS operation; wave j % 8
// waits (bounded) for the eight counts of group j, sums the tiles in wave order and stores the rows - the role rotates, so that the wave that arrives last is not
// the one that falls further behind.  Two tile sets alternate; a wave that is two groups ahead waits (bounded) until the set it wants has been summed.  Both waits
// are for waves that are behind and wait for nobody themselves.
#include "qdma_fmt.h"
#include "host.h"

#define WP_NW 8
#define WP_SPIN (1 << 22)

// The tile-set counters are read and written by inline assembly: an atomic builtin on LDS makes the compiler wait for every direct-to-LDS piece in flight in front
// of it (it cannot tell that the counters and the rings are different memory), which would empty the ring once per row group.
__device__ __forceinline__ uint32_t wp_lds_addr(const void* p) { return (uint32_t)(uintptr_t)p; }      // (the low half of a generic address of LDS is the LDS offset)
__device__ __forceinline__ unsigned wp_lds_peek(const unsigned* p) { unsigned v; asm volatile("ds_read_b32 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=v"(v) : "v"(wp_lds_addr(p)) : "memory"); return v; }
__device__ __forceinline__ unsigned wp_lds_add(unsigned* p, unsigned d) { unsigned v; asm volatile("ds_add_rtn_u32 %0, %1, %2\n\ts_waitcnt lgkmcnt(0)" : "=v"(v) : "v"(wp_lds_addr(p)), "v"(d) : "memory"); return v; }
__device__ __forceinline__ void wp_lds_poke(unsigned* p, unsigned d) { asm volatile("ds_write_b32 %0, %1" :: "v"(wp_lds_addr(p)), "v"(d) : "memory"); }
template <int N> __device__ __forceinline__ void wp_wait_vm() { asm volatile("s_waitcnt vmcnt(%0)" :: "n"(N) : "memory"); }

template <int T_, bool MS, bool SW, int UPW, int NB>
__global__ __launch_bounds__(WP_NW * 64) void qgemm_wp_kernel(const QArgs args, const int M, const int ring_w) {
  const QArgs a = args;
  using F = Fmt<T_>;
  using DF = DmaFmt<T_>;
  typedef typename F::Raw Raw;
  static_assert(!(MS && SW), "the SwiGLU pair is not combined with the q / k / v walk");
  constexpr int SLICE = DF::slot_bytes(UPW);             // bytes of one row that a wave owns
  static_assert(SLICE % 16 == 0 && UPW % 4 == 0, "a wave's run of a row is whole 16-byte pieces and whole steps of four units");
  constexpr int PR = SLICE / 16, PP = PR + (PR % 2 == 0 ? 1 : 0);   // pieces per row, and with the pad piece: an odd pitch in pieces puts sixteen rows on sixteen different bank quads
  constexpr int PIECES = 16 * PP, NI = (PIECES + 63) / 64, REM = PIECES - 64 * (NI - 1), STAGE = PIECES * 16, PITCH = PP * 16;
  constexpr int NST = UPW / 4;                           // steps (4 units x 16 rows) of a wave per row group
  constexpr int GR = SW ? 8 : 16;                        // output rows per row group
  extern __shared__ u32x4 lds[];
  __shared__ __attribute__((aligned(16))) float part[2][WP_NW][256];   // [tile set][wave][16 c + 4 (g ^ (c >> 2)) + i]: lane (g, c) keeps rows 4 g .. 4 g + 3 of column c as one 16-byte piece (the swizzle spreads a quarter wave over all banks)
  __shared__ float nsum[WP_NW][16];
  __shared__ unsigned cnt[2], done[2];
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int r = lane & 15, g = lane >> 4;
  char* ringw = (char*)lds + (size_t)wave * ring_w;
  if (threadIdx.x < 2) { cnt[threadIdx.x] = 0u; done[threadIdx.x] = 0u; }
  uint32_t kc[F::NKC];
  F::consts(kc);
  const long long ngroups = (SW ? a.n[0] : a.ntot) / GR;
  auto seg_of = [&](long long row0, int& sg, long long& local0) {
    sg = 0; local0 = row0;
    if constexpr (MS) { if (local0 >= a.n[0]) { local0 -= a.n[0]; sg = 1; if (a.nseg > 2 && local0 >= a.n[1]) { local0 -= a.n[1]; sg = 2; } } }
  };
  auto rows_of = [&](int sg) -> long long { return !MS ? a.n[0] : sg == 0 ? a.n[0] : sg == 1 ? a.n[1] : a.n[2]; };
  auto w_of = [&](int sg) -> const uint8_t* { return !MS ? a.w[0] : sg == 0 ? a.w[0] : sg == 1 ? a.w[1] : a.w[2]; };
  const long long G = ((long long)blockIdx.x < ngroups) ? (ngroups - blockIdx.x + gridDim.x - 1) / gridDim.x : 0;   // row groups of this workgroup: every wave walks all of them
  __syncthreads();                                       // (the counters are set)
  if (G == 0) return;

  // where this lane's pieces of a group come from: position 64 i + lane of the padded slice = (row, piece); the pad piece repeats the row's last piece
  long long doff[NI];
  bool from_up[NI];                                      // (SW) rows 8 .. 15 come from the up matrix
#pragma unroll
  for (int i = 0; i < NI; i++) {
    const int sigma = 64 * i + lane;
    int rr = sigma / PP, q = sigma - rr * PP;
    rr = rr < 16 ? rr : 15; q = q < PR ? q : PR - 1;
    from_up[i] = SW && rr >= 8;
    doff[i] = (long long)(SW ? (rr & 7) : rr) * a.row_bytes + (long long)wave * SLICE + q * 16;
  }
  auto issue = [&](long long j, int slot) {
    const long long grp = (long long)blockIdx.x + j * gridDim.x;
    int sg; long long l0; seg_of(grp * GR, sg, l0);
    const long long goff = l0 * a.row_bytes;
    const uint8_t* base = w_of(sg) + goff;
    const uint8_t* base_up = SW ? a.w[1] + goff : base;
    char* dst = ringw + slot * STAGE;
#pragma unroll
    for (int i = 0; i < NI; i++) {
      if (i + 1 < NI || REM == 64 || lane < REM)         // (the last instruction fills the rest of the stage and nothing beyond it)
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)((from_up[i] ? base_up : base) + doff[i]), (__attribute__((address_space(3))) void*)(dst + i * 1024), 16, 0, 0);
    }
  };

  // ---- this lane's activation operands (lane (g, c): the eight vectors of unit wave UPW + 4 ss + g of row c, zeros for c >= M): requested first, the weights second
  // (loads return in issue order), turned into the operand layout through the part of the wave's ring that the first groups do not use yet.  As in qgemm_dma.hip the
  // requests are inline assembly and their wait is counted by hand: a compiler-placed wait would also cover the weight pieces behind them.
  u32x4 bfrag[NST][F::XV];
  {
    char* xb = ringw + (size_t)(NB - 1) * STAGE;
    const bool have = r < M;
    auto prologue = [&](auto rows_tag, auto f32_tag, auto norm_tag) __attribute__((always_inline)) {
      constexpr int XR = decltype(rows_tag)::value;      // rows requested (rows at and beyond M repeat row 0 and are dropped)
      constexpr bool F32 = decltype(f32_tag)::value;
      constexpr bool NORM = decltype(norm_tag)::value;
      static_assert(!NORM || F32, "the folded norm reads float32 rows");
      constexpr int NV = F32 ? XR : XR / 2;              // float32: instruction v = row v, lane l = values 4 l .. 4 l + 3; fp16: rows 2 v and 2 v + 1, lane l = piece l & 31 of row 2 v + (l >> 5)
      u32x4 xq[NST][NV];
#pragma unroll
      for (int ss = 0; ss < NST; ss++)
#pragma unroll
        for (int v = 0; v < NV; v++) {
          const int row = F32 ? v : 2 * v + (lane >> 5);
          const int uc = wave * UPW + 4 * ss;
          const char* ptr = F32 ? (const char*)((const float*)a.x + (long long)(row < M ? row : 0) * a.K + 64 * uc + 4 * lane)
                                : (const char*)((const uint16_t*)a.x + (long long)(row < M ? row : 0) * a.K + 64 * uc + 8 * (lane & 31));
          asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(xq[ss][v]) : "v"(ptr) : "memory");
        }
      u32x4 nwq[NORM ? NST : 1];                         // the norm weight of the step's columns (this lane: 4 values)
      if constexpr (NORM) {
#pragma unroll
        for (int ss = 0; ss < NST; ss++) { const float* ptr = a.norm_w + 64 * (wave * UPW + 4 * ss) + 4 * lane; asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(nwq[ss]) : "v"(ptr) : "memory"); }
      }
      // every wave's activation requests are in the CU's queue before any weight request: a CU returns vector-memory data in request order, and without this the
      // activations of the wave that starts last wait behind the weight misses of the seven that started first (its operands were ready 2 us after theirs)
      asm volatile("s_barrier" ::: "memory");
      int issued = 0;
      for (int k = 0; k < NB - 1; k++) if (k < G) { issue(k, k); issued++; }
      qd_wait_vm(issued * NI);
      float sc[NORM ? NV : 1];
      if constexpr (NORM) {
        // nn.RMSNorm (tinygrad/nn/__init__.py:296-304): every wave sums the squares of the values of K that its steps hold, the eight sums meet in LDS
#pragma unroll
        for (int ss = 0; ss < NST; ss++) {
          asm volatile("; landed" : "+v"(nwq[ss]) :: "memory");
#pragma unroll
          for (int v = 0; v < NV; v++) asm volatile("; landed" : "+v"(xq[ss][v]) :: "memory");
        }
        float ps[NV];
#pragma unroll
        for (int v = 0; v < NV; v++) {
          ps[v] = 0.f;
#pragma unroll
          for (int ss = 0; ss < NST; ss++) { const f32x4 f = __builtin_bit_cast(f32x4, xq[ss][v]); ps[v] += f.x * f.x + f.y * f.y + f.z * f.z + f.w * f.w; }
          ps[v] = wave_sum(ps[v]);
        }
        if (lane == 0) {
#pragma unroll
          for (int v = 0; v < NV; v++) nsum[wave][v] = ps[v];
        }
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
#pragma unroll
        for (int v = 0; v < NV; v++) {
          float t = 0.f;
#pragma unroll
          for (int w = 0; w < WP_NW; w++) t += nsum[w][v];
          sc[v] = 1.0f / sqrtf(t / (float)a.K + a.norm_eps);
        }
      }
#pragma unroll
      for (int ss = 0; ss < NST; ss++) {
#pragma unroll
        for (int v = 0; v < NV; v++) asm volatile("; landed" : "+v"(xq[ss][v]) :: "memory");      // no use of the pieces moves in front of the wait
#pragma unroll
        for (int v = 0; v < NV; v++) {
          if constexpr (F32) {
            f32x4 f = __builtin_bit_cast(f32x4, xq[ss][v]);
            if constexpr (NORM) { const f32x4 nw = __builtin_bit_cast(f32x4, nwq[ss]); f.x = (f.x * sc[v]) * nw.x; f.y = (f.y * sc[v]) * nw.y; f.z = (f.z * sc[v]) * nw.z; f.w = (f.w * sc[v]) * nw.w; }
            *(uint2*)(xb + v * 512 + 16 * (((lane >> 1) + v) & 31) + 8 * (lane & 1)) = uint2{f2h_bits(f.x) | (f2h_bits(f.y) << 16), f2h_bits(f.z) | (f2h_bits(f.w) << 16)};
          } else {
            const int row = 2 * v + (lane >> 5);
            *(u32x4*)(xb + row * 512 + 16 * (((lane & 31) + row) & 31)) = xq[ss][v];
          }
        }
        uint32_t nx[F::UW / 2];
        const int c = r < XR ? r : 0;
        const char* src = xb + c * 512;
#pragma unroll
        for (int j = 0; j < 8; j++) { const u32x4 t4 = *(const u32x4*)(src + 16 * ((F::xoff(g, 4 * j) / 8 + c) & 31)); nx[4 * j] = t4.x; nx[4 * j + 1] = t4.y; nx[4 * j + 2] = t4.z; nx[4 * j + 3] = t4.w; }
        float cs[F::NG];
        F::stage(nx, bfrag[ss], cs);
#pragma unroll
        for (int v = 0; v < F::XV; v++) if (!have) bfrag[ss][v] = u32x4{0u, 0u, 0u, 0u};
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");            // the reads of this step are done before the next step (or the ring) writes there
      }
    };
    typedef std::integral_constant<int, 4> R4; typedef std::integral_constant<int, 8> R8; typedef std::integral_constant<int, 16> R16;
    typedef std::true_type Yes; typedef std::false_type No;
    if (a.norm_w) { if (M > 8) prologue(R16{}, Yes{}, Yes{}); else if (M > 4) prologue(R8{}, Yes{}, Yes{}); else prologue(R4{}, Yes{}, Yes{}); }     // (the launch has checked: float32 rows)
    else if (a.x_f32) { if (M > 8) prologue(R16{}, Yes{}, No{}); else if (M > 4) prologue(R8{}, Yes{}, No{}); else prologue(R4{}, Yes{}, No{}); }
    else { if (M > 8) prologue(R16{}, No{}, No{}); else if (M > 4) prologue(R8{}, No{}, No{}); else prologue(R4{}, No{}, No{}); }
  }

  // the summing wave's part: the eight partial tiles of group j in wave order, lane (g, c) rows 4 g .. 4 g + 3 of activation row c, one vector store
  auto store4 = [&](void* yb, long long o, const f32x4 v) __attribute__((always_inline)) {
    if (a.y_f32) *(f32x4*)((float*)yb + o) = v;
    else *(uint2*)((_Float16*)yb + o) = uint2{f2h_bits(v.x) | (f2h_bits(v.y) << 16), f2h_bits(v.z) | (f2h_bits(v.w) << 16)};
  };
  auto reduce_store = [&](long long row0, int p) __attribute__((always_inline)) {
    int sg; long long l0; seg_of(row0, sg, l0);
    const long long nrows = rows_of(sg);
    const int c = r;
    if constexpr (SW) {
      if (g < 2 && c < M) {
        f32x4 gs = {0.f, 0.f, 0.f, 0.f}, us = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int w = 0; w < WP_NW; w++) { gs += *(const f32x4*)&part[p][w][16 * c + 4 * (g ^ (c >> 2))]; us += *(const f32x4*)&part[p][w][16 * c + 4 * ((g + 2) ^ (c >> 2))]; }
        store4(a.y[0], (long long)c * nrows + l0 + 4 * g, f32x4{silu_f(gs.x) * us.x, silu_f(gs.y) * us.y, silu_f(gs.z) * us.z, silu_f(gs.w) * us.w});
      }
    } else {
      if (c < M) {
        const float* rb = a.epilogue == 1 ? (!MS ? a.resid[0] : sg == 0 ? a.resid[0] : sg == 1 ? a.resid[1] : a.resid[2]) : nullptr;
        void* yb = !MS ? a.y[0] : sg == 0 ? a.y[0] : sg == 1 ? a.y[1] : a.y[2];
        const long long o = (long long)c * nrows + l0 + 4 * g;
        f32x4 v = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int w = 0; w < WP_NW; w++) v += *(const f32x4*)&part[p][w][16 * c + 4 * (g ^ (c >> 2))];
        if (rb) v += *(const f32x4*)(rb + o);
        store4(yb, o, v);
      }
    }
  };

  int slot = 0;
  for (long long j = 0; j < G; j++) {
    const long long after = G - 1 - j;
    // this wave's pieces of group j have landed (later groups, and the stores of a sum, may be in flight)
    if constexpr (NB == 2) wp_wait_vm<0>();
    else { static_assert(NB == 3 && NI <= 24, "ring of two or three groups"); if (after >= 1) wp_wait_vm<NI>(); else wp_wait_vm<0>(); }
    if (j + NB - 1 < G) issue(j + NB - 1, slot == 0 ? NB - 1 : slot - 1);
    v4f32 acc0 = {0.f, 0.f, 0.f, 0.f}, acc1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ss = 0; ss < NST; ss++) {
      const Raw buf = DF::from_lds(ringw + slot * STAGE + r * PITCH, 4 * ss + g);
      uint32_t wv[F::NWV];
      F::decode(buf, wv, kc);
      F::to_f16(buf, wv);
#pragma unroll
      for (int v = 0; v < F::XV; v++) {
        const u32x4 av = {wv[4 * v], wv[4 * v + 1], wv[4 * v + 2], wv[4 * v + 3]};
        if (v & 1) acc1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8f16, av), __builtin_bit_cast(v8f16, bfrag[ss][v]), acc1, 0, 0, 0);
        else acc0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8f16, av), __builtin_bit_cast(v8f16, bfrag[ss][v]), acc0, 0, 0, 0);
      }
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");                  // every read of this ring position is done: the next pass requests into it
    slot = slot + 1 == NB ? 0 : slot + 1;
    // the tile set of this group: free once the group two before it has been summed
    const int p = (int)(j & 1);
    const unsigned turn = (unsigned)(j >> 1);
    if (j >= 2) for (int n = 0; wp_lds_peek(&done[p]) != turn && n < WP_SPIN; n++) __builtin_amdgcn_s_sleep(1);
    *(f32x4*)&part[p][wave][16 * r + 4 * (g ^ (r >> 2))] = f32x4{acc0[0] + acc1[0], acc0[1] + acc1[1], acc0[2] + acc1[2], acc0[3] + acc1[3]};
    // (no wait between the tile and the count: LDS executes a wave's operations in order)
    if (wave != (int)(j & 7)) {
      if (lane == 0) asm volatile("ds_add_u32 %0, %1" :: "v"(wp_lds_addr(&cnt[p])), "v"(1u) : "memory");   // counted in; nothing to wait for
    } else {
      // this wave sums group j: the role rotates, so that the wave that arrives last is not the one that falls further behind; the others are ahead of it
      // and wait for nobody, so the (bounded) wait below ends
      if (lane == 0) asm volatile("ds_add_u32 %0, %1" :: "v"(wp_lds_addr(&cnt[p])), "v"(1u) : "memory");
      for (int n = 0; wp_lds_peek(&cnt[p]) != WP_NW && n < WP_SPIN; n++) __builtin_amdgcn_s_sleep(1);
      reduce_store(((long long)blockIdx.x + j * gridDim.x) * GR, p);
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");                // the tiles have been read
      if (lane == 0) { wp_lds_poke(&cnt[p], 0u); wp_lds_poke(&done[p], turn + 1u); }
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

static int wp_cu_count() {
  static int n = 0;
  if (!n) { int dev = 0; hipDeviceProp_t p; n = (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&p, dev) == hipSuccess) ? p.multiProcessorCount : 256; }
  return n;
}

#define WP_STATIC_LDS (2 * WP_NW * 256 * 4 + WP_NW * 16 * 4 + 64)

template <int T, bool MS, bool SW, int UPW, int NB>
static int launch_wp_k(const QArgs& a, int M, hipStream_t s) {
  using DF = DmaFmt<T>;
  constexpr int SLICE = DF::slot_bytes(UPW), PR = SLICE / 16, PP = PR + (PR % 2 == 0 ? 1 : 0), STAGE = 16 * PP * 16;
  const int xb = (M > 8 ? 16 : M > 4 ? 8 : 4) * 512;                   // the activations' way through LDS: behind the ring positions that are requested first
  int ring_w = NB * STAGE; if ((NB - 1) * STAGE + xb > ring_w) ring_w = (NB - 1) * STAGE + xb;
  const size_t lds = (size_t)WP_NW * ring_w;
  if (lds + WP_STATIC_LDS > (size_t)QD_LDS_CU) return -1;
  auto kern = qgemm_wp_kernel<T, MS, SW, UPW, NB>;
  static int static_lds = 0;
  static const hipError_t configured = [&]() {
    hipFuncAttributes fa;
    hipError_t e = hipFuncGetAttributes(&fa, (const void*)kern);
    if (e != hipSuccess) return e;
    static_lds = (int)fa.sharedSizeBytes;
    return hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)(QD_LDS_CU - fa.sharedSizeBytes));
  }();
  TGA_HIP(configured);
  if (lds + (size_t)static_lds > (size_t)QD_LDS_CU) return -1;
  const long long ngroups = SW ? a.n[0] / 8 : a.ntot / 16;
  const long long cus = wp_cu_count();
  const long long grid = ngroups < cus ? ngroups : cus;
  kern<<<dim3((unsigned)grid), dim3(WP_NW * 64), lds, s>>>(a, M, ring_w);
  TGA_LAUNCH_CHECK();
  return 0;
}

template <int T, int UPW>
static int launch_wp_u(const QArgs& a, int M, hipStream_t s) {
  // three groups in flight per wave where the ring holds them, else two
  int rc;
  if constexpr (T != GGML_F16) { if (a.epilogue == 2) { rc = launch_wp_k<T, false, true, UPW, 3>(a, M, s); return rc >= 0 ? rc : launch_wp_k<T, false, true, UPW, 2>(a, M, s); } }
  if (a.epilogue == 2) return -1;
  if (a.nseg > 1) { rc = launch_wp_k<T, true, false, UPW, 3>(a, M, s); return rc >= 0 ? rc : launch_wp_k<T, true, false, UPW, 2>(a, M, s); }
  rc = launch_wp_k<T, false, false, UPW, 3>(a, M, s); return rc >= 0 ? rc : launch_wp_k<T, false, false, UPW, 2>(a, M, s);
}

template <int T>
static int launch_wp(QArgs a, int M, hipStream_t s) {
  using F = Fmt<T>;
  a.nu = a.K / F::UW;
  a.row_bytes = (long long)(a.K / F::BW) * F::BB;
  if (a.K % F::UW != 0 || a.row_bytes % 16 != 0) return -1;
  if constexpr (T != GGML_F16) { if (a.nu == 64) return launch_wp_u<T, 8>(a, M, s); }       // (fp16 rows of 4096 values: a ring of two groups does not fit, and its operands would spill)
  if (a.nu == 32) return launch_wp_u<T, 4>(a, M, s);
  return -1;
}

// Called by tga_qgemm_dma_dispatch with a call it has checked (2 <= M <= 16, matrices of whole row groups at 16-byte aligned addresses, float32 rows where a norm
// folds in).  Returns -1 outside this kernel's range (K other than 2048 / 4096, Q6_K and the formats that are not block pairs, a ring that does not fit LDS,
// outputs that are not 16-byte aligned).
int tga_qgemm_wp_dispatch(int fmt, const QArgs& a, int M, hipStream_t s) {
  static const bool off = getenv("TGA_WP") && atoi(getenv("TGA_WP")) == 0;      // (for A / B runs against the barrier kernel)
  if (off) return -1;
  static const int skip = getenv("TGA_WP_SKIP") ? atoi(getenv("TGA_WP_SKIP")) : 0;   // (A / B: 1 plain, 2 several matrices, 4 SwiGLU pair stay on the barrier kernel)
  if (skip & (a.epilogue == 2 ? 4 : a.nseg > 1 ? 2 : 1)) return -1;
  if (fmt == GGML_F16 && (a.epilogue == 2 || a.K != 2048)) return -1;  // (fp16 rows of 4096 values: a ring of two groups does not fit)
  if (fmt == F_Q4_0P && a.epilogue == 2) return -1;                    // (the Q4_0 SwiGLU pair: the barrier kernel is 0.8 % of a batched 8B step ahead from eight rows on, equal below)
  for (int i = 0; i < (a.epilogue == 2 ? 1 : a.nseg); i++)          // four rows of a column leave as one vector store
    if (((uintptr_t)a.y[i] & 15) != 0 || (a.epilogue == 1 && ((uintptr_t)a.resid[i] & 15) != 0)) return -1;
  switch (fmt) {
    case F_Q4_0P: return launch_wp<F_Q4_0P>(a, M, s);
    case F_Q8_0P: return launch_wp<F_Q8_0P>(a, M, s);
    case GGML_Q4_K: return launch_wp<GGML_Q4_K>(a, M, s);
    case GGML_Q5_K: return launch_wp<GGML_Q5_K>(a, M, s);
    case GGML_Q4_1: return launch_wp<GGML_Q4_1>(a, M, s);
    case GGML_Q5_0: return launch_wp<GGML_Q5_0>(a, M, s);
    case GGML_Q5_1: return launch_wp<GGML_Q5_1>(a, M, s);
    case GGML_F16: return launch_wp<GGML_F16>(a, M, s);
  }
  return -1;
}
