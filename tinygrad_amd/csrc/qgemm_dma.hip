// Small-batch GEMM over Q4_0 / Q8_0 / Q4_1 / Q5_0 / Q5_1 block pairs, Q4_K / Q5_K / Q6_K superblocks and fp16 weights (2 <= M <= 16: the sixteen columns of the MFMA tile) with the weights streamed into LDS by direct-to-LDS loads: the same
// call sites and arithmetic as qgemm.hip (x.linear(W.T) over a lazily dequantized weight: tinygrad/nn/__init__.py:177, tinygrad/mixin/op.py:367-392;
// a unit is decoded once into fp16 weights and v_mfma_f32_16x16x32_f16 multiplies it with all activation rows).
//
// Why a second kernel.  The MFMA operand layout wants lane (g, r) to hold a unit of weight ROW r, so a register load touches sixteen rows
// with 144- or 272-byte runs: measured on a 14336 x 4096 Q8_0 matrix, that lane -> address map streams at 3.4 TB/s where fully contiguous
// 16-byte pieces stream at 5.3 TB/s, and the Q4_0 kernel (half the bytes, the same number of scattered pieces) is no faster than the Q8_0
// one.  Here global memory is read in contiguous 16-byte pieces, 1 KB per wave instruction (global_load_lds_dwordx4: lane l's piece lands at
// LDS base + 16 l), and the operand layout is produced by the LDS reads: each lane picks its unit out of the staged rows.
//
// A slot is 16 weight rows x 16 or 32 units (1024 / 2048 values of K); its rows lie in LDS with a pitch of one piece more than their length, which
// spreads the sixteen rows over the banks.  A stage is two slots: waves 0-3 multiply the steps (4 units x 16 rows each; one or two per
// wave) of the first, waves 4-7 those of the second.  The eight waves of the workgroup (one per CU) issue a stage's pieces together and
// keep nb - 1 stages in flight in a ring of nb.  One barrier per stage orders "all pieces of stage s have landed" before its reads and
// "everyone is done with stage s - 1" before its slots are requested again; the partial tiles of the waves meet in LDS once per row
// group and are reduced after the next stage's barrier.
// A wave meets the same units of K in every row group (K <= 4096: at most two), so its activation operands - lane (g, c): the eight
// vectors of row c's unit, zeros for c >= M - stay in registers for the whole launch; LDS holds nothing but the ring.
// K > 4096 (XS): the activations are streamed too.  A wave reads the 512 bytes of every activation row that its step of the next stage multiplies in
// whole 128-byte lines (eight loads of 1 KB, two rows each: a lane-per-unit read would touch 64 lines per instruction and use 16 bytes of each),
// issued in front of the weight pieces of the stage after (loads return in issue order: the wait that lets the weights of later stages stay in
// flight then covers them), and turns them into the operand layout through a wave-private piece of LDS.
#include "qdma_fmt.h"

// SW: silu(gate) * up (dense SwiGLU, tinygrad/llm/model.py:137) over the two matrices w[0] / w[1]: a row group is eight rows of the gate matrix followed
// by the same eight rows of the up matrix, so the partial tiles of both meet in one reduction and the product is formed before the store.
// SU: units per slot (16 or 32): a longer run of every row per slot streams better (Q4_0: 576-byte runs at 16 units, 1152 at 32) and halves the
// number of stages, a wave then multiplies SU / 16 steps of its slot per stage.
#define QD_XT_PITCH 528                // bytes between activation rows in a wave's transposition buffer (512 + one piece: sixteen rows spread over the banks)
template <int T_, bool MS, int NSS, bool SW, int SU, bool XS = false, bool XF = false>      // XF: (XS) float32 activations
__global__ __launch_bounds__(QD_NW * 64) void qgemm_dma_kernel(const QArgs args, const int M, const int nb) {
  constexpr int QD_SU = SU, SPW = SU / 16;               // steps of one wave per slot
  static_assert(!(MS && SW), "the SwiGLU pair is not combined with the q / k / v walk");
  static_assert(!XS || (SPW == 1 && !MS && !SW), "streamed activations: one step per wave and stage, a single matrix");
  const QArgs a = args;
  using F = Fmt<T_>;
  using DF = DmaFmt<T_>;
  typedef typename F::Raw Raw;
  constexpr int PR = DF::pieces(QD_SU);                  // 16-byte pieces of one row in a slot
  constexpr int SECOND = DF::second_off(QD_SU), STRIDE = DF::stage_stride(QD_SU);
  static_assert(SECOND % 16 == 0 && STRIDE % 16 == 0, "slots are fetched in aligned 16-byte pieces");
  constexpr int PITCH = (PR + DF::PAD) * 16;             // LDS bytes from one row of the slot to the next
  constexpr int SLOTS = 16 * (PR + DF::PAD);
  constexpr int NI = (SLOTS + 63) / 64;                  // wave instructions (1 KB each) per slot
  constexpr int SLOT_BYTES = NI * 1024;
  constexpr int NI2 = 2 * NI;                            // ... per stage
  constexpr int IMAX = (NI2 + QD_NW - 1) / QD_NW;        // instructions of one wave per stage, at most
  constexpr int BASE = NI2 / QD_NW;                      // ... and at least
  extern __shared__ u32x4 lds[];
  __shared__ float part[2][QD_NW][16][17];
  char* ring = (char*)lds;
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int r = lane & 15, g = lane >> 4;
  const int half = wave >> 2, step = wave & 3;           // this wave's slot of a stage and its step inside the slot
  uint32_t kc[F::NKC];
  F::consts(kc);
  const int cu = a.nu, nslots = cu / QD_SU, spg = (nslots + 1) >> 1;   // stages per row group (NSS >= spg)
  constexpr int GR = SW ? 8 : 16;                        // output rows per row group
  const long long ngroups = (SW ? a.n[0] : a.ntot) / GR;
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
    if constexpr (SW) {
      if (t < 256 && wr < 8 && c < M && l0 + wr < nrows) {
        float gate = 0.f, up = 0.f;
#pragma unroll
        for (int w = 0; w < QD_NW; w++) { gate += part[p][w][wr][c]; up += part[p][w][wr + 8][c]; }
        const float v = silu_f(gate) * up;
        const long long o = (long long)c * nrows + l0 + wr;
        if (a.y_f32) ((float*)a.y[0])[o] = v; else ((_Float16*)a.y[0])[o] = (_Float16)v;
      }
      return;
    }
    if (t < 256 && c < M && l0 + wr < nrows) {
      float v = 0.f;
#pragma unroll
      for (int w = 0; w < QD_NW; w++) v += part[p][w][wr][c];
      const long long o = (long long)c * nrows + l0 + wr;
      if (a.epilogue == 1) v += (!MS ? a.resid[0] : sg == 0 ? a.resid[0] : sg == 1 ? a.resid[1] : a.resid[2])[o];
      void* yb = !MS ? a.y[0] : sg == 0 ? a.y[0] : sg == 1 ? a.y[1] : a.y[2];
      if (a.y_f32) ((float*)yb)[o] = v; else ((_Float16*)yb)[o] = (_Float16)v;
    }
  };
  const long long G = ((long long)blockIdx.x < ngroups) ? (ngroups - blockIdx.x + gridDim.x - 1) / gridDim.x : 0;
  const long long S = G * spg;                           // stages of this workgroup
  if (S == 0) return;

  // where this lane's pieces of a stage come from: position 64 j + lane of the two padded slots = (slot, row, piece); the pad piece of a row
  // and the positions past the last row repeat a valid piece (they land in the slot's slack).  When K ends inside a stage (an odd number of
  // slots), the second slot repeats the first: nothing reads it.
  long long doff[IMAX], doff_odd[IMAX];
  bool from_up[IMAX];                                    // (SW) rows 8 .. 15 of the slot come from the up matrix
#pragma unroll
  for (int i = 0; i < IMAX; i++) {
    const int j = wave + QD_NW * i, sl = j >= NI ? 1 : 0;
    const int sigma = 64 * (j - sl * NI) + lane;
    int rr = sigma / (PR + DF::PAD), q = sigma - rr * (PR + DF::PAD);
    rr = rr < 16 ? rr : 15; q = q < PR ? q : PR - 1;
    from_up[i] = SW && rr >= 8;
    doff_odd[i] = (long long)(SW ? (rr & 7) : rr) * a.row_bytes + q * 16;
    doff[i] = doff_odd[i] + sl * SECOND;
  }
  long long ij = 0; int ist = 0, islot = 0;              // issue stream: row group index (of this workgroup), stage in the group, ring position
  auto issue_stage = [&]() {
    const long long grp = (long long)blockIdx.x + ij * gridDim.x;
    int sg; long long l0; seg_of(grp * GR, sg, l0);
    const long long goff = l0 * a.row_bytes + (long long)ist * STRIDE;
    const uint8_t* base = w_of(sg) + goff;
    const uint8_t* base_up = SW ? a.w[1] + goff : base;
    char* dst = ring + (size_t)islot * (2 * SLOT_BYTES);
    const bool two = 2 * ist + 1 < nslots;
#pragma unroll
    for (int i = 0; i < IMAX; i++) {
      const int j = wave + QD_NW * i;
      if (j < NI2)                                                     // (the same for the whole wave)
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)((from_up[i] ? base_up : base) + (two ? doff[i] : doff_odd[i])), (__attribute__((address_space(3))) void*)(dst + j * 1024), 16, 0, 0);
    }
    if (++ist == spg) { ist = 0; ij++; }
    islot = islot + 1 == nb ? 0 : islot + 1;
  };

  // this lane's activation operands: requested first (loads return in issue order), the weights second
  u32x4 bfrag[XS ? 1 : NSS * SPW][F::XV];
  constexpr int NXI = XF ? 16 : 8;                       // (XS) load instructions per stage: one row of 256 float32 or two rows of 256 fp16 each
  u32x4 xin[NXI];                                        // (XS) the wave's activation pieces of the next stage on their way in (requesting them two stages ahead
                                                         // gained nothing: a stage waits 0.1 us for its loads, the rest is issue, LDS round trips and the barrier)
  const int xrows = M > 8 ? 16 : 8;                      // (XS) activation rows in the transposition buffer
  char* xt = ring + (size_t)nb * (2 * SLOT_BYTES) + (size_t)wave * xrows * QD_XT_PITCH;
  auto fetch_x = [&](int st, u32x4 (&xs)[NXI]) __attribute__((always_inline)) {     // stage st of a row group: 256 consecutive values of every activation row
    const int u0 = (2 * st + half) * QD_SU + 4 * step;   // (u0 + 3 < cu wherever the slot exists: K is whole slots)
    const int uc = u0 + 3 < cu ? u0 : cu - 4;
#pragma unroll
    for (int v = 0; v < NXI; v++) {
      if ((XF ? v : 2 * v) < xrows) {                    // (the same for the whole workgroup)
        int row = XF ? v : 2 * v + (lane >> 5); row = row < M ? row : 0;
        const char* p = XF ? (const char*)((const float*)a.x + (long long)row * a.K + 64 * uc + 4 * lane)
                           : (const char*)((const uint16_t*)a.x + (long long)row * a.K + 64 * uc + 8 * (lane & 31));
        asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(xs[v]) : "v"(p) : "memory");
      }
    }
  };
  auto pin_x = [&](u32x4 (&xs)[NXI]) __attribute__((always_inline)) {       // no use of the pieces moves in front of the wait that precedes this
    asm volatile("; landed" : "+v"(xs[0]), "+v"(xs[1]), "+v"(xs[2]), "+v"(xs[3]), "+v"(xs[4]), "+v"(xs[5]), "+v"(xs[6]), "+v"(xs[7]) :: "memory");
    if constexpr (XF) asm volatile("; landed" : "+v"(xs[8]), "+v"(xs[9]), "+v"(xs[10]), "+v"(xs[11]), "+v"(xs[12]), "+v"(xs[13]), "+v"(xs[14]), "+v"(xs[15]) :: "memory");
  };
  if constexpr (XS) {
    fetch_x(0, xin);
    for (int k = 0; k < nb - 1; k++) if (k < S) issue_stage();
  } else {
    // Every activation row's 256 values of a step are read in whole lines (a lane-per-unit read touches 64 lines per instruction and uses 16 bytes
    // of each) and reach the operand layout through LDS: the ring position that the first stages do not use yet, 8 KB per wave, the 16-byte pieces
    // of row c rotated by c so that writes and reads are free of bank conflicts.
    constexpr int NST = NSS * SPW;
    char* xb = ring + (size_t)(nb - 1) * (2 * SLOT_BYTES) + (size_t)wave * 8192;
    bool have[NST], stepok[NST]; int uc[NST];
#pragma unroll
    for (int ss = 0; ss < NST; ss++) {
      const int u0 = (2 * (ss / SPW) + half) * QD_SU + 4 * (step + 4 * (ss % SPW));
      have[ss] = r < M && u0 + g < cu;
      stepok[ss] = u0 + 3 < cu;                          // the step's four units exist (over all waves and steps every unit of a row exactly once)
      uc[ss] = stepok[ss] ? u0 : cu - 4;                 // (K is whole slots of at least 16 units)
    }
    // The requests are inline assembly and the wait is counted by hand: a compiler-placed wait would also cover the weight pieces issued behind
    // them (it cannot count those), i.e. the operands would be formed only after the first stages have landed.  Requests, wait and the writes to
    // LDS are straight-line code per row count (4, 8 or 16 rows: what a workgroup reads of the activations is as much as it reads of a Q4_0
    // matrix at sixteen rows): a request behind a condition would give the compiler a reason to move the pieces between registers while they
    // are on their way (it takes them for present as soon as the request is issued).
    const int mine = (NI2 - wave + QD_NW - 1) / QD_NW;   // this wave's pieces per stage
    // NORM (float32 rows): the rows are RMS-normalised on the way (nn.RMSNorm, tinygrad/nn/__init__.py:296-304: x * rsqrt(mean(x^2) + eps) * weight, the
    // attn_norm / ffn_norm in front of q/k/v and gate/up, tinygrad/llm/model.py:149-150): every wave sums the squares of the 256 values per row that its
    // steps hold, the eight waves' sums meet in LDS (one more barrier), and the values are scaled before they are rounded to fp16.
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
          const char* ptr = F32 ? (const char*)((const float*)a.x + (long long)(row < M ? row : 0) * a.K + 64 * uc[ss] + 4 * lane)
                                : (const char*)((const uint16_t*)a.x + (long long)(row < M ? row : 0) * a.K + 64 * uc[ss] + 8 * (lane & 31));
          asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(xq[ss][v]) : "v"(ptr) : "memory");
        }
      u32x4 nwq[NORM ? NST : 1];                         // the norm weight of the step's columns (this lane: 4 values)
      if constexpr (NORM) {
#pragma unroll
        for (int ss = 0; ss < NST; ss++) { const float* ptr = a.norm_w + 64 * uc[ss] + 4 * lane; asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(nwq[ss]) : "v"(ptr) : "memory"); }
      }
      int issued = 0;
      for (int k = 0; k < nb - 1; k++) if (k < S) { issue_stage(); issued++; }
      qd_wait_vm(issued * mine);
      float sc[NORM ? NV : 1];
      if constexpr (NORM) {
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
          for (int ss = 0; ss < NST; ss++) { const f32x4 f = __builtin_bit_cast(f32x4, xq[ss][v]); ps[v] += stepok[ss] ? f.x * f.x + f.y * f.y + f.z * f.z + f.w * f.w : 0.f; }
          ps[v] = wave_sum(ps[v]);
        }
        if (lane == 0) {
#pragma unroll
          for (int v = 0; v < NV; v++) part[0][wave][v][0] = ps[v];
        }
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
#pragma unroll
        for (int v = 0; v < NV; v++) {
          float t = 0.f;
#pragma unroll
          for (int w = 0; w < QD_NW; w++) t += part[0][w][v][0];
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
        for (int v = 0; v < F::XV; v++) if (!have[ss]) bfrag[ss][v] = u32x4{0u, 0u, 0u, 0u};
      }
    };
    typedef std::integral_constant<int, 4> R4; typedef std::integral_constant<int, 8> R8; typedef std::integral_constant<int, 16> R16;
    typedef std::true_type Yes; typedef std::false_type No;
    if (a.norm_w) { if (M > 8) prologue(R16{}, Yes{}, Yes{}); else if (M > 4) prologue(R8{}, Yes{}, Yes{}); else prologue(R4{}, Yes{}, Yes{}); }     // (the launch has checked: float32 rows)
    else if (a.x_f32) { if (M > 8) prologue(R16{}, Yes{}, No{}); else if (M > 4) prologue(R8{}, Yes{}, No{}); else prologue(R4{}, Yes{}, No{}); }
    else { if (M > 8) prologue(R16{}, No{}, No{}); else if (M > 4) prologue(R8{}, No{}, No{}); else prologue(R4{}, No{}, No{}); }
  }

  v4f32 acc0 = {0.f, 0.f, 0.f, 0.f}, acc1 = {0.f, 0.f, 0.f, 0.f};
  long long cj = 0; int cst = 0, cslot = 0, par = 0;     // compute stream
  long long pend_row0 = -1; int pend_par = 0;            // row group whose partial tiles wait for the next barrier
  auto multiply = [&](const u32x4* bv, int k) {
    const Raw buf = DF::from_lds(ring + (size_t)cslot * (2 * SLOT_BYTES) + half * SLOT_BYTES + r * PITCH + DF::skew(QD_SU, half), 4 * (step + 4 * k) + g);
    uint32_t wv[F::NWV];
    F::decode(buf, wv, kc);
    F::to_f16(buf, wv);
#pragma unroll
    for (int v = 0; v < F::XV; v++) {
      const u32x4 av = {wv[4 * v], wv[4 * v + 1], wv[4 * v + 2], wv[4 * v + 3]};
      if (v & 1) acc1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8f16, av), __builtin_bit_cast(v8f16, bv[v]), acc1, 0, 0, 0);
      else acc0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8f16, av), __builtin_bit_cast(v8f16, bv[v]), acc0, 0, 0, 0);
    }
  };
  auto finish_stage = [&]() __attribute__((always_inline)) {
    cslot = cslot + 1 == nb ? 0 : cslot + 1;
    if (++cst == spg) {                                                // row group complete: the waves' partial tiles go to LDS
#pragma unroll
      for (int i = 0; i < 4; i++) part[par][wave][4 * g + i][r] = acc0[i] + acc1[i];
      pend_row0 = ((long long)blockIdx.x + cj * gridDim.x) * GR; pend_par = par;
      par ^= 1;
      acc0 = v4f32{0.f, 0.f, 0.f, 0.f}; acc1 = v4f32{0.f, 0.f, 0.f, 0.f};
      cst = 0; cj++;
    }
  };
  // (XS) one stage; the activations of stage s sit in register set `set`
  auto xs_stage = [&](long long s, u32x4 (&xs)[NXI]) __attribute__((always_inline)) {
    const long long after = S - 1 - s;
    // queue of this wave: ... x(s), weights(s + 1) | x(s + 1), weights(s + 2) ...: with the weights of stage s + 1 (and nothing else) allowed to be
    // outstanding, the weights of stage s and the activations of stage s have arrived
    qd_wait_vm((int)(after < nb - 2 ? after : nb - 2) * BASE);
    pin_x(xs);
#pragma unroll
    for (int v = 0; v < NXI; v++) {
      if constexpr (XF) {
        if (v < xrows) {
          const f32x4 f = __builtin_bit_cast(f32x4, xs[v]);
          *(uint2*)(xt + v * QD_XT_PITCH + 8 * lane) = uint2{f2h_bits(f.x) | (f2h_bits(f.y) << 16), f2h_bits(f.z) | (f2h_bits(f.w) << 16)};
        }
      } else {
        if (2 * v < xrows) *(u32x4*)(xt + (2 * v + (lane >> 5)) * QD_XT_PITCH + 16 * (lane & 31)) = xs[v];
      }
    }
    // (a __syncthreads() here makes the compiler wait for every outstanding vector-memory operation in front of the barrier)
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    if (pend_row0 >= 0) { store_tile(pend_row0, pend_par); pend_row0 = -1; }
    // one request site in the loop: the compiler must have no reason to copy the pieces from one set of registers to another while they are on
    // their way (it takes them for present as soon as the request is issued)
    fetch_x(cst + 1 == spg ? 0 : cst + 1, xs);                           // (past the last stage: a valid address, never used)
    if (s + nb - 1 < S) issue_stage();
    if (2 * cst + half < nslots) {
      uint32_t nx[F::UW / 2];
      const char* src = xt + (r < xrows ? r : 0) * QD_XT_PITCH;           // (the pieces of unit g in the format's own order: 64 consecutive values except for Q6_K)
#pragma unroll
      for (int j = 0; j < 8; j++) { const u32x4 t4 = *(const u32x4*)(src + 16 * (F::xoff(g, 4 * j) / 8)); nx[4 * j] = t4.x; nx[4 * j + 1] = t4.y; nx[4 * j + 2] = t4.z; nx[4 * j + 3] = t4.w; }
      float c[F::NG];
      F::stage(nx, bfrag[0], c);
#pragma unroll
      for (int v = 0; v < F::XV; v++) if (r >= M) bfrag[0][v] = u32x4{0u, 0u, 0u, 0u};
      multiply(bfrag[0], 0);
    }
    finish_stage();
  };
  if constexpr (XS) {
    for (long long s = 0; s < S; s++) xs_stage(s, xin);
  } else {
  for (long long s = 0; s < S; s++) {
    const long long after = S - 1 - s;
    qd_wait_vm((int)(after < nb - 2 ? after : nb - 2) * BASE);         // this wave's pieces of stage s have landed (later stages may be in flight)
    __syncthreads();                                                   // ... and everyone else's; everyone is done with stage s - 1
    if (pend_row0 >= 0) { store_tile(pend_row0, pend_par); pend_row0 = -1; }
    if (s + nb - 1 < S) issue_stage();                                 // into the ring position stage s - 1 was read from
    if (2 * cst + half < nslots) {                                     // (the slot exists: K may end inside the stage)
#pragma unroll
      for (int k = 0; k < SPW; k++) { if (NSS == 1 || cst == 0) multiply(bfrag[k], k); else multiply(bfrag[(NSS - 1) * SPW + k], k); }
    }
    finish_stage();
  }
  }
  if constexpr (XS) { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); pin_x(xin); }   // the last request is never used: it has arrived before the wave ends
  __syncthreads();
  if (pend_row0 >= 0) store_tile(pend_row0, pend_par);
}

static int qd_cu_count() {
  static int n = 0;
  if (!n) { int dev = 0; hipDeviceProp_t p; n = (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&p, dev) == hipSuccess) ? p.multiProcessorCount : 256; }
  return n;
}

template <int T, bool MS, int NSS, bool SW, int SU, bool XS = false, bool XF = false>
static int launch_qd_k(const QArgs& a, int M, int nb, int per_cu, size_t lds, hipStream_t s) {
  auto kern = qgemm_dma_kernel<T, MS, NSS, SW, SU, XS, XF>;
  static const hipError_t configured = [&]() {
    hipFuncAttributes fa;
    hipError_t e = hipFuncGetAttributes(&fa, (const void*)kern);
    if (e != hipSuccess) return e;
    return hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)(QD_LDS_CU - fa.sharedSizeBytes));
  }();
  TGA_HIP(configured);
  const long long ngroups = SW ? a.n[0] / 8 : a.ntot / 16;
  const long long cap = (long long)qd_cu_count() * per_cu;
  const long long grid = ngroups < cap ? ngroups : cap;
  kern<<<dim3((unsigned)grid), dim3(QD_NW * 64), lds, s>>>(a, M, nb);
  TGA_LAUNCH_CHECK();
  return 0;
}

template <int T, int SU>
static int launch_qd_su(QArgs a, int M, hipStream_t s) {
  using F = Fmt<T>;
  constexpr int STAGE_BYTES = 2 * ((16 * (DmaFmt<T>::pieces(SU) + DmaFmt<T>::PAD) + 63) / 64) * 1024;
  constexpr int per_cu = 1;                                           // one workgroup per CU (two, each with half the ring, were no faster: 17.4 against 14.9 us on Q4_0 14336 x 4096)
  int nb = (int)((QD_LDS_CU / per_cu - (long long)sizeof(float) * 2 * QD_NW * 16 * 17 - 1024) / STAGE_BYTES);
  if (nb > QD_MAX_NB) nb = QD_MAX_NB;                                 // (deeper rings were measured: no faster at four stages, slower at seven)
  if (nb < 2) return -1;
  size_t lds = (size_t)nb * STAGE_BYTES;
  const size_t with_x = (size_t)(nb - 1) * STAGE_BYTES + (size_t)QD_NW * 8192;   // the activations pass through the last ring position and what follows it
  if (with_x > lds) lds = with_x;
  if (lds > (size_t)QD_LDS_CU - sizeof(float) * 2 * QD_NW * 16 * 17 - 1024) return -1;
  if constexpr (T == GGML_Q6_K) {                                     // (one matrix, plain or residual epilogue: the lm-head and single linears)
    if (a.epilogue == 2 || a.nseg > 1) return -1;
    return launch_qd_k<T, false, 1, false, SU>(a, M, nb, per_cu, lds, s);
  } else if constexpr (T == GGML_F16) {                               // (plain or residual epilogue, one to three matrices)
    if (a.epilogue == 2) return -1;
    const bool two = a.K > 2 * F::UW * SU;
    if (a.nseg > 1) return two ? launch_qd_k<T, true, 2, false, SU>(a, M, nb, per_cu, lds, s) : launch_qd_k<T, true, 1, false, SU>(a, M, nb, per_cu, lds, s);
    return two ? launch_qd_k<T, false, 2, false, SU>(a, M, nb, per_cu, lds, s) : launch_qd_k<T, false, 1, false, SU>(a, M, nb, per_cu, lds, s);
  } else if constexpr (SU == 32) {                                    // K <= 4096: at most two slots, one stage per row group
    if (a.epilogue == 2) return launch_qd_k<T, false, 1, true, SU>(a, M, nb, per_cu, lds, s);
    if (a.nseg > 1) return launch_qd_k<T, true, 1, false, SU>(a, M, nb, per_cu, lds, s);
    return launch_qd_k<T, false, 1, false, SU>(a, M, nb, per_cu, lds, s);
  } else {
    const bool two = a.K > 2 * F::UW * SU;
    if (a.epilogue == 2) return two ? launch_qd_k<T, false, 2, true, SU>(a, M, nb, per_cu, lds, s) : launch_qd_k<T, false, 1, true, SU>(a, M, nb, per_cu, lds, s);
    if (a.nseg > 1) return two ? launch_qd_k<T, true, 2, false, SU>(a, M, nb, per_cu, lds, s) : launch_qd_k<T, true, 1, false, SU>(a, M, nb, per_cu, lds, s);
    return two ? launch_qd_k<T, false, 2, false, SU>(a, M, nb, per_cu, lds, s) : launch_qd_k<T, false, 1, false, SU>(a, M, nb, per_cu, lds, s);
  }
}

// K > 4096: activations streamed beside the weights (one matrix, plain or residual epilogue)
template <int T>
static int launch_qd_xs(const QArgs& a, int M, hipStream_t s) {
  constexpr int SU = 16;
  constexpr int STAGE_BYTES = 2 * ((16 * (DmaFmt<T>::pieces(SU) + DmaFmt<T>::PAD) + 63) / 64) * 1024;
  const long long xt_bytes = (long long)QD_NW * (M > 8 ? 16 : 8) * QD_XT_PITCH;
  int nb = (int)((QD_LDS_CU - (long long)sizeof(float) * 2 * QD_NW * 16 * 17 - 1024 - xt_bytes) / STAGE_BYTES);
  if (nb > QD_MAX_NB) nb = QD_MAX_NB;
  if (nb < 2) return -1;
  const size_t lds = (size_t)nb * STAGE_BYTES + (size_t)xt_bytes;
  return a.x_f32 ? launch_qd_k<T, false, 1, false, SU, true, true>(a, M, nb, 1, lds, s) : launch_qd_k<T, false, 1, false, SU, true, false>(a, M, nb, 1, lds, s);
}

template <int T>
static int launch_qd(QArgs a, int M, hipStream_t s) {
  using F = Fmt<T>;
  a.nu = a.K / F::UW;
  a.row_bytes = (long long)(a.K / F::BW) * F::BB;
  if constexpr (T == GGML_Q6_K) {                                        // slots of 32 units (8 superblocks = 1680 bytes: whole 16-byte pieces), K = 2048 or 4096
    if (a.K % (F::UW * 32) != 0) return -1;
    if (a.K > 2 * F::UW * 32) {                                          // beyond 4096: slots of 16 units with the activations streamed beside them (beyond eight rows the ring holds two stages: 4096 x 14336 at 16 rows 27 us, as two launches of eight 47)
      if (a.nseg != 1 || a.epilogue > 1) return -1;
      return launch_qd_xs<T>(a, M, s);
    }
    return launch_qd_su<T, 32>(a, M, s);
  } else if constexpr (T == GGML_F16) {
    if (a.K % (F::UW * 16) != 0 || a.K > 4 * F::UW * 16) return -1;      // whole slots of 16 units (2 KB per row), K <= 4096
    return launch_qd_su<T, 16>(a, M, s);
  } else if constexpr (T == GGML_Q4_K || T == GGML_Q5_K) {
    if (a.K % (F::UW * 16) != 0) return -1;                              // whole slots of 16 units (4 superblocks)
    if (a.K > 4 * F::UW * 16) {
      if (a.nseg != 1 || a.epilogue > 1) return -1;
      return launch_qd_xs<T>(a, M, s);
    }
    // Q4_K: slots of 32 units (K = 2048 or 4096); Q5_K: of 16 (three stages of 32 units and the activations' way through LDS do not fit beside each other)
    if constexpr (T == GGML_Q4_K) { if (a.K % (F::UW * 32) != 0) return -1; return launch_qd_su<T, 32>(a, M, s); }
    else return launch_qd_su<T, 16>(a, M, s);
  } else {
    if (a.K % (F::UW * 16) != 0) return -1;                              // whole slots of 16 units
    if (a.K > 4 * F::UW * 16) {
      if (a.nseg != 1 || a.epilogue > 1) return -1;
      return launch_qd_xs<T>(a, M, s);
    }
    // Q4_0: slots of 32 units where K is whole in them (1152-byte runs, one stage per row group: 14336 x 4096 at M = 4 / 8 14.7 / 15.6 -> 13.5 / 14.4 us);
    // Q8_0 keeps 16 (1088-byte runs already; with 32 the ring holds two stages only: 17.6 / 18.3 against 17.0 / 18.0 us)
    if constexpr (T == F_Q4_0P) { if (a.K % (F::UW * 32) == 0) return launch_qd_su<T, 32>(a, M, s); }
    return launch_qd_su<T, 16>(a, M, s);
  }
}

// Returns -1 when the call is outside this kernel's range (the caller then takes the register-fed MFMA kernel): 2 <= M <= 16, every matrix a multiple of
// 16 rows at a 16-byte aligned address (8 rows for the SwiGLU pair);
// Q4_0 / Q8_0 / Q4_1 / Q5_0 / Q5_1 block pairs: K = 1024, 2048, 3072 or 4096 (larger multiples of 1024 for one matrix); Q4_K / Q5_K: K = 2048 or 4096 (Q5_K: and 1024, 3072), larger
// multiples of 1024 for one matrix; Q6_K: one matrix, K a multiple of 2048; fp16 weights: K <= 4096, no SwiGLU pair.
int tga_qgemm_wp_dispatch(int fmt, const QArgs& a, int M, hipStream_t s);   // qgemm_wp.hip: the same call on wave-private rings (Q8_0, K = 2048 / 4096), -1 outside its range
// what both kernels ask of a call: 2 <= M <= 16, every matrix whole row groups at a 16-byte aligned address, float32 rows where a norm folds in
static bool qd_call_ok(const QArgs& a, int M) {
  if (M < 2 || M > 16 || a.nseg < 1 || a.nseg > 3 || a.epilogue > 2 || a.sel || a.x_staged || a.y_stage_fmt) return false;
  if (a.norm_w && (!a.x_f32 || a.K > 4096 || ((uintptr_t)a.norm_w & 15) != 0)) return false;      // the folded norm: float32 rows that the workgroup's operands cover whole
  if (((uintptr_t)a.x & 15) != 0) return false;
  if (a.epilogue == 2) return a.w[1] && a.n[0] % 8 == 0 && a.n[0] > 0 && (((uintptr_t)a.w[0] | (uintptr_t)a.w[1]) & 15) == 0;   // silu(gate) * up: two matrices of equal shape, eight rows of each per row group
  for (int i = 0; i < a.nseg; i++) if (a.n[i] % 16 != 0 || a.n[i] <= 0 || ((uintptr_t)a.w[i] & 15) != 0) return false;
  return true;
}
// the wave-private kernel or nothing (two rows of a large Q8_0 matrix: there the barrier kernel is slower than the single-row kernel's two-row walk, this one is not)
int tga_qgemm_wp_checked_dispatch(int fmt, const QArgs& a, int M, hipStream_t s) { return qd_call_ok(a, M) ? tga_qgemm_wp_dispatch(fmt, a, M, s) : -1; }
int tga_qgemm_dma_dispatch(int fmt, const QArgs& a, int M, hipStream_t s) {
  if (fmt != F_Q4_0P && fmt != F_Q8_0P && fmt != GGML_Q6_K && fmt != GGML_F16 && fmt != GGML_Q4_K && fmt != GGML_Q5_K && fmt != GGML_Q4_1 && fmt != GGML_Q5_0 && fmt != GGML_Q5_1) return -1;
  if (!qd_call_ok(a, M)) return -1;
  if (const int rc = tga_qgemm_wp_dispatch(fmt, a, M, s); rc >= 0) return rc;
  if (a.epilogue == 2) {
    switch (fmt) {
      case F_Q4_0P: return launch_qd<F_Q4_0P>(a, M, s);
      case F_Q8_0P: return launch_qd<F_Q8_0P>(a, M, s);
      case GGML_Q4_K: return launch_qd<GGML_Q4_K>(a, M, s);
      case GGML_Q5_K: return launch_qd<GGML_Q5_K>(a, M, s);
      case GGML_Q4_1: return launch_qd<GGML_Q4_1>(a, M, s);
      case GGML_Q5_0: return launch_qd<GGML_Q5_0>(a, M, s);
      case GGML_Q5_1: return launch_qd<GGML_Q5_1>(a, M, s);
    }
    return -1;
  }
  switch (fmt) {
    case F_Q4_0P: return launch_qd<F_Q4_0P>(a, M, s);
    case F_Q8_0P: return launch_qd<F_Q8_0P>(a, M, s);
    case GGML_Q6_K: return launch_qd<GGML_Q6_K>(a, M, s);
    case GGML_Q4_K: return launch_qd<GGML_Q4_K>(a, M, s);
    case GGML_Q5_K: return launch_qd<GGML_Q5_K>(a, M, s);
    case GGML_Q4_1: return launch_qd<GGML_Q4_1>(a, M, s);
    case GGML_Q5_0: return launch_qd<GGML_Q5_0>(a, M, s);
    case GGML_Q5_1: return launch_qd<GGML_Q5_1>(a, M, s);
  }
  return launch_qd<GGML_F16>(a, M, s);
}
