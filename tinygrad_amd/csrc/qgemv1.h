// M = 1 dequant-GEMV fast path (decode): see qgemv.hip for the overall design.  This header holds the kernel and its launch
// templates; qgemv1_*.hip instantiate them per weight format (separate translation units compile in parallel).
#pragma once
#include "qfmt.h"
#include "host.h"
#include "moe_gate.h"

#ifndef QG1_WR
#define QG1_WR 8           // row teams (waves) per workgroup when one wave covers a row: one workgroup per CU
#endif
#ifndef QG1_DEPTH
#define QG1_DEPTH 3        // row groups in flight per lane: the loads of the next DEPTH - 1 groups are outstanding while one is multiplied
#endif

// ------------------------------------------------------------------------------------------------ M = 1 fast path
// One activation row: each lane keeps the activations of ITS unit in registers for the whole kernel (no LDS traffic in the
// loop).  A workgroup is WR x WK waves: the WK waves of a row team split K (wave wk owns units 64wk .. 64wk+63) and their
// partial sums meet in LDS once per row group (the only LDS use in the loop: split-K partials); the WR teams own disjoint
// row ranges.  Each team walks its row groups with a register ring of QG1_DEPTH groups.
// Which row groups a team owns.  A CU's vector memory pipeline returns data in request order, so everything a wave asks for waits behind what
// the waves that reached the CU before it have asked for.  Measured with per-wave clock stamps on the 2 x 14336 x 4096 gate/up launch with two
// 4-wave workgroups per CU: the workgroup that arrives second starts 0.2 us later, but holds its activations 1.4 us later, its first weights 2.9 us
// later and ends 2.4 us later than the first (1.3 us on the 4096 x 14336 down projection).  Hence: (a) rows that one wave covers run as ONE 8-wave
// workgroup per CU (QG1_WR) whose waves all hold their activations before any of them asks for weights (prologue 1); (b) where two workgroups per
// CU remain (K split over the waves), the first pass of workgroups owns team_skew row groups more and the second pass as many fewer; (c) a
// launch over one matrix interleaves its teams (team t owns groups t, t + teams, ...), so that the whole chip walks one contiguous window.
// Activations reach the registers through one LDS transpose per workgroup: coalesced 16-byte global loads of the plain row,
// then each lane reads back the 64 (or 32) values of its unit (unit stride padded to spread LDS banks).
// H (rows of at most 32 units, WK = 1): a row occupies half a wave, so each half-wave is a row team of its own (lanes 0-31 and
// 32-63 walk different row ranges; the DPP sum stops at 32 lanes) instead of leaving half of the lanes without loads.
//
// EVERY LOAD IS ISSUED UNCONDITIONALLY, in straight-line code (rows and units clamped to valid ones, surplus results dropped; the
// residual of the epilogue travels with its row group): the compiler places s_waitcnt from a per-path count of outstanding loads and
// takes the most conservative count where paths join, so a load (or a store: they share the counter) inside a branch turns the
// waits behind the join into "wait for everything" and the ring into a one-deep pipeline.  For the same reason the prologue kind
// is a template parameter: with the activation format known at compile time the prologue is one basic block in which the small
// activation reads go out first, the first weight loads second (loads return in issue order; prologue 1 holds them back until the
// workgroup's sum of squares is complete, i.e. until every wave has its activations), and the staging arithmetic runs while the weights
// are in flight.
//   PRO 0  generic: flags read at run time (any activation type, any K); weights first, then the staging loops
//   PRO 1  one float32 row of at most two 8-element pieces per thread with the RMSNorm folded in (kept in registers between the sum of
//          squares and the scaling)
//   PRO 2  activations already in the staged order of this format (written by the producing kernel)
//   PRO 3  one fp16 row of at most two pieces per thread
//   PRO 6  PRO 3 for the expert gate/up jobs of one token with the gating done here: every workgroup computes scores and top-k from the
//          router logits itself (64..1024 floats), so no selection has to cross workgroups inside the router's launch
//   PRO 8  PRO 1 of the q / k / v launch of a decode step with a hint for the attention launch behind it: every lane also reads one dword of a cache
//          line that the attention will ask for (kv_touch)
//   PRO 7  the row is merged from the attention's split partials (one 8-element piece per thread), so the attention has no merge launch
//   PRO 5  PRO 1 for a row of at most one piece per thread that is first completed as x + sum_j p_j y_j (the MoE weighted sum and block
//          residual that precede the next block's attn_norm): the launch that would only add vectors disappears
//
// MR > 1 (several activation rows; instantiated for two; generic prologue, no fused SwiGLU): the same walk over the weights with MR sets of activations in registers;
// a unit is decoded once and multiplied with every row.  Outputs and residuals are (MR, rows) per matrix.
// bx: the workgroup's index among those of this matrix set (blockIdx.x where a launch serves one set, see qgemv1_two_kernel)
// Eight values of one head's attention row from its S split partials: ph = [S][hd] weighted V sums, then (max, sum) pairs of the S splits (six pairs, then
// four floats of padding); merged = sum_s e_s o_s / sum_s e_s l_s with e_s = exp(m_s - max m).
template <int S>
__device__ __forceinline__ void attn_merge_piece(const float* ph, int hd, int d0, f32x4& l, f32x4& h) {
  f32x4 pl[S], phh[S], ml[3];
#pragma unroll
  for (int sp = 0; sp < S; sp++) { pl[sp] = gld16f(ph + sp * hd + d0); phh[sp] = gld16f(ph + sp * hd + d0 + 4); }
#pragma unroll
  for (int j = 0; j < (S + 1) / 2; j++) ml[j] = gld16f(ph + S * hd + 4 * j);
  float pm[S], pls[S];
#pragma unroll
  for (int sp = 0; sp < S; sp++) { pm[sp] = (sp & 1) ? ml[sp >> 1].z : ml[sp >> 1].x; pls[sp] = (sp & 1) ? ml[sp >> 1].w : ml[sp >> 1].y; }
  float mx = pm[0];
#pragma unroll
  for (int sp = 1; sp < S; sp++) mx = fmaxf(mx, pm[sp]);
  l = f32x4{0.f, 0.f, 0.f, 0.f}; h = f32x4{0.f, 0.f, 0.f, 0.f};
  float lsum = 0.f;
#pragma unroll
  for (int sp = 0; sp < S; sp++) {
    const float e = pm[sp] != -INFINITY ? __expf(pm[sp] - mx) : 0.f;
    lsum += e * pls[sp];
    l.x += e * pl[sp].x; l.y += e * pl[sp].y; l.z += e * pl[sp].z; l.w += e * pl[sp].w;
    h.x += e * phh[sp].x; h.y += e * phh[sp].y; h.z += e * phh[sp].z; h.w += e * phh[sp].w;
  }
  const float inv = 1.0f / lsum;
  l.x *= inv; l.y *= inv; l.z *= inv; l.w *= inv; h.x *= inv; h.y *= inv; h.z *= inv; h.w *= inv;
}

// One dword of one line per lane for the attention launch that follows a q / k / v launch (QArgs::touch_*, prologue 8), branch-free: beyond the lines
// there are a lane reads the last one again.  Workgroup bx runs on XCD bx % 8; the attention workgroups of kv head h run on
// XCD h % 8 when the number of kv heads is a multiple of 8 (the host only asks then).  Lines of an XCD: K rows [0, pos) and V rows [0, pos) of each of its
// heads, then the rotation row of pos; thread t of the XCD's workgroups takes line t.
template <int NT>
__device__ __forceinline__ uint32_t kv_touch(const QArgs& a, const unsigned bx, int pos) {
  pos = pos < 0 ? 0 : pos > a.touch_max_ctx - 1 ? a.touch_max_ctx - 1 : pos;
  const int x = bx & 7, t = (int)(bx >> 3) * NT + (int)threadIdx.x;
  const int npl = (pos * a.touch_row_bytes + 127) >> 7;            // lines of the K (or V) rows below pos of one head
  const int heads = (a.touch_n_kv - x + 7) >> 3, nrope = (a.touch_rope_row_bytes + 127) >> 7;
  const int nkv = heads * 2 * npl, total = nkv + nrope;
  const int idx = t < total ? t : total - 1;
  const int hk = idx / (npl > 0 ? npl : 1), line = idx - hk * npl;
  // (addresses by arithmetic, not by selects of pointers: a select between computed pointers can come out as a branch around the load, and a load
  // behind a branch makes the compiler wait for every load in flight where the paths join)
  const uintptr_t kb = (uintptr_t)a.touch_k, vb = (uintptr_t)a.touch_v;
  const uintptr_t kvb = kb ^ ((kb ^ vb) & (uintptr_t)0 - (uintptr_t)(hk & 1));
  const uintptr_t kvp = kvb + ((size_t)(x + 8 * (hk >> 1)) * a.touch_max_ctx * a.touch_row_bytes) + ((size_t)line << 7);
  const uintptr_t rp = (uintptr_t)a.touch_rope + (size_t)pos * a.touch_rope_row_bytes + ((size_t)(idx >= nkv ? idx - nkv : 0) << 7);
  const uintptr_t p = kvp ^ ((kvp ^ rp) & (uintptr_t)0 - (uintptr_t)(idx >= nkv));
  return *(const __attribute__((address_space(1))) uint32_t*)p;   // (a global load: a flat one from an integer address would also count as an LDS operation)
}

template <int T, int R, int WK, int WR, int EPI, bool H, int PRO, int MR = 1>
__device__ __forceinline__ void qgemv1_body(const QArgs& args, const unsigned bx) {
  static_assert(MR == 1 || PRO == 0, "several activation rows: generic prologue");
  // A local copy: its field reads become kernel-argument loads in the entry block, where they merge into a few wide scalar loads
  // issued together (read at their points of use they arrive in dependent stages, each a scalar-cache miss of its own).
  const QArgs a = args;
  int tpos = 0;
  if constexpr (PRO == 8) tpos = *a.touch_pos;                    // (read at the kernel's entry: a scalar load whose miss the prologue hides)
  using F = Fmt<T>;
  typedef typename F::Raw Raw;
  static_assert(WK == 1 || WR == 1, "row teams and K split are not combined");
  static_assert(!H || WK == 1, "half-wave rows need the whole row inside one wave");
  constexpr int HM = H ? 2 : 1;
  constexpr int NT = WK * WR * 64;
  constexpr int NP = F::UW / 2;                                  // dwords (fp16 pairs) per unit
  constexpr int USTRIDE = NP + 4;                                // padded unit stride in dwords
  // Ring depth per launch kind, each measured in the 8B decode step: the SwiGLU pair and the residual epilogue over rows that one wave covers
  // are faster with two row groups per lane (gate/up 15.8 -> 15.0 us, attn_output 5.45 -> 5.26 us), the plain epilogue and the split-K launches
  // with three (q/k/v 8.2 against 8.6 us, down 9.6 against 10.5 us); four is slower everywhere (578 against 607 tok/s).
  constexpr int D = (WK == 1 && !H && EPI != 0) ? 2 : QG1_DEPTH;
  constexpr int NPC = (NT >= 512) ? 1 : 2;                        // 8-element activation pieces per thread in prologues 1 and 3 (rows of at most 8 NT NPC values)
  extern __shared__ uint32_t xlds[];                             // nu * USTRIDE dwords
  __shared__ float part[2][WK][R * MR];
  __shared__ float nred[NT / 64];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wk = (WK > 1) ? wave : 0, wr = (WK > 1) ? 0 : wave;
  const int hl = H ? (lane & 31) : lane, hrow = H ? (lane >> 5) : 0;
  const int u = wk * 64 + hl;
  const bool uvalid = u < a.nu;
  const int uc = uvalid ? u : a.nu - 1;
  const int job = blockIdx.y;
  long long eoff = (a.sel && PRO != 6) ? (long long)a.sel[job] * a.estride : 0;
  const long long yofs = (long long)job * a.ystride;
  const long long xrow = a.sel ? job / a.xdiv : 0;
  constexpr int RS = (EPI == 2) ? 1 : R;                         // output rows per row group
  const long long team = ((long long)bx * WR + wr) * HM + hrow;
  const long long gbase = a.team_base, grem = a.team_rem;       // ngroups / teams and ngroups % teams, from the host
  // (half-wave teams keep equal contiguous ranges and a compile-time row step: their row numbers live in vector registers, where a run-time
  // step turns every load address into 64-bit vector arithmetic - 0.6 us on the 2048-wide fp16 launches of the MoE decode step)
  const long long nfirst = H ? 0 : a.team_first, sk = H ? 0 : a.team_skew;
  const long long g0 = team * gbase + (team < grem ? team : grem) + sk * (team < nfirst ? team : 2 * nfirst - team);
  const long long g1 = g0 + gbase + (team < grem ? 1 : 0) + (team < nfirst ? sk : -sk);
  const long long row_lo = g0 * RS, row_hi = g1 * RS < a.ntot ? g1 * RS : a.ntot;
  const long long rstep = (!H && a.team_stride) ? (long long)a.team_stride * RS : RS;     // rows from one row group of the team to its next
  uint32_t kc[F::NKC];
  F::consts(kc);
  u32x4 xv[MR][F::XV]; float cv[MR][F::NG];
  const int nseg = (EPI == 2) ? 1 : a.nseg;
  int parity = 0;
  uint32_t touched = 0;                                          // (prologue 8: the dword of the cache line this lane touches for the attention launch, see kv_touch)

  // ---- the segment (weight matrix) the team is in
  int seg = 0;
  long long seg_start = 0, lo = 0, hi = 0, cnt = 0, last = 0, seg_n = 0;
  const uint8_t *base0 = nullptr, *base1 = nullptr;
  const float* resid = nullptr;
  auto enter = [&](int sg) {
    seg = sg;
    if (sg == 0) seg_start = 0;
    const long long seg_rows = a.n[sg];
    seg_n = seg_rows;
    lo = row_lo - seg_start; hi = row_hi - seg_start;
    if (lo < 0) lo = 0;
    if (hi > seg_rows) hi = seg_rows;
    seg_start += seg_rows;
    cnt = hi > lo ? (hi - lo + RS - 1) / RS : 0;                 // row groups of this team inside the segment
    if (!H && a.team_stride) {                                   // interleaved teams (one matrix): groups team, team + stride, ...
      lo = team * RS; hi = seg_rows;
      cnt = gbase + (team < grem ? 1 : 0);                       // the stride is the number of teams: team_base groups each, one more for the first team_rem (no division here)
    }
    last = hi > 0 ? hi - 1 : 0;                                  // rows beyond the range reload this one (always a valid row)
    base0 = a.w[sg] + eoff;
    base1 = ((EPI == 2) ? a.w[1] : a.w[sg]) + eoff;
    if constexpr (EPI == 1) resid = a.resid[sg] + yofs;
  };
  struct Grp { Raw w[R]; float res[R * MR]; };
  auto issue = [&](Grp& g, long long row) {
#pragma unroll
    for (int r = 0; r < R; r++) {
      long long rr = (EPI == 2) ? row : row + r;
      rr = rr < last ? rr : last;
      const uint8_t* rp = ((EPI == 2 && r == 1) ? base1 : base0) + rr * a.row_bytes;
      if constexpr (T == GGML_F16) g.w[r] = F::load_nu(rp, uc, a.nu); else g.w[r] = F::load(rp, uc);
    }
    if constexpr (EPI == 1) {
      if constexpr (WK > 1) {                                      // wave 0, lane m R + r stores row + r of activation row m
        const int lm = lane < R * MR ? lane / R : 0, lr = lane < R * MR ? lane % R : 0;
        long long rr = row + lr; rr = rr < last ? rr : last; g.res[0] = resid[lm * seg_n + rr];
      } else {
#pragma unroll
        for (int m = 0; m < MR; m++) {
#pragma unroll
          for (int r = 0; r < R; r++) { long long rr = row + r; rr = rr < last ? rr : last; g.res[m * R + r] = resid[m * seg_n + rr]; }
        }
      }
    }
  };
  // multiply, reduce and store one row group
  auto finish_group = [&](const Grp& g, long long row) {
    float acc[MR][R];
#pragma unroll
    for (int r = 0; r < R; r++) {
      float am[MR];
#pragma unroll
      for (int m = 0; m < MR; m++) am[m] = 0.f;
      if constexpr (MR == 1) unit_dot_reg<T>(g.w[r], xv[0], cv[0], am[0], kc);
      else unit_dot_reg_m<T, MR>(g.w[r], xv, cv, am, kc);
#pragma unroll
      for (int m = 0; m < MR; m++) acc[m][r] = H ? half_sum_lane31(uvalid ? am[m] : 0.f) : wave_sum_lane63(uvalid ? am[m] : 0.f);
    }
    if constexpr (WK > 1) {
      if (lane == 63) {
#pragma unroll
        for (int m = 0; m < MR; m++) {
#pragma unroll
          for (int r = 0; r < R; r++) part[parity][wave][m * R + r] = acc[m][r];
        }
      }
      __syncthreads();
      if (wave == 0) {
        float t = 0.f;
        if (lane < R * MR) {
#pragma unroll
          for (int j = 0; j < WK; j++) t += part[parity][j][lane];
        }
        if constexpr (EPI == 2) {                               // lane 2 m holds the gate sum of activation row m, lane 2 m + 1 its up sum
          const float up = __shfl(t, lane + 1, 64);
          if (lane < R * MR && (lane & 1) == 0) store_swiglu(a, row, t, up, yofs + (lane >> 1) * seg_n);
        } else {
          if constexpr (EPI == 1) t += g.res[0];
          const int lm = lane / R, lr = lane % R;
          if (lane < R * MR && row + lr < hi) store_one<0>(a, seg, row + lr, t, yofs + lm * seg_n);
        }
      }
      parity ^= 1;
    } else {
      if (hl == (H ? 31 : 63)) {
        if constexpr (EPI == 2) {
#pragma unroll
          for (int m = 0; m < MR; m++) store_swiglu(a, row, acc[m][0], acc[m][R - 1], yofs + m * seg_n);
        } else {
#pragma unroll
          for (int m = 0; m < MR; m++) {
#pragma unroll
            for (int r = 0; r < R; r++) if (row + r < hi) store_one<0>(a, seg, row + r, EPI == 1 ? acc[m][r] + g.res[m * R + r] : acc[m][r], yofs + m * seg_n);
          }
        }
      }
    }
  };
  Grp b[D];                                                      // ring of row groups in flight
  // walks the team's row groups of the current segment; group lo is already in flight in b[0]
  auto run_segment = [&]() {
#pragma unroll
    for (int d = 1; d < D - 1; d++) issue(b[d], lo + (long long)d * rstep);
    long long row = lo, g = 0;
    for (; g + D <= cnt; g += D) {
#pragma unroll
      for (int d = 0; d < D; d++) {
        issue(b[(d + D - 1) % D], row + (long long)(D - 1) * rstep);        // the slot freed by the previous group
        finish_group(b[d], row);
        row += rstep;
      }
    }
    // fewer than D groups left: their loads are already in flight (slots 0 .. D - 2), nothing more to issue
#pragma unroll
    for (int d = 0; d < D - 1; d++) {
      if (g + d < cnt) finish_group(b[d], row);                  // (split K: the waves of a workgroup share cnt, so the barrier inside is uniform)
      row += rstep;
    }
  };

  enter(0);
  const int nq = a.K / 8;                                        // 16-byte fp16 pieces in the row
  const f32x4* xr = (const f32x4*)((const float*)a.x + xrow * a.K);
  const u32x4* xh = (const u32x4*)((const uint16_t*)a.x + xrow * a.K);
  auto lds_to_regs = [&]() {
    __syncthreads();
#pragma unroll
    for (int m = 0; m < MR; m++) {
      uint32_t nx[NP];
#pragma unroll
      for (int k = 0; k < NP; k += 4) { const u32x4 v = *(const u32x4*)(xlds + (m * a.nu + uc) * USTRIDE + k); nx[k] = v.x; nx[k + 1] = v.y; nx[k + 2] = v.z; nx[k + 3] = v.w; }
      F::stage(nx, xv[m], cv[m]);
    }
  };
  // piece i (elements 8i .. 8i+7 as 4 fp16 pairs) into LDS: unit F::unit_of(8i) at pair F::pair_of(8i) (4 consecutive pairs stay inside one unit run)
  auto put_piece = [&](int i, const u32x4& v, int m = 0) {
    if constexpr (T == GGML_F16) *(u32x4*)(xlds + (m * a.nu + F::unit_of_nu(8 * i, a.nu)) * USTRIDE + F::pair_of_nu(8 * i, a.nu)) = v;
    else *(u32x4*)(xlds + (m * a.nu + F::unit_of(8 * i)) * USTRIDE + F::pair_of(8 * i)) = v;
  };
  auto pack8 = [](const f32x4& l, const f32x4& h) {
    u32x4 v;
    v.x = f2h_bits(l.x) | (f2h_bits(l.y) << 16); v.y = f2h_bits(l.z) | (f2h_bits(l.w) << 16);
    v.z = f2h_bits(h.x) | (f2h_bits(h.y) << 16); v.w = f2h_bits(h.z) | (f2h_bits(h.w) << 16);
    return v;
  };
  if constexpr (PRO == 2) {
    const u32x4* xs = (const u32x4*)a.x + xrow * (long long)F::XV * a.nu;
#pragma unroll
    for (int t = 0; t < F::XV; t++) xv[0][t] = xs[t * a.nu + uc];
    issue(b[0], lo);
    F::cfromx(xv[0], cv[0]);
  } else if constexpr (PRO == 5) {
    constexpr int CK = 8;                                        // rows of the weighted sum (fewer: the surplus ones reload row 0 with weight 0)
    const int i = (int)threadIdx.x < nq ? (int)threadIdx.x : nq - 1;
    f32x4 l = xr[2 * i], h = xr[2 * i + 1];
    const f32x4 w0 = ((const f32x4*)a.norm_w)[2 * i], w1 = ((const f32x4*)a.norm_w)[2 * i + 1];
    f32x4 yl[CK], yh[CK]; float pj[CK];
#pragma unroll
    for (int j = 0; j < CK; j++) {
      const int jc = j < a.comb_k ? j : 0;
      const f32x4* yr = (const f32x4*)(a.comb_y + (size_t)jc * a.K);
      yl[j] = yr[2 * i]; yh[j] = yr[2 * i + 1];
      pj[j] = a.comb_p[jc];
    }
#pragma unroll
    for (int j = 0; j < CK; j++) {
      const float p = j < a.comb_k ? pj[j] : 0.f;
      l.x += p * yl[j].x; l.y += p * yl[j].y; l.z += p * yl[j].z; l.w += p * yl[j].w;
      h.x += p * yh[j].x; h.y += p * yh[j].y; h.z += p * yh[j].z; h.w += p * yh[j].w;
    }
    if (bx == 0 && blockIdx.y == 0 && (int)threadIdx.x < nq) { ((f32x4*)a.comb_x_out)[2 * i] = l; ((f32x4*)a.comb_x_out)[2 * i + 1] = h; }
    float ss = (int)threadIdx.x < nq ? l.x * l.x + l.y * l.y + l.z * l.z + l.w * l.w + h.x * h.x + h.y * h.y + h.z * h.z + h.w * h.w : 0.f;
    ss = wave_sum(ss);
    if (lane == 0) nred[wave] = ss;
    __syncthreads();
    issue(b[0], lo);                                             // (as in prologue 1: weights once every wave holds its row)
    float tot = 0.f;
#pragma unroll
    for (int j = 0; j < NT / 64; j++) tot += nred[j];
    const float nscale = 1.0f / sqrtf(tot / (float)a.K + a.norm_eps);
    l.x = (l.x * nscale) * w0.x; l.y = (l.y * nscale) * w0.y; l.z = (l.z * nscale) * w0.z; l.w = (l.w * nscale) * w0.w;
    h.x = (h.x * nscale) * w1.x; h.y = (h.y * nscale) * w1.y; h.z = (h.z * nscale) * w1.z; h.w = (h.w * nscale) * w1.w;
    if ((int)threadIdx.x < nq) put_piece((int)threadIdx.x, pack8(l, h));
    lds_to_regs();
  } else if constexpr (PRO == 1 || PRO == 8) {
    f32x4 l4[2], h4[2], w0[2], w1[2];
#pragma unroll
    for (int t = 0; t < NPC; t++) {
      const int i = (int)threadIdx.x + NT * t < nq ? (int)threadIdx.x + NT * t : nq - 1;
      l4[t] = xr[2 * i]; h4[t] = xr[2 * i + 1];
      w0[t] = ((const f32x4*)a.norm_w)[2 * i]; w1[t] = ((const f32x4*)a.norm_w)[2 * i + 1];
    }
    float ss = 0.f;
#pragma unroll
    for (int t = 0; t < NPC; t++) {
      const f32x4 l = l4[t], h = h4[t];
      const float s8 = l.x * l.x + l.y * l.y + l.z * l.z + l.w * l.w + h.x * h.x + h.y * h.y + h.z * h.z + h.w * h.w;
      ss += ((int)threadIdx.x + NT * t < nq) ? s8 : 0.f;
    }
    ss = wave_sum(ss);
    if (lane == 0) nred[wave] = ss;
    __syncthreads();
    // the first weights go out only now, when every wave of the workgroup holds its activations: requested together with them, the weight
    // misses of the waves that started first sit in front of the activation reads of the waves that started last (8B decode 602 -> 609 tok/s)
    issue(b[0], lo);
    if constexpr (PRO == 8) touched = kv_touch<NT>(a, bx, tpos);
    float tot = 0.f;
#pragma unroll
    for (int j = 0; j < NT / 64; j++) tot += nred[j];
    const float nscale = 1.0f / sqrtf(tot / (float)a.K + a.norm_eps);
#pragma unroll
    for (int t = 0; t < NPC; t++) {
      f32x4 l = l4[t], h = h4[t];
      l.x = (l.x * nscale) * w0[t].x; l.y = (l.y * nscale) * w0[t].y; l.z = (l.z * nscale) * w0[t].z; l.w = (l.w * nscale) * w0[t].w;
      h.x = (h.x * nscale) * w1[t].x; h.y = (h.y * nscale) * w1[t].y; h.z = (h.z * nscale) * w1[t].z; h.w = (h.w * nscale) * w1[t].w;
      const int i = (int)threadIdx.x + NT * t;
      if (i < nq) put_piece(i, pack8(l, h));
    }
    lds_to_regs();
  } else if constexpr (PRO == 3) {
    u32x4 v[2];
#pragma unroll
    for (int t = 0; t < NPC; t++) v[t] = xh[(int)threadIdx.x + NT * t < nq ? (int)threadIdx.x + NT * t : nq - 1];
#pragma unroll
    for (int t = 0; t < NPC; t++) { const int i = (int)threadIdx.x + NT * t; if (i < nq) put_piece(i, v[t]); }
    __syncthreads();                                             // every wave holds its pieces: only now the first weights (as in prologue 1)
    issue(b[0], lo);
    lds_to_regs();
  } else if constexpr (PRO == 7) {
    // the row is the merge of the attention's split partials (attn_split1_kernel): thread t merges elements 8t .. 8t + 7 of its head; a split
    // without cached positions carries max = -inf, sum = 0.  One instantiation per number of splits, so that exactly its loads go out, as one batch.
    const int i = (int)threadIdx.x < nq ? (int)threadIdx.x : nq - 1;
    const int hd = 1 << a.attn_hd_log2, head = (8 * i) >> a.attn_hd_log2, d0 = 8 * i - (head << a.attn_hd_log2);
    const float* ph = (const float*)a.x + (size_t)head * (a.attn_S * hd + 16);
    f32x4 l, h;
    switch (a.attn_S) {
      case 1: attn_merge_piece<1>(ph, hd, d0, l, h); break; case 2: attn_merge_piece<2>(ph, hd, d0, l, h); break; case 3: attn_merge_piece<3>(ph, hd, d0, l, h); break;
      case 4: attn_merge_piece<4>(ph, hd, d0, l, h); break; case 5: attn_merge_piece<5>(ph, hd, d0, l, h); break; default: attn_merge_piece<6>(ph, hd, d0, l, h); break;
    }
    if ((int)threadIdx.x < nq) put_piece((int)threadIdx.x, pack8(l, h));
    __syncthreads();                                             // every wave holds its pieces: only now the first weights (as in prologue 3; requested
    issue(b[0], lo);                                             // in front of the partials they cost 2 % of the decode step)
    lds_to_regs();
  } else if constexpr (PRO == 6) {
    __shared__ float tk_lg[1024], tk_sc[1024], tk_tmp[192], tk_p[64];
    __shared__ int tk_sel[64];
    u32x4 v[2];
#pragma unroll
    for (int t = 0; t < 2; t++) v[t] = xh[(int)threadIdx.x + NT * t < nq ? (int)threadIdx.x + NT * t : nq - 1];
    // jobs xrow * k .. xrow * k + k - 1 belong to token xrow: every workgroup gates its own token
    const int slot = job - (int)xrow * a.route_k;
    for (int i = threadIdx.x; i < a.route_E; i += NT) tk_lg[i] = a.route_logits[xrow * a.route_E + i];
    __syncthreads();
    if (wave == 0) gate_topk_wave(tk_lg, a.route_E, a.route_k, a.route_gating, a.route_norm_topk, a.route_scale, tk_sel, tk_p, tk_sc, tk_tmp, lane);
    __syncthreads();
    eoff = (long long)tk_sel[slot] * a.estride;
    enter(0);                                                    // the weight bases of the selected expert
    if (bx == 0 && slot == 0 && (int)threadIdx.x < a.route_k) {
      a.sel[xrow * a.route_k + threadIdx.x] = tk_sel[threadIdx.x]; a.route_probs_out[xrow * a.route_k + threadIdx.x] = tk_p[threadIdx.x];
    }
    issue(b[0], lo);
#pragma unroll
    for (int t = 0; t < 2; t++) { const int i = (int)threadIdx.x + NT * t; if (i < nq) put_piece(i, v[t]); }
    lds_to_regs();
  } else {
    if (a.x_staged) {
      const u32x4* xs = (const u32x4*)a.x + xrow * (long long)F::XV * a.nu;
#pragma unroll
      for (int t = 0; t < F::XV; t++) xv[0][t] = xs[t * a.nu + uc];
      issue(b[0], lo);
      F::cfromx(xv[0], cv[0]);
    } else {
      issue(b[0], lo);
      // Loads of up to four (two) loop iterations are issued as one batch: a load per iteration would cost a memory round trip each.
      float nscale = 1.f;
      if (a.norm_w) {                                            // fused RMSNorm: sum of squares over the workgroup first
        float ss = 0.f;
        for (int p = threadIdx.x; p < 2 * nq; p += NT * 4) {
          f32x4 v[4];
#pragma unroll
          for (int t = 0; t < 4; t++) { const int i = p + NT * t; v[t] = xr[i < 2 * nq ? i : 2 * nq - 1]; }
#pragma unroll
          for (int t = 0; t < 4; t++) if (p + NT * t < 2 * nq) ss += v[t].x * v[t].x + v[t].y * v[t].y + v[t].z * v[t].z + v[t].w * v[t].w;
        }
        ss = wave_sum(ss);
        if (lane == 0) nred[wave] = ss;
        __syncthreads();
        float tot = 0.f;
#pragma unroll
        for (int j = 0; j < NT / 64; j++) tot += nred[j];
        nscale = 1.0f / sqrtf(tot / (float)a.K + a.norm_eps);
      }
      for (int m = 0; m < MR; m++) {
      const f32x4* xr_m = xr + (size_t)m * (a.K / 4);
      const u32x4* xh_m = xh + (size_t)m * (a.K / 8);
      for (int p = threadIdx.x; p < nq; p += NT * 2) {
        u32x4 v[2]; f32x4 lo4[2], hi4[2], w0[2], w1[2];
#pragma unroll
        for (int t = 0; t < 2; t++) {
          const int i = p + NT * t < nq ? p + NT * t : nq - 1;
          if (a.x_f32) {
            lo4[t] = xr_m[2 * i]; hi4[t] = xr_m[2 * i + 1];
            if (a.norm_w) { w0[t] = ((const f32x4*)a.norm_w)[2 * i]; w1[t] = ((const f32x4*)a.norm_w)[2 * i + 1]; }
          } else v[t] = xh_m[i];
        }
#pragma unroll
        for (int t = 0; t < 2; t++) {
          const int i = p + NT * t;
          if (i >= nq) break;
          if (a.x_f32) {
            f32x4 l = lo4[t], h = hi4[t];
            if (a.norm_w) {
              l.x = (l.x * nscale) * w0[t].x; l.y = (l.y * nscale) * w0[t].y; l.z = (l.z * nscale) * w0[t].z; l.w = (l.w * nscale) * w0[t].w;
              h.x = (h.x * nscale) * w1[t].x; h.y = (h.y * nscale) * w1[t].y; h.z = (h.z * nscale) * w1[t].z; h.w = (h.w * nscale) * w1[t].w;
            }
            v[t] = pack8(l, h);
          }
          put_piece(i, v[t], m);
        }
      }
      }
      lds_to_regs();
    }
  }
  run_segment();
  // (a branch around loads is harmless here: the ring is empty between segments)
  for (int sg = 1; sg < nseg; sg++) { enter(sg); if (cnt) { issue(b[0], lo); run_segment(); } }
  if constexpr (PRO == 8) asm volatile("" :: "v"(touched));      // the touch has to be a load that is used: an empty statement takes its register
}

template <int T, int R, int WK, int WR, int EPI, bool H, int PRO, int MR = 1>
__global__ __launch_bounds__(WK * WR * 64) void qgemv1_kernel(const QArgs args) { qgemv1_body<T, R, WK, WR, EPI, H, PRO, MR>(args, blockIdx.x); }

// Two sets of matrices of different block types over the same activation row in one launch (a Q4_K_M file keeps attn_v as Q6_K beside Q4_K attn_q / attn_k;
// tinygrad/llm/model.py:161-163 applies the three linears to one normalised row): the first `split` workgroups walk set a, the others set b.  Rows that one
// wave covers, plain epilogue.
// Behind the branch the compiler reads a set's fields from the kernel-argument segment where they are used: a dozen scalar loads, one after the other, each a
// scalar-cache miss of its own (9.5 us for the 8B shape).  The entry block therefore reads one dword of every 64-byte line of the segment - twelve independent loads,
// one miss time together - so that the later ones hit.  The loads are inline assembly with their wait inside the statement: written in the source (one field per
// line summed into an operand of an empty statement), they made the compiler allocate 256 registers and spill.
template <int TA, int TB, int R, int WR, int PRO>
__global__ __launch_bounds__(WR * 64) void qgemv1_two_kernel(const QArgs a, const QArgs b, const unsigned split) {
  static_assert(2 * sizeof(QArgs) + sizeof(unsigned) > 0x2c0 && 2 * sizeof(QArgs) + sizeof(unsigned) <= 0x300, "twelve lines of kernel arguments");
  {
    const auto ka = __builtin_amdgcn_kernarg_segment_ptr();
    int t0, t1, t2, t3, t4, t5, t6, t7, t8, t9, t10, t11;
    asm volatile("s_load_dword %0, %12, 0x0\n\ts_load_dword %1, %12, 0x40\n\ts_load_dword %2, %12, 0x80\n\ts_load_dword %3, %12, 0xc0\n\ts_load_dword %4, %12, 0x100\n\t"
                 "s_load_dword %5, %12, 0x140\n\ts_load_dword %6, %12, 0x180\n\ts_load_dword %7, %12, 0x1c0\n\ts_load_dword %8, %12, 0x200\n\ts_load_dword %9, %12, 0x240\n\t"
                 "s_load_dword %10, %12, 0x280\n\ts_load_dword %11, %12, 0x2c0\n\t"
                 "s_waitcnt lgkmcnt(0)"
                 : "=&s"(t0), "=&s"(t1), "=&s"(t2), "=&s"(t3), "=&s"(t4), "=&s"(t5), "=&s"(t6), "=&s"(t7), "=&s"(t8), "=&s"(t9), "=&s"(t10), "=&s"(t11) : "s"(ka) : "memory");
  }
  if (blockIdx.x < split) qgemv1_body<TA, R, 1, WR, 0, false, PRO>(a, blockIdx.x);
  else qgemv1_body<TB, R, 1, WR, 0, false, PRO>(b, blockIdx.x - split);
}

// ------------------------------------------------------------------------------------------------ host side
static int fast_cu_count() {
  static int n = 0;
  if (!n) { int dev = 0; hipDeviceProp_t p; n = (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&p, dev) == hipSuccess) ? p.multiProcessorCount : 256; }
  return n;
}

template <int T, int R, int WK, int WR, int EPI, bool H, int PRO, int MR = 1>
static int launch_fast_p(const QArgs& a, long long grid, size_t lds, hipStream_t s) {
  auto kern = qgemv1_kernel<T, R, WK, WR, EPI, H, PRO, MR>;
  if (lds > 48 * 1024) {
    // once per instantiation; the initialisation of a function-local static is serialised by the language, so concurrent first calls are safe
    static const hipError_t configured = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, 150 * 1024 - fmt_tab<Fmt<T>>());
    TGA_HIP(configured);
  }
  kern<<<dim3((unsigned)grid, (unsigned)(a.sel ? a.xdiv_jobs : 1)), dim3(WK * WR * 64), lds, s>>>(a);
  TGA_LAUNCH_CHECK();
  return 0;
}

template <int T, int R, int WK, int WR, int EPI, bool H = false, int MR = 1>
static int launch_fast(QArgs a, hipStream_t s) {
  using F = Fmt<T>;
  constexpr int RS = (EPI == 2) ? 1 : R;
  constexpr int NT = WK * WR * 64;
  const long long ngroups = (a.ntot + RS - 1) / RS;
  const size_t lds = (size_t)MR * a.nu * (F::UW / 2 + 4) * 4;
  // row teams per CU: 8 waves (one 8-wave workgroup or two 4-wave ones), fewer when the staged activations in LDS (160 KB per CU) say so.
  // Measured on the 8B decode step: 8 or 12 waves per CU 570 tok/s, 16 (all wave slots) 564, 4 553.
  int wg_per_cu = (a.sel ? 16 : 8) / (WK * WR); if (wg_per_cu < 1) wg_per_cu = 1;   // (expert jobs share the grid: all 16 wave slots there)
  const int by_lds = (int)((160 * 1024) / (lds + 1024 + fmt_tab<F>())); if (wg_per_cu > by_lds) wg_per_cu = by_lds < 1 ? 1 : by_lds;
  constexpr int TPW = WR * (H ? 2 : 1);                           // row teams per workgroup
  long long max_teams = (long long)fast_cu_count() * wg_per_cu * TPW;
  if (a.sel && a.xdiv_jobs > 1) { max_teams = (max_teams + a.xdiv_jobs - 1) / a.xdiv_jobs; if (max_teams < 1) max_teams = 1; }
  long long per = (ngroups + max_teams - 1) / max_teams;           // row groups per team
  // short rows: a team should own a few row groups, so that the activation staging of its workgroup is paid once per several
  // rows, as long as every CU still gets a workgroup
  long long per_min = ngroups / ((long long)fast_cu_count() * TPW); per_min = per_min < 1 ? 1 : per_min > 4 ? 4 : per_min;
  if (!a.sel && per < per_min) per = per_min;
  long long teams = (ngroups + per - 1) / per;                     // every team gets `per` groups (the last maybe fewer)
  if (!H && WR == 8 && !a.sel) teams = ngroups < max_teams ? ngroups : max_teams;   // one workgroup per CU: the row groups are spread over all CUs
  long long grid = (teams + TPW - 1) / TPW;
  if (grid < 1) grid = 1;
  { const long long nteams = grid * TPW; a.team_base = (int)(ngroups / nteams); a.team_rem = (int)(ngroups % nteams);
    // exactly two workgroups per CU: the pass that reaches the CUs first takes one row group more per team, the second pass one fewer
    const bool two_per_cu = !H && grid == 2LL * fast_cu_count() && !a.sel && a.team_base > 2;
    a.team_skew = two_per_cu ? 1 : 0; a.team_first = two_per_cu ? (int)(nteams / 2) : 0;
    a.team_stride = (!H && !a.team_skew && !a.sel && (EPI == 2 || a.nseg == 1)) ? (int)nteams : 0; }
  // prologue kind (the specialised ones exist for the shapes the decode step uses; everything else takes the generic prologue)
  const bool one_batch = a.K / 8 <= NT * (NT >= 512 ? 1 : 2);
  if constexpr (MR > 1) return launch_fast_p<T, R, WK, WR, EPI, H, 0, MR>(a, grid, lds, s);
  else {
  if constexpr (EPI == 1 && WK == 1 && !H) {
    if (a.attn_S > 0) {
      if (a.K / 8 > NT || a.x_staged || !a.x_f32 || a.sel) return tga_set_error("tga_attn_merge_qlinear: needs one float32 partial row set of at most %d values", 8 * NT);
      return launch_fast_p<T, R, WK, WR, EPI, H, 7>(a, grid, lds, s);
    }
  }
  if (a.attn_S > 0) return tga_set_error("tga_attn_merge_qlinear: shape outside the fused path (K = %d)", a.K);
  if constexpr (EPI == 1) { if (a.x_staged) return launch_fast_p<T, R, WK, WR, EPI, H, 2>(a, grid, lds, s); }
  if constexpr (WK == 1 && EPI == 0) {
    if (a.comb_y) {
      if (a.x_staged || !a.norm_w || !a.x_f32 || a.K / 8 > NT || a.comb_k > 8) return tga_set_error("tga_moe_combine_rmsnorm_qlinear_multi: needs one float32 row of at most %d values and at most 8 summands", 8 * NT);
      return launch_fast_p<T, R, WK, WR, EPI, H, 5>(a, grid, lds, s);
    }
  }
  if (a.comb_y) return tga_set_error("tga_moe_combine_rmsnorm_qlinear_multi: shape outside the fused path (K = %d)", a.K);
  if constexpr (WK == 1 && EPI == 2) {
    if (a.route_logits) {
      if (a.x_staged || a.norm_w || a.x_f32 || !one_batch || a.xdiv != a.route_k || a.xdiv_jobs % a.route_k != 0) return tga_set_error("tga_qlinear_experts_routed: needs fp16 rows of at most %d values and k jobs per row", 16 * NT);
      return launch_fast_p<T, R, WK, WR, EPI, H, 6>(a, grid, lds, s);
    }
  }
  if (a.route_logits) return tga_set_error("tga_qlinear_experts_routed: shape outside the routed path (K = %d)", a.K);
  if constexpr (WK == 1 && EPI != 1) {
    if constexpr (EPI == 0 && !H) { if (!a.x_staged && one_batch && a.norm_w && a.x_f32 && a.touch_pos) return launch_fast_p<T, R, WK, WR, EPI, H, 8>(a, grid, lds, s); }
    if (!a.x_staged && one_batch && a.norm_w && a.x_f32) return launch_fast_p<T, R, WK, WR, EPI, H, 1>(a, grid, lds, s);
    if (!a.x_staged && one_batch && !a.norm_w && !a.x_f32) return launch_fast_p<T, R, WK, WR, EPI, H, 3>(a, grid, lds, s);
  }
  return launch_fast_p<T, R, WK, WR, EPI, H, 0>(a, grid, lds, s);
  }
}

#ifndef QG1_R2_ROWS
#define QG1_R2_ROWS 16
#endif
static constexpr int r2_rows_per_cu() { return QG1_R2_ROWS; }   // two rows per step from 16 rows per CU on (8B decode: q/k/v and attn_output with two rows 508 -> 519 tok/s)
template <int T, int WK, int WR, bool H = false>
static int launch_fast_e(const QArgs& a, hipStream_t s) {
  if (a.epilogue == 2) return launch_fast<T, 2, WK, WR, 2, H>(a, s);
  // two rows per step keep more bytes in flight per lane; a single row when there are too few rows to fill the chip twice, for Q8_0 pairs
  // (68-byte units: no faster with two) and when the waves of a workgroup split K - with the three-deep ring a single row per step is
  // faster there (4096 x 14336: Q4_0 in the 8B decode step 12.5 -> 11.7 us, Q4_K 13.2 -> 12.2, Q6_K 19.3 -> 17.4, Q5_0 16.2 -> 15.2).
  const bool r2 = (T == F_Q4_0P || T == GGML_MXFP4 || T == GGML_Q6_K || T == GGML_Q4_K || T == GGML_Q5_K || T == GGML_Q4_1 || T == GGML_Q5_0 || T == GGML_Q5_1 || T == GGML_IQ4_XS)
                  && WK == 1 && a.ntot >= (long long)fast_cu_count() * r2_rows_per_cu();
  if (a.epilogue == 1) return r2 ? launch_fast<T, 2, WK, WR, 1, H>(a, s) : launch_fast<T, 1, WK, WR, 1, H>(a, s);
  return r2 ? launch_fast<T, 2, WK, WR, 0, H>(a, s) : launch_fast<T, 1, WK, WR, 0, H>(a, s);
}

// entry point per weight format, instantiated in qgemv1_*.hip
template <int T>
int qgemv1_launch_format(QArgs a, hipStream_t s) {
  using F = Fmt<T>;
  a.nu = a.K / F::UW;
  a.row_bytes = (long long)(a.K / F::BW) * F::BB;
  const int waves = (a.nu + 63) / 64;
  if (a.nu <= 32 && !a.attn_S) return launch_fast_e<T, 1, 4, true>(a, s);      // (the merge prologue exists for whole-wave row teams: shorter rows leave lanes without a unit)
  if (waves <= 1) return launch_fast_e<T, 1, QG1_WR>(a, s);
  if (waves <= 2) return launch_fast_e<T, 2, 1>(a, s);
  if (waves <= 4) return launch_fast_e<T, 4, 1>(a, s);
  if (waves <= 8) return launch_fast_e<T, 8, 1>(a, s);
  return launch_fast_e<T, 16, 1>(a, s);
}

// One launch for two sets of matrices of different block types (qgemv1_two_kernel): float32 row with the norm folded in, rows of 33..64 units (one wave per row),
// plain epilogue.  One workgroup per CU, dealt to the sets by their bytes; inside a set the row groups are spread as a launch of its own would.  Returns -1 outside that range.
template <int TA, int TB>
int qgemv1_launch_two(QArgs a, QArgs b, hipStream_t s) {
  using FA = Fmt<TA>; using FB = Fmt<TB>;
  static_assert(FA::UW == FB::UW, "both sets stage the row in units of the same width");
  constexpr int WR = QG1_WR, NT = WR * 64;
  if (a.K != b.K || a.K % FA::BW != 0 || a.K % FB::BW != 0) return -1;
  a.nu = a.K / FA::UW; b.nu = b.K / FB::UW;
  a.row_bytes = (long long)(a.K / FA::BW) * FA::BB; b.row_bytes = (long long)(b.K / FB::BW) * FB::BB;
  if (a.nu <= 32 || a.nu > 64 || a.K / 8 > NT) return -1;
  for (const QArgs* q : {&a, &b})
    if (q->epilogue || q->sel || q->x_staged || q->y_stage_fmt || !q->norm_w || !q->x_f32 || q->comb_y || q->route_logits || q->ntot <= 0) return -1;
  const size_t lds = (size_t)a.nu * (FA::UW / 2 + 4) * 4;
  const long long cus = fast_cu_count();
  const int R = (a.ntot + b.ntot >= cus * r2_rows_per_cu()) ? 2 : 1;
  // the split that makes the longest team shortest (row groups come whole: dealing the workgroups by bytes alone left the 58 workgroups of a 1024-row Q6_K attn_v
  // with two row groups per team where 64 have one: 11.4 us for the 8B shape); among equals the one that leaves set a the most workgroups
  const long long nga = (a.ntot + R - 1) / R, ngb = (b.ntot + R - 1) / R;
  long long gb = 1, best = -1;
  for (long long g = 1; g < cus; g++) {
    const long long ta = (nga + (cus - g) * WR - 1) / ((cus - g) * WR) * a.row_bytes, tb = (ngb + g * WR - 1) / (g * WR) * b.row_bytes;
    const long long t = ta > tb ? ta : tb;
    if (best < 0 || t < best) { best = t; gb = g; }
  }
  long long ga = cus - gb;
  auto fit = [&](QArgs& q, long long& g) {                       // no more workgroups than the set has row groups for; row groups per team and the remainder
    const long long ngroups = (q.ntot + R - 1) / R, most = (ngroups + WR - 1) / WR;
    if (g > most) g = most;
    const long long nteams = g * WR;
    q.team_base = (int)(ngroups / nteams); q.team_rem = (int)(ngroups % nteams);
    q.team_skew = 0; q.team_first = 0;
    q.team_stride = q.nseg == 1 ? (int)nteams : 0;
  };
  fit(a, ga); fit(b, gb);
  if (R == 2) qgemv1_two_kernel<TA, TB, 2, WR, 1><<<dim3((unsigned)(ga + gb)), dim3(NT), lds, s>>>(a, b, (unsigned)ga);
  else qgemv1_two_kernel<TA, TB, 1, WR, 1><<<dim3((unsigned)(ga + gb)), dim3(NT), lds, s>>>(a, b, (unsigned)ga);
  TGA_LAUNCH_CHECK();
  return 0;
}

// Two activation rows on the same kernel (one weight row per step, generic prologue): plain, residual or SwiGLU epilogue, rows that one wave
// covers or K split over four waves.  Returns -1 outside that range.
template <int T, int MR>
static int qgemv1_launch_multi_m(const QArgs& a, int waves, hipStream_t s) {
  if (a.epilogue == 2) return waves <= 1 ? launch_fast<T, 2, 1, QG1_WR, 2, false, MR>(a, s) : launch_fast<T, 2, 4, 1, 2, false, MR>(a, s);   // a row group = the gate row and the up row
  if (waves <= 1) return a.epilogue == 1 ? launch_fast<T, 1, 1, QG1_WR, 1, false, MR>(a, s) : launch_fast<T, 1, 1, QG1_WR, 0, false, MR>(a, s);
  return a.epilogue == 1 ? launch_fast<T, 1, 4, 1, 1, false, MR>(a, s) : launch_fast<T, 1, 4, 1, 0, false, MR>(a, s);
}
template <int T>
int qgemv1_launch_multi(QArgs a, int M, hipStream_t s) {
  using F = Fmt<T>;
  a.nu = a.K / F::UW;
  a.row_bytes = (long long)(a.K / F::BW) * F::BB;
  const int waves = (a.nu + 63) / 64;
  if (a.nu <= 32 || waves > 4 || a.epilogue > 2 || a.sel || a.x_staged || a.y_stage_fmt || a.norm_w || a.comb_y || a.route_logits) return -1;
  // two rows only: every further row adds 3 us on a 14336 x 4096 matrix (the dot2 chains and lane reductions of a wave do not overlap
  // enough with two waves per SIMD; Q4_0: 9.8 / 13.0 / 15.7 / 18.7 us at M = 1..4), so from three rows on the matrix-core kernels win
  if (M == 2) return qgemv1_launch_multi_m<T, 2>(a, waves, s);
  return -1;
}
