// Weight formats as they lie in LDS after direct-to-LDS loads (global_load_lds_dwordx4: lane l's 16-byte piece lands at LDS base + 16 l), shared by the
// small-batch kernels that stream the weights through LDS (qgemm_dma.hip, qgemm_wp.hip): per format the geometry of a run of units of one row and the
// read that picks one unit out of it, and the counted wait on vector-memory operations.
#pragma once
#include "qfmt.h"
#include <type_traits>

typedef _Float16 v8f16 __attribute__((ext_vector_type(8)));
typedef float v4f32 __attribute__((ext_vector_type(4)));

#define QD_NW 8                       // waves per workgroup
#define QD_LDS_CU (160 * 1024)
#define QD_MAX_NB 3

// slot_bytes(su): bytes of su units of one row; PAD: 16-byte pieces between the rows of a slot in LDS (the pitch spreads sixteen rows over the banks);
// from_lds(row, u): unit u of a slot's row.
// Geometry of a slot whose rows are whole 16-byte pieces at 16-byte aligned offsets: pieces(su) per row, the second slot of a stage second_off(su) bytes
// behind the first, stage_stride(su) bytes of a row per stage, the slot's first unit skew(su, half) bytes into the staged row.
template <class D> struct DmaPlain {
  static constexpr int pieces(int su) { return D::slot_bytes(su) / 16; }
  static constexpr int second_off(int su) { return D::slot_bytes(su); }
  static constexpr int stage_stride(int su) { return 2 * D::slot_bytes(su); }
  static constexpr int skew(int, int) { return 0; }
};
template <int T> struct DmaFmt;
template <> struct DmaFmt<F_Q4_0P> : DmaPlain<DmaFmt<F_Q4_0P>> {
  static constexpr int PAD = 1;
  static constexpr int slot_bytes(int su) { return su * 36; }
  static __device__ __forceinline__ Fmt<F_Q4_0P>::Raw from_lds(const char* row, int u) {
    const uint32_t* p = (const uint32_t*)(row + 36 * u);
    Fmt<F_Q4_0P>::Raw r;
    r.a = u32x4{p[0], p[1], p[2], p[3]}; r.b = u32x4{p[4], p[5], p[6], p[7]}; r.c = p[8];
    return r;
  }
};
template <> struct DmaFmt<F_Q8_0P> : DmaPlain<DmaFmt<F_Q8_0P>> {
  static constexpr int PAD = 1;
  static constexpr int slot_bytes(int su) { return su * 68; }
  static __device__ __forceinline__ Fmt<F_Q8_0P>::Raw from_lds(const char* row, int u) {
    const uint32_t* p = (const uint32_t*)(row + 68 * u);
    Fmt<F_Q8_0P>::Raw r;
    r.a = u32x4{p[0], p[1], p[2], p[3]}; r.b = u32x4{p[4], p[5], p[6], p[7]}; r.c = u32x4{p[8], p[9], p[10], p[11]}; r.d = u32x4{p[12], p[13], p[14], p[15]}; r.e = p[16];
    return r;
  }
};

// fp16 weights (model.py:376 keeps dense tensors as fp16): a unit is 64 consecutive weights = eight aligned pieces, nothing to decode
template <> struct DmaFmt<GGML_F16> : DmaPlain<DmaFmt<GGML_F16>> {
  static constexpr int PAD = 1;
  static constexpr int slot_bytes(int su) { return su * 128; }
  static __device__ __forceinline__ Fmt<GGML_F16>::Raw from_lds(const char* row, int u) {
    const u32x4* p = (const u32x4*)(row + 128 * u);
    Fmt<GGML_F16>::Raw r;
#pragma unroll
    for (int i = 0; i < 8; i++) r.q[i] = p[i];
    return r;
  }
};
// Q6_K (gguf.py:68-72): four units = one superblock of 210 bytes, so a slot is 32 units = 8 superblocks = 105 pieces and a wave's step of four units is one
// superblock; superblocks are 2-byte aligned in the slot's row: every 16-byte piece is read as its enclosing aligned dwords and funnel-shifted (by 0 or 16 bits,
// the same for the whole wave), as Fmt<GGML_Q6_K>::load does from global memory.
__device__ __forceinline__ u32x4 lds16_a2(const char* p, uint32_t& tail_dword, uint32_t& sh) {
  const uint32_t a = (uint32_t)(uintptr_t)p; sh = (a & 2u) * 8u;
  const uint32_t* q = (const uint32_t*)(p - (a & 3u));
  const uint32_t v0 = q[0], v1 = q[1], v2 = q[2], v3 = q[3], e = q[4];
  tail_dword = e;
  return u32x4{__builtin_amdgcn_alignbit(v1, v0, sh), __builtin_amdgcn_alignbit(v2, v1, sh), __builtin_amdgcn_alignbit(v3, v2, sh), __builtin_amdgcn_alignbit(e, v3, sh)};
}
template <> struct DmaFmt<GGML_Q6_K> {
  static constexpr int PAD = 2;                          // pitches of 107 and 55 pieces = 428 and 220 dwords = 44 and 28 mod 64: sixteen rows on sixteen different bank quads
  // Slots of 16 units (K beyond 4096, an even number of slots): 4 superblocks = 840 bytes start 8 bytes off a 16-byte boundary in every second slot.  A stage
  // (1680 bytes of a row) is fetched as two windows of 53 aligned pieces, [0, 848) and [832, 1680): the second slot's units start 8 bytes into its window.
  static constexpr int pieces(int su) { return su == 32 ? 105 : 53; }
  static constexpr int second_off(int su) { return su == 32 ? 1680 : 832; }
  static constexpr int stage_stride(int su) { return su / 4 * 210 * 2; }
  static constexpr int skew(int su, int half) { return su == 32 ? 0 : 8 * half; }
  static __device__ __forceinline__ Fmt<GGML_Q6_K>::Raw from_lds(const char* row, int u) {
    const char* p = row + 210 * (u >> 2); const int h = (u >> 1) & 1, g = u & 1;
    uint32_t tail, sh;
    Fmt<GGML_Q6_K>::Raw r;
    r.a = lds16_a2(p + 64 * h + 16 * g, tail, sh); r.b = lds16_a2(p + 64 * h + 32 + 16 * g, tail, sh); r.h = lds16_a2(p + 128 + 32 * h + 16 * g, tail, sh);
    const u32x4 sc = lds16_a2(p + 192, tail, sh);          // sc[0..15]; the tail dword holds d (bytes 208, 209)
    r.sc0 = h ? sc.z : sc.x; r.sc1 = h ? sc.w : sc.y;
    r.d = (uint32_t)g | (__builtin_amdgcn_alignbit(0u, tail, sh) << 16);
    return r;
  }
};

// Q4_K / Q5_K (gguf.py:57-67): four units = one superblock of 144 / 176 bytes = 9 / 11 aligned pieces; a wave's step of four units is one superblock per row
// (lane group g: sub-block pair g), every read is an aligned 16-byte piece.
template <bool FIVE> struct DmaFmtK45 : DmaPlain<DmaFmtK45<FIVE>> {
  using F = FmtK45<FIVE>;
  static constexpr int PAD = 1;                          // pitches of 37 / 73 (Q4_K) and 45 / 89 (Q5_K) pieces: sixteen rows on sixteen different bank quads
  static constexpr int slot_bytes(int su) { return su / 4 * F::BB; }
  static __device__ __forceinline__ typename F::Raw from_lds(const char* row, int u) {
    const char* b = row + F::BB * (u >> 2); const int p = u & 3;
    typename F::Raw r;
    r.hdr = *(const u32x4*)b; r.q0 = *(const u32x4*)(b + F::QS + 32 * p); r.q1 = *(const u32x4*)(b + F::QS + 32 * p + 16);
    if constexpr (FIVE) { r.h0 = *(const u32x4*)(b + 16); r.h1 = *(const u32x4*)(b + 32); }
    r.p = (uint32_t)p;
    return r;
  }
};
template <> struct DmaFmt<GGML_Q4_K> : DmaFmtK45<false> {};
template <> struct DmaFmt<GGML_Q5_K> : DmaFmtK45<true> {};

// Q4_1 / Q5_0 / Q5_1 block pairs (gguf.py:47-55): units of 40 / 44 / 48 bytes at 4-byte aligned offsets of the slot's row; 16 units are 40 / 44 / 48 pieces
// (pitches of 41 / 45 / 49 pieces = 36 / 52 / 4 mod 64 dwords: sixteen rows on sixteen different bank quads)
template <int KIND> struct DmaFmtL : DmaPlain<DmaFmtL<KIND>> {
  using F = FmtL<KIND>;
  static constexpr int PAD = 1;
  static constexpr int slot_bytes(int su) { return su * F::BB; }
  static __device__ __forceinline__ typename F::Raw from_lds(const char* row, int u) {
    const uint32_t* p = (const uint32_t*)(row + F::BB * u);
    typename F::Raw r;
    r.a = u32x4{p[0], p[1], p[2], p[3]}; r.b = u32x4{p[4], p[5], p[6], p[7]};
#pragma unroll
    for (int i = 0; i < F::ND - 8; i++) r.t[i] = p[8 + i];
    return r;
  }
};
template <> struct DmaFmt<GGML_Q4_1> : DmaFmtL<0> {};
template <> struct DmaFmt<GGML_Q5_0> : DmaFmtL<1> {};
template <> struct DmaFmt<GGML_Q5_1> : DmaFmtL<2> {};

// at most n vector-memory operations of this wave still outstanding (n is the same for the whole wave).  Behind it, the registers of inline-assembly
// requests are passed through an empty asm statement with the comment "; landed": no use of them can move in front of the wait, and the comment marks
// the place in the generated assembly for tests/test_isa_invariants.py
__device__ __forceinline__ void qd_wait_vm(int n) {
  switch (n) {
#define QD_W(k) case k: asm volatile("s_waitcnt vmcnt(" #k ")" ::: "memory"); break;
    QD_W(1) QD_W(2) QD_W(3) QD_W(4) QD_W(5) QD_W(6) QD_W(7) QD_W(8) QD_W(9) QD_W(10) QD_W(11) QD_W(12) QD_W(13) QD_W(14) QD_W(15) QD_W(16)
    QD_W(17) QD_W(18) QD_W(19) QD_W(20) QD_W(21) QD_W(22) QD_W(23) QD_W(24)
#undef QD_W
    default: asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); break;
  }
}
