// Block dequant kernels: bit-exact restatement of ggml_data_to_tensor (tinygrad/llm/gguf.py:23-119) for Q4_0 (:46), Q4_1 (:47-49), Q5_0 / Q5_1 (:50-55), Q8_0 (:56),
// Q4_K / Q5_K (:57-67), Q6_K (:68-72), IQ3_XXS / IQ3_S / IQ2_S (:73-95), IQ4_XS (:96-104), MXFP4 (:105-114) and Q1_0 (:115-118).  One thread produces 4 consecutive output elements (one 16-byte or 8-byte store), so
// stores are fully coalesced; the packed bytes are re-read through L1/L2 (this kernel is a load-time / test utility, the
// decode path never materialises weights).
#include "deq.h"
#include "host.h"

template <int T, bool F16>
__global__ __launch_bounds__(256) void dequant_kernel(const uint8_t* __restrict__ blocks, void* __restrict__ out, int64_t n4) {
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n4; i += (int64_t)gridDim.x * 256) {
    const int64_t e = i * 4, blk = e / Deq<T>::NEL; const int e0 = (int)(e % Deq<T>::NEL);
    float o[4];
    Deq<T>::get4(blocks + blk * Deq<T>::NBY, e0, o);
    if (F16) {
      // keep the float32 result opaque: folding the multiply into v_fma_mixlo_f16 (product + 0) would turn -0.0 into +0.0
#pragma unroll
      for (int q = 0; q < 4; q++) asm volatile("" : "+v"(o[q]));
      u32x2 v = {f2h_bits(o[0]) | (f2h_bits(o[1]) << 16), f2h_bits(o[2]) | (f2h_bits(o[3]) << 16)};
      ((u32x2*)out)[i] = v;
    } else {
      f32x4 v = {o[0], o[1], o[2], o[3]};
      ((f32x4*)out)[i] = v;
    }
  }
}

template <int T> static int launch_dequant(const void* blocks, int64_t n, void* out, int out_dtype, hipStream_t s) {
  TGA_REQUIRE(n % Deq<T>::NEL == 0, "tga_dequant: n=%lld is not a multiple of the block size %d", (long long)n, Deq<T>::NEL);
  if (n == 0) return 0;
  const int64_t n4 = n / 4;
  const int grid = (int)((n4 + 255) / 256 < 65536 ? (n4 + 255) / 256 : 65536);
  if (out_dtype == TGA_F32) dequant_kernel<T, false><<<grid, 256, 0, s>>>((const uint8_t*)blocks, out, n4);
  else dequant_kernel<T, true><<<grid, 256, 0, s>>>((const uint8_t*)blocks, out, n4);
  TGA_LAUNCH_CHECK();
  return 0;
}

extern "C" int tga_dequant(int ggml_type, const void* blocks, int64_t n, void* out, int out_dtype, void* stream) {
  TGA_REQUIRE(out_dtype == TGA_F32 || out_dtype == TGA_F16, "tga_dequant: out_dtype must be TGA_F32 or TGA_F16");
  TGA_REQUIRE(n >= 0 && (n == 0 || (blocks && out)), "tga_dequant: null pointer");
  hipStream_t s = (hipStream_t)stream;
  switch (ggml_type) {
    case GGML_Q4_0: return launch_dequant<GGML_Q4_0>(blocks, n, out, out_dtype, s);
    case GGML_Q4_1: return launch_dequant<GGML_Q4_1>(blocks, n, out, out_dtype, s);
    case GGML_Q5_0: return launch_dequant<GGML_Q5_0>(blocks, n, out, out_dtype, s);
    case GGML_Q5_1: return launch_dequant<GGML_Q5_1>(blocks, n, out, out_dtype, s);
    case GGML_Q8_0: return launch_dequant<GGML_Q8_0>(blocks, n, out, out_dtype, s);
    case GGML_Q4_K: return launch_dequant<GGML_Q4_K>(blocks, n, out, out_dtype, s);
    case GGML_Q5_K: return launch_dequant<GGML_Q5_K>(blocks, n, out, out_dtype, s);
    case GGML_Q6_K: return launch_dequant<GGML_Q6_K>(blocks, n, out, out_dtype, s);
    case GGML_MXFP4: return launch_dequant<GGML_MXFP4>(blocks, n, out, out_dtype, s);
    case GGML_IQ4_XS: return launch_dequant<GGML_IQ4_XS>(blocks, n, out, out_dtype, s);
    case GGML_IQ3_XXS: return launch_dequant<GGML_IQ3_XXS>(blocks, n, out, out_dtype, s);
    case GGML_IQ3_S: return launch_dequant<GGML_IQ3_S>(blocks, n, out, out_dtype, s);
    case GGML_IQ2_S: return launch_dequant<GGML_IQ2_S>(blocks, n, out, out_dtype, s);
    case GGML_Q1_0: return launch_dequant<GGML_Q1_0>(blocks, n, out, out_dtype, s);
  }
  return tga_set_error("GGML type '%d' is not supported!", ggml_type);   // message of tinygrad/llm/gguf.py:119
}
