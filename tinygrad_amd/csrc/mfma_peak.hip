// Register-only peak of the scaled FP8 MFMA (v_mfma_scale_f32_16x16x128_f8f6f4), the method of extra/mmapeak/mmapeak.py:16-52,97-109:
// every wave issues `loops` x 200 MFMAs on operands that never leave registers (eight independent accumulators, so consecutive
// instructions do not wait on each other); FLOPs = waves x loops x 200 x 2 x 16 x 16 x 128.
#include "common.h"
#include "host.h"

typedef int i32x8 __attribute__((ext_vector_type(8)));

__global__ __launch_bounds__(256) void mfma_peak_kernel(int loops, float* out) {
  i32x8 a, b;
#pragma unroll
  for (int i = 0; i < 8; i++) { a[i] = 0x38383838 + (int)threadIdx.x * 0x01010101 * (i & 1); b[i] = 0x3C3C3C3C; }   // finite E4M3 bytes
  f32x4 acc[8];
#pragma unroll
  for (int i = 0; i < 8; i++) acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};
  const int sc = 0x7F7F7F7F;                                   // E8M0 scale 1.0 in every byte
  for (int l = 0; l < loops; l++) {
#pragma unroll
    for (int j = 0; j < 25; j++) {
#pragma unroll
      for (int i = 0; i < 8; i++) acc[i] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, acc[i], 0, 0, 0, sc, 0, sc);
    }
  }
  f32x4 s = acc[0];
#pragma unroll
  for (int i = 1; i < 8; i++) s += acc[i];
  if (s.x + s.y + s.z + s.w == 12345.678f) out[0] = s.x;      // keeps the chain live
}

// Launches n_workgroups x 4 waves; the caller times the launch (events) and divides tga_mfma_peak_flops by the duration.
extern "C" int tga_mfma_peak(int n_workgroups, int loops, float* scratch, void* stream) {
  TGA_REQUIRE(n_workgroups > 0 && loops > 0 && scratch, "tga_mfma_peak: bad argument");
  mfma_peak_kernel<<<n_workgroups, 256, 0, (hipStream_t)stream>>>(loops, scratch);
  TGA_LAUNCH_CHECK();
  return 0;
}
