// Host-side helpers shared by the C-ABI translation units.
#pragma once
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdarg.h>
#include "../../include/tinygrad_amd.h"

int tga_set_error(const char* fmt, ...);   // stores the per-thread message, returns 1
extern "C" int tga_route_scratch_setup(int device);   // mxfp8.hip: looks up the static routing workspace of the current device (tga_init calls it)
int tga_qgemm64_setup(int device);                          // qgemm64.hip: allocates the prefill GEMM workspace of the current device (tga_init calls it)
void tga_qgemm64_release(hipStream_t stream);               // qgemm64.hip: a stream that is being destroyed gives its workspace slot back

#define TGA_HIP(expr) do { hipError_t _e = (expr); if (_e != hipSuccess) \
  return tga_set_error("HIP Error %d, %s  [%s at %s:%d]", (int)_e, hipGetErrorString(_e), #expr, __FILE__, __LINE__); } while (0)
#define TGA_REQUIRE(cond, ...) do { if (!(cond)) return tga_set_error(__VA_ARGS__); } while (0)
// kernel launches report configuration errors through hipGetLastError
#define TGA_LAUNCH_CHECK() TGA_HIP(hipGetLastError())
