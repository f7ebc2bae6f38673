// Host-side helpers shared by the C-ABI translation units.
#pragma once
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdarg.h>
#include "../../include/tinygrad_amd.h"

int tga_set_error(const char* fmt, ...);   // stores the per-thread message, returns 1
extern "C" int tga_route_scratch_setup(int device);   // mxfp8.hip: looks up the static routing workspace of the current device (tga_init calls it)

#define TGA_HIP(expr) do { hipError_t _e = (expr); if (_e != hipSuccess) \
  return tga_set_error("HIP Error %d, %s  [%s at %s:%d]", (int)_e, hipGetErrorString(_e), #expr, __FILE__, __LINE__); } while (0)
#define TGA_REQUIRE(cond, ...) do { if (!(cond)) return tga_set_error(__VA_ARGS__); } while (0)
// kernel launches report configuration errors through hipGetLastError
#define TGA_LAUNCH_CHECK() TGA_HIP(hipGetLastError())
