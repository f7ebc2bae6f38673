// The M = 1 dequant-GEMV kernel with two activation rows (qgemv1.h, MR = 2) for the Q4_0 / Q8_0 block pairs and Q6_K: the load pattern of the
// single-row kernel (one weight row per wave instruction group, lane = unit) streams better than the matrix-core kernels' sixteen-row
// pattern, and a second row of dot2 work per decoded unit still fits under the stream (Q8_0 14336 x 4096: 17.2 us against 19.1 us on the
// LDS-staged dot2 kernel; Q4_0: 13.0 us).
#include "qgemv1.h"

template int qgemv1_launch_multi<F_Q4_0P>(QArgs, int, hipStream_t);
template int qgemv1_launch_multi<F_Q8_0P>(QArgs, int, hipStream_t);
template int qgemv1_launch_multi<GGML_Q6_K>(QArgs, int, hipStream_t);

// Returns -1 when the call is outside this path's range (the caller falls back to the matrix-core or the LDS-staged kernel).
int tga_qgemv1_multi_dispatch(int fmt, const QArgs& a, int M, hipStream_t s) {
  if (M != 2 || a.K % 8 || ((uintptr_t)a.x & 15) != 0) return -1;
  if (a.ntot * (long long)a.K < (1ll << 25)) return -1;              // small matrices: the LDS-staged kernel's shorter prologue wins (Q8_0 4096 x 4096: 8.9 against 9.2 us)
  switch (fmt) {
    case F_Q4_0P: return qgemv1_launch_multi<F_Q4_0P>(a, M, s);
    case F_Q8_0P: return qgemv1_launch_multi<F_Q8_0P>(a, M, s);
    case GGML_Q6_K: return qgemv1_launch_multi<GGML_Q6_K>(a, M, s);
  }
  return -1;
}
