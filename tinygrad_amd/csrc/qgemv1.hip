// M = 1 dequant-GEMV fast path: dispatch over the weight formats (kernel and launch templates in qgemv1.h, one translation unit per
// group of formats in qgemv1_*.hip).
#include "qgemv1.h"

extern template int qgemv1_launch_format<F_Q4_0P>(QArgs, hipStream_t);
extern template int qgemv1_launch_format<F_Q8_0P>(QArgs, hipStream_t);
extern template int qgemv1_launch_format<GGML_F16>(QArgs, hipStream_t);
extern template int qgemv1_launch_format<GGML_MXFP4>(QArgs, hipStream_t);
extern template int qgemv1_launch_format<GGML_Q6_K>(QArgs, hipStream_t);
extern template int qgemv1_launch_format<GGML_Q4_K>(QArgs, hipStream_t);
extern template int qgemv1_launch_format<GGML_Q5_K>(QArgs, hipStream_t);
extern template int qgemv1_launch_format<GGML_Q4_1>(QArgs, hipStream_t);
extern template int qgemv1_launch_format<GGML_Q5_0>(QArgs, hipStream_t);
extern template int qgemv1_launch_format<GGML_Q5_1>(QArgs, hipStream_t);
extern template int qgemv1_launch_format<GGML_IQ4_XS>(QArgs, hipStream_t);
extern template int qgemv1_launch_format<GGML_IQ3_XXS>(QArgs, hipStream_t);
extern template int qgemv1_launch_format<GGML_IQ3_S>(QArgs, hipStream_t);
extern template int qgemv1_launch_format<GGML_IQ2_S>(QArgs, hipStream_t);
extern template int qgemv1_launch_format<GGML_Q1_0>(QArgs, hipStream_t);

// Returns -1 when the shape is outside the fast path (caller falls back to the LDS-staged kernel).
int tga_qgemv1_dispatch(int fmt, const QArgs& a, hipStream_t s) {
  const int uw = (fmt == GGML_MXFP4) ? 32 : 64;
  if (fmt == GGML_F16 && a.K % 64) return -1;
  if ((a.K / uw + 63) / 64 > 16 || a.K % 8) return -1;
  if ((fmt == GGML_IQ3_XXS || fmt == GGML_IQ3_S || fmt == GGML_IQ2_S || fmt == GGML_Q1_0) && a.K > 32768) return -1;   // (their tables share the LDS with the row)
  if (((uintptr_t)a.x & 15) != 0) return a.x_staged ? tga_set_error("tga_qlinear: staged activations must be 16-byte aligned") : -1;   // 16-byte activation loads
  switch (fmt) {
    case F_Q4_0P: return qgemv1_launch_format<F_Q4_0P>(a, s);
    case F_Q8_0P: return qgemv1_launch_format<F_Q8_0P>(a, s);
    case GGML_Q6_K: return qgemv1_launch_format<GGML_Q6_K>(a, s);
    case GGML_Q4_K: return qgemv1_launch_format<GGML_Q4_K>(a, s);
    case GGML_Q5_K: return qgemv1_launch_format<GGML_Q5_K>(a, s);
    case GGML_Q4_1: return qgemv1_launch_format<GGML_Q4_1>(a, s);
    case GGML_Q5_0: return qgemv1_launch_format<GGML_Q5_0>(a, s);
    case GGML_Q5_1: return qgemv1_launch_format<GGML_Q5_1>(a, s);
    case GGML_IQ4_XS: return qgemv1_launch_format<GGML_IQ4_XS>(a, s);
    case GGML_IQ3_XXS: return qgemv1_launch_format<GGML_IQ3_XXS>(a, s);
    case GGML_IQ3_S: return qgemv1_launch_format<GGML_IQ3_S>(a, s);
    case GGML_IQ2_S: return qgemv1_launch_format<GGML_IQ2_S>(a, s);
    case GGML_Q1_0: return qgemv1_launch_format<GGML_Q1_0>(a, s);
    case GGML_MXFP4: return qgemv1_launch_format<GGML_MXFP4>(a, s);
    case GGML_F16: return qgemv1_launch_format<GGML_F16>(a, s);
  }
  return -1;
}
