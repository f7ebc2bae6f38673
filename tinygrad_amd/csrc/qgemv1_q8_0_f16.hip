// M = 1 dequant-GEMV kernels of these weight formats (template in qgemv1.h)
#include "qgemv1.h"

template int qgemv1_launch_format<F_Q8_0P>(QArgs, hipStream_t);
template int qgemv1_launch_format<GGML_F16>(QArgs, hipStream_t);
