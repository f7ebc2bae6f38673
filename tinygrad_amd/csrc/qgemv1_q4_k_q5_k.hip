// M = 1 dequant-GEMV kernels of these weight formats (template in qgemv1.h)
#include "qgemv1.h"

template int qgemv1_launch_format<GGML_Q4_K>(QArgs, hipStream_t);
template int qgemv1_launch_format<GGML_Q5_K>(QArgs, hipStream_t);
