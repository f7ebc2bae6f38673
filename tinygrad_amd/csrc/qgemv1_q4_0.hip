// M = 1 dequant-GEMV kernels of these weight formats (template in qgemv1.h)
#include "qgemv1.h"

template int qgemv1_launch_format<F_Q4_0P>(QArgs, hipStream_t);
