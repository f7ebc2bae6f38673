// M = 1 dequant-GEMV fast path: IQ4_XS (instantiations of qgemv1.h).
#include "qgemv1.h"
template int qgemv1_launch_format<GGML_IQ4_XS>(QArgs, hipStream_t);
