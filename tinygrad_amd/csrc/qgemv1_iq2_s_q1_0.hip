// M = 1 dequant-GEMV fast path: IQ2_S, Q1_0 (instantiations of qgemv1.h).
#include "qgemv1.h"
template int qgemv1_launch_format<GGML_IQ2_S>(QArgs, hipStream_t);
template int qgemv1_launch_format<GGML_Q1_0>(QArgs, hipStream_t);
