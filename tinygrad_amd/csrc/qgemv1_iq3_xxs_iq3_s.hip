// M = 1 dequant-GEMV fast path: IQ3_XXS, IQ3_S (instantiations of qgemv1.h).
#include "qgemv1.h"
template int qgemv1_launch_format<GGML_IQ3_XXS>(QArgs, hipStream_t);
template int qgemv1_launch_format<GGML_IQ3_S>(QArgs, hipStream_t);
