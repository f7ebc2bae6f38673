// One launch for attn_q / attn_k of one block type and attn_v of another (Q4_K_M / Q5_K_M files: Q6_K attn_v in half of the blocks); template in qgemv1.h
#include "qgemv1.h"

int tga_qgemv1_two_dispatch(int fmt_a, int fmt_b, const QArgs& a, const QArgs& b, hipStream_t s) {
  if (fmt_a == GGML_Q4_K && fmt_b == GGML_Q6_K) return qgemv1_launch_two<GGML_Q4_K, GGML_Q6_K>(a, b, s);
  if (fmt_a == GGML_Q5_K && fmt_b == GGML_Q6_K) return qgemv1_launch_two<GGML_Q5_K, GGML_Q6_K>(a, b, s);
  return -1;
}
