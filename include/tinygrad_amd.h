/* C-ABI of libtinygrad_amd.so: hand-written gfx950 kernels for the quantized-weight linear path.
 *
 * Plain pointers and sizes only.  Every device pointer is memory the CALLER owns (allocated with tga_malloc or any HIP
 * allocation of the same process); no entry point allocates or frees an output.  All work is enqueued on `stream`
 * (a hipStream_t passed as void*, NULL = the null stream) and is asynchronous unless stated.
 * Return value: 0 on success, non-zero on failure with the message available from tga_last_error() (per thread).
 *
 * Citations name the reference interface each entry point replaces (paths relative to the tinygrad tree).
 */
#ifndef TINYGRAD_AMD_H
#define TINYGRAD_AMD_H
#include <stddef.h>
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

/* ggml type ids, as in tinygrad/llm/gguf.py:20-21 */
#define TGA_F32 0
#define TGA_F16 1
#define TGA_Q4_0 2
#define TGA_Q4_1 3
#define TGA_Q5_0 6
#define TGA_Q5_1 7
#define TGA_Q8_0 8
#define TGA_Q4_K 12
#define TGA_Q5_K 13
#define TGA_Q6_K 14
#define TGA_IQ3_XXS 18
#define TGA_IQ3_S 21
#define TGA_IQ2_S 22
#define TGA_IQ4_XS 23
#define TGA_MXFP4 39
#define TGA_Q1_0 41     /* (every block type above is read in place by the linear entry points and expanded by tga_dequant) */
/* activation dtype code: fp16 values in the staged order of the consuming weight (see tga_stage_activation) */
#define TGA_F16_STAGED 101

/* ---- runtime: replaces HIPDevice / HIPAllocator / HIPProgram timing in tinygrad/runtime/ops_hip.py:12-70 ---- */
const char* tga_last_error(void);
int tga_init(int device);                                  /* hipSetDevice + kernel attribute set-up; ops_hip.py:14-20.  Also allocates, once per device, the 160 MB workspace of the 17 .. 128 row linears */
int tga_device_name(char* buf, size_t len);
int tga_malloc(void** ptr, size_t nbytes);                 /* ops_hip.py:60-62 */
int tga_free(void* ptr);                                   /* ops_hip.py:63 */
int tga_memcpy_h2d(void* dst, const void* src, size_t n);  /* ops_hip.py:64-66, synchronous */
int tga_memcpy_d2h(void* dst, const void* src, size_t n);  /* ops_hip.py:67-69, synchronous */
int tga_memcpy_d2d(void* dst, const void* src, size_t n, void* stream);
/* device-to-device copy done by a plain kernel (n bytes, 16-byte aligned): a known-size yardstick for hardware traffic counters. */
int tga_copy_kernel(void* dst, const void* src, size_t n, void* stream);
int tga_memset(void* dst, int value, size_t n, void* stream);   /* hipMemsetAsync; refused (error) on a stream that is capturing */
int tga_sync(void);                                        /* ops_hip.py:22-24 hipDeviceSynchronize */
int tga_stream_create(void** stream);
int tga_stream_destroy(void* stream);                      /* waits for the stream's work, gives its slot of that workspace back, destroys it */
int tga_stream_sync(void* stream);
int tga_event_create(void** ev);                           /* ops_hip.py:49-57 wait=True timing */
int tga_event_destroy(void* ev);
int tga_event_record(void* ev, void* stream);
int tga_event_sync(void* ev);
int tga_event_elapsed_ms(void* start, void* stop, float* ms);
/* Replay support (the reference replays a captured kernel list per token: tinygrad/engine/jit.py:163-198). */
int tga_graph_begin(void* stream);
int tga_graph_end(void* stream, void** graph_exec);
int tga_graph_launch(void* graph_exec, void* stream);
int tga_graph_destroy(void* graph_exec);
/* The same replay without hipGraphLaunch: tga_graph_begin, the launches, then tga_cmdlist_end keeps the captured kernel launches (function, grid,
 * block, dynamic LDS, argument values) and tga_cmdlist_launch enqueues them one after the other on the stream, in capture order.  Only kernel
 * launches captured on one stream are accepted.  Per kernel this costs less on the GPU than a graph node does (0.3-0.5 us measured). */
int tga_cmdlist_end(void* stream, void** cmdlist);
int tga_cmdlist_launch(void* cmdlist, void* stream);
int tga_cmdlist_size(void* cmdlist);
int tga_cmdlist_destroy(void* cmdlist);

/* ---- block dequant: ggml_data_to_tensor, tinygrad/llm/gguf.py:23-119 (types 2, 3, 6, 7, 8, 12, 13, 14, 23, 39, 41) ----
 * blocks: device pointer to the raw GGUF tensor bytes; n: number of elements (multiple of the block size).
 * out_dtype TGA_F32: bit-exact ggml_data_to_tensor result.  TGA_F16: that result cast to fp16 round-to-nearest-even,
 * i.e. the weight the model path holds after tinygrad/llm/model.py:376. */
int tga_dequant(int ggml_type, const void* blocks, int64_t n, void* out, int out_dtype, void* stream);

/* ---- fused dequant + linear: nn.Linear.__call__ over a lazily dequantized GGUF weight,
 * tinygrad/nn/__init__.py:177 -> Tensor.dot tinygrad/mixin/op.py:367-392 (float32 accumulation, dtype.py:212-216).
 *   y[m, n] = sum_k x[m, k] * W[n, k],   W = dequant(w) as (N, K) row-major with quant blocks along K (gguf.py:148).
 * x: (M, K) row-major, x_dtype TGA_F16 or TGA_F32 (F32 activations are rounded to fp16 before the multiply).
 * y: (M, N) row-major, y_dtype TGA_F16 or TGA_F32.  1 <= M <= 8 (the decode range); 9 <= M <= 16 is taken too, for prefill chunks: one launch where the
 * LDS-fed matrix-core kernel applies (Q4_0 / Q8_0 / Q4_1 / Q5_0 / Q5_1 / Q4_K / Q5_K, K a multiple of 1024 (Q4_K: of 2048 up to 4096), rows a multiple of 16; K beyond 4096: one matrix, plain or residual epilogue; Q6_K: one matrix, K a multiple of 2048), otherwise two calls of at most eight rows; 17 <= M <= 128 (plain fp16 / float32 activations; a prefill step) is one pass over the weights on a matrix-core tile of two, four or eight column groups where it applies (Q4_0 / Q8_0 pairs, Q4_K, Q5_K, Q6_K, IQ4_XS, fp16; K a multiple of 256 up to 32768; several matrices: each a multiple of 16 rows; staged rows and split-K partial sums in the per-device workspace of tga_init, one slot per stream), otherwise blocks of sixteen rows.  Dense fp16 weights (TGA_F16, K % 64 == 0) are served too.  K must be a multiple of the type's block size
 * (Q4_1 / Q5_0 / Q5_1 are served as block pairs: K % 64 == 0).
 * w must be 2-byte aligned for Q4_0/Q8_0/Q6_K and 4-byte aligned for Q4_K/Q5_K/Q4_1/Q5_0/Q5_1 (GGUF aligns tensor data to 32 bytes,
 * gguf.py:144-148). */
int tga_qlinear(int ggml_type, const void* w, const void* x, int x_dtype, void* y, int y_dtype,
                int M, int64_t N, int64_t K, void* stream);

/* Several weights sharing one activation in ONE launch (attn_q/k/v at tinygrad/llm/model.py:168; ffn_gate/ffn_up at :137).
 * nseg <= 3; segment i is an (n[i], K) weight of type ggml_type written to y[i] as (M, n[i]).
 * epilogue: 0 = plain store; 1 = y[i] = resid[i] + x W^T in float32 (the residual adds at model.py:149-150; requires
 * y_dtype TGA_F32; resid[i] may alias y[i]); 2 = SwiGLU: nseg must be 2 with n[0] == n[1], and the single output
 * y[0] = silu(x Wgate^T) * (x Wup^T) (model.py:137), resid ignored. */
int tga_qlinear_multi(int ggml_type, int nseg, const void* const* w, void* const* y, const int64_t* n,
                      const void* x, int x_dtype, int y_dtype, int M, int64_t K,
                      int epilogue, const void* const* resid, int y_stage_type, int64_t y_stage_K, void* stream);

/* tga_qlinear_multi at M = 1 with the RMSNorm that precedes it folded in (attn_norm -> attn_q/k/v and ffn_norm -> ffn_gate/up,
 * tinygrad/llm/model.py:149-150; output_norm -> output, :362; nn.RMSNorm tinygrad/nn/__init__.py:296-304): x is the float32
 * row BEFORE the norm, the kernel multiplies W by fp16((x * rsqrt(mean(x^2) + norm_eps)) * norm_weight).  Needs the M = 1 fast
 * path (K % 64 == 0, K <= 65536, 16-byte aligned x and norm_weight, 4-byte aligned weights); other arguments as above. */
int tga_rmsnorm_qlinear_multi(const float* norm_weight, float norm_eps, int ggml_type, int nseg, const void* const* w, void* const* y, const int64_t* n,
                              const void* x, int y_dtype, int64_t K, int epilogue, const void* const* resid,
                              int y_stage_type, int64_t y_stage_K, void* stream);

/* tga_rmsnorm_qlinear_multi with the plain epilogue for matrices of DIFFERENT block types over the same row: segment i has type ggml_types[i].  A Q4_K_M / Q5_K_M
 * file keeps attn_v as Q6_K beside Q4_K / Q5_K attn_q / attn_k in half of its blocks, and tinygrad/llm/model.py:161-163 applies the three linears to one
 * normalised row.  Runs of equal consecutive types are one launch each; a (Q4_K | Q5_K) run followed by a Q6_K run shares ONE launch when K is 2304..4096
 * and x, norm_weight are 16-byte aligned.  Results are those of tga_rmsnorm_qlinear_multi per run; the shared launch is another build of the same walk and may round
 * a float32 sum differently (within 2e-6 of the largest output). */
int tga_rmsnorm_qlinear_mixed(const float* norm_weight, float norm_eps, int nseg, const int32_t* ggml_types, const void* const* w, void* const* y, const int64_t* n,
                              const float* x, int y_dtype, int64_t K, void* stream);

/* The same for M rows (batched decode steps and prefill chunks): x (M, K) float32 BEFORE the norm.  One launch where the LDS-fed small-batch kernel applies
 * (Q4_0 / Q8_0 / Q4_1 / Q5_0 / Q5_1 / Q4_K / Q5_K / Q6_K / fp16, 2 <= M <= 8, K <= 4096: the norm is folded into its prologue); otherwise tga_rmsnorm_rows into xn_scratch_f16 (M, K) followed by
 * tga_qlinear_multi on it (M up to 128).  xn_scratch_f16 is clobbered or left untouched accordingly. */
int tga_rmsnorm_qlinear_rows(const float* norm_weight, float norm_eps, int ggml_type, int nseg, const void* const* w, void* const* y, const int64_t* n,
                             const float* x, void* xn_scratch_f16, int y_dtype, int M, int64_t K, int epilogue, const void* const* resid, void* stream);

/* tga_rmsnorm_qlinear_multi on the row x_in + sum_j probs[j] * y_experts[j]: the MoE weighted sum over the selected experts' outputs and
 * the block residual (tinygrad/llm/model.py:130, 150) folded into the next block's attn_norm -> attn_q/k/v launch (or output_norm -> output).
 * The completed row is written to x_out, which must not alias x_in.  y_experts (k, K) and probs (k) float32, k <= 8, K <= 2048, plain epilogue. */
int tga_moe_combine_rmsnorm_qlinear_multi(const float* y_experts, const float* probs, int k, const float* x_in, float* x_out,
                                          const float* norm_weight, float norm_eps, int ggml_type, int nseg, const void* const* w, void* const* y,
                                          const int64_t* n, int y_dtype, int64_t K, void* stream);

/* Staged activations (no counterpart in the reference; an M = 1 fast path): the decode GEMV keeps each lane's activations in
 * registers in the order its in-register decode produces weights, which is a fixed permutation of the row that depends on the
 * weight's (ggml_type, K).  tga_stage_activation writes that permutation as fp16 (K values); a linear then takes it with
 * x_dtype = TGA_F16_STAGED and skips its own staging.  Producers can emit the order directly: tga_rmsnorm / tga_attention_decode
 * (stage_type, stage_K) and tga_qlinear_multi with the SwiGLU epilogue (y_stage_type != 0: the fp16 output, of length y_stage_K, is written in the
 * staged order of a consumer weight of that type whose K = y_stage_K).  Requires K % 64 == 0 (Q4_K / Q5_K / Q6_K: % 256). */
int tga_stage_activation(int ggml_type, const void* x, int x_dtype, int64_t K, void* out_f16, void* stream);

/* ExpertWeights.__call__ (tinygrad/llm/model.py:21-27) over a stacked (n_experts, N, K) weight kept in GGUF blocks: for job j
 * (one (token, slot) pair) y[j, :] = x[j / jobs_per_x_row, :] @ W[sel[j]]^T; only the selected experts' bytes are read.
 * With w_up != NULL the output is silu(x Wgate[e]^T) * (x Wup[e]^T) (model.py:129), w being the gate stack.
 * sel: n_jobs int32 expert ids in device memory.  x: (ceil(n_jobs / jobs_per_x_row), K); y: (n_jobs, N). */
int tga_qlinear_experts(int ggml_type, const void* w, const void* w_up, int64_t n_experts, const int32_t* sel, int n_jobs,
                        int jobs_per_x_row, const void* x, int x_dtype, void* y, int y_dtype, int64_t N, int64_t K, void* stream);

/* The expert gate/up jobs of ONE token with the gating inside the launch: every workgroup computes scores, pairwise top-k and weights from
 * the router logits (tinygrad/llm/model.py:112-128; gating as tga_moe_gate) for itself, job j multiplies the j-th selected expert:
 * y[j] = silu(x Wgate[e_j]^T) * (x Wup[e_j]^T).  The selection and the weights are written to sel_out / probs_out (k entries each) for
 * the launches that follow.  x: one fp16 row of at most 4096 values; logits: n_experts float32 (tga_moe_router with k = 0 writes them). */
int tga_qlinear_experts_routed(int ggml_type, const void* w_gate, const void* w_up, int64_t n_experts, const float* logits, int k,
                               int gating, int norm_topk_prob, float scale, int32_t* sel_out, float* probs_out,
                               const void* x_f16, void* y, int y_dtype, int64_t N, int64_t K, void* stream);
/* The same for n_tokens tokens in one launch (the (B, T, k) selection of ExpertWeights.__call__, model.py:21-27, gated per token as model.py:112-128):
 * jobs t k .. t k + k - 1 are token t's, gated from row t of logits (n_tokens, n_experts); x (n_tokens, K) fp16, y (n_tokens k, N),
 * sel_out / probs_out (n_tokens, k). */
int tga_qlinear_experts_routed_rows(int ggml_type, const void* w_gate, const void* w_up, int64_t n_experts, const float* logits, int n_tokens, int k,
                                    int gating, int norm_topk_prob, float scale, int32_t* sel_out, float* probs_out,
                                    const void* x_f16, void* y, int y_dtype, int64_t N, int64_t K, void* stream);

/* Expert gating of FFNBlock._feed_forward (model.py:112-128): scores by ExpertGating (1 SOFTMAX, 2 SIGMOID, 3 SOFTMAX_WEIGHT,
 * 4 SQRT_SOFTPLUS; model.py:9-13), pairwise_topk selection (model.py:35-41: ascending, lower index wins ties), probabilities
 * gathered / renormalised / scaled.  logits (n_tokens, n_experts) float32 -> sel (n_tokens, k) int32, probs (n_tokens, k). */
int tga_moe_gate(const float* logits, int n_tokens, int n_experts, int k, int gating, int norm_topk_prob, float scale,
                 int32_t* sel, float* probs, void* stream);
/* The same with the expert selection bias of model.py:113, 123 (`exp_probs_b`): experts are ranked by score + selection_bias[e] (n_experts
 * float32), the probabilities are gathered from the unbiased scores; with a bias the SOFTMAX + norm_topk_prob shortcut of model.py:116-117
 * does not apply, as in the reference. */
int tga_moe_gate_biased(const float* logits, const float* selection_bias, int n_tokens, int n_experts, int k, int gating, int norm_topk_prob, float scale,
                        int32_t* sel, float* probs, void* stream);
/* Router of ONE token in one launch (model.py:112-128 with the block's ffn_norm, :150): h = fp16(RMSNorm(x) * norm_weight) (norm_weight
 * NULL: h = fp16(x)), logits = h @ Wr^T for a dense fp16 router weight (n_experts, dim), then gating + top-k as tga_moe_gate.
 * xn_out_f16 (dim fp16, the activation of the expert GEMVs) may be NULL.  logits_ws: n_experts floats (the logits, readable
 * afterwards) followed by one int32 arrival counter that must be ZERO before the first call (each call leaves it zero); calls
 * sharing one workspace must not overlap.  dim % 8 == 0, dim <= 16384, n_experts <= 1024, k <= 64.
 * k = 0: logits only (sel / probs may be NULL, the counter is not touched): for a consumer that gates for itself (tga_qlinear_experts_routed). */
int tga_moe_router(const float* x, const float* norm_weight, float norm_eps, const void* router_w_f16, int dim, int n_experts, int k,
                   int gating, int norm_topk_prob, float scale, void* xn_out_f16, float* logits_ws, int32_t* sel, float* probs, void* stream);
/* tga_moe_router with k = 0 over `rows` tokens in one launch: xn (rows, dim) fp16 = ffn_norm(x) (model.py:150) and logits (rows, n_experts) = xn . router^T
 * (ffn_gate_inp, model.py:112); the gating is left to the consumer (tga_qlinear_experts_routed_rows or tga_moe_gate). */
int tga_moe_router_rows(const float* x, const float* norm_weight, float norm_eps, const void* router_w_f16, int rows, int dim, int n_experts,
                        void* xn_out_f16, float* logits, void* stream);
/* out[t] = resid[t] + sum_s probs[t, s] * y[t, s, :]  (model.py:130 and the residual add :150); resid may be NULL or alias out. */
int tga_moe_combine(const float* y, const float* probs, const float* resid, int n_tokens, int k, int dim, float* out, void* stream);

/* ---- decode-step neighbours of the linears (batch 1), tinygrad/llm/model.py:144-204, 358-364 ----
 * `state` is a 64-byte device record {int32 pos, token, step, n_prompt, error, vocab, pad[10]} so that one captured launch sequence
 * serves every position (the reference binds a symbolic start_pos into its replayed graph, model.py:464-484).  vocab = rows of the
 * embedding table (0: token ids are not checked).  error is a bit mask the kernels set instead of reading or writing out of bounds:
 * bit 0 = tga_embed_row met a token id outside [0, vocab) and read row 0; bit 1 = tga_attention_decode met pos outside [0, max_ctx)
 * and did nothing.  The caller checks and clears it after synchronising. */

/* token_embd(tokens).float() for the token in state (model.py:359): dequantizes one row of a Q4_0 / Q4_1 / Q5_0 / Q5_1 / Q8_0 /
 * Q4_K / Q5_K / Q6_K / MXFP4 / F16 / F32 table (bit-exact block decode, as tga_dequant, rounded to fp16: the reference's table is an fp16 weight, model.py:376). */
int tga_embed_row(const void* table, int ggml_type, int dim, const void* state, float* out, void* stream);

/* nn.RMSNorm (tinygrad/nn/__init__.py:296-304): (x * rsqrt(mean(x^2) + eps)) * weight; writes fp16 and/or fp32 (either may be NULL).
 * stage_type != 0: the fp16 output is written in the staged order of a consumer weight of that ggml type with K = dim. */
int tga_rmsnorm(const float* x, const float* weight, int dim, float eps, void* out_f16, float* out_f32, int stage_type, void* stream);

/* One token of TransformerBlock._attention after the q/k/v projections (model.py:180-197): half-split RoPE of q and k with the
 * freqs_cis table rope_table[max_ctx][head_dim] = cos half | sin half (model.py:16-19, 29-33), fp16 KV append at state.pos
 * (cache layout [n_kv_heads][max_ctx][head_dim]), GQA scaled-dot-product attention over positions 0..pos with softmax in
 * float32 (tinygrad/mixin/rand.py:298-327).  head_dim is 64, 128 or 256.  Two launches: softmax partials per 64-position split,
 * then their merge per query head.  partials: workspace of at least n_heads * ceil(max_ctx/64) * (head_dim + 2) floats that carries
 * the split partials from the first launch to the second; calls sharing one workspace must not overlap.
 * stage_type != 0: out_f16 is written in the staged order of a consumer weight of that type with K = n_heads * head_dim. */
int tga_attention_decode(const float* q, const float* k, const float* v, void* cache_k, void* cache_v, float* partials, const void* state,
                         int n_heads, int n_kv_heads, int head_dim, int max_ctx, const float* rope_table, void* out_f16, float* out_f32, int stage_type, void* stream);

/* tga_attention_decode with the q / k RMSNorm of the reference applied before RoPE (attn_q_norm / attn_k_norm, float32 weights, both
 * NULL for no norm).  norm_per_head = 0: one norm over all n_heads * head_dim (n_kv_heads * head_dim) values, weights of that length
 * (model.py:169, OLMoE); norm_per_head = 1: one norm per head over its head_dim values, weights of head_dim values shared by all heads
 * (model.py:180, Qwen3).  q and k must be 16-byte aligned when the norm is on. */
int tga_attention_decode_normed(const float* q, const float* k, const float* v, const float* q_norm_weight, const float* k_norm_weight, float norm_eps,
                                int norm_per_head, void* cache_k, void* cache_v, float* partials, const void* state,
                                int n_heads, int n_kv_heads, int head_dim, int max_ctx, const float* rope_table, void* out_f16, float* out_f32, int stage_type, void* stream);

/* tga_attention_decode as ONE launch whose consumer merges (model.py:167-198 up to the softmax-weighted V sums; _normed: with the q / k RMSNorm of
 * tga_attention_decode_normed, over the whole rows or per head, q and k 16-byte aligned).  A workgroup serves one query
 * head and one split of the cache; tga_attention_split_plan reports the number of splits for max_ctx: at most six, 0 when the cache is too long for this path
 * (max_ctx beyond 3072).  partials: n_heads * (n_splits * head_dim + 16) floats, per head [n_splits][head_dim] weighted V sums followed by the splits'
 * (max, sum) pairs; 16-byte aligned.  A split that starts beyond state.pos leaves an empty partial (max -inf, sum 0).  The merge is tga_attn_merge_qlinear's. */
int tga_attention_split_plan(int max_ctx, int* n_splits);
int tga_attention_decode_split(const float* q, const float* k, const float* v, void* cache_k, void* cache_v, float* partials, const void* state,
                               int n_heads, int n_kv_heads, int head_dim, int max_ctx, const float* rope_table, void* stream);
int tga_attention_decode_split_normed(const float* q, const float* k, const float* v, const float* q_norm_weight, const float* k_norm_weight, float norm_eps, int norm_per_head,
                                      void* cache_k, void* cache_v, float* partials, const void* state,
                                      int n_heads, int n_kv_heads, int head_dim, int max_ctx, const float* rope_table, void* stream);
/* attn_output + residual (model.py:198, 149) over the attention row that tga_attention_decode_split left as partials: y = resid + merge(partials) W^T, float32,
 * y may be resid.  The merge per head - sum_s e_s o_s / sum_s e_s l_s with e_s = exp(m_s - max m), rounded to fp16 - happens while the launch stages its
 * activation row.  K = n_heads * head_dim <= 4096 (rows of at most 64 units, one wave per row); block types with a single-row kernel except MXFP4; n_splits 1..6. */
int tga_attn_merge_qlinear(int ggml_type, const void* w, float* y, int64_t N, int64_t K, const float* resid, const float* partials, int n_splits, int head_dim, void* stream);

/* tga_rmsnorm_qlinear_multi (single row) for the q / k / v launch of a decode step, with a hint for the attention launch behind it (no counterpart in the
 * reference): every lane also reads one dword of one 128-byte line of the cached K / V rows below state.pos and of the rotation row of that position, each on
 * the XCD whose attention workgroups will read it, so that the attention finds them in L2.  Same results as tga_rmsnorm_qlinear_multi; caches
 * [n_kv_heads][max_ctx][head_dim] fp16, rope_table [max_ctx][head_dim] float32.  The hint is dropped unless n_kv_heads is a multiple of 8. */
int tga_rmsnorm_qlinear_multi_touch(const float* norm_weight, float norm_eps, int ggml_type, int nseg, const void* const* w, void* const* y, const int64_t* n,
                                    const void* x, int y_dtype, int64_t K, int epilogue, const void* const* resid,
                                    const void* state, const void* cache_k, const void* cache_v, const void* rope_table, int n_kv_heads, int head_dim, int max_ctx,
                                    void* stream);
/* argmax(-1) with first-max tie rule (tinygrad/mixin/op.py:866-891) + the bookkeeping of Transformer.generate (model.py:475-484):
 * while state.pos + 1 < state.n_prompt the next input token is prompt[pos + 1]; otherwise the argmax token is stored at
 * out_tokens[state.step] and fed back.  scratch_v / scratch_i: 256 floats / 256 int32. */
int tga_argmax_step(const float* logits, int n, float* scratch_v, int* scratch_i, void* state, const int* prompt, int* out_tokens, int max_tokens, void* stream);
/* prompt step that skips the output projection: token = prompt[pos + 1], pos += 1. */
int tga_advance_prompt(void* state, const int* prompt, void* stream);

/* ---- batched decode: 2..8 sequences in lockstep at one position (the reference's (B, T) token batch, tinygrad/llm/model.py:358-364 with
 * B > 1; ExpertWeights.__call__ over a (B, T, k) selection, :21-27).  The dense linears take tga_qlinear_multi with M = B. ---- */

/* token_embd(tokens) for n_rows tokens listed in device memory (model.py:359): out (n_rows, dim) float32.  state: the decode record, only
 * for its vocab / error fields (ids outside [0, vocab) read row 0 and set error bit 0). */
int tga_embed_rows(const void* table, int ggml_type, int dim, const int32_t* tokens, int n_rows, void* state, float* out, void* stream);
/* out[i] = fp16(silu(gate[i]) * up[i]) over n float32 values: the feed-forward activation of tinygrad/llm/model.py:137 for a block whose ffn_gate and ffn_up are of
 * different block types (two linear launches, then this; equal types take the SwiGLU epilogue of tga_qlinear_multi instead). */
int tga_silu_mul(const float* gate, const float* up, int64_t n, void* out_f16, void* stream);
/* tga_rmsnorm over `rows` rows of dim values (one workgroup per row); outputs (rows, dim). */
int tga_rmsnorm_rows(const float* x, const float* weight, int rows, int dim, float eps, void* out_f16, float* out_f32, int stage_type, void* stream);
/* tga_moe_combine followed by tga_rmsnorm_rows in one launch: every row of x is completed IN PLACE as x[t] + sum_s probs[t, s] * y[t, s, :] (the weighted
 * sum over the selected experts' outputs and the block residual, tinygrad/llm/model.py:130, 150; the same sums in the same order as tga_moe_combine) and the
 * next block's attn_norm - or output_norm - is taken of the completed row (nn.RMSNorm, tinygrad/nn/__init__.py:296-304).  y (rows, k, dim), probs (rows, k). */
int tga_moe_combine_rmsnorm_rows(const float* y, const float* probs, float* x, const float* weight, int rows, int k, int dim, float eps, void* out_f16,
                                 float* out_f32, void* stream);
/* tga_attention_decode_normed for `batch` sequences at the shared position state.pos: q (batch, n_heads * head_dim), k / v (batch, n_kv_heads *
 * head_dim), caches (batch, n_kv_heads, max_ctx, head_dim) fp16, partials batch times the single-sequence workspace, outputs (batch, n_heads * head_dim). */
int tga_attention_decode_batched(int batch, const float* q, const float* k, const float* v, const float* q_norm_weight, const float* k_norm_weight, float norm_eps,
                                 int norm_per_head, void* cache_k, void* cache_v, float* partials, const void* state,
                                 int n_heads, int n_kv_heads, int head_dim, int max_ctx, const float* rope_table, void* out_f16, float* out_f32, void* stream);
/* Attention for `rows` consecutive positions state.pos .. state.pos + rows - 1 of ONE sequence (the chunked prefill of Transformer.generate,
 * tinygrad/llm/model.py:464, 476-481; causal mask `_attention`, model.py:227-229): q (rows, n_heads * head_dim), k / v (rows, n_kv_heads * head_dim),
 * one cache (n_kv_heads, max_ctx, head_dim) fp16.  A first launch rotates and appends every row's key / value, a second attends from the cache (row r sees the
 * positions up to its own; more than eight rows of head_dim 64 / 128 without q / k norm: on the matrix cores, probabilities rounded to fp16), a third merges the splits.  partials: rows times the single-sequence workspace.  Outputs (rows, n_heads * head_dim). */
int tga_attention_prefill_chunk(int rows, const float* q, const float* k, const float* v, const float* q_norm_weight, const float* k_norm_weight, float norm_eps,
                                int norm_per_head, void* cache_k, void* cache_v, float* partials, const void* state,
                                int n_heads, int n_kv_heads, int head_dim, int max_ctx, const float* rope_table, void* out_f16, float* out_f32, void* stream);
/* tga_attention_prefill_chunk for 17 .. 128 rows whose fp16 output is ONE buffer for all rows in the layout the prefill GEMM multiplies from, for a consumer
 * (attn_output) of block type consumer_type with K = n_heads * head_dim (a multiple of 256): 16 * (rows <= 32 ? 2 : 4) rows x K fp16 values; the rows at and beyond
 * `rows` are not written (zero them once). */
int tga_attention_prefill_chunk_staged(int rows, const float* q, const float* k, const float* v, const float* q_norm_weight, const float* k_norm_weight, float norm_eps,
                                       int norm_per_head, void* cache_k, void* cache_v, float* partials, const void* state,
                                       int n_heads, int n_kv_heads, int head_dim, int max_ctx, const float* rope_table, void* out_rows_staged, int consumer_type, void* stream);
/* ---- a prefill step of 17 .. 128 rows (model.py:464, 476-481) with the rows handed from launch to launch in the layout the prefill GEMM multiplies from: no
 * counterpart in the reference (its scheduler fuses what it fuses); the results equal those of tga_rmsnorm_qlinear_rows / tga_qlinear_multi on plain rows up to the
 * order of a float32 sum.  tga_qlinear_multi takes such rows with x_dtype TGA_F16_STAGED and M > 16, and writes them from the SwiGLU epilogue with y_stage_type. ---- */
/* *ncg = column groups of sixteen rows (2 or 4: the buffer of the rows holds 16 * ncg x K fp16 values) when a linear of this type with rows of K values takes M rows
 * in that layout, 0 when it does not. */
int tga_rows_staged_plan(int ggml_type, int64_t K, int M, int* ncg);
/* y = y + x W^T (attn_output, ffn_down: model.py:149-150) for one matrix over rows in that layout.  When the kernel splits K, the sum over the splits is left to the
 * caller's next launch: *partials / *ks / *np describe the partial tiles (in the stream's workspace: valid until the next call with 17 .. 128 rows on this stream) and y
 * is untouched; *ks = 0: y is complete. */
int tga_qlinear_rows_deferred(int ggml_type, const void* w, int64_t N, int64_t K, const void* x_staged, int M, float* y, const float** partials, int* ks, int* np, void* stream);
/* nn.RMSNorm (tinygrad/nn/__init__.py:296-304) of `rows` float32 rows, written as fp16 in that layout for a consumer of consumer_type (and to xn_out_f16 as plain
 * rows when given).  partials != NULL: every row is first completed in place with what tga_qlinear_rows_deferred left. */
int tga_rmsnorm_rows_stage(float* x, const float* partials, int ks, int np, const float* weight, float eps, int rows, int dim, int consumer_type, void* xn_out_f16, void* staged_out, void* stream);
/* x += the sum of those partial tiles in the order of K (what the deferred call's own reduce launch would have done). */
int tga_rows_add_partials(float* x, const float* partials, int ks, int np, int rows, int dim, void* stream);
/* After a chunk of `rows` prompt positions: state.pos += rows and tokens[r] = prompt[state.pos + r] (entries past max_ctx - 1 read the last one): the
 * input ids of the next chunk (model.py:477-480 slices the prompt on the host; here the captured step advances itself). */
int tga_chunk_advance(void* state, const int32_t* prompt, int rows, int32_t* tokens, int max_ctx, void* stream);
/* tga_argmax_step / tga_advance_prompt for a batch: while state.pos + 1 < state.n_prompt the next token of sequence b is prompts[b * prompt_stride +
 * pos + 1]; otherwise (logits != NULL) the first index of the maximum of logits row b (model.py:364 at temperature 0) goes to tokens[b] and
 * out_tokens[state.step * batch + b].  Then pos += 1 (and step += 1 when tokens were sampled).  logits NULL: a prompt step without lm-head. */
int tga_argmax_rows_step(const float* logits, int batch, int n, void* state, const int32_t* prompts, int prompt_stride, int32_t* tokens, int32_t* out_tokens,
                         int max_steps, void* stream);
/* Groups the (token, slot) jobs of a batch by expert: table = n_experts records of 16 int32 {number of jobs that selected the expert (at most 8:
 * the experts of one token are distinct, model.py:35-41, and a batch has at most 8 tokens), their job indices}.  flags: one int32 the caller
 * zeroes; bit 0 is set when an expert was selected by more than 8 jobs, bit 1 for an expert id outside [0, n_experts) (such jobs are dropped). */
int tga_expert_jobs(const int32_t* sel, int n_jobs, int n_experts, int32_t* table, int32_t* flags, void* stream);
/* ExpertWeights.__call__ (model.py:21-27) for the jobs of a batch with every selected expert streamed ONCE: for each expert with jobs, one
 * small-batch GEMM on the matrix cores over its (N, K) weight and the fp16 activation rows of its jobs (job j reads row j / jobs_per_x_row of
 * x_f16, writes row j of y (n_jobs, N)); w_up != NULL: y = silu(x Wgate[e]^T) * (x Wup[e]^T) (model.py:129).  Weights are rounded to fp16 once
 * (the reference's fp16 weight cast, model.py:376), products accumulate in float32.  table from tga_expert_jobs. */
int tga_qlinear_experts_grouped(int ggml_type, const void* w, const void* w_up, int64_t n_experts, const int32_t* table, int n_jobs, int jobs_per_x_row,
                                const void* x_f16, void* y, int y_dtype, int64_t N, int64_t K, void* stream);

/* ---- MXFP8 MoE prefill path: extra/gemm/cdna_asm_gemm.py, extra/gemm/moe_routing.py, extra/gemm/moe_gemm.py ---- */

/* quantize_mxfp8 (cdna_asm_gemm.py:149-159): per 32 block along K, e8 = clamp(floor(log2(max(amax, 1e-38))) + 127, 0, 254),
 * q = E4M3(clamp(x * 2^(127 - e8), +-448)) (RNE, tinygrad/dtype.py:237-260).  x: (rows, K) bf16 (x_is_bf16) or float32.
 * q: (rows, K) bytes; e8: (rows, K/32) bytes; packed (may be NULL): mx_pack layout (K/128, rows) uint32 (cdna_asm_gemm.py:161-163). */
int tga_quantize_mxfp8(const void* x, int x_is_bf16, int64_t rows, int64_t K, void* q, void* e8, void* packed, void* stream);
/* fused_silu_mul_quantize_mxfp8 (extra/llama_kernels/fused_silu_mul_quantize_mxfp8/__init__.py:11-49, 91-104): act = w1 * sigmoid(w1) * w3 in
 * float32 from two (rows, K) bf16 tensors (sigmoid = 1 / (1 + exp2(-w1 * log2 e))), quantized as tga_quantize_mxfp8 without an intermediate
 * tensor; outputs as there. */
int tga_silu_mul_quantize_mxfp8(const void* x_w1_bf16, const void* x_w3_bf16, int64_t rows, int64_t K, void* q, void* e8, void* packed, void* stream);
/* transpose_quantize_mxfp8 (extra/llama_kernels/transpose_quantize_mxfp8/__init__.py:24-37): the outputs of tga_quantize_mxfp8 for the
 * transpose of g without forming it.  g: (M, N) bf16, M % 32 == 0, N % 64 == 0 (the reference asks N % 256); q: (N, M) bytes; e8: (N, M/32)
 * bytes; packed (may be NULL; needs M % 128 == 0): (M/128, N) uint32. */
int tga_transpose_quantize_mxfp8(const void* g_bf16, int64_t M, int64_t N, void* q, void* e8, void* packed, void* stream);

/* route (moe_routing.py:109-122) for one device group: top-k (descending, lower index first among equals), weights =
 * softmax(top values), per-expert counts padded to 256 -> off (E+1), dest_row[j] = off[e_j] + stable rank of assignment j among
 * those of expert e_j in flattened (token, slot) order.  scratch: int32[n_tokens*k + ceil(n_tokens*k/1024)*n_experts]. */
int tga_moe_route(const float* logits, int n_tokens, int n_experts, int k, float* weights, int32_t* topi, int32_t* dest_row, int32_t* off,
                  int32_t* counts, int32_t* scratch, void* stream);
/* tga_moe_route without a workspace argument and without any allocation (no counterpart in the reference; for callers that cannot
 * allocate: code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  The ranks and per-chunk counts live in a
 * 512 KiB device array inside the library, one copy per GPU, held until the process ends; tga_init(device) must have run on the current
 * device.  Limits: n_tokens * k <= 65536 and n_tokens * k + ceil(n_tokens * k / 1024) * n_experts <= 131072, else an error and no launch.
 * Nothing in the workspace has to start at zero (every word read was written by the same call), but all calls on one GPU share it: calls
 * that overlap on one GPU (two streams, two threads) race.  Same results as tga_moe_route. */
int tga_moe_route_static(const float* logits, int n_tokens, int n_experts, int k, float* weights, int32_t* topi, int32_t* dest_row, int32_t* off,
                         int32_t* counts, void* stream);
/* dispatch (moe_routing.py:124-126): xg[dest_row[j], :] = x[j / k, :] (bf16 rows); rows no assignment maps to are zero-filled. */
int tga_moe_dispatch(const void* x_bf16, const int32_t* dest_row, const int32_t* off, const int32_t* counts, int n_tokens, int k, int n_experts,
                     int64_t m_l, int D, void* xg_bf16, void* stream);
/* combine (moe_routing.py:128-131): out[t] = sum_s bf16(weights[t,s]) * z[dest_row[t*k+s]] in bf16 products, float32 sum, bf16 out. */
int tga_moe_combine_rows(const void* z_bf16, const int32_t* dest_row, const float* weights, int n_tokens, int k, int D, void* out_bf16, void* stream);

/* grouped_mx_gemm's kernel (moe_gemm.py:31-48, 112-134), same operand list and order as the reference's custom kernel:
 * C (M,N) bf16 = A (M,K) e4m3 . B[e(tile)] (E,N,K) e4m3 ^T with E8M0 1x32 scales x_e8 (M,K/32), w_e8 (E,N,K/32); e(tile) from
 * expert_off (E+1) as Routing.rows_e (moe_routing.py:98-104).  x_si / w_si (the mx_pack copies) are accepted and unused.
 * Requires M % 256 == 0, N % 256 == 0, K % 128 == 0 (moe_gemm.py:120).  Every 256-row tile of C is written: the tiles at or beyond
 * expert_off[E] are multiplied with expert E - 1, which is what rows_e assigns them (dispatch leaves those rows of A zero, so they come out 0). */
int tga_grouped_mxfp8_gemm(void* C, const void* A, const void* B, const void* x_si, const void* w_si, const void* x_e8, const void* w_e8,
                           const int32_t* expert_off, int64_t M, int64_t N, int64_t K, int n_experts, void* stream);
/* The same product restricted to the routed tiles (rows below expert_off[E]); the rows of C beyond keep their contents.  For callers that
 * only gather routed rows afterwards (combine, moe_routing.py:128-131): M is the worst-case m_l, of which a fifth is unrouted at benchmark
 * configuration 5's size.  No packed-scale operands (they are unused). */
int tga_grouped_mxfp8_gemm_routed(void* C, const void* A, const void* B, const void* x_e8, const void* w_e8, const int32_t* expert_off,
                                  int64_t M, int64_t N, int64_t K, int n_experts, void* stream);
/* The routed-tiles product for callers that also know how many rows of every expert are routed (Routing.counts, moe_routing.py:109-127): inside an
 * expert's range the rows at or beyond its count are padding (dispatch zeroes them); their 16-row groups are not multiplied and their rows of C are
 * written as zeros.  With zero padding rows of A and finite weights that is the reference's result; when the padding rows of A are not zero
 * (e.g. the second GEMM of a feed-forward whose first GEMM added an expert bias to them) these rows differ from it - combine never reads them. */
int tga_grouped_mxfp8_gemm_counts(void* C, const void* A, const void* B, const void* x_e8, const void* w_e8, const int32_t* expert_off, const int32_t* counts,
                                  int64_t M, int64_t N, int64_t K, int n_experts, void* stream);
/* Device symbol for a pre-compiled PROGRAM bound through Tensor.custom_kernel (tinygrad/tensor.py:390-396, extra/gemm/moe_gemm.py:36-48):
 *   extern "C" __global__ void tga_grouped_mxfp8_gemm_kernel(bf16* C, const fp8* A, const fp8* B, const uint32_t* x_si, const uint32_t* w_si,
 *                                                            const uint8_t* x_e8, const uint8_t* w_e8, const int32_t* expert_off,
 *                                                            int M, int N, int K, int E);
 * one pointer per buffer in the order of the sink's sources, the scalar variables after them (tinygrad/uop/ops.py:1194-1198); launch
 * 512 threads x (M / 256) * (N / 256) workgroups with no dynamic LDS.  Same arithmetic as tga_grouped_mxfp8_gemm, which launches it through
 * the runtime API.  The code object is inside libtinygrad_amd.so; tga_kernel_symbol returns its host-side handle for hipLaunchKernel. */
int tga_kernel_symbol(const char* name, const void** host_function);
/* HIPProgram.__call__ (tinygrad/runtime/ops_hip.py:36-57): launches a kernel handle from tga_kernel_symbol; grid[3] counts workgroups,
 * block[3] threads, args is an array of pointers to the argument values in declaration order; no dynamic LDS. */
int tga_launch_kernel(const void* host_function, const uint32_t* grid, const uint32_t* block, void** args, void* stream);
/* bias add after a grouped GEMM (examples/mlperf/models/gpt_oss.py:219-224, `+ (onehot @ bias.float()).cast(bf16)`): in place,
 * h[r, :] = bf16(h[r, :] + bf16(bias[e(r), :])) with e(r) the expert of row r's 256-row tile (moe_routing.py:98-104: the tiles at or beyond
 * expert_off[E] belong to expert E - 1); bias (E, N) float32.  M % 256 == 0. */
int tga_add_expert_bias(void* h_bf16, const float* bias, const int32_t* expert_off, int64_t M, int64_t N, int n_experts, void* stream);
/* clamped interleaved SwiGLU between the two grouped GEMMs (examples/mlperf/models/gpt_oss.py:94-98), bf16 (rows, 2I) -> (rows, I). */
int tga_swiglu_interleaved(const void* h_bf16, int64_t rows, int two_inter, float limit, float alpha, void* y_bf16, void* stream);

/* Measured peak of the scaled FP8 MFMA (method of extra/mmapeak/mmapeak.py:16-52,97-109): n_workgroups x 4 waves each issue
 * loops x 200 register-only v_mfma_scale_f32_16x16x128_f8f6f4; FLOPs = n_workgroups * 4 * loops * 200 * 65536; the caller times it. */
int tga_mfma_peak(int n_workgroups, int loops, float* scratch, void* stream);

/* ---- synthetic-model writer (no counterpart in the reference, whose weights always come from GGUF files): fills `out` with
 * n_elements random-init weights U(-amp, amp) (nn.Linear's init range, tinygrad/nn/__init__.py:173-174) already quantized to
 * GGUF blocks of ggml_type (TGA_Q4_0: ggml's reference rule; TGA_Q6_K: absmax rule; TGA_Q4_K: min/max rule; TGA_F16: plain fp16 cast); TGA_F32 fills the
 * constant `amp`; TGA_MXFP4 ignores amp: uniform E2M1 codes with E8M0 bytes uniform in [119, 123] (block scales 2^-8 .. 2^-4). */
int tga_synth_weights(int ggml_type, void* out, int64_t n_elements, uint32_t seed, float amp, void* stream);

#ifdef __cplusplus
}
#endif
#endif
