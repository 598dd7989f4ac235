// C interface of the gfx950 kernel library.  Every function takes device
// pointers and a HIP stream, checks its arguments on the host, launches
// asynchronously, and returns 0 or a negative code; fmsamd_last_error()
// then holds the reason.  Nothing here allocates device memory.
#pragma once

#include <hip/hip_runtime.h>

#define FMSAMD_ABI_VERSION 10

// element types
#define FMS_F32 0
#define FMS_BF16 1

// activations of the gated feed-forward
#define FMS_ACT_SILU 0
#define FMS_ACT_GELU 1       // with the error function
#define FMS_ACT_RELU 2
#define FMS_ACT_IDENTITY 3
#define FMS_ACT_SIGMOID 4
#define FMS_ACT_TANH 5
#define FMS_ACT_MISH 6       // x tanh(log(1 + e^x))
#define FMS_ACT_GELU_TANH 7  // the tanh approximation
#define FMS_ACT_LAST FMS_ACT_GELU_TANH

#ifdef __cplusplus
extern "C" {
#endif

const char* fmsamd_last_error();
int fmsamd_abi_version();

// resid[t, :] = float(table[ids[t], :]) * scale
int fmsamd_embed(const int* ids, const void* table, int table_dtype, float* out, int n_tokens, int width, int vocab,
                 float scale, hipStream_t stream);

// resid += branch (float32 sum, written back unless `rows` is given); out = norm(resid) * weight + bias.
// branch, weight, bias and rows may be null.  act_dtype is the type of branch and out.
int fmsamd_add_norm(float* resid, const void* branch, int act_dtype, const void* weight, const void* bias,
                    int weight_dtype, void* out, const int* rows, int n_out, int width, float eps, int use_mean,
                    hipStream_t stream);

// out[t, j] = act(gu[t, j] + b[j]) * (gu[t, hidden + j] + b[hidden + j])
int fmsamd_gated_act(const void* gu, const void* bias, int bias_dtype, void* out, int dtype, int n_tokens, int hidden,
                     int act, hipStream_t stream);

// positions[i] += 1 where seq_of_token[i] >= 0
int fmsamd_advance_positions(int* positions, const int* seq_of_token, int n, hipStream_t stream);

int fmsamd_cast(const void* in, int in_dtype, void* out, int out_dtype, long n, hipStream_t stream);
int fmsamd_bias_add(void* x, int dtype, const void* bias, int bias_dtype, int rows, int cols, hipStream_t stream);

// cos/sin of position * freqs[i], float32, [max_pos, half]
int fmsamd_rope_table(const float* freqs, float* cos_t, float* sin_t, int max_pos, int half, hipStream_t stream);

// Rotate the queries of qkv in place; rotate the keys and write keys and values into the paged cache
// (k_cache/v_cache null: queries only).  cos_t null: no rotation.  value_dim (0: head_dim): the size of a value if it
// is not the size of a key; the rows are then [H*D | K*D | K*value_dim] and the value pages [kv head][value_dim][token].
int fmsamd_rope_kv_write(void* qkv, int dtype, long row_stride, const int* positions, const int* seq_of_token,
                         const int* block_table, int table_stride, const float* cos_t, const float* sin_t,
                         int rot_dim, int max_pos, void* k_cache, void* v_cache, int n_tokens, int nheads, int kvheads,
                         int head_dim, int value_dim, hipStream_t stream);

// causal attention over the cache; any element type, any even head size up to 256.  Further terms of the scores:
// slopes (float32 [nheads] or null): score += slopes[head] * (key position - query position); soft_cap (0: none):
// score = soft_cap * tanh(score / soft_cap), before the slope term.  value_dim (0: head_dim): values and output heads
// of another size than the keys.  Which keys a query sees beside the causal rule: the last `window` (0: all), of which the
// sequence's first `keep_first` keys are exempt; or (chunk > 0, no window) the keys of the query's own run of `chunk`
// positions, counted from the sequence's start.  sink (float32 [nheads] or null): a logit per head that joins the softmax's
// denominator and has neither key nor value.  dist_bias (float32 [nheads, dist_len] or null): score +=
// dist_bias[head][min(distance, dist_len - 1)], not scaled and not capped.
int fmsamd_attn_generic(const void* q, long q_stride, void* out, long out_stride, int dtype, const int* positions,
                        const int* seq_of_token, const int* block_table, int table_stride, const void* k_cache,
                        const void* v_cache, int n_tokens, int nheads, int kvheads, int head_dim, float scale,
                        int window, const float* slopes, float soft_cap, int value_dim, int chunk, int keep_first,
                        const float* sink, const float* dist_bias, int dist_len, hipStream_t stream);

// soft_cap (0: none) of the two bfloat16 kernels: scores become soft_cap * tanh(score / soft_cap); chunk and sink as in
// fmsamd_attn_generic; so are keep_first and dist_bias (the prefill kernel has them for head sizes up to 64, and for 128).
// bfloat16 prefill: the step is cut into query blocks of at most fmsamd_attn_prefill_qblock(...) consecutive
// tokens of one sequence; the same number goes into the call as qblock_tokens
int fmsamd_attn_prefill_qblock(int nheads, int kvheads, int head_dim, int n_tokens);
int fmsamd_attn_prefill_bf16(const void* q, long q_stride, void* out, long out_stride, const int* positions,
                             const int* seq_of_token, const int* qblock_start, const int* qblock_len, int n_qblocks,
                             int qblock_tokens, const int* block_table, int table_stride, const void* k_cache, const void* v_cache,
                             int n_tokens, int nheads, int kvheads, int head_dim, float scale, int window,
                             float soft_cap, int chunk, const float* sink, int keep_first, const float* dist_bias,
                             int dist_len, hipStream_t stream);

// bfloat16 decode: one token per sequence.  The context bound max_context is cut into splits of
// `pages_per_split` pages, and every sequence deals its own pages out evenly over that many blocks of `waves`
// waves (which take them in turn and merge in LDS); with more than one split a second kernel merges the
// partial results.  staged != 0 (head size 128 only): pages are loaded in contiguous kilobytes and turned into
// the MFMA layout in LDS, which streams faster when there is much to read.  row_order (or null): the token rows in
// the order in which the blocks are to take them, e.g. longest context first; the result does not depend on it.
long fmsamd_attn_decode_workspace(int n_tokens, int nheads, int head_dim, int n_splits);
int fmsamd_attn_decode_bf16(const void* q, long q_stride, void* out, long out_stride, void* workspace,
                            long workspace_bytes, const int* positions, const int* seq_of_token,
                            const int* block_table, int table_stride, const void* k_cache, const void* v_cache,
                            int n_tokens, int nheads, int kvheads, int head_dim, float scale, int window,
                            int max_context, int pages_per_split, int waves, int staged, const int* row_order,
                            float soft_cap, int chunk, const float* sink, int keep_first, const float* dist_bias,
                            int dist_len, hipStream_t stream);

// c[M, N] = a[M, K] w[N, K]^T (+ bias[N])
int fmsamd_gemm_f32(const float* a, long lda, const float* w, const float* bias, float* c, long ldc, int M, int N,
                    int K, hipStream_t stream);
int fmsamd_gemm_bf16(const void* a, long lda, const void* w, const void* bias, int bias_dtype, void* c, int out_dtype,
                     long ldc, int M, int N, int K, hipStream_t stream);
// The same product for any K and any row stride (the MFMA kernels need multiples of 8): element loads and
// float32 FMA.  Slow; it exists so that no width a configuration allows is refused.
int fmsamd_gemm_bf16_any(const void* a, long lda, const void* w, const void* bias, int bias_dtype, void* c,
                         int out_dtype, long ldc, int M, int N, int K, hipStream_t stream);
// A row norm left to the product that reads the rows: the rows hold stream * norm weight, and the sums of
// squares of the stream come as `count` partial sums per row (partials[m * count + i]).  The product is
// multiplied by rsqrt(sum / K + eps) of its row before the bias.  A null pointer (or null partials): none.
typedef struct {
  const float* partials;
  int count;
  float eps;
} fmsamd_row_scale;

// At most 192 rows: the weights stream once through MFMA registers.  From 17 rows on the product needs a
// workspace of fmsamd_gemm_skinny_workspace(M, rows of W, K) bytes (slices of K meet there).
long fmsamd_gemm_skinny_workspace(int M, int rows, int K);
int fmsamd_gemm_skinny_bf16(const void* x, long ldx, const void* w, const void* bias, int bias_dtype, void* out,
                            int out_dtype, long ldo, int M, int N, int K, const fmsamd_row_scale* row_scale,
                            void* workspace, long workspace_bytes, hipStream_t stream);
int fmsamd_gemm_skinny_gated_bf16(const void* x, long ldx, const void* w, const void* bias, int bias_dtype, void* out,
                                  int out_dtype, long ldo, int M, int hidden, int K, int act,
                                  const fmsamd_row_scale* row_scale, void* workspace, long workspace_bytes,
                                  hipStream_t stream);
// resid += x W^T (+ bias) in float32; scaled = resid * norm_w in bfloat16; partials[M, partial_count] = sums
// of squares of resid by groups of columns (partial_count as fmsamd_gemm_skinny_residual_partials(M, N, K) says;
// every entry is written).  At most 192 rows.
int fmsamd_gemm_skinny_residual_partials(int M, int N, int K);
int fmsamd_gemm_skinny_residual_bf16(const void* x, long ldx, const void* w, const void* bias, int bias_dtype,
                                     float* resid, long ldr, const void* norm_w, int norm_w_dtype, void* scaled,
                                     long ldo, float* partials, int partial_count, int M, int N, int K,
                                     const fmsamd_row_scale* row_scale, void* workspace, long workspace_bytes,
                                     hipStream_t stream);

// qkv = x W^T (+ bias) for at most 192 rows with the rotation and the cache write fused into the epilogue;
// only the query columns of `out` are written
int fmsamd_qkv_rope_skinny_bf16(const void* x, long ldx, const void* w, const void* bias, int bias_dtype, void* out,
                                long ldo, int M, int K, const int* positions, const int* seq_of_token,
                                const int* block_table, int table_stride, const float* cos_t, const float* sin_t,
                                int rot_dim, int max_pos, void* k_cache, void* v_cache, int nheads, int kvheads,
                                int head_dim, const fmsamd_row_scale* row_scale, void* workspace, long workspace_bytes,
                                hipStream_t stream);

// token choice; rng_state is [rows][2] uint64 (seed, counter), advanced by the kernel
int fmsamd_sample(const float* logits, long ld, int rows, int vocab, int do_sample, float temperature, int top_k,
                  void* rng_state, int* out_tokens, hipStream_t stream);

// greedy choice over many blocks per row; workspace of fmsamd_argmax_workspace(rows, vocab) bytes
long fmsamd_argmax_workspace(int rows, int vocab);
int fmsamd_argmax(const float* logits, long ld, int rows, int vocab, void* workspace, long workspace_bytes,
                  int* out_tokens, hipStream_t stream);

// The greedy choice of fmsamd_argmax without a workspace, for callers that cannot allocate device memory:
// code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart
// in the reference.  The partial results of the first stage go to an array of FMSAMD_ARGMAX_STATIC_BYTES
// that the library holds on every GPU it runs on until the process ends; rows * ceil(vocab / 2048) * 8 bytes
// must fit (32768 partial results: 256 rows of a vocabulary of 262144, 1024 rows of one of 65536), larger
// inputs are refused.  The call allocates nothing and frees nothing.  All calls on one GPU share that GPU's
// array: calls that overlap in time on one GPU (two streams, two threads) race; calls on one stream do not.
// The first call on a device looks the array's address up (hipGetSymbolAddress), so make it outside a capture.
#define FMSAMD_ARGMAX_STATIC_BYTES (256 * 1024)
int fmsamd_argmax_static(const float* logits, long ld, int rows, int vocab, int* out_tokens, hipStream_t stream);

// Measurements of the GPU itself, for a benchmark's "of the measured peak": a pure read of `bytes` bytes by
// `blocks` blocks, and blocks x 4 waves x iterations x 8 matrix instructions on registers (*flops: how many
// floating-point operations that is).  `out` is a float on the device that may be written.
// contiguous: every block reads one stretch of the buffer instead of the grid sweeping it together; large: 32x32x16
// products instead of 16x16x32.
int fmsamd_probe_read(const void* buffer, long bytes, int blocks, int contiguous, float* out, hipStream_t stream);
int fmsamd_probe_mfma(int blocks, int iterations, int large, float* out, double* flops, hipStream_t stream);

// ---- norms behind a branch, further activations (norm_chain.hip) ----------------------------------------------
// resid += branch / rms(branch) * branch_weight (float32, written back unless `rows` is given);
// out = resid / rms(resid) * weight (out null: the sum only).  Both weights have weight_dtype; either may be null.
int fmsamd_norm_add_norm(float* resid, const void* branch, int act_dtype, const void* branch_weight, float branch_eps,
                         const void* weight, int weight_dtype, float eps, void* out, const int* rows, int n_out, int width,
                         hipStream_t stream);
// The same for norms that may take the mean off and add a shift: with N(v; w, b, mean) = (v - [mean of v]) /
// sqrt([variance or mean square of v] + eps) * w + b, resid += N(branch; branch_weight, branch_bias, branch_mean) and
// out = N(resid; weight, bias, mean).  The four vectors have weight_dtype; any may be null.
int fmsamd_norm_add_norm_affine(float* resid, const void* branch, int act_dtype, const void* branch_weight,
                                const void* branch_bias, float branch_eps, int branch_mean, const void* weight,
                                const void* bias, int weight_dtype, float eps, int use_mean, void* out, const int* rows,
                                int n_out, int width, hipStream_t stream);
// out[t, 0:n] = x[t, col0 : col0 + n] / rms * weight for float32 rows ldx apart
int fmsamd_rms_norm_cols(const float* x, long ldx, int col0, int n, const void* weight, int weight_dtype, float eps,
                         void* out, int out_dtype, long ldo, int rows, hipStream_t stream);
// out[t, 0:n] = a z / rms(z) + b z^2 / rms(z^2) + c z^3 / rms(z^3) + e (powers element by element) for float32 rows ldz apart
int fmsamd_poly_norm(const float* z, long ldz, int n, float a, float b, float c, float e, float eps, void* out, int out_dtype,
                     long ldo, int rows, hipStream_t stream);
// out = act(x), act one of FMS_ACT_*
int fmsamd_activate(const void* x, void* out, int dtype, long n, int act, hipStream_t stream);
// gu [T, 2 * hidden] (gate first): out = g' sigmoid(alpha g') (u' + shift), g' = min(g, limit), u' = clamp(u, +-limit)
int fmsamd_clamped_gated_act(const void* gu, void* out, int dtype, int n_tokens, int hidden, float limit, float alpha,
                             float shift, hipStream_t stream);

// ---- attention over a latent cache (latent_attention.hip) ---------------------------------------------------------
// The cache holds one row [rank + rot] per token: pages [page][token in page][rank + rot].
// vt_cache (or null): the latent once more, transposed, pages [page][rank][token in page], for the MFMA kernel.
// down: float32 rows whose columns col0 .. col0 + rank + rot are the latent before its norm and the shared key part
// before its rotation; the normed latent and the rotated part are written into the token's page.
int fmsamd_latent_kv_write(const float* down, long ld, int col0, int rank, int rot, const void* norm_weight,
                           int weight_dtype, float eps, const int* positions, const int* seq_of_token,
                           const int* block_table, int table_stride, const float* cos_t, const float* sin_t, int max_pos,
                           void* cache, void* vt_cache, int cache_dtype, int n_tokens, hipStream_t stream);
// qa[t, h, rank : rank + rot] = rotate(q[t, h, dim : dim + rot]); q rows hold nheads x (dim + rot), qa rows nheads x (rank + rot)
int fmsamd_latent_q_rotate(const void* q, long ldq, int dtype, int nheads, int dim, int rot, void* qa, long ldqa, int rank,
                           const int* positions, const float* cos_t, const float* sin_t, int max_pos, int n_tokens,
                           hipStream_t stream);
// y[t, h, 0:N] = W[h] x[t, h, 0:K] (W [nheads, N, K]), times sigmoid(gate[t * ldg + h]) if gate is given
int fmsamd_headwise_linear(const void* x, long ldx, long x_head_stride, const void* w, void* y, long ldy,
                           long y_head_stride, const float* gate, long ldg, int dtype, int n_tokens, int nheads, int N,
                           int K, hipStream_t stream);
// out[t, h, 0:rank] = sum_j p_j cache[j, 0:rank], p = softmax over the visible keys j (and the sink, if given: float32
// [nheads], unscaled, in the denominator only) of scale * qa[t, h, :] . cache[j, :]
int fmsamd_latent_attn_generic(const void* qa, long ldq, void* out, long ldo, int dtype, const int* positions,
                               const int* seq_of_token, const int* block_table, int table_stride, const void* cache,
                               const float* sink, int n_tokens, int nheads, int rank, int rot, float scale, int window,
                               hipStream_t stream);

// The same attention for bfloat16 on the matrix cores (sizes: fmsamd_latent_attn_mfma_fits).  n_splits 0: prompts;
// n_splits >= 1: single tokens, every (token, 16 heads) dealt over n_splits blocks of four waves, partial results in
// a workspace of fmsamd_latent_attn_workspace(...) bytes, merged by a second kernel.
long fmsamd_latent_attn_workspace(int n_tokens, int nheads, int rank, int n_splits);
int fmsamd_latent_attn_mfma_fits(int rank, int rot);
int fmsamd_latent_attn_mfma(const void* qa, long ldq, void* out, long ldo, void* workspace, long workspace_bytes,
                            const int* positions, const int* seq_of_token, const int* block_table, int table_stride,
                            const void* cache, const void* vt_cache, const float* sink, int n_tokens, int nheads, int rank,
                            int rot, float scale, int window, int n_splits, hipStream_t stream);

// ---- experts (experts.hip) -----------------------------------------------------------------------------------------
// ids: the `top` largest logits of every token; weights: FMS_ROUTE_SOFTMAX the softmax over the chosen logits,
// FMS_ROUTE_SIGMOID each chosen logit's sigmoid, FMS_ROUTE_SIGMOID_NORMED those divided by their sum.
#define FMS_ROUTE_SOFTMAX 0
#define FMS_ROUTE_SIGMOID 1
#define FMS_ROUTE_SIGMOID_NORMED 2
int fmsamd_moe_route(const float* logits, long ld, int n_tokens, int n_experts, int top, int score, int* ids, float* weights,
                     hipStream_t stream);
// Rows of a tile of (token, choice) pairs of one expert: 64 where experts have many rows and the matrix-core kernel can
// run (wide_ok), else 16; the most tiles there can be; the pairs sorted by expert and cut into tiles:
// order [n_pairs], tiles [max_tiles][3] = (expert, first row in order, rows).
int fmsamd_moe_tile_rows(int n_pairs, int n_experts, int wide_ok);
int fmsamd_moe_max_tiles(int n_pairs, int n_experts, int tile_rows);
int fmsamd_moe_group(const int* ids, int n_pairs, int n_experts, int* order, int* tiles, int max_tiles, int tile_rows,
                     hipStream_t stream);
// stage 0: y[sorted pair] = act(s x Wg^T, s x Wu^T) (w1, w2 = gate, up [E, N, K]; s = in_scale[pair], or 1 if null: a
// weight on the expert's input, applied to the float32 sums); stage 1: y[pair] = x W^T, float32
// With w2 null at stage 0 the experts have no gate: y[sorted pair] = act(s x W1^T), act one of FMS_ACT_*.
int fmsamd_moe_experts(int stage, const void* x, long ldx, const void* w1, const void* w2, void* y, int dtype,
                       const int* order, const int* tiles, int max_tiles, int tile_rows, int top, int N, int K, float limit,
                       float alpha, float shift, const float* in_scale, int act, hipStream_t stream);
// weights null: the plain sum of a token's rows.  ids (or null) [T, top] with n_experts: a choice of n_experts or more is
// an identity expert, whose output is the token's input x_in [T, ldx] (of the output's type) instead of a row of y.
int fmsamd_moe_combine(const float* y, const float* weights, int top, const void* shared, const float* shared_gate, long ldg,
                       void* out, int dtype, int n_tokens, int width, const int* ids, int n_experts, const void* x_in, long ldx,
                       hipStream_t stream);
// Routing over groups: s = softmax over all n_outputs logits; outputs are chosen by s + correction (float32 [n_outputs] or
// null) among the `keep` groups (of `groups` equal runs of neighbours) whose largest choice score is largest; the weights
// are the chosen outputs' s over their sum (+ 1e-20), times scale.
int fmsamd_moe_route_grouped(const float* logits, long ld, int n_tokens, int n_outputs, int top, const float* correction,
                             int groups, int keep, float scale, int* ids, float* weights, hipStream_t stream);

// ---- steps around attention (attention_extras.hip) ------------------------------------------------------------------
// float32 rows [q (nq) | k (nk) | v (nv)]: out = [q / rms(q) * wq | k / rms(k) * wk | v], each norm over its whole run of
// columns; rows whose seq_of_token is negative are skipped (seq_of_token null: none are).  norm_dim > 0: the norms run
// over every run of norm_dim columns (a head) by itself, with weights of norm_dim entries that all heads share.
// v_first (rows of out's type, ld_first apart, or null) and v_lambda (one float32 number on the device): the values
// leave as (1 - lambda) v + lambda v_first.
int fmsamd_qk_projection_norm(const float* proj, long ld, int nq, int nk, int nv, const void* wq, const void* wk,
                              int weight_dtype, float eps, void* out, int out_dtype, long ldo, const int* seq_of_token,
                              int n_tokens, int norm_dim, const void* v_first, long ld_first, const void* v_lambda,
                              hipStream_t stream);
// out = x * act(gate) * scale (gate: float32 logits or null); group > 1: one gate column for every run of `group` columns
// of x (a gate per head)
int fmsamd_gate_mul(const void* x, long ldx, const float* gate, long ldg, int act, float scale, void* out, long ldo,
                    int dtype, int n_tokens, int cols, int group, hipStream_t stream);
int fmsamd_scale_f32(float* x, long n, float s, hipStream_t stream);
// out[t, 0:n] = x[t, 0:n] (x: float32 rows ldx apart, already offset to the first column) in out_dtype
int fmsamd_cast_cols(const float* x, long ldx, void* out, int out_dtype, long ldo, int n_tokens, int n, hipStream_t stream);

// ---- the gated delta rule (delta_rule.hip) ------------------------------------------------------------------------------
// proj: float32 rows whose first C = 2*kv_heads*dim + heads*vdim columns are the q, k and v channels before the
// convolution and whose columns col_b .. col_b + heads are the logits of beta; a: rows with the decay's input at col_a
// (heads columns, or heads*dim if per_channel); conv_w [C, taps]; conv_state [slots][taps-1][C] is read, then updated.
// Writes qkv [T, C] (convolved, silu, q and k unit vectors per head, q times q_scale), beta [T, heads] and
// decay [T, heads (*dim)] = exp(-exp(a_log) softplus(a + dt_bias)), and kq [T, kv_heads] = k . q of the finished vectors.
int fmsamd_delta_prepare(const float* proj, long ld, int col_b, const float* a, long lda, int col_a, const void* conv_w,
                         int conv_dtype, int taps, const float* a_log, const float* dt_bias, float* conv_state,
                         const int* seq_of_token, const int* slot_ids, float* qkv, float* beta, float* decay, float* kq,
                         int n_tokens, int heads, int kv_heads, int dim, int vdim, int per_channel, float q_scale,
                         hipStream_t stream);
// The recurrence over every sequence's tokens of the step (seq_starts [n_seqs + 1]); state [slots][heads][vdim][dim]
// is read and written; out [T, heads*vdim].  single_tokens != 0: the caller knows that no sequence brings more than one
// token, and the kernel stages accordingly (the result is the same either way).
int fmsamd_delta_rule(const float* qkv, const float* beta, const float* decay, const float* kq, float* state, float* out,
                      const int* seq_starts, const int* seq_of_token, const int* slot_ids, int n_seqs, int heads,
                      int kv_heads, int dim, int vdim, int per_channel, int single_tokens, hipStream_t stream);
// out[t, h, :] = o[t, h, :] / rms * weight * act(gate[t, h, :]) * out_scale
int fmsamd_gated_head_norm(const float* o, const float* gate, long ldg, const void* weight, int weight_dtype, float eps,
                           int act, float out_scale, void* out, int out_dtype, long ldo, const int* seq_of_token,
                           int n_tokens, int heads, int vdim, hipStream_t stream);

// ---- norms behind the branches only, short convolutions (post_norm.hip) --------------------------------------------
// resid += gnorm(branch) * branch_weight (branch null: nothing is added; written back unless `rows` is given), where gnorm
// divides each of branch_groups equal consecutive parts of a row by its own root mean square (branch_groups 0: the branch
// is added as it is); then out is nothing, the
// stream in the activation type, or gnorm(resid) * weight with `groups` parts.
#define FMS_CHAIN_NONE 0
#define FMS_CHAIN_CAST 1
#define FMS_CHAIN_NORM 2
int fmsamd_group_norm_chain(float* resid, const void* branch, int act_dtype, const void* branch_weight, int branch_weight_dtype,
                            int branch_groups, float branch_eps, const void* weight, int weight_dtype, int groups, float eps,
                            void* out, int out_mode, const int* rows, int n_out, int width, hipStream_t stream);
// out[t, c] = (x[t, c] if add_input) + bias[c] + sum_j conv_w[c, j] x[t - taps + 1 + j, c] over a sequence's own tokens; the
// inputs before the step come from conv_state [slots][taps-1][channels] (float32), which is then moved on.  x: float32 rows.
// single_tokens: the caller knows that every sequence brings one token (a short step then needs no second kernel for the state).
int fmsamd_short_conv(const float* x, long ld, int channels, const void* conv_w, const void* bias, int weight_dtype, int taps,
                      float* conv_state, const int* seq_of_token, const int* slot_ids, int add_input, void* out, int out_dtype,
                      long ldo, int n_tokens, int single_tokens, hipStream_t stream);

// ---- the real-gated linear recurrent unit (rglru.hip) -------------------------------------------------------------------
// u: float32 rows; ra_t, ri_t [blocks][in][out] (transposed square matrices), ra_b, ri_b, lam float32 [channels];
// a = exp(-c sigmoid(Ra u + ba) softplus(lam)), b = sqrt(1 - a^2) sigmoid(Ri u + bi) u, both float32 [T, channels].
int fmsamd_rglru_gates(const float* u, long ldu, const void* ra_t, const float* ra_b, const void* ri_t, const float* ri_b,
                       int weight_dtype, const float* lam, float c, const int* seq_of_token, float* a_out, float* b_out,
                       int n_tokens, int channels, int blocks, hipStream_t stream);
// S <- a S + b over every sequence's tokens of the step (seq_starts [n_seqs + 1]), from and into state [slots][channels];
// out[t] = S * act(y[t]) (y: float32 rows ldy apart).
int fmsamd_rglru_scan(const float* a, const float* b, const float* y, long ldy, int act, float* state, const int* seq_starts,
                      const int* seq_of_token, const int* slot_ids, void* out, int out_dtype, long ldo, int n_seqs, int channels,
                      hipStream_t stream);
// Long sequences: the same walk in chunks of token rows that run side by side.  fmsamd_rglru_scan_chunk says how many rows a
// chunk has for a step (0: walk sequence by sequence); workspace: float32 [(2 * ceil(n_tokens / chunk) + n_seqs) * channels].
int fmsamd_rglru_scan_chunk(int n_tokens, int n_seqs);
int fmsamd_rglru_scan_chunked(const float* a, const float* b, const float* y, long ldy, int act, float* state, const int* seq_starts,
                              const int* seq_of_token, const int* slot_ids, void* out, int out_dtype, long ldo, int n_tokens,
                              int n_seqs, int channels, int chunk, float* workspace, hipStream_t stream);

#ifdef __cplusplus
}
#endif
