// C entry points of the kernel library.  Every function takes device pointers and a HIP
// stream, launches asynchronously on it, returns 0 on success and a non-zero code after
// leaving a message for ia_last_error().  dtype arguments: 0 = float32, 1 = bfloat16.
#pragma once

#include <hip/hip_runtime.h>

#define IA_ABI_VERSION 1

#ifdef __cplusplus
extern "C" {
#endif

const char* ia_last_error(void);
int ia_abi_version(void);

int ia_embed_gather(void* out, const void* table, const int* ids, int n, int hidden, int vocab,
                    int dtype, hipStream_t stream);
int ia_gather_rows(void* out, const void* x, const int* rows, int n, int cols, int dtype,
                   hipStream_t stream);
int ia_rmsnorm(void* out, const void* x, const float* w, float eps, int rows, int cols,
               int add_one, int dtype, hipStream_t stream);
int ia_add_rmsnorm(void* out, void* x, const void* delta, const float* w, float eps, int rows,
                   int cols, int add_one, int dtype, hipStream_t stream);
int ia_add_inplace(void* x, const void* delta, long long n, int dtype, hipStream_t stream);
int ia_fill_normal(void* out, long long n, unsigned long long seed, double mean, double std,
                   int dtype, hipStream_t stream);
int ia_widen_bf16(float* out, const void* x, long long n, hipStream_t stream);
// rows of [gate | up] -> act(gate) * up; act: 1 SiLU, 2 GELU in its tanh form (the same numbers name the activation
// in the `dual` argument of the products below, where 0 means a plain product)
int ia_gate_mul(void* out, const void* gu, int rows, int inter, int act, int dtype, hipStream_t stream);
// x[row][c] += bias[c] in place (x and bias in the same precision)
int ia_add_bias(void* x, const void* bias, int rows, int cols, int dtype, hipStream_t stream);
// A pure streaming read of `bytes` bytes by `blocks` blocks (one word of `out` a block): the measurement script's
// measured memory roof.  Nothing of the engine calls it.
int ia_stream_read(unsigned* out, const void* x, long long bytes, int blocks, hipStream_t stream);
int ia_rope_table(float* cos_out, float* sin_out, const int* positions, const float* inv_freq,
                  int n, int half, hipStream_t stream);

int ia_qk_rope_kv(void* q_out, void* k_cache, void* v_cache, const void* qkv,
                  const float* q_norm_w, const float* k_norm_w, const float* cos_t,
                  const float* sin_t, const int* slots, int n, int nq, int nkv, int d, int rot,
                  int interleaved, int page_size, float eps, int add_one, int dtype,
                  hipStream_t stream);

// The same on rows of any layout (`ld_` elements a row: queries from q_off, keys from k_off, values of width dv from v_off; k_off < 0:
// no keys or values, the layer reads another layer's cache)
int ia_qk_rope_kv_strided(void* q_out, void* k_cache, void* v_cache, const void* proj, const float* q_norm_w,
                          const float* k_norm_w, const float* cos_t, const float* sin_t, const int* slots, int n,
                          int ld_, int q_off, int k_off, int v_off, int nq, int nkv, int d, int dv, int rot,
                          int interleaved, int page_size, float eps, int add_one, int dtype, hipStream_t stream);

// d: the keys' width, dv: the values' (v_cache [pages, nkv, dv, page_size], out [n, nq, dv])
// sink: 1 adds exp(0) to the softmax's denominator (a key of score 0 that has no value); the same in the matrix-core kernels.
// sinks: with sink, null or [nq] 32-bit values s_h, one a query head: the term is exp(s_h) instead (not scaled); mask_chunk > 0: a
// query sees the keys of its own chunk of that many positions only (chunks counted from position 0), up to itself.
// workspace: null, or ia_attention_generic_workspace(...) floats when that is not 0 (steps of few tokens: a wave a
// segment of keys and a merge kernel, the same bits as without); max_kv_len: an upper bound of positions + 1
int ia_attention_generic(void* out, const void* q, const void* k_cache, const void* v_cache,
                         const int* positions, const int* token_seq, const int* block_table,
                         int n, int max_pages, int nq, int nkv, int d, int dv, int page_size, int window,
                         float scale, int dtype, float* workspace, int max_kv_len, int sink, int mask_chunk,
                         const float* sinks, hipStream_t stream);
long long ia_attention_generic_workspace(int n, int nq, int nkv, int d, int dv, int max_kv_len);

int ia_gemm_tiled(void* out, const void* x, const void* w, int M, int N, int K, int in_dtype,
                  int out_dtype, hipStream_t stream);
// bias: bfloat16 [N] ([2 N] with dual), or null
// (ia_gemm_tiled at up to 64 rows: the shape of its kernel for few rows, 100 * output features + staged rows a wave:
// 816, 808, 416 or 1608; 0: the kernel's own rule)
int ia_gemm_rows_tune(int shape);
int ia_gemm_skinny_bf16(void* out, const void* x, const void* w, const void* bias, int M, int N, int K,
                        int out_dtype, int dual, hipStream_t stream);
// Large bfloat16 products through the vendor's library, hipBLASLt, called directly (vendor_gemm.hip).  ia_vendor_gemm_init
// opens the library at `path` (the copy the process already holds) once; ia_vendor_gemm_bf16: out [M, N] = x [M, K] . w [N, K]^T,
// contiguous, with `workspace_bytes` of device memory for kernels that want some.
#define IA_VENDOR_NO_KERNEL 2     // ia_vendor_gemm_bf16: the library's search names no kernel for this shape
int ia_vendor_gemm_init(const char* path);
int ia_vendor_gemm_ready(void);
int ia_vendor_gemm_bf16(void* out, const void* x, const void* w, int M, int N, int K, void* workspace,
                        long long workspace_bytes, hipStream_t stream);
// Large bfloat16 products in tiles of 256 x 256 (gemm_mfma.hip); K a multiple of 64; with `dual` w is [gate; up]
// and out = act(x . gate^T) * (x . up^T).
int ia_gemm_mfma_bf16(void* out, const void* x, const void* w, int M, int N, int K, int dual, hipStream_t stream);
// Tuning knobs of the skinny product (tests switch the staged variants off with stage = 0); the defaults are
// (2048, 8, 5, 8, 1).
void ia_gemm_skinny_tune(int target_waves, int min_ksteps, int rot_mul, int min_waves, int stage);
// The skinny product with a residual stream around it (decode steps; see gemm.hip): adds itself to `resid`
// and leaves the rows' sums of squares and the rows times the next norm's weight, and / or takes such rows
// and finishes their norm.
// (the sums of squares come block by block: ia_gemm_skinny_blocks(N) blocks of ia_gemm_skinny_block_rows(N)
// neighbouring features each, a choice that depends on N and on the chip's number of compute units)
int ia_gemm_skinny_blocks(int N);
int ia_gemm_skinny_block_rows(int N);
int ia_gemm_skinny_stream(void* out, const void* x, const void* w, const void* bias, int M, int N, int K, int out_dtype,
                          int dual, void* resid, float* sums_out, void* scaled_out, const float* next_w,
                          int add_one, const float* sums_in, int n_sums, float eps, hipStream_t stream);

// Products of 17 to 128 bfloat16 rows (gemm_mid.hip); K a multiple of 128.  out_mode 0: out [M, N] bfloat16; 1: float;
// 2: out [ia_gemm_mid_splits(N, K)][M][N] float, the sums of each split of k, to be added up by the reader
// (ia_sum_partials, ia_add_rmsnorm_partials).  dual: w = [gate; up], out = act(x . gate^T) * (x . up^T), mode 0.
int ia_gemm_mid_splits(int N, int K);
// whether the weight's blocks fill the chip evenly, one a compute unit (dual: [gate; up] of N features each)
int ia_gemm_mid_fills(int N, int K, int dual);
// (a fixed pipeline for measurements and tests: k steps of a chunk, 2 or 4, and stages, 2 to 4; (0, 0): the kernel's own
// rule; no product depends on it bit for bit); anything else is an error and changes nothing
int ia_gemm_mid_tune(int kc, int ns);
// (how a block's waves share its products, for measurements and tests: 0 the kernel's own rule, 1 a tile of weight rows a
// wave over all rows of the step, 2 two tiles a wave over half of the rows wherever the shape allows; the same bits)
int ia_gemm_mid_blocking(int how);
// (a fixed shape of the blocks for measurements and tests: waves a block, 2 to 8 (0: the kernel's own rule), ways k is split
// and stages, 2 or 3 (2: four waves only); the caller's partial sums must have as many splits); a shape that has no
// kernel is an error and changes nothing
int ia_gemm_mid_plan(int waves, int splits, int stages);
int ia_gemm_mid_bf16(void* out, const void* x, const void* w, int M, int N, int K, int out_mode, int dual,
                     hipStream_t stream);
// the same for up to 16 rows that are a norm's input times its weight, with their sums of squares sums_in [M][n_sums]: every sum
// of the product is multiplied by the row's rsqrt(sum of sums_in / K + eps); out_mode 0 or 1
int ia_gemm_mid_bf16_scaled(void* out, const void* x, const void* w, int M, int N, int K, int out_mode, int dual,
                            const float* sums_in, int n_sums, float eps, hipStream_t stream);
int ia_sum_partials(void* out, const float* part, int splits, int M, int N, hipStream_t stream);
// x += (sum of the splits, rounded to bfloat16) in place, out = rmsnorm(x) * w; bfloat16 rows of up to 8192 features.
int ia_add_rmsnorm_partials(void* out, void* x, const float* part, int splits, const float* w, float eps,
                            int rows, int cols, int add_one, hipStream_t stream);

long long ia_argmax_workspace(int rows, int vocab);
int ia_argmax(int* out, const float* logits, void* workspace, int rows, int vocab, hipStream_t stream);
// The arg max without any allocation.  It has no counterpart in the reference; it is for callers that cannot
// allocate device memory: code under HIP graph capture, tight serving loops, harnesses that forbid it.  The
// two-step kernels' candidates go to an array of ia_argmax_static_capacity() 32-bit words (64 KiB) that the
// library holds in each GPU's memory until the process ends, instead of a workspace of the caller's; sizes for
// which ia_argmax_workspace(rows, vocab) exceeds that are refused with an error (about 430 rows at a
// vocabulary of 152 k).  No hipMalloc, hipFree or allocating library call happens inside.  All calls on one GPU
// share that GPU's array: calls that overlap on one GPU (two streams, two threads) race; calls on one stream do not.
long long ia_argmax_static_capacity(void);
int ia_argmax_static(int* out, const float* logits, int rows, int vocab, hipStream_t stream);
int ia_penalize(float* logits, int rows, int vocab, const int* window, int w, const float* rep,
                const float* freq, const float* pres, const int* bias_ids, const float* bias_vals,
                int nb, hipStream_t stream);
int ia_window_push(int* window, int rows, int w, const int* caps, const int* tokens, hipStream_t stream);
long long ia_sample_workspace(int rows, int vocab);
int ia_sample_max_top(void);
// n_top, lp_out [rows, 1 + max_top], lp_ids [rows, max_top]: all null, or the log-probabilities asked for per row
int ia_sample(int* out, const float* logits, void* workspace, int rows, int vocab,
              const float* temperature, const int* top_k, const float* top_p, const float* min_p,
              const float* u, const int* n_top, float* lp_out, int* lp_ids, hipStream_t stream);

// ---- several residual streams a token (streams.hip) ------------------------------------------------------------
// streams: 32-bit [n, S, W].  One call adds a sub-layer's output into the streams (x_t <- sum_s mix[s][t] x_s +
// out[t] * scale * y; y null: skipped; y may be K rows a token with 32-bit weights yw) and forms the next
// sub-layer's input h = rmsnorm(sum_s in[s] x_s) * w (h null: skipped; rows: only these rows, for a call without y).
int ia_streams_step(float* streams, const void* y, const float* yw, int K, const float* scale,
                    const float* mix, const float* outc, const float* inc, const float* w, float eps,
                    void* h, const int* rows, int n, int S, int W, int y_dtype, int h_dtype, hipStream_t stream);
int ia_streams_open(float* streams, const void* x, int n, int S, int W, int dtype, hipStream_t stream);
int ia_softcap(float* x, long long n, float cap, hipStream_t stream);

// ---- latent attention (latent.hip) -------------------------------------------------------------------------------
int ia_latent_prep(void* q_out, void* k_cache, void* v_cache, const void* proj, const float* norm_w,
                   const float* cos_t, const float* sin_t, const int* slots, int n, int H, int d, int r,
                   int rank, int rd, int q_off, int down_off, int ld_proj, int page_size, float eps,
                   float mag, int interleaved, const void* qrows, int ld_q, int dtype, hipStream_t stream);
// out[t][j] = x[t][x_off + j] / sqrt(mean_j x[t][x_off + j]^2 + eps) * w[j], j < cols: the RMS norm of a slice of rows of pitch x_ld
int ia_norm_slice(void* out, const void* x, long long x_ld, int x_off, const float* w, float eps, int rows, int cols,
                  int dtype, hipStream_t stream);
// out[t][h][j] = sum_i w[h][j][i] x[t][h][i], optionally times sigmoid(gate[t][h][j]), or, with g_per_head, sigmoid(gate[t][h])
int ia_head_product(void* out, const void* x, const void* w, const void* gate, int n, int H, int n_out,
                    int k_in, long long x_ld, int x_off, int x_head, long long o_ld, int o_off, int o_head,
                    long long g_ld, int g_off, int g_per_head, int x_dtype, int w_dtype, int out_dtype, hipStream_t stream);

// ---- gated linear recurrence behind a short convolution (recurrence.hip) ----------------------------------------
// u_lo: null, or a bfloat16 copy of u (for products that take it in that precision)
int ia_conv_step(float* u, void* u_lo, const void* x, const void* taps, const void* bias, const float* state,
                 const int* token_seq, const int* cu_tokens, const int* state_slots, int n, int width, int k,
                 long long x_ld, int x_off, int dtype, hipStream_t stream);
int ia_rglru_scan(void* out, float* state, const float* u, const float* z, const void* bias_r,
                  const void* bias_i, const void* lam, const void* branch, const void* x,
                  const int* cu_tokens, const int* state_slots, int n_seqs, int width, int bw, int k,
                  float decay, long long b_ld, int b_off, long long x_ld, int x_off, int dtype,
                  hipStream_t stream);
// the same for long portions: chunks of 64 tokens side by side (rounding apart, the same result); `work` holds
// ia_rglru_chunked_workspace(...) 32-bit words
long long ia_rglru_chunked_workspace(int n, int n_seqs, int width);
int ia_rglru_scan_chunked(void* out, float* state, float* work, const float* u, const float* z,
                          const void* bias_r, const void* bias_i, const void* lam, const void* branch,
                          const void* x, const int* cu_tokens, const int* state_slots, int n, int n_seqs,
                          int width, int bw, int k, float decay, long long b_ld, int b_off, long long x_ld,
                          int x_off, int dtype, hipStream_t stream);

// ---- routed experts (experts.hip) --------------------------------------------------------------------------------
// score_fn: 0 sigmoid, 1 softmax over all experts.  tile: rows of a row tile, 32, 64 or 128 (the plan, gate_up and down
// of one call agree).  tiled: the weights are stored as tiles of 64 features x 64 k values, zero-padded: w_gu
// [E][2][ceil(ff / 64)][ceil(W / 64)][64][64], w_down [E][ceil(W / 64)][ceil(ff / 64)][64][64] (bfloat16, matrix cores);
// else w_gu [E][2 ff][W], w_down [E][W][ff].
// choice_bias: null, or [E] 32-bit values that count in the choice only (score + bias picks, the score weighs).  The plan
// gives a pair whose choice is E or beyond (an output of the router that names no expert with weights) no place and no tile.
int ia_route(int* sel, float* weight, const void* h, const void* router, int n, int W, int E, int top,
             float scale, int score_fn, int renorm, const float* choice_bias, int gates, float* gate_out, int dtype,
             hipStream_t stream);
int ia_route_tiles(int pairs, int E);
int ia_route_plan(int* order, int* tile_expert, int* tile_first, int* tile_rows, int* meta, const int* sel,
                  int pairs, int E, int tile, hipStream_t stream);
int ia_experts_gate_up(void* act, const void* h, const void* w_gu, const int* order, const int* tile_expert,
                       const int* tile_first, const int* tile_rows, const int* meta, int pairs, int E, int top,
                       int W, int ff, float limit, float alpha, int tile, int tiled, const float* in_weight, int dtype,
                       hipStream_t stream);
int ia_experts_down(float* y, const void* act, const void* w_down, const int* order, const int* tile_expert,
                    const int* tile_first, const int* tile_rows, const int* meta, int pairs, int E, int W,
                    int ff, int tile, int tiled, int dtype, hipStream_t stream);

// A 32-bit residual stream whose sub-layers stand between two norms (sandwich.hip): x += rmsnorm(s1 y1 + s2 y2) * w_post;
// x += e_rows + e_vec; h = rmsnorm(x) * w_pre.  Every half may be null.  With `rows` only the named rows are read and the
// stream is not written.  y_dtype: precision of y1, y2, e_rows; h_dtype: of h.
int ia_sandwich_step(float* x, const void* y1, float s1, const void* y2, float s2, const float* w_post,
                     const void* e_rows, const float* e_vec, const float* w_pre, float eps_post, float eps, void* h,
                     const int* rows, int n, int W, int y_dtype, int h_dtype, hipStream_t stream);
// act over every element in place: 1 SiLU, 2 GELU in its tanh form, 3 the exact GELU
int ia_activation(void* x, long long n, int act, int dtype, hipStream_t stream);

// A 32-bit residual stream whose sub-layers all read one normed copy (parallel.hip): x += y1 + y2 + sum_k [routed_w[k]] routed[k]
// + y3_scale y3; x += rmsnorm(enter) * enter_w; h = norm(x) (a layer norm with weight and bias, or with center 0 an RMS norm):
// every part optional, one kernel.  y_dtype: of y1, y2, y3, enter; h_dtype: of xr (the new x once more) and h.  rows: only these
// rows through the norm, nothing added, the stream left alone.
int ia_parallel_step(float* x, const void* y1, const void* y2, const void* y3, int y1_splits, int y2_splits, int y3_splits,
                     const float* y3_scale, const float* routed, const float* routed_w, int top, const void* enter,
                     const float* enter_w, float enter_eps, void* xr, const float* norm_w, const float* norm_b, float norm_eps,
                     int center, void* h, const int* rows, int n, int W, int y_dtype, int h_dtype, hipStream_t stream);
// out[t][c] = act(g[t][c]) * e[t][e_off + c]; act: 1 SiLU, 2 GELU in its tanh form
int ia_gate_rows(void* out, const void* g, const void* e, int rows, int cols, long long e_ld, int e_off, int act, int dtype,
                 hipStream_t stream);
// A 32-bit residual stream that is normed after every sum (postnorm.hip): x <- rmsnorm(alpha x + y + sum_k routed_w[k] *
// routed[k] + y2) * w, written back in 32-bit and to h (h_dtype; null: not wanted); every addend may be null.  routed
// [n, top, W] 32-bit with weights [n, top]; a pair whose sel (null: none) is real_experts or more stands for the stream's
// own row.  rows: only these rows are read, the stream is left alone and h gets one row for each.
// y_splits, y2_splits: 1, or y (y2) is a 32-bit product still split along its k, [splits, n, W], added up here.
int ia_postnorm_step(float* x, float alpha, const void* y, const void* y2, int y_splits, int y2_splits, const float* routed,
                     const float* routed_w, const int* sel, int top, int real_experts, const float* w, float eps,
                     void* h, const int* rows, int n, int W, int y_dtype, int h_dtype, hipStream_t stream);
// out (32-bit) = table[ids] * scale; h (null: not wanted): the same rows in the table's precision
int ia_embed_gather_scaled(float* out, void* h, const void* table, const int* ids, int n, int hidden, int vocab,
                           float scale, int dtype, hipStream_t stream);
// a[row][c] *= sigmoid(g[row * g_ld + g_off + c]) in place, a [rows, cols]
int ia_sigmoid_gate(void* a, const void* g, int rows, int cols, int g_ld, int g_off, int group, int dtype, hipStream_t stream);
// rows of [gate | up] -> g' * sigmoid(slope g') * (u' + 1) with g' = min(gate, limit), u' = clamp(up, -limit, limit)
int ia_clamped_gate_mul(void* out, const void* gu, int rows, int inter, float limit, float slope, int dtype,
                        hipStream_t stream);
int ia_scale(float* x, long long n, float factor, hipStream_t stream);
// Mixers with a matrix state a head (linear_state.hip).  A request's state is its row of `state` [slots][row_floats];
// every kernel takes the offset of its part of the row.
int ia_conv_act_step(void* out, const void* x, const void* taps, const void* bias, float* state,
                     long long row_floats, long long tail_off, const int* token_seq, const int* cu_tokens,
                     const int* state_slots, int n, int n_seqs, int C, int k, long long x_ld, int x_off, int act,
                     int dtype, hipStream_t stream);
int ia_exp_gates(float* log_a, float* b, float* floor_, float* state, long long row_floats, long long m_off,
                 const void* proj, long long p_ld, int i_off, int f_off, const float* bias_i,
                 const float* bias_f, float cap, const int* cu_tokens, const int* state_slots, int H,
                 int n_seqs, int max_q_len, int dtype, hipStream_t stream);
int ia_step_gates(float* log_a, float* b, const void* proj, long long p_ld, int dt_off, const float* dt_bias,
                  const float* a_log, int n, int H, int dtype, hipStream_t stream);
// S <- a S + b k v^T, o = S^T q (+ skip v); `den` not null: one more column of S whose value is always 1.
// log_a: [n][H] logarithms of the decays (a_per_token 1) or the decays themselves, [H] (a_per_token 0).
// chunk > 0: portions run in chunks of that many tokens side by side (workspace: ia_linear_scan_workspace floats; max_q_len:
// an upper bound of a request's tokens); the results differ from the walk (chunk 0) by rounding.
int ia_linear_scan(float* out, float* den, float* state, long long row_floats, long long s_off,
                   const void* q, long long q_ld, int q_off, int q_heads,
                   const void* k, long long k_ld, int k_off, int k_heads,
                   const void* v, long long v_ld, int v_off,
                   const float* log_a, int a_per_token, const float* b, const float* skip,
                   const int* cu_tokens, const int* state_slots, int n_seqs, int H, int dim, int vdim,
                   float q_scale, float k_scale, int chunk, int max_q_len, float* workspace, int dtype,
                   hipStream_t stream);
long long ia_linear_scan_workspace(int n_seqs, int max_q_len, int chunk, int H, int dim, int vdim, int normaliser);
// 1 (the default): what a chunk's start contributes is formed on the matrix cores in true 32-bit (keys up to 128, chunks up
// to 64 tokens); 0: on the vector units
void ia_linear_scan_tune(int carry_mfma);
// [o / (max(|den|, floor) + 1e-6)] [* act(gate)] -> RMS norm in groups of `group` features [* w] [* act(gate)]; act: 1 SiLU, 4 sigmoid
int ia_group_norm_gate(void* out, const float* o, const float* den, const float* floor_, int head,
                       const void* gate, long long g_ld, int g_off, int act, int gate_first, const float* w,
                       float eps, int n, int inner, int group, int dtype, hipStream_t stream);

// Built per head size (-DIA_HEAD_DIM) into a library of its own.
int ia_attention_mfma_head_dim(void);
int ia_attention_mfma_value_dim(void);     // the values' width this library was built for (IA_VALUE_DIM; the keys' unless given)
long long ia_attention_mfma_workspace(int n, int nq, int splits);
int ia_attention_mfma(void* out, float* workspace, const void* q, const void* k_cache,
                      const void* v_cache, const int* block_table, const int* cu_tokens,
                      const int* positions, int n, int seq_begin, int n_seqs, int token_begin,
                      int n_tokens, int max_q_len, int max_kv_len, int max_pages,
                      int nq, int nkv, int d, int page_size, int window, float scale,
                      int splits, int chunk, int sink, int mask_chunk, const float* sinks, hipStream_t stream);
// Decode steps (one token a request, head sizes in steps of 64): per-head norm, rotation, cache write, attention
// and the merge of the key splits in one kernel.  `workspace` holds ia_attention_decode_workspace() floats;
// `counters` holds at least ia_attention_decode_counters() 32-bit words that are zero before the call and zero
// again after it (calls that share them must not overlap).
int ia_attention_mfma_has_fused(void);
long long ia_attention_decode_workspace(int n, int nq, int nkv, int splits);
long long ia_attention_decode_counters(int n, int nq, int nkv, int splits);
int ia_attention_mfma_decode_fused(void* out, float* workspace, const void* qkv, void* k_cache,
                                   void* v_cache, const int* block_table, const int* cu_tokens,
                                   const int* positions, const int* slots, const float* q_norm_w,
                                   const float* k_norm_w, const float* cos_t, const float* sin_t,
                                   float eps, int add_one, int n, int seq_begin, int n_seqs,
                                   int token_begin, int n_tokens, int max_kv_len, int max_pages,
                                   int nq, int nkv, int d, int page_size, int window, float scale,
                                   int splits, int chunk, int sink, int* counters, int n_counters, hipStream_t stream);

#ifdef __cplusplus
}
#endif
