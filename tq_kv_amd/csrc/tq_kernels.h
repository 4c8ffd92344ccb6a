/* C entry points of the gfx950 kernel library.
 *
 * In the manner of the reference's C boundary (tq-kv/include/tq_kv.h:27-84): plain
 * C types, int32 status (0 ok, -1 error), a message for the last error.  Pointers
 * are device pointers unless said otherwise; `stream` is a hipStream_t.  Every
 * entry point checks its sizes on the host and refuses what its kernel does not
 * handle; none allocates.
 *
 * dtype codes: 0 = float32, 1 = bfloat16.
 */
#pragma once
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

const char* tqk_last_error(void);
int tqk_abi_version(void);
int tqk_page_size(void);                /* positions per cache page, as the kernels were built */
int tqk_skinny_max_rows(void);          /* most rows the skinny products (tqk_fused_*) take */
int tqk_mid_max_rows(void);             /* most rows tqk_mid_store and tqk_mid_gated take */
int tqk_attention_max_head_dim(void);   /* the largest head size any attention kernel here takes (tqk_attention's) */

/* Two probes of the GPU at hand, for a bench to set its figures against (the caller times the launches): a plain streaming read of
 * `bytes` bytes (a multiple of 16, 16-byte aligned) by `blocks` blocks of `threads` threads (blocks 0: two of 256 per compute unit;
 * the caller tries several shapes and keeps the best), and `turns` times four 32x32x16 bfloat16 matrix-core
 * products per wave on operands that stay in registers (*flops_out, on the host: the operations of the launch).  sink: 4 bytes of
 * device memory. */
int tqk_probe_read(const void* src, long long bytes, int blocks, int threads, void* sink, void* stream);
int tqk_probe_mfma(long long turns, void* sink, double* flops_out, void* stream);

/* dst row r = src row rows[r], rows of row_bytes bytes each (at most 65535 rows) */
int tqk_gather_rows(const void* src, const int32_t* rows, int n_rows, long long row_bytes, void* dst, void* stream);
/* x[r, :] += bias in place; x [n_rows, n], bias [n] */
int tqk_add_bias(void* x, int x_dtype, const void* bias, int bias_dtype, int n_rows, int n, void* stream);
/* dst[i] = src[i] in another dtype */
int tqk_convert(const void* src, int src_dtype, void* dst, int dst_dtype, long long n, void* stream);
/* A bfloat16 weight [n, k] (k a multiple of 32; `parts` stacked weights of n / parts rows) in the order the lanes of the
 * few-row kernels take it: out [parts * ceil(n / parts / 16)][k / 32][64][8], see tqk_fused_store. */
int tqk_pack_weight(const void* w, void* out, int n, int k, int parts, void* stream);
/* and back: rows [n, k] from the packed copy (for products of many rows, which the library takes from rows) */
int tqk_unpack_weight(const void* packed, void* rows, int n, int k, int parts, void* stream);

/* out[t, :] = scale * float(table[ids[t], :]); ids outside [0, vocab) give zeros.  copy_bf16
 * (optional): the same values as bfloat16 [tokens, hidden], times copy_weight [hidden]
 * (bfloat16) if given.  ss_out (optional, at most 16 tokens): ss_out[t] = sum of out[t]^2. */
int tqk_embed(const void* table, int table_dtype, const int32_t* ids, int n_tokens,
              int hidden, int vocab, float scale, float* out, void* copy_bf16, const void* copy_weight,
              float* ss_out, void* stream);

/* In place on float32 logits [rows, vocab]: l = (l + bias[v]) * scale, then, if cap > 0,
 * l = cap * tanh(l / cap).  bias (float32 [vocab]) may be null. */
int tqk_finish_logits(float* logits, int n_rows, int vocab, const float* bias, float scale, float cap, void* stream);

/* out[i] = std_dev * z(key, i) (+ 1 if plus_one), i < n: standard normal values that are a
 * function of the 64-bit key and the index alone, the same bits as the host's recipe gives
 * (tq_kv_amd/weights/random_init.py).  out: float32 or bfloat16 (rounded to nearest even). */
int tqk_random_normal(void* out, int dtype, long long n, uint64_t key, float std_dev, int plus_one, void* stream);

/* Row r (row index rows[r], or r if rows is NULL):
 *   v = (h ? h[row] : 0) + (delta ? delta[row] : 0);  if write_back: h[row] = v;
 *   out[r] = v / sqrt(mean(v^2) + eps) * weight          (all in float32)
 * delta and out have dtype act_dtype. */
int tqk_add_rmsnorm(float* h, const void* delta, int act_dtype, const void* weight,
                    int weight_dtype, float eps, const int32_t* rows, int n_rows,
                    int hidden, void* out, int write_back, void* stream);
/* the same, the update being a product's sums over n_sums pieces of its K (tqk_mid_store with
 * finish == 0): float32 [n_sums][sum_rows][hidden], added up in order and rounded to the
 * activation type first */
int tqk_add_rmsnorm_sums(float* h, const float* sums, int n_sums, int sum_rows, int act_dtype, const void* weight,
                         int weight_dtype, float eps, const int32_t* rows, int n_rows,
                         int hidden, void* out, int write_back, void* stream);

/* y[M,N] = x[M,K] w[N,K]^T (+ bias[N]); float32 accumulation in a fixed order that
 * does not depend on M.  Any sizes.  scratch: tqk_gemm_scratch_bytes(...) bytes of device
 * memory, 16-byte aligned (may be null: then, or where that is 0, the tiled kernel runs). */
size_t tqk_gemm_scratch_bytes(int x_dtype, int w_dtype, int bias_dtype, int y_dtype, int M, int N, int K);
int tqk_gemm(const void* x, int x_dtype, const void* w, int w_dtype, const void* bias,
             int bias_dtype, void* y, int y_dtype, int M, int N, int K, void* scratch, void* stream);

/* Skinny products (up to 16 rows, bfloat16, K a multiple of 32) with the small operations
 * around them folded in.  A norm between two products is split over them: the one that adds
 * to the stream h writes xw = bfloat16(h * weight of the next norm) and the sums of h^2 in
 * pieces (tqk_fused_residual, tqk_embed); the one that consumes the norm takes xw and the
 * pieces (ss_parts [n_ss_parts, 16]) and divides its result by sqrt(sum / K + eps).
 * w is [N, K] row by row, or with w_packed in the order the lanes take it:
 * [tile of 16 rows][K/32][64 lanes][8 values], lane = 16 * ((k % 32) / 8) + row % 16, the rows
 * padded with zeros to whole tiles (a gated weight: gate rows, then up rows, each padded). */
int tqk_fused_store(const void* x, const int32_t* x_rows, const float* ss_parts, int n_ss_parts, float eps,
                    const void* w, int w_packed, void* y, int y_dtype, int M, int N, int K, void* stream);
/* y[M, N/2] = silu(gate) * up, w = gate rows then up rows */
int tqk_fused_gated(const void* x, const float* ss_parts, int n_ss_parts, float eps, const void* w, int w_packed, void* y,
                    int M, int N, int K, void* stream);
/* h[M,N] += bfloat16(x w^T) in float32; xw_out = bfloat16(h * next_norm_w) or bfloat16(h);
 * ss_out (optional) [tqk_fused_residual_parts(N, K), 16] */
int tqk_fused_residual_parts(int N, int K);
int tqk_fused_residual_wf32(const void* x, const void* w, int w_packed, float* h, const float* next_norm_w, void* xw_out,
                            float* ss_out, int M, int N, int K, void* stream);        /* the same, the norm's weight in float32 */
int tqk_fused_residual(const void* x, const void* w, int w_packed, float* h, const void* next_norm_w, void* xw_out,
                       float* ss_out, int M, int N, int K, void* stream);
/* q, k, v of a decoding step: + bias, rotation (halves over the whole head) at tok_pos[m],
 * q to q_out [M, heads, head_dim], k and v into the cache page of sequence m */
int tqk_fused_qkv(const void* x, const float* ss_parts, int n_ss_parts, float eps, const void* w, int w_packed, const void* bias,
                  const float* cos_table, const float* sin_table, int max_positions,
                  const int32_t* tok_pos, const int32_t* page_table, int table_width,
                  void* keys, void* values, int n_pages, void* q_out,
                  int M, int n_heads, int n_kv_heads, int head_dim, int K, void* stream);

/* Products of up to 128 rows (bfloat16, K a multiple of 32) from the packed copy of the weight.
 * K is cut into tqk_mid_splits(N, K, gated) pieces; where that is more than 1, scratch is
 * float32 [pieces][M][N], 16-byte aligned.  finish == 0: with more than one piece the pieces'
 * sums stay in scratch (tqk_add_rmsnorm_sums adds them up) and y is not written. */
int tqk_mid_splits(int N, int K, int gated);
int tqk_mid_store(const void* x, const void* w_packed, void* y, int y_dtype, int M, int N, int K, void* scratch,
                  int finish, void* stream);
/* y[M, N/2] = silu(gate) * up, w = gate rows then up rows, packed in two parts */
int tqk_mid_gated(const void* x, const void* w_packed, void* y, int M, int N, int K, void* scratch, void* stream);

/* For each token t and head: add bias, rotate q and k heads by the angle table row
 * tok_pos[t] (style 0: none, 1: halves (j, j+rot/2), 2: pairs (2j, 2j+1)), write q to
 * q_out [tokens, heads, head_dim] and, if write_kv, k and v into the pages of the
 * token's sequence: keys [n_pages, kv_heads, 64, head_dim], values transposed inside a
 * page, [n_pages, kv_heads, head_dim, 64], position p of the page at place
 * (p & 32) | ((p >> 2 & 3) << 3) | ((p >> 4 & 1) << 2) | (p & 3). */
int tqk_rope_store(const void* qkv, int act_dtype, const void* bias, int bias_dtype,
                   const float* cos_table, const float* sin_table, int rot_dim, int style,
                   int max_positions, const int32_t* tok_seq, const int32_t* tok_pos,
                   const int32_t* page_table, int table_width, int n_seqs, void* keys, void* values,
                   int n_pages, void* q_out, int n_tokens, int n_heads, int n_kv_heads,
                   int head_dim, int write_kv, void* stream);
/* the same with the q, k, v product given as its sums over n_sums pieces of K (tqk_mid_store with
 * finish == 0), float32 [n_sums][n_tokens][(heads + 2 kv heads) * head_dim]; only where
 * tqk_rope_store_takes_sums says so */
int tqk_rope_store_takes_sums(int act_dtype, int has_bias, int bias_dtype, int rot_dim, int style, int head_dim);
int tqk_rope_store_sums(const float* sums, int n_sums, const void* bias, int bias_dtype,
                        const float* cos_table, const float* sin_table, int rot_dim, int style,
                        int max_positions, const int32_t* tok_seq, const int32_t* tok_pos,
                        const int32_t* page_table, int table_width, int n_seqs, void* keys, void* values,
                        int n_pages, void* q_out, int n_tokens, int n_heads, int n_kv_heads,
                        int head_dim, int write_kv, void* stream);

/* Softmax attention of each token's query over its sequence's cached positions
 * lo..tok_pos[t], lo = max(0, tok_pos - window + 1) if window > 0 else 0.  One wave
 * per (token, head); float32 throughout; out [tokens, heads*head_dim]. */
int tqk_attention(const void* q, const void* keys, const void* values, int act_dtype,
                  const int32_t* tok_seq, const int32_t* tok_pos, const int32_t* page_table,
                  int table_width, int n_seqs, int n_pages, int window, float scale, void* out,
                  int n_tokens, int n_heads, int n_kv_heads, int head_dim, void* stream);

/* Decoding: sequence b's one new token (query row b, position tok_pos[b]) over its pages,
 * bfloat16, MFMA; n_parts partitions take the sequence's live pages in turn.  With
 * one partition the result goes straight to out [seqs, heads*head_dim]; with more, the
 * partitions' results go to part_out [seqs, heads, n_parts, head_dim] and part_ml [seqs,
 * heads, n_parts, 2] (float32) and a second kernel merges them into out. */
int tqk_attention_decode_supported(int head_dim);
int tqk_attention_decode(const void* q, const void* keys, const void* values, const int32_t* tok_pos,
                         const int32_t* page_table, int table_width, int n_seqs, int n_pages, int window,
                         float scale, int n_parts, void* part_out, void* part_ml,
                         void* out, int n_heads, int n_kv_heads, int head_dim, void* stream);

/* Prompts: tiles of up to tile_queries (16, 32, 64 or 128) consecutive queries of one sequence
 * (tile i: sequence tile_seq[i], first packed token tile_tok0[i], tile_count[i] queries, none more
 * than tile_queries) over the sequence's pages, causal with optional window, bfloat16, MFMA; the
 * tiles are best listed longest reach first.  seq_start + seq_new is the number of positions a
 * sequence's cache holds after this step.  tqk_attention_prefill_tile: the tile size that suits
 * a step of n_tokens. */
int tqk_attention_prefill_supported(int head_dim);
int tqk_attention_prefill_tile(int n_tokens, int n_heads, int n_kv_heads, int head_dim);
int tqk_attention_prefill(const void* q, const void* keys, const void* values, const int32_t* tok_pos,
                          const int32_t* page_table, int table_width, int n_seqs, int n_pages,
                          const int32_t* tile_seq, const int32_t* tile_tok0, const int32_t* tile_count,
                          int n_tiles, int tile_queries, const int32_t* seq_start, const int32_t* seq_new,
                          int window, float scale, void* out, int n_tokens, int n_heads, int n_kv_heads,
                          int head_dim, void* stream);
/* The same with a cap on the scores: cap > 0 makes them cap tanh(scale q.k / cap) before the softmax. */
int tqk_attention_prefill_capped(const void* q, const void* keys, const void* values, const int32_t* tok_pos,
                                 const int32_t* page_table, int table_width, int n_seqs, int n_pages,
                                 const int32_t* tile_seq, const int32_t* tile_tok0, const int32_t* tile_count,
                                 int n_tiles, int tile_queries, const int32_t* seq_start, const int32_t* seq_new,
                                 int window, float scale, float cap, void* out, int n_tokens, int n_heads, int n_kv_heads,
                                 int head_dim, void* stream);

/* out[t, i] = silu(gate_up[t, i]) * gate_up[t, inter + i] */
int tqk_swiglu(const void* gate_up, void* out, int act_dtype, int n_tokens, int inter, void* stream);

/* Gates of feed-forwards other than SiLU.  gate: 0 g sigmoid(g) u; 1 max(g, 0) u; 2 g' sigmoid(alpha g') (u' + 1) with
 * g' = min(g, limit) and u' = clamp(u, -limit, limit); 3 gelu_tanh(g) u; 4 max(g, 0)^2 u.  tqk_gated_act is tqk_swiglu, and
 * tqk_fused_gated_act and tqk_mid_gated_act are tqk_fused_gated and tqk_mid_gated, with the gate named. */
int tqk_gated_act(const void* gate_up, void* out, int act_dtype, int n_tokens, int inter, int gate, float limit, float alpha,
                  void* stream);
int tqk_fused_gated_act(const void* x, const float* ss_parts, int n_ss_parts, float eps, const void* w, int w_packed, void* y,
                        int M, int N, int K, int gate, float limit, float alpha, void* stream);
int tqk_mid_gated_act(const void* x, const void* w_packed, void* y, int M, int N, int K, void* scratch, int gate, float limit,
                      float alpha, void* stream);

/* Attention through a low-rank latent (latent.hip).  Every position leaves one cache row [rk + dr]: the normed
 * latent and one rotated key part, shared by all heads; pages are [n_pages][64][rk + dr].
 * tqk_latent_split: row t of proj (row_stride values) begins [q_rank | kv_rank + rot_dim (absent when kv_rank == 0) | n_gate].  cq_out
 * [tokens, q_rank] = RMS norm of the first part times q_norm_w; the second part goes into the cache row of the token's
 * position (RMS norm times kv_norm_w of its first kv_rank values, rotation in halves of the first rot_dims of the
 * others by the angle table row tok_pos[t]; `turned`, if given, gets the latent a second time, pages [n_pages][kv_rank][64]
 * with a page's positions at the places of the standard value pages, see tqk_rope_store); gate_out [tokens, n_gate] = sigmoid of the last part, float32. */
int tqk_latent_max_rank(void);          /* the largest latent (rk) tqk_latent_attention takes */
int tqk_latent_max_row(void);           /* the largest cache row (rk + dr) it takes */
int tqk_latent_split(const void* proj, int act_dtype, int row_stride, int q_rank, int kv_rank, int rot_dim, int n_gate, const void* q_norm_w,
                     const void* kv_norm_w, int norm_dtype, float eps, const float* cos_table, const float* sin_table,
                     int rot_dims, int max_positions, const int32_t* tok_seq, const int32_t* tok_pos,
                     const int32_t* page_table, int table_width, void* cache, void* turned, int n_pages, void* cq_out,
                     float* gate_out, int n_tokens, void* stream);
/* qa [tokens, heads, rk + dr] float32: qa[:rk] = W_uk,h^T q[:dn] (w_uk [heads * dn, rk]), qa[rk:] = q[dn:] rotated;
 * tail_only: the rotated part alone (the product is someone else's: tqk_head_product) */
int tqk_latent_absorb(const void* q, int act_dtype, const void* w_uk, int w_dtype, int n_heads, int dn, int dr, int rk,
                      const float* cos_table, const float* sin_table, int rot_dims, int max_positions,
                      const int32_t* tok_pos, float* qa, int n_tokens, int tail_only, void* stream);
/* out [tokens, heads, rk] float32 = softmax over the visible positions of (qa . row) * scale, times row[:rk];
 * visible: lo..tok_pos[t], lo = max(0, tok_pos - window + 1) if window > 0 else 0 */
int tqk_latent_attention(const float* qa, const void* cache, int cache_dtype, const int32_t* tok_seq, const int32_t* tok_pos,
                         const int32_t* page_table, int table_width, int n_seqs, int n_pages, int window, float scale,
                         float* out, int n_tokens, int n_heads, int rk, int dr, void* stream);
/* the same on the matrix cores, for a bfloat16 cache with its turned copy, where tqk_latent_attention_mfma_supported says so */
int tqk_latent_attention_mfma_supported(int rk, int dr);
/* n_parts > 1: a token's pages are dealt out to that many waves and merged by a second kernel; part_o float32 [tokens,
 * heads, n_parts, rk] and part_ml [tokens, heads, n_parts, 2] are its scratch.  tqk_latent_attention_parts: a good number. */
int tqk_latent_attention_parts(int n_tokens, int n_heads, int table_width, int window);
int tqk_latent_attention_mfma(const float* qa, const void* cache, const void* turned, const int32_t* tok_seq, const int32_t* tok_pos,
                              const int32_t* page_table, int table_width, int n_seqs, int n_pages, int window, float scale,
                              float* out, int n_tokens, int n_heads, int rk, int dr, int n_parts, float* part_o, float* part_ml,
                              void* stream);
/* the same for steps of several tokens per sequence: tiles of up to 4 consecutive tokens of one sequence, a block a tile */
int tqk_latent_attention_tiles(const float* qa, const void* cache, const void* turned, const int32_t* tok_pos,
                               const int32_t* page_table, int table_width, int n_seqs, int n_pages, const int32_t* tile_seq,
                               const int32_t* tile_tok0, const int32_t* tile_count, int n_tiles, int window, float scale,
                               float* out, int n_tokens, int n_heads, int rk, int dr, void* stream);
/* y [tokens, heads * dv] = gate[t, h] * W_uv,h o[t, h] (w_uv [heads * dv, rk]; gate may be null) */
int tqk_latent_values(const float* o, const void* w_uv, int w_dtype, const float* gate, int n_heads, int rk, int dv, void* y,
                      int y_dtype, int n_tokens, void* stream);

/* A feed-forward of routed experts (moe.hip).  tqk_moe_route: idx, weight [tokens, top]: the `top` experts with the
 * largest softmax(W_r x) and that score times scale.  tqk_moe_group: pair p = (token, choice) gets row pair_pos[p]
 * among its expert's rows, sorted_tok[row] names the row's token; tile lists of tqk_moe_max_tiles(pairs, experts)
 * entries and their number *n_tiles, all on the device.  tqk_moe_product: rows (x[x_rows[row]] or x[row]) of every
 * tile times its expert's weight (w + expert * expert_stride: [N, K], gated: gate rows then up rows [2 N, K]) into
 * y [pairs, N]; gated 0: the product alone, 1: gate and up, 2: one product [N, K] with the gate's function of it alone (u = 1:
 * relu2 gives max(z, 0)^2).  tqk_moe_route with renormalize: the chosen weights are divided by their sum (the softmax over
 * the chosen logits alone); with gate_w [hidden] (of the router's type, or null) it also writes gate_out[t] = sigmoid(x[t] . gate_w).
 * tqk_moe_combine: out[t] = sum_k weight[t, k] y[pair_pos[t, k]] + shared_scale[t] * shared[t]
 * (shared may be null; shared_scale null: 1).  tqk_moe_route's mode: bit 1 is that renormalising, bit 2 makes the scores
 * sigmoid(z) of every expert on its own instead of the softmax.  tqk_moe_scale_rows: rows[pair_pos[p]] = weight[p] * x[p / top]
 * and unit[p] = 1, for experts whose input carries the weight. */
int tqk_moe_scale_rows(const void* x, int act_dtype, const int32_t* pair_pos, const float* weight, int top, void* rows, float* unit,
                       int n_tokens, int hidden, void* stream);
int tqk_moe_max_experts(void);
int tqk_moe_tile_rows(void);
int tqk_moe_max_tiles(int n_pairs, int n_experts, int tile_m);
int tqk_moe_route(const void* x, int act_dtype, const void* w_router, int w_dtype, int n_experts, int hidden, int top, float scale,
                  int mode, int32_t* idx, float* weight, const void* gate_w, float* gate_out, int n_tokens, void* stream);
int tqk_moe_group(const int32_t* idx, int n_tokens, int top, int n_experts, int tile_m, int32_t* pair_pos, int32_t* sorted_tok,
                  int32_t* tile_expert, int32_t* tile_row0, int32_t* tile_rows, int32_t* n_tiles, void* stream);
int tqk_moe_product(const void* x, int act_dtype, const int32_t* x_rows, const void* w, int w_dtype, long long expert_stride, void* y,
                    int N, int K, int gated, int gate, float limit, float alpha, const int32_t* tile_expert,
                    const int32_t* tile_row0, const int32_t* tile_rows, const int32_t* n_tiles, int max_tiles, void* stream);
/* Many small products on the matrix cores (grouped.hip), bfloat16 weights, K a multiple of 8: the experts' products over
 * tiles of up to tile_m rows (16, 32 or 64, what tqk_moe_group was given; tqk_moe_product takes tqk_moe_tile_rows()), and
 * y[t, h, :N] = scale[t, h] * W_h x[t, h, :K] for every token and head (x bfloat16 or float32, w [heads][N][K], y
 * bfloat16 or float32, strides in values, scale float32 [tokens, heads] or null). */
int tqk_grouped_supported(int K);
int tqk_moe_product_mfma(const void* x, const int32_t* x_rows, const void* w, long long expert_stride, void* y, int N, int K,
                         int gated, int gate, float limit, float alpha, const int32_t* tile_expert, const int32_t* tile_row0,
                         const int32_t* tile_rows, const int32_t* n_tiles, int max_tiles, int tile_m, void* stream);
int tqk_head_product(const void* x, int x_f32, long long x_row_stride, long long x_head_stride, const void* w, void* y, int y_f32,
                     long long y_row_stride, long long y_head_stride, const float* scale, int n_tokens, int n_heads, int N, int K,
                     void* stream);
int tqk_moe_combine(const void* y, int act_dtype, const int32_t* pair_pos, const float* weight, int top, const void* shared,
                    const float* shared_scale, void* out, int n_tokens, int hidden, void* stream);

/* Around the residual stream (stream_ops.hip).  tqk_pair_embed: h[t] += table[(prev * mul_prev + token * mul_cur) mod buckets],
 * table [buckets + 1, hidden], the last row for a sequence's first token; prev is the token before it in the step or, for the
 * first token a step brings of a sequence that has begun, last[slot].  tqk_remember_tokens: last[slot] = the last token the step
 * brings of each sequence (its own launch: the first token of a sequence's piece reads what the last one writes; in a step of one
 * token a sequence tqk_pair_embed does it itself, `remember`).  copy_bf16 (or null): the stream's rows after the addition, as bfloat16.
 * tqk_norm_add: h[t] += y[t] / sqrt(mean(y[t]^2) + eps) * weight (weight null: h[t] += y[t]; y null: nothing is added), and
 * copy[t] = h[t] in the activation type (copy may be null).  tqk_unary_act: out = f(x), f a gate's function with u = 1.
 * tqk_row_gate: out[t] = sigmoid(x[t] . w), float32. */
int tqk_pair_embed(const void* table, int table_dtype, int buckets, long long mul_prev, long long mul_cur, const int32_t* tokens,
                   const int32_t* tok_seq, const int32_t* tok_pos, const int32_t* seq_slot, const int32_t* seq_start,
                   int32_t* last, float* h, int n_tokens, int hidden, int vocab, void* copy_bf16, int remember, void* stream);
int tqk_remember_tokens(const int32_t* tokens, const int32_t* cu, const int32_t* seq_new, const int32_t* seq_slot, int32_t* last,
                        int n_seqs, void* stream);
int tqk_norm_add(float* h, const void* y, int act_dtype, const void* weight, int weight_dtype, float eps, void* copy, int n_tokens,
                 int hidden, void* stream);
int tqk_unary_act(const void* x, void* out, int act_dtype, long long n, int kind, float limit, float alpha, void* stream);
int tqk_row_gate(const void* x, int act_dtype, const void* w, int w_dtype, float* out, int n_tokens, int hidden, void* stream);

/* Attention with keys of key_dim and values of value_dim per head (attention_masked.hip).  tqk_normed_rope_store: a row of qkv is
 * [heads * key_dim | kv_heads * key_dim | kv_heads * value_dim]; every query and key head is divided by its root mean square
 * (eps inside the root) and multiplied by q_norm_w / k_norm_w [key_dim] (null: no norm), then its first rot_dim elements are
 * rotated in halves by the angle table row tok_pos[t]; values become (1 - mix[0]) v + mix[0] mix_with[t] where mix_with
 * [tokens, kv_heads * value_dim] is given, and are written to mix_keep (if given) as they go to the cache.  Pages: keys
 * [n_pages, kv_heads, 64, key_dim], values [n_pages, kv_heads, value_dim, 64] with the places of tqk_rope_store.
 * tqk_attention_masked: a query at position i sees j <= i with i - j < window or j < keep_first (window 0: all); scores
 * scale q.k, then cap tanh(s / cap) if cap > 0; sink [heads] (or null) adds exp(sink_h) to the softmax's denominator.
 * One wave per (token, head), float32 throughout; out [tokens, heads * value_dim]. */
int tqk_normed_rope_store(const void* qkv, int act_dtype, const void* q_norm_w, const void* k_norm_w, int w_dtype, float eps,
                          const float* cos_table, const float* sin_table, int rot_dim, int max_positions, const void* mix,
                          const void* mix_with, void* mix_keep, const int32_t* tok_seq, const int32_t* tok_pos,
                          const int32_t* page_table, int table_width, void* keys, void* values, void* q_out, int n_tokens,
                          int n_heads, int n_kv_heads, int key_dim, int value_dim, int write_kv, void* stream);
int tqk_attention_masked_max_dim(void);
int tqk_attention_masked(const void* q, const void* keys, const void* values, int act_dtype, const int32_t* tok_seq,
                         const int32_t* tok_pos, const int32_t* page_table, int table_width, int n_seqs, int n_pages, int window,
                         int keep_first, float scale, float cap, const void* sink, int sink_dtype, void* out, int n_tokens,
                         int n_heads, int n_kv_heads, int key_dim, int value_dim, void* stream);

/* The same on the matrix cores (attention_masked_mfma.hip), bfloat16, key_dim a multiple of 8, both sizes up to 256.  n_tiles > 0:
 * tiles of up to tile_queries = tqk_attention_masked_mfma_tile(...) consecutive queries of one sequence (lists on the device; tok_pos and q by packed
 * token, page_table by sequence of the step).  Else rows: row r is a token of its own at position tok_pos[r] whose pages are
 * page_table row r, dealt out to n_parts partitions (part_out float32 [rows, heads, n_parts, value_dim] and part_ml [rows, heads,
 * n_parts, 2] where n_parts > 1; a second kernel merges them). */
int tqk_attention_masked_mfma_supported(int key_dim, int value_dim);
int tqk_attention_masked_mfma_tile(int n_tokens, int n_heads, int n_kv_heads, int key_dim, int value_dim);
int tqk_attention_masked_mfma(const void* q, const void* keys, const void* values, const int32_t* tok_pos, const int32_t* page_table,
                              int table_width, int n_pages, int window, int keep_first, float scale, float cap, const void* sink,
                              int sink_dtype, const int32_t* tile_seq, const int32_t* tile_tok0, const int32_t* tile_count, int n_tiles,
                              int tile_queries, int n_rows, int n_parts, void* part_out, void* part_ml, void* out, int n_heads, int n_kv_heads,
                              int key_dim, int value_dim, void* stream);

/* Bias, rotation, then a norm without a weight (attention_masked.hip): rows of qkv are [heads * key_dim | kv heads * key_dim | kv heads *
 * value_dim]; bias (optional) has a row's layout; q and k are turned (style 1: in halves, 2: element 2i with 2i + 1, 0: not at all) and then,
 * if normed, every head is divided by its root mean square (eps inside the root).  q goes to q_out, keys and values into the pages. */
int tqk_rope_norm_store(const void* qkv, int act_dtype, const void* bias, int bias_dtype, const float* cos_table, const float* sin_table,
                        int rot_dim, int style, int max_positions, int normed, float eps, const int32_t* tok_seq, const int32_t* tok_pos,
                        const int32_t* page_table, int table_width, void* keys, void* values, void* q_out, int n_tokens, int n_heads,
                        int n_kv_heads, int key_dim, int value_dim, int write_kv, void* stream);

/* Mixers with a fixed-size state (recurrent.hip).  A step is a packed batch: token t belongs to sequence tok_seq[t] of the step at position
 * tok_pos[t]; sequence s brings seq_new[s] tokens from packed row cu[s] on, had seq_start[s] positions before, and its state is row seq_slot[s]
 * (rows state_stride floats apart).  Small parameters are float32.
 *
 * tqk_conv_state: out[t, c] = act(bias[c] + sum_k w[c, k] in(t - (taps - 1 - k), c)), in = x + in_bias for the step's rows (x: rows x_stride
 * values apart, any float dtype) and the state's [taps - 1][channels] (oldest first) for what came before; activation 0: none, 1: silu.
 * tqk_conv_state_update: the state after the step (call it after every reader of the old one).
 * tqk_conv_state_step: both in one launch for a step in which every sequence brings one token. */
#define TQK_CONV_MAX_TAPS 8
int tqk_conv_max_taps(void);
int tqk_conv_state(const void* x, int x_dtype, long long x_stride, const float* in_bias, const float* w, const float* bias, int taps,
                   int activation, const float* state, long long state_stride, const int32_t* tok_seq, const int32_t* tok_pos,
                   const int32_t* seq_slot, const int32_t* seq_start, float* out, int n_tokens, int channels, void* stream);
int tqk_conv_state_update(const void* x, int x_dtype, long long x_stride, const float* in_bias, int taps, float* state, long long state_stride,
                          const int32_t* cu, const int32_t* seq_new, const int32_t* seq_slot, int n_seqs, int channels, void* stream);
int tqk_conv_state_step(const void* x, int x_dtype, long long x_stride, const float* in_bias, const float* w, const float* bias, int taps,
                        int activation, float* state, long long state_stride, const int32_t* tok_seq, const int32_t* seq_slot, float* out,
                        int n_tokens, int channels, void* stream);
/* Gates of a real-gated linear recurrent unit: r = sigmoid(Wa u + ba), i = sigmoid(Wi u + bi) with block-diagonal Wa, Wi given as
 * [blocks][in][out]; a = exp(decay_c r) (decay_c = -8 softplus(lam), per channel); g = sqrt(1 - a^2) i u. */
int tqk_rglru_gates(const float* u, const float* wa_t, const float* wi_t, const float* ba, const float* bi, const float* decay_c, float* a_out,
                    float* g_out, int n_tokens, int width, int blocks, void* stream);
/* (the same; the order of the sum over the inputs may depend on the step's size: steps of few tokens deal the inputs out to slices of threads) */
int tqk_rglru_gates_any_order(const float* u, const float* wa_t, const float* wi_t, const float* ba, const float* bi, const float* decay_c,
                              float* a_out, float* g_out, int n_tokens, int width, int blocks, void* stream);
/* S_t = a_t S_(t-1) + g_t per sequence and channel from the state (one float a channel), which is left at the last S;
 * out_t = S_t gelu_tanh(y_t + y_bias) in the activation dtype. */
int tqk_linear_scan(const float* a, const float* g, const void* y, int act_dtype, long long y_stride, const float* y_bias, float* state,
                    long long state_stride, const int32_t* cu, const int32_t* seq_new, const int32_t* seq_slot, void* out, int n_seqs,
                    int width, void* stream);
/* The selective state-space recurrence with one decay per head: xbc rows are [x: heads * p_dim | B: groups * n_state | C: groups * n_state];
 * dt = softplus(dt_raw[t, h] + dt_bias[h]); S_t = exp(-exp(a_log[h]) dt) S_(t-1) + dt B_t x_t^T; y_t = S_t^T C_t + d_skip[h] x_t.
 * The state of a slot: [heads][n_state][p_dim] float32. */
int tqk_ssm_max_state(void);
int tqk_ssm_scan(const float* xbc, long long xbc_stride, const void* dt_raw, int dt_dtype, long long dt_stride, const float* dt_bias,
                 const float* a_log, const float* d_skip, float* state, long long state_stride, const int32_t* cu, const int32_t* seq_new,
                 const int32_t* seq_slot, float* y_out, int n_seqs, int heads, int groups, int n_state, int p_dim, void* stream);
/* The same recurrences for steps that bring many tokens of a sequence, in chunks of consecutive tokens of one sequence (chunk c: packed rows
 * chunk_row0[c] .. + chunk_count[c]; sequence s owns chunks seq_first[s] .. seq_first[s + 1], in order).  mode 1: every chunk from a zero
 * state; its last state goes to chunk_l / chunk_state, the product of its decays to chunk_p / chunk_decay.  tqk_chunk_carry: per sequence
 * S <- p S + local over its chunks, from the sequence's state row, leaving in each chunk's place the state it starts from and in the state
 * row the last (element e of per_seq decays with chunk_p[c * p_stride + e / p_div]).  mode 2: every chunk again from that state, writing
 * the outputs.  tqk_ssm_steps: dt = softplus(raw + bias) and decay = exp(-exp(a_log) dt) per (token, head), which tqk_ssm_chunks takes. */
int tqk_linear_chunks(const float* a, const float* g, const void* y, int act_dtype, long long y_stride, const float* y_bias,
                      const int32_t* chunk_row0, const int32_t* chunk_count, int n_chunks, float* chunk_p, float* chunk_l, void* out, int mode,
                      int width, void* stream);
int tqk_chunk_carry(const float* chunk_p, long long p_stride, int p_div, float* chunk_l, const int32_t* seq_first, const int32_t* seq_slot,
                    float* state, long long state_stride, int n_seqs, long long per_seq, void* stream);
int tqk_ssm_steps(const void* dt_raw, int dt_dtype, long long dt_stride, const float* dt_bias, const float* a_log, float* dt_out,
                  float* decay_out, int n_tokens, int heads, void* stream);
int tqk_ssm_chunks(const float* xbc, long long xbc_stride, const float* dt, const float* decay, const float* d_skip, const int32_t* chunk_row0,
                   const int32_t* chunk_count, int n_chunks, float* chunk_state, float* chunk_decay, float* y_out, int mode, int heads,
                   int groups, int n_state, int p_dim, void* stream);
/* out = norm_parts(y silu(z)) w: `parts` equal parts of a row, each divided by its own root mean square. */
int tqk_gated_part_norm(const float* y, const void* z, int act_dtype, long long z_stride, const float* w, float eps, void* out, int n_tokens,
                        int size, int parts, void* stream);
/* h[i] += x[i], float32 */
int tqk_add_rows(float* h, const float* x, long long n, void* stream);

/* out[r] = lowest index of the largest value of logits[r, :]; scratch: at least
 * tqk_argmax_scratch_floats(n_rows, vocab) floats of device memory. */
int tqk_argmax_scratch_floats(int n_rows, int vocab);
int tqk_argmax(const float* logits, int n_rows, int vocab, int32_t* out, float* scratch, void* stream);

/* tqk_argmax_static, the variant that allocates nothing: csrc/tq_no_alloc.h */

/* In place: for every token in the history of the row's request, once per occurrence,
 * l > 0 ? l / penalty : l * penalty.  hist, times [n_req, hist_cap], hist_len [n_req]: the
 * history as tqk_append_history keeps it (times: for each entry how often the penalty is
 * applied on its behalf; zeros with hist_len 0 to start with). */
int tqk_repeat_penalty(float* logits, int n_rows, int vocab, const int32_t* row_req,
                       const int32_t* hist, const int32_t* times, int hist_cap, const int32_t* hist_len,
                       int n_req, float penalty, void* stream);

/* tokens[r] goes to the end of the history of request row_req[r] (dropped when that is full);
 * rows of one call name different requests. */
int tqk_append_history(const int32_t* tokens, const int32_t* row_req, int32_t* hist, int32_t* times,
                       int hist_cap, int32_t* hist_len, int n_rows, void* stream);

/* One draw per row from softmax(logits / temperature) cut to top_k (0: off) and top_p
 * (>= 1: off), by inverse CDF over the kept tokens in order of id with uniforms[r].
 * scratch: tqk_sample_scratch_bytes(n_rows, vocab, top_k, top_p) bytes of device memory, 8-byte
 * aligned (may be null where that is 0). */
size_t tqk_sample_scratch_bytes(int n_rows, int vocab, int top_k, float top_p);
int tqk_sample(const float* logits, int n_rows, int vocab, float temperature, int top_k, float top_p,
               const float* uniforms, int32_t* out, void* scratch, void* stream);

/* The residual stream in several copies, a layer norm with weight and bias, the previous token mixed into a mixer's input (streams.hip).
 * X [tokens, copies, width] float32.  tqk_streams_step: where y is given, X'[t, r] = sum_s mix[s, r] X[t, s] + out_w[r] y[t]; then, where
 * in_w is given, u = sum_s in_w[s] X'[t, s] goes to u_out (if given) and (u - mean) / sqrt(var + eps) norm_w + norm_b to n_out (if given);
 * wide != 0 lets a row have more threads (another order of its sums than with wide == 0).
 * tqk_add_layer_norm: out[i] = that norm of h[rows[i]] + delta[rows[i]] (rows null: row i; h or delta may be null; write_back leaves
 * the sum in h).  tqk_token_shift: out[t] = n[t] + (n[t - 1] - n[t]) mu, with the sequence's state row in place of n[t - 1] for the first
 * token a step brings of it; remember != 0 (steps of one token a sequence) also leaves n[t] in the state.  tqk_shift_remember: the state
 * of every sequence becomes n of the last token the step brings of it. */
int tqk_streams_max(void);
int tqk_streams_fill(const float* h, float* X, int n_streams, int n_tokens, int width, void* stream);
int tqk_streams_step(float* X, int n_streams, const void* y, int y_dtype, const float* mix, const float* out_w, const float* in_w,
                     const float* norm_w, const float* norm_b, float eps, float* u_out, void* n_out, int n_dtype, int n_tokens, int width,
                     int wide, void* stream);
int tqk_add_layer_norm(float* h, const void* delta, int delta_dtype, const int32_t* rows, int n_rows, const float* weight, const float* bias,
                       float eps, void* out, int out_dtype, int width, int write_back, void* stream);
int tqk_token_shift(const float* n, const float* mu, float* state, long long state_stride, const int32_t* tok_seq, const int32_t* tok_pos,
                    const int32_t* seq_start, const int32_t* seq_slot, void* out, int out_dtype, int n_tokens, int width, int remember,
                    void* stream);
int tqk_shift_remember(const float* n, float* state, long long state_stride, const int32_t* cu, const int32_t* seq_new, const int32_t* seq_slot,
                       int n_seqs, int width, void* stream);

/* Linear attention with a decaying state (linear_attention.hip): per head S_t = diag(a_t) S_(t-1) + k_t v_t^T, o_t = S_t^T q_t, the state
 * of a slot [heads][d][dv] float32.  q, k, v: rows `stride` elements apart, heads side by side.  The decay: z [tokens, heads * d] float32
 * with z_bias gives a = sigmoid(z + bias)^inv_tau per key channel; z null: head_decay[h] for the whole head.  q and k are turned by
 * tok_pos through cos, sin [max_pos, rot_dim / 2] (style 1: halves, 2: pairs; cos null: not turned) and multiplied by q_scale, k_scale.
 * mode 0: every sequence's tokens in order from its state row, which is written back (cu, seq_new, seq_slot; n_items sequences).
 * mode 1 and 2: chunks as tqk_ssm_chunks takes them (chunk_row0, chunk_count; n_items chunks), between them tqk_chunk_carry with
 * p_stride heads * d, p_div dv and per_seq heads * d * dv.  out [tokens, heads, dv] float32.
 * tqk_head_norm_gate: out[t, h] = o[t, h] / rms(o[t, h]) * weight (null: 1) * silu(gate[t, h]) (null: 1). */
int tqk_linear_attention_max_dim(void);
int tqk_linear_attention(const void* q, const void* k, const void* v, int act_dtype, long long stride, const float* z, long long z_stride,
                         const float* z_bias, float inv_tau, const float* head_decay, float q_scale, float k_scale, const float* cos,
                         const float* sin, int rot_dim, int style, int max_pos, const int32_t* tok_pos, float* state, long long state_stride,
                         const int32_t* cu, const int32_t* seq_new, const int32_t* seq_slot, const int32_t* chunk_row0,
                         const int32_t* chunk_count, float* chunk_state, float* chunk_decay, float* out, int mode, int n_items, int heads,
                         int d, int dv, void* stream);
int tqk_head_norm_gate(const float* o, const float* weight, float eps, const void* gate, int gate_dtype, long long gate_stride, void* out,
                       int out_dtype, int n_tokens, int heads, int dv, void* stream);

/* Attention over a window plus pooled blocks (pooled_attention.hip).  Pages: keys [kv heads][page + tqk_pooled_rows(pool)][d], values
 * likewise with dv; a block's means lie behind the positions of the page that holds its last position.  tqk_pooled_store: qkv
 * [tokens, (heads + kv heads) d + kv heads dv]; normed: q and k heads are divided by their root mean square (times q_weight, k_weight
 * [d] if given); then their first rot_dim elements are turned (style 0: not); vcos given: values are turned over all dv elements in
 * the same layout.  tqk_pool_blocks: the means of the blocks that end among the step's positions.  tqk_pooled_attention: row r
 * (sequence row_seq[r], position row_pos[r]) sees positions j with 0 <= pos - j < window and every block that ends at or before
 * pos - window; sink [heads] float32 or null; vcos given: the output is turned back by the row's position. */
int tqk_pooled_attention_max_dim(void);
int tqk_pooled_rows(int pool);
int tqk_pooled_store(const void* qkv, int dtype, const float* q_weight, const float* k_weight, int normed, float eps, const float* cos,
                     const float* sin, int rot_dim, int style, const float* vcos, const float* vsin, int max_pos, const int32_t* tok_seq,
                     const int32_t* tok_pos, const int32_t* table, int width, void* keys, void* values, void* q_out, int n_tokens,
                     int heads, int kv_heads, int d, int dv, int pool, void* stream);
int tqk_pool_blocks(void* keys, void* values, int dtype, const int32_t* seq_start, const int32_t* seq_new, const int32_t* table, int width,
                    int n_seqs, int max_new, int pool, int kv_heads, int d, int dv, void* stream);
int tqk_pooled_attention(const void* q, const void* keys, const void* values, int dtype, const int32_t* row_seq, const int32_t* row_pos,
                         const int32_t* table, int width, int window, int pool, float scale, const float* sink, const float* vcos,
                         const float* vsin, int style, int max_pos, void* out, int n_rows, int heads, int kv_heads, int d, int dv,
                         void* stream);
/* The same attention on the matrix cores for steps that bring several tokens of a sequence (pooled_attention_mfma.hip; bfloat16, head
 * sizes that are multiples of 32 up to 256): tiles of tqk_pooled_attention_tile(heads, kv_heads) consecutive queries of one sequence
 * (sequence of the step, first packed token, number of queries). */
int tqk_pooled_attention_tiles_supported(int d, int dv);
int tqk_pooled_attention_tile(int heads, int kv_heads);
int tqk_pooled_attention_tiles(const void* q, const void* keys, const void* values, const int32_t* tok_pos, const int32_t* table, int width,
                               int window, int pool, float scale, const float* sink, const float* vcos, const float* vsin, int style,
                               int max_pos, const int32_t* tile_seq, const int32_t* tile_tok0, const int32_t* tile_count, int n_tiles,
                               int tile_queries, void* out, int heads, int kv_heads, int d, int dv, void* stream);
/* out[t] = c (x[t] / rms(x[t]) wx + y[t] / rms(y[t]) wy) over rows of `width` elements (streams.hip) */
int tqk_normed_pair_sum(const void* x, const void* y, int dtype, const float* wx, const float* wy, float eps, float c, void* out, int out_dtype,
                        int n_tokens, int width, void* stream);

#ifdef __cplusplus
}
#endif
