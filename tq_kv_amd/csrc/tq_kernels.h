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

/* out[t, i] = silu(gate_up[t, i]) * gate_up[t, inter + i] */
int tqk_swiglu(const void* gate_up, void* out, int act_dtype, int n_tokens, int inter, void* stream);

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

#ifdef __cplusplus
}
#endif
