// C interface of the kernel library.  Every function returns 0 on success, a negative
// value when it refuses its arguments or a launch fails; fl_last_error() then gives
// the reason.  Pointers are device pointers unless a name says otherwise; `stream` is a
// hipStream_t.  dtype codes: 0 = float32, 1 = bfloat16.
#pragma once
#include <hip/hip_runtime.h>

#ifdef __cplusplus
extern "C" {
#endif

const char* fl_last_error(void);
int fl_abi_version(void);
int fl_compute_units(void);        // compute units of the current device: what the kernels' plans count blocks against

// ---- plain kernels (plain.hip) ----
int fl_embed(const void* table, int dtype, const int* tokens, float* out, int n, int H, int V,
             hipStream_t stream);
int fl_rmsnorm(const float* x, const float* delta, float* resid_out, const int* rows,
               const float* w, void* out, int out_dtype, int n_rows, int H, float eps,
               hipStream_t stream);
int fl_add_inplace(float* x, const float* delta, long n, hipStream_t stream);
int fl_gemm_plain(const void* x, const void* w, void* out, int in_dtype, int out_dtype, int M,
                  int N, int K, hipStream_t stream);
int fl_rope_kv_write(const void* qkv, int in_dtype, int ld, const int* positions,
                     const int* tok_seq, const int* block_table, int max_blocks, void* q_out,
                     void* cache_base, int dtype, int n, int nh, int nkv, int hd, int page_size,
                     int n_pages, int rot, float theta, int write_cache, const float* cs, int paired,
                     int n_parts, long part_stride, hipStream_t stream);
// cs[n][rot / 2][2]: cosine and sine of every (token, rotation pair) of a step
int fl_rope_table(const int* positions, int n, int rot, float theta, float* cs, hipStream_t stream);
// the same from frequencies of the caller's own: cs = magnitude * (cos, sin)(position * inv_freq[i]), inv_freq[rot / 2] double
int fl_rope_table_ladder(const int* positions, int n, int rot, const double* inv_freq, float magnitude,
                         float* cs, hipStream_t stream);
int fl_attn_plain(const void* q, void* out, const void* cache_base, int dtype,
                  const int* positions, const int* tok_seq, const int* block_table,
                  int max_blocks, int n, int nh, int nkv, int hd, int page_size, int n_pages,
                  float scale, int window, hipStream_t stream);
int fl_attn_max_head_dim(void);             // the largest head size the attention kernels take
int fl_silu_mul(const void* gu, int in_dtype, void* out, int out_dtype, int n, int I,
                hipStream_t stream);
int fl_feed_tokens(int* tokens, const int* ids, const int* src, int n, hipStream_t stream);
int fl_argmax(const float* logits, int* out, int rows, int V, hipStream_t stream);
int fl_sample(const float* logits, const float* inv_temp, const float* uniform, int* out,
              int rows, int V, hipStream_t stream);
// The same draw through top-k, top-p and min-p for the rows that ask for them (top_k[r] >= 1 as a float,
// 0 < top_p[r] < 1, min_p[r] > 0); other rows are left to fl_sample.  At most fl_sample_filtered_max_k()
// candidates are kept.  stash: rows * V values of scratch for vocabularies beyond 32,768, or null.
int fl_sample_filtered(const float* logits, const float* inv_temp, const float* uniform, const float* top_k,
                       const float* top_p, const float* min_p, int* out, int rows, int V, unsigned* stash,
                       hipStream_t stream);
int fl_sample_filtered_max_k(void);
int fl_sample_filtered_max_vocab(void);      // the largest vocabulary fl_sample_filtered takes
// Penalties over the tokens a request has generated (counts[slot][V], 16-bit, one row per state slot) and
// logit bias, in place on the step's logits before the draw; slot[r] < 0 (as a float): the row has none.
int fl_sample_penalise(float* logits, int rows, int V, const unsigned short* counts, const float* slot,
                       const float* repetition, const float* presence, const float* frequency, hipStream_t stream);
int fl_sample_bias(float* logits, int V, int n, const float* row, const float* token, const float* value,
                   hipStream_t stream);
int fl_sample_count(unsigned short* counts, int V, int rows, const float* slot, const int* ids, hipStream_t stream);
int fl_sample_history(unsigned short* counts, int V, int slot, const int* tokens, int n, hipStream_t stream);

// ---- attention over one cached latent per token (latent.hip) ----
// RMS norm of columns col0 .. col0 + width - 1 of float rows; with a block table the result goes to the
// page row of the token's position (pool [n_pages][page_size][width]), else to out [n][width]
int fl_norm_slice(const float* x, int ld, int col0, int width, const float* w, float eps, void* out,
                  int out_dtype, int n, const int* positions, const int* tok_seq, const int* block_table,
                  int max_blocks, int page_size, int n_pages, hipStream_t stream);
// one small product per head: out[t][h][:] = x[t][h][:] W_h (transposed: W_h^T), optionally times the sigmoid of a gate logit per head
int fl_heads_matmul(const float* x, int ldx, const void* w, int w_dtype, void* out, int out_dtype, int n,
                    int H, int K, int J, int transposed, const float* gate, int ldg, int gate_col0,
                    hipStream_t stream);
// z[t][h][:] = softmax_j(scale * qa[t][h] . c_j) c_j over the latent rows j <= position of the token's request
int fl_latent_attention(const float* qa, float* z, const void* pool, int dtype, const int* positions,
                        const int* tok_seq, const int* block_table, int max_blocks, int n, int H, int R,
                        int page_size, int n_pages, float scale, int window, hipStream_t stream);
int fl_latent_max_width(void);
// the same on the matrix cores for bfloat16 pools (latent_tuned.hip): qa bfloat16 [n][H][R], z float [n][H][R]
int fl_latent_attention_mfma(const void* qa, float* z, const void* pool, const int* positions,
                             const int* tok_seq, const int* block_table, int max_blocks, int n, int H, int R,
                             int page_size, int n_pages, float scale, int window, int n_split, float* part_o,
                             float* part_ml, hipStream_t stream);
int fl_latent_attention_mfma_takes(int R, int page_size);
// the same for prompt portions: blocks of four waves that share their keys through LDS; tiles [n_tiles][4] =
// (first token, tokens, first group of 16 heads, groups), tokens x groups <= 4, the tokens of one request
int fl_latent_attention_shared(const void* qa, float* z, const void* pool, const int* positions,
                               const int* tok_seq, const int* block_table, int max_blocks, int H, int R,
                               int page_size, int n_pages, float scale, int window, const int* tiles, int n_tiles,
                               hipStream_t stream);
long fl_latent_attention_shared_lds(int R);
// and for steps of few rows: a block of four waves per (token, 16 heads, part of the keys) that deal the latent's dims out among them
int fl_latent_attention_dealt(const void* qa, float* z, const void* pool, const int* positions,
                              const int* tok_seq, const int* block_table, int max_blocks, int n, int H, int R,
                              int page_size, int n_pages, float scale, int window, int n_split, float* part_o,
                              float* part_ml, hipStream_t stream);
// out[t][h][j] = sum_k x[t][h][k] w[h][j][k] on the matrix cores (w bfloat16 [H][J][K])
int fl_heads_matmul_mfma(const void* x, int x_dtype, int ldx, const void* w, void* out, int out_dtype, int n,
                         int H, int K, int J, const float* gate, int ldg, int gate_col0, hipStream_t stream);
int fl_heads_matmul_mfma_takes(int K, int J);

// ---- the mLSTM recurrence (mlstm.hip) ----
int fl_mlstm_scan(const float* proj, int ld, int col_q, int col_k, int col_v, int col_i, int col_f,
                  const float* bias_i, const float* bias_f, float cap, float q_scale, float* state,
                  const int* seq_q_start, const int* seq_q_len, const int* seq_slots, float* out, float* factors,
                  int n_seqs, int H, int D, int Dv, hipStream_t stream);
int fl_mlstm_max_dim(void);
long fl_mlstm_state_floats(int D, int Dv);
int fl_headnorm_gate(const float* x, const float* w, const float* gate, int ldg, int gate_col0, void* out,
                     int out_dtype, int n, int H, int Dv, float eps, int gate_kind, hipStream_t stream);

// ---- routed experts, activations, re-entry of the stream (moe.hip) ----
int fl_moe_route(const float* logits, int ld, int col0, int n, int E, int top, int kind, int renorm,
                 int* place, int* src_row, float* src_scale, float* pair_w, int* tiles, int max_tiles,
                 hipStream_t stream);
// the same for a router whose choice goes by softmax + correction inside the best groups of experts and whose last
// n_identity outputs are identity experts (E counts all outputs); weights = chosen softmax / their sum * scale
int fl_moe_route_grouped(const float* logits, int ld, int col0, int n, int E, int n_identity, int top,
                         const float* correction, int n_groups, int keep_groups, float scale, int* place,
                         int* src_row, float* src_scale, float* pair_w, int* tiles, int max_tiles,
                         hipStream_t stream);
// y[p] = src_scale[p] * x[src_row[p]] for the sorted places of identity experts' tiles
int fl_moe_identity(const void* x, int dtype, const int* src_row, const float* src_scale, float* y,
                    const int* tiles, int max_tiles, int W, hipStream_t stream);
int fl_moe_tile_rows(void);
int fl_moe_gemm(const void* x, int dtype, const int* src_row, const float* src_scale, const void* w,
                float* out, const int* tiles, int max_tiles, int N, int K, hipStream_t stream);
// fl_moe_gemm on the matrix cores (bfloat16 x and w; moe_tuned.hip); n_rows: the sorted pairs of the step (few: the
// form that only streams the weights)
int fl_moe_gemm_mfma(const void* x, const int* src_row, const float* src_scale, const void* w, float* out,
                     const int* tiles, int max_tiles, int n_rows, int N, int K, hipStream_t stream);
int fl_moe_gemm_mfma_takes(int N, int K);
// out[m][f] = sum_k x[m][k] w[f][k] for few features f: one wave per output, float sums in a fixed order
int fl_gemm_few(const void* x, const void* w, float* out, int dtype, int M, int N, int K, hipStream_t stream);
int fl_moe_combine(const float* y, const int* place, int top, const float* shared, const float* gate, int ldg,
                   int gate_col, float* delta, int n, int W, hipStream_t stream);
int fl_activation(const float* x, void* out, int out_dtype, long total, int kind, hipStream_t stream);
int fl_concat_cast(const float* a, const float* b, void* out, int out_dtype, int n, int W, hipStream_t stream);
int fl_add_rowvec(float* x, const float* v, int n, int W, hipStream_t stream);

// ---- tuned bf16 kernels ----
// nw_hint: waves per block that split K (0: chosen from the sizes)
// epilogue: 0 = plain product; 1 = SwiGLU over interleaved gate/up rows, out_cols <= N / 2
int fl_gemm_skinny(const void* x, const void* w_packed, void* out, int out_dtype, int M, int N, int K,
                   int nw_hint, int epilogue, int out_cols, hipStream_t stream);

// The same product fused with the norms around it (at most 16 rows).  in_ssq (or null): [M, in_parts]
// partial sums of squares; every row of the result is multiplied by rsqrt(sum / K + eps).
// epilogue 2: resid[M, N] += the product, xg[M, N] = bf16(resid * g), out_ssq[M, ceil(N / 16)] = the
// blocks' sums of resid^2; nothing is stored in out.
int fl_gemm_skinny_fused(const void* x, const void* w_packed, void* out, int out_dtype, int M, int N, int K,
                         int epilogue, int out_cols, const float* in_ssq, int in_parts, float eps,
                         float* resid, const float* g, void* xg, float* out_ssq, hipStream_t stream);
int fl_gemm_skinny_scale_parts(int N, int K, int in_parts);

// 17 to 64 rows, K a multiple of 32; a shape with fl_gemm_mid_splits > 1 needs a float workspace
// of splits * M * N values
int fl_gemm_mid(const void* x, const void* w_packed, void* out, float* workspace, int out_dtype,
                int M, int N, int K, int epilogue, int out_cols, hipStream_t stream);
int fl_gemm_mid_splits(int M, int N, int K);
// for tests and measurements: waves per block (0, 4, 8) and K-splits (0 = chosen) from the caller
int fl_gemm_mid_ex(const void* x, const void* w_packed, void* out, float* workspace, int out_dtype,
                   int M, int N, int K, int epilogue, int out_cols, const float* in_ssq, int in_parts,
                   float eps, int waves, int forced_splits, hipStream_t stream);
int fl_gemm_mid_splits_ex(int M, int N, int K, int waves, int forced);
// The same fused with the norms around it, as fl_gemm_skinny_fused: a row scale from partial sums of
// squares, and the product added to the residual stream with the next norm left in factors
// (out_ssq[M, fl_gemm_mid_parts(N)]; the workspace holds splits * M * N floats, also for one split).
int fl_gemm_mid_scaled(const void* x, const void* w_packed, void* out, float* workspace, int out_dtype,
                       int M, int N, int K, int epilogue, int out_cols, const float* in_ssq, int in_parts,
                       float eps, hipStream_t stream);
int fl_gemm_mid_residual(const void* x, const void* w_packed, float* workspace, int M, int N, int K,
                         float* resid, const float* g, void* xg, float* out_ssq, hipStream_t stream);
int fl_gemm_mid_partials(const void* x, const void* w_packed, float* workspace, int M, int N, int K,
                         const float* in_ssq, int in_parts, float eps, hipStream_t stream);
int fl_gemm_mid_parts(int N);
// The adding half of fl_gemm_mid_residual for any number of rows: part[splits][M][N] -> resid, xg, out_ssq.
int fl_reduce_residual(const float* part, float* resid, const float* g, void* xg, float* out_ssq, int M, int N,
                       int splits, hipStream_t stream);

int fl_gemm_tiled(const void* x, const void* w_packed, void* out, float* workspace, int out_dtype,
                  int M, int N, int K, int epilogue, int out_cols, hipStream_t stream);
int fl_gemm_tiled_splits(int M, int N, int K);
// for tests and measurements: block shape (0 = chosen, 3 = 256 features x 128 tokens, 7 = 192 x 128,
// 8 = 128 x 128; with eight waves 10 = 256 x 256, 6 = 128 x 256) and K-splits (0 = chosen) from the caller
int fl_gemm_tiled_ex(const void* x, const void* w_packed, void* out, float* workspace, int out_dtype,
                     int M, int N, int K, int epilogue, int out_cols, const float* in_ssq, int in_parts,
                     float eps, int variant, int forced_splits, hipStream_t stream);
int fl_gemm_tiled_splits_ex(int M, int N, int K, int forced);
int fl_gemm_tiled_shape(int M, int N, int K, int may_split);
int fl_gemm_tiled_residual_ex(const void* x, const void* w_packed, float* workspace, int M, int N, int K, float* resid,
                              const float* g, void* xg, float* out_ssq, int variant, hipStream_t stream);
int fl_gemm_tiled_parts_ex(int M, int N, int K, int variant);
int fl_gemm_tiled_rope_ex(const void* x, const void* w_packed, int M, int N, int K, const float* in_ssq,
                          int in_parts, float eps, const int* positions, const int* tok_seq,
                          const int* block_table, int max_blocks, const float* cs, void* q_out, void* cache_base,
                          int nh, int nkv, int hd, int page_size, int n_pages, int rot, int write_cache, int variant,
                          hipStream_t stream);
// The joined q/k/v projection (rows of w in paired order) with rotation and the stores of q and the
// cache rows in the product's kernel: at most 16 rows, and many rows (shapes whose K is not split).
int fl_gemm_skinny_rope(const void* x, const void* w_packed, int M, int N, int K, const float* in_ssq,
                        int in_parts, float eps, const int* positions, const int* tok_seq,
                        const int* block_table, int max_blocks, const float* cs, void* q_out,
                        void* cache_base, int nh, int nkv, int hd, int page_size, int n_pages, int rot,
                        int write_cache, hipStream_t stream);
int fl_gemm_tiled_rope(const void* x, const void* w_packed, int M, int N, int K, const float* in_ssq,
                       int in_parts, float eps, const int* positions, const int* tok_seq,
                       const int* block_table, int max_blocks, const float* cs, void* q_out, void* cache_base,
                       int nh, int nkv, int hd, int page_size, int n_pages, int rot, int write_cache,
                       hipStream_t stream);
// The tiled product fused with the norms around it, as fl_gemm_skinny_fused.  The residual form leaves
// out_ssq[M, fl_gemm_tiled_residual_parts(M, N, K)] and needs a workspace of splits * M * N floats where K is split.
int fl_gemm_tiled_scaled(const void* x, const void* w_packed, void* out, float* workspace, int out_dtype,
                         int M, int N, int K, int epilogue, int out_cols, const float* in_ssq, int in_parts,
                         float eps, hipStream_t stream);
int fl_gemm_tiled_residual(const void* x, const void* w_packed, float* workspace, int M, int N, int K, float* resid,
                           const float* g, void* xg, float* out_ssq, hipStream_t stream);
int fl_gemm_tiled_parts(int M, int N, int K);
// The K-splits left apart in workspace[fl_gemm_tiled_splits(M, N, K)][M][N], each scaled by in_ssq's row scale.
int fl_gemm_tiled_partials(const void* x, const void* w_packed, float* workspace, int M, int N, int K,
                           const float* in_ssq, int in_parts, float eps, hipStream_t stream);
int fl_gemm_tiled_residual_parts(int M, int N, int K);
int fl_attn_decode(const void* q, void* out, float* part_o, float* part_ml, const void* cache_base,
                   const int* items, int n_items, const int* block_table, int max_blocks, int nh, int nkv, int hd, int page_size,
                   int n_pages, float scale, int window, int n_split, hipStream_t stream);
// fl_attn_decode with splits per row: items[i] = (row, position, request, split + 256 * splits), a row's
// splits one after the other from split 0 on (up to 255 of them; 1: no split), row < 0: unused place.
// part_o: n_items * nh * (hd rounded up to 32) floats, part_ml: n_items * nh * 2.  firsts[r] = (row,
// index of the row's first item, its splits, 0), n_rows of them; null: every row has one split,
// nothing is merged (and no workspace needed).
int fl_attn_decode_items(const void* q, void* out, float* part_o, float* part_ml, const void* cache_base,
                         const int* items, int n_items, const int* block_table, int max_blocks, int nh, int nkv,
                         int hd, int page_size, int n_pages, float scale, int window, const int* firsts, int n_rows,
                         hipStream_t stream);
// fl_attn_decode for callers that cannot allocate device memory (code under graph capture, tight
// serving loops, harnesses that forbid it).  It has no counterpart in the reference.  The splits'
// partial results, which fl_attn_decode takes as part_o / part_ml, go to an array of
// FL_ATTN_DECODE_STATIC_FLOATS floats (8 MiB) that is part of the library's image on every GPU it
// runs on; the call allocates and frees nothing.  It refuses n_items * nh * n_split * (hd rounded
// up to 32, + 2) floats beyond that size.  Every call on a GPU uses that GPU's one array: calls
// that overlap on one GPU (two streams, two threads) race; calls on one stream do not.  Nothing in
// the array has to start at zero: every slot a call reads was written by the same call before.
#define FL_ATTN_DECODE_STATIC_FLOATS (2u << 20)
int fl_attn_decode_static(const void* q, void* out, const void* cache_base, const int* items, int n_items,
                          const int* block_table, int max_blocks, int nh, int nkv, int hd, int page_size,
                          int n_pages, float scale, int window, int n_split, hipStream_t stream);
long fl_attn_decode_static_capacity(void);
int fl_attn_prefill(const void* q, void* out, const void* cache_base, const int* tiles, int n_tiles,
                    const int* positions, const int* block_table, int max_blocks, int nh, int nkv, int hd,
                    int page_size, int n_pages, float scale, int window, int qt_hint, float* part_o, float* part_ml,
                    int n_split, hipStream_t stream);
// Block-table entries of a request that a block of fl_attn_prefill can keep at a head size, and whether
// it takes a cache shape with tables max_blocks wide (with a window only the window's pages count).
int fl_attn_prefill_max_pages(int hd);
int fl_attn_prefill_takes(int hd, int page_size, int max_blocks, int window);
int fl_attn_prefill_splits(int n_tiles, int nh, int nkv, int hd, int max_keys);
int fl_attn_prefill_heads(int n_tiles, int nh, int nkv, int hd, int max_keys);      // query heads per wave: the qt_hint to pass
int fl_attn_prefill_workspace(int n_rows, int nh, int hd, int n_split, long* o_floats, long* ml_floats);
int fl_attn_decode_workspace(int n_items, int nh, int hd, int n_split, long* o_floats, long* ml_floats);

// ---- products that add to the residual stream and norm it with Dynamic Tanh in their epilogue ----
// resid[M, N] += x w^T; xn[M, N] = bf16(tanh(alpha[0] * resid) * g + bias) (bias may be null).  fl_gemm_skinny_dyt: at
// most 16 rows; fl_gemm_tiled_dyt: shapes whose K is not split (fl_gemm_tiled_splits(M, N, K) == 1).
int fl_gemm_skinny_dyt(const void* x, const void* w_packed, int M, int N, int K, float* resid,
                       const float* alpha, const float* g, const float* bias, void* xn, hipStream_t stream);
int fl_gemm_tiled_dyt(const void* x, const void* w_packed, int M, int N, int K, float* resid,
                      const float* alpha, const float* g, const float* bias, void* xn, hipStream_t stream);
// the same from a product's K-splits left apart (part[splits][M][N]), as fl_reduce_residual
int fl_reduce_dyt(const float* part, float* resid, const float* alpha, const float* g, const float* bias, void* xn,
                  int M, int N, int splits, hipStream_t stream);

// ---- the same attention kernels with capped scores: score <- softcap * tanh(score / softcap) ----
int fl_attn_plain_capped(const void* q, void* out, const void* cache_base, int dtype,
                         const int* positions, const int* tok_seq, const int* block_table,
                         int max_blocks, int n, int nh, int nkv, int hd, int page_size, int n_pages,
                         float scale, int window, float softcap, hipStream_t stream);
int fl_attn_decode_items_capped(const void* q, void* out, float* part_o, float* part_ml, const void* cache_base,
                                const int* items, int n_items, const int* block_table, int max_blocks, int nh,
                                int nkv, int hd, int page_size, int n_pages, float scale, int window,
                                float softcap, const int* firsts, int n_rows, hipStream_t stream);
int fl_attn_prefill_capped(const void* q, void* out, const void* cache_base, const int* tiles,
                           int n_tiles, const int* positions, const int* block_table,
                           int max_blocks, int nh, int nkv, int hd, int page_size, int n_pages,
                           float scale, int window, float softcap, int qt_hint, float* part_o, float* part_ml,
                           int n_split, hipStream_t stream);

// ---- rows of the residual stream and of mixers' outputs (stream_ops.hip) ----
// out = tanh(alpha * (x + delta)) * w + b (Dynamic Tanh); resid_out, rows as for fl_rmsnorm
int fl_dyt(const float* x, const float* delta, float* resid_out, const int* rows, const float* alpha,
           const float* w, const float* b, void* out, int out_dtype, int n_rows, int H, hipStream_t stream);
int fl_embed_scaled(const void* table, int dtype, const int* tokens, float* out, int n, int H, int V, float scale,
                    hipStream_t stream);
// out[r][i] = act(gu[r][i]) * gu[r][I + i]; kinds as fl_activation
int fl_gated_act(const float* gu, void* out, int out_dtype, int n, int I, int kind, hipStream_t stream);
// out = ca * a / rms(a) * wa + cb * b / rms(b) * wb per row
int fl_norm_mix(const float* a, const float* wa, float ca, const float* b, const float* wb, float cb, float* out,
                int n, int H, float eps, hipStream_t stream);
// out[t][h][j < Dv] = x[t][h][j] * g(gate[t][gate_col0 + h * Dv + j]), heads of x ldh wide; g: 0 none, 1 sigmoid, 2 silu
int fl_heads_gate(const void* x, int dtype, int ldh, const float* gate, int ldg, int gate_col0, int kind, void* out,
                  int n, int H, int Dv, hipStream_t stream);

// ---- between a joined q/k/v projection and attention (qkv_prepare.hip) ----
int fl_qkv_prepare(const float* proj, int ld, int col_q, int col_k, int col_v, const int* positions,
                   const int* tok_seq, const int* block_table, int max_blocks, void* q_out, void* cache_base,
                   int dtype, int n, int nh, int nkv, int D, int Dv, int hdp, int page_size, int n_pages, int rot,
                   int interleaved, const float* cs, const float* qnorm_w, const float* knorm_w, int head_norm,
                   const float* q_head_gain, const float* k_head_gain, float eps, float* v_first, int vmix_mode,
                   const float* lambda, int write_cache, float* row_scales, const float* bias, hipStream_t stream);

// ---- linear recurrences with a matrix state per head (linear_scan.hip) ----
int fl_linear_scan_max_dim(void);
int fl_conv_max_taps(void);
int fl_linear_scan(const float* q, int ldq, const float* k, int ldk, const float* v, int ldv,
                   const float* head_decay, const float* tok_decay, const float* beta, int ldg, float* state,
                   long slot_stride, const int* seq_q_start, const int* seq_q_len, const int* seq_slots,
                   float* out, int n_seqs, int H, int G, int D, int Dv, hipStream_t stream);
int fl_conv_prepare(const float* proj, int ld, int col0, int col_b, int col_a, const float* conv_w,
                    const float* a_log, const float* dt_bias, float* conv_state, long slot_stride,
                    const int* tok_seq, const int* seq_q_start, const int* seq_q_len, const int* seq_slots,
                    float* prep, float* gates, int n, int n_seqs, int G, int H, int D, int Dv, int taps,
                    float q_scale, float unit_eps, hipStream_t stream);
// fl_linear_scan's delta rule with a decay per token, head and key dim (decay rows ldd wide, heads x D; beta rows ldb wide)
int fl_linear_scan_delta_channel(const float* q, int ldq, const float* k, int ldk, const float* v, int ldv,
                                 const float* decay, int ldd, const float* beta, int ldb, float* state,
                                 long slot_stride, const int* seq_q_start, const int* seq_q_len,
                                 const int* seq_slots, float* out, int n_seqs, int H, int G, int D, int Dv,
                                 hipStream_t stream);
// out[t][h * D + d] = exp(-exp(a_log[h]) * softplus(a[t][col + h * D + d] + dt_bias[h * D + d]))
int fl_channel_decay(const float* a, int ld, int col, const float* a_log, const float* dt_bias, float* out,
                     int n, int H, int D, hipStream_t stream);
// out[t][f] = sum_r x[t][col + r] * w[f][r]: the second factor of a projection of low rank, given as it is stored
// (w_rows [N][R]: a step of few tokens reads it) and transposed (wt [R][N]); x float, the factor in dtype
int fl_lowrank_expand(const float* x, int ld, int col, const void* w_rows, const void* wt, int dtype, float* out,
                      int n, int N, int R, hipStream_t stream);
int fl_rotate_scale(const float* proj, int ld, int col_a, int col_b, const float* cs, int rot, int interleaved,
                    float scale_a, float scale_b, float* out_a, float* out_b, int n, int H, int D,
                    hipStream_t stream);

// ---- layer norm, learned positions, forget gates per key dim, attention whose heads' scores are mixed ----
// out = (v - mean) / sqrt(var + eps) * w + b of v = x (+ delta); resid_out, rows as for fl_rmsnorm; b may be null
int fl_layernorm(const float* x, const float* delta, float* resid_out, const int* rows, const float* w,
                 const float* b, void* out, int out_dtype, int n, int H, float eps, hipStream_t stream);
// resid += layernorm(delta); cast (or null) receives the new resid in cast_dtype
int fl_layernorm_add(const float* delta, const float* w, const float* b, float* resid, void* cast, int cast_dtype,
                     int n, int H, float eps, hipStream_t stream);
// out[t] = table[tokens[t]] + pos_table[positions[t]] (both tables in dtype, the sum float)
int fl_embed_positions(const void* table, const void* pos_table, int dtype, const int* tokens, const int* positions,
                       float* out, int n, int H, int V, int P, hipStream_t stream);
int fl_cast_rows(const float* x, void* out, int out_dtype, long total, hipStream_t stream);
int fl_scale_inplace(float* x, long total, float s, hipStream_t stream);
// out[r][i] = act(x[r][i] + bias[i]); kinds as fl_activation (3: the square of relu)
int fl_bias_activation(const float* x, const float* bias, void* out, int out_dtype, int n, int width, int kind,
                       hipStream_t stream);
// fl_linear_scan with a forget gate f per token, head and key dim: S <- diag(f) S + (1 - f) v^T, o = S^T q
int fl_linear_scan_channel(const float* q, int ldq, const float* f, int ldf, const float* v, int ldv, float* state,
                           long slot_stride, const int* seq_q_start, const int* seq_q_len, const int* seq_slots,
                           float* out, int n_seqs, int H, int D, int Dv, hipStream_t stream);
// q_out = silu(proj[col_q ..]), f_out = lower + (1 - lower) * sigmoid(proj[col_f ..] + bias), HD values per row
int fl_forget_gates(const float* proj, int ld, int col_q, int col_f, const float* bias, const float* lower,
                    float* q_out, float* f_out, int n, int HD, hipStream_t stream);
// Softmax attention over the paged cache with a distance bias slope_g * (i - j) taken off every head's score,
// the heads' scores mixed by talk [nh][nh], and a sink per head in the denominator (each may be null).
// part_keys > 0: a token's keys are dealt out to n_parts blocks of part_keys keys and joined afterwards
// (part_acc [n][n_parts][nh][hd], part_ml [n][n_parts][nh][2], float).
int fl_attn_mixed_max_heads(int hd);
int fl_attn_mixed(const void* q, void* out, const void* cache_base, int dtype, const int* positions,
                  const int* tok_seq, const int* block_table, int max_blocks, int n, int nh, int nkv, int hd,
                  int page_size, int n_pages, float scale, int window, int keep_first, int chunk, const float* slopes,
                  const float* talk, const float* sink, int part_keys, int n_parts, float* part_acc, float* part_ml,
                  hipStream_t stream);
int fl_attn_mixed_tiled_fits(int nh, int hd, int page_size);
int fl_attn_mixed_tiled(const void* q, void* out, const void* cache_base, const int* positions, const int* block_table,
                        int max_blocks, const int* seq_q_start, const int* seq_q_len, int n_seqs, int n_tiles, int n,
                        int nh, int nkv, int hd, int page_size, int n_pages, float scale, int window, int keep_first, int chunk,
                        const float* slopes, const float* talk, const float* sink, int part_keys, int n_parts, float* part_acc, float* part_ml,
                        hipStream_t stream);

// ---- hyper-connections: a residual stream in S copies (hyper.hip) ----
// xs [n][S][W] float.  y given: x_t <- sum_s mix[s][t] x_s + out_w[t] * (y + y_bias), y_bias [W] or null.  in_w given: u = sum_s in_w[s] x_s (the new
// copies) into u_out, and with a gain normed = u / sqrt(mean(u^2) + eps) * gain in out_dtype.  rows (n_rows of them):
// the tokens that are read, one output row each (only without y).
int fl_hyper_step(float* xs, int n, int S, int W, const float* y, const float* y_bias, const float* mix, const float* out_w,
                  const float* in_w, const int* rows, int n_rows, float* u_out, const float* gain, float eps,
                  void* normed, int out_dtype, hipStream_t stream);
int fl_hyper_spread(const float* x, float* xs, int n, int S, int W, hipStream_t stream);
int fl_scaled_sum(const float* a, float ca, const float* b, float cb, float* out, long total, hipStream_t stream);
int fl_softcap_inplace(float* x, long total, float cap, hipStream_t stream);

// ---- step programs (program.hip): launches recorded once, replayed with one call ----
typedef union FlArg { void* p; long l; int i; float f; } FlArg;
void* fl_program_new(void);
void fl_program_free(void* program);
int fl_program_size(const void* program);
// name: a launch function the recorder knows (every function above that takes a stream); args: its
// arguments in order, the stream's value is ignored
int fl_program_append(void* program, const char* name, const FlArg* args, int n_args);
int fl_program_run(const void* program, hipStream_t stream, int* failed_at);
// What the recorder knows: launch functions register themselves (FL_RECORDABLE in recordable.h puts a
// registrar beside a definition); a launch function of another library is added with
// fl_program_register, `call` being a function that unpacks the recorded arguments and calls it with
// the stream given.  fl_program_knows: the number of arguments (stream included) or -1.
typedef int (*FlTrampoline)(const FlArg* args, hipStream_t stream);
int fl_program_register(const char* name, FlTrampoline call, int n_args);
int fl_program_knows(const char* name);

#ifdef __cplusplus
}
#endif
