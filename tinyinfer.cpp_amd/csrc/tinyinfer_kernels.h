// The C interface of the kernel libraries: what `ops/kernels.py` binds through ctypes, and what a
// C or C++ program may link against.  One shared library per source file (libti_<name>.<hash>.so,
// built by build.py); each also exports `const char* ti_last_error()`.
//
// Conventions.  Every pointer is device memory of the GPU that `stream` belongs to.  Every function
// returns 0 on success, 3 for sizes its kernels do not serve (nothing was launched; use the more
// general function) and another non-zero value for an error; `ti_last_error()` of the same library
// then holds the message.  Nothing here allocates: scratch comes in through arguments.
// dtype codes: 0 = float32, 1 = bfloat16.  Epilogue codes `epi`: 0 store f32, 1 add into f32,
// 2 store in the operand dtype, 3 SwiGLU over stacked [gate; up] rows.
//
// Shapes: M tokens (rows) of a step; H residual width; a cache pool of one layer is
// [pages][2][n_kv][P][hd] with keys as [row][hd] and values transposed as [hd][row]; `table` is
// int32 [requests][table_stride] of page ids (-1: none), `slot[m]` the table row of token m, `pos[m]`
// its position.
#pragma once
#include <hip/hip_runtime.h>

#ifdef __cplusplus
extern "C" {
#endif

// ---- libti_core: embedding, norms, rotation, cache write (templated on the storage dtype)
int ti_embed(int dtype, const void* table, const int* tok, float* x, int M, int H, int V, hipStream_t stream);
// the same; a token below zero stands for fed[-1 - token], an id an earlier kernel on the stream left (fed may be null)
int ti_embed_fed(int dtype, const void* table, const int* tok, const int* fed, int n_fed, float* x, int M, int H, int V,
                 hipStream_t stream);
// out[r] = rmsnorm(x[rows ? rows[r] : r]) * w, in `out_dtype`
int ti_rmsnorm(int out_dtype, const float* x, const float* w, const int* rows, void* out, int n_rows, int H, float eps,
               hipStream_t stream);
// x[r] += partial[0][r] + ... + partial[KS - 1][r] (partial: [KS][n_rows][H], what a product with a
// split K left), written back, then the same norm of the new x.  Returns 3 for what it does not serve.
int ti_rmsnorm_add_partials(int out_dtype, float* x, const float* partial, int KS, const float* w, void* out,
                            int n_rows, int H, float eps, hipStream_t stream);
// half-split rotation in place on f32 [M, heads, hd] (rows `row_stride` floats apart)
int ti_rope_neox(float* x, const int* pos, const float* inv_freq, int M, int heads, int hd, long row_stride,
                 hipStream_t stream);
// table[p][k] = (cos, sin)(p * inv_freq[k]) for p < n_pos
int ti_rope_table(float* table, const float* inv_freq, int half, int n_pos, hipStream_t stream);
// qkv f32 [M, (n_head + 2 n_kv) hd]: per-head norm (weights may be null), rotation (inv_freq may be
// null; rope_table [table_len][hd/2][2] may be null), q to q_out, k and v into the cache pages
int ti_qk_norm_rope_kv_write(int dtype, const float* qkv, const float* q_w, const float* k_w, const float* inv_freq,
                             const float* rope_table, int table_len, const int* pos, const int* slot, const int* table,
                             int table_stride, void* pool, void* q_out, int M, int n_head, int n_kv, int hd,
                             int page_size, float eps, hipStream_t stream);
// the per-head norm alone, in place
int ti_qk_norm_inplace(float* qkv, int row_width, const float* q_w, const float* k_w, int M, int n_head, int n_kv, int hd,
                       float eps, hipStream_t stream);
// zero `bytes` bytes (whole four-byte words) with a kernel
int ti_fill_zero(void* p, long bytes, hipStream_t stream);
// random values, element i a pure function of (seed, i).  dtype 0 / 1: kind 0 normal(a, b), 1 uniform
// [a, b), 2 constant a; dtype 2 (int32): uniform integers in [a, b)
int ti_fill_random(int dtype, void* p, long n, int kind, float a, float b, unsigned long seed, hipStream_t stream);

// ---- libti_gemm_generic: out (op)= A W^T for any sizes, float32 or bfloat16, fixed summation order
int ti_gemm_generic(int dtype, const void* A, const void* W, void* out, int M, int N, int K, long lda, int epi,
                    hipStream_t stream);

// ---- libti_gemm_bf16: the same on the matrix cores (K a multiple of 8)
int ti_gemm_bf16(const void* A, const void* W, void* out, int M, int N, int K, long lda, int epi, hipStream_t stream);
// The adding product for 17..64 rows and a weight of few rows: MFMAs fed straight from memory, K
// split over workgroups whose sums go through `partial` (workspace of partial_bytes).  defer = 0:
// they are added to out here (served: products large enough to gain even so); defer = 1: they stay
// in partial [*splits][M][N] and the caller adds them (ti_gemm_bf16_partials_add, or
// ti_rmsnorm_add_partials on the way to the next norm); defer = 2: as 1, but added here.
// Returns 3 for what it does not serve.
int ti_gemm_bf16_add_split(const void* A, const void* W, void* out, int M, int N, int K, long lda, int epi,
                         void* partial, long partial_bytes, int defer, int* splits, hipStream_t stream);
int ti_gemm_bf16_partials_add(float* out, const float* partial, int KS, long count, hipStream_t stream);
// out = A W^T stored in 32-bit for 17..64 rows times a large weight of few tiles: K split over workgroups
// (partial: workspace of partial_bytes), the shares added up by a kernel of its own; 3: not served
int ti_gemm_bf16_store_split(const void* A, const void* W, void* out, int M, int N, int K, long lda, void* partial,
                             long partial_bytes, hipStream_t stream);
// the kernel of ti_gemm_bf16_add_split alone, for tests: any epilogue, 1..64 rows, K split ks ways
int ti_gemm_bf16_mblocks_any(const void* A, const void* W, void* out, int M, int N, int K, long lda, int epi,
                             void* partial, int ks, hipStream_t stream);
// the kernel for up to 16 rows that takes the token rows through LDS in pieces, alone, for tests: any
// epilogue, K a multiple of 64 split ks ways (adding epilogue only; partial f32 [ks][M][N])
int ti_gemm_bf16_pieces_any(const void* A, const void* W, void* out, int M, int N, int K, long lda, int epi,
                            void* partial, int ks, hipStream_t stream);
// out (op)= rmsnorm(x; nw, eps) W^T for M <= 16, K a multiple of 64
int ti_gemm_bf16_normed(const float* x, const float* nw, float eps, const void* W, void* out, int M, int N, int K, int epi,
                        hipStream_t stream);
// the q/k/v product of a step (M > 16) that finishes its heads itself: see ti_qk_norm_rope_kv_write
int ti_gemm_bf16_qkv_prep(const void* A, const void* W, int M, int K, long lda, const float* q_w, const float* k_w,
                          float eps, const float* inv_freq, const float* rope_table, int table_len, const int* pos,
                          const int* slot, const int* table, int table_stride, void* pool, void* q_out, int n_head,
                          int n_kv, int hd, int page_size, hipStream_t stream);

// ---- libti_attention_generic: paged causal attention of every row, any head size in steps of 16
int ti_attention_rows(int dtype, const void* q, const void* pool, const int* table, int table_stride, const int* pos,
                      const int* slot, void* out, int M, int n_head, int n_kv, int hd, int page_size, float scale,
                      int window, hipStream_t stream);

// the same for keys and values of different sizes (dk, dv up to 256, any value in that range) and soft-capped scores:
// s = (q . k) scale, then softcap tanh(s / softcap) if softcap > 0.  A page is K [n_kv][P][dk] | V [n_kv][dv][P].
int ti_attention_capped_rows(int dtype, const void* q, const void* pool, const int* table, int table_stride,
                             const int* pos, const int* slot, void* out, int M, int n_head, int n_kv, int dk, int dv,
                             int page_size, float scale, float softcap, int window, hipStream_t stream);

// ---- libti_pointwise: element-wise kernels of layers beyond the pre-norm transformer block
// x[m, 2i] += sin(pos[m] inv_freq[i]), x[m, 2i + 1] += cos(pos[m] inv_freq[i])
int ti_add_sinusoid(float* x, const int* pos, const float* inv_freq, int M, int H, hipStream_t stream);
// x[m, :] += v
int ti_add_row(float* x, const float* v, int M, int H, hipStream_t stream);
// out = xIELU(z) with act = (p, q): z > 0: softplus(p) z^2 + z/2; else (1/2 + softplus(q)) (exp(z) - 1 - z) + z/2
int ti_xielu(int out_dtype, const float* z, const float* act, void* out, long n, hipStream_t stream);
// x[m, c] += a[m, c] sa[c] + b[m, c] sb[c]  (b may be null; a scale that is null is 1)
int ti_scaled_add(float* x, const float* a, const float* sa, const float* b, const float* sb, int M, int H,
                  hipStream_t stream);
// qkv f32 [M, n_head dk + n_kv dk + n_kv dv]: q times 1 + coef ln(floor((pos + 1) / every) + 1) to q_out, k and v into
// the pages (layout as ti_attention_capped_rows reads it)
int ti_qkv_split_write(int dtype, const float* qkv, const int* pos, const int* slot, const int* table, int table_stride,
                       void* pool, void* q_out, int M, int n_head, int n_kv, int dk, int dv, int page_size, float coef,
                       int every, hipStream_t stream);

// the same split with a bias on every column of qkv first (f32 [n_head dk + n_kv (dk + dv)], null: none) and the rotation of
// the first rot_dims entries of every query and key head (entry i with entry i + rot_dims / 2; cos and sin times mag;
// rope_table [table_len][rot_dims / 2][2] may be null; inv_freq null: no rotation)
int ti_qkv_prep_write(int dtype, const float* qkv, const float* bias, const float* inv_freq, const float* rope_table,
                      int table_len, float mag, int rot_dims, const int* pos, const int* slot, const int* table,
                      int table_stride, void* pool, void* q_out, int M, int n_head, int n_kv, int dk, int dv, int page_size,
                      float coef, int every, hipStream_t stream);
// out[r] = tanh(alpha[0] x[rows ? rows[r] : r]) * w + b (b may be null), in `out_dtype`
int ti_dyt(int out_dtype, const float* x, const float* alpha, const float* w, const float* b, const int* rows, void* out,
           int n_rows, int H, hipStream_t stream);
// z f32 [R, 2F] = [gate | up], rows ldz floats apart, bias f32 [2F] (null: none) added first.  kind 0: silu(g) u;
// kind 1: g = min(g, limit), u = clamp(u, -limit, limit), g sigmoid(alpha g) (u + 1).  out [R, F] in `out_dtype`
int ti_gated_act(int out_dtype, const float* z, long ldz, const float* bias, void* out, long R, int F, int kind, float limit,
                 float alpha, hipStream_t stream);
// out [M, 2H] = [a | b] rounded to `out_dtype` (a, b f32 [M, H])
int ti_concat_round(int out_dtype, const float* a, const float* b, void* out, int M, int H, hipStream_t stream);

// ---- libti_latent_attention: attention over cached latents (a token keeps [c (R) | kr (r)]; a head's key is [W_uk c | kr],
// its value W_uv c, neither ever formed per token)
// proj f32 [M, ld]: queries [H][d + r] from column 0, [latent (R) | shared key part (r)] from column off_kv.  The latent is
// RMS-normed (norm_w [R], eps) and goes with the rotated key part into the token's row of pool [pages][P][R + r]; the heads'
// last r query entries are rotated in place.  Rotation as in ti_qkv_prep_write (rot_dims <= r).  A page has page_elems
// elements: with P (2 R + r) or more it also holds the latents transposed, [R][P], behind its P rows
int ti_latent_prep(int dtype, float* proj, int ld, int off_kv, const float* norm_w, float eps, const float* inv_freq,
                   const float* rope_table, int table_len, float mag, int rot_dims, const int* pos, const int* slot,
                   const int* table, int table_stride, void* pool, long page_elems, int M, int H, int d, int r, int R, int page_size,
                   hipStream_t stream);
// qa f32 [M, H, R + r] = [W_uk_h^T q_h[:d] | q_h[d:]] with w_uk [H d][R] in `dtype`
int ti_latent_absorb(int dtype, const float* proj, int ld, const void* w_uk, float* qa, int M, int H, int d, int r, int R,
                     hipStream_t stream);
// o f32 [M, H, R] = sum_j p_j c_j over the row's visible positions (window <= 0: all up to its own), p the softmax of
// (qa . [c_j | kr_j]) scale with exp(sink[h]) joining the denominator (sink null: none)
int ti_latent_attention_rows(int dtype, const float* qa, const void* pool, long page_elems, const int* table, int table_stride, const int* pos,
                             const int* slot, const float* sink, float* out, int M, int H, int R, int r, int page_size,
                             float scale, int window, hipStream_t stream);
// out [M, H dv] = W_uv_h o[m, h] with w_uv [H dv][R], both in `dtype`
int ti_latent_expand(int dtype, const float* o, const void* w_uv, void* out, int M, int H, int R, int dv, hipStream_t stream);
// dst [H][cols][rows] = src [H][rows][cols] transposed head by head
int ti_latent_transpose(int dtype, const void* src, void* dst, int H, int rows, int cols, hipStream_t stream);

// ---- libti_latent_attention_bf16: the same on the matrix cores, over pages that hold the latents a second time transposed
// 1 if the sizes are served (R % 16, (R + r) % 8, d % 8, (d + r) % 4, dv % 16, pages of a multiple of 16 rows, R <= 512, R + r <= 576)
int ti_latent_bf16_served(int H, int d, int r, int R, int dv, int page_size);
// qa bf16 [M, H, R + r] from w_uk_t bf16 [H][R][d] (ti_latent_transpose of w_uk)
int ti_latent_absorb_bf16(const float* proj, int ld, const void* w_uk_t, void* qa, int M, int H, int d, int r, int R, hipStream_t stream);
// o bf16 [M, H, R] for the tiles int32 [n][3] = (entry, first row, rows <= 64) of entries int32 [.][4] = (row0, tokens, start, -);
// the block table's row of a tile is its entry's.  use_lds: a tile's four wavefronts share every pair of key blocks through LDS
int ti_latent_attention_tiles_bf16(const void* qa, const void* pool, long page_elems, const int* table, int table_stride,
                                   const int* tiles, const int* entries, const float* sink, void* o, int n_tiles, int H, int R, int r,
                                   int page_size, float scale, int window, int use_lds, hipStream_t stream);
// ... and for single rows (rows int32 [n], null: every row): 16 heads a wavefront; n_splits workgroups share a row's keys
// (part: ti_latent_attention_rows_scratch floats)
int ti_latent_attention_rows_bf16(const void* qa, const void* pool, long page_elems, const int* table, int table_stride, const int* pos,
                                  const int* slot, const int* rows, const float* sink, void* o, int n_rows, int H, int R, int r,
                                  int page_size, float scale, int window, float* part, int n_splits, hipStream_t stream);
long ti_latent_attention_rows_scratch(int n_rows, int H, int R, int r, int n_splits);
// out bf16 [M, H dv] = W_uv_h o[m, h] from o bf16 [M, H, R]
int ti_latent_expand_bf16(const void* o, const void* w_uv, void* out, int M, int H, int R, int dv, hipStream_t stream);

// ---- libti_recurrent: the mLSTM cell as a scan over each request's tokens of the step
// proj f32 [M, ld] holds, from the columns off_* on, the heads' q and k [heads][dk], v [heads][dv] and the gates'
// pre-activations i, f [heads]; state f32, slot_stride floats per slot: [heads][dk dv + dk + 1] (S [dk][dv], n, m);
// entries int32 [n_entries][4] = (first row, tokens, -, state slot); o f32 [M, heads dv] (not yet normed)
int ti_mlstm_scan(const float* proj, int ld, int off_q, int off_k, int off_v, int off_i, int off_f, const float* bias_i,
                  const float* bias_f, float* state, long slot_stride, const int* entries, int n_entries, float* o,
                  int heads, int dk, int dv, float cap, float q_scale, hipStream_t stream);
// the same with long portions cut into chunks that run side by side: chunks int32 [n_chunks][4] = (entry, first row,
// tokens, 1 if the entry's first chunk + 2 if its last) in the entries' order, spans int32 [n_entries][2] = (an entry's
// first chunk, its chunks), chunk_buf f32 [n_chunks][heads][dk dv + dk + 3] scratch.  The same values up to rounding.
int ti_mlstm_scan_chunked(const float* proj, int ld, int off_q, int off_k, int off_v, int off_i, int off_f,
                          const float* bias_i, const float* bias_f, float* state, long slot_stride, const int* entries,
                          int n_entries, const int* chunks, int n_chunks, const int* spans, float* chunk_buf, float* o,
                          int heads, int dk, int dv, float cap, float q_scale, hipStream_t stream);
// out = o / rms(o per head) * w * sigmoid(gate), gate in rows of ld floats from column off_g on
int ti_gated_head_norm(int out_dtype, const float* o, const float* gate, int ld, int off_g, const float* w, void* out,
                       int M, int heads, int dv, float eps, hipStream_t stream);

// libti_attention_bf16: sinks (float [n_head] in device memory, null: none) for the calling thread's next calls of the
// matrix-core attention entry points: exp(sink[head]) joins the softmax's denominator where a column is finished
void ti_attention_bf16_sink(const float* sink);

// ---- libti_hyper: the layer norm, and a residual kept in several streams
// out[r] = layernorm(sum_s coef[s] x_s[rows ? rows[r] : r]) * w (mean and variance, no bias), in `out_dtype`; the streams lie
// stream_stride floats apart; coef null: the first stream alone.  out may be x (float32, one stream).  H up to 16384
int ti_mixed_layernorm(int out_dtype, const float* x, long stream_stride, int S, const float* coef, const int* rows,
                       const float* w, void* out, int n_rows, int H, float eps, hipStream_t stream);
// u[i] = sum_s coef[s] x_s[i] (coef null: the plain sum)
int ti_hyper_combine(const float* x, long stream_stride, int S, const float* coef, float* u, long n, hipStream_t stream);
// every stream a copy of x
int ti_hyper_spread(const float* x, float* streams, long stream_stride, int S, long n, hipStream_t stream);
// x_t <- sum_s mix[s, t] x_s + back[t] y, every t at once from the old streams; y2 (null: none): the output is f1 y + f2 y2
int ti_hyper_write(float* streams, long stream_stride, int S, const float* mix, const float* back, const float* y, const float* y2,
                   float f1, float f2, long n, hipStream_t stream);
// the same write and, in the same pass, out = layernorm(sum_t coef[t] x_t) * w of the new streams (what ti_mixed_layernorm gives)
int ti_hyper_write_read(int out_dtype, float* streams, long stream_stride, int S, const float* mix, const float* back, const float* y,
                        const float* y2, float f1, float f2, const float* coef, const float* w, void* out, int M, int H, float eps,
                        hipStream_t stream);

// ---- libti_gated_attention: attention with per-head norms, values from the keys or mixed with another layer's, a sink, a gate
// proj f32 [M, ld] holds q (n_head x dk), k (n_kv x dk) and v (n_kv x dv; off_v < 0: the values are the keys as projected) from
// the given columns on.  q_w / k_w (null: none): RMS norm of every head before the rotation of its first rot_dims entries.
// mix_mode 1: the values also go to v_kept f32 [M, n_kv dv]; 2: v <- (1 - lambda) v + lambda v_kept (lambda: one float in
// device memory).  q to q_out, k and v into the pages K [n_kv][P][dk] | V [n_kv][dv_rows][P] (dv_rows >= dv, 0: dv; rows of a
// value head beyond dv are written as zeros: values padded to the keys' size for kernels that hold both at one size)
int ti_gated_qkv_prep(int dtype, const float* proj, int ld, int off_q, int off_k, int off_v, const float* q_w, const float* k_w,
                      float eps, const float* inv_freq, const float* rope_table, int table_len, float mag, int rot_dims,
                      int mix_mode, const float* mix_lambda, float* v_kept, const int* pos, const int* slot, const int* table,
                      int table_stride, void* pool, void* q_out, int M, int n_head, int n_kv, int dk, int dv, int dv_rows,
                      int page_size, hipStream_t stream);
// out (T [M, n_head dv]) = src (T [M, n_head src_dv], the first dv of every head) times sigmoid(gate), gate f32 rows of gate_ld
// floats: entry h dv + d (gate_mode 1) or h (gate_mode 2); gate null: times one; src may be out where src_dv = dv
int ti_sigmoid_gate(int dtype, const void* src, int src_dv, void* out, const float* gate, int gate_ld, int gate_mode, int M,
                    int n_head, int dv, hipStream_t stream);
// causal softmax attention of every row over such pages; sink f32 [n_head] (null: none) joins the denominator; gate (null:
// none) f32 rows of gate_ld floats, the output times sigmoid of entry h dv + d (gate_mode 1) or h (gate_mode 2)
int ti_gated_attention_rows(int dtype, const void* q, const void* pool, const int* table, int table_stride, const int* pos,
                            const int* slot, const float* sink, const float* gate, int gate_ld, int gate_mode, void* out, int M,
                            int n_head, int n_kv, int dk, int dv, int dv_rows, int page_size, float scale, int window,
                            hipStream_t stream);

// ---- libti_linear_attention: linear attention with a fixed decay per head, and the gated norm behind it
// S_t = decay_h S_(t-1) + k_t v_t^T, o_t = S_t^T q_t with q, k, v = silu of the given columns of proj f32 [M, ld]; state f32
// [slots][heads][dk][dv]; entry_meta [n_entries][4] = (row0, tokens, start, slot); o f32 [M, heads dv]
int ti_decay_scan(const float* proj, int ld, int off_q, int off_k, int off_v, const float* decay, float* state, long slot_stride,
                  const int* entry_meta, int n_entries, float* o, int heads, int dk, int dv, hipStream_t stream);
// the same with the entries' tokens in chunks that run side by side (chunks [n_chunks][4] = (entry, first row, tokens, 1: the
// entry's first chunk + 2: its last), spans [n_entries][2] = (first chunk, chunks); scratch float [n_chunks][heads][dk dv])
int ti_decay_scan_chunked(const float* proj, int ld, int off_q, int off_k, int off_v, const float* decay, float* state,
                          long slot_stride, const int* entry_meta, int n_entries, const int* chunks, int n_chunks, const int* spans,
                          float* scratch, float* o, int heads, int dk, int dv, hipStream_t stream);
// out = o / rms(o over the whole row) * w * sigmoid(gate), gate in rows of ld floats from column off_g on
int ti_gated_row_norm(int out_dtype, const float* o, const float* gate, int ld, int off_g, const float* w, void* out, int M, int W,
                      float eps, hipStream_t stream);

// ---- libti_residual: layers that norm what a sublayer returns
// x[m] (+)= y'[m] / sqrt(mean(y'[m]^2) + eps) * g; y'[m] = y[m], or with `gather` (int32 [M][n_gather]) the sum of
// the rows y[gather[m][k]] in ascending k (gather null and n_gather > 1: of the rows y[m n_gather + k]).  accumulate 0: x is overwritten (y may be x itself).  rounded (may be null):
// [M][H] of rounded_dtype, the new x rounded for the product that reads it next
int ti_norm_residual(float* x, const float* y, const float* g, const int* gather, int n_gather, int M, int H, float eps,
                     int accumulate, void* rounded, int rounded_dtype, hipStream_t stream);
// out = x rounded to out_dtype
int ti_round_rows(int out_dtype, const float* x, void* out, long n, hipStream_t stream);
// x *= s
int ti_scale(float* x, float s, long n, hipStream_t stream);

// ---- libti_diff_attention: a short convolution over time with carried state, and differential attention
// out[m, c] = sum_j taps[c][j] u(pos[m] - (K - 1) + j)[c]; u f32 [M, C] holds the step's rows, state f32
// [slots][K - 1][C] the K - 1 rows before each entry's start (entries int32 [n][4] = (row0, tokens, start, slot);
// entry_of[m]: the entry of row m), which the call then replaces by the last K - 1 rows up to the step's end
int ti_short_conv(const float* u, const float* taps, float* state, const int* entries, int n_entries, const int* entry_of,
                  const int* pos, float* out, int M, int C, int K, hipStream_t stream);
// qkv f32 [M, n_head 2 dk + n_kv 2 dk + n_kv dv] (each query head and kv head holds two maps of dk): per map RMS
// norm with the weights q_w / k_w [dk] (may be null), rotation of the first rot_dims entries (entry i with entry
// i + rot_dims / 2; cos and sin times mag; rope_table [table_len][rot_dims / 2][2] may be null), q to q_out, k and v
// into pages K [n_kv][P][2 dk] | V [n_kv][dv][P]
// With taps f32 [C][K] (C the width of qkv; null: none) every channel first passes the short convolution of ti_short_conv,
// in the same kernel (state, entries, entry_of as there; the state is moved on afterwards): the same bits as the two calls
int ti_diff_qk_prep(int dtype, const float* qkv, const float* taps, float* state, const int* entries, int n_entries,
                    const int* entry_of, int K, const float* q_w, const float* k_w, float eps, const float* inv_freq,
                    const float* rope_table, int table_len, float mag, int rot_dims, const int* pos, const int* slot,
                    const int* table, int table_stride, void* pool, void* q_out, int M, int n_head, int n_kv, int dk, int dv,
                    int page_size, hipStream_t stream);
// out[m, h] = (a1 - lambda a2) / rms(a1 - lambda a2) * out_scale, a1 and a2 the softmax attention of the head's two
// maps over the keys that are not later than pos[m], in its block of `block` positions (0: none) and inside the window
int ti_diff_attention_rows(int dtype, const void* q, const void* pool, const int* table, int table_stride, const int* pos,
                           const int* slot, void* out, int M, int n_head, int n_kv, int dk, int dv, int page_size, float scale,
                           int block, int window, float lambda, float eps, float out_scale, hipStream_t stream);

// ---- libti_diff_attention_bf16: the same attention on the matrix cores (dk, dv in {32, 64, 128}, pages of 16 n rows);
// 3: sizes not served.  tiles int32 [n_tiles][3] = (entry, first row, rows <= 64) of entries int32 [.][4] = (row0, tokens,
// start, -); the block table's row of an entry is the entry's index
int ti_diff_attention_tiles_bf16(const void* q, const void* pool, const int* table, int table_stride, const int* tiles,
                                 const int* entries, void* out, int n_tiles, int n_head, int n_kv, int dk, int dv,
                                 int page_size, float scale, int block, int window, float lambda, float eps, float out_scale,
                                 int use_lds, hipStream_t stream);
// (use_lds 1: the four wavefronts of a tile share the keys and values they read through LDS; 0: each fetches its own)
// single rows (rows int32 [n_rows], or null: rows 0 .. n_rows - 1); at most 16 query heads a kv head.  n_splits > 1: so many
// workgroups share a row's keys and leave their shares in part (f32, ti_diff_attention_rows_scratch floats) for a kernel that
// merges them
int ti_diff_attention_rows_bf16(const void* q, const void* pool, const int* table, int table_stride, const int* pos,
                                const int* slot, const int* rows, void* out, int n_rows, int n_head, int n_kv, int dk, int dv,
                                int page_size, float scale, int block, int window, float lambda, float eps, float out_scale,
                                float* part, int n_splits, hipStream_t stream);
long ti_diff_attention_rows_scratch(int n_rows, int n_kv, int dv, int n_splits);

// ---- libti_moe: a mixture of experts
// scores (score_kind 0: sigmoid, 1: softmax over the experts, 2: the logits themselves, the weights then being the softmax over
// the chosen logits alone) of h [M, W] against router f32 [E, W] in 32-bit; the `top`
// largest per token (ties: the lower index) to ids int32 [M, top] and wts f32 [M, top] (renormalize: divided by their sum)
int ti_moe_route(int dtype, const void* h, const float* router, int* ids, float* wts, int M, int W, int E, int top,
                 int score_kind, int renormalize, hipStream_t stream);
// the same for a grouped router: correction f32 [E] (null: none) joins the scores for the choice only; the experts form
// n_groups groups of neighbours, a group's score the sum of its two largest choice scores, and only experts of the `keep`
// best groups can be chosen (n_groups <= 1: no groups); weights: the chosen experts' uncorrected scores, divided by their
// sum + sum_floor where `renormalize`, times weight_scale
int ti_moe_route_grouped(int dtype, const void* h, const float* router, const float* correction, int* ids, float* wts, int M,
                         int W, int E, int top, int score_kind, int renormalize, int n_groups, int keep, float weight_scale,
                         float sum_floor, hipStream_t stream);
// y f32 [M, W] = sum_k down[e_k] relu(up[e_k] (s_k h))^2 (scale_input) or sum_k s_k down[e_k] relu(up[e_k] h)^2;
// up [E][F][W], down [E][W][F] in the dtype of h; act: scratch of that dtype, [M top][F]; part: f32 [M top][W].  A workgroup
// per expert and 16 outputs walks its weights once for all the pairs that chose the expert: steps of few tokens, and float32.
// A token's rows of part are added in ascending order into y where y is given, else left to the caller
int ti_moe_experts_rows(int dtype, const void* h, const int* ids, const float* wts, const void* up, const void* down, void* act,
                        float* part, float* y, int M, int W, int F, int E, int top, int scale_input, hipStream_t stream);

// experts with a gate: y[m] = sum_k s_k down[e_k] act(gate[e_k] h, up[e_k] h); gate_up [E][2F][W] holds an expert's gate rows
// above its up rows.  act_kind 0: silu(g) u; 1: g = min(g, limit), u = clamp(u, -limit, limit), g sigmoid(alpha g) (u + 1).
// z: f32 scratch [M top][2F]; act, part, y as above
int ti_moe_experts_rows_gated(int dtype, const void* h, const int* ids, const float* wts, const void* gate_up, const void* down,
                              float* z, void* act, float* part, float* y, int M, int W, int F, int E, int top, int act_kind,
                              float limit, float alpha, hipStream_t stream);

// ---- libti_moe_bf16: the experts for steps of many tokens, on the matrix cores: the (token, expert) pairs are laid out expert
// by expert in tiles of 128 rows and both products run over the tiles.  Scratch: meta int32 [ti_moe_grouped_meta_ints(M top, E)],
// where int32 [M top] (the row of every pair), rows bf16 [M top][W], act bf16 [M top][F], out f32 [M top][W].  y (may be
// null): the tokens' sums; without it the caller adds the rows out[where[m top + k]] in ascending k.  3: sizes not served
long ti_moe_grouped_meta_ints(int n_pairs, int E);
int ti_moe_experts_grouped_bf16(const void* h, const int* ids, const float* wts, const void* up, const void* down, int* meta,
                                int* where, void* rows, void* act, float* out, float* y, int M, int W, int F, int E, int top,
                                int scale_input, hipStream_t stream);

// the gated experts of ti_moe_experts_rows_gated over such tiles; z: f32 scratch [M top][2F]; y is written (the tokens' weighted sums)
int ti_moe_experts_grouped_gated_bf16(const void* h, const int* ids, const float* wts, const void* gate_up, const void* down,
                                      int* meta, int* where, void* rows, float* z, void* act, float* out, float* y, int M, int W,
                                      int F, int E, int top, int act_kind, float limit, float alpha, hipStream_t stream);

// ---- libti_attention_bf16: the same on the matrix cores (head sizes 32, 64, 128; pages of 16 n rows)
// rows of single tokens; n_splits > 1 needs part_o f32 [n_rows, n_head, n_splits, hd] and part_ml f32
// [n_rows, n_head, n_splits, 2]
int ti_attention_decode_bf16(const void* q, const void* pool, const int* table, int table_stride, const int* pos,
                             const int* slot, const int* rows, void* out, float* part_o, float* part_ml, int n_rows,
                             int n_head, int n_kv, int hd, int page_size, float scale, int window, int n_splits,
                             hipStream_t stream);
// the same from the 32-bit projections: norm, rotation and the cache write of the row's own key and
// value happen inside (head sizes 64 and 128, at most 16 q heads per kv head).  slot may be null
// (both entry points) where row m of the step is row m of the block tables and a table row has at
// most 1,024 entries: the page ids are then fetched beside the position, not behind it
int ti_attention_decode_prepared_bf16(const float* qkv, int row_width, const float* q_w, const float* k_w, float eps,
                                      const float* inv_freq, const float* rope_table, int table_len, void* pool,
                                      int write_kv, const int* table, int table_stride, const int* pos,
                                      const int* slot, void* out, float* part_o, float* part_ml, int n_rows,
                                      int n_head, int n_kv, int hd, int page_size, float scale, int window,
                                      int n_splits, hipStream_t stream);
// portions of prompts: tiles int32 [n_tiles][2] = (entry, first row) of 128 rows each, entries int32
// [n_entries][4] = (row0, n_tokens, start_pos, -)
int ti_attention_prefill_bf16(const void* q, const void* pool, const int* table, int table_stride, const int* tiles,
                              const int* entries, void* out, int n_tiles, int n_head, int n_kv, int hd, int page_size,
                              float scale, int window, hipStream_t stream);
// the same for launches of few tiles (head sizes 64, 128): tiles of 64 rows ordered from the most visible
// keys to the fewest; a workgroup takes tile b and tile n_tiles - 1 - b, so that all have about the same work
// n_splits > 1 (up to 8): the keys of every tile are cut into that many runs, each with a workgroup of its
// own, for launches of few tiles against a long context; their results go through part_o [n_rows][n_head]
// [n_splits][hd] and part_ml [n_rows][n_head][n_splits][2] and are merged into out for all n_rows rows of the
// step (rows of no tile get what lies in the buffers: whoever owns them writes them afterwards).
// paired = 0: the same kernel with a workgroup per tile, for launches that fit the chip in one round.
int ti_attention_prefill_paired_bf16(const void* q, const void* pool, const int* table, int table_stride,
                                     const int* tiles, const int* entries, void* out, int n_tiles, int n_head,
                                     int n_kv, int hd, int page_size, float scale, int window, int n_rows,
                                     float* part_o, float* part_ml, int n_splits, int paired, hipStream_t stream);

// the three above with soft-capped scores: s <- softcap tanh(s / softcap) before the softmax (softcap <= 0: none)
int ti_attention_decode_capped_bf16(const void* q, const void* pool, const int* table, int table_stride, const int* pos,
                                    const int* slot, const int* rows, void* out, float* part_o, float* part_ml, int n_rows,
                                    int n_head, int n_kv, int hd, int page_size, float scale, float softcap, int window,
                                    int n_splits, hipStream_t stream);
int ti_attention_prefill_capped_bf16(const void* q, const void* pool, const int* table, int table_stride, const int* tiles,
                                     const int* entries, void* out, int n_tiles, int n_head, int n_kv, int hd, int page_size,
                                     float scale, float softcap, int window, hipStream_t stream);
int ti_attention_prefill_paired_capped_bf16(const void* q, const void* pool, const int* table, int table_stride,
                                            const int* tiles, const int* entries, void* out, int n_tiles, int n_head,
                                            int n_kv, int hd, int page_size, float scale, float softcap, int window,
                                            int n_rows, float* part_o, float* part_ml, int n_splits, int paired,
                                            hipStream_t stream);

// ---- libti_sampling
// out[r] = lowest index of the largest logit; scratch: 2 * 64 * n_rows four-byte words (two stages:
// 64 workgroups per row, then one) or null (one workgroup reads a whole row)
int ti_argmax(const float* logits, int* out, void* scratch, int n_rows, int V, hipStream_t stream);
// ti_argmax for callers that cannot allocate (code under HIP graph capture, tight serving loops,
// harnesses that forbid hipMalloc): the same two-stage kernels with their partial results in a
// device array of the library itself (128 KiB on each GPU it runs on, kept until the process ends)
// instead of a workspace argument.  At most 256 rows, else an error.  It calls no hipMalloc, hipFree or
// allocating routine; calls that overlap on one GPU share the array and race.  It has no counterpart in
// the reference: it is there for callers that cannot allocate.
int ti_argmax_static(const float* logits, int* out, int n_rows, int V, hipStream_t stream);
// temperature, top-k (0: all), top-p and one uniform number per row.  scratch: ti_sample_scratch_bytes(n_rows)
// bytes, zero before the first call and touched by nothing else since (the kernels leave them at zero; calls
// that overlap on one workspace race), or null: then one workgroup walks a whole row, as it does for the rows
// that have no top-k cut.
long ti_sample_scratch_bytes(int n_rows);
int ti_sample(const float* logits, const float* temp, const int* top_k, const float* top_p, const float* uni, int* out,
              void* scratch, int n_rows, int V, hipStream_t stream);


// ---- libti_measure: what the GPU delivers, for the bench tool's fractions
// reads `bytes` bytes (a multiple of 16) once with `blocks` workgroups of 256 threads; sink: `blocks` words
int ti_measure_read(const void* p, long bytes, void* sink, int blocks, hipStream_t stream);
// `blocks` workgroups of four wavefronts, each wavefront `iters` rounds of four 32x32x16 bfloat16 MFMAs on
// registers: blocks * 4 * iters * 4 * 32,768 flops
int ti_measure_mfma(int blocks, int iters, void* sink, hipStream_t stream);
// `blocks` workgroups of one wavefront each read one word every `stride` bytes of [p, p + bytes)
int ti_measure_touch(const void* p, long bytes, long stride, void* sink, int blocks, hipStream_t stream);

#ifdef __cplusplus
}
#endif
