// C interface of the kernel library.  Every function returns 0 on success; on a
// non-zero return ri_last_error() holds the reason and nothing was launched.
// Pointers are device pointers unless said otherwise; `stream` is a hipStream_t.
// dtype arguments take RiDtype codes: 0 = float32, 1 = bfloat16.
#pragma once
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

const char* ri_last_error(void);
int ri_abi_version(void);
// Compute units of the current device (256 where there is none): what the launch-sizing rules count against.
int ri_compute_units(void);

// out[t, :] = table[ids[t], :] as float32.  ids are int32 and must be < vocab (checked by the caller).
int ri_embed_gather(float* out, const void* table, int table_dtype, const int32_t* ids,
                    int tokens, int dim, void* stream);

// r = residual[src] (+ pending[src]); if rows == NULL: src = row and residual[row] = r is written back;
// else src = rows[row] and nothing is written back.  out[row] = r * rsqrt(mean(r^2) + eps) * gain.
// residual float32, pending of pending_dtype (may be NULL), gain float32, out of out_dtype.
// pending may be `parts` tensors [parts][total_rows][dim] that are added one after the other.
int ri_add_rmsnorm(void* out, int out_dtype, float* residual, const void* pending, int pending_dtype, int parts,
                   int total_rows, const float* gain, float eps, const int32_t* rows, int n_rows, int dim,
                   int tiled, void* stream);

// Plain residual add on gathered rows, no norm: out[row] = residual[src] + pending[src], float32.
// With rows == NULL out may be residual itself (an add in place).
int ri_add_rows(float* out, const float* residual, const void* pending, int pending_dtype,
                const int32_t* rows, int n_rows, int dim, void* stream);

// Per-head RMSNorm of q and k (gains may be NULL: no norm), rotate-half position encoding of the first
// rot_dim elements of each head (inv_freq NULL: none), in place for q, and write of k and v into the pages.
// qkv: [tokens, (heads + 2 kv_heads) * head_dim] of act_dtype.  tok_pos/tok_seq: int32 [tokens].
// page_table: int32 [seqs, table_width].  k_pages: [pages, kv_heads, page_size, head_dim], v_pages (transposed
// inside a page): [pages, kv_heads, head_dim, page_size], both of cache_dtype.
// cu_seqlens (int32 [seqs + 1], may be NULL), seqs and max_new (most new tokens of a sequence) let values be
// written a page at a time; without them every element is written on its own.
// k_pages and v_pages both NULL: nothing goes to the cache; k is normed and rotated in place like q (for a
// caller that changes q and k once more before a second call moves k and v into their pages).
int ri_qk_norm_rope_kv_write(void* qkv, int act_dtype, const float* q_gain, const float* k_gain, float eps,
                             const float* inv_freq, int rot_dim, const int32_t* tok_pos, const int32_t* tok_seq,
                             const int32_t* cu_seqlens, int seqs, int max_new,
                             const int32_t* page_table, int table_width, void* k_pages, void* v_pages,
                             int cache_dtype, int tokens, int heads, int kv_heads, int head_dim, int page_size,
                             int num_pages, void* stream);

// Causal grouped-query attention of each new token over its sequence's pages (any number of new tokens
// per sequence).  q is read from qkv rows (row stride q_stride elements); out: [tokens, heads * head_dim].
// window <= 0: all keys 0..pos; else keys max(0, pos - window + 1)..pos.  v_dim: the size of a value head
// (v_pages: [pages, kv_heads, v_dim, page_size]; out: [tokens, heads * v_dim]).  softcap > 0: a score s becomes
// softcap * tanh(s / softcap) before the softmax.  slopes (float32 [heads] or NULL): a distance bias, the score of
// query head h at position p for the key at position j becomes s - slopes[h] * (p - j).
int ri_attention(void* out, const void* q, int act_dtype, int q_stride, const void* k_pages, const void* v_pages,
                 int cache_dtype, const int32_t* tok_pos, const int32_t* tok_seq, const int32_t* page_table,
                 int table_width, int tokens, int heads, int kv_heads, int head_dim, int v_dim, int page_size,
                 int window, float scale, float softcap, const float* slopes, void* stream);

// Queries and keys for an attention without rotation, keys and values into their pages, from the fused
// projection qkv: [tokens, heads * dim + kv_heads * dim + kv_heads * vdim].  Per-head RMS norm of q and k (gains
// may be NULL), then q *= 1 + temp_coef * ln(floor((pos + 1) / temp_every) + 1) in place (temp_coef 0: none).
// k_pages: [pages, kv_heads, page_size, dim]; v_pages: [pages, kv_heads, vdim, page_size].
// cu_seqlens (int32 [seqs + 1], may be NULL), seqs and max_new (most new tokens of a sequence) let values be
// written a page at a time.
int ri_qk_norm_temper_kv_write(void* qkv, int act_dtype, const float* q_gain, const float* k_gain, float eps,
                               float temp_coef, int temp_every, const int32_t* tok_pos, const int32_t* tok_seq,
                               const int32_t* cu_seqlens, int seqs, int max_new,
                               const int32_t* page_table, int table_width, void* k_pages, void* v_pages,
                               int cache_dtype, int tokens, int heads, int kv_heads, int dim, int vdim, int page_size,
                               void* stream);

// Several residual streams per token (streams: [total_rows, n_streams, dim] float32), the write that waits for
// them, the read and the norm, in one kernel.  For row r (rows == NULL: every row, and the new streams are stored;
// else row rows[r], nothing stored):
//   pending != NULL:  y = sum of its parts [parts, total_rows, dim];  x_t <- sum_s mix[s * n + t] x_s + out_coef[t] y
//   u = sum_t in_coef[t] x_t;  out[r] = norm(u): norm_kind 0 none, 1 RMS (gain), 2 layer norm (gain, bias or NULL).
// mix, out_coef, in_coef NULL: the identity, ones, ones (n_streams 1: residual += pending, then the norm).
// fresh != NULL: [total_rows, dim], the one row every stream starts from; the call spreads it into `streams`.
int ri_streams_read_norm(void* out, int out_dtype, float* streams, const float* fresh, int n_streams,
                         const void* pending, int pending_dtype, int parts, int total_rows, const float* mix,
                         const float* out_coef, const float* in_coef, const float* gain, const float* bias, float eps,
                         int norm_kind, const int32_t* rows, int n_rows, int dim, void* stream);

// out[t, :] = norm(table[ids[t], :] + positions[tok_pos[t], :]) as float32 (positions may be NULL; norm kinds as
// above).  Both tables of table_dtype.
int ri_embed_positions_norm(float* out, const void* table, const void* positions, int table_dtype, const int32_t* ids,
                            const int32_t* tok_pos, const float* gain, const float* bias, float eps, int norm_kind,
                            int tokens, int dim, void* stream);

// Gated linear attention.  proj: [tokens, row] of act_dtype with, for each of `heads` heads, q and k of `dim`
// and v of `vdim` at the column offsets q_off, k_off, v_off (head h at off + h * size); z: float32
// [tokens, heads * dim], the decay's pre-activation without its bias (z_bias: [heads * dim] or NULL).  Per head,
// with alpha = exp(log_sigmoid(z + bias) / tau):   S <- diag(alpha_t) S + k_t v_t^T,   o_t = S^T (q_t * q_scale).
// state: float32 [slots, heads, dim, vdim], read at the sequence's slot before its first token of the step and
// written back after its last.  cu_seqlens: [seqs + 1] over the flat tokens; slots: [seqs].  out: float32
// [tokens, heads * vdim].  With more tokens than sequences (a prompt) z is overwritten by the decays.
int ri_gla_scan(float* out, const void* proj, int act_dtype, int row, int q_off, int k_off, int v_off, float* z,
                const float* z_bias, float tau, float q_scale, float* state, const int32_t* cu_seqlens,
                const int32_t* slots, int seqs, int tokens, int heads, int dim, int vdim, void* stream);

// out[t, h, :] = rms_norm(o[t, h, :]) * gain * silu(gate[t, h, :]): o float32 [tokens, heads * vdim]; gate read
// from proj rows at column g_off; out of act_dtype [tokens, heads * vdim].
int ri_gla_norm_gate(void* out, const float* o, const void* proj, int act_dtype, int row, int g_off, const float* gain,
                     float eps, int tokens, int heads, int vdim, void* stream);

// One new token a sequence (token b is sequence b's): the recurrence's step, the per-head RMS norm and the gate in
// one kernel; out of act_dtype [seqs, heads * vdim].  ri_gla_step_fits: whether it takes these head sizes.
int ri_gla_step_fits(int dim, int vdim);
int ri_gla_step(void* out, const void* proj, int act_dtype, int row, int q_off, int k_off, int v_off, int g_off,
                const float* z, const float* z_bias, float tau, float q_scale, float* state, const int32_t* slots,
                const float* gain, float eps, int seqs, int heads, int dim, int vdim, void* stream);
// The step of the linear attention with a fixed decay per head (q, k, v through silu): float32 out [seqs, heads * vdim],
// neither normed nor gated; head sizes as ri_gla_step_fits says.
int ri_decay_step(float* out, const void* proj, int act_dtype, int row, int q_off, int k_off, int v_off,
                  const float* head_decay, float q_scale, float* state, const int32_t* slots, int seqs, int heads, int dim,
                  int vdim, void* stream);

// ri_decay_scan over prompts in chunks of 64 tokens (three launches: every chunk's own sum, the walk from chunk to
// chunk, every chunk's outputs), where ri_decay_chunks_fit says the head sizes are taken (multiples of 4 up to 128;
// the offsets and the row multiples of 4 too).  max_new: the most new tokens of a sequence; workspace: float32 of at
// least ri_decay_chunks_workspace(...) floats.  The results differ from ri_decay_scan's by rounding alone.
int ri_decay_chunks_fit(int dim, int vdim);
long ri_decay_chunks_workspace(int seqs, int tokens, int heads, int dim, int vdim);
int ri_decay_scan_chunked(float* out, const void* proj, int act_dtype, int row, int q_off, int k_off, int v_off,
                          const float* head_decay, float q_scale, float* state, const int32_t* cu_seqlens,
                          const int32_t* slots, int seqs, int tokens, int max_new, int heads, int dim, int vdim,
                          float* workspace, long workspace_floats, void* stream);

// The gated delta rule.  proj: [tokens, row] of act_dtype with the projections of q and k (kv_heads heads of dim each)
// and v (heads heads of vdim) side by side from column q_off on: `channels` = 2 kv_heads dim + heads vdim columns.
// ri_delta_prepare: per channel the causal convolution over time with taps [channels, ntaps] (last column: the
// current token's) and silu, the inputs before a step's first token taken from tails [slots, ntaps - 1, channels]
// (float32; zeros at a sequence's start); q and k made unit vectors per head (x / sqrt(sum x^2 + 1e-6)), q also
// times dim^(-1/2); qkv: float32 [tokens, channels].  gates: float32 [tokens, 2 heads]: g = exp(-exp(a_log) *
// softplus(a + dt_bias)) then beta = sigmoid(b), from ab [tokens, 2 heads] (a then b).  Then the tails are moved on
// by the step's tokens.
int ri_delta_prepare(float* qkv, float* gates, const void* proj, int act_dtype, int row, int q_off, const float* taps,
                     int ntaps, float* tails, const float* ab, const float* a_log, const float* dt_bias,
                     const int32_t* tok_seq, const int32_t* cu_seqlens, const int32_t* slots, int seqs, int tokens,
                     int heads, int kv_heads, int dim, int vdim, void* stream);
// Per sequence and head, over the sequence's new tokens in order: S <- g S; u = beta (v - S^T k); S <- S + k u^T;
// o = S^T q.  state: float32 [slots, heads, dim, vdim]; out: float32 [tokens, heads * vdim].
int ri_delta_max_dim();
// slices: over how many lanes a column's rows are spread, 4 or 8; 0: by the size of the launch.
int ri_delta_scan(float* out, const float* qkv, const float* gates, float* state, const int32_t* cu_seqlens,
                  const int32_t* slots, int seqs, int tokens, int heads, int kv_heads, int dim, int vdim, int slices,
                  void* stream);

// One new token a sequence (token b is sequence b's; cu_seqlens is 0, 1, .., seqs): ri_delta_prepare, ri_delta_scan, the
// per-head RMS norm over vdim with `gain` and the gate silu(g) (read from proj rows at column g_off) in one kernel, then
// the tails moved on; out of act_dtype [seqs, heads * vdim].  ri_delta_step_fits: whether it takes these head sizes.
int ri_delta_step_fits(int dim, int vdim);
int ri_delta_step(void* out, const void* proj, int act_dtype, int row, int q_off, int g_off, const float* taps, int ntaps,
                  float* tails, const float* ab, const float* a_log, const float* dt_bias, float* state,
                  const int32_t* cu_seqlens, const int32_t* slots, const float* gain, float eps, int seqs, int heads,
                  int kv_heads, int dim, int vdim, void* stream);

// A mixture of experts' router.  z: float32 [tokens, experts] router logits; s = sigmoid(z); the `top` experts with
// the largest s + correction (the lower index on a tie) are chosen; their weights are their s divided by the sum of
// the chosen s (+ 1e-20).  ids: int32 [tokens, top] in the order chosen; weights: float32 [tokens, top]; dense:
// float32 [tokens, experts], the weight of every expert, zero where it was not chosen.
int ri_experts_route(int32_t* ids, float* weights, float* dense, const float* z, const float* correction, int tokens,
                     int experts, int top, void* stream);
// The experts' activation on the gate and up branches of all experts side by side: gu [tokens, experts, 2, ff]
// (gate then up); g = min(gate, limit), u = clamp(up, -limit, limit);
// out[t, e, i] = dense[t, e] * g * sigmoid(1.702 g) * (u + 1), zero for experts that the token did not choose
// (dense NULL: every weight 1).
int ri_experts_activate(void* out, const void* gu, int dtype, const float* dense, int tokens, int experts, int ff,
                        float limit, void* stream);

// Many tokens: the assignments (token t's k-th expert is assignment t * top + k) sorted by expert and, inside an
// expert, by token.  dest[p]: the row of assignment p; offsets[e]: where expert e's rows begin (experts + 1
// entries); rank and counts: workspaces of `pairs` and `experts` entries.  ri_experts_gather copies every
// assignment's token row (bfloat16, dim a multiple of 8) to its place; ri_experts_combine adds a token's rows of y
// (bfloat16 [pairs, dim]) times the router's weights, in the order chosen, into float32 out [tokens, dim].
int ri_experts_sort(int32_t* dest, int32_t* offsets, int32_t* rank, int32_t* counts, const int32_t* ids, int pairs,
                    int experts, void* stream);
int ri_experts_gather(void* rows, const void* x, const int32_t* dest, int pairs, int top, int dim, void* stream);
int ri_experts_combine(float* out, const void* y, const int32_t* dest, const float* weights, int tokens, int top, int dim,
                       void* stream);

// The experts of a few tokens, reading only the rows of the experts chosen (bfloat16): x [tokens, dim]; gu
// [experts * 2 * ff, dim] (every expert's gate rows, then its up rows); down [dim, experts * ff]; ids and weights
// [tokens, top] from ri_experts_route; act: workspace [tokens * top, ff] bfloat16; out: float32 [tokens, dim], the
// weighted sum of the chosen experts' outputs, added in the order chosen.
int ri_experts_few_tokens(float* out, void* act, const void* x, const void* gu, const void* down, const int32_t* ids,
                          const float* weights, int tokens, int experts, int top, int ff, int dim, float limit,
                          void* stream);

// out[i] = max(y[i], 0)^2.
int ri_relu_squared(void* out, const void* y, int dtype, long total, void* stream);
// out[i] = 0.5 y (1 + tanh(sqrt(2 / pi) (y + 0.044715 y^3))), in float32.
int ri_gelu_tanh(void* out, const void* y, int dtype, long total, void* stream);
// out[i] = 0.5 y (1 + erf(y / sqrt(2))), in float32.
int ri_gelu_erf(void* out, const void* y, int dtype, long total, void* stream);

// The same attention on the matrix cores, for bfloat16, pages of 32 tokens and head_dim 32, 64 or 128 (softcap and
// slopes as in ri_attention; slopes NULL: no distance bias).
// Prefill form: any number of new tokens per sequence (cu_seqlens: int32 [seqs + 1] over the flat tokens,
// max_new: the most new tokens of any sequence); at most 64 query heads per kv head.
int ri_attention_prefill_bf16(void* out, const void* qkv, int q_stride, const void* k_pages, const void* v_pages,
                              const int32_t* cu_seqlens, const int32_t* tok_pos, const int32_t* page_table,
                              int table_width, int seqs, int max_new, int heads, int kv_heads, int head_dim,
                              int page_size, int window, float scale, float softcap, const float* slopes, void* stream);
// (softcap > 0, here and in the decode form: a score s becomes softcap * tanh(s / softcap) before the softmax)

// Decode form: exactly one new token per sequence; keys in chunks of 256 (in a step of few workgroups each cut into
// 2 or 4 pieces), joined by a second kernel.
// workspace: float32 [seqs, heads, max_chunks * pieces, head_dim + 2]; max_chunks >= ri_attention_decode_chunks(longest
// sequence after this step), pieces = ri_attention_decode_pieces(seqs, kv_heads, heads, max_chunks); at most 16
// query heads per kv head.
int ri_attention_decode_chunks(int max_len);
int ri_attention_decode_pieces(int seqs, int kv_heads, int heads, int max_chunks);
// Whether ri_attention_decode_bf16 takes a step of this size with its streaming kernel (a workgroup walks a
// whole run of a sequence's pages; no join when a sequence is one run): the number of runs per sequence, or
// 0 for one workgroup per chunk.
int ri_attention_decode_streams(int seqs, int kv_heads, int max_chunks);
int ri_attention_decode_bf16(void* out, float* workspace, const void* qkv, int q_stride, const void* k_pages,
                             const void* v_pages, const int32_t* cu_seqlens, const int32_t* tok_pos,
                             const int32_t* page_table, int table_width, int seqs, int max_chunks, int heads,
                             int kv_heads, int head_dim, int page_size, int window, float scale, float softcap,
                             const float* slopes, int tiled_out, void* stream);
// The same with the first keep_first keys visible behind a window and a number per head (sinks, may be NULL) whose
// exponential joins the softmax's denominator; for steps that ri_attention_decode_streams says do not stream.
int ri_attention_decode_kept_bf16(void* out, float* workspace, const void* qkv, int q_stride, const void* k_pages,
                                  const void* v_pages, const int32_t* cu_seqlens, const int32_t* tok_pos,
                                  const int32_t* page_table, int table_width, int seqs, int max_chunks, int heads,
                                  int kv_heads, int head_dim, int page_size, int window, float scale, float softcap,
                                  const float* slopes, int tiled_out, int keep_first, const float* sinks, void* stream);

// tiled_out (both decode forms): the result [seqs, heads * head_dim] is written in the matrix cores' operand order
// (see tiled_at in common.h) for the packed product that reads it.
// The decode attention of a layer from the raw fused projection (which is not changed): per-head norm (gains
// may be NULL) and rotation (inv_freq may be NULL) of the new token's q and k, its k and v into their pages
// and attention in chunks of 256 keys in one kernel, the join in a second.
int ri_attention_decode_fused_bf16(void* out, float* workspace, const void* qkv, int q_stride, const float* q_gain,
                                   const float* k_gain, float eps, const float* inv_freq, void* k_pages,
                                   void* v_pages, const int32_t* tok_pos, const int32_t* page_table, int table_width,
                                   int seqs, int max_chunks, int heads, int kv_heads, int head_dim, int page_size,
                                   int window, float scale, int tiled_out, void* stream);

// out[M, N] (float32) = x[M, K] (float32) . w[N, K]^T, w float32 or bfloat16; true 32-bit arithmetic.
int ri_gemm_f32(float* out, const float* x, const void* w, int w_dtype, int m, int n, int k, void* stream);

// out[M, N] (out_dtype) = x[M, K] . w[N, K]^T for bfloat16 x and w, float32 accumulation, M <= 8.
// swiglu != 0: w is [2 * N, K] = gate rows then up rows and out[m, n] = silu(gate) * up.
int ri_gemv_bf16(void* out, int out_dtype, const void* x, const void* w, int m, int n, int k, int swiglu,
                 void* stream);

// The same with the weights packed ahead of time into MFMA tiles: [ceil(n/16)][ceil(k/32)][64 lanes][8],
// lane l of a tile holding row l % 16, k 8 * (l / 16)..+8, zero beyond n and k; with swiglu the up matrix's
// ceil(n/16) row tiles follow the gate's.
// parts > 1 cuts K into that many pieces whose float32 sums go to out[part][m][n] (the consumer adds them in
// order); it needs out_dtype float32 and no swiglu.
// tiled: bit 0, the rows of x lie in the matrix cores' operand order (tiles of 32 columns, each 64 lanes x 8
// elements, lane l holding row l % 16 and the columns 8 * (l / 16) ..+8 of the tile); bit 1, the bfloat16
// result is to lie so (a product writes it for the next one, which then loads a tile as one kilobyte).
int ri_gemm_skinny_packed_bf16(void* out, int out_dtype, const void* x, const void* wpacked, int m, int n, int k,
                               int swiglu, int parts, int tiled, void* stream);

// The same product for 17 to 64 rows of x (it takes fewer too): every weight fragment meets two or four
// tiles of 16 rows of x.  No parts, no links.
int ri_gemm_mid_packed_bf16(void* out, int out_dtype, const void* x, const void* wpacked, int m, int n, int k,
                            int swiglu, int tiled, void* stream);

// The two decode-size products linked to the RMSNorms around them, so that those need no kernels of their
// own.  W . norm(r) with norm(r) = r * inv * g equals inv * (W . (r * g)), inv = 1 / sqrt(mean(r^2) + eps):
//   consumer side (ssq_in != NULL): x holds bfloat16(r * g) and ssq_in[m][n_in] partial sums of r[m]^2 over
//     a row of `dim` elements; the result rows are scaled by inv (before the activation with swiglu).
//   producer side (residual != NULL): the result is added into residual[m][n] (float32, in place), the new
//     value times next_gain[n] goes to xg_out[m][n] (bfloat16) and each workgroup's sum of its squares to
//     ssq_out[m][partials]; out is not written.  No swiglu on this side.
// ri_*_partials: the number of partial sums a row gets from a product with these sizes.
int ri_gemv_bf16_partials(int n, int k);
int ri_gemv_bf16_linked(void* out, int out_dtype, const void* x, const void* w, int m, int n, int k, int swiglu,
                        const float* ssq_in, int n_in, float eps, int dim, float* residual, const float* next_gain,
                        void* xg_out, float* ssq_out, void* stream);
int ri_gemm_skinny_packed_bf16_partials(int n);
int ri_gemm_skinny_packed_bf16_linked(void* out, int out_dtype, const void* x, const void* wpacked, int m, int n,
                                      int k, int swiglu, const float* ssq_in, int n_in, float eps, int dim,
                                      float* residual, const float* next_gain, void* xg_out, float* ssq_out,
                                      int tiled, void* stream);

// out[m, :] = bfloat16(xg[m, :] * inv[m]), inv[m] = 1 / sqrt(sum_j ssq[m, j] / dim + eps): finishes a norm whose
// scaling was left to a product (xg = bfloat16(r * gain) and n_in partial sums of r^2 per row), for a reader
// that cannot do it.  x_tiled: xg lies in the matrix cores' order (at most 64 rows); out is always in rows.
int ri_finish_norm(void* out, const void* xg, const float* ssq, int n_in, float eps, int dim, int rows, int x_tiled,
                   void* stream);

// The packed product for 17 to 64 rows of x: the three or four wavefronts of a workgroup, on as many
// neighbouring row tiles, share the tiles of x through LDS.  parts > 1 cuts K into that many stretches whose
// float32 sums go to out[parts][m][n]; ri_gemm_wide_packed_bf16_plan says how many wavefronts and parts fill
// the machine most evenly for a matrix (with swiglu: never parts).  tiled as in ri_gemm_skinny_packed_bf16.
// 65 to 128 rows of x: every wavefront takes two neighbouring row tiles; float32 sums in plain rows, no
// activation, x in plain rows, depth 1.  129 to 256 rows: two such passes.  With the activation 65 to 128 rows
// are taken with five to eight wavefronts a workgroup (K whole, plain rows in and out, depth 1).  ri_gemm_wide_stretch_plan: wavefronts and stretches for a product of m
// rows without the activation.
int ri_gemm_wide_packed_bf16_plan(int n, int k, int swiglu, int* waves, int* parts);
int ri_gemm_wide_stretch_plan(int m, int n, int k, int* waves, int* parts);
int ri_gemm_wide_packed_bf16(void* out, int out_dtype, const void* x, const void* wpacked, int m, int n, int k,
                             int swiglu, int parts, int tiled, int depth, int waves, void* stream);
// (depth: 1 or 2 slices of eight weight fragments that a wavefront keeps in flight.  With parts > 1 and swiglu
// the parts are [parts][m][2 n]: gate sums then up sums, the activation left to ri_sum_parts.)
// out[m, i] = sum over p, in order, of parts[p][m][i] (float32 parts; out float32 or bfloat16, in rows or, for
// bfloat16 and at most 64 rows, in the matrix cores' order).  swiglu: the parts' rows are 2 x width, gate sums
// then up sums, and out[m, i] = silu(sum gate) * (sum up).
int ri_sum_parts(void* out, int out_dtype, const float* parts, int n_parts, int rows, int width, int swiglu, int tiled,
                 void* stream);

// x[t, i] += bias[i] in place (bias float32 [dim], x of dtype [rows, dim]).
int ri_add_bias(void* x, int dtype, const float* bias, int rows, int dim, void* stream);

// out[t, i] = silu(y[t, i]) * y[t, inter + i]; y: [tokens, 2 * inter].
// tiled: the bfloat16 result (at most 64 rows, inter a multiple of 8) in the matrix cores' order.
int ri_swiglu(void* out, const void* y, int dtype, int tokens, int inter, int tiled, void* stream);

// ids[r] = first index of the maximum of logits[r, :] (float32).  workspace: ri_argmax_workspace_bytes(rows).
int ri_argmax_workspace_bytes(int rows);
int ri_argmax(int32_t* ids, const float* logits, void* workspace, int rows, int vocab, void* stream);

// ri_argmax for callers that cannot allocate device memory (code under HIP graph capture, tight serving
// loops, harnesses that forbid hipMalloc): the workspace is a device array built into the library, half a
// megabyte that each GPU the library runs on holds until the process ends, for at most
// ri_argmax_static_max_rows() = 1024 rows; more rows are refused.  It calls no allocating routine.  The
// reference has no counterpart (its argmax allocates its result: src/cuda/ops.rs:251-260).  Every call on a GPU uses
// that GPU's one array: calls that overlap on one GPU (two streams, two threads) race; calls in stream order
// do not.  Same result as ri_argmax.
int ri_argmax_static_max_rows(void);
int ri_argmax_static(int32_t* ids, const float* logits, int rows, int vocab, void* stream);

// Next-token selection, one row of float32 logits per sequence: repetition penalty over the token ids
// marked in seen (a byte per vocabulary entry; row seen_rows[r] of it, or row r when seen_rows is NULL;
// seen may be NULL), greedy when temperature <= 0, else temperature, top-k (0: off), top-p (1: off) and
// one draw with uniform[r] in [0, 1).
int ri_sample(int32_t* out, const float* logits, const uint8_t* seen, const int32_t* seen_rows, const float* uniform,
              int rows, int vocab, float temperature, int top_k, float top_p, float penalty, void* stream);

// seen[rows[i], tokens[i]] = 1 for i < n.
// The same selection (temperature > 0 only) with every row cut over many workgroups and one launch per
// pass: the form for large vocabularies, where one workgroup's loads in flight bound a pass.  The same
// token as ri_sample for the same arguments.  workspace: ri_sample_split_workspace_bytes(rows) bytes, any
// contents.
long ri_sample_split_workspace_bytes(int rows);
int ri_sample_split(int32_t* out, const float* logits, const uint8_t* seen, const int32_t* seen_rows,
                    const float* uniform, void* workspace, int rows, int vocab, float temperature, int top_k,
                    float top_p, float penalty, void* stream);

int ri_mark_seen(uint8_t* seen, const int32_t* rows, const int32_t* tokens, int n, int vocab, void* stream);

// ---- the host side of the cache (no device call; handles are opaque; int results: 0, or 1 with the error
// text set, unless said otherwise)
// A pool of pages and every slot's table of them [num_slots][max_pages_per_slot] (-1: unmapped), pages handed
// out lowest number first.  window 0: every key stays; else pages behind the window go back at ri_pool_trim.
void* ri_pool_new(int num_pages, int page_size, int num_slots, int max_pages_per_slot, int window);   // NULL: error
void ri_pool_delete(void* pool);
int32_t* ri_pool_tables(void* pool);
int ri_pool_free_count(void* pool);
int ri_pool_pages_needed(void* pool, int slot, long length_before, long new_tokens);                  // the count
int ri_pool_reserve(void* pool, int slot, long length_before, long new_tokens);
int ri_pool_trim(void* pool, int slot, long length);
// The first `tokens` positions of every sequence stay mapped however far a window has moved on.
int ri_pool_keep_first(void* pool, int tokens);
int ri_pool_release(void* pool, int slot);
int ri_pool_check(void* pool);
// Slots, every slot's length, and the pools (not owned) that the slots hold pages in.
void* ri_cache_new(void* const* pools, int num_pools, int num_slots, int max_seq_len);                // NULL: error
void ri_cache_delete(void* cache);
int ri_cache_acquire(void* cache);                                       // the slot, or -1
int ri_cache_release(void* cache, int slot);
int ri_cache_is_held(void* cache, int slot);                             // 0 or 1
int ri_cache_check_held(void* cache, int slot);
int ri_cache_free_slots(void* cache);                                    // the count
long ri_cache_length(void* cache, int slot);                             // the length, or -1
long ri_cache_longest(void* cache, const int32_t* slots, int n);        // the longest of them, or -1
int ri_cache_reserve(void* cache, const int32_t* slots, const int32_t* counts, int n);     // all or nothing
int ri_cache_commit(void* cache, const int32_t* slots, const int32_t* counts, int n);
int ri_cache_check(void* cache);
// A step's layout as one block of int32 words, every piece on a 16-byte boundary: tokens, each token's
// sequence and position, sequence starts (n + 1), slots, lengths after the step, wanted rows, one page
// table [n][width] per pool; offsets[7 + pools] says where each piece begins.  Returns the words used, -1 on
// error.  Between ri_cache_reserve and ri_cache_commit of the same step.
long ri_cache_plan_step(void* cache, const int32_t* slots, const int32_t* counts, int n, const int32_t* tokens,
                        const int32_t* want_rows, int n_want, int vocab, int width, int32_t* words, long capacity,
                        int64_t* offsets);

// ---- layers whose norm sits behind the residual sum (postnorm.hip)
// residual <- norm(alpha * residual + y + y_bias), the norm a layer norm (kind 2, with bias) or an RMS norm (kind 1); y
// [rows, dim] or float32 [parts, rows, dim]; act: the new residual in the activations' format, or NULL.
int ri_scaled_sum_norm(float* residual, void* act, int act_dtype, const void* y, int y_dtype, int parts,
                       const float* y_bias, float alpha, const float* gain, const float* bias, float eps, int kind,
                       int rows, int dim, void* stream);
// out [rows, ff] = g sigmoid(1.702 g) (u + 1), g = min(gate + b_gate, limit), u = clamp(up + b_up, -limit, limit), for
// gu [rows, gate | up]; the biases may be NULL.
int ri_glu_clamped_bias(void* out, const void* gu, int dtype, const float* b_gate, const float* b_up, float limit,
                        int rows, int ff, void* stream);
// out [tokens, experts * ff] = dense[t, e] * act(u[t, e, :]); kind 0: exact GELU, 1: its tanh form, 2: squared ReLU;
// dense NULL: every weight 1.
int ri_experts_activate_plain(void* out, const void* u, int dtype, const float* dense, int dense_stride, int tokens,
                              int experts, int ff, int kind, void* stream);
// x <- cap * tanh(x / cap) in place.
int ri_softcap_rows(float* x, float cap, long total, void* stream);

// ---- attention over a cached latent (latent.hip)
int ri_latent_prepare(void* proj, int act_dtype, int stride, int q_off, int kv_off, const float* gain, float eps,
                      const float* inv_freq, const int32_t* tok_pos, const int32_t* tok_seq, const int32_t* page_table,
                      int table_width, void* k_pages, void* v_pages, int cache_dtype, int page_size, int tokens, int heads,
                      int dim, int rot, int rank, void* stream);
// out[t, out_off + h * out_head + 0..n) = scale * sigmoid(gates[t, g_off + h]) * x[t, x_off + h * x_head + 0..k) W_h, W
// [heads, k, n]; the extra elements of x behind k are copied behind n; gates may be NULL.
int ri_head_products(void* out, int out_dtype, int out_stride, int out_off, int out_head, const void* x, int x_dtype,
                     int x_stride, int x_off, int x_head, const void* w, int w_dtype, const void* gates, int g_stride,
                     int g_off, float scale, int tokens, int heads, int k, int n, int extra, void* stream);
// The attention over the cached latent on the matrix cores (latent_mfma.hip): bfloat16, pages of 32, (key_dim, rank) one of
// (576, 512), (288, 256), (160, 128).  chunks > 1: a token's pages in chunks of chunk_pages that run side by side, joined by a
// second launch; partial: float32 workspace [tokens][heads][chunks][rank + 2].
int ri_latent_attention_mfma_fits(int key_dim, int rank, int page_size);
int ri_latent_attention_mfma(void* out, const void* q, int q_stride, const void* k_pages, const void* v_pages,
                             const int32_t* tok_pos, const int32_t* tok_seq, const int32_t* page_table, int table_width,
                             int tokens, int heads, int key_dim, int rank, int page_size, float scale, const float* sinks,
                             float* partial, int chunks, int chunk_pages, void* stream);

// ---- windowed attention whose heads talk (talking_attention.hip)
int ri_whole_norm_kv_write(void* proj, int act_dtype, int stride, int q_off, int k_off, const float* q_gain,
                           const float* k_gain, float eps, const int32_t* tok_pos, const int32_t* tok_seq,
                           const int32_t* page_table, int table_width, void* k_pages, void* v_pages, int cache_dtype,
                           int page_size, int tokens, int heads, int kv_heads, int dim, void* stream);
// shares > 1: out is float32 [shares][tokens][out_stride] partial sums for the caller to add; stats: float32 workspace
// [tokens][heads][2].
int ri_talking_attention_shares(int tokens, int longest);
int ri_talking_attention(void* out, int out_dtype, int out_stride, int out_off, float out_scale, int shares, float* stats,
                         const void* q, int act_dtype, int q_stride, int q_off, const void* k_pages, const void* v_pages,
                         int cache_dtype, const int32_t* tok_pos, const int32_t* tok_seq, const int32_t* page_table,
                         int table_width, int tokens, int heads, int kv_heads, int dim, int page_size, int window, float scale,
                         const float* r1, const float* r2, const float* talk, void* stream);
// The same attention on the matrix cores (talking_mfma.hip): bfloat16, pages of 32, heads of 32, 64 or 128, a multiple of 8
// heads up to 32; tiles: the sum over the sequences of their new tokens in sixteens, rounded up.
int ri_talking_attention_mfma_fits(int heads, int kv_heads, int dim, int page_size);
int ri_talking_attention_mfma(void* out, float* stats, const void* q, int q_stride, int q_off, const void* k_pages,
                              const void* v_pages, const int32_t* tok_pos, const int32_t* cu_seqlens, int seqs,
                              const int32_t* page_table, int table_width, int tiles, int heads, int kv_heads, int dim,
                              int page_size, int window, float scale, const float* r1, const float* r2, const float* talk,
                              void* stream);

// ---- time mixing (timemix.hip)
int ri_shift_mix(void* out, int out_dtype, const float* x, const float* kept, const float* mu, int n_mix,
                 const int32_t* tok_seq, const int32_t* cu_seqlens, const int32_t* slots, int tokens, int width, void* stream);
int ri_shift_keep(float* kept, const float* x, const int32_t* cu_seqlens, const int32_t* slots, int seqs, int width,
                  void* stream);
int ri_timemix_max_dim();
int ri_tanh_rows(void* out, int out_dtype, const float* x, long total, void* stream);
int ri_timemix_scan(void* out, int out_stride, int out_off, float out_scale, const void* r, const void* k, const void* v,
                    const void* g, int act_dtype, const float* z, const float* w0, const float* u, const float* gain,
                    float eps, float* state, const int32_t* cu_seqlens, const int32_t* slots, int seqs, int heads, int dim,
                    void* stream);
// The same walk with a wavefront on 16 columns of the state (heads of up to 128); o: float32 workspace [tokens, heads * dim]; z is overwritten with the decays.
int ri_timemix_scan_cols_fits(int dim);
int ri_timemix_scan_cols(void* out, int out_stride, int out_off, float out_scale, float* o, const void* r, const void* k,
                         const void* v, const void* g, int act_dtype, float* z, const float* w0, const float* u,
                         const float* gain, float eps, float* state, const int32_t* cu_seqlens, const int32_t* slots, int tokens,
                         int seqs, int heads, int dim, void* stream);

// ---- the state-space mixer (ssd.hip)
// update_tails 0: the convolution; 1: the tails move on by the step's tokens (call it after the convolution).
int ri_causal_conv_silu(float* out, const void* proj, int act_dtype, int stride, int col0, const float* taps_w,
                        const float* bias, float* tails, int taps, const int32_t* tok_seq, const int32_t* cu_seqlens,
                        const int32_t* slots, int tokens, int seqs, int channels, int update_tails, void* stream);
int ri_ssd_scan(float* out, const float* xbc, int channels, int b_off, int c_off, const void* proj, int act_dtype, int stride,
                int z_off, int dt_off, const float* dt_bias, const float* a_log, const float* d_skip, float* state,
                const int32_t* cu_seqlens, const int32_t* slots, int seqs, int heads, int groups, int n, int vdim,
                void* stream);
// The same walk with a wavefront on 16 columns of the state, for states of up to 128 rows.
int ri_ssd_scan_cols_fits(int n, int vdim);
int ri_ssd_scan_cols(float* out, const float* xbc, int channels, int b_off, int c_off, const void* proj, int act_dtype, int stride,
                     int z_off, int dt_off, const float* dt_bias, const float* a_log, const float* d_skip, float* state,
                     const int32_t* cu_seqlens, const int32_t* slots, int seqs, int heads, int groups, int n, int vdim,
                     void* stream);
int ri_group_rms_norm(void* out, int out_dtype, const float* x, const float* gain, float eps, int rows, int width, int parts,
                      void* stream);

#ifdef __cplusplus
}
#endif
