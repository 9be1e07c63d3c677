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
// window <= 0: all keys 0..pos; else keys max(0, pos - window + 1)..pos.
int ri_attention(void* out, const void* q, int act_dtype, int q_stride, const void* k_pages, const void* v_pages,
                 int cache_dtype, const int32_t* tok_pos, const int32_t* tok_seq, const int32_t* page_table,
                 int table_width, int tokens, int heads, int kv_heads, int head_dim, int page_size, int window,
                 float scale, void* stream);

// The same attention on the matrix cores, for bfloat16, pages of 32 tokens and head_dim 32, 64 or 128.
// Prefill form: any number of new tokens per sequence (cu_seqlens: int32 [seqs + 1] over the flat tokens,
// max_new: the most new tokens of any sequence); at most 64 query heads per kv head.
int ri_attention_prefill_bf16(void* out, const void* qkv, int q_stride, const void* k_pages, const void* v_pages,
                              const int32_t* cu_seqlens, const int32_t* tok_pos, const int32_t* page_table,
                              int table_width, int seqs, int max_new, int heads, int kv_heads, int head_dim,
                              int page_size, int window, float scale, void* stream);

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
                             int kv_heads, int head_dim, int page_size, int window, float scale, int tiled_out, void* stream);

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

#ifdef __cplusplus
}
#endif
