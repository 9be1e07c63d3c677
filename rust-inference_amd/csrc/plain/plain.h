// Plain C++ twins of the kernel families: scalar host code, one function per operation, float32
// arithmetic in the order the reference's CPU path uses, no tiling and no cache tricks.  They are what
// a kernel is meant to compute, written so that it can be read in a minute; the CPU tests hold them
// against the float64 numpy implementation under tests/plain, and the host sampler uses the selection
// functions for logits that never were on a GPU.  Built for the host alone (no GPU code in here).
#pragma once
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

// bfloat16 <-> float32 (round to nearest even, NaN stays quiet NaN: the reference's src/dtype.rs:75-89)
uint16_t ri_plain_f32_to_bf16(float f);
float ri_plain_bf16_to_f32(uint16_t b);

// out[t, :] = table[ids[t], :]; returns 1 for an id outside the table (src/ops/embedding.rs:10-42)
int ri_plain_embedding(float* out, const float* table, const int32_t* ids, int tokens, int vocab, int dim);

// y = x * (1 / sqrt(mean(x^2) + eps)) * gain over groups of `dim` elements (src/ops/norm.rs:7-32)
void ri_plain_rms_norm(float* out, const float* x, const float* gain, int rows, int dim, float eps);
// residual += pending, then the norm of the sum (src/ops/norm.rs:35-62)
void ri_plain_add_rms_norm(float* out, float* residual, const float* pending, const float* gain, int rows, int dim,
                           float eps);

// inv_freq[i] = 1 / theta^(2 i / rot_dim), i < rot_dim / 2, in float32 (src/ops/rope.rs:20)
void ri_plain_rope_inv_freq(float* inv_freq, int rot_dim, float theta);
// rotate-half on x[tokens, heads, head_dim] in place: pairs (i, i + rot_dim/2) of the first rot_dim elements,
// angle = f32(pos) * inv_freq[i] (src/ops/rope.rs:39, :73-74)
void ri_plain_rope(float* x, const int32_t* positions, const float* inv_freq, int tokens, int heads, int head_dim,
                   int rot_dim);

// out = x . w^T, float32 sums in the order of k (src/ops/linear.rs:7-19; src/cpu/linear.rs:158-198)
void ri_plain_linear(float* out, const float* x, const float* w, int m, int n, int k);
// out[t, i] = silu(y[t, i]) * y[t, inter + i] (src/ops/elementwise.rs:9-12, :35-52)
void ri_plain_swiglu(float* out, const float* y, int tokens, int inter);

// Causal grouped-query attention of q[tokens, heads, head_dim] over a paged cache: k_pages
// [pages, kv_heads, page_size, head_dim], v_pages [pages, kv_heads, head_dim, page_size] (values transposed
// inside a page), page_table [seqs, table_width].  The query of token t, at position tok_pos[t] of sequence
// tok_seq[t], sees keys lo..pos with lo = 0 or pos - window + 1; score = (q . k) * scale; online softmax
// with running maximum and sum (src/attention.rs:33-150).
void ri_plain_attention(float* out, const float* q, const float* k_pages, const float* v_pages, const int32_t* tok_pos,
                        const int32_t* tok_seq, const int32_t* page_table, int table_width, int tokens, int heads,
                        int kv_heads, int head_dim, int page_size, int window, float scale);

// first index of the maximum (src/sampling.rs:131-139)
int ri_plain_argmax(const float* row, int n);

// The sampler's generator: xorshift64* seeded through the splitmix64 finaliser (src/sampling.rs:33-53)
uint64_t ri_plain_rng_seed(uint64_t seed);
uint64_t ri_plain_rng_next(uint64_t* state);
float ri_plain_rng_next_f32(uint64_t* state);
// One token from a row of logits (src/sampling.rs:73-127): repetition penalty over the ids in history,
// greedy when temperature <= 0, else temperature, top-k, sort (falling value, rising id), softmax, top-p
// prefix, one draw from *rng.  Returns the token, or -1 when vocab < 1.
int ri_plain_sample(const float* logits, int vocab, const int32_t* history, int n_history, float temperature, int top_k,
                    float top_p, float penalty, uint64_t* rng);

#ifdef __cplusplus
}
#endif
