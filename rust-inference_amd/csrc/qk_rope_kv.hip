// Per-head q/k RMSNorm, rotate-half position encoding and the write of keys and values into
// their pages, in one pass over the fused qkv projection.  One wavefront per (token, head).
//
// The reference does this in four launches and rounds to 16 bits after each
// (src/cuda/kernels.cu:98-108 norm, :127-142 rotation, :322-336 page write); here a q or k
// element is normed and rotated in float32 and rounded once.
#include "api.h"
#include "common.h"

#define QK_MAX_PAIRS 4   // pairs per lane: head_dim / 2 <= 64 * QK_MAX_PAIRS

template <typename TA, typename TC>
__global__ void qk_norm_rope_kv_write_kernel(
    TA* __restrict__ qkv, const float* __restrict__ q_gain, const float* __restrict__ k_gain, float eps,
    const float* __restrict__ inv_freq, const int32_t* __restrict__ tok_pos,
    const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ page_table, int table_width,
    TC* __restrict__ k_pages, TC* __restrict__ v_pages, int tokens, int heads, int kv_heads, int head_dim,
    int page_size) {
    const int lane = threadIdx.x & (RI_WAVE - 1);
    const int waves_per_block = blockDim.x / RI_WAVE;
    const int all_heads = heads + 2 * kv_heads;
    const long item = (long)blockIdx.x * waves_per_block + threadIdx.x / RI_WAVE;
    if (item >= (long)tokens * all_heads) return;          // whole wavefront leaves together
    const int t = (int)(item / all_heads), hh = (int)(item % all_heads);
    const int half = head_dim / 2;
    TA* x = qkv + (size_t)t * all_heads * head_dim + (size_t)hh * head_dim;

    const int pos = tok_pos[t];
    TC* dst = nullptr;          // where a k head goes
    if (hh >= heads) {
        const int kvh = (hh - heads) % kv_heads;
        const int page = page_table[(size_t)tok_seq[t] * table_width + pos / page_size];
        const size_t head_base = ((size_t)page * kv_heads + kvh) * page_size * head_dim;
        if (hh >= heads + kv_heads) {
            // v: a copy, no norm and no rotation, transposed inside the page: [head_dim][page_size]
            TC* vt = v_pages + head_base + pos % page_size;
            for (int d = lane; d < head_dim; d += RI_WAVE) from_f32(vt + (size_t)d * page_size, to_f32(x[d]));
            return;
        }
        dst = k_pages + head_base + (size_t)(pos % page_size) * head_dim;
    }

    // lane owns pairs i = lane, lane + 64, ...: elements (i, i + half)
    float x1[QK_MAX_PAIRS], x2[QK_MAX_PAIRS];
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < QK_MAX_PAIRS; ++j) {
        const int i = lane + j * RI_WAVE;
        x1[j] = x2[j] = 0.f;
        if (i < half) {
            x1[j] = to_f32(x[i]);
            x2[j] = to_f32(x[i + half]);
            ss += x1[j] * x1[j] + x2[j] * x2[j];
        }
    }
    const float* gain = hh < heads ? q_gain : k_gain;
    float inv = 1.0f;
    if (gain) inv = 1.0f / sqrtf(wave_sum(ss) / (float)head_dim + eps);
#pragma unroll
    for (int j = 0; j < QK_MAX_PAIRS; ++j) {
        const int i = lane + j * RI_WAVE;
        if (i >= half) continue;
        float a = x1[j], b = x2[j];
        if (gain) { a = a * inv * gain[i]; b = b * inv * gain[i + half]; }
        // pairs (i, i + half); angle = f32(pos) * inv_freq[i] as a float32 product
        // (the reference: src/ops/rope.rs:39, :73-74)
        if (inv_freq) {
            float sn, cs;
            sincosf((float)pos * inv_freq[i], &sn, &cs);
            const float ra = a * cs - b * sn, rb = b * cs + a * sn;
            a = ra; b = rb;
        }
        if (dst) { from_f32(dst + i, a); from_f32(dst + i + half, b); }
        else     { from_f32(x + i, a);   from_f32(x + i + half, b); }
    }
}

template <typename TA, typename TC>
static void launch_qk(void* qkv, const float* q_gain, const float* k_gain, float eps, const float* inv_freq,
                      int rot_dim, const int32_t* tok_pos, const int32_t* tok_seq, const int32_t* page_table,
                      int table_width, void* k_pages, void* v_pages, int tokens, int heads, int kv_heads,
                      int head_dim, int page_size, hipStream_t s) {
    const long items = (long)tokens * (heads + 2 * kv_heads);
    const int waves = 4;
    const unsigned grid = (unsigned)((items + waves - 1) / waves);
    qk_norm_rope_kv_write_kernel<TA, TC><<<grid, waves * RI_WAVE, 0, s>>>(
        (TA*)qkv, q_gain, k_gain, eps, inv_freq, tok_pos, tok_seq, page_table, table_width,
        (TC*)k_pages, (TC*)v_pages, tokens, heads, kv_heads, head_dim, page_size);
}

extern "C" int ri_qk_norm_rope_kv_write(void* qkv, int act_dtype, const float* q_gain, const float* k_gain, float eps,
                                        const float* inv_freq, int rot_dim, const int32_t* tok_pos,
                                        const int32_t* tok_seq, const int32_t* page_table, int table_width,
                                        void* k_pages, void* v_pages, int cache_dtype, int tokens, int heads,
                                        int kv_heads, int head_dim, int page_size, int num_pages, void* stream) {
    RI_REQUIRE(tokens > 0 && heads > 0 && kv_heads > 0, "qk_norm_rope_kv_write: tokens %d, heads %d, kv heads %d",
               tokens, heads, kv_heads);
    RI_REQUIRE(head_dim >= 2 && head_dim % 2 == 0 && head_dim <= 2 * RI_WAVE * QK_MAX_PAIRS,
               "qk_norm_rope_kv_write: head_dim %d must be even and at most %d", head_dim, 2 * RI_WAVE * QK_MAX_PAIRS);
    RI_REQUIRE(!inv_freq || rot_dim == head_dim,
               "qk_norm_rope_kv_write: rotation of %d of %d elements: only whole heads are rotated here", rot_dim,
               head_dim);
    RI_REQUIRE(page_size > 0 && table_width > 0 && num_pages > 0, "qk_norm_rope_kv_write: page geometry");
    RI_REQUIRE((long)tokens * (heads + 2 * kv_heads) / 4 < 2147483647L, "qk_norm_rope_kv_write: too many tokens");
    RI_REQUIRE(act_dtype == cache_dtype && (act_dtype == RI_F32 || act_dtype == RI_BF16),
               "qk_norm_rope_kv_write: activations (%d) and cache (%d) must share float32 or bfloat16", act_dtype,
               cache_dtype);
    hipStream_t s = (hipStream_t)stream;
    if (act_dtype == RI_F32)
        launch_qk<float, float>(qkv, q_gain, k_gain, eps, inv_freq, rot_dim, tok_pos, tok_seq, page_table,
                                table_width, k_pages, v_pages, tokens, heads, kv_heads, head_dim, page_size, s);
    else
        launch_qk<bf16_t, bf16_t>(qkv, q_gain, k_gain, eps, inv_freq, rot_dim, tok_pos, tok_seq, page_table,
                                  table_width, k_pages, v_pages, tokens, heads, kv_heads, head_dim, page_size, s);
    RI_LAUNCH_CHECK("qk_norm_rope_kv_write");
    return 0;
}
