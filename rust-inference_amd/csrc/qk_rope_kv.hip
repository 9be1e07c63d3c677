// Per-head q/k RMSNorm, rotate-half position encoding and the write of keys and values into
// their pages, in one pass over the fused qkv projection.  One wavefront per (token, head) in the
// general kernel; prompts of head sizes that allow it go through the 16-byte kernels further down.
//
// The reference does this in four launches and rounds to 16 bits after each
// (src/cuda/kernels.cu:98-108 norm, :127-142 rotation, :322-336 page write); here a q or k
// element is normed and rotated in float32 and rounded once.
#include "api.h"
#include "common.h"

#define QK_MAX_PAIRS 4   // pairs per lane: head_dim / 2 <= 64 * QK_MAX_PAIRS
#define QK_MAX_TAIL 8    // elements per lane behind the rotated part: head_dim <= 64 * QK_MAX_TAIL

template <typename TA, typename TC>
__global__ void qk_norm_rope_kv_write_kernel(
    TA* __restrict__ qkv, const float* __restrict__ q_gain, const float* __restrict__ k_gain, float eps,
    const float* __restrict__ inv_freq, int rot_dim, const int32_t* __restrict__ tok_pos,
    const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ page_table, int table_width,
    TC* __restrict__ k_pages, TC* __restrict__ v_pages, int tokens, int heads, int kv_heads, int head_dim,
    int page_size) {
    const int lane = threadIdx.x & (RI_WAVE - 1);
    const int waves_per_block = blockDim.x / RI_WAVE;
    const int all_heads = heads + 2 * kv_heads;
    const long item = (long)blockIdx.x * waves_per_block + threadIdx.x / RI_WAVE;
    if (item >= (long)tokens * all_heads) return;          // whole wavefront leaves together
    const int t = (int)(item / all_heads), hh = (int)(item % all_heads);
    // the first rot_dim elements of a head are rotated in pairs (i, i + rot_dim / 2); the rest, if any, is
    // normed only (a rotation over part of the head).  Without a rotation the pairing only shares out the work.
    const int half = rot_dim / 2;
    TA* x = qkv + (size_t)t * all_heads * head_dim + (size_t)hh * head_dim;

    const int pos = tok_pos[t];
    TC* dst = nullptr;          // where a k head goes
    if (hh >= heads && k_pages == nullptr) {
        if (hh >= heads + kv_heads) return;            // no pages given: k is changed in place like q, v is left alone
    } else if (hh >= heads) {
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

    // lane owns pairs i = lane, lane + 64, ...: elements (i, i + half), and of the elements behind the
    // rotated part every 64th
    float x1[QK_MAX_PAIRS], x2[QK_MAX_PAIRS], xt[QK_MAX_TAIL];
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
#pragma unroll
    for (int j = 0; j < QK_MAX_TAIL; ++j) {
        const int i = 2 * half + lane + j * RI_WAVE;
        xt[j] = 0.f;
        if (i < head_dim) {
            xt[j] = to_f32(x[i]);
            ss += xt[j] * xt[j];
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
#pragma unroll
    for (int j = 0; j < QK_MAX_TAIL; ++j) {
        const int i = 2 * half + lane + j * RI_WAVE;
        if (i >= head_dim) continue;
        const float a = gain ? xt[j] * inv * gain[i] : xt[j];
        if (dst) from_f32(dst + i, a);
        else     from_f32(x + i, a);
    }
}

// ------------------------------------------------------------------ the same in 16-byte pieces
// For head sizes whose half is 8 lanes' worth of eight elements or a power-of-two fraction of it
// (head_dim 16, 32, 64, 128, 256, 512 ...): a lane takes eight consecutive pairs (d, d + half) of one
// head, so head_dim / 16 lanes make a head and a wavefront works on 1024 / head_dim heads at once, every
// load and store 16 bytes (32 for float32).  Values are not written here but by the page-wise kernel
// below, which transposes whole pages through LDS instead of scattering single elements.
template <typename T> struct Vec8;
template <> struct Vec8<float> {
    __device__ static void load(const float* p, float* o) {
        const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
        o[0] = a.x; o[1] = a.y; o[2] = a.z; o[3] = a.w; o[4] = b.x; o[5] = b.y; o[6] = b.z; o[7] = b.w;
    }
    __device__ static void store(float* p, const float* v) {
        *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
        *reinterpret_cast<float4*>(p + 4) = make_float4(v[4], v[5], v[6], v[7]);
    }
};
template <> struct Vec8<bf16_t> {
    __device__ static void load(const bf16_t* p, float* o) {
        const uint4 v = *reinterpret_cast<const uint4*>(p);
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            o[2 * i] = __uint_as_float(w[i] << 16);
            o[2 * i + 1] = __uint_as_float(w[i] & 0xFFFF0000u);
        }
    }
    __device__ static void store(bf16_t* p, const float* v) {
        *reinterpret_cast<uint4*>(p) = make_uint4(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]),
                                                  pack_bf16x2(v[4], v[5]), pack_bf16x2(v[6], v[7]));
    }
};

template <typename TA, typename TC>
__global__ void __launch_bounds__(256)
qk_norm_rope_k_write_vec_kernel(
    TA* __restrict__ qkv, const float* __restrict__ q_gain, const float* __restrict__ k_gain, float eps,
    const float* __restrict__ inv_freq, const int32_t* __restrict__ tok_pos, const int32_t* __restrict__ tok_seq,
    const int32_t* __restrict__ page_table, int table_width, TC* __restrict__ k_pages, int heads, int kv_heads,
    int head_dim, int page_size) {
    extern __shared__ float cs_sn[];                         // cos[half] then sin[half] of this token
    const int lane = threadIdx.x & (RI_WAVE - 1), wave = threadIdx.x / RI_WAVE;
    const int t = blockIdx.x;
    const int half = head_dim / 2;
    const int lanes_per_head = half / 8;                     // a power of two, at most 64
    const int heads_at_once = RI_WAVE / lanes_per_head;
    const int pos = tok_pos[t];
    const int page = page_table[(size_t)tok_seq[t] * table_width + pos / page_size];
    if (inv_freq)
        for (int i = threadIdx.x; i < half; i += blockDim.x) sincosf((float)pos * inv_freq[i], &cs_sn[half + i], &cs_sn[i]);
    __syncthreads();
    const int qk_heads = heads + kv_heads;
    TA* row = qkv + (size_t)t * (heads + 2 * kv_heads) * head_dim;
    const int sub = lane / lanes_per_head, piece = lane % lanes_per_head;     // head within the group, 8 pairs of it
    for (int h0 = wave * heads_at_once; h0 < qk_heads; h0 += 4 * heads_at_once) {
        const int hh = h0 + sub;
        if (hh >= qk_heads) continue;                        // lanes of a head stay together: shuffles below are safe
        TA* x = row + (size_t)hh * head_dim + piece * 8;
        float a[8], b[8];
        Vec8<TA>::load(x, a);
        Vec8<TA>::load(x + half, b);
        const float* gain = hh < heads ? q_gain : k_gain;
        if (gain) {
            float ss = 0.f;
#pragma unroll
            for (int e = 0; e < 8; ++e) ss += a[e] * a[e] + b[e] * b[e];
            for (int m = lanes_per_head / 2; m > 0; m >>= 1) ss += __shfl_xor(ss, m, RI_WAVE);
            const float inv = 1.0f / sqrtf(ss / (float)head_dim + eps);
            float ga[8], gb[8];
            Vec8<float>::load(gain + piece * 8, ga);
            Vec8<float>::load(gain + half + piece * 8, gb);
#pragma unroll
            for (int e = 0; e < 8; ++e) { a[e] = a[e] * inv * ga[e]; b[e] = b[e] * inv * gb[e]; }
        }
        if (inv_freq) {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float cs = cs_sn[piece * 8 + e], sn = cs_sn[half + piece * 8 + e];
                const float ra = a[e] * cs - b[e] * sn, rb = b[e] * cs + a[e] * sn;
                a[e] = ra; b[e] = rb;
            }
        }
        if (hh < heads) {
            Vec8<TA>::store(x, a);
            Vec8<TA>::store(x + half, b);
        } else {
            TC* dst = k_pages + (((size_t)page * kv_heads + (hh - heads)) * page_size + pos % page_size) * head_dim
                      + piece * 8;
            Vec8<TC>::store(dst, a);
            Vec8<TC>::store(dst + half, b);
        }
    }
}

// Values into their pages, a page at a time: one workgroup per (page touched by this step, sequence,
// kv head) reads the page's new tokens as rows, turns them through LDS and writes channel rows.
#define VW_TOKENS 32      // tokens of a page handled at once (pages of other sizes are walked in such pieces)
template <typename TA, typename TC>
__global__ void __launch_bounds__(256)
v_write_pages_kernel(const TA* __restrict__ qkv, const int32_t* __restrict__ cu_seqlens,
                     const int32_t* __restrict__ tok_pos, const int32_t* __restrict__ page_table, int table_width,
                     TC* __restrict__ v_pages, int heads, int kv_heads, int head_dim, int page_size) {
    extern __shared__ float tile[];                          // [VW_TOKENS][head_dim + 1]
    const int b = blockIdx.y, kvh = blockIdx.z;
    const int t_begin = cu_seqlens[b], n = cu_seqlens[b + 1] - t_begin;
    const int start = tok_pos[t_begin];                      // the sequence's new tokens sit at start .. start + n - 1
    const int first = (start / VW_TOKENS + blockIdx.x) * VW_TOKENS;      // this workgroup's 32 positions
    const int lo = max(first, start), hi = min(first + VW_TOKENS - 1, start + n - 1);
    if (lo > hi) return;
    const int stride = head_dim + 1;
    const size_t v_off = (size_t)(heads + kv_heads + kvh) * head_dim;
    const size_t row_len = (size_t)(heads + 2 * kv_heads) * head_dim;
    if constexpr (sizeof(TA) == 2 && sizeof(TC) == 2) {
        // 32 new tokens of 16-bit values with a head of whole 16-byte pieces: 16 bytes a thread each way (a
        // prompt's full pages; the same bits as below, a third of the time)
        if (lo == first && hi == first + VW_TOKENS - 1 && head_dim % 8 == 0 && page_size % 8 == 0) {
            const int pieces = head_dim / 8;
            for (int e = threadIdx.x; e < VW_TOKENS * pieces; e += blockDim.x) {
                const int tt = e / pieces, d = (e - tt * pieces) * 8;
                const uint4 v = *reinterpret_cast<const uint4*>(qkv + (size_t)(t_begin + first - start + tt) * row_len + v_off + d);
                const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    tile[tt * stride + d + 2 * j] = __uint_as_float(w[j] << 16);
                    tile[tt * stride + d + 2 * j + 1] = __uint_as_float(w[j] & 0xFFFF0000u);
                }
            }
            __syncthreads();
            const int page = page_table[(size_t)b * table_width + first / page_size];
            TC* base = v_pages + ((size_t)page * kv_heads + kvh) * page_size * head_dim + first % page_size;
            for (int e = threadIdx.x; e < head_dim * (VW_TOKENS / 8); e += blockDim.x) {
                const int d = e / (VW_TOKENS / 8), t8 = (e - d * (VW_TOKENS / 8)) * 8;
                uint32_t w[4];
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    w[j] = (__float_as_uint(tile[(t8 + 2 * j) * stride + d]) >> 16) |
                           (__float_as_uint(tile[(t8 + 2 * j + 1) * stride + d]) & 0xFFFF0000u);
                *reinterpret_cast<uint4*>(base + (size_t)d * page_size + t8) = make_uint4(w[0], w[1], w[2], w[3]);
            }
            return;
        }
    }
    for (int e = threadIdx.x; e < (hi - lo + 1) * head_dim; e += blockDim.x) {
        const int tt = e / head_dim, d = e - tt * head_dim;
        tile[(lo - first + tt) * stride + d] = to_f32(qkv[(size_t)(t_begin + lo - start + tt) * row_len + v_off + d]);
    }
    __syncthreads();
    const int page = page_table[(size_t)b * table_width + first / page_size];
    TC* base = v_pages + ((size_t)page * kv_heads + kvh) * page_size * head_dim + first % page_size;
    for (int e = threadIdx.x; e < head_dim * VW_TOKENS; e += blockDim.x) {
        const int d = e / VW_TOKENS, tt = e - d * VW_TOKENS;
        if (first + tt >= lo && first + tt <= hi) from_f32(base + (size_t)d * page_size + tt, tile[tt * stride + d]);
    }
}

static bool vec_path_fits(int head_dim, int page_size) {
    const int half = head_dim / 2;
    if (half % 8) return false;
    const int lph = half / 8;
    // (the page-wise value writer holds 32 tokens of a head in LDS: 64 KB at most without asking for more)
    return lph <= 64 && (lph & (lph - 1)) == 0 && page_size % VW_TOKENS == 0 &&
           (size_t)VW_TOKENS * (head_dim + 1) * sizeof(float) <= 65536;
}

template <typename TA, typename TC>
static void launch_qk(void* qkv, const float* q_gain, const float* k_gain, float eps, const float* inv_freq,
                      int rot_dim, const int32_t* tok_pos, const int32_t* tok_seq, const int32_t* cu_seqlens,
                      int seqs, int max_new, const int32_t* page_table, int table_width, void* k_pages,
                      void* v_pages, int tokens, int heads, int kv_heads, int head_dim, int page_size,
                      hipStream_t s) {
    // one new token per sequence: a single launch that writes the few values element by element is cheaper
    // than two
    const bool whole = head_dim % 2 == 0 && (!inv_freq || rot_dim == head_dim);      // what the 16-byte kernels rotate
    if (cu_seqlens && max_new > 1 && whole && k_pages && vec_path_fits(head_dim, page_size)) {
        qk_norm_rope_k_write_vec_kernel<TA, TC><<<tokens, 256, head_dim * sizeof(float), s>>>(
            (TA*)qkv, q_gain, k_gain, eps, inv_freq, tok_pos, tok_seq, page_table, table_width, (TC*)k_pages, heads,
            kv_heads, head_dim, page_size);
        // a sequence's max_new tokens touch at most this many 32-token pieces
        dim3 grid((max_new + VW_TOKENS - 2) / VW_TOKENS + 1, seqs, kv_heads);
        v_write_pages_kernel<TA, TC><<<grid, 256, VW_TOKENS * (head_dim + 1) * sizeof(float), s>>>(
            (const TA*)qkv, cu_seqlens, tok_pos, page_table, table_width, (TC*)v_pages, heads, kv_heads, head_dim,
            page_size);
        return;
    }
    const long items = (long)tokens * (heads + 2 * kv_heads);
    const int waves = 4;
    qk_norm_rope_kv_write_kernel<TA, TC><<<(unsigned)((items + waves - 1) / waves), waves * RI_WAVE, 0, s>>>(
        (TA*)qkv, q_gain, k_gain, eps, inv_freq, inv_freq ? rot_dim : (head_dim & ~1), tok_pos, tok_seq, page_table,
        table_width, (TC*)k_pages, (TC*)v_pages, tokens, heads, kv_heads, head_dim, page_size);
}

extern "C" int ri_qk_norm_rope_kv_write(void* qkv, int act_dtype, const float* q_gain, const float* k_gain, float eps,
                                        const float* inv_freq, int rot_dim, const int32_t* tok_pos,
                                        const int32_t* tok_seq, const int32_t* cu_seqlens, int seqs, int max_new,
                                        const int32_t* page_table, int table_width,
                                        void* k_pages, void* v_pages, int cache_dtype, int tokens, int heads,
                                        int kv_heads, int head_dim, int page_size, int num_pages, void* stream) {
    RI_REQUIRE(tokens > 0 && heads > 0 && kv_heads > 0, "qk_norm_rope_kv_write: tokens %d, heads %d, kv heads %d",
               tokens, heads, kv_heads);
    RI_REQUIRE(head_dim >= 1 && head_dim <= 2 * RI_WAVE * QK_MAX_PAIRS,
               "qk_norm_rope_kv_write: head_dim %d must be between 1 and %d", head_dim, 2 * RI_WAVE * QK_MAX_PAIRS);
    RI_REQUIRE(!inv_freq || (rot_dim >= 2 && rot_dim % 2 == 0 && rot_dim <= head_dim),
               "qk_norm_rope_kv_write: a rotation of %d of %d elements: the rotated part is even and no longer than "
               "the head", rot_dim, head_dim);
    RI_REQUIRE((k_pages == nullptr) == (v_pages == nullptr), "qk_norm_rope_kv_write: key pages without value pages");
    RI_REQUIRE(k_pages == nullptr || (page_size > 0 && table_width > 0 && num_pages > 0),
               "qk_norm_rope_kv_write: page geometry");
    RI_REQUIRE((long)tokens * (heads + 2 * kv_heads) / 4 < 2147483647L, "qk_norm_rope_kv_write: too many tokens");
    RI_REQUIRE(!cu_seqlens || (seqs > 0 && seqs <= 65535 && max_new > 0 && kv_heads <= 65535),
               "qk_norm_rope_kv_write: seqs %d, max_new %d", seqs, max_new);
    RI_REQUIRE(act_dtype == cache_dtype && (act_dtype == RI_F32 || act_dtype == RI_BF16),
               "qk_norm_rope_kv_write: activations (%d) and cache (%d) must share float32 or bfloat16", act_dtype,
               cache_dtype);
    hipStream_t s = (hipStream_t)stream;
    if (act_dtype == RI_F32)
        launch_qk<float, float>(qkv, q_gain, k_gain, eps, inv_freq, rot_dim, tok_pos, tok_seq, cu_seqlens, seqs,
                                max_new, page_table, table_width, k_pages, v_pages, tokens, heads, kv_heads, head_dim,
                                page_size, s);
    else
        launch_qk<bf16_t, bf16_t>(qkv, q_gain, k_gain, eps, inv_freq, rot_dim, tok_pos, tok_seq, cu_seqlens, seqs,
                                  max_new, page_table, table_width, k_pages, v_pages, tokens, heads, kv_heads,
                                  head_dim, page_size, s);
    RI_LAUNCH_CHECK("qk_norm_rope_kv_write");
    return 0;
}
