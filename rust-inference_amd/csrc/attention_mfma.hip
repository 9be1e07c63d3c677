// Attention over the paged bfloat16 cache on the matrix cores (MFMA 16x16x32), for pages of 32 tokens.
//
// One wavefront works on up to 16 * NT "columns": a column is one (new token, query head) pair of
// one sequence and one kv head, so the query heads that share a kv head share every key and value
// it loads.  For one page of 32 keys and one tile of 16 columns:
//
//   S^T[key, col] = K[key, :] . Q[col, :]         2 MFMA tiles of 16 keys, head_dim / 32 steps each
//   online softmax per column in float32         running maximum m, running sum l (base-2 exponent)
//   O^T[d, col] += V^T[d, key] . P^T[key, col]    head_dim / 16 MFMA tiles, 32 keys deep
//
// Both products take their operands straight from global memory in the lane order MFMA wants:
// keys lie as [token][head_dim] and values transposed as [head_dim][token] inside a page.  The two
// key tiles take rows {0-3, 8-11, 16-19, 24-27} and {4-7, 12-15, 20-23, 28-31} of the page, so that
// after them lane group j (lanes 16 j .. 16 j + 15) holds the scores of keys 8 j .. 8 j + 7 of its
// column: exactly the B operand of the second product, with no exchange between lanes.
//
// The mask is positional: the query at position p sees keys lo..p, lo = 0 or p - window + 1
// (the reference: src/attention.rs:73, :117-118).  Scores are scaled after the dot product
// (src/attention.rs:28, :121-127); statistics and accumulators are float32; the weights enter the
// second product rounded to bfloat16 and the running sum is taken of the rounded weights, so they
// still sum to one.
//
// Prefill: one wavefront per tile of tokens, walking the sequence's pages in order.  Decode (one new
// token per sequence): the keys are cut into chunks of 256 at fixed places, one workgroup per chunk
// (its eight wavefronts take one page each), partial results go to a workspace and a second kernel
// joins them in chunk order.  Neither order depends on the batch or on how tokens were cut.
#include "api.h"
#include "common.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;

union Frag {
    bf16x8 v;
    uint4 u;
    uint32_t w[4];
};

#define PAGE 32
#define DECODE_CHUNK 256          // keys per workgroup of the decode kernel: 8 pages
#define DECODE_WAVES 8            // wavefronts of a decode workgroup: one page each

template <int DH>
struct PageFrags {
    Frag k[2][DH / 32];           // two tiles of 16 keys, head_dim / 32 steps
    Frag v[DH / 16];              // head_dim / 16 tiles of 16 channels, 32 keys deep
};

template <int DH>
__device__ __forceinline__ void load_page(PageFrags<DH>& f, const bf16_t* __restrict__ k_pages,
                                          const bf16_t* __restrict__ v_pages, long phys, int kv_heads, int kvh,
                                          int lane) {
    const int i = lane & 15, jg = lane >> 4;
    const bf16_t* kbase = k_pages + (phys * kv_heads + kvh) * (long)(PAGE * DH);
    const bf16_t* vbase = v_pages + (phys * kv_heads + kvh) * (long)(PAGE * DH);
#pragma unroll
    for (int kt = 0; kt < 2; ++kt) {
        const int row = (i >> 2) * 8 + kt * 4 + (i & 3);
#pragma unroll
        for (int ks = 0; ks < DH / 32; ++ks)
            f.k[kt][ks].u = *reinterpret_cast<const uint4*>(kbase + row * DH + ks * 32 + jg * 8);
    }
#pragma unroll
    for (int dt = 0; dt < DH / 16; ++dt)
        f.v[dt].u = *reinterpret_cast<const uint4*>(vbase + (dt * 16 + i) * PAGE + jg * 8);
}

// The state of NT tiles of 16 columns.  Lane l belongs to column l % 16 of every tile.
template <int DH, int NT>
struct Columns {
    Frag q[NT][DH / 32];
    floatx4 o[NT][DH / 16];
    float m[NT], l[NT];
    int qpos[NT], lo[NT];         // the column's query position (-1: no such column) and first visible key
};

template <int DH, int NT>
__device__ __forceinline__ void process_page(Columns<DH, NT>& c, const PageFrags<DH>& f, int page, int lane,
                                             float scale_log2) {
    const int jg = lane >> 4;
    const int key0 = page * PAGE + jg * 8;
#pragma unroll
    for (int j = 0; j < NT; ++j) {
        floatx4 s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < DH / 32; ++ks) {
            s0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f.k[0][ks].v, c.q[j][ks].v, s0, 0, 0, 0);
            s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f.k[1][ks].v, c.q[j][ks].v, s1, 0, 0, 0);
        }
        float s[8] = {s0[0], s0[1], s0[2], s0[3], s1[0], s1[1], s1[2], s1[3]};
        float mx = -INFINITY;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const int key = key0 + e;
            s[e] = (key <= c.qpos[j] && key >= c.lo[j]) ? s[e] * scale_log2 : -INFINITY;
            mx = fmaxf(mx, s[e]);
        }
        mx = fmaxf(mx, __shfl_xor(mx, 16, RI_WAVE));
        mx = fmaxf(mx, __shfl_xor(mx, 32, RI_WAVE));
        const float m_new = fmaxf(c.m[j], mx);
        const float m_safe = m_new == -INFINITY ? 0.f : m_new;     // a column that has seen no key yet
        const float corr = exp2f(c.m[j] - m_safe);                  // 0 while m is -inf
        Frag p;
        float ps = 0.f;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const bf16_t a = f32_to_bf16(exp2f(s[2 * e] - m_safe));
            const bf16_t b = f32_to_bf16(exp2f(s[2 * e + 1] - m_safe));
            p.w[e] = (uint32_t)a | ((uint32_t)b << 16);
            ps += bf16_to_f32(a) + bf16_to_f32(b);
        }
        ps += __shfl_xor(ps, 16, RI_WAVE);
        ps += __shfl_xor(ps, 32, RI_WAVE);
        c.l[j] = c.l[j] * corr + ps;
        c.m[j] = m_new;
#pragma unroll
        for (int dt = 0; dt < DH / 16; ++dt) {
            c.o[j][dt] *= corr;
            c.o[j][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f.v[dt].v, p.v, c.o[j][dt], 0, 0, 0);
        }
    }
}

template <int DH, int NT>
__device__ __forceinline__ void init_columns(Columns<DH, NT>& c) {
#pragma unroll
    for (int j = 0; j < NT; ++j) {
        c.m[j] = -INFINITY;
        c.l[j] = 0.f;
        c.qpos[j] = -1;
        c.lo[j] = 0;
#pragma unroll
        for (int ks = 0; ks < DH / 32; ++ks) c.q[j][ks].u = make_uint4(0, 0, 0, 0);
#pragma unroll
        for (int dt = 0; dt < DH / 16; ++dt) c.o[j][dt] = floatx4{0.f, 0.f, 0.f, 0.f};
    }
}

// ------------------------------------------------------------------ prefill
template <int DH, int NT>
__global__ void __launch_bounds__(256)
attn_prefill_mfma_kernel(bf16_t* __restrict__ out, const bf16_t* __restrict__ qkv, int q_stride,
                         const bf16_t* __restrict__ k_pages, const bf16_t* __restrict__ v_pages,
                         const int32_t* __restrict__ cu_seqlens, const int32_t* __restrict__ tok_pos,
                         const int32_t* __restrict__ page_table, int table_width, int heads, int kv_heads,
                         int window, float scale_log2) {
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int b = blockIdx.y, kvh = blockIdx.z;
    const int group = heads / kv_heads;
    const int tile_tokens = (16 * NT) / group;               // tokens per wavefront
    const int t_end = cu_seqlens[b + 1];
    const int t0 = cu_seqlens[b] + (blockIdx.x * 4 + wave) * tile_tokens;
    if (t0 >= t_end) return;                                 // the whole wavefront leaves; no barrier below
    const int nt = min(tile_tokens, t_end - t0);

    Columns<DH, NT> c;
    init_columns<DH, NT>(c);
    const int jg = lane >> 4;
#pragma unroll
    for (int j = 0; j < NT; ++j) {
        const int col = j * 16 + (lane & 15);
        const int tl = col / group, g = col - tl * group;
        if (tl < nt) {
            const int tok = t0 + tl;
            c.qpos[j] = tok_pos[tok];
            c.lo[j] = window > 0 ? max(0, c.qpos[j] - window + 1) : 0;
            const bf16_t* qp = qkv + (long)tok * q_stride + (kvh * group + g) * DH + jg * 8;
#pragma unroll
            for (int ks = 0; ks < DH / 32; ++ks) c.q[j][ks].u = *reinterpret_cast<const uint4*>(qp + ks * 32);
        }
    }
    const int first_pos = tok_pos[t0], last_pos = tok_pos[t0 + nt - 1];
    const int p_lo = window > 0 ? max(0, first_pos - window + 1) / PAGE : 0;
    const int p_hi = last_pos / PAGE;
    const int32_t* table = page_table + (long)b * table_width;

    PageFrags<DH> fa, fb;                                    // the page in work and the one being fetched
    load_page<DH>(fa, k_pages, v_pages, table[p_lo], kv_heads, kvh, lane);
    for (int p = p_lo; p <= p_hi; p += 2) {
        if (p + 1 <= p_hi) load_page<DH>(fb, k_pages, v_pages, table[p + 1], kv_heads, kvh, lane);
        process_page<DH, NT>(c, fa, p, lane, scale_log2);
        if (p + 1 > p_hi) break;
        if (p + 2 <= p_hi) load_page<DH>(fa, k_pages, v_pages, table[p + 2], kv_heads, kvh, lane);
        process_page<DH, NT>(c, fb, p + 1, lane, scale_log2);
    }

#pragma unroll
    for (int j = 0; j < NT; ++j) {
        const int col = j * 16 + (lane & 15);
        const int tl = col / group, g = col - tl * group;
        if (tl >= nt) continue;
        const float inv = 1.0f / c.l[j];
        bf16_t* op = out + ((long)(t0 + tl) * heads + kvh * group + g) * DH + jg * 4;
#pragma unroll
        for (int dt = 0; dt < DH / 16; ++dt) {
            uint2 w;
            w.x = (uint32_t)f32_to_bf16(c.o[j][dt][0] * inv) | ((uint32_t)f32_to_bf16(c.o[j][dt][1] * inv) << 16);
            w.y = (uint32_t)f32_to_bf16(c.o[j][dt][2] * inv) | ((uint32_t)f32_to_bf16(c.o[j][dt][3] * inv) << 16);
            *reinterpret_cast<uint2*>(op + dt * 16) = w;
        }
    }
}

// ------------------------------------------------------------------ decode: chunks of 256 keys, then a join
// Workspace: [seqs, heads, max_chunks, DH + 2] float32: the unnormalised output, then m and l.
template <int DH>
__global__ void __launch_bounds__(DECODE_WAVES * 64)
attn_decode_mfma_kernel(float* __restrict__ ws, const bf16_t* __restrict__ qkv, int q_stride,
                        const bf16_t* __restrict__ k_pages, const bf16_t* __restrict__ v_pages,
                        const int32_t* __restrict__ tok_pos, const int32_t* __restrict__ page_table, int table_width,
                        int heads, int kv_heads, int window, float scale_log2, int max_chunks) {
    __shared__ float o_lds[DECODE_WAVES][DH * 17];           // [d * 17 + col]: no bank conflicts either way
    __shared__ float ml_lds[DECODE_WAVES][2][16];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int chunk = blockIdx.x, b = blockIdx.y, kvh = blockIdx.z;
    const int group = heads / kv_heads;
    const int tok = b;                                       // one new token per sequence: token b is sequence b's
    const int qpos = tok_pos[tok];
    const int lo = window > 0 ? max(0, qpos - window + 1) : 0;
    if (chunk * DECODE_CHUNK > qpos || chunk * DECODE_CHUNK + DECODE_CHUNK - 1 < lo) return;   // whole workgroup

    const int page = chunk * (DECODE_CHUNK / PAGE) + wave;   // this wavefront's page
    const bool has = page * PAGE <= qpos && page * PAGE + PAGE - 1 >= lo;
    PageFrags<DH> f;
    if (has) load_page<DH>(f, k_pages, v_pages, page_table[(long)b * table_width + page], kv_heads, kvh, lane);

    Columns<DH, 1> c;
    init_columns<DH, 1>(c);
    const int jg = lane >> 4, col = lane & 15;
    if (col < group) {
        c.qpos[0] = qpos;
        c.lo[0] = lo;
        const bf16_t* qp = qkv + (long)tok * q_stride + (kvh * group + col) * DH + jg * 8;
#pragma unroll
        for (int ks = 0; ks < DH / 32; ++ks) c.q[0][ks].u = *reinterpret_cast<const uint4*>(qp + ks * 32);
    }
    if (has) process_page<DH, 1>(c, f, page, lane, scale_log2);

#pragma unroll
    for (int dt = 0; dt < DH / 16; ++dt)
#pragma unroll
        for (int r = 0; r < 4; ++r) o_lds[wave][(dt * 16 + jg * 4 + r) * 17 + col] = c.o[0][dt][r];
    if (jg == 0) {
        ml_lds[wave][0][col] = c.m[0];
        ml_lds[wave][1][col] = c.l[0];
    }
    __syncthreads();
    for (int idx = threadIdx.x; idx < group * DH; idx += DECODE_WAVES * 64) {
        const int g = idx / DH, d = idx - g * DH;
        float m = -INFINITY;
#pragma unroll
        for (int w = 0; w < DECODE_WAVES; ++w) m = fmaxf(m, ml_lds[w][0][g]);
        float acc = 0.f, l = 0.f;
#pragma unroll
        for (int w = 0; w < DECODE_WAVES; ++w) {
            const float mw = ml_lds[w][0][g];
            const float f2 = mw == -INFINITY ? 0.f : exp2f(mw - m);
            acc += o_lds[w][d * 17 + g] * f2;
            l += ml_lds[w][1][g] * f2;
        }
        float* dst = ws + (((long)b * heads + kvh * group + g) * max_chunks + chunk) * (DH + 2);
        dst[d] = acc;
        if (d == 0) {
            dst[DH] = m;
            dst[DH + 1] = l;
        }
    }
}

template <int DH>
__global__ void __launch_bounds__(DH)
attn_decode_join_kernel(bf16_t* __restrict__ out, const float* __restrict__ ws,
                        const int32_t* __restrict__ tok_pos, int heads, int window, int max_chunks) {
    const int b = blockIdx.x, h = blockIdx.y, d = threadIdx.x;
    const int tok = b;
    const int qpos = tok_pos[tok];
    const int lo = window > 0 ? max(0, qpos - window + 1) : 0;
    const int c_lo = lo / DECODE_CHUNK, c_hi = qpos / DECODE_CHUNK;
    const float* base = ws + ((long)b * heads + h) * max_chunks * (DH + 2);
    float m = -INFINITY;
    for (int c = c_lo; c <= c_hi; ++c) m = fmaxf(m, base[c * (DH + 2) + DH]);
    float acc = 0.f, l = 0.f;
    for (int c = c_lo; c <= c_hi; ++c) {
        const float mc = base[c * (DH + 2) + DH];
        const float f = mc == -INFINITY ? 0.f : exp2f(mc - m);
        acc += base[c * (DH + 2) + d] * f;
        l += base[c * (DH + 2) + DH + 1] * f;
    }
    out[((long)tok * heads + h) * DH + d] = f32_to_bf16(acc / l);
}

// ------------------------------------------------------------------ host side
static int check_common(const char* name, int heads, int kv_heads, int head_dim, int page_size, int q_stride,
                        int table_width) {
    RI_REQUIRE(heads > 0 && kv_heads > 0 && heads % kv_heads == 0, "%s: heads %d, kv heads %d", name, heads, kv_heads);
    RI_REQUIRE(head_dim == 32 || head_dim == 64 || head_dim == 128,
               "%s: head_dim %d (this kernel is built for 32, 64 and 128)", name, head_dim);
    RI_REQUIRE(page_size == PAGE, "%s: pages of %d tokens (this kernel takes %d)", name, page_size, PAGE);
    RI_REQUIRE(q_stride >= heads * head_dim && q_stride % 8 == 0, "%s: q row stride %d", name, q_stride);
    RI_REQUIRE(table_width > 0, "%s: page table width %d", name, table_width);
    RI_REQUIRE(kv_heads <= 65535, "%s: %d kv heads exceed one launch", name, kv_heads);
    return 0;
}

// column tiles per wavefront: 64 columns for head_dim up to 64, 32 for 128 (registers)
static int prefill_tiles(int head_dim) { return head_dim <= 64 ? 4 : 2; }

extern "C" int ri_attention_prefill_bf16(void* out, const void* qkv, int q_stride, const void* k_pages,
                                         const void* v_pages, const int32_t* cu_seqlens, const int32_t* tok_pos,
                                         const int32_t* page_table, int table_width, int seqs, int max_new,
                                         int heads, int kv_heads, int head_dim, int page_size, int window,
                                         float scale, void* stream) {
    if (check_common("attention_prefill_bf16", heads, kv_heads, head_dim, page_size, q_stride, table_width)) return 1;
    const int group = heads / kv_heads;
    const int nt_tiles = prefill_tiles(head_dim);
    RI_REQUIRE(group <= 16 * nt_tiles, "attention_prefill_bf16: %d query heads per kv head (at most %d)", group,
               16 * nt_tiles);
    RI_REQUIRE(seqs > 0 && seqs <= 65535 && max_new > 0, "attention_prefill_bf16: seqs %d, max_new %d", seqs, max_new);
    const int tile_tokens = (16 * nt_tiles) / group;
    dim3 grid((max_new + 4 * tile_tokens - 1) / (4 * tile_tokens), seqs, kv_heads);
    const float scale_log2 = scale * 1.4426950408889634f;
    hipStream_t s = (hipStream_t)stream;
#define RI_PREFILL_CASE(DH, NT)                                                                                  \
    case DH:                                                                                                     \
        attn_prefill_mfma_kernel<DH, NT><<<grid, 256, 0, s>>>(                                                   \
            (bf16_t*)out, (const bf16_t*)qkv, q_stride, (const bf16_t*)k_pages, (const bf16_t*)v_pages,          \
            cu_seqlens, tok_pos, page_table, table_width, heads, kv_heads, window, scale_log2);                  \
        break;
    switch (head_dim) {
        RI_PREFILL_CASE(32, 4)
        RI_PREFILL_CASE(64, 4)
        RI_PREFILL_CASE(128, 2)
    }
#undef RI_PREFILL_CASE
    RI_LAUNCH_CHECK("attention_prefill_bf16");
    return 0;
}

extern "C" int ri_attention_decode_chunks(int max_len) { return (max_len + DECODE_CHUNK - 1) / DECODE_CHUNK; }

extern "C" int ri_attention_decode_bf16(void* out, float* workspace, const void* qkv, int q_stride,
                                        const void* k_pages, const void* v_pages, const int32_t* cu_seqlens,
                                        const int32_t* tok_pos, const int32_t* page_table, int table_width, int seqs,
                                        int max_chunks, int heads, int kv_heads, int head_dim, int page_size,
                                        int window, float scale, void* stream) {
    if (check_common("attention_decode_bf16", heads, kv_heads, head_dim, page_size, q_stride, table_width)) return 1;
    const int group = heads / kv_heads;
    RI_REQUIRE(group <= 16, "attention_decode_bf16: %d query heads per kv head (at most 16)", group);
    RI_REQUIRE(seqs > 0 && seqs <= 65535 && max_chunks > 0 && heads <= 65535,
               "attention_decode_bf16: seqs %d, chunks %d, heads %d", seqs, max_chunks, heads);
    dim3 grid(max_chunks, seqs, kv_heads);
    const float scale_log2 = scale * 1.4426950408889634f;
    hipStream_t s = (hipStream_t)stream;
#define RI_DECODE_CASE(DH)                                                                                        \
    case DH:                                                                                                      \
        attn_decode_mfma_kernel<DH><<<grid, DECODE_WAVES * 64, 0, s>>>(                                           \
            workspace, (const bf16_t*)qkv, q_stride, (const bf16_t*)k_pages, (const bf16_t*)v_pages,             \
            tok_pos, page_table, table_width, heads, kv_heads, window, scale_log2, max_chunks);                   \
        attn_decode_join_kernel<DH><<<dim3(seqs, heads), DH, 0, s>>>((bf16_t*)out, workspace, tok_pos, heads,    \
                                                                      window, max_chunks);                        \
        break;
    switch (head_dim) {
        RI_DECODE_CASE(32)
        RI_DECODE_CASE(64)
        RI_DECODE_CASE(128)
    }
#undef RI_DECODE_CASE
    RI_LAUNCH_CHECK("attention_decode_bf16");
    return 0;
}
