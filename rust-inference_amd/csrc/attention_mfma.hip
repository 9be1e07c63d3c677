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
// second product rounded to bfloat16, the running sum is taken of them before the rounding.  (Letting
// the reference point of the exponents lag behind the running maximum, so that the accumulators are
// rescaled only rarely, was tried and changed no timing: the rescaling is not what the kernel waits for.)
//
// Prefill: one wavefront per tile of tokens, walking the sequence's pages in order; the four
// wavefronts of a workgroup share the pages through LDS.  The walk is one page ahead with the scores: the
// matrix cores take the next page's scores while the vector unit turns this page's into weights, and this
// page's value product while it finds the next page's maxima (3 to 6% over one page at a time at 2,048 to
// 32,768 tokens; the same bits).  Decode (one new
// token per sequence): the keys are cut into chunks of 256 at fixed places, one workgroup per chunk
// (its eight wavefronts take one page each), partial results go to a workspace and a second kernel
// joins them in chunk order.  Neither order depends on the batch or on how tokens were cut.
#include <type_traits>

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
#define DECODE_CHUNK 256          // keys per workgroup of the decode kernel: 8 pages; the unit of every count of chunks
#define DECODE_WAVES 8            // wavefronts of a decode workgroup: one page each
// (a step with few workgroups cuts every chunk into 2 or 4 pieces, workgroups of 4 or 2 wavefronts: CW below)

// The maximum over the four lanes of a column (lanes l, l ^ 16, l ^ 32, l ^ 48), in every one of them, by the
// two lane-swap instructions of gfx950: v_permlane32_swap exchanges the upper half of its first operand with
// the lower half of its second, v_permlane16_swap the odd rows of 16 lanes of the first with the even rows
// of the second; given the same value twice, the two results hold a lane's own value and its partner's.
// They stay in the vector unit, where a shuffle through LDS (ds_bpermute) costs a round trip that the softmax
// of a page waits for twice, but take three vector instructions a step where the shuffle takes one.  Timed
// on prompts of 1,024 to 2,048 tokens, the swaps win by 8-10% at head size 64 and by 4-8% with two tiles a
// wavefront at head size 128; with one tile at head size 128 (many wavefronts a SIMD, whose vector
// instructions are what is short) the shuffles win by 1-4%.  SWAP chooses.
template <bool SWAP>
__device__ __forceinline__ float column_max(float v) {
    if (!SWAP) {
        v = fmaxf(v, __shfl_xor(v, 16, RI_WAVE));
        return fmaxf(v, __shfl_xor(v, 32, RI_WAVE));
    }
    typedef unsigned __attribute__((ext_vector_type(2))) pair_t;
    {
        const unsigned u = __float_as_uint(v);
        const pair_t r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
        const unsigned a = r.x, b = r.y;
        v = fmaxf(__uint_as_float(a), __uint_as_float(b));
    }
    {
        const unsigned u = __float_as_uint(v);
        const pair_t r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
        const unsigned a = r.x, b = r.y;
        v = fmaxf(__uint_as_float(a), __uint_as_float(b));
    }
    return v;
}

template <int DH>
struct PageFrags {
    Frag k[2][DH / 32];           // two tiles of 16 keys, head_dim / 32 steps
    Frag v[DH / 16];              // head_dim / 16 tiles of 16 channels, 32 keys deep
};

// `wanted` false: the fragments will not be used (the decode kernels keep their loads out of branches and ask
// for a page even where a wavefront has none); every lane then reads the page's first 16 bytes, which costs
// the memory system one line instead of sixteen kilobytes.
template <int DH>
__device__ __forceinline__ void load_page(PageFrags<DH>& f, const bf16_t* __restrict__ k_pages,
                                          const bf16_t* __restrict__ v_pages, long phys, int kv_heads, int kvh,
                                          int lane, bool wanted = true) {
    const int w = wanted ? 1 : 0;
    const int i = (lane & 15) * w, jg = (lane >> 4) * w;
    const bf16_t* kbase = k_pages + (phys * kv_heads + kvh) * (long)(PAGE * DH);
    const bf16_t* vbase = v_pages + (phys * kv_heads + kvh) * (long)(PAGE * DH);
#pragma unroll
    for (int kt = 0; kt < 2; ++kt) {
        const int row = (i >> 2) * 8 + (kt * 4 + (i & 3)) * w;
#pragma unroll
        for (int ks = 0; ks < DH / 32; ++ks)
            f.k[kt][ks].u = load_stream16(kbase + row * DH + (ks * 32) * w + jg * 8);
    }
#pragma unroll
    for (int dt = 0; dt < DH / 16; ++dt)
        f.v[dt].u = load_stream16(vbase + ((dt * 16) * w + i) * PAGE + jg * 8);
}

// The state of NT tiles of 16 columns.  Lane l belongs to column l % 16 of every tile.
template <int DH, int NT>
struct Columns {
    Frag q[NT][DH / 32];
    floatx4 o[NT][DH / 16];
    float m[NT], l[NT];
    int qpos[NT], lo[NT];         // the column's query position (-1: no such column) and first visible key
};

// One page for NT tiles of columns, in two halves so that the key fragments and the value fragments
// need not be in registers at the same time.  `open` says that every key of the page is visible to
// every column of this wavefront (the usual case away from the diagonal and the window's edge): no
// mask then.  The running sum l stays per lane (the lane's own eight keys of every page) and is added
// up over the four lane groups once at the end; the running maximum is shared by a column's lanes at
// every page.
template <int DH, int NT>
__device__ __forceinline__ void scores_and_weights(Columns<DH, NT>& c, const Frag (&kf)[2][DH / 32], Frag (&p)[NT],
                                                   int page, int lane, float scale_log2, bool open) {
    const int jg = lane >> 4;
    const int key0 = page * PAGE + jg * 8;
#pragma unroll
    for (int j = 0; j < NT; ++j) {
        floatx4 s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < DH / 32; ++ks) {
            s0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[0][ks].v, c.q[j][ks].v, s0, 0, 0, 0);
            s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[1][ks].v, c.q[j][ks].v, s1, 0, 0, 0);
        }
        float s[8] = {s0[0], s0[1], s0[2], s0[3], s1[0], s1[1], s1[2], s1[3]};
        if (!open) {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const int key = key0 + e;
                if (key > c.qpos[j] || key < c.lo[j]) s[e] = -INFINITY;
            }
        }
        float mx = fmaxf(fmaxf(fmaxf(s[0], s[1]), fmaxf(s[2], s[3])), fmaxf(fmaxf(s[4], s[5]), fmaxf(s[6], s[7])));
        mx = column_max<(NT >= 2 || DH < 128)>(mx);
        const float m_new = fmaxf(c.m[j], mx * scale_log2);        // the scale is positive: max commutes with it
        const float m_safe = m_new == -INFINITY ? 0.f : m_new;     // a column that has seen no key yet
        float ps[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float a = __builtin_amdgcn_exp2f(fmaf(s[2 * e], scale_log2, -m_safe));
            const float b = __builtin_amdgcn_exp2f(fmaf(s[2 * e + 1], scale_log2, -m_safe));
            p[j].w[e] = pack_bf16x2(a, b);
            ps[e] = a + b;
        }
        if (__any(m_new != c.m[j])) {                               // a new maximum somewhere in the wavefront
            const float corr = __builtin_amdgcn_exp2f(c.m[j] - m_safe);      // 0 while m is -inf
            c.l[j] *= corr;
#pragma unroll
            for (int dt = 0; dt < DH / 16; ++dt) c.o[j][dt] *= corr;
            c.m[j] = m_new;
        }
        c.l[j] += (ps[0] + ps[1]) + (ps[2] + ps[3]);
    }
}

template <int DH, int NT>
__device__ __forceinline__ void weighted_values(Columns<DH, NT>& c, const Frag (&vf)[DH / 16], const Frag (&p)[NT]) {
#pragma unroll
    for (int j = 0; j < NT; ++j)
#pragma unroll
        for (int dt = 0; dt < DH / 16; ++dt)
            c.o[j][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[dt].v, p[j].v, c.o[j][dt], 0, 0, 0);
}

template <int DH, int NT>
__device__ __forceinline__ void process_page(Columns<DH, NT>& c, const PageFrags<DH>& f, int page, int lane,
                                             float scale_log2, bool open) {
    Frag p[NT];
    scores_and_weights<DH, NT>(c, f.k, p, page, lane, scale_log2, open);
    weighted_values<DH, NT>(c, f.v, p);
}

// The columns' sums over all their lanes: call once after the last page.
template <int DH, int NT>
__device__ __forceinline__ void finish_columns(Columns<DH, NT>& c) {
#pragma unroll
    for (int j = 0; j < NT; ++j) {
        c.l[j] += __shfl_xor(c.l[j], 16, RI_WAVE);
        c.l[j] += __shfl_xor(c.l[j], 32, RI_WAVE);
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

// The same work in four pieces, for a loop that takes the scores of the next page while it weighs this one
// (the prefill's): the results are those of scores_and_weights and weighted_values bit for bit.
template <int DH, int NT>
__device__ __forceinline__ void scores_of(const Columns<DH, NT>& c, const Frag (&kf)[2][DH / 32], float (&s)[NT][8]) {
#pragma unroll
    for (int j = 0; j < NT; ++j) {
        floatx4 s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < DH / 32; ++ks) {
            s0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[0][ks].v, c.q[j][ks].v, s0, 0, 0, 0);
            s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[1][ks].v, c.q[j][ks].v, s1, 0, 0, 0);
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            s[j][e] = s0[e];
            s[j][4 + e] = s1[e];
        }
    }
}

template <int DH, int NT>
__device__ __forceinline__ void mask_scores(const Columns<DH, NT>& c, float (&s)[NT][8], int page, int lane) {
    const int key0 = page * PAGE + (lane >> 4) * 8;
#pragma unroll
    for (int j = 0; j < NT; ++j)
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const int key = key0 + e;
            if (key > c.qpos[j] || key < c.lo[j]) s[j][e] = -INFINITY;
        }
}

// The columns' running maxima with a page's scores taken in (c.m itself stays as it is).
template <int DH, int NT>
__device__ __forceinline__ void maxima_with(const Columns<DH, NT>& c, const float (&s)[NT][8], float (&m_new)[NT],
                                            float scale_log2) {
#pragma unroll
    for (int j = 0; j < NT; ++j) {
        float mx = fmaxf(fmaxf(fmaxf(s[j][0], s[j][1]), fmaxf(s[j][2], s[j][3])),
                         fmaxf(fmaxf(s[j][4], s[j][5]), fmaxf(s[j][6], s[j][7])));
        mx = column_max<(NT >= 2 || DH < 128)>(mx);
        m_new[j] = fmaxf(c.m[j], mx * scale_log2);
    }
}

// Moves the reference point of the exponents to the new maxima (sums and accumulators are rescaled where a
// maximum rose anywhere in the wavefront) and returns in ref what the next weights subtract.
template <int DH, int NT>
__device__ __forceinline__ void move_reference(Columns<DH, NT>& c, const float (&m_new)[NT], float (&ref)[NT]) {
#pragma unroll
    for (int j = 0; j < NT; ++j) {
        ref[j] = m_new[j] == -INFINITY ? 0.f : m_new[j];           // a column that has seen no key yet
        if (__any(m_new[j] != c.m[j])) {
            const float corr = __builtin_amdgcn_exp2f(c.m[j] - ref[j]);      // 0 while m is -inf
            c.l[j] *= corr;
#pragma unroll
            for (int dt = 0; dt < DH / 16; ++dt) c.o[j][dt] *= corr;
            c.m[j] = m_new[j];
        }
    }
}

// A page's weights from its scores and the reference point that already holds its maximum.
template <int DH, int NT>
__device__ __forceinline__ void weights_of(Columns<DH, NT>& c, const float (&s)[NT][8], const float (&ref)[NT],
                                           Frag (&p)[NT], float scale_log2) {
#pragma unroll
    for (int j = 0; j < NT; ++j) {
        float ps[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float a = __builtin_amdgcn_exp2f(fmaf(s[j][2 * e], scale_log2, -ref[j]));
            const float b = __builtin_amdgcn_exp2f(fmaf(s[j][2 * e + 1], scale_log2, -ref[j]));
            p[j].w[e] = pack_bf16x2(a, b);
            ps[e] = a + b;
        }
        c.l[j] += (ps[0] + ps[1]) + (ps[2] + ps[3]);
    }
}

// ------------------------------------------------------------------ prefill
// A workgroup of four wavefronts takes 4 * (16 NT / group) consecutive tokens of one sequence and one kv
// head.  The pages of keys and values go through LDS, fetched once for all four wavefronts and
// double-buffered: while a page is in work the next one is on its way from global memory.  In LDS a key
// row is padded to head_dim + 16 elements and a value row (one channel, 32 tokens) to 48.  A fragment
// read takes 16 bytes per lane with lanes 0-15 on 16 consecutive rows; timed alone, such reads run at the
// full LDS rate (2.0 ns per wavefront read per CU) exactly when the row stride is 32 bytes modulo 64
// (96, 160, 288 here), at 3.4-3.5 ns for every other stride that is not a multiple of 128 (a pad of 8
// elements among them), and at 6.8 and 13.5 ns for multiples of 128 and 256.  The key rows of a page are
// stored in the order the two MFMA tiles take them (rows {0-3, 8-11, 16-19, 24-27}, then the rest).
template <int DH>
struct LdsPage {
    static constexpr int KS = DH + 16;                       // key row stride, elements
    static constexpr int VS = PAGE + 16;                     // value row stride, elements
    static constexpr int CHUNKS = 4 * DH;                    // 16-byte pieces of a key page (and of a value page)
    static constexpr int PER_THREAD = (CHUNKS + 255) / 256;
};

template <int DH>
__device__ __forceinline__ void stage_store_key(bf16_t* k_lds, int c, const uint4& k) {
    const int krow = c / (DH / 8), kcol = c % (DH / 8);                  // key row 0..31, 16-byte column
    const int w = krow & 7;
    const int lrow = (w >= 4 ? 16 : 0) + (krow >> 3) * 4 + (w & 3);
    *reinterpret_cast<uint4*>(k_lds + lrow * LdsPage<DH>::KS + kcol * 8) = k;
}

template <int DH>
__device__ __forceinline__ void stage_store_value(bf16_t* v_lds, int c, const uint4& v) {
    const int vrow = c / 4, vcol = c % 4;                                // channel 0..DH-1, 16-byte column
    *reinterpret_cast<uint4*>(v_lds + vrow * LdsPage<DH>::VS + vcol * 8) = v;
}

template <int DH>
__device__ __forceinline__ void key_frags_from_lds(Frag (&kf)[2][DH / 32], const bf16_t* k_lds, int lane) {
    const int i = lane & 15, jg = lane >> 4;
#pragma unroll
    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int ks = 0; ks < DH / 32; ++ks)
            kf[kt][ks].u = *reinterpret_cast<const uint4*>(k_lds + (kt * 16 + i) * LdsPage<DH>::KS + ks * 32 + jg * 8);
}

template <int DH>
__device__ __forceinline__ void value_frags_from_lds(Frag (&vf)[DH / 16], const bf16_t* v_lds, int lane) {
    const int i = lane & 15, jg = lane >> 4;
#pragma unroll
    for (int dt = 0; dt < DH / 16; ++dt)
        vf[dt].u = *reinterpret_cast<const uint4*>(v_lds + (dt * 16 + i) * LdsPage<DH>::VS + jg * 8);
}

template <int DH, int NT>
__global__ void __launch_bounds__(256, 2)
attn_prefill_mfma_kernel(bf16_t* __restrict__ out, const bf16_t* __restrict__ qkv, int q_stride,
                         const bf16_t* __restrict__ k_pages, const bf16_t* __restrict__ v_pages,
                         const int32_t* __restrict__ cu_seqlens, const int32_t* __restrict__ tok_pos,
                         const int32_t* __restrict__ page_table, int table_width, int heads, int kv_heads,
                         int window, float scale_log2) {
    __shared__ __attribute__((aligned(16))) bf16_t k_lds[2][PAGE * LdsPage<DH>::KS];
    __shared__ __attribute__((aligned(16))) bf16_t v_lds[2][DH * LdsPage<DH>::VS];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    // The kv head is the fastest grid index: consecutive workgroups go to consecutive XCDs, so the
    // workgroups that walk the same keys and values (one kv head of one sequence) meet in one XCD's L2.
    const int kvh = blockIdx.x, b = blockIdx.z;
    const int group = heads / kv_heads;
    const int tile_tokens = (16 * NT) / group;               // tokens per wavefront
    const int t_end = cu_seqlens[b + 1];
    // the last tokens of a sequence see the most keys: their workgroups are launched first
    const int t_wg = cu_seqlens[b] + (int)(gridDim.y - 1 - blockIdx.y) * 4 * tile_tokens;
    if (t_wg >= t_end) return;                               // the whole workgroup leaves
    const int t0 = t_wg + wave * tile_tokens;
    const int nt = max(0, min(tile_tokens, t_end - t0));     // a wavefront without tokens still helps to fetch

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
    // pages the workgroup walks (every wavefront takes them all)
    const int wg_first = tok_pos[t_wg], wg_last = tok_pos[min(t_end, t_wg + 4 * tile_tokens) - 1];
    const int p_lo = window > 0 ? max(0, wg_first - window + 1) / PAGE : 0;
    const int p_hi = wg_last / PAGE;
    // a page is open to the whole wavefront when its last key is at or before the first token's position
    // and its first key inside the last token's window; wavefronts with unused columns mask always
    const bool full = nt * group == 16 * NT;
    const int min_qpos = (nt > 0 && full) ? tok_pos[t0] : -1;
    const int max_lo = (nt > 0 && window > 0) ? max(0, tok_pos[t0 + nt - 1] - window + 1) : 0;
    const int32_t* table = page_table + (long)b * table_width;

    // What this thread carries of a page on its way from global memory to LDS: up to two 16-byte pieces
    // of the key page and of the value page, in plain registers.
    static_assert(LdsPage<DH>::PER_THREAD <= 2, "a page is at most two pieces per thread");
    constexpr bool TWO = LdsPage<DH>::PER_THREAD > 1;
    const int c0 = threadIdx.x;
    const bool has0 = c0 < LdsPage<DH>::CHUNKS;
    uint4 sk0 = make_uint4(0, 0, 0, 0), sk1 = sk0, sv0 = sk0, sv1 = sk0;
#define RI_STAGE_LOAD(PAGES, R0, R1, PHYS)                                                           \
    {                                                                                                \
        const long base_ = ((long)(PHYS) * kv_heads + kvh) * (long)(PAGE * DH);                      \
        if (has0) R0 = *reinterpret_cast<const uint4*>(PAGES + base_ + c0 * 8);                      \
        if (TWO) R1 = *reinterpret_cast<const uint4*>(PAGES + base_ + (c0 + 256) * 8);               \
    }
    // The loop is one page ahead with the scores: a turn takes the scores of page p + 1 while it turns the
    // scores of page p into weights (the matrix cores work on the one while the vector unit works on the
    // other), then the value product of page p while it finds the maxima of page p + 1.  Keys are staged
    // two pages ahead and values one; in turn i the keys read lie in buffer i % 2 and the values in the other,
    // and the pages that arrive are written to the buffers that are not read, so one barrier a turn is enough.
    // Every wavefront takes every page of the workgroup (those outside its own tokens' sight are masked
    // whole and add nothing), and the page numbers of the loads are clamped: no branch in a turn but the mask
    // and the move of the reference point, so that each half of a turn is one stretch of code to schedule.
#define RI_TURN_LOADS(P)                                                                             \
    RI_STAGE_LOAD(k_pages, sk0, sk1, table[min((P) + 2, p_hi)]);                                     \
    RI_STAGE_LOAD(v_pages, sv0, sv1, table[min((P) + 1, p_hi)]);
#define RI_TURN_STORES(I)                                                                            \
    {                                                                                                \
        if (has0) stage_store_key<DH>(k_lds[((I) & 1) ^ 1], c0, sk0);                                \
        if (TWO) stage_store_key<DH>(k_lds[((I) & 1) ^ 1], c0 + 256, sk1);                           \
        if (has0) stage_store_value<DH>(v_lds[(I) & 1], c0, sv0);                                    \
        if (TWO) stage_store_value<DH>(v_lds[(I) & 1], c0 + 256, sv1);                               \
        __syncthreads();                /* what arrived is in place; what was read may be overwritten */ \
    }
#define RI_PAGE_OPEN(Q) ((Q) * PAGE + PAGE - 1 <= min_qpos && (Q) * PAGE >= max_lo)
    RI_STAGE_LOAD(k_pages, sk0, sk1, table[p_lo]);
    {
        if (has0) stage_store_key<DH>(k_lds[0], c0, sk0);
        if (TWO) stage_store_key<DH>(k_lds[0], c0 + 256, sk1);
    }
    __syncthreads();
    float s_cur[NT][8], ref[NT], m_new[NT];
    {                                                        // turn 0: the first page's scores and maxima
        RI_TURN_LOADS(p_lo - 1);
        Frag kf[2][DH / 32];
        key_frags_from_lds<DH>(kf, k_lds[0], lane);
        scores_of<DH, NT>(c, kf, s_cur);
        if (!RI_PAGE_OPEN(p_lo)) mask_scores<DH, NT>(c, s_cur, p_lo, lane);
        maxima_with<DH, NT>(c, s_cur, m_new, scale_log2);
        move_reference<DH, NT>(c, m_new, ref);
        RI_TURN_STORES(0);
    }
    // A turn with the next page open to every column of the wavefront has no mask in it; pages are open in
    // one stretch (behind the window's edge, before the diagonal), so the turns come as three loops.
    auto turn = [&](int p, auto masked) {
        const int i = p - p_lo + 1;
        RI_TURN_LOADS(p);
        Frag w[NT];
        float s_next[NT][8];
        {
            Frag kf[2][DH / 32];
            key_frags_from_lds<DH>(kf, k_lds[i & 1], lane);
            scores_of<DH, NT>(c, kf, s_next);
            weights_of<DH, NT>(c, s_cur, ref, w, scale_log2);
        }
        if (decltype(masked)::value) mask_scores<DH, NT>(c, s_next, p + 1, lane);
        {
            Frag vf[DH / 16];
            value_frags_from_lds<DH>(vf, v_lds[(i & 1) ^ 1], lane);
            weighted_values<DH, NT>(c, vf, w);
            maxima_with<DH, NT>(c, s_next, m_new, scale_log2);
        }
        move_reference<DH, NT>(c, m_new, ref);
#pragma unroll
        for (int j = 0; j < NT; ++j)
#pragma unroll
            for (int e = 0; e < 8; ++e) s_cur[j][e] = s_next[j][e];
        RI_TURN_STORES(i);
    };
    int p = p_lo;
    for (; p < p_hi && !RI_PAGE_OPEN(p + 1); ++p) turn(p, std::true_type());
    for (; p < p_hi && RI_PAGE_OPEN(p + 1); ++p) turn(p, std::false_type());
    for (; p < p_hi; ++p) turn(p, std::true_type());
    {                                                        // the last page's weights and value product
        const int i = p_hi - p_lo + 1;
        Frag w[NT], vf[DH / 16];
        weights_of<DH, NT>(c, s_cur, ref, w, scale_log2);
        value_frags_from_lds<DH>(vf, v_lds[(i & 1) ^ 1], lane);
        weighted_values<DH, NT>(c, vf, w);
    }
#undef RI_TURN_LOADS
#undef RI_TURN_STORES
#undef RI_PAGE_OPEN
#undef RI_STAGE_LOAD
    finish_columns<DH, NT>(c);

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
// CW: wavefronts, and pages, of a workgroup; `chunk` counts pieces of CW pages, `max_chunks` such pieces.
template <int DH, int CW>
__global__ void __launch_bounds__(CW * 64)
attn_decode_mfma_kernel(float* __restrict__ ws, const bf16_t* __restrict__ qkv, int q_stride,
                        const bf16_t* __restrict__ k_pages, const bf16_t* __restrict__ v_pages,
                        const int32_t* __restrict__ tok_pos, const int32_t* __restrict__ page_table, int table_width,
                        int heads, int kv_heads, int window, float scale_log2, int max_chunks) {
    __shared__ float o_lds[CW][DH * 17];           // [d * 17 + col]: no bank conflicts either way
    __shared__ float ml_lds[CW][2][16];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int b = blockIdx.x, kvh = blockIdx.y, chunk = blockIdx.z;      // chunks last: the empty ones start last
    const int group = heads / kv_heads;
    const int tok = b;                                       // one new token per sequence: token b is sequence b's
    // The position and this wavefront's entry of the page table are asked for together: neither address
    // depends on the other's value, and each is a trip to memory that the page's loads would wait for in turn.
    const int page = chunk * CW + wave;   // this wavefront's page
    const int qpos = tok_pos[tok];
    const int phys = max(page_table[(long)b * table_width + min(page, table_width - 1)], 0);   // not mapped: page 0, unused
    const int lo = window > 0 ? max(0, qpos - window + 1) : 0;
    if (chunk * (CW * PAGE) > qpos || chunk * (CW * PAGE) + CW * PAGE - 1 < lo) return;   // whole workgroup

    // No load sits in a branch (the compiler counts loads in flight only along code without branches): a
    // wavefront without a page of its own fetches page `phys` all the same, a lane without a column the
    // group's last query, and neither is used.
    const bool has = page * PAGE <= qpos && page * PAGE + PAGE - 1 >= lo;
    Columns<DH, 1> c;
    init_columns<DH, 1>(c);
    const int jg = lane >> 4, col = lane & 15;
    {
        const bf16_t* qp = qkv + (long)tok * q_stride + (kvh * group + min(col, group - 1)) * DH + jg * 8;
#pragma unroll
        for (int ks = 0; ks < DH / 32; ++ks) c.q[0][ks].u = *reinterpret_cast<const uint4*>(qp + ks * 32);
    }
    PageFrags<DH> f;
    load_page<DH>(f, k_pages, v_pages, phys, kv_heads, kvh, lane, has);
    if (col < group) {
        c.qpos[0] = qpos;
        c.lo[0] = lo;
    } else {
#pragma unroll
        for (int ks = 0; ks < DH / 32; ++ks) c.q[0][ks].u = make_uint4(0, 0, 0, 0);
    }
    if (has) process_page<DH, 1>(c, f, page, lane, scale_log2, false);
    finish_columns<DH, 1>(c);

#pragma unroll
    for (int dt = 0; dt < DH / 16; ++dt)
#pragma unroll
        for (int r = 0; r < 4; ++r) o_lds[wave][(dt * 16 + jg * 4 + r) * 17 + col] = c.o[0][dt][r];
    if (jg == 0) {
        ml_lds[wave][0][col] = c.m[0];
        ml_lds[wave][1][col] = c.l[0];
    }
    __syncthreads();
    for (int idx = threadIdx.x; idx < group * DH; idx += CW * 64) {
        const int g = idx / DH, d = idx - g * DH;
        float m = -INFINITY;
#pragma unroll
        for (int w = 0; w < CW; ++w) m = fmaxf(m, ml_lds[w][0][g]);
        float acc = 0.f, l = 0.f;
#pragma unroll
        for (int w = 0; w < CW; ++w) {
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

// The join reads only the chunks that hold visible keys (it takes the position for that: reading every
// chunk's marker instead was tried and was slower).  Also tried and not kept: two pages per wavefront
// (chunks of 512 keys: 26 us against 24 us for both kernels at 8 sequences of 2,090 keys), and spare
// workgroups of the join reading the next product's weights ahead into the memory-side cache (that
// product got 2 us faster, the join 3 us slower).
// A sequence of up to JOIN_SERIAL chunks is joined by one pass in chunk order.  A longer one is cut into
// JOIN_PARTS runs of consecutive chunks of equal length (the last may be shorter); every run is joined in
// chunk order by itself and the runs then in run order.  The cut depends on the sequence's own number
// of chunks and on nothing else: PB, the runs a workgroup works on side by side, only says which
// threads do the work.  (One thread per channel walking 128 chunks, 32,768 keys, took 60 us, twice as
// long as the attention kernel before it.)
#define JOIN_SERIAL 16
#define JOIN_PARTS 8

// G chunks of a run from `cb` on, all their loads asked for before any is used: the largest maximum, and the
// chunks' results added in chunk order with the run's maximum `m`.
template <int DH, int G>
__device__ __forceinline__ void join_max(const float* __restrict__ base, int cb, int c1, float& m) {
    float mc[G];
#pragma unroll
    for (int i = 0; i < G; ++i) mc[i] = base[min(cb + i, c1) * (DH + 2) + DH];
#pragma unroll
    for (int i = 0; i < G; ++i)
        if (cb + i <= c1) m = fmaxf(m, mc[i]);
}

template <int DH, int G>
__device__ __forceinline__ void join_sum(const float* __restrict__ base, int cb, int c1, int d, float m, float& acc,
                                         float& l) {
    float o[G], mc[G], lc[G];
#pragma unroll
    for (int i = 0; i < G; ++i) {
        const float* at = base + min(cb + i, c1) * (DH + 2);
        o[i] = at[d];
        mc[i] = at[DH];
        lc[i] = at[DH + 1];
    }
#pragma unroll
    for (int i = 0; i < G; ++i) {
        if (cb + i <= c1) {
            const float f = mc[i] == -INFINITY ? 0.f : exp2f(mc[i] - m);
            acc += o[i] * f;
            l += lc[i] * f;
        }
    }
}

template <int DH, int PB>
__global__ void __launch_bounds__(DH * PB)
attn_decode_join_kernel(bf16_t* __restrict__ out, const float* __restrict__ ws, const int32_t* __restrict__ tok_pos,
                        int heads, int window, int max_chunks, int chunk_keys, int tiled) {
    __shared__ float part_o[JOIN_PARTS][DH];
    __shared__ float part_ml[JOIN_PARTS][2];
    const int b = blockIdx.x, h = blockIdx.y;                       // token b is sequence b's one new token
    const int d = threadIdx.x % DH, tp = threadIdx.x / DH;
    const int qpos = tok_pos[b];
    const int lo = window > 0 ? max(0, qpos - window + 1) : 0;
    // window < 0: the entries are the runs of the streaming kernel, all of them written
    const int c_lo = window < 0 ? 0 : lo / chunk_keys, c_hi = window < 0 ? max_chunks - 1 : qpos / chunk_keys;
    const int n = c_hi - c_lo + 1;
    const int parts = n <= JOIN_SERIAL ? 1 : JOIN_PARTS;
    const int per = (n + parts - 1) / parts;
    const float* base = ws + ((long)b * heads + h) * max_chunks * (DH + 2);
    for (int p = tp; p < parts; p += PB) {
        const int c0 = c_lo + p * per, c1 = min(c_hi, c0 + per - 1);
        // Sixteen chunks' loads are asked for at once while the run has sixteen more, then four at a time, each
        // from an address pulled back into the run, and what lies past the run's end is left out where it would
        // be used: a loop that fetches a chunk and then uses it makes a trip to memory for every chunk.  The
        // sums are the same operations in the same order as such a loop's.
        float m = -INFINITY;
        int cb = c0;
        for (; cb + JOIN_SERIAL - 1 <= c1; cb += JOIN_SERIAL) join_max<DH, JOIN_SERIAL>(base, cb, c1, m);
        for (; cb <= c1; cb += 4) join_max<DH, 4>(base, cb, c1, m);
        float acc = 0.f, l = 0.f;
        cb = c0;                                                    // always in chunk order
        for (; cb + JOIN_SERIAL - 1 <= c1; cb += JOIN_SERIAL) join_sum<DH, JOIN_SERIAL>(base, cb, c1, d, m, acc, l);
        for (; cb <= c1; cb += 4) join_sum<DH, 4>(base, cb, c1, d, m, acc, l);
        if (parts == 1) {                                           // the whole workgroup is here or nowhere
            out[tiled ? tiled_at(b, h * DH + d, heads * DH / 32) : ((size_t)b * heads + h) * DH + d] = f32_to_bf16(acc / l);
            return;
        }
        part_o[p][d] = acc;
        if (d == 0) {
            part_ml[p][0] = m;
            part_ml[p][1] = l;
        }
    }
    if (parts == 1) return;
    __syncthreads();
    if (tp != 0) return;
    float m = -INFINITY;
    for (int p = 0; p < parts; ++p) m = fmaxf(m, part_ml[p][0]);
    float acc = 0.f, l = 0.f;
    for (int p = 0; p < parts; ++p) {                               // always in run order
        const float mp = part_ml[p][0];
        const float f = mp == -INFINITY ? 0.f : exp2f(mp - m);
        acc += part_o[p][d] * f;
        l += part_ml[p][1] * f;
    }
    out[tiled ? tiled_at(b, h * DH + d, heads * DH / 32) : ((size_t)b * heads + h) * DH + d] = f32_to_bf16(acc / l);
}

// The join of up to CAP chunks (JOIN_SERIAL) with every load asked for at once, before the position is known:
// the chunks' results and markers lie at places that depend on the grid alone, so one trip to memory
// fetches them all (those of chunks the sequence has not reached are fetched and not used), where the
// loop above makes three trips in turn (the position, the maxima, the results).  The same operations in
// the same order as that loop: the results are equal bit for bit.
template <int DH, int CAP>
__global__ void __launch_bounds__(DH)
attn_decode_join_small_kernel(bf16_t* __restrict__ out, const float* __restrict__ ws, const int32_t* __restrict__ tok_pos,
                              int heads, int window, int max_chunks, int chunk_keys, int tiled) {
    const int b = blockIdx.x, h = blockIdx.y, d = threadIdx.x;
    const float* base = ws + ((long)b * heads + h) * max_chunks * (DH + 2);
    float o[CAP], mc[CAP], lc[CAP];
#pragma unroll
    for (int c = 0; c < CAP; ++c) {
        o[c] = 0.f;
        mc[c] = -INFINITY;
        lc[c] = 0.f;
        if (c < max_chunks) {
            o[c] = base[c * (DH + 2) + d];
            mc[c] = base[c * (DH + 2) + DH];
            lc[c] = base[c * (DH + 2) + DH + 1];
        }
    }
    const int qpos = tok_pos[b];
    const int lo = window > 0 ? max(0, qpos - window + 1) : 0;
    // window < 0: the entries are not chunks at fixed places but the runs of the streaming kernel, all of
    // them written (an empty run as a maximum of -inf)
    const int c_lo = window < 0 ? 0 : lo / chunk_keys, c_hi = window < 0 ? max_chunks - 1 : qpos / chunk_keys;
    float m = -INFINITY;
#pragma unroll
    for (int c = 0; c < CAP; ++c)
        if (c >= c_lo && c <= c_hi) m = fmaxf(m, mc[c]);
    float acc = 0.f, l = 0.f;
#pragma unroll
    for (int c = 0; c < CAP; ++c) {                          // always in chunk order
        if (c >= c_lo && c <= c_hi) {
            const float f = mc[c] == -INFINITY ? 0.f : exp2f(mc[c] - m);
            acc += o[c] * f;
            l += lc[c] * f;
        }
    }
    out[tiled ? tiled_at(b, h * DH + d, heads * DH / 32) : ((size_t)b * heads + h) * DH + d] = f32_to_bf16(acc / l);
}

template <int DH>
static void launch_join(bf16_t* out, const float* ws, const int32_t* tok_pos, int seqs, int heads, int window,
                        int max_chunks, int tiled, hipStream_t s, int chunk_keys = DECODE_CHUNK) {
    if (max_chunks <= JOIN_SERIAL)
        attn_decode_join_small_kernel<DH, JOIN_SERIAL><<<dim3(seqs, heads), DH, 0, s>>>(out, ws, tok_pos, heads, window,
                                                                                     max_chunks, chunk_keys, tiled);
    else
        attn_decode_join_kernel<DH, JOIN_PARTS><<<dim3(seqs, heads), DH * JOIN_PARTS, 0, s>>>(out, ws, tok_pos, heads,
                                                                                           window, max_chunks, chunk_keys, tiled);
}

// ------------------------------------------------------------------ decode: the new token's own q, k and v
// One head of the raw projection: per-head RMSNorm (when there is a gain), rotation (when there are
// frequencies), rounded to bfloat16 into LDS.  The loads are apart from the arithmetic, so that a kernel can ask
// for them before it asks for its pages and take the norm while the pages are on their way: every load is
// issued by every lane from an address inside the row, none inside a branch (the compiler counts loads in
// flight only along code without branches; anything else makes it wait for all of them).
__device__ float ri_zero_row[256];                           // what an absent gain or frequency table is read from

template <int DH>
struct HeadLoads {
    float x1, x2, g1, g2, f;                                 // the pair (d, d + DH/2), its gains, its frequency
};

template <int DH>
__device__ __forceinline__ HeadLoads<DH> fetch_head(const bf16_t* __restrict__ x, const float* __restrict__ gain,
                                                    const float* __restrict__ inv_freq, int lane) {
    static_assert(DH <= 128 && (DH & (DH - 1)) == 0, "one (d, d + DH/2) pair per lane");
    constexpr int HALF = DH / 2;
    const int d = lane & (HALF - 1);                         // lanes beyond HALF repeat the first ones' loads
    const float* gp = gain ? gain : ri_zero_row;
    const float* fp = inv_freq ? inv_freq : ri_zero_row;
    HeadLoads<DH> h;
    h.x1 = bf16_to_f32(x[d]);
    h.x2 = bf16_to_f32(x[d + HALF]);
    h.g1 = gp[d];
    h.g2 = gp[d + HALF];
    h.f = fp[d];
    return h;
}

template <int DH>
__device__ __forceinline__ void finish_head(bf16_t* dst_lds, const HeadLoads<DH>& h, bool normed, bool rotated,
                                            float eps, int pos, int lane) {
    constexpr int HALF = DH / 2;
    const bool mine = lane < HALF;
    float x1 = h.x1, x2 = h.x2;
    if (normed) {
        const float inv = 1.0f / sqrtf(wave_sum(mine ? x1 * x1 + x2 * x2 : 0.f) / (float)DH + eps);
        x1 = x1 * inv * h.g1;
        x2 = x2 * inv * h.g2;
    }
    if (rotated) {
        float sn, cs;
        sincosf((float)pos * h.f, &sn, &cs);
        const float a = x1 * cs - x2 * sn, b = x2 * cs + x1 * sn;
        x1 = a;
        x2 = b;
    }
    if (mine) {
        dst_lds[lane] = f32_to_bf16(x1);
        dst_lds[lane + HALF] = f32_to_bf16(x2);
    }
}

// ------------------------------------------------------------------ decode, streaming
// When the step has keys enough to fill the machine without cutting every sequence into chunks of 256 (many
// sequences, or very long ones), a workgroup walks a whole run of a sequence's pages instead: its four
// wavefronts take every fourth page, each with the next page's loads in flight while it works on the one it
// has, and keep their running maximum, sum and output across pages as the prefill kernel does.  The memory
// system then sees one long stream per wavefront rather than a burst per workgroup with a start and an end
// around it.  A sequence is cut into `splits` runs of whole chunks by its own length alone; with one run the
// kernel writes the output itself and no join follows, with more the runs' results go to the workspace
// [seqs, heads, splits, DH + 2] and the join adds them in run order (more than 16 of them in eight groups
// side by side, as it does with chunks).
// W wavefronts a workgroup: four, two workgroups a compute unit, where the step has workgroups enough; eight in
// one workgroup a compute unit for steps that have one run for every compute unit and few more (a wavefront's
// walk is then half as long, and there is no join).

// FUSED: qkv is the raw projection; the kernel norms and rotates the group's queries for itself, and the
// workgroup whose run ends at the new token's position makes the new key and value and stores them into their
// page before any page is read.
template <int DH, bool FUSED, int W>
__global__ void __launch_bounds__(W * 64, W == 4 ? 2 : 1)
attn_decode_stream_kernel(bf16_t* __restrict__ out, float* __restrict__ ws, const bf16_t* __restrict__ qkv, int q_stride,
                          const float* __restrict__ q_gain, const float* __restrict__ k_gain, float eps,
                          const float* __restrict__ inv_freq, bf16_t* k_pages, bf16_t* v_pages,
                          const int32_t* __restrict__ tok_pos, const int32_t* __restrict__ page_table, int table_width,
                          int heads, int kv_heads, int window, float scale_log2, int splits, int tiled) {
    static_assert(!FUSED || DH <= 128, "one (d, d + DH/2) pair per lane");
    __shared__ float o_lds[W][DH * 17];
    __shared__ float ml_lds[W][2][16];
    __shared__ __attribute__((aligned(16))) bf16_t q_lds[FUSED ? 16 : 1][DH];
    __shared__ __attribute__((aligned(16))) bf16_t knew[DH];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int b = blockIdx.x, kvh = blockIdx.y, split = blockIdx.z;
    const int group = heads / kv_heads;
    const int qpos = tok_pos[b];                             // token b is sequence b's one new token
    const int lo = window > 0 ? max(0, qpos - window + 1) : 0;
    const int c_lo = lo / DECODE_CHUNK, c_hi = qpos / DECODE_CHUNK;
    const int per = (c_hi - c_lo + splits) / splits;         // chunks per run: by the sequence's own length
    const int c0 = c_lo + split * per, c1 = min(c_hi, c0 + per - 1);
    const int p_first = max(c0 * (DECODE_CHUNK / PAGE), lo / PAGE);
    const int p_last = min(c1 * (DECODE_CHUNK / PAGE) + DECODE_CHUNK / PAGE - 1, qpos / PAGE);   // below p_first: an empty run
    const int32_t* table = page_table + (long)b * table_width;

    // This wavefront's pages are p_first + wave + W * j, j = 0 .. n_mine - 1, taken in blocks of
    // 64 * HELD: lane l of held[i] holds the table's entry for page j = block + 64 * i + l of the block, fetched
    // before the block begins, so that a page's address never waits for a trip to memory of its own.  No load
    // of the walk sits in a branch (the compiler counts loads in flight only along code without branches, and
    // otherwise waits for the page just asked for before it works on the one it has): an index past the end
    // is pulled back to the last page, an entry that is not mapped reads page 0, and neither is used.
    constexpr int HELD = 4;
    const int mine = p_first + wave;
    const int n_mine = mine <= p_last ? (p_last - mine) / W + 1 : 0;
    int held[HELD];
    auto fetch_table = [&](int j0) {
#pragma unroll
        for (int i = 0; i < HELD; ++i) {
            const int j = min(j0 + 64 * i + lane, max(n_mine - 1, 0));
            held[i] = max(table[min(mine + W * j, table_width - 1)], 0);
        }
    };
    auto phys_of = [&](int r) -> long {                      // r: the page's number inside the block
        int v = __builtin_amdgcn_readlane(held[0], r & 63);
#pragma unroll
        for (int i = 1; i < HELD; ++i) {
            const int w = __builtin_amdgcn_readlane(held[i], r & 63);
            v = (r >> 6) == i ? w : v;
        }
        return (long)v;
    };
    auto open_page = [&](int pg) -> bool { return pg * PAGE + PAGE - 1 <= qpos && pg * PAGE >= lo; };
    // The group's queries and, where the run ends at the new token, its key and value.  These go into their
    // page before the workgroup reads any page: the barrier makes them visible to the wavefront that will
    // read that page, the last of the run, so nothing has to be patched into fragments afterwards.
    Columns<DH, 1> c;
    init_columns<DH, 1>(c);
    const int jg = lane >> 4, col = lane & 15;
    fetch_table(0);
    if (FUSED) {
        const bf16_t* row = qkv + (long)b * q_stride;
        const int page_new = qpos / PAGE;
        HeadLoads<DH> hq[16 / W];                            // up to 16 query heads a kv head: 16 / W a wavefront
#pragma unroll
        for (int i = 0; i < 16 / W; ++i)
            hq[i] = fetch_head<DH>(row + (kvh * group + min(wave + W * i, group - 1)) * DH, q_gain, inv_freq, lane);
        const HeadLoads<DH> hk = fetch_head<DH>(row + (heads + kvh) * DH, k_gain, inv_freq, lane);
        const bf16_t* v_row = row + (heads + kv_heads + kvh) * DH;
        const bf16_t v0 = v_row[lane & (DH - 1)], v1 = v_row[(lane + 64) & (DH - 1)];
#pragma unroll
        for (int i = 0; i < 16 / W; ++i)
            if (wave + W * i < group)
                finish_head<DH>(q_lds[wave + W * i], hq[i], q_gain != nullptr, inv_freq != nullptr, eps, qpos, lane);
        if (p_first <= p_last && p_last == page_new) {       // this run holds the new token's position
            const int slot = qpos % PAGE;
            const long head_base = ((long)table[page_new] * kv_heads + kvh) * (long)(PAGE * DH);
            if (wave == W - 1) {                  // the key: norm, rotation, into its page
                finish_head<DH>(knew, hk, k_gain != nullptr, inv_freq != nullptr, eps, qpos, lane);
                __builtin_amdgcn_wave_barrier();
                for (int d = lane; d < DH; d += 64) k_pages[head_base + (long)slot * DH + d] = knew[d];
            } else if (wave == W - 2) {           // the value: a copy, transposed inside the page
                if (lane < DH) v_pages[head_base + (long)lane * PAGE + slot] = v0;
                if (lane + 64 < DH) v_pages[head_base + (long)(lane + 64) * PAGE + slot] = v1;
            }
        }
        __syncthreads();
#pragma unroll
        for (int ks = 0; ks < DH / 32; ++ks)
            c.q[0][ks].u = *reinterpret_cast<const uint4*>(&q_lds[min(col, group - 1)][ks * 32 + jg * 8]);
    } else {
        const bf16_t* qp = qkv + (long)b * q_stride + (kvh * group + min(col, group - 1)) * DH + jg * 8;
#pragma unroll
        for (int ks = 0; ks < DH / 32; ++ks) c.q[0][ks].u = *reinterpret_cast<const uint4*>(qp + ks * 32);
    }
    if (col < group) {
        c.qpos[0] = qpos;
        c.lo[0] = lo;
    } else {
#pragma unroll
        for (int ks = 0; ks < DH / 32; ++ks) c.q[0][ks].u = make_uint4(0, 0, 0, 0);
    }
    PageFrags<DH> fa, fb;
    for (int j0 = 0; j0 < n_mine; j0 += 64 * HELD) {
        if (j0 > 0) fetch_table(j0);
        const int n_blk = min(n_mine - j0, 64 * HELD);
        load_page<DH>(fa, k_pages, v_pages, phys_of(0), kv_heads, kvh, lane);
        for (int r = 0; r < n_blk; r += 2) {
            const int pa = mine + W * (j0 + r), pb = pa + W;
            load_page<DH>(fb, k_pages, v_pages, phys_of(min(r + 1, n_blk - 1)), kv_heads, kvh, lane, r + 1 < n_blk);
            process_page<DH, 1>(c, fa, pa, lane, scale_log2, open_page(pa));
            load_page<DH>(fa, k_pages, v_pages, phys_of(min(r + 2, n_blk - 1)), kv_heads, kvh, lane, r + 2 < n_blk);
            if (r + 1 < n_blk) process_page<DH, 1>(c, fb, pb, lane, scale_log2, open_page(pb));
        }
    }
    finish_columns<DH, 1>(c);

#pragma unroll
    for (int dt = 0; dt < DH / 16; ++dt)
#pragma unroll
        for (int r = 0; r < 4; ++r) o_lds[wave][(dt * 16 + jg * 4 + r) * 17 + col] = c.o[0][dt][r];
    if (jg == 0) {
        ml_lds[wave][0][col] = c.m[0];
        ml_lds[wave][1][col] = c.l[0];
    }
    __syncthreads();
    for (int idx = threadIdx.x; idx < group * DH; idx += W * 64) {
        const int g = idx / DH, d = idx - g * DH;
        float m = -INFINITY;
#pragma unroll
        for (int w = 0; w < W; ++w) m = fmaxf(m, ml_lds[w][0][g]);
        float acc = 0.f, l = 0.f;
#pragma unroll
        for (int w = 0; w < W; ++w) {              // always in wavefront order
            const float mw = ml_lds[w][0][g];
            const float f2 = mw == -INFINITY ? 0.f : exp2f(mw - m);
            acc += o_lds[w][d * 17 + g] * f2;
            l += ml_lds[w][1][g] * f2;
        }
        const int h = kvh * group + g;
        if (splits == 1) {                                   // the new token sees itself at least: l > 0
            out[tiled ? tiled_at(b, h * DH + d, heads * DH / 32) : ((size_t)b * heads + h) * DH + d] = f32_to_bf16(acc / l);
        } else {
            float* dst = ws + (((long)b * heads + h) * splits + split) * (DH + 2);
            dst[d] = acc;
            if (d == 0) {
                dst[DH] = m;
                dst[DH + 1] = l;
            }
        }
    }
}

// Runs per sequence of the streaming kernel for a step of `seqs` sequences of up to `max_chunks` chunks, or 0
// where the kernel of one workgroup per chunk is the faster one.  It depends on the step's size alone: one
// run where there are 512 (sequence, kv head) pairs or more; else, from 64 chunks (16,384 keys) on, as many
// runs as bring the workgroups to about a thousand, of eight chunks (64 pages, 16 a wavefront) at least, if
// that still makes 512 workgroups.
// Measured at 8 kv heads of 128: with 64 sequences of 2,080 keys one run per sequence (512 workgroups, no
// join) takes 94 us where the chunks and their join take 97 + 6; 8 sequences of 32,800 keys in 16 runs make
// the step 2% shorter, 4 of them 2%, one sequence of 131,000 keys in 64 runs 10%.  Fewer or shorter streams
// do not keep the memory busy (one sequence of 131,000 keys in 16 runs: 12% longer; runs of four chunks: no
// gain), and runs that need a join lose at a few thousand keys (2 runs at 48 sequences of 2,080 keys: -2.5%;
// 4 runs at 16 sequences of 4,100: -1.5%; 32 sequences of 4,100 gain 2.5% and are left to the chunks with them;
// one run a sequence at 16 sequences of 16 to 1,300 keys, 128 workgroups and no join: 7% of a small model's step
// longer than the chunks with their join).
// (The counts of workgroups above were measured on 256 compute units and are kept per compute unit: two of
// them for each to stream at all, four for each where runs are joined.)
// (One run a sequence from 1.8 workgroups a compute unit, 58 sequences of 8 kv heads, instead of two: a step of 58 and
// 62 sequences 0.5 to 2.4% shorter at Qwen3-8B sizes, 1.2% longer at 58 at Qwen3-0.6B sizes; from 1.6, 52 sequences, 0.6 to
// 2.5% longer: left at two.)
#define STREAM_WORKGROUPS_PER_CU 4
#define STREAM_MIN_PER_CU 2
#define STREAM_MIN_CHUNKS 8
#define STREAM_JOINED_FROM 64
// Eight wavefronts a workgroup and one run a sequence: where the step has a workgroup for four fifths of the compute
// units or more but for none a second one (a second round on a few units doubles the kernel's time, and with half the
// units idle the others pull no faster), for sequences of up to STREAM_WIDE_MAX_CHUNKS chunks.
#ifndef STREAM_WIDE_MAX_CHUNKS
#define STREAM_WIDE_MAX_CHUNKS 16
#endif
#ifndef STREAM_WIDE_BELOW
#define STREAM_WIDE_BELOW 5       // from this share of the compute units below their number
#define STREAM_WIDE_ABOVE 0       // to this share above it (0: to their number itself)
#endif
static bool stream_wide(int seqs, int kv_heads, int max_chunks) {
    const long rows = (long)seqs * kv_heads;
    const long cus = ri_compute_units();
    const long lo = cus - (STREAM_WIDE_BELOW ? cus / STREAM_WIDE_BELOW : 0), hi = cus + (STREAM_WIDE_ABOVE ? cus / STREAM_WIDE_ABOVE : 0);
    return rows >= lo && rows <= hi && rows < STREAM_MIN_PER_CU * cus && max_chunks <= STREAM_WIDE_MAX_CHUNKS;
}

static int stream_splits(int seqs, int kv_heads, int max_chunks) {
    const long rows = (long)seqs * kv_heads;
    const long cus = ri_compute_units();
    if (rows >= STREAM_MIN_PER_CU * cus || stream_wide(seqs, kv_heads, max_chunks)) return 1;
    if (max_chunks < STREAM_JOINED_FROM) return 0;
    const long splits = min((STREAM_WORKGROUPS_PER_CU * cus + rows - 1) / rows, (long)max_chunks / STREAM_MIN_CHUNKS);
    if (splits < 2 || rows * splits < STREAM_MIN_PER_CU * cus) return 0;
    return (int)splits;
}

extern "C" int ri_attention_decode_streams(int seqs, int kv_heads, int max_chunks) {
    return stream_splits(seqs, kv_heads, max_chunks);
}

// ------------------------------------------------------------------ decode, everything in one kernel
// The decode step's attention from the raw projection: per-head RMSNorm and rotation of the new token's q
// and k, the write of its k and v into their page, and the attention over chunks of 256 keys, in one
// kernel; the join of the chunks follows as a second one.  Every workgroup norms and rotates the group's
// queries for itself (a few hundred elements); the workgroup whose chunk holds the new token's position
// also makes the new key and value, stores them for later steps and patches them into the fragments it
// has just read from the page (the page in memory does not have them yet).  (Joining inside the same
// kernel, by the workgroup that finishes last, was tried: the device-wide fences it needs write the
// whole L2 back and cost many times what the second launch costs.)
template <int DH, int CW>
__global__ void __launch_bounds__(CW * 64)
attn_decode_fused_kernel(float* __restrict__ ws, const bf16_t* __restrict__ qkv, int q_stride, const float* __restrict__ q_gain,
                         const float* __restrict__ k_gain, float eps, const float* __restrict__ inv_freq,
                         bf16_t* __restrict__ k_pages, bf16_t* __restrict__ v_pages,
                         const int32_t* __restrict__ tok_pos, const int32_t* __restrict__ page_table, int table_width,
                         int heads, int kv_heads, int window, float scale_log2, int max_chunks) {
    static_assert(DH <= 128, "one (d, d + DH/2) pair per lane");
    __shared__ float o_lds[CW][DH * 17];
    __shared__ float ml_lds[CW][2][16];
    __shared__ __attribute__((aligned(16))) bf16_t q_lds[16][DH];
    __shared__ __attribute__((aligned(16))) bf16_t knew[DH];
    __shared__ __attribute__((aligned(16))) bf16_t vnew[DH];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int b = blockIdx.x, kvh = blockIdx.y, chunk = blockIdx.z;      // chunks last: the empty ones start last
    const int group = heads / kv_heads;
    // 1. What needs nothing but the workgroup's indices is asked for first: the heads this wavefront will norm
    // (two of the group's queries at most, and the new key), the new value, the position and this wavefront's
    // entry of the page table.  An entry that is not mapped reads page 0, which is never used then.
    const bf16_t* row = qkv + (long)b * q_stride;
    const int g0 = min(wave, group - 1), g1 = min(wave + CW, group - 1);
    const HeadLoads<DH> hq0 = fetch_head<DH>(row + (kvh * group + g0) * DH, q_gain, inv_freq, lane);
    const HeadLoads<DH> hq1 = fetch_head<DH>(row + (kvh * group + g1) * DH, q_gain, inv_freq, lane);
    const HeadLoads<DH> hk = fetch_head<DH>(row + (heads + kvh) * DH, k_gain, inv_freq, lane);
    const bf16_t* v_row = row + (heads + kv_heads + kvh) * DH;
    const bf16_t v0 = v_row[lane & (DH - 1)], v1 = v_row[(lane + 64) & (DH - 1)];
    const int page = chunk * CW + wave;
    const int qpos = tok_pos[b];                             // token b is sequence b's one new token
    const int phys = max(page_table[(long)b * table_width + min(page, table_width - 1)], 0);
    const int lo = window > 0 ? max(0, qpos - window + 1) : 0;
    if (chunk * (CW * PAGE) > qpos || chunk * (CW * PAGE) + CW * PAGE - 1 < lo) return;   // whole workgroup
    const bool owner = chunk == qpos / (CW * PAGE);         // this chunk holds the new token's position

    // 2. this wavefront's page is on its way while the queries are made (a wavefront without a page of its own
    // fetches page `phys` all the same and leaves it unused)
    const bool has = page * PAGE <= qpos && page * PAGE + PAGE - 1 >= lo;
    PageFrags<DH> f;
    load_page<DH>(f, k_pages, v_pages, phys, kv_heads, kvh, lane, has);
    const long phys_new = owner ? page_table[(long)b * table_width + qpos / PAGE] : 0;

    // 3. queries of the group; in the owner also the new key and value
    if (wave < group) finish_head<DH>(q_lds[wave], hq0, q_gain != nullptr, inv_freq != nullptr, eps, qpos, lane);
    if (wave + CW < group)
        finish_head<DH>(q_lds[wave + CW], hq1, q_gain != nullptr, inv_freq != nullptr, eps, qpos, lane);
    if (owner) {
        const int slot = qpos % PAGE;
        const long head_base = (phys_new * kv_heads + kvh) * (long)(PAGE * DH);
        if (wave == CW - 1) {                      // the key: norm, rotation, into LDS and into its page
            finish_head<DH>(knew, hk, k_gain != nullptr, inv_freq != nullptr, eps, qpos, lane);
            __builtin_amdgcn_wave_barrier();
            for (int d = lane; d < DH; d += 64) k_pages[head_base + (long)slot * DH + d] = knew[d];
        } else if (wave == CW - 2) {               // the value: a copy, transposed inside the page
            if (lane < DH) {
                vnew[lane] = v0;
                v_pages[head_base + (long)lane * PAGE + slot] = v0;
            }
            if (lane + 64 < DH) {
                vnew[lane + 64] = v1;
                v_pages[head_base + (long)(lane + 64) * PAGE + slot] = v1;
            }
        }
    }
    __syncthreads();

    // 4. this wavefront's page against the group's queries
    Columns<DH, 1> c;
    init_columns<DH, 1>(c);
    const int jg = lane >> 4, col = lane & 15;
    if (col < group) {
        c.qpos[0] = qpos;
        c.lo[0] = lo;
#pragma unroll
        for (int ks = 0; ks < DH / 32; ++ks)
            c.q[0][ks].u = *reinterpret_cast<const uint4*>(&q_lds[col][ks * 32 + jg * 8]);
    }
    if (has && page == qpos / PAGE) {                        // the new token's key and value are not in memory yet
        const int r = qpos % PAGE;
        const int i_new = (r >> 3) * 4 + (r & 3);            // the fragment row that holds key r
        if (col == i_new) {
#pragma unroll
            for (int ks = 0; ks < DH / 32; ++ks) {
                const uint4 kv = *reinterpret_cast<const uint4*>(&knew[ks * 32 + jg * 8]);
                if ((r & 7) >= 4) f.k[1][ks].u = kv; else f.k[0][ks].u = kv;
            }
        }
        if (jg == (r >> 3)) {                                // lanes whose eight keys include key r
            const int e = r & 7;
#pragma unroll
            for (int dt = 0; dt < DH / 16; ++dt) {
                const uint32_t v = vnew[dt * 16 + col];
                uint32_t w[4] = {f.v[dt].u.x, f.v[dt].u.y, f.v[dt].u.z, f.v[dt].u.w};
#pragma unroll
                for (int k = 0; k < 4; ++k)
                    if (k == (e >> 1)) w[k] = (e & 1) ? ((w[k] & 0x0000FFFFu) | (v << 16)) : ((w[k] & 0xFFFF0000u) | v);
                f.v[dt].u = make_uint4(w[0], w[1], w[2], w[3]);
            }
        }
    }
    if (has) process_page<DH, 1>(c, f, page, lane, scale_log2, false);
    finish_columns<DH, 1>(c);

#pragma unroll
    for (int dt = 0; dt < DH / 16; ++dt)
#pragma unroll
        for (int r = 0; r < 4; ++r) o_lds[wave][(dt * 16 + jg * 4 + r) * 17 + col] = c.o[0][dt][r];
    if (jg == 0) {
        ml_lds[wave][0][col] = c.m[0];
        ml_lds[wave][1][col] = c.l[0];
    }
    __syncthreads();
    for (int idx = threadIdx.x; idx < group * DH; idx += CW * 64) {
        const int g = idx / DH, d = idx - g * DH;
        float m = -INFINITY;
#pragma unroll
        for (int w = 0; w < CW; ++w) m = fmaxf(m, ml_lds[w][0][g]);
        float acc = 0.f, l = 0.f;
#pragma unroll
        for (int w = 0; w < CW; ++w) {
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

// Column tiles per wavefront: at most 64 columns for head_dim up to 64, 32 for 128 (registers); fewer when
// that leaves the launch with less than four workgroups a compute unit (few query heads per kv head, a
// prompt of a few thousand tokens: at 32 query and 8 kv heads of 128, 2,048 tokens take 81 us with 1,024
// workgroups of half the columns against 95 us with 512; from 4,096 tokens on the full tiles win).  A
// column's arithmetic does not depend on the tile it sits in, only the grid does.
// Tiles are halved while the launch has fewer workgroups than this many for each compute unit (measured with
// 256 of them: a prompt of 3,072 tokens at Qwen3-8B sizes takes 105 us with two tiles a wavefront in 768
// workgroups, 126 us with one tile in 1,536; at 2,048 tokens one tile in 1,024 workgroups takes 57 us, two in
// 512 take 67).
#define PREFILL_MIN_WGS_PER_CU 3
static int prefill_tiles(int head_dim, int group, int max_new, int seqs, int kv_heads) {
    int nt = head_dim <= 64 ? 4 : 2;
    while (nt > 1 && group <= 16 * (nt / 2)) {
        const int tile_tokens = (16 * nt) / group;
        const long wgs = (long)((max_new + 4 * tile_tokens - 1) / (4 * tile_tokens)) * seqs * kv_heads;
        if (wgs >= (long)PREFILL_MIN_WGS_PER_CU * ri_compute_units()) break;
        nt /= 2;
    }
    return nt;
}

extern "C" int ri_attention_prefill_bf16(void* out, const void* qkv, int q_stride, const void* k_pages,
                                         const void* v_pages, const int32_t* cu_seqlens, const int32_t* tok_pos,
                                         const int32_t* page_table, int table_width, int seqs, int max_new,
                                         int heads, int kv_heads, int head_dim, int page_size, int window,
                                         float scale, void* stream) {
    if (check_common("attention_prefill_bf16", heads, kv_heads, head_dim, page_size, q_stride, table_width)) return 1;
    const int group = heads / kv_heads;
    RI_REQUIRE(seqs > 0 && seqs <= 65535 && max_new > 0, "attention_prefill_bf16: seqs %d, max_new %d", seqs, max_new);
    const int nt_tiles = prefill_tiles(head_dim, group, max_new, seqs, kv_heads);
    RI_REQUIRE(group <= 16 * nt_tiles, "attention_prefill_bf16: %d query heads per kv head (at most %d)", group,
               16 * nt_tiles);
    const int tile_tokens = (16 * nt_tiles) / group;
    const int tiles = (max_new + 4 * tile_tokens - 1) / (4 * tile_tokens);
    RI_REQUIRE(tiles <= 65535, "attention_prefill_bf16: %d tiles of tokens exceed one launch", tiles);
    dim3 grid(kv_heads, tiles, seqs);
    const float scale_log2 = scale * 1.4426950408889634f;
    hipStream_t s = (hipStream_t)stream;
#define RI_PREFILL_CASE(DH, NT)                                                                                  \
    case DH * 8 + NT:                                                                                            \
        attn_prefill_mfma_kernel<DH, NT><<<grid, 256, 0, s>>>(                                                   \
            (bf16_t*)out, (const bf16_t*)qkv, q_stride, (const bf16_t*)k_pages, (const bf16_t*)v_pages,          \
            cu_seqlens, tok_pos, page_table, table_width, heads, kv_heads, window, scale_log2);                  \
        break;
    switch (head_dim * 8 + nt_tiles) {
        RI_PREFILL_CASE(32, 4)
        RI_PREFILL_CASE(32, 2)
        RI_PREFILL_CASE(32, 1)
        RI_PREFILL_CASE(64, 4)
        RI_PREFILL_CASE(64, 2)
        RI_PREFILL_CASE(64, 1)
        RI_PREFILL_CASE(128, 2)
        RI_PREFILL_CASE(128, 1)
    }
#undef RI_PREFILL_CASE
    RI_LAUNCH_CHECK("attention_prefill_bf16");
    return 0;
}

extern "C" int ri_attention_decode_chunks(int max_len) { return (max_len + DECODE_CHUNK - 1) / DECODE_CHUNK; }

// Pieces that the chunk kernels cut every chunk into: 1, or 2 or 4 (workgroups of four or two wavefronts, one page
// each) while the step's workgroups, counted by the bound on the lengths, stay within one for every compute unit and
// the pieces of a sequence within what the join fetches at once (past that the cut loses what it gains).  A
// workgroup norms two query heads a wavefront at most, so a kv head's query heads bound the cut too.
#ifndef DECODE_SPLIT_FILL
#define DECODE_SPLIT_FILL 1
#endif
static int decode_pieces(int seqs, int kv_heads, int group, int max_chunks) {
    if (stream_splits(seqs, kv_heads, max_chunks) > 0) return 1;
    const long wgs = (long)seqs * kv_heads * max_chunks, cus = ri_compute_units();
    int pieces = 1;
    while (pieces < 4 && wgs * pieces * 2 <= DECODE_SPLIT_FILL * cus && max_chunks * pieces * 2 <= JOIN_SERIAL &&
           group <= 2 * (DECODE_WAVES / (pieces * 2)))
        pieces *= 2;
    return pieces;
}

// The workspace of a decode attention call has room for max_chunks times this many results a sequence and head.
extern "C" int ri_attention_decode_pieces(int seqs, int kv_heads, int heads, int max_chunks) {
    return decode_pieces(seqs, kv_heads, heads / (kv_heads > 0 ? kv_heads : 1), max_chunks);
}

extern "C" int ri_attention_decode_bf16(void* out, float* workspace, const void* qkv, int q_stride,
                                        const void* k_pages, const void* v_pages, const int32_t* cu_seqlens,
                                        const int32_t* tok_pos, const int32_t* page_table, int table_width, int seqs,
                                        int max_chunks, int heads, int kv_heads, int head_dim, int page_size,
                                        int window, float scale, int tiled_out, void* stream) {
    if (check_common("attention_decode_bf16", heads, kv_heads, head_dim, page_size, q_stride, table_width)) return 1;
    RI_REQUIRE(!tiled_out || (seqs <= 64 && head_dim % 32 == 0), "attention_decode_bf16: tiled rows are at most 64 (%d)", seqs);
    const int group = heads / kv_heads;
    RI_REQUIRE(group <= 16, "attention_decode_bf16: %d query heads per kv head (at most 16)", group);
    RI_REQUIRE(seqs > 0 && max_chunks > 0 && max_chunks <= 65535 && heads <= 65535,
               "attention_decode_bf16: seqs %d, chunks %d, heads %d", seqs, max_chunks, heads);
    dim3 grid(seqs, kv_heads, max_chunks);
    const float scale_log2 = scale * 1.4426950408889634f;
    hipStream_t s = (hipStream_t)stream;
    const int splits = stream_splits(seqs, kv_heads, max_chunks);
    const bool wide = stream_wide(seqs, kv_heads, max_chunks);
    if (splits > 0) {
        dim3 sgrid(seqs, kv_heads, splits);
#define RI_STREAM_CASE(DH)                                                                                        \
    case DH:                                                                                                      \
        if (wide)                                                                                                 \
            attn_decode_stream_kernel<DH, false, 8><<<sgrid, 8 * 64, 0, s>>>(                                     \
                (bf16_t*)out, workspace, (const bf16_t*)qkv, q_stride, nullptr, nullptr, 0.f, nullptr,            \
                (bf16_t*)k_pages, (bf16_t*)v_pages, tok_pos, page_table, table_width, heads, kv_heads, window,    \
                scale_log2, splits, tiled_out);                                                                   \
        else                                                                                                      \
            attn_decode_stream_kernel<DH, false, 4><<<sgrid, 4 * 64, 0, s>>>(                                     \
                (bf16_t*)out, workspace, (const bf16_t*)qkv, q_stride, nullptr, nullptr, 0.f, nullptr,            \
                (bf16_t*)k_pages, (bf16_t*)v_pages, tok_pos, page_table, table_width, heads, kv_heads, window,    \
                scale_log2, splits, tiled_out);                                                                   \
        if (splits > 1) launch_join<DH>((bf16_t*)out, workspace, tok_pos, seqs, heads, -1, splits, tiled_out, s); \
        break;
        switch (head_dim) {
            RI_STREAM_CASE(32)
            RI_STREAM_CASE(64)
            RI_STREAM_CASE(128)
        }
#undef RI_STREAM_CASE
        RI_LAUNCH_CHECK("attention_decode_bf16 (streaming)");
        return 0;
    }
    const int pieces = decode_pieces(seqs, kv_heads, group, max_chunks), all = max_chunks * pieces;
    const dim3 pgrid(seqs, kv_heads, all);
#define RI_DECODE_CASE(DH, CW)                                                                                    \
    case DH * 16 + CW:                                                                                            \
        attn_decode_mfma_kernel<DH, CW><<<pgrid, CW * 64, 0, s>>>(                                                \
            workspace, (const bf16_t*)qkv, q_stride, (const bf16_t*)k_pages, (const bf16_t*)v_pages,             \
            tok_pos, page_table, table_width, heads, kv_heads, window, scale_log2, all);                          \
        launch_join<DH>((bf16_t*)out, workspace, tok_pos, seqs, heads, window, all, tiled_out, s, CW * PAGE);     \
        break;
    switch (head_dim * 16 + DECODE_WAVES / pieces) {
        RI_DECODE_CASE(32, 8)
        RI_DECODE_CASE(32, 4)
        RI_DECODE_CASE(32, 2)
        RI_DECODE_CASE(64, 8)
        RI_DECODE_CASE(64, 4)
        RI_DECODE_CASE(64, 2)
        RI_DECODE_CASE(128, 8)
        RI_DECODE_CASE(128, 4)
        RI_DECODE_CASE(128, 2)
    }
#undef RI_DECODE_CASE
    RI_LAUNCH_CHECK("attention_decode_bf16");
    return 0;
}

// The decode attention of a layer from the raw fused projection (which is not changed): q/k norm, rotation,
// the new token's k and v into their pages and attention in chunks in one kernel, then the join.
extern "C" int ri_attention_decode_fused_bf16(void* out, float* workspace, const void* qkv, int q_stride,
                                              const float* q_gain, const float* k_gain, float eps,
                                              const float* inv_freq, void* k_pages, void* v_pages,
                                              const int32_t* tok_pos, const int32_t* page_table, int table_width,
                                              int seqs, int max_chunks, int heads, int kv_heads, int head_dim,
                                              int page_size, int window, float scale, int tiled_out, void* stream) {
    if (check_common("attention_decode_fused_bf16", heads, kv_heads, head_dim, page_size, q_stride, table_width))
        return 1;
    RI_REQUIRE(!tiled_out || (seqs <= 64 && head_dim % 32 == 0), "attention_decode_fused_bf16: tiled rows are at most 64 (%d)", seqs);
    const int group = heads / kv_heads;
    RI_REQUIRE(group <= 16, "attention_decode_fused_bf16: %d query heads per kv head (at most 16)", group);
    RI_REQUIRE(seqs > 0 && max_chunks > 0 && max_chunks <= 65535 && heads <= 65535,
               "attention_decode_fused_bf16: seqs %d, chunks %d, heads %d", seqs, max_chunks, heads);
    RI_REQUIRE(q_stride >= (heads + 2 * kv_heads) * head_dim, "attention_decode_fused_bf16: qkv row stride %d",
               q_stride);
    dim3 grid(seqs, kv_heads, max_chunks);
    const float scale_log2 = scale * 1.4426950408889634f;
    hipStream_t s = (hipStream_t)stream;
    const int splits = stream_splits(seqs, kv_heads, max_chunks);
    const bool wide = stream_wide(seqs, kv_heads, max_chunks);
    if (splits > 0) {
        dim3 sgrid(seqs, kv_heads, splits);
#define RI_STREAM_CASE(DH)                                                                                        \
    case DH:                                                                                                      \
        if (wide)                                                                                                 \
            attn_decode_stream_kernel<DH, true, 8><<<sgrid, 8 * 64, 0, s>>>(                                      \
                (bf16_t*)out, workspace, (const bf16_t*)qkv, q_stride, q_gain, k_gain, eps, inv_freq,             \
                (bf16_t*)k_pages, (bf16_t*)v_pages, tok_pos, page_table, table_width, heads, kv_heads, window,    \
                scale_log2, splits, tiled_out);                                                                   \
        else                                                                                                      \
            attn_decode_stream_kernel<DH, true, 4><<<sgrid, 4 * 64, 0, s>>>(                                      \
                (bf16_t*)out, workspace, (const bf16_t*)qkv, q_stride, q_gain, k_gain, eps, inv_freq,             \
                (bf16_t*)k_pages, (bf16_t*)v_pages, tok_pos, page_table, table_width, heads, kv_heads, window,    \
                scale_log2, splits, tiled_out);                                                                   \
        if (splits > 1) launch_join<DH>((bf16_t*)out, workspace, tok_pos, seqs, heads, -1, splits, tiled_out, s); \
        break;
        switch (head_dim) {
            RI_STREAM_CASE(32)
            RI_STREAM_CASE(64)
            RI_STREAM_CASE(128)
        }
#undef RI_STREAM_CASE
        RI_LAUNCH_CHECK("attention_decode_fused_bf16 (streaming)");
        return 0;
    }
    const int pieces = decode_pieces(seqs, kv_heads, group, max_chunks), all = max_chunks * pieces;
    const dim3 pgrid(seqs, kv_heads, all);
#define RI_FUSED_CASE(DH, CW)                                                                                     \
    case DH * 16 + CW:                                                                                            \
        attn_decode_fused_kernel<DH, CW><<<pgrid, CW * 64, 0, s>>>(                                               \
            workspace, (const bf16_t*)qkv, q_stride, q_gain, k_gain, eps, inv_freq, (bf16_t*)k_pages,             \
            (bf16_t*)v_pages, tok_pos, page_table, table_width, heads, kv_heads, window, scale_log2, all);        \
        launch_join<DH>((bf16_t*)out, workspace, tok_pos, seqs, heads, window, all, tiled_out, s, CW * PAGE);     \
        break;
    switch (head_dim * 16 + DECODE_WAVES / pieces) {
        RI_FUSED_CASE(32, 8)
        RI_FUSED_CASE(32, 4)
        RI_FUSED_CASE(32, 2)
        RI_FUSED_CASE(64, 8)
        RI_FUSED_CASE(64, 4)
        RI_FUSED_CASE(64, 2)
        RI_FUSED_CASE(128, 8)
        RI_FUSED_CASE(128, 4)
        RI_FUSED_CASE(128, 2)
    }
#undef RI_FUSED_CASE
    RI_LAUNCH_CHECK("attention_decode_fused_bf16");
    return 0;
}
