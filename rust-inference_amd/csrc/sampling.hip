// Next-token selection on the device, one workgroup per row of logits: repetition penalty, greedy
// when the temperature is not positive, else temperature, top-k, top-p and one draw, with the
// meaning of every stage taken from the reference's host sampler (src/sampling.rs:73-127):
//
//   penalty   every token id seen before: a positive logit is divided, any other multiplied (:76-88)
//   order     candidates by falling scaled logit, rising id among equal values (:99)
//   top-k     the first k of that order (:95-98)
//   softmax   exp(s - max) over the kept candidates (:101-104)
//   top-p     the shortest prefix of the order whose mass reaches top_p, normalised again (:105-117)
//   draw      the first candidate whose running mass exceeds r, r uniform in [0, 1) from the host's
//             generator (:119-127)
//
// Nothing is sorted.  The order is a 56-bit key per candidate (the float's bits made monotone, then
// 2^24 - 1 - id), and "the first candidate whose running count or mass passes a target" is found by
// descending that key eight bits at a time: a histogram of the candidates that share the prefix found
// so far, then a scan of its 256 bins from the top (the id bits are settled in one step as a rule: see
// descend).  Masses are 40-bit fixed-point integers, so every
// sum is exact and independent of the order of addition: the same logits and the same r give the
// same token on every run.  Lanes add into 16 copies of the histogram, so that
// the many candidates that share a bin do not queue up on one LDS address.
#include "api.h"
#include "common.h"

#define SMP_THREADS 1024
#define SMP_COPIES 16
#define SMP_ID_BITS 24
#define SMP_FIXED 1099511627776.0f      // 2^40
#define SMP_TIES 2048                   // candidates of one value whose ids are listed rather than descended

typedef unsigned long long u64;

__device__ __forceinline__ uint32_t ordered_bits(float f) {
    // larger float <=> larger unsigned; -0.0 and +0.0 compare equal like the floats do
    uint32_t u = __float_as_uint(f == 0.f ? 0.f : f);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

struct RowView {
    const float* logits;
    const uint8_t* seen;     // may be NULL
    float penalty, temperature;      // temperature: the divisor of every logit (1 when the row is taken greedily)
    bool wide;               // the row starts on a 16-byte boundary and the vocabulary is a multiple of 4
    __device__ __forceinline__ float penalise(float l, bool was_seen) const {
        return was_seen ? (l > 0.f ? l / penalty : l * penalty) : l;
    }
};

// f(i, penalised logit of token i) for every token of the row, each token once, the workgroup's threads
// sharing the work.  One pass over a row is bound by the latency of its loads, not by their volume (a
// row is a few hundred KB in the L2 cache), so the loads are 16 bytes wide where the row allows it and
// SMP_UNROLL of them are in flight per thread before the first value is used.
#define SMP_UNROLL 4
template <typename F>
__device__ __forceinline__ void for_each_logit(const RowView& row, int begin, int end, int threads, F&& f) {
    if (row.wide) {                                       // begin is a multiple of 4, end one or the vocabulary's end
        const float4* lp = reinterpret_cast<const float4*>(row.logits);
        const uint32_t* sp = reinterpret_cast<const uint32_t*>(row.seen);
        const int end4 = end / 4;
        for (int i0 = begin / 4 + threadIdx.x; i0 < end4; i0 += threads * SMP_UNROLL) {
            float4 v[SMP_UNROLL];
            uint32_t sn[SMP_UNROLL];
#pragma unroll
            for (int u = 0; u < SMP_UNROLL; ++u) {
                const int i = i0 + u * threads;
                v[u] = i < end4 ? lp[i] : make_float4(0.f, 0.f, 0.f, 0.f);
                sn[u] = (sp && i < end4) ? sp[i] : 0u;
            }
#pragma unroll
            for (int u = 0; u < SMP_UNROLL; ++u) {
                const int i = i0 + u * threads;
                if (i < end4) {
                    f(4 * i, row.penalise(v[u].x, sn[u] & 0x000000FFu));
                    f(4 * i + 1, row.penalise(v[u].y, sn[u] & 0x0000FF00u));
                    f(4 * i + 2, row.penalise(v[u].z, sn[u] & 0x00FF0000u));
                    f(4 * i + 3, row.penalise(v[u].w, sn[u] & 0xFF000000u));
                }
            }
        }
    } else {
        for (int i = begin + threadIdx.x; i < end; i += threads)
            f(i, row.penalise(row.logits[i], row.seen && row.seen[i]));
    }
}

// The fixed-point mass of a candidate, exp(s - smax) * 2^40 cut to an integer: one function, used wherever
// a mass is wanted, so that every pass sees the same number.  The exponential is the hardware's base-2
// one (its argument is at most 0, its last bit or two are its own: the masses define the distribution that
// is drawn from, and they differ from the exact ones by parts in ten million).  The float, at least 1
// and below 2^41, is widened by hand: 24 bits of mantissa shifted into place.
__device__ __forceinline__ u64 fixed_mass(float s, float smax) {
    const float x = __builtin_amdgcn_exp2f((s - smax) * 1.44269504088896341f) * SMP_FIXED;
    const uint32_t bits = __float_as_uint(x);
    const int e = (int)(bits >> 23) - 127;                   // x is not negative and not above 2^40 (1 + 2^-22)
    if (e < 0) return 0;
    const u64 mant = (u64)((bits & 0x007FFFFFu) | 0x00800000u);
    return e >= 23 ? mant << (e - 23) : mant >> (23 - e);
}

__device__ __forceinline__ u64 composite(float s, int id) {
    return ((u64)ordered_bits(s) << SMP_ID_BITS) | (u64)((1 << SMP_ID_BITS) - 1 - id);
}

__device__ __forceinline__ float value_of_ordered(uint32_t ob) {      // the inverse of ordered_bits
    return __uint_as_float((ob & 0x80000000u) ? (ob & 0x7FFFFFFFu) : ~ob);
}

// One digit of a descent: from the 256 bins of the candidates that share the prefix found so far, the
// highest bin b whose candidates bring the running weight past the target:
//   shared[0] = weight above bin b, shared[1] = b, shared[2] = weight down to and including bin b.
// The first wavefront does it, four bins a lane, with a suffix sum over the lanes.
__device__ __forceinline__ void pick_bin(const u64* bins, u64 above, u64 target, u64* shared) {
    if (threadIdx.x < 64) {
        const int lane = threadIdx.x;
        const u64 b0 = bins[4 * lane], b1 = bins[4 * lane + 1], b2 = bins[4 * lane + 2], b3 = bins[4 * lane + 3];
        const u64 mine = b0 + b1 + b2 + b3;
        u64 sfx = mine;                                         // this lane's bins and all higher lanes'
        for (int d = 1; d < 64; d <<= 1) {
            const u64 o = __shfl_down(sfx, d, 64);
            if (lane + d < 64) sfx += o;
        }
        const u64 a3 = above + (sfx - mine);                    // weight above bin 4 lane + 3
        const u64 a2 = a3 + b3, a1 = a2 + b2, a0 = a1 + b1;
        int hit = -1;
        u64 hit_above = 0, hit_bin = 0;
        if (a3 + b3 > target)      { hit = 4 * lane + 3; hit_above = a3; hit_bin = b3; }
        else if (a2 + b2 > target) { hit = 4 * lane + 2; hit_above = a2; hit_bin = b2; }
        else if (a1 + b1 > target) { hit = 4 * lane + 1; hit_above = a1; hit_bin = b1; }
        else if (a0 + b0 > target) { hit = 4 * lane;     hit_above = a0; hit_bin = b0; }
        const u64 any = __ballot(hit >= 0);
        const int top = any ? 63 - __clzll((long long)any) : 0;       // nothing passes the target: bin 0
        if (lane == top) {
            if (!any) { hit = 0; hit_above = a0; hit_bin = b0; }
            shared[0] = hit_above;
            shared[1] = (u64)hit;
            shared[2] = hit_above + hit_bin;
        }
    }
}

// Finds the key c* with  sum_{c > c*} w  <=  target  <  sum_{c >= c*} w  over the candidates with
// key >= floor_key, w = 1 (count) or the fixed-point mass.  Returns c*; *incl = sum_{c >= c*} w.
//
// Four passes settle the 32 value bits.  What is left are the candidates whose value is exactly that
// (nearly always one): a fifth pass lists their ids, they all weigh the same, and the one wanted is found
// by its rank.  Only if the list overflows (a row of equal logits) the id bits are descended like the
// value bits.
//
// prefix: the bits of c* found so far, in place; above: the weight of the candidates above the prefix's
// bucket; first_shift: the digit to go on with (48, prefix and above 0: from the start); list_ties false:
// the id bits are descended at once (the caller has found the list too short already).
template <bool MASS>
__device__ u64 descend_from(const RowView& row, int vocab, float smax, u64 floor_key, u64 target, u64 prefix, u64 above,
                            int first_shift, bool list_ties, u64* hist, u64* bins, u64* shared, int* ties,
                            int* tie_count, u64* incl) {
    for (int shift = first_shift; shift >= 0; shift -= 8) {
        if (list_ties && shift == SMP_ID_BITS - 8) {          // the value is known: list the ids that have it
            if (threadIdx.x == 0) *tie_count = 0;
            __syncthreads();
            const uint32_t value_bits = (uint32_t)(prefix >> SMP_ID_BITS);
            for_each_logit(row, 0, vocab, SMP_THREADS, [&](int i, float l) {
                const float s = l / row.temperature;
                if (ordered_bits(s) == value_bits && composite(s, i) >= floor_key) {
                    const int k = atomicAdd(tie_count, 1);
                    if (k < SMP_TIES) ties[k] = i;
                }
            });
            __syncthreads();
            const int n = *tie_count;
            if (n >= 1 && n <= SMP_TIES) {                      // (none: cannot be, the bucket was chosen for its weight)
                const float s = value_of_ordered(value_bits);
                const u64 w = MASS ? fixed_mass(s, smax) : 1;
                u64 j = w ? (target - above) / w : 0;           // so many of the tied candidates lie above c*
                if (j > (u64)(n - 1)) j = (u64)(n - 1);
                for (int k = threadIdx.x; k < n; k += SMP_THREADS) {      // ids rise as keys fall: the j-th smallest id
                    const int id = ties[k];
                    int rank = 0;
                    for (int q = 0; q < n; ++q) rank += ties[q] < id;
                    if ((u64)rank == j) {
                        shared[0] = prefix | (u64)((1 << SMP_ID_BITS) - 1 - id);
                        shared[1] = above + (j + 1) * w;
                    }
                }
                __syncthreads();
                prefix = shared[0];
                *incl = shared[1];
                __syncthreads();
                return prefix;
            }
        }
        for (int i = threadIdx.x; i < 256 * SMP_COPIES; i += SMP_THREADS) hist[i] = 0;
        __syncthreads();
        const u64 hi_mask = shift == 48 ? 0 : (~(u64)0) << (shift + 8);
        for_each_logit(row, 0, vocab, SMP_THREADS, [&](int i, float l) {
            const float s = l / row.temperature;
            const u64 c = composite(s, i);
            if (c >= floor_key && (c & hi_mask) == (prefix & hi_mask)) {
                const u64 w = MASS ? fixed_mass(s, smax) : 1;
                atomicAdd(&hist[((c >> shift) & 255) * SMP_COPIES + (threadIdx.x & (SMP_COPIES - 1))], w);
            }
        });
        __syncthreads();
        if (threadIdx.x < 256) {
            u64 t = 0;
            for (int k = 0; k < SMP_COPIES; ++k) t += hist[threadIdx.x * SMP_COPIES + k];
            bins[threadIdx.x] = t;
        }
        __syncthreads();
        pick_bin(bins, above, target, shared);
        __syncthreads();
        above = shared[0];
        prefix |= shared[1] << shift;
        *incl = shared[2];
        __syncthreads();
    }
    return prefix;
}

template <bool MASS>
__device__ u64 descend(const RowView& row, int vocab, float smax, u64 floor_key, u64 target, u64* hist, u64* bins,
                       u64* shared, int* ties, int* tie_count, u64* incl) {
    return descend_from<MASS>(row, vocab, smax, floor_key, target, 0, 0, 48, true, hist, bins, shared, ties, tie_count,
                              incl);
}

__device__ __forceinline__ RowView row_view(const float* logits, const uint8_t* seen, const int32_t* seen_rows, int r,
                                            int vocab, float temperature, float penalty) {
    RowView row;
    row.logits = logits + (size_t)r * vocab;
    row.seen = (seen && penalty != 1.0f) ? seen + (size_t)(seen_rows ? seen_rows[r] : r) * vocab : nullptr;
    row.penalty = penalty;
    row.temperature = temperature > 0.f ? temperature : 1.0f;      // logit / temperature, a true division (src/sampling.rs:93-94)
    row.wide = vocab % 4 == 0 && ((uintptr_t)row.logits & 15) == 0 && ((uintptr_t)row.seen & 3) == 0;
    return row;
}

__global__ void __launch_bounds__(SMP_THREADS)
sample_kernel(int32_t* __restrict__ out, const float* __restrict__ logits, const uint8_t* __restrict__ seen,
              const int32_t* __restrict__ seen_rows, const float* __restrict__ uniform, int vocab, float temperature,
              int top_k, float top_p, float penalty) {
    __shared__ u64 hist[256 * SMP_COPIES];
    __shared__ u64 bins[256];
    __shared__ u64 shared[4];
    __shared__ int ties[SMP_TIES];
    __shared__ int tie_count;
    __shared__ float fscratch[16];
    __shared__ int iscratch[16];
    const RowView row = row_view(logits, seen, seen_rows, blockIdx.x, vocab, temperature, penalty);

    if (!(temperature > 0.f)) {                            // greedy: the first maximum (src/sampling.rs:131-139)
        float v = -INFINITY;
        int idx = 0x7FFFFFFF;
        for_each_logit(row, 0, vocab, SMP_THREADS, [&](int i, float l) {
            if (l > v || (l == v && i < idx)) { v = l; idx = i; }
        });
        for (int m = RI_WAVE / 2; m > 0; m >>= 1) {
            const float ov = __shfl_xor(v, m, RI_WAVE);
            const int oi = __shfl_xor(idx, m, RI_WAVE);
            if (ov > v || (ov == v && oi < idx)) { v = ov; idx = oi; }
        }
        if ((threadIdx.x & 63) == 0) { fscratch[threadIdx.x >> 6] = v; iscratch[threadIdx.x >> 6] = idx; }
        __syncthreads();
        if (threadIdx.x == 0) {
            for (int w = 1; w < SMP_THREADS / 64; ++w)
                if (fscratch[w] > v || (fscratch[w] == v && iscratch[w] < idx)) { v = fscratch[w]; idx = iscratch[w]; }
            out[blockIdx.x] = idx == 0x7FFFFFFF ? 0 : idx;
        }
        return;
    }

    float smax = -INFINITY;
    for_each_logit(row, 0, vocab, SMP_THREADS, [&](int, float l) { smax = fmaxf(smax, l / row.temperature); });
    smax = block_max(smax, fscratch);

    u64 floor_key = 0, incl = 0;
    if (top_k > 0 && top_k < vocab)                       // the k-th candidate of the order closes the kept set
        floor_key = descend<false>(row, vocab, smax, 0, (u64)(top_k - 1), hist, bins, shared, ties, &tie_count, &incl);
    // total mass of the kept set: descend to the very last candidate (target = everything but one unit)
    // would cost seven more passes; one exact integer sum does it
    u64 z = 0;
    for_each_logit(row, 0, vocab, SMP_THREADS, [&](int i, float l) {
        const float s = l / row.temperature;
        if (composite(s, i) >= floor_key) z += fixed_mass(s, smax);
    });
    for (int m = RI_WAVE / 2; m > 0; m >>= 1) z += __shfl_xor(z, m, RI_WAVE);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) bins[threadIdx.x >> 6] = z;
    __syncthreads();
    z = 0;
    for (int w = 0; w < SMP_THREADS / 64; ++w) z += bins[w];
    __syncthreads();

    if (top_p < 1.0f) {                                    // shortest prefix whose mass reaches top_p * z
        u64 want = (u64)ceil((double)top_p * (double)z);
        if (want < 1) want = 1;
        if (want > z) want = z;
        floor_key = descend<true>(row, vocab, smax, floor_key, want - 1, hist, bins, shared, ties, &tie_count, &incl);
        z = incl;                                          // the kept mass, to be normalised by
    }
    const u64 target = (u64)((double)uniform[blockIdx.x] * (double)z);     // r < 1, so target < z
    const u64 pick = descend<true>(row, vocab, smax, floor_key, target < z ? target : z - 1, hist, bins, shared, ties,
                                  &tie_count, &incl);
    if (threadIdx.x == 0) out[blockIdx.x] = (1 << SMP_ID_BITS) - 1 - (int)(pick & ((1 << SMP_ID_BITS) - 1));
}

extern "C" int ri_sample(int32_t* out, const float* logits, const uint8_t* seen, const int32_t* seen_rows,
                         const float* uniform, int rows, int vocab, float temperature, int top_k, float top_p,
                         float penalty, void* stream) {
    RI_REQUIRE(rows > 0 && vocab > 0 && vocab < (1 << SMP_ID_BITS), "sample: rows %d, vocab %d (below %d)", rows, vocab,
               1 << SMP_ID_BITS);
    RI_REQUIRE(top_k >= 0 && top_p > 0.f && penalty > 0.f, "sample: top_k %d, top_p %g, penalty %g", top_k,
               (double)top_p, (double)penalty);
    RI_REQUIRE(!(temperature > 0.f) || uniform != nullptr, "sample: a positive temperature needs uniform draws");
    sample_kernel<<<rows, SMP_THREADS, 0, (hipStream_t)stream>>>(out, logits, seen, seen_rows, uniform, vocab,
                                                                 temperature, top_k, top_p, penalty);
    RI_LAUNCH_CHECK("sample");
    return 0;
}

// ------------------------------------------------------------------ the same selection, a row over many workgroups
// One workgroup has one compute unit's loads in flight, and a pass over a large vocabulary is bound by
// exactly that.  Here every pass is a launch of its own and a row is cut into slices, one workgroup each:
//
//   max          the largest scaled logit of the row (atomic maximum of the ordered bits)
//   per descent  (top-k, top-p, draw: those that are asked for, in this order)
//     digit 0..3   a histogram of the slice's candidates in LDS, added into the row's in the workspace
//     ties         the ids of the candidates that have the value found, appended to the row's list
//     finish       one workgroup a row: the candidate by its rank among the ties (or, if the list is too
//                  short for them, the id digits over the whole row as in the kernel above); the last
//                  descent's is the token
//
// No kernel hands a state to the next: each replays the digits found so far from the histograms in the
// workspace, which are complete when it starts.  All sums are of integers, so the token is the one that
// the one-workgroup kernel finds.
#define SW_THREADS 256
#define SW_COPIES 4
#define SW_DESCENTS 3                                              // 0: top-k, 1: top-p, 2: the draw
// a row's workspace, in 64-bit words
#define SW_HIST 0                                                  // [descent][digit 0..3][256]
#define SW_RESULT (SW_DESCENTS * 4 * 256)                          // [descent][2]: the key found, the weight down to it
#define SW_SMAX (SW_RESULT + SW_DESCENTS * 2)                      // ordered bits of the largest scaled logit
#define SW_TIE_COUNT (SW_SMAX + 1)                                 // [descent]
#define SW_TIES (SW_TIE_COUNT + SW_DESCENTS)                       // [descent][SMP_TIES] ids, 32 bits each
#define SW_WORDS (SW_TIES + SW_DESCENTS * SMP_TIES / 2)

struct SplitPlan {
    const float* logits;
    const uint8_t* seen;
    const int32_t* seen_rows;
    const float* uniform;
    u64* ws;
    int vocab, slice;              // slice: tokens per workgroup, a multiple of 4
    float temperature;
    int top_k;
    float top_p, penalty;
};

struct Descent {
    u64 floor_key, target, prefix, above, incl;
};

// The sum of 256 bins in LDS, for every thread (a workgroup of at least 64 threads).
__device__ __forceinline__ u64 bins_total(const u64* bins, u64* shared) {
    if (threadIdx.x < 64) {
        u64 t = bins[4 * threadIdx.x] + bins[4 * threadIdx.x + 1] + bins[4 * threadIdx.x + 2] + bins[4 * threadIdx.x + 3];
        for (int d = 32; d > 0; d >>= 1) t += __shfl_xor(t, d, 64);
        if (threadIdx.x == 0) shared[3] = t;
    }
    __syncthreads();
    const u64 t = shared[3];
    __syncthreads();
    return t;
}

// Where descent `desc` of this row stands after `digits` of its value digits, from the workspace.
__device__ void replay(const SplitPlan& p, const u64* ws_row, int r, int desc, int digits, u64* bins, u64* shared,
                       Descent& d) {
    const bool has_k = p.top_k > 0 && p.top_k < p.vocab, has_p = p.top_p < 1.0f;
    d.floor_key = desc == 0 ? 0 : (desc == 2 && has_p) ? ws_row[SW_RESULT + 2] : has_k ? ws_row[SW_RESULT] : 0;
    d.target = d.prefix = d.above = d.incl = 0;
    if (digits == 0) return;
    const u64* hist = ws_row + SW_HIST + (size_t)desc * 4 * 256;
    if (desc == 0) {
        d.target = (u64)(p.top_k - 1);
    } else {
        u64 z;                                                     // the mass of the kept candidates
        if (desc == 2 && has_p) {
            z = ws_row[SW_RESULT + 3];
        } else {                                                   // this descent's first histogram holds them all
            if (threadIdx.x < 256) bins[threadIdx.x] = hist[threadIdx.x];
            __syncthreads();
            z = bins_total(bins, shared);
        }
        if (desc == 1) {                                           // shortest prefix whose mass reaches top_p * z
            u64 want = (u64)ceil((double)p.top_p * (double)z);
            if (want < 1) want = 1;
            if (want > z) want = z;
            d.target = want - 1;
        } else {
            const u64 t = (u64)((double)p.uniform[r] * (double)z);  // r < 1, so t < z
            d.target = t < z ? t : z - 1;
        }
    }
    for (int dd = 0; dd < digits; ++dd) {
        if (threadIdx.x < 256) bins[threadIdx.x] = hist[dd * 256 + threadIdx.x];
        __syncthreads();
        pick_bin(bins, d.above, d.target, shared);
        __syncthreads();
        d.above = shared[0];
        d.prefix |= shared[1] << (48 - 8 * dd);
        d.incl = shared[2];
        __syncthreads();
    }
}

__global__ void split_fill_kernel(u64* ws, long words) {
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < words) ws[i] = 0;
}

__global__ void __launch_bounds__(SW_THREADS)
split_max_kernel(SplitPlan p) {
    __shared__ float fscratch[16];
    const int r = blockIdx.y, begin = blockIdx.x * p.slice, end = min(p.vocab, begin + p.slice);
    const RowView row = row_view(p.logits, p.seen, p.seen_rows, r, p.vocab, p.temperature, p.penalty);
    float smax = -INFINITY;
    for_each_logit(row, begin, end, SW_THREADS, [&](int, float l) { smax = fmaxf(smax, l / row.temperature); });
    smax = block_max(smax, fscratch);
    if (threadIdx.x == 0 && begin < end)
        atomicMax(reinterpret_cast<unsigned int*>(p.ws + (size_t)r * SW_WORDS + SW_SMAX), ordered_bits(smax));
}

__device__ __forceinline__ float row_smax(const u64* ws_row) {
    return value_of_ordered((uint32_t)ws_row[SW_SMAX]);
}

// digit 0..3: the slice's share of the histogram; digit 4: its share of the list of ties.
template <bool MASS>
__global__ void __launch_bounds__(SW_THREADS)
split_pass_kernel(SplitPlan p, int desc, int digit) {
    __shared__ u64 hist[256 * SW_COPIES];
    __shared__ u64 bins[256];
    __shared__ u64 shared[4];
    const int r = blockIdx.y, begin = blockIdx.x * p.slice, end = min(p.vocab, begin + p.slice);
    u64* ws_row = p.ws + (size_t)r * SW_WORDS;
    const RowView row = row_view(p.logits, p.seen, p.seen_rows, r, p.vocab, p.temperature, p.penalty);
    const float smax = row_smax(ws_row);
    Descent d;
    replay(p, ws_row, r, desc, digit, bins, shared, d);
    if (digit == 4) {
        const uint32_t value_bits = (uint32_t)(d.prefix >> SMP_ID_BITS);
        unsigned int* count = reinterpret_cast<unsigned int*>(ws_row + SW_TIE_COUNT + desc);
        int* ties = reinterpret_cast<int*>(ws_row + SW_TIES) + (size_t)desc * SMP_TIES;
        for_each_logit(row, begin, end, SW_THREADS, [&](int i, float l) {
            const float s = l / row.temperature;
            if (ordered_bits(s) == value_bits && composite(s, i) >= d.floor_key) {
                const unsigned int k = atomicAdd(count, 1u);
                if (k < SMP_TIES) ties[k] = i;
            }
        });
        return;
    }
    const int shift = 48 - 8 * digit;
    for (int i = threadIdx.x; i < 256 * SW_COPIES; i += SW_THREADS) hist[i] = 0;
    __syncthreads();
    const u64 hi_mask = shift == 48 ? 0 : (~(u64)0) << (shift + 8);
    for_each_logit(row, begin, end, SW_THREADS, [&](int i, float l) {
        const float s = l / row.temperature;
        const u64 c = composite(s, i);
        if (c >= d.floor_key && (c & hi_mask) == (d.prefix & hi_mask)) {
            const u64 w = MASS ? fixed_mass(s, smax) : 1;
            atomicAdd(&hist[((c >> shift) & 255) * SW_COPIES + (threadIdx.x & (SW_COPIES - 1))], w);
        }
    });
    __syncthreads();
    u64 t = 0;
    for (int k = 0; k < SW_COPIES; ++k) t += hist[threadIdx.x * SW_COPIES + k];     // SW_THREADS is 256: a bin a thread
    if (t) atomicAdd(ws_row + SW_HIST + ((size_t)desc * 4 + digit) * 256 + threadIdx.x, t);
}

template <bool MASS>
__global__ void __launch_bounds__(SMP_THREADS)
split_finish_kernel(SplitPlan p, int desc, int32_t* out) {
    __shared__ u64 hist[256 * SMP_COPIES];
    __shared__ u64 bins[256];
    __shared__ u64 shared[4];
    __shared__ int lds_ties[SMP_TIES];
    __shared__ int lds_tie_count;
    const int r = blockIdx.x;
    u64* ws_row = p.ws + (size_t)r * SW_WORDS;
    const float smax = row_smax(ws_row);
    Descent d;
    replay(p, ws_row, r, desc, 4, bins, shared, d);
    const int n = (int)(unsigned int)ws_row[SW_TIE_COUNT + desc];
    u64 key, incl;
    if (n >= 1 && n <= SMP_TIES) {
        const int* ties = reinterpret_cast<const int*>(ws_row + SW_TIES) + (size_t)desc * SMP_TIES;
        for (int k = threadIdx.x; k < n; k += SMP_THREADS) lds_ties[k] = ties[k];
        __syncthreads();
        const float s = value_of_ordered((uint32_t)(d.prefix >> SMP_ID_BITS));
        const u64 w = MASS ? fixed_mass(s, smax) : 1;
        u64 j = w ? (d.target - d.above) / w : 0;              // so many of the tied candidates lie above c*
        if (j > (u64)(n - 1)) j = (u64)(n - 1);
        for (int k = threadIdx.x; k < n; k += SMP_THREADS) {   // ids rise as keys fall: the j-th smallest id
            const int id = lds_ties[k];
            int rank = 0;
            for (int q = 0; q < n; ++q) rank += lds_ties[q] < id;
            if ((u64)rank == j) {
                shared[0] = d.prefix | (u64)((1 << SMP_ID_BITS) - 1 - id);
                shared[1] = d.above + (j + 1) * w;
            }
        }
        __syncthreads();
        key = shared[0];
        incl = shared[1];
    } else {                                                   // more ties than the list holds: the id digits
        const RowView row = row_view(p.logits, p.seen, p.seen_rows, r, p.vocab, p.temperature, p.penalty);
        key = descend_from<MASS>(row, p.vocab, smax, d.floor_key, d.target, d.prefix, d.above, SMP_ID_BITS - 8, false,
                                 hist, bins, shared, lds_ties, &lds_tie_count, &incl);
    }
    if (threadIdx.x == 0) {
        ws_row[SW_RESULT + 2 * desc] = key;
        ws_row[SW_RESULT + 2 * desc + 1] = incl;
        if (out) out[r] = (1 << SMP_ID_BITS) - 1 - (int)(key & ((1 << SMP_ID_BITS) - 1));
    }
}

extern "C" long ri_sample_split_workspace_bytes(int rows) { return (long)rows * SW_WORDS * (long)sizeof(u64); }

extern "C" int ri_sample_split(int32_t* out, const float* logits, const uint8_t* seen, const int32_t* seen_rows,
                               const float* uniform, void* workspace, int rows, int vocab, float temperature, int top_k,
                               float top_p, float penalty, void* stream) {
    RI_REQUIRE(rows > 0 && rows <= 65535 && vocab > 0 && vocab < (1 << SMP_ID_BITS),
               "sample_split: rows %d, vocab %d (below %d)", rows, vocab, 1 << SMP_ID_BITS);
    RI_REQUIRE(top_k >= 0 && top_p > 0.f && penalty > 0.f, "sample_split: top_k %d, top_p %g, penalty %g", top_k,
               (double)top_p, (double)penalty);
    RI_REQUIRE(temperature > 0.f && uniform != nullptr && workspace != nullptr,
               "sample_split: a positive temperature, uniform draws and a workspace are needed");
    hipStream_t s = (hipStream_t)stream;
    // slices: enough workgroups to fill the machine, none with less than 1,024 tokens
    int slices = (1024 + rows - 1) / rows;
    if (slices > 64) slices = 64;
    if (slices > (vocab + 1023) / 1024) slices = (vocab + 1023) / 1024;
    if (slices < 1) slices = 1;
    const int slice = ((vocab + slices - 1) / slices + 3) / 4 * 4;
    slices = (vocab + slice - 1) / slice;
    SplitPlan p = {logits, seen, seen_rows, uniform, (u64*)workspace, vocab, slice, temperature, top_k, top_p, penalty};
    const long words = (long)rows * SW_WORDS;
    split_fill_kernel<<<(unsigned)((words + 255) / 256), 256, 0, s>>>(p.ws, words);
    const dim3 grid(slices, rows);
    split_max_kernel<<<grid, SW_THREADS, 0, s>>>(p);
    const bool has_k = top_k > 0 && top_k < vocab, has_p = top_p < 1.0f;
    if (has_k) {
        for (int digit = 0; digit <= 4; ++digit) split_pass_kernel<false><<<grid, SW_THREADS, 0, s>>>(p, 0, digit);
        split_finish_kernel<false><<<rows, SMP_THREADS, 0, s>>>(p, 0, nullptr);
    }
    if (has_p) {
        for (int digit = 0; digit <= 4; ++digit) split_pass_kernel<true><<<grid, SW_THREADS, 0, s>>>(p, 1, digit);
        split_finish_kernel<true><<<rows, SMP_THREADS, 0, s>>>(p, 1, nullptr);
    }
    for (int digit = 0; digit <= 4; ++digit) split_pass_kernel<true><<<grid, SW_THREADS, 0, s>>>(p, 2, digit);
    split_finish_kernel<true><<<rows, SMP_THREADS, 0, s>>>(p, 2, out);
    RI_LAUNCH_CHECK("sample_split");
    return 0;
}

// seen[rows[i], tokens[i]] = 1: the history of the repetition penalty as a byte per vocabulary entry.
__global__ void mark_seen_kernel(uint8_t* __restrict__ seen, const int32_t* __restrict__ rows,
                                 const int32_t* __restrict__ tokens, int n, int vocab) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n && tokens[i] >= 0 && tokens[i] < vocab) seen[(size_t)rows[i] * vocab + tokens[i]] = 1;
}

extern "C" int ri_mark_seen(uint8_t* seen, const int32_t* rows, const int32_t* tokens, int n, int vocab, void* stream) {
    RI_REQUIRE(n > 0 && vocab > 0, "mark_seen: n %d, vocab %d", n, vocab);
    mark_seen_kernel<<<(n + 255) / 256, 256, 0, (hipStream_t)stream>>>(seen, rows, tokens, n, vocab);
    RI_LAUNCH_CHECK("mark_seen");
    return 0;
}
