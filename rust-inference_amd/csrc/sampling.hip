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
// so far, then a scan of its 256 bins from the top.  Masses are 40-bit fixed-point integers, so every
// sum is exact and independent of the order of addition: the same logits and the same r give the
// same token on every run.  Lanes add into 16 copies of the histogram, so that
// the many candidates that share a bin do not queue up on one LDS address.
#include "api.h"
#include "common.h"

#define SMP_THREADS 1024
#define SMP_COPIES 16
#define SMP_ID_BITS 24
#define SMP_FIXED 1099511627776.0f      // 2^40

typedef unsigned long long u64;

__device__ __forceinline__ uint32_t ordered_bits(float f) {
    // larger float <=> larger unsigned; -0.0 and +0.0 compare equal like the floats do
    uint32_t u = __float_as_uint(f == 0.f ? 0.f : f);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

struct RowView {
    const float* logits;
    const uint8_t* seen;     // may be NULL
    float penalty, inv_temperature;
    __device__ __forceinline__ float penalised(int i) const {
        float l = logits[i];
        if (seen && seen[i]) l = l > 0.f ? l / penalty : l * penalty;
        return l;
    }
    __device__ __forceinline__ float scaled(int i) const { return penalised(i) * inv_temperature; }
};

__device__ __forceinline__ u64 composite(float s, int id) {
    return ((u64)ordered_bits(s) << SMP_ID_BITS) | (u64)((1 << SMP_ID_BITS) - 1 - id);
}

// Finds the key c* with  sum_{c > c*} w  <=  target  <  sum_{c >= c*} w  over the candidates with
// key >= floor_key, w = 1 (count) or the fixed-point mass.  Returns c*; *incl = sum_{c >= c*} w.
template <bool MASS>
__device__ u64 descend(const RowView& row, int vocab, float smax, u64 floor_key, u64 target, u64* hist, u64* bins,
                       u64* shared, u64* incl) {
    u64 prefix = 0;            // the bits of c* found so far, in place
    u64 above = 0;             // weight of the candidates above the prefix's bucket
    for (int shift = 48; shift >= 0; shift -= 8) {
        for (int i = threadIdx.x; i < 256 * SMP_COPIES; i += SMP_THREADS) hist[i] = 0;
        __syncthreads();
        const u64 hi_mask = shift == 48 ? 0 : (~(u64)0) << (shift + 8);
        for (int i = threadIdx.x; i < vocab; i += SMP_THREADS) {
            const float s = row.scaled(i);
            const u64 c = composite(s, i);
            if (c >= floor_key && (c & hi_mask) == (prefix & hi_mask)) {
                const u64 w = MASS ? (u64)(expf(s - smax) * SMP_FIXED) : 1;
                atomicAdd(&hist[((c >> shift) & 255) * SMP_COPIES + (threadIdx.x & (SMP_COPIES - 1))], w);
            }
        }
        __syncthreads();
        if (threadIdx.x < 256) {
            u64 t = 0;
            for (int k = 0; k < SMP_COPIES; ++k) t += hist[threadIdx.x * SMP_COPIES + k];
            bins[threadIdx.x] = t;
        }
        __syncthreads();
        if (threadIdx.x == 0) {
            u64 acc = above;
            int b = 255;
            for (; b > 0; --b) {
                if (acc + bins[b] > target) break;
                acc += bins[b];
            }
            shared[0] = acc;                   // weight above bucket b
            shared[1] = (u64)b;
            shared[2] = acc + bins[b];         // weight down to and including bucket b
        }
        __syncthreads();
        above = shared[0];
        prefix |= shared[1] << shift;
        *incl = shared[2];
        __syncthreads();
    }
    return prefix;
}

__global__ void __launch_bounds__(SMP_THREADS)
sample_kernel(int32_t* __restrict__ out, const float* __restrict__ logits, const uint8_t* __restrict__ seen,
              const int32_t* __restrict__ seen_rows, const float* __restrict__ uniform, int vocab, float temperature,
              int top_k, float top_p, float penalty) {
    __shared__ u64 hist[256 * SMP_COPIES];
    __shared__ u64 bins[256];
    __shared__ u64 shared[4];
    __shared__ float fscratch[16];
    __shared__ int iscratch[16];
    RowView row;
    row.logits = logits + (size_t)blockIdx.x * vocab;
    row.seen = (seen && penalty != 1.0f)
                   ? seen + (size_t)(seen_rows ? seen_rows[blockIdx.x] : (int)blockIdx.x) * vocab : nullptr;
    row.penalty = penalty;
    row.inv_temperature = temperature > 0.f ? 1.0f / temperature : 1.0f;

    if (!(temperature > 0.f)) {                            // greedy: the first maximum (src/sampling.rs:131-139)
        float v = -INFINITY;
        int idx = 0x7FFFFFFF;
        for (int i = threadIdx.x; i < vocab; i += SMP_THREADS) {
            const float l = row.penalised(i);
            if (l > v || (l == v && i < idx)) { v = l; idx = i; }
        }
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
    for (int i = threadIdx.x; i < vocab; i += SMP_THREADS) smax = fmaxf(smax, row.scaled(i));
    smax = block_max(smax, fscratch);

    u64 floor_key = 0, incl = 0;
    if (top_k > 0 && top_k < vocab)                       // the k-th candidate of the order closes the kept set
        floor_key = descend<false>(row, vocab, smax, 0, (u64)(top_k - 1), hist, bins, shared, &incl);
    // total mass of the kept set: descend to the very last candidate (target = everything but one unit)
    // would cost seven more passes; one exact integer sum does it
    u64 z = 0;
    for (int i = threadIdx.x; i < vocab; i += SMP_THREADS) {
        const float s = row.scaled(i);
        if (composite(s, i) >= floor_key) z += (u64)(expf(s - smax) * SMP_FIXED);
    }
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
        floor_key = descend<true>(row, vocab, smax, floor_key, want - 1, hist, bins, shared, &incl);
        z = incl;                                          // the kept mass, to be normalised by
    }
    const u64 target = (u64)((double)uniform[blockIdx.x] * (double)z);     // r < 1, so target < z
    const u64 pick = descend<true>(row, vocab, smax, floor_key, target < z ? target : z - 1, hist, bins, shared, &incl);
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
