// Decode-size products for bfloat16: out[M, N] = x[M, K] . w[N, K]^T with M <= 8 rows of x.
// The weights are the traffic: each wavefront streams a row of w (or a fixed share of one) with
// 16-byte loads and keeps M float32 accumulators, so every weight byte is read once per call.
// Optional SwiGLU epilogue for the fused gate|up matrix.  Lane l owns k = 8 * (l + 64 * i) ..+8: the
// order of each row's sum is fixed by K and N alone.
#include "api.h"
#include "common.h"

#define GV_WAVES 4          // wavefronts per workgroup, one output row (or gate/up pair) each per turn

__device__ __forceinline__ void unpack8(const uint4 v, float* o) {
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        o[2 * i] = __uint_as_float(w[i] << 16);
        o[2 * i + 1] = __uint_as_float(w[i] & 0xFFFF0000u);
    }
}

__device__ __forceinline__ float silu_f(float z) { return z / (1.0f + expf(-z)); }

// KS wavefronts share a row, each taking a contiguous 1/KS of K (a multiple of 512 elements, so that
// every lane's 16-byte pieces stay aligned and the split depends on K alone); their sums are added
// through LDS in wavefront order.  More wavefronts in flight per byte: it pays when the matrix has few
// rows or long ones.
// Partial sums of squares a thread fetches ahead of the weights.  A row has as many as the product before
// wrote workgroups (up to 4,096 at Qwen3-8B sizes); what is not fetched ahead is fetched after the stream, one
// more trip to memory at the end of every workgroup.  Sixteen a thread cover 4,096 (decode at batch 1: +1.5%);
// where a row has 1,024 at most, four do, and the registers of more cost a small model 1.5%.
#define GV_PRE_FEW 4
#define GV_PRE_MANY 16
// Steps of 512 k whose loads a wavefront with one row of x asks for together (see the loop below), for the
// plain product and for the gate|up pair.
#ifndef GV_AHEAD_PLAIN
#define GV_AHEAD_PLAIN 4
#endif
#ifndef GV_AHEAD_GATED
#define GV_AHEAD_GATED 4
#endif

template <int MT, bool SWIGLU, typename TO, int KS, int GV_PRE>
__global__ void __launch_bounds__(GV_WAVES * RI_WAVE)
gemv_bf16_kernel(TO* __restrict__ out, const bf16_t* __restrict__ x, const bf16_t* __restrict__ w, int M, int N, int K,
                 NormLink link) {
    __shared__ float red[2][GV_WAVES][MT];
    __shared__ float scratch[16];
    __shared__ float sq_lds[GV_WAVES][MT];
    const int lane = threadIdx.x & (RI_WAVE - 1);
    const int wave = threadIdx.x / RI_WAVE;
    const int n = blockIdx.x * (GV_WAVES / KS) + wave / KS;
    const int part = wave % KS;
    const int slice = ((K + KS - 1) / KS + 511) / 512 * 512;
    const int k_begin = part * slice, k_end = min(K, k_begin + slice);
    const bool row_ok = n < N;
    const bf16_t* wr = w + (size_t)(row_ok ? n : 0) * K;
    const bf16_t* wu = SWIGLU ? w + (size_t)(N + (row_ok ? n : 0)) * K : nullptr;

    // Loads whose values are wanted only after the weights have streamed are issued here, so that their
    // latency hides behind the stream: a row's partial sums of squares (up to GV_PRE per thread; more are
    // fetched afterwards), and the element of the residual stream and the gain that the result meets.
    float pre[MT][GV_PRE];
    if (link.ssq_in) {
#pragma unroll
        for (int m = 0; m < MT; ++m)
#pragma unroll
            for (int j = 0; j < GV_PRE; ++j) {
                const int p = threadIdx.x + j * GV_WAVES * RI_WAVE;
                pre[m][j] = (m < M && p < link.n_in) ? link.ssq_in[(size_t)m * link.n_in + p] : 0.f;
            }
    }
    float res_pre[MT], gain_pre = 0.f;
    if (link.residual && row_ok && part == 0) {
        gain_pre = link.next_gain[n];
#pragma unroll
        for (int m = 0; m < MT; ++m) res_pre[m] = m < M ? link.residual[(size_t)m * N + n] : 0.f;
    }

    float acc[MT] = {}, accu[MT] = {};
    if (row_ok) {
        // GV_AHEAD steps of 512 k at a time with all their loads asked for before the first is used: a wavefront
        // then has GV_AHEAD (twice that with the up row) kilobytes of weights in flight instead of one.  The
        // compiler keeps loads in flight only across code without branches, so the steps of a round are
        // unrolled by hand and the rest of K, if any, follows one step at a time.  The same sums in the same order.
        constexpr int GV_AHEAD = MT == 1 ? (SWIGLU ? GV_AHEAD_GATED : GV_AHEAD_PLAIN) : (MT == 2 ? 2 : 1);
        int k = k_begin + lane * 8;
        if (GV_AHEAD > 1) {
            for (; k + (GV_AHEAD - 1) * RI_WAVE * 8 < k_end; k += GV_AHEAD * RI_WAVE * 8) {
                uint4 wq[GV_AHEAD], uq[GV_AHEAD], xq[GV_AHEAD][MT];
#pragma unroll
                for (int a = 0; a < GV_AHEAD; ++a) {
                    wq[a] = load_stream16(wr + k + a * RI_WAVE * 8);
                    if (SWIGLU) uq[a] = load_stream16(wu + k + a * RI_WAVE * 8);
#pragma unroll
                    for (int m = 0; m < MT; ++m)
                        xq[a][m] = *reinterpret_cast<const uint4*>(x + (size_t)(m < M ? m : 0) * K + k + a * RI_WAVE * 8);
                }
#pragma unroll
                for (int a = 0; a < GV_AHEAD; ++a) {
                    float wv[8], uv[8];
                    unpack8(wq[a], wv);
                    if (SWIGLU) unpack8(uq[a], uv);
#pragma unroll
                    for (int m = 0; m < MT; ++m) {       // (rows beyond M repeat row 0 and are never stored: no branch here)
                        float xv[8];
                        unpack8(xq[a][m], xv);
#pragma unroll
                        for (int e = 0; e < 8; ++e) {
                            acc[m] = fmaf(xv[e], wv[e], acc[m]);
                            if (SWIGLU) accu[m] = fmaf(xv[e], uv[e], accu[m]);
                        }
                    }
                }
            }
        }
        for (; k < k_end; k += RI_WAVE * 8) {
            float wv[8], uv[8];
            unpack8(load_stream16(wr + k), wv);
            if (SWIGLU) unpack8(load_stream16(wu + k), uv);
#pragma unroll
            for (int m = 0; m < MT; ++m) {
                if (m < M) {
                    float xv[8];
                    unpack8(*reinterpret_cast<const uint4*>(x + (size_t)m * K + k), xv);
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        acc[m] = fmaf(xv[e], wv[e], acc[m]);
                        if (SWIGLU) accu[m] = fmaf(xv[e], uv[e], accu[m]);
                    }
                }
            }
        }
    }
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        acc[m] = wave_sum(acc[m]);
        if (SWIGLU) accu[m] = wave_sum(accu[m]);
    }
    if (KS > 1) {
        if (lane == 0) {
#pragma unroll
            for (int m = 0; m < MT; ++m) {
                red[0][wave][m] = acc[m];
                if (SWIGLU) red[1][wave][m] = accu[m];
            }
        }
        __syncthreads();
        if (part == 0) {
#pragma unroll
            for (int m = 0; m < MT; ++m) {
                acc[m] = 0.f;
                accu[m] = 0.f;
                for (int p = 0; p < KS; ++p) {
                    acc[m] += red[0][wave + p][m];
                    if (SWIGLU) accu[m] += red[1][wave + p][m];
                }
            }
        }
    }
    // rows of x that still want their 1 / rms: add up the partial sums of squares, always in this order
    float inv[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m) inv[m] = 1.0f;
    if (link.ssq_in) {
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            if (m < M) {
                float sq = 0.f;
#pragma unroll
                for (int j = 0; j < GV_PRE; ++j) sq += pre[m][j];
                for (int p = threadIdx.x + GV_PRE * GV_WAVES * RI_WAVE; p < link.n_in; p += GV_WAVES * RI_WAVE)
                    sq += link.ssq_in[(size_t)m * link.n_in + p];
                inv[m] = 1.0f / sqrtf(block_sum(sq, scratch) / (float)link.dim + link.eps);
            }
        }
    }
    const bool writer = lane == 0 && row_ok && part == 0;
    float sq[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        sq[m] = 0.f;
        if (writer && m < M) {
            float v = SWIGLU ? silu_f(acc[m] * inv[m]) * (accu[m] * inv[m]) : acc[m] * inv[m];
            if (link.residual) {
                const size_t at = (size_t)m * N + n;
                v += res_pre[m];
                link.residual[at] = v;                      // this element belongs to this wavefront alone
                link.xg_out[at] = f32_to_bf16(v * gain_pre);
                sq[m] = v * v;
            } else {
                from_f32(out + (size_t)m * N + n, v);
            }
        }
    }
    if (link.residual) {                                    // the workgroup's share of every row's sum of squares
        if (lane == 0) {
#pragma unroll
            for (int m = 0; m < MT; ++m) sq_lds[wave][m] = sq[m];
        }
        __syncthreads();
        if (threadIdx.x < MT && threadIdx.x < M) {
            float total = 0.f;
            for (int wv = 0; wv < GV_WAVES; ++wv) total += sq_lds[wv][threadIdx.x];
            link.ssq_out[(size_t)threadIdx.x * gridDim.x + blockIdx.x] = total;
        }
    }
}

// How many wavefronts share a row: measured on MI355X with one row of x (decode at batch 1).  A wavefront that
// asks for four steps' loads at a time streams a row of 4,096 elements and more fastest alone (Qwen3-8B sizes,
// tok/s at batch 1 with four, two and one wavefront on the rows of 12,288 elements: 308.5, 312.0, 313.4; with two
// on the gate|up rows of 4,096: 303.0); shorter rows have no such rounds, and there two wavefronts a row keep
// more loads in flight for a small matrix.
static int gemv_k_split(int n, int k) {
    if (k >= 4096) return 1;
    if ((long)n * k <= 4096L * 4096L) return 2;
    return 1;
}

static unsigned gemv_grid(int n, int k) {
    const int rows_per_wg = GV_WAVES / gemv_k_split(n, k);
    return (unsigned)((n + rows_per_wg - 1) / rows_per_wg);
}

template <int MT, bool SWIGLU, int KS>
static void launch_gemv_ks(void* out, int out_dtype, const void* x, const void* w, int m, int n, int k,
                           const NormLink& link, hipStream_t s) {
    const unsigned grid = gemv_grid(n, k);
    // one row of x whose norm is still to finish, with more partial sums than four a thread cover
    const bool many = MT == 1 && link.ssq_in && link.n_in > GV_PRE_FEW * GV_WAVES * RI_WAVE;
    if (out_dtype == RI_F32) {
        if (many) gemv_bf16_kernel<MT, SWIGLU, float, KS, MT == 1 ? GV_PRE_MANY : GV_PRE_FEW><<<grid, GV_WAVES * RI_WAVE, 0, s>>>(
            (float*)out, (const bf16_t*)x, (const bf16_t*)w, m, n, k, link);
        else gemv_bf16_kernel<MT, SWIGLU, float, KS, GV_PRE_FEW><<<grid, GV_WAVES * RI_WAVE, 0, s>>>(
            (float*)out, (const bf16_t*)x, (const bf16_t*)w, m, n, k, link);
    } else {
        if (many) gemv_bf16_kernel<MT, SWIGLU, bf16_t, KS, MT == 1 ? GV_PRE_MANY : GV_PRE_FEW><<<grid, GV_WAVES * RI_WAVE, 0, s>>>(
            (bf16_t*)out, (const bf16_t*)x, (const bf16_t*)w, m, n, k, link);
        else gemv_bf16_kernel<MT, SWIGLU, bf16_t, KS, GV_PRE_FEW><<<grid, GV_WAVES * RI_WAVE, 0, s>>>(
            (bf16_t*)out, (const bf16_t*)x, (const bf16_t*)w, m, n, k, link);
    }
}

template <int MT, bool SWIGLU>
static void launch_gemv(void* out, int out_dtype, const void* x, const void* w, int m, int n, int k,
                        const NormLink& link, hipStream_t s) {
    switch (gemv_k_split(n, k)) {
        case 4: launch_gemv_ks<MT, SWIGLU, 4>(out, out_dtype, x, w, m, n, k, link, s); break;
        case 2: launch_gemv_ks<MT, SWIGLU, 2>(out, out_dtype, x, w, m, n, k, link, s); break;
        default: launch_gemv_ks<MT, SWIGLU, 1>(out, out_dtype, x, w, m, n, k, link, s); break;
    }
}

static int gemv_run(void* out, int out_dtype, const void* x, const void* w, int m, int n, int k, int swiglu,
                    const NormLink& link, hipStream_t s) {
    const int mt = m <= 1 ? 1 : m <= 2 ? 2 : m <= 4 ? 4 : 8;
#define RI_GEMV_CASE(MT)                                                             \
    case MT:                                                                         \
        if (swiglu) launch_gemv<MT, true>(out, out_dtype, x, w, m, n, k, link, s);   \
        else        launch_gemv<MT, false>(out, out_dtype, x, w, m, n, k, link, s);  \
        break;
    switch (mt) {
        RI_GEMV_CASE(1)
        RI_GEMV_CASE(2)
        RI_GEMV_CASE(4)
        RI_GEMV_CASE(8)
    }
#undef RI_GEMV_CASE
    RI_LAUNCH_CHECK("gemv_bf16");
    return 0;
}

extern "C" int ri_gemv_bf16(void* out, int out_dtype, const void* x, const void* w, int m, int n, int k, int swiglu,
                            void* stream) {
    RI_REQUIRE(m > 0 && m <= 8, "gemv_bf16: %d rows of x, this kernel takes 1 to 8", m);
    RI_REQUIRE(n > 0 && k > 0 && k % 8 == 0, "gemv_bf16: n %d, k %d (k must be a multiple of 8)", n, k);
    RI_REQUIRE(out_dtype == RI_F32 || out_dtype == RI_BF16, "gemv_bf16: out dtype %d", out_dtype);
    NormLink link = {};
    return gemv_run(out, out_dtype, x, w, m, n, k, swiglu, link, (hipStream_t)stream);
}

// Number of workgroups (and so of partial sums of squares per row) of a linked product with n output columns.
extern "C" int ri_gemv_bf16_partials(int n, int k) { return (int)gemv_grid(n, k); }

extern "C" int ri_gemv_bf16_linked(void* out, int out_dtype, const void* x, const void* w, int m, int n, int k,
                                   int swiglu, const float* ssq_in, int n_in, float eps, int dim, float* residual,
                                   const float* next_gain, void* xg_out, float* ssq_out, void* stream) {
    RI_REQUIRE(m > 0 && m <= 8, "gemv_bf16_linked: %d rows of x, this kernel takes 1 to 8", m);
    RI_REQUIRE(n > 0 && k > 0 && k % 8 == 0, "gemv_bf16_linked: n %d, k %d (k must be a multiple of 8)", n, k);
    RI_REQUIRE(out_dtype == RI_F32 || out_dtype == RI_BF16, "gemv_bf16_linked: out dtype %d", out_dtype);
    RI_REQUIRE(!ssq_in || (n_in > 0 && dim > 0), "gemv_bf16_linked: %d partial sums over %d elements", n_in, dim);
    RI_REQUIRE(!residual || (next_gain && xg_out && ssq_out && !swiglu),
               "gemv_bf16_linked: a product that feeds the residual stream needs the next gain and both outputs");
    RI_REQUIRE(residual || out, "gemv_bf16_linked: no output");
    NormLink link = {ssq_in, n_in, eps, dim, residual, next_gain, (bf16_t*)xg_out, ssq_out};
    return gemv_run(out, out_dtype, x, w, m, n, k, swiglu, link, (hipStream_t)stream);
}
