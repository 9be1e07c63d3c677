// Decode-size products for bfloat16: out[M, N] = x[M, K] . w[N, K]^T with M <= 8 rows of x.
// The weights are the traffic: each wavefront streams whole rows of w with 16-byte loads and keeps
// M float32 accumulators, so every weight byte is read once per call.  Optional SwiGLU epilogue for
// the fused gate|up matrix.  Lane l owns k = 8 * (l + 64 * i) ..+8: the order of each row's sum is
// fixed by K alone.
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

template <int MT, bool SWIGLU, typename TO>
__global__ void __launch_bounds__(GV_WAVES * RI_WAVE)
gemv_bf16_kernel(TO* __restrict__ out, const bf16_t* __restrict__ x, const bf16_t* __restrict__ w, int M, int N, int K) {
    const int lane = threadIdx.x & (RI_WAVE - 1);
    const int n = blockIdx.x * GV_WAVES + threadIdx.x / RI_WAVE;
    if (n >= N) return;
    const bf16_t* wr = w + (size_t)n * K;
    const bf16_t* wu = SWIGLU ? w + (size_t)(N + n) * K : nullptr;
    float acc[MT] = {}, accu[MT] = {};
    for (int k = lane * 8; k < K; k += RI_WAVE * 8) {
        float wv[8], uv[8];
        unpack8(*reinterpret_cast<const uint4*>(wr + k), wv);
        if (SWIGLU) unpack8(*reinterpret_cast<const uint4*>(wu + k), uv);
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
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        const float g = wave_sum(acc[m]);
        const float u = SWIGLU ? wave_sum(accu[m]) : 0.f;
        if (lane == 0 && m < M) from_f32(out + (size_t)m * N + n, SWIGLU ? silu_f(g) * u : g);
    }
}

template <int MT, bool SWIGLU>
static void launch_gemv(void* out, int out_dtype, const void* x, const void* w, int m, int n, int k, hipStream_t s) {
    const unsigned grid = (n + GV_WAVES - 1) / GV_WAVES;
    if (out_dtype == RI_F32)
        gemv_bf16_kernel<MT, SWIGLU, float><<<grid, GV_WAVES * RI_WAVE, 0, s>>>((float*)out, (const bf16_t*)x,
                                                                                (const bf16_t*)w, m, n, k);
    else
        gemv_bf16_kernel<MT, SWIGLU, bf16_t><<<grid, GV_WAVES * RI_WAVE, 0, s>>>((bf16_t*)out, (const bf16_t*)x,
                                                                                 (const bf16_t*)w, m, n, k);
}

extern "C" int ri_gemv_bf16(void* out, int out_dtype, const void* x, const void* w, int m, int n, int k, int swiglu,
                            void* stream) {
    RI_REQUIRE(m > 0 && m <= 8, "gemv_bf16: %d rows of x, this kernel takes 1 to 8", m);
    RI_REQUIRE(n > 0 && k > 0 && k % 8 == 0, "gemv_bf16: n %d, k %d (k must be a multiple of 8)", n, k);
    RI_REQUIRE(out_dtype == RI_F32 || out_dtype == RI_BF16, "gemv_bf16: out dtype %d", out_dtype);
    hipStream_t s = (hipStream_t)stream;
    const int mt = m <= 1 ? 1 : m <= 2 ? 2 : m <= 4 ? 4 : 8;
#define RI_GEMV_CASE(MT)                                                       \
    case MT:                                                                   \
        if (swiglu) launch_gemv<MT, true>(out, out_dtype, x, w, m, n, k, s);   \
        else        launch_gemv<MT, false>(out, out_dtype, x, w, m, n, k, s);  \
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
