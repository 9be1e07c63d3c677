// out[M, N] = x[M, K] . w[N, K]^T in true 32-bit arithmetic: float32 multiply-adds on the vector
// units, no matrix-core or reduced-precision mode.  w may be stored as bfloat16 and is widened
// exactly.  Every output element is one sequential sum over k = 0..K-1, so a row's result does
// not depend on how many other rows are in the call.  This is the correctness path; it is tiled
// through LDS but not tuned.
#include "api.h"
#include "common.h"

#define GT_M 64
#define GT_N 64
#define GT_K 16

template <typename TW>
__global__ void __launch_bounds__(256)
gemm_f32_kernel(float* __restrict__ out, const float* __restrict__ x, const TW* __restrict__ w, int M, int N, int K) {
    __shared__ float xs[GT_K][GT_M + 4];
    __shared__ float ws[GT_K][GT_N + 4];
    const int tid = threadIdx.x, tx = tid % 16, ty = tid / 16;
    const int m0 = blockIdx.y * GT_M, n0 = blockIdx.x * GT_N;
    float acc[4][4] = {};
    for (int k0 = 0; k0 < K; k0 += GT_K) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int e = tid + i * 256, r = e / GT_K, kk = e % GT_K;
            const int k = k0 + kk;
            xs[kk][r] = (m0 + r < M && k < K) ? x[(size_t)(m0 + r) * K + k] : 0.f;
            ws[kk][r] = (n0 + r < N && k < K) ? to_f32(w[(size_t)(n0 + r) * K + k]) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < GT_K; ++kk) {
            float a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) { a[i] = xs[kk][ty * 4 + i]; b[i] = ws[kk][tx * 4 + i]; }
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int m = m0 + ty * 4 + i, n = n0 + tx * 4 + j;
            if (m < M && n < N) out[(size_t)m * N + n] = acc[i][j];
        }
}

extern "C" int ri_gemm_f32(float* out, const float* x, const void* w, int w_dtype, int m, int n, int k, void* stream) {
    RI_REQUIRE(m > 0 && n > 0 && k > 0, "gemm_f32: m %d, n %d, k %d", m, n, k);
    RI_REQUIRE(w_dtype == RI_F32 || w_dtype == RI_BF16, "gemm_f32: weight dtype %d", w_dtype);
    dim3 grid((n + GT_N - 1) / GT_N, (m + GT_M - 1) / GT_M);
    RI_REQUIRE(grid.y <= 65535, "gemm_f32: %d rows exceed one launch", m);
    hipStream_t s = (hipStream_t)stream;
    if (w_dtype == RI_F32)
        gemm_f32_kernel<float><<<grid, 256, 0, s>>>(out, x, (const float*)w, m, n, k);
    else
        gemm_f32_kernel<bf16_t><<<grid, 256, 0, s>>>(out, x, (const bf16_t*)w, m, n, k);
    RI_LAUNCH_CHECK("gemm_f32");
    return 0;
}
