// Row-wise kernels: embedding gather, fused residual add + RMSNorm, SwiGLU, argmax.
// One workgroup per row; all statistics in float32.
#include <mutex>

#include "api.h"
#include "common.h"

// ------------------------------------------------------------------ embedding
// out[t, :] = table[ids[t], :] (the reference: src/cuda/kernels.cu:90-95), widened to float32
// because the residual stream is kept in 32-bit.
template <typename TW>
__global__ void embed_gather_kernel(float* __restrict__ out, const TW* __restrict__ table,
                                    const int32_t* __restrict__ ids, int dim) {
    const int t = blockIdx.x;
    const TW* row = table + (size_t)ids[t] * dim;
    float* o = out + (size_t)t * dim;
    for (int d = threadIdx.x; d < dim; d += blockDim.x) o[d] = to_f32(row[d]);
}

extern "C" int ri_embed_gather(float* out, const void* table, int table_dtype, const int32_t* ids,
                               int tokens, int dim, void* stream) {
    RI_REQUIRE(tokens > 0 && dim > 0, "embed_gather: tokens %d, dim %d", tokens, dim);
    RI_REQUIRE(table_dtype == RI_F32 || table_dtype == RI_BF16, "embed_gather: table dtype %d", table_dtype);
    hipStream_t s = (hipStream_t)stream;
    if (table_dtype == RI_F32)
        embed_gather_kernel<float><<<tokens, 256, 0, s>>>(out, (const float*)table, ids, dim);
    else
        embed_gather_kernel<bf16_t><<<tokens, 256, 0, s>>>(out, (const bf16_t*)table, ids, dim);
    RI_LAUNCH_CHECK("embed_gather");
    return 0;
}

// ------------------------------------------------------------------ residual add + RMSNorm
// r = residual + pending is the new residual stream; out = r * (1 / sqrt(mean(r^2) + eps)) * gain,
// multiplied in that order (the reference: src/ops/norm.rs:7-10, :25-30, :53-58).  The sum stays in
// float32 and is not rounded before the variance is taken.
template <typename TP, typename TO>
__global__ void add_rmsnorm_kernel(TO* __restrict__ out, float* __restrict__ residual, const TP* __restrict__ pending,
                                   int parts, size_t part_stride, const float* __restrict__ gain, float eps,
                                   const int32_t* __restrict__ rows, int dim) {
    __shared__ float scratch[16];
    const int row = blockIdx.x;
    const size_t src = (size_t)(rows ? rows[row] : row) * dim;
    const bool write_back = rows == nullptr;
    float ss = 0.f;
    for (int d = threadIdx.x; d < dim; d += blockDim.x) {
        float v = residual[src + d];
        if (pending)
            for (int p = 0; p < parts; ++p) v += to_f32(pending[p * part_stride + src + d]);
        if (write_back && pending) residual[src + d] = v;
        ss += v * v;
    }
    const float inv = 1.0f / sqrtf(block_sum(ss, scratch) / (float)dim + eps);
    TO* o = out + (size_t)row * dim;
    for (int d = threadIdx.x; d < dim; d += blockDim.x) {
        float v = residual[src + d];                       // written by this same thread when write_back
        if (pending && !write_back)
            for (int p = 0; p < parts; ++p) v += to_f32(pending[p * part_stride + src + d]);
        from_f32(o + d, v * inv * gain[d]);
    }
}

// The same for rows of up to 8192 elements (a multiple of 4): every thread loads its elements in
// 16-byte pieces up front and keeps them in registers, so the loads of a row are in flight together
// and the row is read once.  The sum of squares is taken per thread over its own elements, then over
// the workgroup in a fixed order.
__device__ __forceinline__ float4 load4(const float* p) { return *reinterpret_cast<const float4*>(p); }
__device__ __forceinline__ float4 load4(const bf16_t* p) {
    const uint2 w = *reinterpret_cast<const uint2*>(p);
    return make_float4(__uint_as_float(w.x << 16), __uint_as_float(w.x & 0xFFFF0000u), __uint_as_float(w.y << 16),
                       __uint_as_float(w.y & 0xFFFF0000u));
}
__device__ __forceinline__ void store4(float* p, float4 v) { *reinterpret_cast<float4*>(p) = v; }
__device__ __forceinline__ void store4(bf16_t* p, float4 v) {
    uint2 w;
    w.x = (uint32_t)f32_to_bf16(v.x) | ((uint32_t)f32_to_bf16(v.y) << 16);
    w.y = (uint32_t)f32_to_bf16(v.z) | ((uint32_t)f32_to_bf16(v.w) << 16);
    *reinterpret_cast<uint2*>(p) = w;
}

// Every load is issued whatever the indices are, from an address pulled back inside the row, and a value from
// outside is dropped afterwards: a load inside a branch or inside a loop of unknown length makes the compiler
// wait for each one before the next is asked for (a norm over four parts of a split product took sixteen
// trips to memory in turn that way).  PQ parts are fetched together; the sum is taken in the order of the parts.
template <typename TP, typename TO, int VPT, int PQ>
__global__ void __launch_bounds__(256)
add_rmsnorm_vec_kernel(TO* __restrict__ out, float* __restrict__ residual, const TP* __restrict__ pending,
                       int parts, size_t part_stride, const float* __restrict__ gain, float eps,
                       const int32_t* __restrict__ rows, int dim, int tiled) {
    __shared__ float scratch[16];
    const int row = blockIdx.x;
    const size_t src = (size_t)(rows ? rows[row] : row) * dim;
    const bool write_back = rows == nullptr && pending != nullptr;
    float4 v[VPT], g[VPT];
    int at[VPT];
    bool ok[VPT];
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        const int d = (i * 256 + threadIdx.x) * 4;
        ok[i] = d < dim;
        at[i] = ok[i] ? d : 0;
        v[i] = load4(residual + src + at[i]);
        g[i] = load4(gain + at[i]);
    }
    if (pending) {
        for (int q0 = 0; q0 < parts; q0 += PQ) {                 // the parts of a split product, always in this order
            float4 p[PQ][VPT];
#pragma unroll
            for (int j = 0; j < PQ; ++j) {
                const size_t base = (size_t)min(q0 + j, parts - 1) * part_stride + src;
#pragma unroll
                for (int i = 0; i < VPT; ++i) p[j][i] = load4(pending + base + at[i]);
            }
#pragma unroll
            for (int j = 0; j < PQ; ++j) {
                const bool live = q0 + j < parts;
#pragma unroll
                for (int i = 0; i < VPT; ++i) {
                    v[i].x = live ? v[i].x + p[j][i].x : v[i].x;
                    v[i].y = live ? v[i].y + p[j][i].y : v[i].y;
                    v[i].z = live ? v[i].z + p[j][i].z : v[i].z;
                    v[i].w = live ? v[i].w + p[j][i].w : v[i].w;
                }
            }
        }
    }
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        if (ok[i]) {
            if (write_back) store4(residual + src + at[i], v[i]);
            ss += v[i].x * v[i].x + v[i].y * v[i].y + v[i].z * v[i].z + v[i].w * v[i].w;
        }
    }
    const float inv = 1.0f / sqrtf(block_sum(ss, scratch) / (float)dim + eps);
    TO* o = out + (size_t)row * dim;
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        if (ok[i])                                           // four columns of one chunk of eight either way
            store4(tiled ? out + tiled_at(row, at[i], (dim + 31) / 32) : o + at[i],
                   make_float4(v[i].x * inv * g[i].x, v[i].y * inv * g[i].y, v[i].z * inv * g[i].z,
                               v[i].w * inv * g[i].w));
    }
}

template <typename TP, typename TO, int VPT>
static void launch_add_rmsnorm_vec(TO* out, float* residual, const TP* pending, int parts, size_t ps, const float* gain,
                                   float eps, const int32_t* rows, int n_rows, int dim, int tiled, hipStream_t s) {
    if (parts > 1)
        add_rmsnorm_vec_kernel<TP, TO, VPT, 4><<<n_rows, 256, 0, s>>>(out, residual, pending, parts, ps, gain, eps, rows, dim, tiled);
    else
        add_rmsnorm_vec_kernel<TP, TO, VPT, 1><<<n_rows, 256, 0, s>>>(out, residual, pending, parts, ps, gain, eps, rows, dim, tiled);
}

template <typename TP, typename TO>
static void launch_add_rmsnorm_typed(TO* out, float* residual, const TP* pending, int parts, size_t ps,
                                     const float* gain, float eps, const int32_t* rows, int n_rows, int dim,
                                     int tiled, hipStream_t s) {
    if (dim % 4 == 0 && dim <= 1024)
        launch_add_rmsnorm_vec<TP, TO, 1>(out, residual, pending, parts, ps, gain, eps, rows, n_rows, dim, tiled, s);
    else if (dim % 4 == 0 && dim <= 2048)
        launch_add_rmsnorm_vec<TP, TO, 2>(out, residual, pending, parts, ps, gain, eps, rows, n_rows, dim, tiled, s);
    else if (dim % 4 == 0 && dim <= 4096)
        launch_add_rmsnorm_vec<TP, TO, 4>(out, residual, pending, parts, ps, gain, eps, rows, n_rows, dim, tiled, s);
    else if (dim % 4 == 0 && dim <= 8192)
        launch_add_rmsnorm_vec<TP, TO, 8>(out, residual, pending, parts, ps, gain, eps, rows, n_rows, dim, tiled, s);
    else
        add_rmsnorm_kernel<TP, TO><<<n_rows, 256, 0, s>>>(out, residual, pending, parts, ps, gain, eps, rows, dim);
}

template <typename TP>
static void launch_add_rmsnorm(void* out, int out_dtype, float* residual, const TP* pending, int parts, size_t ps,
                               const float* gain, float eps, const int32_t* rows, int n_rows, int dim, int tiled,
                               hipStream_t s) {
    if (out_dtype == RI_F32)
        launch_add_rmsnorm_typed<TP, float>((float*)out, residual, pending, parts, ps, gain, eps, rows, n_rows, dim, 0, s);
    else
        launch_add_rmsnorm_typed<TP, bf16_t>((bf16_t*)out, residual, pending, parts, ps, gain, eps, rows, n_rows, dim,
                                             tiled, s);
}

extern "C" int ri_add_rmsnorm(void* out, int out_dtype, float* residual, const void* pending, int pending_dtype,
                              int parts, int total_rows, const float* gain, float eps, const int32_t* rows, int n_rows,
                              int dim, int tiled, void* stream) {
    RI_REQUIRE(n_rows > 0 && dim > 0, "add_rmsnorm: rows %d, dim %d", n_rows, dim);
    RI_REQUIRE(parts >= 1 && parts <= 64 && total_rows >= 1, "add_rmsnorm: %d parts of %d rows", parts, total_rows);
    const size_t ps = (size_t)total_rows * dim;
    RI_REQUIRE(out_dtype == RI_F32 || out_dtype == RI_BF16, "add_rmsnorm: out dtype %d", out_dtype);
    RI_REQUIRE(pending_dtype == RI_F32 || pending_dtype == RI_BF16, "add_rmsnorm: pending dtype %d", pending_dtype);
    RI_REQUIRE(!tiled || (out_dtype == RI_BF16 && dim % 4 == 0 && dim <= 8192 && n_rows <= 64),
               "add_rmsnorm: tiled rows are bfloat16, at most 64, of a multiple of 4 up to 8192 elements (%d of %d)",
               n_rows, dim);
    hipStream_t s = (hipStream_t)stream;
    if (pending_dtype == RI_F32)
        launch_add_rmsnorm<float>(out, out_dtype, residual, (const float*)pending, parts, ps, gain, eps, rows, n_rows,
                                  dim, tiled, s);
    else
        launch_add_rmsnorm<bf16_t>(out, out_dtype, residual, (const bf16_t*)pending, parts, ps, gain, eps, rows, n_rows,
                                   dim, tiled, s);
    RI_LAUNCH_CHECK("add_rmsnorm");
    return 0;
}

// (out may be residual itself when rows is NULL: every element is read and then written by one thread)
template <typename TP>
__global__ void add_rows_kernel(float* out, const float* residual,
                                const TP* __restrict__ pending, const int32_t* __restrict__ rows, int dim) {
    const int row = blockIdx.x;
    const size_t src = (size_t)(rows ? rows[row] : row) * dim;
    for (int d = threadIdx.x; d < dim; d += blockDim.x) {
        float v = residual[src + d];
        if (pending) v += to_f32(pending[src + d]);
        out[(size_t)row * dim + d] = v;
    }
}

extern "C" int ri_add_rows(float* out, const float* residual, const void* pending, int pending_dtype,
                           const int32_t* rows, int n_rows, int dim, void* stream) {
    RI_REQUIRE(n_rows > 0 && dim > 0, "add_rows: rows %d, dim %d", n_rows, dim);
    hipStream_t s = (hipStream_t)stream;
    if (pending_dtype == RI_F32)
        add_rows_kernel<float><<<n_rows, 256, 0, s>>>(out, residual, (const float*)pending, rows, dim);
    else if (pending_dtype == RI_BF16)
        add_rows_kernel<bf16_t><<<n_rows, 256, 0, s>>>(out, residual, (const bf16_t*)pending, rows, dim);
    else
        RI_REQUIRE(false, "add_rows: pending dtype %d", pending_dtype);
    RI_LAUNCH_CHECK("add_rows");
    return 0;
}

// ------------------------------------------------------------------ a norm that a product was to finish
// out[m, :] = bfloat16(xg[m, :] * inv[m]) with inv[m] = 1 / sqrt(sum_j ssq[m, j] / dim + eps): the rows of a
// norm that was left to the product after it (see NormLink in common.h), for a reader that cannot take the
// norm over.  The partial sums are added in a fixed order.  xg lies in rows or in the matrix cores' order.
__global__ void finish_norm_kernel(bf16_t* __restrict__ out, const bf16_t* __restrict__ xg, const float* __restrict__ ssq,
                                   int n_in, float eps, int dim, int x_tiled) {
    __shared__ float scratch[16];
    const int m = blockIdx.x;
    float part = 0.f;
    for (int j = threadIdx.x; j < n_in; j += blockDim.x) part += ssq[(size_t)m * n_in + j];
    const float inv = 1.0f / sqrtf(block_sum(part, scratch) / (float)dim + eps);
    const int k_tiles = (dim + 31) / 32;
    for (int d = threadIdx.x; d < dim; d += blockDim.x) {
        const bf16_t v = x_tiled ? xg[tiled_at(m, d, k_tiles)] : xg[(size_t)m * dim + d];
        out[(size_t)m * dim + d] = f32_to_bf16(bf16_to_f32(v) * inv);
    }
}

extern "C" int ri_finish_norm(void* out, const void* xg, const float* ssq, int n_in, float eps, int dim, int rows,
                              int x_tiled, void* stream) {
    RI_REQUIRE(rows > 0 && dim > 0 && n_in > 0, "finish_norm: rows %d, dim %d, %d partial sums", rows, dim, n_in);
    RI_REQUIRE(!x_tiled || rows <= 64, "finish_norm: %d rows in the matrix cores' order (64 at most)", rows);
    finish_norm_kernel<<<rows, 256, 0, (hipStream_t)stream>>>((bf16_t*)out, (const bf16_t*)xg, ssq, n_in, eps, dim, x_tiled);
    RI_LAUNCH_CHECK("finish_norm");
    return 0;
}

// ------------------------------------------------------------------ SwiGLU
// silu(z) = z / (1 + exp(-z)) (the reference: src/ops/elementwise.rs:9-12); gate = silu(gate) * up.
__device__ __forceinline__ float silu(float z) { return z / (1.0f + expf(-z)); }

template <typename T>
__global__ void swiglu_kernel(T* __restrict__ out, const T* __restrict__ y, int inter, long total) {
    const long e = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= total) return;
    const long t = e / inter;
    const int i = (int)(e - t * inter);
    const T* row = y + t * 2 * inter;
    from_f32(out + e, silu(to_f32(row[i])) * to_f32(row[inter + i]));
}

// Eight bfloat16 elements per thread with 16-byte loads and stores, for inter a multiple of 8.
// tiled: the result lies in the matrix cores' order (at most 64 rows): eight columns from a multiple of 8 on are
// neighbours there too.
__global__ void swiglu_bf16x8_kernel(bf16_t* __restrict__ out, const bf16_t* __restrict__ y, int inter8, long total8,
                                     int tiled) {
    const long e = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= total8) return;
    const long t = e / inter8;
    const int i = (int)(e - t * inter8);
    const uint4 g = *reinterpret_cast<const uint4*>(y + (t * 2 * inter8 + i) * 8);
    const uint4 u = *reinterpret_cast<const uint4*>(y + (t * 2 * inter8 + inter8 + i) * 8);
    const uint32_t gw[4] = {g.x, g.y, g.z, g.w}, uw[4] = {u.x, u.y, u.z, u.w};
    uint32_t o[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const float a = silu(__uint_as_float(gw[k] << 16)) * __uint_as_float(uw[k] << 16);
        const float b = silu(__uint_as_float(gw[k] & 0xFFFF0000u)) * __uint_as_float(uw[k] & 0xFFFF0000u);
        o[k] = pack_bf16x2(a, b);
    }
    const size_t at = tiled ? tiled_at((int)t, i * 8, (inter8 * 8 + 31) / 32) : (size_t)e * 8;
    *reinterpret_cast<uint4*>(out + at) = make_uint4(o[0], o[1], o[2], o[3]);
}

extern "C" int ri_swiglu(void* out, const void* y, int dtype, int tokens, int inter, int tiled, void* stream) {
    RI_REQUIRE(tokens > 0 && inter > 0, "swiglu: tokens %d, inter %d", tokens, inter);
    RI_REQUIRE(!tiled || (dtype == RI_BF16 && inter % 8 == 0 && tokens <= 64),
               "swiglu: a tiled result is bfloat16, at most 64 rows and a multiple of 8 wide");
    const long total = (long)tokens * inter;
    RI_REQUIRE((total + 255) / 256 <= 2147483647L, "swiglu: %ld elements exceed one launch", total);
    const unsigned grid = (unsigned)((total + 255) / 256);
    hipStream_t s = (hipStream_t)stream;
    if (dtype == RI_F32)
        swiglu_kernel<float><<<grid, 256, 0, s>>>((float*)out, (const float*)y, inter, total);
    else if (dtype == RI_BF16 && inter % 8 == 0)
        swiglu_bf16x8_kernel<<<(unsigned)((total / 8 + 255) / 256), 256, 0, s>>>((bf16_t*)out, (const bf16_t*)y,
                                                                                  inter / 8, total / 8, tiled);
    else if (dtype == RI_BF16)
        swiglu_kernel<bf16_t><<<grid, 256, 0, s>>>((bf16_t*)out, (const bf16_t*)y, inter, total);
    else
        RI_REQUIRE(false, "swiglu: dtype %d", dtype);
    RI_LAUNCH_CHECK("swiglu");
    return 0;
}

// ------------------------------------------------------------------ bias
// x[t, i] += bias[i] in place, the sum in float32 (for parts with biased products; the reference's family
// has none: src/models/qwen3.rs:60-69).
template <typename T>
__global__ void add_bias_kernel(T* __restrict__ x, const float* __restrict__ bias, int dim) {
    T* row = x + (size_t)blockIdx.x * dim;
    for (int d = threadIdx.x; d < dim; d += blockDim.x) from_f32(row + d, to_f32(row[d]) + bias[d]);
}

extern "C" int ri_add_bias(void* x, int dtype, const float* bias, int rows, int dim, void* stream) {
    RI_REQUIRE(rows > 0 && dim > 0, "add_bias: rows %d, dim %d", rows, dim);
    RI_REQUIRE(dtype == RI_F32 || dtype == RI_BF16, "add_bias: dtype %d", dtype);
    hipStream_t s = (hipStream_t)stream;
    if (dtype == RI_F32) add_bias_kernel<float><<<rows, 256, 0, s>>>((float*)x, bias, dim);
    else add_bias_kernel<bf16_t><<<rows, 256, 0, s>>>((bf16_t*)x, bias, dim);
    RI_LAUNCH_CHECK("add_bias");
    return 0;
}

// ------------------------------------------------------------------ argmax
// First index of the row maximum: of equal values the lower index wins
// (the reference: src/ops/reduce.rs:18-25, src/cuda/kernels.cu:182, :189).  A NaN never wins.
__device__ __forceinline__ void better(float& v, int& i, float ov, int oi) {
    if (ov > v || (ov == v && oi < i)) { v = ov; i = oi; }
}

// Stage one: every workgroup takes a slice of the row and writes its best (value, index);
// stage two: one workgroup per row picks the best of the slices.  Slices are in index order and
// equal values keep the lower index, so the result is the first maximum of the row.
#define ARGMAX_SLICES 64

__device__ __forceinline__ void block_best(float& v, int& idx, float* sv, int* si) {
    for (int m = RI_WAVE / 2; m > 0; m >>= 1) {
        float ov = __shfl_xor(v, m, RI_WAVE);
        int oi = __shfl_xor(idx, m, RI_WAVE);
        better(v, idx, ov, oi);
    }
    const int lane = threadIdx.x & (RI_WAVE - 1), wave = threadIdx.x / RI_WAVE;
    if (lane == 0) { sv[wave] = v; si[wave] = idx; }
    __syncthreads();
    if (threadIdx.x == 0)
        for (int w = 1; w < (int)(blockDim.x / RI_WAVE); ++w) better(v, idx, sv[w], si[w]);
}

__global__ void argmax_slices_kernel(float* __restrict__ part_v, int32_t* __restrict__ part_i,
                                     const float* __restrict__ logits, int vocab, int per_slice) {
    __shared__ float sv[16];
    __shared__ int si[16];
    const float* row = logits + (size_t)blockIdx.y * vocab;
    const int begin = blockIdx.x * per_slice, end = min(vocab, begin + per_slice);
    float v = -INFINITY;
    int idx = 0x7FFFFFFF;
    for (int i = begin + threadIdx.x; i < end; i += blockDim.x) better(v, idx, row[i], i);
    block_best(v, idx, sv, si);
    if (threadIdx.x == 0) {
        part_v[blockIdx.y * ARGMAX_SLICES + blockIdx.x] = v;
        part_i[blockIdx.y * ARGMAX_SLICES + blockIdx.x] = idx;
    }
}

__global__ void argmax_pick_kernel(int32_t* __restrict__ ids, const float* __restrict__ part_v,
                                   const int32_t* __restrict__ part_i) {
    float v = part_v[blockIdx.x * ARGMAX_SLICES + threadIdx.x];
    int idx = part_i[blockIdx.x * ARGMAX_SLICES + threadIdx.x];
    for (int m = RI_WAVE / 2; m > 0; m >>= 1) {
        float ov = __shfl_xor(v, m, RI_WAVE);
        int oi = __shfl_xor(idx, m, RI_WAVE);
        better(v, idx, ov, oi);
    }
    if (threadIdx.x == 0) ids[blockIdx.x] = idx == 0x7FFFFFFF ? 0 : idx;
}

extern "C" int ri_argmax_workspace_bytes(int rows) { return rows * ARGMAX_SLICES * 8; }

extern "C" int ri_argmax(int32_t* ids, const float* logits, void* workspace, int rows, int vocab, void* stream) {
    RI_REQUIRE(rows > 0 && rows <= 65535 && vocab > 0, "argmax: rows %d, vocab %d", rows, vocab);
    float* part_v = (float*)workspace;
    int32_t* part_i = (int32_t*)(part_v + (size_t)rows * ARGMAX_SLICES);
    const int per_slice = (vocab + ARGMAX_SLICES - 1) / ARGMAX_SLICES;
    hipStream_t s = (hipStream_t)stream;
    argmax_slices_kernel<<<dim3(ARGMAX_SLICES, rows), 256, 0, s>>>(part_v, part_i, logits, vocab, per_slice);
    argmax_pick_kernel<<<rows, ARGMAX_SLICES, 0, s>>>(ids, part_v, part_i);
    RI_LAUNCH_CHECK("argmax");
    return 0;
}

// ---- the same argmax for callers that cannot allocate device memory
// The (value, index) pairs of stage one lie in a file-scope device array instead of a workspace the caller
// brings.  In host code the array's name stands for the symbol, not for its device address: the address is
// asked for once per device (each GPU holds its own copy at its own address) and only that pointer is used
// afterwards.  Every call on a GPU shares that GPU's array, so calls that overlap on one GPU race.
#define ARGMAX_STATIC_MAX_ROWS 1024
#define ARGMAX_STATIC_MAX_DEVICES 64
static __device__ __align__(256) unsigned char scratch[ARGMAX_STATIC_MAX_ROWS * ARGMAX_SLICES * 8];

static void* g_scratch_of_device[ARGMAX_STATIC_MAX_DEVICES];      // per device: the array's address there
static std::mutex g_scratch_mutex;

// The address of `scratch` on the current device (looked up at the first call on that device).
static int scratch_of_current_device(void** out) {
    int device = -1;
    hipError_t e = hipGetDevice(&device);
    RI_REQUIRE(e == hipSuccess, "argmax_static: hipGetDevice: %s", hipGetErrorString(e));
    RI_REQUIRE(device >= 0 && device < ARGMAX_STATIC_MAX_DEVICES, "argmax_static: device %d is beyond the %d this library "
               "keeps an address for", device, ARGMAX_STATIC_MAX_DEVICES);
    std::lock_guard<std::mutex> hold(g_scratch_mutex);
    if (g_scratch_of_device[device] == nullptr) {
        void* ptr = nullptr;
        e = hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch));
        RI_REQUIRE(e == hipSuccess && ptr != nullptr, "argmax_static: hipGetSymbolAddress on device %d: %s", device,
                   hipGetErrorString(e));
        g_scratch_of_device[device] = ptr;
    }
    *out = g_scratch_of_device[device];
    return 0;
}

extern "C" int ri_argmax_static_max_rows(void) { return ARGMAX_STATIC_MAX_ROWS; }

extern "C" int ri_argmax_static(int32_t* ids, const float* logits, int rows, int vocab, void* stream) {
    RI_REQUIRE(rows > 0 && vocab > 0, "argmax_static: rows %d, vocab %d", rows, vocab);
    RI_REQUIRE(rows <= ARGMAX_STATIC_MAX_ROWS, "argmax_static: %d rows, the built-in scratch holds %d at most "
               "(use ri_argmax with a workspace of the caller's)", rows, ARGMAX_STATIC_MAX_ROWS);
    void* ptr = nullptr;
    if (int rc = scratch_of_current_device(&ptr)) return rc;
    // stage one writes every (value, index) pair that stage two reads: nothing has to start at zero
    return ri_argmax(ids, logits, ptr, rows, vocab, stream);
}
