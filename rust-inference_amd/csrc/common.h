// Shared device helpers for the gfx950 kernels: number formats, 64-lane reductions,
// launch checking.  Everything here is written for CDNA4 wavefronts of 64 lanes.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define RI_WAVE 64

// dtype codes of the C interface
enum RiDtype { RI_F32 = 0, RI_BF16 = 1 };

typedef uint16_t bf16_t;   // bfloat16 carried as its bits

// A bfloat16 is the upper half of a 32-bit float (the reference: src/dtype.rs:75-77).
__device__ __forceinline__ float bf16_to_f32(bf16_t b) { return __uint_as_float(((uint32_t)b) << 16); }

// Round to nearest, ties to even; a NaN stays a quiet NaN (the reference: src/dtype.rs:82-89).
// gfx950 converts in hardware (v_cvt_pk_bf16_f32) with exactly this rounding.
__device__ __forceinline__ bf16_t f32_to_bf16(float f) {
    const __bf16 h = (__bf16)f;
    return *reinterpret_cast<const bf16_t*>(&h);
}

// Two floats to two bfloat16 in one 32-bit word, the first in the low half.
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
    typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2_t;
    const bf16x2_t v = {(__bf16)lo, (__bf16)hi};
    return *reinterpret_cast<const uint32_t*>(&v);
}

// Rows of activations in the order the matrix cores take them as a B operand: tiles of 16 rows x 32 columns,
// each 64 lanes x 8 elements (lane l: row l % 16, columns 8 * (l / 16) ..+8 of the tile), the tiles of a row
// tile one after the other, row tile after row tile.  A product or a norm that writes its result this way
// spares the product after it loads that touch sixteen cache lines for half of each: a tile is one kilobyte
// in a row.  k_tiles is the number of column tiles, ceil(columns / 32).  TILED_X: x lies so; TILED_OUT: the
// bfloat16 result is to lie so.
#define TILED_X 1
#define TILED_OUT 2
__device__ __forceinline__ size_t tiled_at(int m, int n, int k_tiles) {
    return (((size_t)(m >> 4) * k_tiles + (n >> 5)) * 64 + (m & 15) + 16 * ((n & 31) >> 3)) * 8 + (n & 7);
}

// One kilobyte of zeros: what a lane reads in place of a fragment piece that lies outside its matrix (rows beyond
// M, columns beyond K), lane l at ri_zero_fragment + 8 * l.  The kernels keep their loads out of branches (the
// compiler counts loads in flight only along code without branches) and choose the address instead; dropping a
// loaded value afterwards works too, but makes the compiler wait for the load where the value is dropped.
static __device__ bf16_t ri_zero_fragment[512];             // (never written; not const, which would move it to another address space and make every such load a flat one)

// A 16-byte load of data that is read once (a weight matrix streaming through): marked non-temporal, so
// that it does not displace what the caches hold to be used again.
__device__ __forceinline__ uint4 load_stream16(const void* p) {
    typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));
    const u32x4_t v = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(p));
    return make_uint4(v.x, v.y, v.z, v.w);
}

__device__ __forceinline__ float to_f32(float v) { return v; }
__device__ __forceinline__ float to_f32(bf16_t v) { return bf16_to_f32(v); }
__device__ __forceinline__ void from_f32(float* p, float v) { *p = v; }
__device__ __forceinline__ void from_f32(bf16_t* p, float v) { *p = f32_to_bf16(v); }

// Sum over the 64 lanes of a wavefront; every lane gets the result.  The order of
// the additions is fixed, so the result does not depend on anything but the inputs.
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int m = RI_WAVE / 2; m > 0; m >>= 1) v += __shfl_xor(v, m, RI_WAVE);
    return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int m = RI_WAVE / 2; m > 0; m >>= 1) v = fmaxf(v, __shfl_xor(v, m, RI_WAVE));
    return v;
}

// Sum over a workgroup of up to 1024 threads (a multiple of 64).  `scratch` is an LDS
// array of at least 16 floats.  All threads get the result.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
    const int lane = threadIdx.x & (RI_WAVE - 1), wave = threadIdx.x / RI_WAVE;
    const int nwaves = (blockDim.x + RI_WAVE - 1) / RI_WAVE;
    v = wave_sum(v);
    __syncthreads();                      // scratch may still be read from an earlier call
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    float total = 0.f;
    for (int w = 0; w < nwaves; ++w) total += scratch[w];
    return total;
}

__device__ __forceinline__ float block_max(float v, float* scratch) {
    const int lane = threadIdx.x & (RI_WAVE - 1), wave = threadIdx.x / RI_WAVE;
    const int nwaves = (blockDim.x + RI_WAVE - 1) / RI_WAVE;
    v = wave_max(v);
    __syncthreads();
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    float total = -INFINITY;
    for (int w = 0; w < nwaves; ++w) total = fmaxf(total, scratch[w]);
    return total;
}

// How a decode-size product is linked to the RMSNorms around it, so that the norms need no kernels
// of their own.  y = W . norm(r) with norm(r) = r * inv * g is computed as inv * (W . (r * g)): the
// producer of r leaves xg = bfloat16(r * g) and partial sums of r^2; the consumer adds the partial
// sums up (always in the same order), and scales its result rows by inv = 1 / sqrt(mean(r^2) + eps).
struct NormLink {
    // consumer side: the rows of x are xg, not yet scaled.  ssq_in: [M][n_in] partial sums of squares over
    // a row of `dim` elements; NULL: x is what it is.
    const float* ssq_in;
    int n_in;
    float eps;
    int dim;
    // producer side: the result is a branch's output.  residual[m][n] += result (float32, in place),
    // xg_out[m][n] = bfloat16(residual * next_gain[n]), ssq_out[m][workgroup] = the workgroup's sum of
    // residual^2; NULL: the result is stored as it is.
    float* residual;
    const float* next_gain;
    bf16_t* xg_out;
    float* ssq_out;
};

// ---- host side: error text of the last refused or failed call (per thread)
void ri_set_error(const char* fmt, ...);

#define RI_REQUIRE(cond, ...)                 \
    do {                                      \
        if (!(cond)) {                        \
            ri_set_error(__VA_ARGS__);        \
            return 1;                         \
        }                                     \
    } while (0)

#define RI_LAUNCH_CHECK(name)                                                   \
    do {                                                                        \
        hipError_t e_ = hipGetLastError();                                      \
        if (e_ != hipSuccess) {                                                 \
            ri_set_error("%s: launch failed: %s", name, hipGetErrorString(e_)); \
            return 2;                                                           \
        }                                                                       \
    } while (0)
