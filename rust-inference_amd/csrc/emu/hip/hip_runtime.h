// A stand-in for <hip/hip_runtime.h> that runs the kernels of this library on the CPU, thread by thread, so
// that their memory accesses can be checked against guarded buffers without a GPU (kernels/build.py:
// build_emulated).  It is no general HIP emulator: it knows what these kernels use.  A workgroup's threads are
// coroutines of one host thread; __syncthreads and every instruction that moves data between the lanes of a
// wavefront (shuffles, votes, lane reads, lane swaps, the matrix-core product) make the threads meet, so the
// values the kernels compute are the real ones, page numbers read from tables included, and a load issued from
// a wrong address touches the guard page behind its buffer.  Workgroups run one after the other.
#pragma once
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#include <type_traits>

#define RI_EMULATED 1
#define __global__
#define __device__
#define __host__
#define __forceinline__ inline __attribute__((always_inline))
#define __shared__ static
#define __launch_bounds__(...)
#define __align__(n) __attribute__((aligned(n)))
#define HIP_SYMBOL(x) x

struct dim3 {
    unsigned x, y, z;
    constexpr dim3(unsigned x_ = 1, unsigned y_ = 1, unsigned z_ = 1) : x(x_), y(y_), z(z_) {}
};
struct uint2 { unsigned x, y; };
struct alignas(16) uint4 { unsigned x, y, z, w; };
struct alignas(16) float4 { float x, y, z, w; };
static inline uint4 make_uint4(unsigned x, unsigned y, unsigned z, unsigned w) { return uint4{x, y, z, w}; }
static inline float4 make_float4(float x, float y, float z, float w) { return float4{x, y, z, w}; }

typedef void* hipStream_t;
enum hipError_t { hipSuccess = 0, hipErrorNoDevice = 100 };
enum hipDeviceAttribute_t { hipDeviceAttributeMultiprocessorCount = 63 };
static inline hipError_t hipGetLastError() { return hipSuccess; }
static inline const char* hipGetErrorString(hipError_t) { return "no error (emulated)"; }
// There is no device, unless the environment names a number of compute units (RI_EMU_COMPUTE_UNITS): then
// there is one, of that size, so that the rules which size launches by the machine choose on a few thousand keys
// what they choose on an MI355X from tens of thousands on.
static inline int emu_compute_units() {
    const char* s = getenv("RI_EMU_COMPUTE_UNITS");
    return s ? atoi(s) : 0;
}
static inline hipError_t hipGetDevice(int* dev) {
    if (emu_compute_units() <= 0) return hipErrorNoDevice;
    *dev = 0;
    return hipSuccess;
}
static inline hipError_t hipDeviceGetAttribute(int* value, hipDeviceAttribute_t, int) {
    if (emu_compute_units() <= 0) return hipErrorNoDevice;
    *value = emu_compute_units();
    return hipSuccess;
}
template <class T>
static inline hipError_t hipGetSymbolAddress(void** p, T& symbol) { *p = (void*)&symbol; return hipSuccess; }
static inline hipError_t hipMalloc(void**, size_t) { return hipErrorNoDevice; }

namespace emu {
struct Thread {
    dim3 idx;
    int linear, lane, wave;
};
extern Thread* self;                       // the emulated thread that is running
extern dim3 block_idx, block_dim, grid_dim;
void* dyn_shared();                        // the workgroup's dynamic shared memory
void barrier();                            // all live threads of the workgroup meet
// Every live lane of the calling thread's wavefront hands in `bytes` bytes; returns when all have, with all
// 64 lanes' values in `all` (lane l at all + l * bytes; lanes that do not exist or have ended: zeros) and the
// lanes that handed one in as a bit mask.
uint64_t wave_gather(const void* mine, size_t bytes, void* all);
struct Body { virtual void run() = 0; virtual ~Body() {} };
void launch(const char* name, dim3 grid, dim3 block, size_t dyn_shared_bytes, Body& body);
template <class F>
struct BodyOf : Body {
    F f;
    explicit BodyOf(F&& g) : f(static_cast<F&&>(g)) {}
    void run() override { f(); }
};
template <class F>
void launch_fn(const char* name, dim3 grid, dim3 block, size_t shmem, F&& f) {
    BodyOf<F> b(static_cast<F&&>(f));
    launch(name, grid, block, shmem, b);
}
}  // namespace emu

#define threadIdx (emu::self->idx)
#define blockIdx emu::block_idx
#define blockDim emu::block_dim
#define gridDim emu::grid_dim
// kernel<<<grid, block, shared, stream>>>(args) is rewritten by the build into this
#define RI_EMU_LAUNCH(kernel, grid, block, shmem, stream, ...) \
    emu::launch_fn(#kernel, dim3(grid), dim3(block), (size_t)(shmem), [&]() { kernel(__VA_ARGS__); })

static inline void __syncthreads() { emu::barrier(); }

// ---- bits and numbers
static inline float __uint_as_float(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static inline uint32_t __float_as_uint(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float __int_as_float(int32_t u) { float f; memcpy(&f, &u, 4); return f; }
static inline int32_t __float_as_int(float f) { int32_t u; memcpy(&u, &f, 4); return u; }
static inline int __clz(int x) { return x == 0 ? 32 : __builtin_clz((unsigned)x); }
static inline int __clzll(long long x) { return x == 0 ? 64 : __builtin_clzll((unsigned long long)x); }
static inline float rsqrtf(float x) { return 1.0f / sqrtf(x); }
template <class A, class B>
static inline typename std::common_type<A, B>::type min(A a, B b) {
    typedef typename std::common_type<A, B>::type T;
    return (T)b < (T)a ? (T)b : (T)a;
}
template <class A, class B>
static inline typename std::common_type<A, B>::type max(A a, B b) {
    typedef typename std::common_type<A, B>::type T;
    return (T)a < (T)b ? (T)b : (T)a;
}
#define __builtin_amdgcn_exp2f(x) exp2f(x)
#define __builtin_amdgcn_sched_barrier(x) ((void)0)

// ---- atomics: one host thread runs everything
template <class T> static inline T atomicAdd(T* p, T v) { T o = *p; *p = o + v; return o; }
template <class T> static inline T atomicMax(T* p, T v) { T o = *p; if (v > o) *p = v; return o; }

// ---- between the lanes of a wavefront
template <class T>
static inline T __shfl_xor(T v, int mask, int width = 64) {
    T all[64];
    emu::wave_gather(&v, sizeof(T), all);
    const int lane = emu::self->lane, other = lane ^ mask;
    return (other / width == lane / width && other < 64) ? all[other] : v;
}
template <class T>
static inline T __shfl_down(T v, unsigned delta, int width = 64) {
    T all[64];
    emu::wave_gather(&v, sizeof(T), all);
    const int lane = emu::self->lane, other = lane + (int)delta;
    return (other / width == lane / width && other < 64) ? all[other] : v;
}
template <class T>
static inline T __shfl(T v, int src, int width = 64) {
    T all[64];
    emu::wave_gather(&v, sizeof(T), all);
    const int lane = emu::self->lane, other = (lane / width) * width + (src % width);
    return all[other];
}
static inline int emu_readlane(int v, int lane) {
    int all[64];
    emu::wave_gather(&v, sizeof(int), all);
    return all[lane & 63];
}
static inline int emu_readfirstlane(int v) {
    int all[64];
    const uint64_t live = emu::wave_gather(&v, sizeof(int), all);
    return all[__builtin_ctzll(live)];
}
#define __builtin_amdgcn_readlane(v, l) emu_readlane((int)(v), (l))
#define __builtin_amdgcn_readfirstlane(v) emu_readfirstlane((int)(v))
// The lanes of a wavefront run in step on the GPU, so what one lane has written to LDS another lane reads
// after it without more than this barrier for the compiler; here the lanes are threads that must really meet.
static inline void emu_wave_barrier() {
    char mine = 0, all[64];
    emu::wave_gather(&mine, 1, all);
}
#define __builtin_amdgcn_wave_barrier() emu_wave_barrier()
static inline int __any(int pred) {
    int all[64];
    const uint64_t live = emu::wave_gather(&pred, sizeof(int), all);
    for (int l = 0; l < 64; ++l)
        if (((live >> l) & 1) && all[l]) return 1;
    return 0;
}
static inline unsigned long long __ballot(int pred) {
    int all[64];
    const uint64_t live = emu::wave_gather(&pred, sizeof(int), all);
    unsigned long long m = 0;
    for (int l = 0; l < 64; ++l)
        if (((live >> l) & 1) && all[l]) m |= 1ull << l;
    return m;
}

// v_permlane32_swap: the upper 32 lanes of the first operand change places with the lower 32 lanes of the
// second; v_permlane16_swap: the odd rows of 16 lanes of the first with the even rows of the second.  Both
// return {first, second} after the exchange.
typedef unsigned emu_u32x2 __attribute__((ext_vector_type(2)));
static inline emu_u32x2 emu_permlane_swap(unsigned a, unsigned b, int row) {
    unsigned in[2] = {a, b}, all[64][2];
    emu::wave_gather(in, sizeof(in), all);
    const int lane = emu::self->lane;
    const bool odd = (lane / row) & 1;
    emu_u32x2 out;
    out.x = odd ? all[lane - row][1] : a;          // an odd row of the first takes the even row of the second
    out.y = odd ? b : all[lane + row][0];          // an even row of the second takes the odd row of the first
    return out;
}
#define __builtin_amdgcn_permlane32_swap(a, b, fi, bc) emu_permlane_swap((a), (b), 32)
#define __builtin_amdgcn_permlane16_swap(a, b, fi, bc) emu_permlane_swap((a), (b), 16)

// MFMA 16x16x32 bfloat16: D[16 x 16] = A[16 x 32] . B[32 x 16] + C.  Lane l holds A[l % 16][8 * (l / 16) ..+8],
// B[8 * (l / 16) ..+8][l % 16] and D[4 * (l / 16) + i][l % 16] for i = 0..3.
template <class V8, class V4>
static inline V4 emu_mfma_16x16x32_bf16(V8 a, V8 b, V4 c) {
    struct Pair { uint16_t a[8], b[8]; } mine, all[64];
    memcpy(mine.a, &a, 16);
    memcpy(mine.b, &b, 16);
    emu::wave_gather(&mine, sizeof(mine), all);
    const int lane = emu::self->lane, col = lane & 15, rows = 4 * (lane >> 4);
    V4 d = c;
    for (int i = 0; i < 4; ++i) {
        float sum = 0.f;
        for (int k = 0; k < 32; ++k) {
            const float av = __uint_as_float((uint32_t)all[(rows + i) + 16 * (k >> 3)].a[k & 7] << 16);
            const float bv = __uint_as_float((uint32_t)all[col + 16 * (k >> 3)].b[k & 7] << 16);
            sum += av * bv;
        }
        d[i] = c[i] + sum;
    }
    return d;
}
#define __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, x, y, z) emu_mfma_16x16x32_bf16((a), (b), (c))
