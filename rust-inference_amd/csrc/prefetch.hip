// Pulling a weight matrix toward the compute units ahead of the product that reads it.
//
// A decode step is a chain of products that each stream one matrix from HBM, and every link of the chain
// starts with nothing on its way: the launch, the first loads' trip to memory and the tail of the kernel
// before are time in which HBM delivers nothing.  The matrices themselves depend on nothing, so a second
// chain of these kernels, beside the products on a stream of its own, reads the next product's matrix
// while the current product runs: the bytes land in the memory-side cache (256 MB on MI355X, shared by all
// compute units), from which the product then streams them faster and without the first trip to HBM.
// The loaded values are thrown away; the kernel writes nothing (the store below needs an exact 32-bit
// pattern of xor-ed weights and is there so that the loads cannot be dropped).
#include "api.h"
#include "common.h"

#define PF_THREADS 256
#define PF_UNROLL 8

__global__ void __launch_bounds__(PF_THREADS)
prefetch_kernel(const uint4* __restrict__ p, size_t n16, uint32_t* __restrict__ sink) {
    const size_t stride = (size_t)gridDim.x * PF_THREADS;
    size_t i = (size_t)blockIdx.x * PF_THREADS + threadIdx.x;
    uint32_t acc = 0;
    for (; i + (PF_UNROLL - 1) * stride < n16; i += PF_UNROLL * stride) {
        uint4 v[PF_UNROLL];
#pragma unroll
        for (int u = 0; u < PF_UNROLL; ++u) v[u] = p[i + u * stride];
#pragma unroll
        for (int u = 0; u < PF_UNROLL; ++u) acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
    }
    for (; i < n16; i += stride) {
        const uint4 v = p[i];
        acc ^= v.x ^ v.y ^ v.z ^ v.w;
    }
    if (acc == 0x9E3779B9u && sink != nullptr) *sink = acc;
}

extern "C" int ri_prefetch(const void* data, long bytes, int workgroups, void* sink, void* stream) {
    RI_REQUIRE(data != nullptr && bytes > 0, "prefetch: %ld bytes", bytes);
    RI_REQUIRE((uintptr_t)data % 16 == 0, "prefetch: the data must start on a 16-byte boundary");
    RI_REQUIRE(workgroups > 0 && workgroups <= 65535, "prefetch: %d workgroups", workgroups);
    prefetch_kernel<<<workgroups, PF_THREADS, 0, (hipStream_t)stream>>>((const uint4*)data, (size_t)bytes / 16,
                                                                        (uint32_t*)sink);
    RI_LAUNCH_CHECK("prefetch");
    return 0;
}
