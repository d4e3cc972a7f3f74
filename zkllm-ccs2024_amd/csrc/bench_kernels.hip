// Measurement helpers: the VALU integer multiply-add peak that the Montgomery kernels are priced
// against, and a plain copy kernel of known size used to scale the profiler's byte counters.
#include <cstring>
#include "field.hpp"
#include "rt.hpp"
#include "../../include/zkllm_hip.h"

using namespace zk;

// 16 independent 32x32+64 multiply-add chains per lane (one v_mad_u64_u32 each step), no memory
// traffic in the loop.  Total multiply-adds = threads * 16 * iters.
__global__ void __launch_bounds__(256) k_mad_peak(unsigned long long* __restrict__ out, uint32_t seed, uint32_t iters) {
    const uint32_t t = blockIdx.x * 256 + threadIdx.x;
    uint32_t a = seed * 2654435761u + t, b = (seed ^ t) | 1u;
    unsigned long long acc[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = t + i;
    for (uint32_t it = 0; it < iters; ++it) {
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[i] = (unsigned long long)a * (uint32_t)(b + i) + acc[i];
        a += (uint32_t)acc[0];      // keeps the multiplicands loop-variant
    }
    unsigned long long s = 0;
#pragma unroll
    for (int i = 0; i < 16; ++i) s ^= acc[i];
    if (s == 0x1234567ull) out[t] = s;    // practically never taken; defeats dead-code elimination
}

__global__ void __launch_bounds__(256) k_copy16(uint4* __restrict__ dst, const uint4* __restrict__ src, size_t n16) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n16) dst[i] = src[i];
}

extern "C" {

// Runs the multiply-add peak kernel and reports multiply-adds per second.
int zk_bench_mad_peak(uint32_t blocks, uint32_t iters, double* mad_per_s_host, void* stv) {
    hipStream_t st = (hipStream_t)stv;
    ZK_ARG(blocks >= 1 && iters >= 1, "zk_bench_mad_peak: empty launch");
    Scratch out((size_t)blocks * 256 * 8, st);
    if (out.rc) return out.rc;
    hipEvent_t e0, e1;
    ZK_HIP(hipEventCreate(&e0));
    ZK_HIP(hipEventCreate(&e1));
    hipLaunchKernelGGL(k_mad_peak, dim3(blocks), dim3(256), 0, st, out.as<unsigned long long>(), 1u, iters / 8 + 1);   // warm-up
    ZK_HIP(hipEventRecord(e0, st));
    hipLaunchKernelGGL(k_mad_peak, dim3(blocks), dim3(256), 0, st, out.as<unsigned long long>(), 2u, iters);
    ZK_HIP(hipEventRecord(e1, st));
    ZK_HIP(hipEventSynchronize(e1));
    float ms = 0;
    ZK_HIP(hipEventElapsedTime(&ms, e0, e1));
    ZK_HIP(hipEventDestroy(e0));
    ZK_HIP(hipEventDestroy(e1));
    *mad_per_s_host = (double)blocks * 256.0 * 16.0 * iters / (ms * 1e-3);
    return 0;
}
// dst = src, bytes must be a multiple of 16 (reads `bytes`, writes `bytes`)
int zk_bench_copy(void* dst, const void* src, size_t bytes, void* st) {
    ZK_ARG(bytes % 16 == 0, "zk_bench_copy: bytes must be a multiple of 16");
    const size_t n16 = bytes / 16;
    if (n16) {
        hipLaunchKernelGGL(k_copy16, dim3(cdiv(n16, 256)), dim3(256), 0, (hipStream_t)st, (uint4*)dst, (const uint4*)src, n16);
        ZK_LAUNCH_CHECK();
    }
    return 0;
}

}  // extern "C"
