// Harness utilities for the single-translation-unit test / bench mains (the role of the
// reference's projects/common.cuh: HIP_CHECK :29-41, alloc + copy :45-60, random tensors :86-105).
// Test infrastructure: the host GEMM oracle is included from the repository's oracle/ directory.
#pragma once

#include <hip/hip_runtime.h>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "../../../oracle/sg_oracle.c"

using fp8 = unsigned char;   // OCP E4M3 storage
using bf16 = uint16_t;       // bf16 bits

#ifndef HIP_CHECK
#define HIP_CHECK(error)                                                                                  \
    if ((error) != hipSuccess) {                                                                          \
        fprintf(stderr, "Hip error: '%s'(%d) at %s:%d\n", hipGetErrorString(error), error, __FILE__, __LINE__); \
        exit(EXIT_FAILURE);                                                                               \
    }
#endif

template <typename T>
void tensor_h2d(const T* host, T*& dev, size_t n) {
    HIP_CHECK(hipMalloc(&dev, n * sizeof(T)));
    HIP_CHECK(hipMemcpy(dev, host, n * sizeof(T), hipMemcpyHostToDevice));
}

// U[-1, 1) rounded to E4M3 with saturation, as the reference's random_host_tensor<fp8> (common.cuh:97-105)
inline void random_host_fp8(std::vector<fp8>& x, size_t n) {
    x.resize(n);
    for (size_t i = 0; i < n; i++) {
        const float y = static_cast<float>(rand()) / static_cast<float>(RAND_MAX);
        x[i] = orc_e4m3_encode(2 * (y - 0.5f));
    }
}
inline float random_host_scale() { return static_cast<float>(rand()) / static_cast<float>(RAND_MAX) - 0.5f; }

// U[-1, 1) floats, as the reference's random_host_tensor<float> (common.cuh:86-95)
inline void random_host_f32(std::vector<float>& x, size_t n) {
    x.resize(n);
    for (size_t i = 0; i < n; i++) x[i] = 2 * (static_cast<float>(rand()) / static_cast<float>(RAND_MAX) - 0.5f);
}

// The role of the reference's flush_device_cache (common.cuh:141-158: a kernel that sweeps an L2-sized buffer):
// here a fill of 640 MB, more than twice the 256 MB memory-side cache, so the next launch finds nothing of its
// operands in any cache.  The buffer is allocated once.
inline void flush_device_cache() {
    static void* sweep = nullptr;
    const size_t bytes = (size_t)640 << 20;
    if (!sweep) HIP_CHECK(hipMalloc(&sweep, bytes));
    HIP_CHECK(hipMemsetAsync(sweep, 0, bytes, 0));
}
