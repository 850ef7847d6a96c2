// async_gemm<out> for the single-translation-unit harness: same name and argument list as the reference's launcher
// (projects/async_gemm_sparse/sparse_k.cu:45-69; no scale, fp32 or bf16 output), running the producer/consumer LDS
// ring with the role split of core.cu.  D is overwritten.  Shapes the ring cannot take (k not a multiple of the
// 256-byte stage) end the process with a message, as the reference does for shapes off its tile grid (:54-58).
#pragma once
#include "./core.cu"
#include "../../../../rocm_dev_amd/csrc/sg_ring_kernel.h"

template <typename out_dtype>
void async_gemm(const unsigned char* A, const unsigned char* B, out_dtype* D, const int m, const int n, const int k) {
    static_assert(sizeof(out_dtype) == 4 || sizeof(out_dtype) == 2, "fp32 or bf16 output");
    if (k % 256 != 0 || n % 2 != 0 || m > 32) {
        std::cerr << "m, n or k is off the ring's tile grid (m <= 32, n even, k % 256 == 0): " << m << ", " << n << ", " << k
                  << std::endl;
        exit(1);
    }
    sg::RingArgs ra{};
    sg::StreamArgs& a = ra.g;
    a.A = A; a.B = B; a.D = D; a.scale = nullptr;
    a.m = m; a.n = n; a.k = k; a.b_stride = k;
    a.split_k = 1;
    a.waves = CONSUMERS;
    a.n_tiles = (n + 16 * B_LANES - 1) / (16 * B_LANES);
    a.m_tiles = 1;
    a.out_f32 = sizeof(out_dtype) == 4;
    sg::set_reciprocals(a);
    ra.a_producers = A_PRODUCERS;
    ra.b_producers = B_PRODUCERS;
    ra.consumers = CONSUMERS;
    ra.qsize = QSIZE;

    const int mt = m <= 16 ? 1 : 2;
    const int xu = mt == 2 ? 8 : ((m + 3) / 4 <= 1 ? 1 : ((m + 3) / 4 <= 2 ? 2 : 4));
    const size_t slot = (size_t)(B_LANES * 4 + xu) * 1024;
    const size_t flags = ((size_t)(2 * B_LANES * QSIZE + 2) * sizeof(int) + 1023) & ~(size_t)1023;
    const size_t lds = (size_t)QSIZE * slot + 2u * B_LANES * mt * CONSUMERS * 1024 + flags + 4096;
    if (lds > 159 * 1024) {
        std::cerr << "ring of " << lds << " bytes does not fit LDS" << std::endl;
        exit(1);
    }
    int cus = 256;
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, 0) == hipSuccess) cus = prop.multiProcessorCount;
    size_t per_cu = (159 * 1024) / lds;
    per_cu = per_cu < 1 ? 1 : (per_cu > 4 ? 4 : per_cu);
    size_t grid = (size_t)cus * per_cu;
    if (grid > (size_t)a.n_tiles) grid = (size_t)a.n_tiles;
    const unsigned threads = (A_PRODUCERS + B_PRODUCERS + CONSUMERS) * 64;

    auto launch = [&](auto kernel) {
        if (lds > 48 * 1024)
            (void)hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        kernel<<<dim3((unsigned)grid), dim3(threads), lds, 0>>>(ra);
    };
    if (mt == 2) launch(sg::ring_gemm_kernel<2, B_LANES, 8, true>);
    else if (xu == 1) launch(sg::ring_gemm_kernel<1, B_LANES, 1, true>);
    else if (xu == 2) launch(sg::ring_gemm_kernel<1, B_LANES, 2, true>);
    else launch(sg::ring_gemm_kernel<1, B_LANES, 4, true>);
}
