// bench main: "w0, w1, ..., End of warmup, t0, t1, ..., " on stdout, microseconds per launch - the protocol of the
// reference's projects/async_gemm_16x16x64/bench.cu:24-66 (argv = m n k; cache flushed before every timed launch).
// The operands are created once, not once per iteration, and the counts are 100 warm-up + 250 timed launches.
// Every value carries a spare trailing zero because the reference's parser drops the last three characters of the
// stream (bench.py:49).
#include "./../common.cuh"
#include "./src.cu"

#include <cassert>

int main(int argc, char** argv) {
    HIP_CHECK(hipSetDevice(0));
    const int iterations = 250, warmups = 100;
    assert(argc == 4);
    const int m = atoi(argv[1]), n = atoi(argv[2]), k = atoi(argv[3]);

    std::vector<fp8> hA, hB;
    random_host_fp8(hA, (size_t)m * k);
    random_host_fp8(hB, (size_t)n * k);
    fp8 *dA, *dB;
    float* dD;
    tensor_h2d<fp8>(hA.data(), dA, (size_t)m * k);
    tensor_h2d<fp8>(hB.data(), dB, (size_t)n * k);
    HIP_CHECK(hipMalloc(&dD, (size_t)m * n * sizeof(float)));

    hipEvent_t start, stop;
    HIP_CHECK(hipEventCreate(&start));
    HIP_CHECK(hipEventCreate(&stop));
    for (int iter = 0; iter < iterations + warmups; iter++) {
        flush_device_cache();
        HIP_CHECK(hipDeviceSynchronize());
        HIP_CHECK(hipEventRecord(start));
        async_gemm<float>(dA, dB, dD, m, n, k);
        HIP_CHECK(hipEventRecord(stop));
        HIP_CHECK(hipEventSynchronize(stop));
        float t;
        HIP_CHECK(hipEventElapsedTime(&t, start, stop));
        if (iter == warmups) printf("End of warmup, ");
        printf("%.3f0, ", t * 1000);
    }
    return 0;
}
