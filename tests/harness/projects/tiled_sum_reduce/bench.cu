// bench main: "w0, w1, ..., End of warmup, t0, t1, ..., " on stdout, microseconds per launch - the protocol of the
// reference's projects/tiled_sum_reduce/bench.cu:28-69 (argv = b m n; cache flushed before every timed launch).
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
    const int b = atoi(argv[1]), m = atoi(argv[2]), n = atoi(argv[3]);
    const size_t mn = (size_t)m * n;

    std::vector<float> hA, hB;
    random_host_f32(hA, (size_t)b * mn);
    random_host_f32(hB, (size_t)b * mn);
    float *dA, *dB, *dD;
    tensor_h2d<float>(hA.data(), dA, (size_t)b * mn);
    tensor_h2d<float>(hB.data(), dB, (size_t)b * mn);
    HIP_CHECK(hipMalloc(&dD, mn * sizeof(float)));

    hipEvent_t start, stop;
    HIP_CHECK(hipEventCreate(&start));
    HIP_CHECK(hipEventCreate(&stop));
    for (int iter = 0; iter < iterations + warmups; iter++) {
        flush_device_cache();
        HIP_CHECK(hipDeviceSynchronize());
        HIP_CHECK(hipEventRecord(start));
        tiled_sum_reduce(dA, dB, dD, b, m, n);
        HIP_CHECK(hipEventRecord(stop));
        HIP_CHECK(hipEventSynchronize(stop));
        float t;
        HIP_CHECK(hipEventElapsedTime(&t, start, stop));
        if (iter == warmups) printf("End of warmup, ");
        printf("%.3f0, ", t * 1000);
    }
    return 0;
}
