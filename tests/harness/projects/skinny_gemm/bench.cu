// bench main: "w0, w1, ..., End of warmup, t0, t1, ..., " on stdout, one value per event pair
// in microseconds per GEMM - the protocol of the reference's projects/skinny_gemm/bench.cu:38-75
// (100 warm-up + 250 timed iterations, BATCH = 4 back-to-back launches on 4 different weight
// matrices per event pair).  Weights rotate through enough copies that more than 512 MB pass
// between two uses of a matrix.  Every value carries a spare trailing zero because the
// reference's parser drops the last three characters of the stream (bench.py:49).
#include "./../common.cuh"
#include "./skinny_gemm_caller.cu"

#include <cassert>

#define MUL 4
#define BATCH 4

int main(int argc, char** argv) {
    HIP_CHECK(hipSetDevice(0));
    const int warmups = (MUL * 100) / BATCH;
    const int iterations = (MUL * 250) / BATCH;
    assert(argc == 4);
    const int m = atoi(argv[1]), n = atoi(argv[2]), k = atoi(argv[3]);

    size_t copies = (size_t)(640e6 / ((double)n * k)) + 1;
    copies = ((copies + BATCH - 1) / BATCH) * BATCH;
    std::vector<fp8> hA, hB;
    random_host_fp8(hA, (size_t)m * k);
    random_host_fp8(hB, (size_t)n * k);
    fp8 *dA, *dB;
    bf16* dD;
    float* dScale;
    const float hScale = random_host_scale();
    tensor_h2d<fp8>(hA.data(), dA, (size_t)m * k);
    HIP_CHECK(hipMalloc(&dB, copies * (size_t)n * k));
    for (size_t c = 0; c < copies; c++)
        HIP_CHECK(hipMemcpy(dB + c * (size_t)n * k, hB.data(), (size_t)n * k, hipMemcpyHostToDevice));
    tensor_h2d<float>(&hScale, dScale, 1);
    HIP_CHECK(hipMalloc(&dD, (size_t)m * n * sizeof(bf16)));

    hipEvent_t start, stop;
    HIP_CHECK(hipEventCreate(&start));
    HIP_CHECK(hipEventCreate(&stop));
    size_t next = 0;
    for (int iter = 0; iter < iterations + warmups; iter++) {
        HIP_CHECK(hipDeviceSynchronize());
        HIP_CHECK(hipEventRecord(start));
        for (int i = 0; i < BATCH; i++) {
            skinny_gemm_fastpath(dA, dB + next * (size_t)n * k, dD, dScale, m, n, k);
            next = (next + 1) % copies;
        }
        HIP_CHECK(hipEventRecord(stop));
        HIP_CHECK(hipEventSynchronize(stop));
        float t;
        HIP_CHECK(hipEventElapsedTime(&t, start, stop));
        if (iter == warmups) printf("End of warmup, ");
        printf("%.3f0, ", t * 1000 / BATCH);
    }
    return 0;
}
