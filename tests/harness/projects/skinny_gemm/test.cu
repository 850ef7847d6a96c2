// test main: GPU result against the host loop on rand() inputs, one JSON object on stdout
// {"max_delta": ..., "total_delta": ...} - the protocol of the reference's
// projects/skinny_gemm/test.cu:43-114 (argv = m n k, srand(0), scale in U[-0.5, 0.5)).
#include "./../common.cuh"
#include "./skinny_gemm_caller.cu"

#include <cassert>

int main(int argc, char** argv) {
    HIP_CHECK(hipSetDevice(0));
    srand(0);
    assert(argc == 4);
    const int m = atoi(argv[1]), n = atoi(argv[2]), k = atoi(argv[3]);

    std::vector<fp8> hA, hB;
    random_host_fp8(hA, (size_t)m * k);
    random_host_fp8(hB, (size_t)n * k);
    const float hScale = random_host_scale();

    std::vector<bf16> host_ref((size_t)m * n), host_result((size_t)m * n);
    orc_gemm_omp(hA.data(), hB.data(), host_ref.data(), hScale, m, n, k, k);

    fp8 *dA, *dB;
    bf16* dD;
    float* dScale;
    tensor_h2d<fp8>(hA.data(), dA, (size_t)m * k);
    tensor_h2d<fp8>(hB.data(), dB, (size_t)n * k);
    tensor_h2d<float>(&hScale, dScale, 1);
    HIP_CHECK(hipMalloc(&dD, (size_t)m * n * sizeof(bf16)));
    HIP_CHECK(hipMemset(dD, 0xff, (size_t)m * n * sizeof(bf16)));   // NaN pattern: D must be overwritten

    HIP_CHECK(hipDeviceSynchronize());
    const int rc = skinny_gemm_fastpath(dA, dB, dD, dScale, m, n, k);
    HIP_CHECK(hipDeviceSynchronize());
    if (rc != 0) {
        std::cout << "{\"max_delta\": nan, \"total_delta\": nan, \"return_code\": " << rc << "}";
        return 0;
    }
    HIP_CHECK(hipMemcpy(host_result.data(), dD, (size_t)m * n * sizeof(bf16), hipMemcpyDeviceToHost));

    float max_delta, total_delta;
    orc_delta_metrics_bf16(host_result.data(), host_ref.data(), (size_t)m * n, &max_delta, &total_delta);
    std::cout << "{\"max_delta\": " << max_delta << ", \"total_delta\": " << total_delta << "}";
    return 0;
}
