// test main: GPU result against the host loop on rand() inputs, one JSON object on stdout
// {"max_delta": ..., "total_delta": ...} - the protocol of the reference's projects/async_gemm_16x16x64/test.cu:41-96
// (argv = m n k, fp32 output, no scale).  The host loop is the oracle's restatement of test.cu:7-38.
#include "./../common.cuh"
#include "./src.cu"

#include <cassert>
#include <cmath>

#define OUTD float

int main(int argc, char** argv) {
    HIP_CHECK(hipSetDevice(0));
    assert(argc == 4);
    const int m = atoi(argv[1]), n = atoi(argv[2]), k = atoi(argv[3]);

    std::vector<fp8> hA, hB;
    random_host_fp8(hA, (size_t)m * k);
    random_host_fp8(hB, (size_t)n * k);
    std::vector<OUTD> host_ref((size_t)m * n), host_result((size_t)m * n);
    orc_gemm_f32(hA.data(), hB.data(), host_ref.data(), 1.0f, m, n, k, k);

    fp8 *dA, *dB;
    OUTD* dD;
    tensor_h2d<fp8>(hA.data(), dA, (size_t)m * k);
    tensor_h2d<fp8>(hB.data(), dB, (size_t)n * k);
    HIP_CHECK(hipMalloc(&dD, (size_t)m * n * sizeof(OUTD)));
    HIP_CHECK(hipMemset(dD, 0xff, (size_t)m * n * sizeof(OUTD)));   // NaN pattern: D must be overwritten

    HIP_CHECK(hipDeviceSynchronize());
    async_gemm<OUTD>(dA, dB, dD, m, n, k);
    HIP_CHECK(hipDeviceSynchronize());
    HIP_CHECK(hipMemcpy(host_result.data(), dD, (size_t)m * n * sizeof(OUTD), hipMemcpyDeviceToHost));

    float sum_delta = 0.0f, max_delta = 0.0f;
    for (size_t i = 0; i < (size_t)m * n; i++) {
        const float delta = std::fabs((float)host_result[i] - (float)host_ref[i]);
        sum_delta += delta;
        max_delta = (delta > max_delta || delta != delta) ? delta : max_delta;
    }
    std::cout << "{\"max_delta\": " << max_delta << ", \"total_delta\": " << sum_delta << "}";
    return 0;
}
