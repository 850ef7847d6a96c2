// test main: GPU batch sum against the host loop on rand() inputs, one JSON object on stdout
// {"max_delta": ..., "total_delta": ...} - the protocol of the reference's projects/tiled_sum_reduce/test.cu:28-69
// (argv = b m n).  The host loop is the oracle's restatement of test.cu:5-26; the result must be bit-identical.
#include "./../common.cuh"
#include "./src.cu"

#include <cassert>
#include <cmath>
#include <iostream>

int main(int argc, char** argv) {
    HIP_CHECK(hipSetDevice(0));
    assert(argc == 4);
    const int b = atoi(argv[1]), m = atoi(argv[2]), n = atoi(argv[3]);
    const size_t mn = (size_t)m * n;

    std::vector<float> hA, hB, host_ref(mn), host_result(mn);
    random_host_f32(hA, (size_t)b * mn);
    random_host_f32(hB, (size_t)b * mn);
    orc_tiled_sum_reduce(hA.data(), hB.data(), host_ref.data(), b, m, n);

    float *dA, *dB, *dD;
    tensor_h2d<float>(hA.data(), dA, (size_t)b * mn);
    tensor_h2d<float>(hB.data(), dB, (size_t)b * mn);
    HIP_CHECK(hipMalloc(&dD, mn * sizeof(float)));
    HIP_CHECK(hipMemset(dD, 0xff, mn * sizeof(float)));   // NaN pattern: D must be overwritten

    HIP_CHECK(hipDeviceSynchronize());
    tiled_sum_reduce(dA, dB, dD, b, m, n);
    HIP_CHECK(hipDeviceSynchronize());
    HIP_CHECK(hipMemcpy(host_result.data(), dD, mn * sizeof(float), hipMemcpyDeviceToHost));

    float sum_delta = 0.0f, max_delta = 0.0f;
    for (size_t i = 0; i < mn; i++) {
        const float delta = std::fabs(host_result[i] - host_ref[i]);
        sum_delta += delta;
        max_delta = (delta > max_delta || delta != delta) ? delta : max_delta;
    }
    std::cout << "{\"max_delta\": " << max_delta << ", \"total_delta\": " << sum_delta << "}";
    return 0;
}
