// tiled_sum_reduce for the single-translation-unit harness: same name and argument list as the reference's launcher
// (projects/tiled_sum_reduce_async/src.cu:179-200), on the library's LDS-queue kernel, included as source.  D is overwritten.
#pragma once
#include "../../../../rocm_dev_amd/csrc/sg_tsr.hip"

inline void tiled_sum_reduce(const float* A, const float* B, float* D, const int b, const int m, const int n) {
    const int rc = sg::launch_tiled_sum_reduce_ring(A, B, D, b, m, n, nullptr);
    if (rc != 0) {
        std::fprintf(stderr, "tiled_sum_reduce: return code %d\n", rc);
        std::exit(1);
    }
}
