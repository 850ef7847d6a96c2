// Builds the reference's OWN host loops into oracle/_ref/libref_host.so, from the sources where they lie:
// host_skinny_gemm (projects/skinny_gemm/test.cu:7-39) and host_tiled_sum_reduce
// (projects/tiled_sum_reduce/test.cu:5-26).  Test infrastructure: tests/test_reference_host.py uses it to
// check that the oracle's restatement (sg_oracle.c) follows the same loop order, scale placement and cast.
// The kernels those files also hold are compiled for the reference's own target (gfx942) because the host
// side refers to them, but nothing here launches them; their main()s - which begin with hipSetDevice - are
// renamed and never called.
#include <cstdlib>
#include <cstring>

#define main reference_skinny_gemm_test_main
#include "projects/skinny_gemm/test.cu"
#undef main

namespace tsr {
#define main reference_tsr_test_main
#include "projects/tiled_sum_reduce/test.cu"
#undef main
}  // namespace tsr

extern "C" {

// D[m][n] fp32 = (float)(acc * scale), E4M3 FNUZ operands, as the reference decodes them
void ref_host_skinny_gemm_f32(const unsigned char* A, const unsigned char* B, float* D, float scale, int m, int n, int k) {
    float* out = nullptr;
    host_skinny_gemm<float>(A, B, out, &scale, m, n, k);
    std::memcpy(D, out, sizeof(float) * (size_t)m * n);
    std::free(out);
}

// the same with the reference's own output type (fp16 bits)
void ref_host_skinny_gemm_f16(const unsigned char* A, const unsigned char* B, unsigned short* D, float scale, int m, int n, int k) {
    half* out = nullptr;
    host_skinny_gemm<half>(A, B, out, &scale, m, n, k);
    std::memcpy(D, out, sizeof(half) * (size_t)m * n);
    std::free(out);
}

// D[m*n] = sum over the batch of (A + B), in batch order
void ref_host_tiled_sum_reduce(const float* A, const float* B, float* D, int b, int m, int n) {
    float* out = nullptr;
    tsr::host_tiled_sum_reduce(A, B, out, b, m, n);
    std::memcpy(D, out, sizeof(float) * (size_t)m * n);
    std::free(out);
}

}  // extern "C"
