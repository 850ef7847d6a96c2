// One v_mfma_f32_16x16x128_f8f6f4 per test: A[16][128], B[16][128] (E4M3 codes, row-major by logical k), C[16][16] -> D[16][16].
// Logical k of lane l, byte j: 32*(l/16) + j (the register layout of the instruction).
#include <hip/hip_runtime.h>
#include <stdint.h>
typedef int i32x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
__global__ void probe(const uint8_t* A, const uint8_t* B, const float* C, float* D, int tests) {
    const int lane = threadIdx.x;
    for (int t = blockIdx.x; t < tests; t += gridDim.x) {
        const uint8_t* a = A + (size_t)t * 2048 + (lane % 16) * 128 + 32 * (lane / 16);
        const uint8_t* b = B + (size_t)t * 2048 + (lane % 16) * 128 + 32 * (lane / 16);
        i32x8 av = *reinterpret_cast<const i32x8*>(a);
        i32x8 bv = *reinterpret_cast<const i32x8*>(b);
        f32x4 c;
        for (int e = 0; e < 4; e++) c[e] = C[(size_t)t * 256 + (4 * (lane / 16) + e) * 16 + lane % 16];
        f32x4 d = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(av, bv, c, 0, 0, 0, 0, 0, 0);
        for (int e = 0; e < 4; e++) D[(size_t)t * 256 + (4 * (lane / 16) + e) * 16 + lane % 16] = d[e];
    }
}
extern "C" int run_probe(const uint8_t* A, const uint8_t* B, const float* C, float* D, int tests) {
    probe<<<dim3(256), dim3(64)>>>(A, B, C, D, tests);
    return (int)hipDeviceSynchronize();
}
