// Test helper: dumps what ROCm's hip_fp8.h *host* software casts produce for OCP E4M3.
// The reference's host oracle decodes and encodes through these same header functions
// (projects/skinny_gemm/test.cu:33,57 and projects/common.cuh:103, there in FNUZ mode);
// this program calls them in __HIP_E4M3 (OCP) mode so the oracle's tables can be pinned
// against the library the reference depends on.  No GPU call is made.
//
//   hipfp8_host_cast decode            -> 256 lines "code value" (fp16 widened to float)
//   hipfp8_host_cast encode < floats   -> one code per input line (hex float bits in)
#include <hip/hip_fp8.h>
#include <hip/hip_fp16.h>
#include <cstdio>
#include <cstring>
#include <cstdint>

int main(int argc, char** argv) {
    if (argc == 2 && !strcmp(argv[1], "decode")) {
        for (int c = 0; c < 256; c++) {
            __half_raw h = __hip_cvt_fp8_to_halfraw((__hip_fp8_storage_t)c, __HIP_E4M3);
            float f = (float)h.data;
            uint32_t u;
            memcpy(&u, &f, 4);
            printf("%d %08x\n", c, u);
        }
        return 0;
    }
    if (argc == 2 && !strcmp(argv[1], "encode")) {
        unsigned u;
        while (scanf("%x", &u) == 1) {
            float f;
            memcpy(&f, &u, 4);
            printf("%d\n", (int)__hip_cvt_float_to_fp8(f, __HIP_SATFINITE, __HIP_E4M3));
        }
        return 0;
    }
    fprintf(stderr, "usage: %s decode | encode\n", argv[0]);
    return 2;
}
