// fp32 batch sum for gfx950:  D[m,n] = sum_b (A[b,m,n] + B[b,m,n]).
//
// Restates tiled_sum_reduce/src.cu:11-50: per element the batches are visited in order and
// each step adds (A + B) to the running sum, so the result is bit-identical to the host
// loop in tiled_sum_reduce/test.cu:5-26.  The reference gives every wave an 8 x 64 tile of
// 8 scalar loads per lane; here a lane owns four consecutive floats (one 128-bit load per
// operand per batch) and UNROLL batches are kept in flight, which is what a pure streaming
// kernel needs on HBM3E.  Any m, n: the tail is handled element-wise.
#include "sg_device.h"
#include "sg_host.h"

namespace sg {

constexpr int kTsrUnroll = 4;

__global__ void __launch_bounds__(256) tiled_sum_reduce_kernel(const float* __restrict__ A, const float* __restrict__ B,
                                                               float* __restrict__ D, int b, size_t mn) {
    const size_t i4 = ((size_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (i4 >= mn) return;
    if (i4 + 4 <= mn && (mn & 3) == 0) {
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
        const float* a = A + i4;
        const float* bb = B + i4;
        int ib = 0;
        for (; ib + kTsrUnroll <= b; ib += kTsrUnroll) {
            f32x4 va[kTsrUnroll], vb[kTsrUnroll];
#pragma unroll
            for (int u = 0; u < kTsrUnroll; u++) {
                va[u] = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(a + (size_t)(ib + u) * mn));
                vb[u] = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(bb + (size_t)(ib + u) * mn));
            }
#pragma unroll
            for (int u = 0; u < kTsrUnroll; u++)
#pragma unroll
                for (int e = 0; e < 4; e++) acc[e] = __fadd_rn(acc[e], __fadd_rn(va[u][e], vb[u][e]));
        }
        for (; ib < b; ib++) {
            const f32x4 va = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(a + (size_t)ib * mn));
            const f32x4 vb = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(bb + (size_t)ib * mn));
#pragma unroll
            for (int e = 0; e < 4; e++) acc[e] = __fadd_rn(acc[e], __fadd_rn(va[e], vb[e]));
        }
        *reinterpret_cast<f32x4*>(D + i4) = acc;
    } else {
        for (size_t i = i4; i < mn && i < i4 + 4; i++) {
            float acc = 0.f;
            for (int ib = 0; ib < b; ib++) acc = __fadd_rn(acc, __fadd_rn(A[(size_t)ib * mn + i], B[(size_t)ib * mn + i]));
            D[i] = acc;
        }
    }
}

int launch_tiled_sum_reduce(const float* A, const float* B, float* D, int b, int m, int n, hipStream_t stream) {
    if (!A || !B || !D || b < 0 || m <= 0 || n <= 0) return SG_BAD_ARGUMENT;
    if ((reinterpret_cast<uintptr_t>(A) | reinterpret_cast<uintptr_t>(B) | reinterpret_cast<uintptr_t>(D)) & 15u)
        return SG_BAD_ALIGNMENT;
    const size_t mn = (size_t)m * n;
    const unsigned grid = (unsigned)((mn + 1023) / 1024);
    tiled_sum_reduce_kernel<<<grid, 256, 0, stream>>>(A, B, D, b, mn);
    return hipGetLastError() == hipSuccess ? SG_SUCCESS : SG_LAUNCH_FAILED;
}

}  // namespace sg
