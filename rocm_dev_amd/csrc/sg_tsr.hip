// fp32 batch sum for gfx950:  D[m,n] = sum_b (A[b,m,n] + B[b,m,n]).
//
// Restates tiled_sum_reduce/src.cu:11-50: per element the batches are visited in order and
// each step adds (A + B) to the running sum, so the result is bit-identical to the host
// loop in tiled_sum_reduce/test.cu:5-26.  The reference gives every wave an 8 x 64 tile of
// 8 scalar loads per lane; here a lane owns CH pieces of four consecutive floats, 4 KB apart,
// so that a workgroup reads CH * 4 KB contiguous bytes of every operand and batch.  The 2*b
// streams of this kernel start whole multiples of m*n*4 bytes apart - typically the same
// channel and bank, different rows - and what decides the rate is how much of a DRAM row a
// stream takes per visit: 32 KB per workgroup and stream (CH = 8) with one batch in flight
// reaches 6.4-7.0 TB/s on 8-16 batches of 16-32 MB, 4 KB with four batches in flight 5.3-5.6.
// Small problems keep CH = 1, which gives them enough workgroups.  Any m, n: the tail is
// handled element-wise.
#include "sg_device.h"
#include "sg_host.h"

namespace sg {

template <int CH>
__global__ void __launch_bounds__(256) tiled_sum_reduce_kernel(const float* __restrict__ A, const float* __restrict__ B,
                                                               float* __restrict__ D, int b, size_t mn) {
    if ((mn & 3) == 0 && (size_t)(blockIdx.x + 1) * (1024 * CH) <= mn) {
        const size_t base = (size_t)blockIdx.x * (1024 * CH) + threadIdx.x * 4;
        f32x4 acc[CH];
#pragma unroll
        for (int c = 0; c < CH; c++) acc[c] = f32x4{0.f, 0.f, 0.f, 0.f};
        for (int ib = 0; ib < b; ib++) {
            f32x4 va[CH], vb[CH];
#pragma unroll
            for (int c = 0; c < CH; c++) {
                va[c] = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(A + (size_t)ib * mn + base + c * 1024));
                vb[c] = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(B + (size_t)ib * mn + base + c * 1024));
            }
#pragma unroll
            for (int c = 0; c < CH; c++)
#pragma unroll
                for (int e = 0; e < 4; e++) acc[c][e] = __fadd_rn(acc[c][e], __fadd_rn(va[c][e], vb[c][e]));
        }
#pragma unroll
        for (int c = 0; c < CH; c++) *reinterpret_cast<f32x4*>(D + base + c * 1024) = acc[c];
    } else {
        // the last, partial workgroup, or m*n not a multiple of four (batches then start at unaligned addresses):
        // one float per lane and step, neighbouring lanes on neighbouring floats
        const size_t first = (size_t)blockIdx.x * (1024 * CH) + threadIdx.x;
        for (int j = 0; j < 4 * CH; j++) {
            const size_t i = first + (size_t)j * 256;
            if (i >= mn) break;
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
    // 32 KB per workgroup and stream once that still leaves two workgroups for every CU
    const int ch = mn >= ((size_t)4 << 20) ? 8 : 1;
    const size_t per_wg = (size_t)1024 * ch;
    const size_t grid = (mn + per_wg - 1) / per_wg;
    if (grid > 0x7fffffffu) return SG_BAD_ARGUMENT;
    if (ch == 8) tiled_sum_reduce_kernel<8><<<(unsigned)grid, 256, 0, stream>>>(A, B, D, b, mn);
    else tiled_sum_reduce_kernel<1><<<(unsigned)grid, 256, 0, stream>>>(A, B, D, b, mn);
    return hipGetLastError() == hipSuccess ? SG_SUCCESS : SG_LAUNCH_FAILED;
}

}  // namespace sg
