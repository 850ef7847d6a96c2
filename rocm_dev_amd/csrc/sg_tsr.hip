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
//
// tiled_sum_reduce_async/src.cu:13-177 stages the same sum through an LDS queue: producer waves copy
// batch slices of A and B into QSIZE slots, consumer waves wait on flag bytes, add and free the slots.
// Its counterpart here (tiled_sum_reduce_ring_kernel) keeps the queue and drops the flags: every wave
// fills its own slots with direct-to-LDS loads (global_load_lds_dwordx4, 1 KB per instruction, no
// registers in between), DEPTH batches ahead, and consumes them in batch order behind s_waitcnt
// vmcnt - loads complete in issue order, so the counter is the queue's head.  Same sums, same order.
#include "sg_device.h"
#include "sg_host.h"
#include "sg_lds_kernel.h"

namespace sg {

// the part of [first, first + count) below mn, one float per lane and step, batches in order
__device__ __forceinline__ void tiled_sum_reduce_elementwise(const float* A, const float* B, float* D, int b, size_t mn,
                                                             size_t first, int steps, int stride) {
    for (int j = 0; j < steps; j++) {
        const size_t i = first + (size_t)j * stride;
        if (i >= mn) break;
        float acc = 0.f;
        for (int ib = 0; ib < b; ib++) acc = __fadd_rn(acc, __fadd_rn(A[(size_t)ib * mn + i], B[(size_t)ib * mn + i]));
        D[i] = acc;
    }
}

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
        tiled_sum_reduce_elementwise(A, B, D, b, mn, (size_t)blockIdx.x * (1024 * CH) + threadIdx.x, 4 * CH, 256);
    }
}

// LDS-queue variant.  WAVES waves per workgroup, each owning P pieces of 1 KB (256 floats), contiguous, of every
// operand and batch: a stage is one batch = 2*P load instructions into a slot of 2*P KB, DEPTH slots per wave.
// A lane reads back exactly the 16 bytes it asked for, so nothing is shared between lanes and the only ordering
// needed is the wave's own vmcnt (the loads) and lgkmcnt (the LDS reads, which the additions wait for before the
// slot is refilled).
template <int WAVES, int P, int DEPTH>
__global__ void __launch_bounds__(WAVES * 64) tiled_sum_reduce_ring_kernel(const float* __restrict__ A, const float* __restrict__ B,
                                                                           float* __restrict__ D, int b, size_t mn) {
    constexpr int PER_STAGE = 2 * P, STAGE_BYTES = PER_STAGE * 1024, WG_FLOATS = WAVES * P * 256;
    static_assert((DEPTH - 1) * PER_STAGE <= 63, "vmcnt is a 6-bit counter");
    extern __shared__ __align__(16) uint8_t tsr_ring[];
    if ((mn & 3) != 0 || (size_t)(blockIdx.x + 1) * WG_FLOATS > mn) {
        tiled_sum_reduce_elementwise(A, B, D, b, mn, (size_t)blockIdx.x * WG_FLOATS + threadIdx.x, WG_FLOATS / (WAVES * 64),
                                     WAVES * 64);
        return;
    }
    const int wave = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6), lane = (int)threadIdx.x & 63;
    const size_t base = (size_t)blockIdx.x * WG_FLOATS + (size_t)wave * (P * 256) + lane * 4;
    const unsigned ring = lds_addr(tsr_ring) + (unsigned)wave * (DEPTH * STAGE_BYTES);
    const uint8_t* mine = tsr_ring + (size_t)wave * (DEPTH * STAGE_BYTES) + lane * 16;

    auto issue = [&](int ib) {
        const unsigned slot = ring + (unsigned)(ib % DEPTH) * STAGE_BYTES;
        const float* a = A + (size_t)ib * mn + base;
        const float* bb = B + (size_t)ib * mn + base;
#pragma unroll
        for (int u = 0; u < P; u++) {
            dma_1kb_stream(a + u * 256, slot + u * 1024);
            dma_1kb_stream(bb + u * 256, slot + (P + u) * 1024);
        }
    };
    f32x4 acc[P];
#pragma unroll
    for (int u = 0; u < P; u++) acc[u] = f32x4{0.f, 0.f, 0.f, 0.f};
    auto consume = [&](int ib) {
        const uint8_t* slot = mine + (size_t)(ib % DEPTH) * STAGE_BYTES;
#pragma unroll
        for (int u = 0; u < P; u++) {
            const f32x4 va = *reinterpret_cast<const f32x4*>(slot + u * 1024);
            const f32x4 vb = *reinterpret_cast<const f32x4*>(slot + (P + u) * 1024);
#pragma unroll
            for (int e = 0; e < 4; e++) acc[u][e] = __fadd_rn(acc[u][e], __fadd_rn(va[e], vb[e]));
        }
    };
    // prologue: up to DEPTH batches in flight; batches beyond b are never issued, so the waits below count
    // what is really outstanding
    const int ahead = b < DEPTH ? b : DEPTH;
    for (int ib = 0; ib < ahead; ib++) issue(ib);
    int ib = 0;
    for (; ib + DEPTH < b; ib++) {
        wait_vmcnt<(DEPTH - 1) * PER_STAGE>();
        consume(ib);
        // the additions above have waited for the LDS reads of this slot: it may be overwritten
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        issue(ib + DEPTH);
    }
    for (; ib < b; ib++) {                       // the last min(b, DEPTH) batches: b - 1 - ib younger stages in flight
        wait_vmcnt_upto((b - 1 - ib) * PER_STAGE);
        consume(ib);
    }
    wait_vmcnt<0>();
#pragma unroll
    for (int u = 0; u < P; u++) *reinterpret_cast<f32x4*>(D + base + u * 256) = acc[u];
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

int launch_tiled_sum_reduce_ring(const float* A, const float* B, float* D, int b, int m, int n, hipStream_t stream) {
    if (!A || !B || !D || b < 0 || m <= 0 || n <= 0) return SG_BAD_ARGUMENT;
    if ((reinterpret_cast<uintptr_t>(A) | reinterpret_cast<uintptr_t>(B) | reinterpret_cast<uintptr_t>(D)) & 15u)
        return SG_BAD_ALIGNMENT;
    const size_t mn = (size_t)m * n;
    // 32 KB of every operand and batch per workgroup (eight waves x 4 KB), two batches in flight: 128 KB of LDS,
    // one workgroup per CU; small problems take 4 KB per workgroup, four batches in flight
    if (mn >= ((size_t)4 << 20)) {
        constexpr int WAVES = 8, P = 4, DEPTH = 2;
        static bool configured[64] = {};
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return SG_LAUNCH_FAILED;
        constexpr unsigned lds = WAVES * DEPTH * 2 * P * 1024;
        if (!configured[dev]) {
            if (hipFuncSetAttribute(reinterpret_cast<const void*>(tiled_sum_reduce_ring_kernel<WAVES, P, DEPTH>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
                return SG_LAUNCH_FAILED;
            configured[dev] = true;
        }
        const size_t grid = (mn + WAVES * P * 256 - 1) / (WAVES * P * 256);
        if (grid > 0x7fffffffu) return SG_BAD_ARGUMENT;
        tiled_sum_reduce_ring_kernel<WAVES, P, DEPTH><<<(unsigned)grid, WAVES * 64, lds, stream>>>(A, B, D, b, mn);
    } else {
        constexpr int WAVES = 4, P = 1, DEPTH = 4;
        const size_t grid = (mn + WAVES * P * 256 - 1) / (WAVES * P * 256);
        tiled_sum_reduce_ring_kernel<WAVES, P, DEPTH><<<(unsigned)grid, WAVES * 64, WAVES * DEPTH * 2 * P * 1024, stream>>>(A, B, D, b, mn);
    }
    return hipGetLastError() == hipSuccess ? SG_SUCCESS : SG_LAUNCH_FAILED;
}

}  // namespace sg
