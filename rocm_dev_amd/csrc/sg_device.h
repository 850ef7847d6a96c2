// Device-side building blocks shared by the gfx950 kernels: vector types, bf16 rounding,
// OCP E4M3 conversion helpers and cache-policy loads.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace sg {

typedef long  i64x2 __attribute__((ext_vector_type(2)));
typedef int   i32x2 __attribute__((ext_vector_type(2)));
typedef int   i32x4 __attribute__((ext_vector_type(4)));
typedef int   i32x8 __attribute__((ext_vector_type(8)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

constexpr int kWave = 64;

__device__ __forceinline__ int lane_id() { return threadIdx.x & 63; }
__device__ __forceinline__ int wave_id() { return __builtin_amdgcn_readfirstlane(threadIdx.x >> 6); }

// fp32 -> bf16 bits, round to nearest even; NaN stays a quiet NaN.
__device__ __forceinline__ uint32_t bf16_bits(float x) {
    uint32_t u = __float_as_uint(x);
    uint32_t r = (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
    return ((u & 0x7fffffffu) > 0x7f800000u) ? ((u >> 16) | 0x40u) : r;
}
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
    return bf16_bits(lo) | (bf16_bits(hi) << 16);
}
__device__ __forceinline__ float bf16_lo(uint32_t w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }

// 16-byte global loads.  The streaming flavour marks the line non-temporal: weights are
// read exactly once, so they should not displace the activations held in L2.
__device__ __forceinline__ i64x2 load16(const void* p) { return *reinterpret_cast<const i64x2*>(p); }
__device__ __forceinline__ i64x2 load16_stream(const void* p) {
    return __builtin_nontemporal_load(reinterpret_cast<const i64x2*>(p));
}

// D = A x B + C on gfx950's FP8 matrix core: 16 x 16 outputs, 128 bytes of K per instruction, both operands OCP E4M3
// (format codes 0/0).  The builtin is the block-scaled form; with both scale operands the constant 0 the compiler
// emits the plain v_mfma_f32_16x16x128_f8f6f4 - no scale-load instruction in front of every MFMA, bit-identical
// results to unit scales (E8M0 byte 127), and about 7 % more sustained throughput on real data (less power).
__device__ __forceinline__ f32x4 mfma_e4m3_16x16x128(const i32x8& a, const i32x8& b, const f32x4& c) {
    return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, c, 0, 0, 0, 0, 0, 0);
}


// n / d for a divisor whose reciprocal the host has prepared: inv = floor(2^32 / d) (0xffffffff for d = 1).
// The product's high word is the quotient or one below it for every 32-bit n, so one correction step makes
// it exact.  Five scalar instructions where the compiler's general division is about thirty, among them a
// reciprocal on the vector unit whose result has to travel back to the scalar unit - at the top of a
// kernel whose one wave per SIMD has nothing else to issue meanwhile.
__host__ __device__ __forceinline__ unsigned div_reciprocal(unsigned d) {
    return d <= 1 ? 0xffffffffu : (unsigned)(0x100000000ull / d);
}
__device__ __forceinline__ unsigned fast_div(unsigned n, unsigned d, unsigned inv) {
    const unsigned q = __umulhi(n, inv);
    return n - q * d >= d ? q + 1 : q;
}

// Workgroups are dispatched round-robin over the 8 XCDs (workgroup b runs on XCD b % 8), each with its own
// L2.  A 16-row tile writes only 32 bytes of every output row, so the four tiles that share a 128-byte line of
// D should pass through the same L2, which then merges them before they reach memory: workgroup b is given
// position xcd_order(b) in tile order, where all workgroups of one XCD are neighbours.
constexpr int kXcds = 8;
__device__ __forceinline__ int xcd_order(int b, int groups) {
    const int x = b % kXcds, i = b / kXcds;
    const int q = groups / kXcds, rem = groups % kXcds;
    return x * q + (x < rem ? x : rem) + i;
}

}  // namespace sg
