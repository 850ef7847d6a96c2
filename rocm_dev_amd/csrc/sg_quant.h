// Per-row E4M3 quantisation arithmetic shared by the row encoder (sg_codec.hip) and the GEMM that
// quantises its bf16 activations itself (sg_lds_kernel.h): one definition, so both produce the same bits.
//
//   scale[r] = absmax(row r) / 448   (1 for an all-zero row; NaNs do not take part in the maximum)
//   code     = e4m3_rne_sat( fp32(x) / scale[r] ),  a NaN quotient -> 0x7f
//
// The quotient must be the correctly rounded fp32 quotient (the E4M3 rounding that follows makes a one-ulp
// slip visible at a tie).  An IEEE divide is about ten VALU operations; rows whose maximum has a biased
// exponent in [60, 190] use y = 1 / s once and Markstein's correction per element,
//   q = x*y;  r = fma(-s, q, x);  q' = fma(r, y, q),
// which equals the IEEE quotient for every bf16 x below such a bf16 maximum wherever |q| >= 2^-12 (checked
// exhaustively on the CPU; smaller quotients all encode to zero).  Other rows take the IEEE divide.
#pragma once

#include "sg_device.h"

namespace sg {

// Both E4M3 NaN codes (0x7f, 0xff) -> 0x7f in all four bytes: the sign of a NaN quotient (NaN input, inf / inf)
// depends on how the division is carried out, so the encoder's contract fixes it.
__device__ __forceinline__ uint32_t canonical_nan_codes(int packed) {
    const uint32_t u = (uint32_t)packed;
    const uint32_t nan_sign = ((u & 0x7f7f7f7fu) + 0x01010101u) & 0x80808080u;   // bit 7 of every byte whose low seven bits are ones
    return u & ~nan_sign;
}

// largest |x| of eight bf16 values, NaNs ignored (fmaxf returns the other operand)
__device__ __forceinline__ float absmax8_bf16(const u32x4 raw, float amax) {
#pragma unroll
    for (int j = 0; j < 4; j++) {
        amax = fmaxf(amax, fabsf(bf16_lo(raw[j])));
        amax = fmaxf(amax, fabsf(bf16_hi(raw[j])));
    }
    return amax;
}

struct RowQuant {
    float s;      // the row's scale
    float y;      // 1 / s, correctly rounded
    bool fast;    // Markstein's correction applies
};
__device__ __forceinline__ RowQuant row_quant(float amax) {
    RowQuant r;
    r.s = (amax == 0.0f) ? 1.0f : __fdiv_rn(amax, 448.0f);
    r.y = __fdiv_rn(1.0f, r.s);
    const uint32_t aexp = (__float_as_uint(amax) >> 23) & 0xffu;
    r.fast = (aexp >= 60u && aexp <= 190u);
    return r;
}

// eight bf16 values -> eight E4M3 codes (k order preserved: byte j of the result is element j)
__device__ __forceinline__ u32x2 quantize8_bf16(const u32x4 raw, const RowQuant r) {
    float q[8];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const float x0 = bf16_lo(raw[j]), x1 = bf16_hi(raw[j]);
        if (r.fast) {
            const float q0 = __fmul_rn(x0, r.y), q1 = __fmul_rn(x1, r.y);
            // copysign: for x = -0 the correction step would return +0, the divide gives -0
            q[2 * j] = copysignf(__fmaf_rn(__fmaf_rn(-r.s, q0, x0), r.y, q0), x0);
            q[2 * j + 1] = copysignf(__fmaf_rn(__fmaf_rn(-r.s, q1, x1), r.y, q1), x1);
        } else {
            q[2 * j] = __fdiv_rn(x0, r.s);
            q[2 * j + 1] = __fdiv_rn(x1, r.s);
        }
    }
    int w0 = __builtin_amdgcn_cvt_pk_fp8_f32(q[0], q[1], 0, false);
    w0 = __builtin_amdgcn_cvt_pk_fp8_f32(q[2], q[3], w0, true);
    int w1 = __builtin_amdgcn_cvt_pk_fp8_f32(q[4], q[5], 0, false);
    w1 = __builtin_amdgcn_cvt_pk_fp8_f32(q[6], q[7], w1, true);
    return u32x2{canonical_nan_codes(w0), canonical_nan_codes(w1)};
}

}  // namespace sg
