// Per-row FP8 codec for gfx950: the local compute on either side of an FP8 all-reduce
// exchange.  All three kernels are pure HBM streaming; arithmetic per element is kept to a
// handful of VALU operations so the memory pipe stays the limit.
//
//   encode  scales[r] = absmax(X[r,:]) / 448 (1 for an all-zero row);
//           Q[r,c]    = e4m3_rne_sat( fp32(X[r,c]) / scales[r] )          (bit exact)
//   decode  Y[r,c]    = bf16( dec(Q[r,c]) * scales[r] )
//   reduce  Y[r,c]    = bf16( sum_i dec(Q_i[r,c]) * scales_i[r] ), fp32, buffer order,
//           multiply and add rounded separately (no fused multiply-add)
//
// The quotient x / s must be the correctly rounded fp32 quotient, because the E4M3
// rounding that follows makes a one-ulp slip visible at a tie.  A hardware IEEE divide is
// about ten VALU operations per element, too many for a streaming kernel, so the kernel
// divides once per row (y = 1/s, correctly rounded) and per element uses Markstein's
// correction  q = x*y;  r = fma(-s, q, x);  q' = fma(r, y, q).  x and the row maximum are
// bf16 values; for every bf16 maximum with biased exponent 60..190 and every bf16 x below
// it this sequence has been checked exhaustively on the CPU against the IEEE quotient
// wherever |q| >= 2^-12 (smaller quotients all encode to zero).  Rows whose maximum lies
// outside that exponent window take the plain IEEE divide.
#include "sg_device.h"
#include "sg_host.h"
#include "sg_quant.h"

namespace sg {

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));

__device__ __forceinline__ uint32_t cvt_bf16x2(float lo, float hi) {
    f32x2 v = {lo, hi};
    bf16x2_t h = __builtin_convertvector(v, bf16x2_t);
    return __builtin_bit_cast(uint32_t, h);
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o));
    return v;
}

// One workgroup per row.  Thread t holds chunks t, t+T, ... of 8 bf16 each (CH of them),
// so the row is read from memory exactly once.
template <int CH>
__global__ void __launch_bounds__(256) fp8_encode_rows_kernel(const uint16_t* __restrict__ X, uint8_t* __restrict__ Q,
                                                              float* __restrict__ scales, int cols) {
    __shared__ float wmax[4];
    const int row = blockIdx.x;
    const int T = blockDim.x;
    const int t = threadIdx.x;
    const int nchunks = cols >> 3;
    const u32x4* xrow = reinterpret_cast<const u32x4*>(X + (size_t)row * cols);

    u32x4 raw[CH];
#pragma unroll
    for (int c = 0; c < CH; c++) {
        const int idx = c * T + t;
        raw[c] = u32x4{0u, 0u, 0u, 0u};
        if (idx < nchunks) raw[c] = __builtin_nontemporal_load(xrow + idx);
    }

    float amax = 0.0f;
#pragma unroll
    for (int c = 0; c < CH; c++) amax = absmax8_bf16(raw[c], amax);
    amax = wave_max(amax);
    const int nw = T >> 6;
    if (nw > 1) {
        if (lane_id() == 0) wmax[threadIdx.x >> 6] = amax;
        __syncthreads();
        amax = wmax[0];
        for (int w = 1; w < nw; w++) amax = fmaxf(amax, wmax[w]);
    }

    const RowQuant rq = row_quant(amax);
    if (t == 0) scales[row] = rq.s;

    u32x2* qrow = reinterpret_cast<u32x2*>(Q + (size_t)row * cols);
#pragma unroll
    for (int c = 0; c < CH; c++) {
        const int idx = c * T + t;
        const u32x2 out = quantize8_bf16(raw[c], rq);
        if (idx < nchunks) __builtin_nontemporal_store(out, qrow + idx);
    }
}

// Rows too long to hold in registers: two passes over the row (the second mostly from L2).
__global__ void __launch_bounds__(256) fp8_encode_rows_long_kernel(const uint16_t* __restrict__ X, uint8_t* __restrict__ Q,
                                                                   float* __restrict__ scales, int cols) {
    __shared__ float wmax[4];
    const int row = blockIdx.x;
    const int t = threadIdx.x;
    const int nchunks = cols >> 3;
    const u32x4* xrow = reinterpret_cast<const u32x4*>(X + (size_t)row * cols);
    float amax = 0.0f;
    for (int idx = t; idx < nchunks; idx += 256) {
        const u32x4 raw = xrow[idx];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            amax = fmaxf(amax, fabsf(bf16_lo(raw[j])));
            amax = fmaxf(amax, fabsf(bf16_hi(raw[j])));
        }
    }
    amax = wave_max(amax);
    if (lane_id() == 0) wmax[threadIdx.x >> 6] = amax;
    __syncthreads();
    amax = fmaxf(fmaxf(wmax[0], wmax[1]), fmaxf(wmax[2], wmax[3]));
    const float s = (amax == 0.0f) ? 1.0f : __fdiv_rn(amax, 448.0f);
    if (t == 0) scales[row] = s;
    u32x2* qrow = reinterpret_cast<u32x2*>(Q + (size_t)row * cols);
    for (int idx = t; idx < nchunks; idx += 256) {
        const u32x4 raw = xrow[idx];
        float q[8];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            q[2 * j] = __fdiv_rn(bf16_lo(raw[j]), s);
            q[2 * j + 1] = __fdiv_rn(bf16_hi(raw[j]), s);
        }
        int w0 = __builtin_amdgcn_cvt_pk_fp8_f32(q[0], q[1], 0, false);
        w0 = __builtin_amdgcn_cvt_pk_fp8_f32(q[2], q[3], w0, true);
        int w1 = __builtin_amdgcn_cvt_pk_fp8_f32(q[4], q[5], 0, false);
        w1 = __builtin_amdgcn_cvt_pk_fp8_f32(q[6], q[7], w1, true);
        qrow[idx] = u32x2{canonical_nan_codes(w0), canonical_nan_codes(w1)};
    }
}

// 16 codes per thread: one 16-byte load, two 16-byte stores.  cols % 16 == 0, so a chunk
// never straddles two rows.
__global__ void __launch_bounds__(256) fp8_decode_rows_kernel(const uint8_t* __restrict__ Q, const float* __restrict__ scales,
                                                              uint16_t* __restrict__ Y, int cols, size_t nchunks) {
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= nchunks) return;
    const int chunks_per_row = cols >> 4;
    const int row = (int)(idx / chunks_per_row);
    const float s = scales[row];
    const u32x4 q = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(Q) + idx);
    u32x4 o[2];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const f32x2 lo = __builtin_amdgcn_cvt_pk_f32_fp8(q[j], false);
        const f32x2 hi = __builtin_amdgcn_cvt_pk_f32_fp8(q[j], true);
        o[j >> 1][2 * (j & 1)] = cvt_bf16x2(__fmul_rn(lo.x, s), __fmul_rn(lo.y, s));
        o[j >> 1][2 * (j & 1) + 1] = cvt_bf16x2(__fmul_rn(hi.x, s), __fmul_rn(hi.y, s));
    }
    // plain stores: with 32 bytes per lane the non-temporal hint costs a third of the bandwidth
    // (measured 3.9 vs 6.0 TB/s for this 1-read : 2-write pattern)
    u32x4* y = reinterpret_cast<u32x4*>(Y) + 2 * idx;
    y[0] = o[0];
    y[1] = o[1];
}

template <int NBUF>
__global__ void __launch_bounds__(256) fp8_reduce_rows_kernel(const uint8_t* __restrict__ Q, const float* __restrict__ scales,
                                                              uint16_t* __restrict__ Y, int nbuf_rt, size_t q_buf_stride,
                                                              int rows, int cols, size_t nchunks) {
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= nchunks) return;
    const int nbuf = NBUF > 0 ? NBUF : nbuf_rt;
    const int chunks_per_row = cols >> 4;
    const int row = (int)(idx / chunks_per_row);
    float acc[16];
#pragma unroll
    for (int e = 0; e < 16; e++) acc[e] = 0.0f;

    auto accumulate = [&](const u32x4 q, const float s) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const f32x2 lo = __builtin_amdgcn_cvt_pk_f32_fp8(q[j], false);
            const f32x2 hi = __builtin_amdgcn_cvt_pk_f32_fp8(q[j], true);
            acc[4 * j + 0] = __fadd_rn(acc[4 * j + 0], __fmul_rn(lo.x, s));
            acc[4 * j + 1] = __fadd_rn(acc[4 * j + 1], __fmul_rn(lo.y, s));
            acc[4 * j + 2] = __fadd_rn(acc[4 * j + 2], __fmul_rn(hi.x, s));
            acc[4 * j + 3] = __fadd_rn(acc[4 * j + 3], __fmul_rn(hi.y, s));
        }
    };

    if (NBUF > 0) {
        u32x4 q[NBUF > 0 ? NBUF : 1];
        float s[NBUF > 0 ? NBUF : 1];
#pragma unroll
        for (int b = 0; b < NBUF; b++) {
            q[b] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(Q + (size_t)b * q_buf_stride) + idx);
            s[b] = scales[(size_t)b * rows + row];
        }
#pragma unroll
        for (int b = 0; b < NBUF; b++) accumulate(q[b], s[b]);
    } else {
        for (int b = 0; b < nbuf; b++) {
            const u32x4 q = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(Q + (size_t)b * q_buf_stride) + idx);
            accumulate(q, scales[(size_t)b * rows + row]);
        }
    }

    u32x4 o[2];
#pragma unroll
    for (int j = 0; j < 8; j++) o[j >> 2][j & 3] = cvt_bf16x2(acc[2 * j], acc[2 * j + 1]);
    // plain stores: with 32 bytes per lane the non-temporal hint costs a third of the bandwidth
    // (measured 3.9 vs 6.0 TB/s for this 1-read : 2-write pattern)
    u32x4* y = reinterpret_cast<u32x4*>(Y) + 2 * idx;
    y[0] = o[0];
    y[1] = o[1];
}

static bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

int launch_fp8_encode_rows(const void* X, uint8_t* Q, float* scales, int rows, int cols, hipStream_t stream) {
    if (!X || !Q || !scales || rows <= 0 || cols <= 0 || (cols & 15)) return SG_BAD_ARGUMENT;
    if (!aligned16(X) || !aligned16(Q)) return SG_BAD_ALIGNMENT;
    const int nchunks = cols >> 3;
    const uint16_t* x = reinterpret_cast<const uint16_t*>(X);
    int threads = 256;
    if (nchunks <= 64) threads = 64;
    else if (nchunks <= 128) threads = 128;
    const int ch = (nchunks + threads - 1) / threads;
    if (ch <= 1) fp8_encode_rows_kernel<1><<<rows, threads, 0, stream>>>(x, Q, scales, cols);
    else if (ch <= 2) fp8_encode_rows_kernel<2><<<rows, threads, 0, stream>>>(x, Q, scales, cols);
    else if (ch <= 4) fp8_encode_rows_kernel<4><<<rows, threads, 0, stream>>>(x, Q, scales, cols);
    else if (ch <= 8) fp8_encode_rows_kernel<8><<<rows, threads, 0, stream>>>(x, Q, scales, cols);
    else fp8_encode_rows_long_kernel<<<rows, 256, 0, stream>>>(x, Q, scales, cols);
    return hipGetLastError() == hipSuccess ? SG_SUCCESS : SG_LAUNCH_FAILED;
}

int launch_fp8_decode_rows(const uint8_t* Q, const float* scales, void* Y, int rows, int cols, hipStream_t stream) {
    if (!Q || !scales || !Y || rows <= 0 || cols <= 0 || (cols & 15)) return SG_BAD_ARGUMENT;
    if (!aligned16(Q) || !aligned16(Y)) return SG_BAD_ALIGNMENT;
    const size_t nchunks = (size_t)rows * (cols >> 4);
    const unsigned grid = (unsigned)((nchunks + 255) / 256);
    fp8_decode_rows_kernel<<<grid, 256, 0, stream>>>(Q, scales, reinterpret_cast<uint16_t*>(Y), cols, nchunks);
    return hipGetLastError() == hipSuccess ? SG_SUCCESS : SG_LAUNCH_FAILED;
}

int launch_fp8_reduce_rows(const uint8_t* Q, const float* scales, void* Y, int nbuf, size_t q_buf_stride, int rows,
                           int cols, hipStream_t stream) {
    if (!Q || !scales || !Y || nbuf <= 0 || rows <= 0 || cols <= 0 || (cols & 15)) return SG_BAD_ARGUMENT;
    if (!aligned16(Q) || !aligned16(Y) || (q_buf_stride & 15)) return SG_BAD_ALIGNMENT;
    if (nbuf > 1 && q_buf_stride < (size_t)rows * cols) return SG_BAD_ARGUMENT;
    const size_t nchunks = (size_t)rows * (cols >> 4);
    const unsigned grid = (unsigned)((nchunks + 255) / 256);
    uint16_t* y = reinterpret_cast<uint16_t*>(Y);
    if (nbuf == 8)
        fp8_reduce_rows_kernel<8><<<grid, 256, 0, stream>>>(Q, scales, y, nbuf, q_buf_stride, rows, cols, nchunks);
    else if (nbuf == 4)
        fp8_reduce_rows_kernel<4><<<grid, 256, 0, stream>>>(Q, scales, y, nbuf, q_buf_stride, rows, cols, nchunks);
    else if (nbuf == 2)
        fp8_reduce_rows_kernel<2><<<grid, 256, 0, stream>>>(Q, scales, y, nbuf, q_buf_stride, rows, cols, nchunks);
    else
        fp8_reduce_rows_kernel<0><<<grid, 256, 0, stream>>>(Q, scales, y, nbuf, q_buf_stride, rows, cols, nchunks);
    return hipGetLastError() == hipSuccess ? SG_SUCCESS : SG_LAUNCH_FAILED;
}

}  // namespace sg
