// 2:4 prune + compress of a dense E4M3 weight matrix for gfx950: the producer side of the format
// sg_sparse24_gemm reads (values [n][k/2], one metadata nibble per group of four k).
//
// Per group of four consecutive codes the two with the largest magnitude are kept (magnitude =
// code & 0x7f, which orders E4M3 values by |x|; ties keep the lower position, so an input that is
// already 2:4 keeps its non-zeros and pads with the lowest free positions).  Kept codes are stored
// in k order; the nibble is first | second << 2 with first < second, the group with the lower k in
// the low nibble of the byte.  No counterpart in the reference, which has no compressed format.
//
// A lane handles 16 codes (four groups): one 16-byte load, one 8-byte value store, one 2-byte
// metadata store, all contiguous across the lanes of a wave.  HBM-bound: 1.625 bytes per code.
#include "sg_device.h"
#include "sg_host.h"

namespace sg {

__device__ __forceinline__ void pick_two(uint32_t word, uint32_t& kept, uint32_t& nibble) {
    uint32_t mag[4];
#pragma unroll
    for (int i = 0; i < 4; i++) mag[i] = (word >> (8 * i)) & 0x7fu;
    // largest magnitude, then the largest among the rest; strict '>' keeps the lower position on ties
    int i0 = 0;
#pragma unroll
    for (int i = 1; i < 4; i++) i0 = mag[i] > mag[i0] ? i : i0;
    int i1 = i0 == 0 ? 1 : 0;
#pragma unroll
    for (int i = 0; i < 4; i++) i1 = (i != i0 && mag[i] > mag[i1]) ? i : i1;
    const int first = i0 < i1 ? i0 : i1, second = i0 < i1 ? i1 : i0;
    kept = ((word >> (8 * first)) & 0xffu) | (((word >> (8 * second)) & 0xffu) << 8);
    nibble = (uint32_t)first | ((uint32_t)second << 2);
}

__global__ void __launch_bounds__(256) sparse24_compress_kernel(const uint8_t* __restrict__ B, uint8_t* __restrict__ vals,
                                                                uint8_t* __restrict__ meta, int n, int k, int b_stride) {
    const int per_row = k >> 4;                                    // 16-code pieces per row
    const size_t piece = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (piece >= (size_t)n * per_row) return;
    const size_t row = piece / per_row;
    const int col = (int)(piece - row * per_row);
    const u32x4 w = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(B + row * (size_t)b_stride + (size_t)col * 16));
    uint32_t kept[4], nib[4];
#pragma unroll
    for (int g = 0; g < 4; g++) pick_two(w[g], kept[g], nib[g]);
    u32x2 v = {kept[0] | (kept[1] << 16), kept[2] | (kept[3] << 16)};
    *reinterpret_cast<u32x2*>(vals + row * (size_t)(k >> 1) + (size_t)col * 8) = v;
    const uint16_t m16 = (uint16_t)(nib[0] | (nib[1] << 4) | (nib[2] << 8) | (nib[3] << 12));
    *reinterpret_cast<uint16_t*>(meta + row * (size_t)(k >> 3) + (size_t)col * 2) = m16;
}

int launch_sparse24_compress(const uint8_t* B, uint8_t* vals, uint8_t* meta, int n, int k, int b_stride, hipStream_t stream) {
    const size_t pieces = (size_t)n * (k >> 4);
    const size_t grid = (pieces + 255) / 256;
    if (grid > 0x7fffffffu) return SG_BAD_ARGUMENT;
    sparse24_compress_kernel<<<(unsigned)grid, 256, 0, stream>>>(B, vals, meta, n, k, b_stride);
    return report_hip("sparse24_compress_kernel launch", hipGetLastError()) == hipSuccess ? SG_SUCCESS : SG_LAUNCH_FAILED;
}

}  // namespace sg
