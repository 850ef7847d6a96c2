// Profiling aid: streams a weight matrix the way the persistent LDS-ring GEMM does - same tiles per workgroup, same
// K split over eight waves, same 4 rows x 256 B direct-to-LDS loads with the streaming hint, two ring slots per
// wave - and does nothing else: no activations, no matrix instructions, no stores.  What it sustains is the ceiling
// of that access pattern, the yardstick the GEMM's own streaming rate is read against.
#pragma once

#include "sg_lds_kernel.h"

namespace sg {

// SEG: contiguous bytes a DMA instruction takes from one row - 256 (4 rows per instruction, the GEMM's pattern), 512
// (2 rows) or 1024 (1 row); a wave's stage is always 4 KB = 4 instructions: 16 rows x 256 B, 8 x 512 B or 4 x 1 KB.
template <int SEG>
__global__ void __launch_bounds__(512) read_stream_kernel(const uint8_t* B, int n, int k, int b_stride, unsigned* sink) {
    extern __shared__ __attribute__((aligned(1024))) uint8_t ring[];   // [wave][2][4 KB]
    constexpr int DEPTH = 2, PER_STAGE = 4, STAGE_BYTES = 4096;
    const int lane = lane_id(), wave = wave_id(), waves = (int)blockDim.x >> 6;
    constexpr int ROWS_PER_INSTR = 1024 / SEG, TILE_ROWS = 4 * ROWS_PER_INSTR;   // 16, 8 or 4 rows per tile
    const int blocks = k / SEG;
    const TileRun run = persistent_tile_run((n + TILE_ROWS - 1) / TILE_ROWS);
    const int per_tile = wave < blocks ? (blocks - wave + waves - 1) / waves : 0;
    const int total = per_tile * run.count;
    const int src_row = (lane * 16) / SEG, src_col = (lane * 16) % SEG;   // 16 bytes per lane, lanes in address order
    const unsigned my_ring_lds = lds_addr(ring + (size_t)wave * (DEPTH * STAGE_BYTES));
    const uint8_t* my_ring = ring + (size_t)wave * (DEPTH * STAGE_BYTES);
    auto issue = [&](int i) __attribute__((always_inline)) {
        const int j = i / per_tile;
        const int kb = wave + (i - j * per_tile) * waves;
        const int n0 = (run.first + j) * TILE_ROWS;
        const unsigned slot = my_ring_lds + (unsigned)(i % DEPTH) * STAGE_BYTES;
#pragma unroll
        for (int u = 0; u < 4; u++) {
            int row = n0 + ROWS_PER_INSTR * u + src_row;
            row = row < n ? row : n - 1;
            dma_1kb_stream(B + (size_t)row * b_stride + (size_t)kb * SEG + src_col, slot + u * 1024);
        }
    };
    unsigned seen = 0;
    auto consume = [&](int i) __attribute__((always_inline)) {
        seen ^= *reinterpret_cast<const unsigned*>(my_ring + (size_t)(i % DEPTH) * STAGE_BYTES + 16 * lane);
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    };
    const int pro = total < DEPTH ? total : DEPTH;
    for (int d = 0; d < pro; d++) issue(d);
    for (int i = 0; i < total; i++) {
        if (i + DEPTH <= total) wait_vmcnt<(DEPTH - 1) * PER_STAGE>();
        else wait_vmcnt<0>();
        consume(i);
        if (i + DEPTH < total) issue(i + DEPTH);
    }
    // the words read decide nothing: the store keeps the loop from being optimised away and never happens for real data
    if (seen == 0x9e3779b9u && sink) *sink = seen;
}

}  // namespace sg
