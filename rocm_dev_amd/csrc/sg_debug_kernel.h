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

// Profiling aid: what one CU can take in through direct-to-LDS loads when part of the stream misses the XCD's L2 and
// part of it hits.  Every wave issues 1 KB loads (8 rows x 128 B, rows 8 KB apart: the mid-batch kernel's pattern)
// into its own LDS slots, DEPTH instructions in flight, until a wall-clock deadline, and counts them.
//   cold stream: a region of its own per wave, walked once (streaming hint) - L2 misses
//   hot stream:  one window per XCD (workgroup id % 8) that all its workgroups walk from different starts - L2 hits
// cold_waves >= 0: waves [0, cold_waves) stream cold, the others hot.  cold_waves < 0: every wave alternates
// hot_per_cold hot instructions with one cold one.  counts[0], counts[1]: cold and hot instructions of all workgroups.
template <int DEPTH>
__global__ void __launch_bounds__(1024) cu_ingest_kernel(const uint8_t* cold, unsigned cold_region, const uint8_t* hot, unsigned hot_window,
                                                          int ticks, int cold_waves, int hot_per_cold, unsigned long long* counts) {
    extern __shared__ __attribute__((aligned(1024))) uint8_t ring[];
    constexpr unsigned PITCH = 8192;
    const int lane = lane_id(), wave = wave_id(), waves = (int)blockDim.x >> 6;
    const int slots = 128 / waves;                                    // 1 KB slots per wave out of 128 KB (waves is a power of two)
    const unsigned my_lds = lds_addr(ring + (size_t)wave * slots * 1024);
    const size_t lane_off = (size_t)(lane >> 3) * PITCH + (size_t)(lane & 7) * 16;
    const uint8_t* cbase = cold + ((size_t)blockIdx.x * waves + wave) * cold_region + lane_off;
    const uint8_t* hbase = hot + (size_t)(blockIdx.x & 7) * hot_window + lane_off;
    const unsigned cmask = cold_region - 1, hmask = hot_window - 1;   // both sizes are powers of two, at least 8 rows
    unsigned cpos = 0, hpos = (unsigned)((((blockIdx.x >> 3) * waves + wave) * 8u * PITCH) & hmask);
    // along the row in 128-byte steps, then on to the next eight rows, wrapping inside the region
    auto advance = [](unsigned pos, unsigned mask) __attribute__((always_inline)) {
        unsigned in_row = (pos & (PITCH - 1)) + 128, grp = pos & ~(PITCH * 8 - 1);
        if (in_row == PITCH) { in_row = 0; grp += PITCH * 8; }
        return (grp + in_row) & mask;
    };
    int slot = 0;
    unsigned n_cold = 0, n_hot = 0;
    auto load_cold = [&]() __attribute__((always_inline)) {
        dma_1kb_stream(cbase + cpos, my_lds + (unsigned)slot * 1024);
        cpos = advance(cpos, cmask);
        slot = (slot + 1) & (slots - 1);
        n_cold++;
        wait_vmcnt<DEPTH - 1>();
    };
    auto load_hot = [&]() __attribute__((always_inline)) {
        dma_1kb(hbase + hpos, my_lds + (unsigned)slot * 1024);
        hpos = advance(hpos, hmask);
        slot = (slot + 1) & (slots - 1);
        n_hot++;
        wait_vmcnt<DEPTH - 1>();
    };
    // the clock is read once per batch of loads: a read per load would bound the loop by the read's own latency
    const unsigned long long t_end = __builtin_amdgcn_s_memrealtime() + (unsigned long long)ticks;
    if (cold_waves >= 0 && wave < cold_waves) {
        while (__builtin_amdgcn_s_memrealtime() < t_end)
            for (int rep = 0; rep < 16; rep++) load_cold();
    } else if (cold_waves >= 0) {
        while (__builtin_amdgcn_s_memrealtime() < t_end)
            for (int rep = 0; rep < 16; rep++) load_hot();
    } else {
        while (__builtin_amdgcn_s_memrealtime() < t_end)
            for (int rep = 0; rep < 4; rep++) {
                for (int h = 0; h < hot_per_cold; h++) load_hot();
                load_cold();
            }
    }
    wait_vmcnt<0>();
    if (lane == 0) {
        if (n_cold) atomicAdd(&counts[0], n_cold);
        if (n_hot) atomicAdd(&counts[1], n_hot);
    }
}

}  // namespace sg
