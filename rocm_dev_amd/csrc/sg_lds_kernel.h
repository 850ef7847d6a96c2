// LDS-ring FP8 skinny GEMM for gfx950:  D[m,n] = scale * sum_k A[m,k] * B[n,k].
//
// Why LDS.  HBM3E wants long contiguous runs: a wave instruction that reads 4 rows x 256
// contiguous bytes sustains about 15 % more bandwidth than one that reads 16 rows x 64
// bytes (what the MFMA register layout would ask for).  So both operands are fetched with
// the wide pattern by gfx950's direct-to-LDS loads (global_load_lds_dwordx4: no VGPR
// staging, tracked by vmcnt) into a ring of stages, and read back from LDS in the MFMA
// layout.
//
// One stage = 256 bytes of K ("K block") for the 16*RG weight rows and the activation rows
// of the tile.  One DMA instruction moves 4 rows x 256 B = 1 KB; the hardware puts lane l's
// 16 bytes at  ring slot base + 16*l.  Which global chunk a lane fetches is ours to choose,
// and a permutation inside each 64-byte run costs nothing in the memory system, so
// instruction u (rows 4u..4u+3 of a 16-row group) lets lane l = 4*q + p fetch
//     row 4u + (q % 4),  K bytes  64*(q / 4) + 16*((p + u) % 4) .. +15,
// i.e. it rotates the four 16-byte pieces of every 64-byte run by u.  The MFMA read of
// lane (r = l%16, g = l/16) for 64-byte chunk kc is then the 16 bytes at
//     1024*(r/4) + 64*(4*kc + r%4) + 16*((g - r/4) & 3),
// and the sixteen lanes of one ds_read_b128 pass (same g, r = 0..15) hit sixteen different
// 4-bank groups: no bank conflicts, no padding.
//
// Ring protocol.  Every wave is producer and consumer of its own ring: it issues the DMAs
// of DEPTH stages ahead, waits with s_waitcnt vmcnt(n) until the oldest stage has landed
// (loads complete in order), consumes it, and refills the slot.  Nothing but the wave's own
// counters is involved, so there are no flags to poll and no barrier until the epilogue.
// (The variant with separate producer and consumer waves is sg_ring_kernel.h.)
//
// The DMA is issued from inline assembly so that the compiler's wait-count insertion does
// not see it: it would otherwise wait for ALL outstanding DMAs before every LDS read.
#pragma once

#include "sg_device.h"
#include "sg_epilogue.h"
#include "sg_quant.h"

namespace sg {

__device__ __forceinline__ unsigned lds_addr(const void* p) {
    return (unsigned)(uintptr_t)(__attribute__((address_space(3))) const void*)p;
}

// 64 lanes x 16 bytes from global memory to LDS [lds_base + 16*lane]; lds_base is wave-uniform.
__device__ __forceinline__ void dma_1kb(const void* gptr, unsigned lds_base) {
    lds_base = __builtin_amdgcn_readfirstlane(lds_base);
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(gptr), "s"(lds_base) : "memory", "m0");
}
__device__ __forceinline__ void dma_1kb_stream(const void* gptr, unsigned lds_base) {
    lds_base = __builtin_amdgcn_readfirstlane(lds_base);
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off nt" ::"v"(gptr), "s"(lds_base) : "memory", "m0");
}
// The same with the address split into a wave-uniform 64-bit base (scalar registers) and a 32-bit per-lane
// offset: advancing along K is then one scalar add per stage instead of a 64-bit vector add per instruction.
__device__ __forceinline__ void dma_1kb_at(const void* sbase, unsigned voff, unsigned lds_base) {
    lds_base = __builtin_amdgcn_readfirstlane(lds_base);
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(voff), "s"(sbase), "s"(lds_base)
                 : "memory", "m0");
}
__device__ __forceinline__ void dma_1kb_stream_at(const void* sbase, unsigned voff, unsigned lds_base) {
    lds_base = __builtin_amdgcn_readfirstlane(lds_base);
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1 nt" ::"v"(voff), "s"(sbase), "s"(lds_base)
                 : "memory", "m0");
}
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
    static_assert(N >= 0 && N <= 63, "vmcnt is a 6-bit counter");
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// waits until at most n (a run-time value, clamped to 63) vector-memory operations are outstanding
__device__ __forceinline__ void wait_vmcnt_upto(int n) {
    if (n >= 48) wait_vmcnt<48>();
    else if (n >= 32) wait_vmcnt<32>();
    else if (n >= 24) wait_vmcnt<24>();
    else if (n >= 16) wait_vmcnt<16>();
    else if (n >= 12) wait_vmcnt<12>();
    else if (n >= 8) wait_vmcnt<8>();
    else if (n >= 4) wait_vmcnt<4>();
    else wait_vmcnt<0>();
}

// Drains the last DEPTH stages: stage D of them still has DEPTH-1-D younger stages in flight.
template <int D, int DEPTH, int PER_STAGE, class Consume>
__device__ __forceinline__ void drain_ring(Consume& consume, int i) {
    wait_vmcnt<(DEPTH - 1 - D) * PER_STAGE>();
    consume(i + D);
    if constexpr (D + 1 < DEPTH) drain_ring<D + 1, DEPTH, PER_STAGE>(consume, i);
}
// ... with another consumer for the very last stage (the one that may be a half block)
template <int D, int DEPTH, int PER_STAGE, class Consume, class ConsumeLast>
__device__ __forceinline__ void drain_ring(Consume& consume, ConsumeLast& consume_last, int i) {
    wait_vmcnt<(DEPTH - 1 - D) * PER_STAGE>();
    if constexpr (D + 1 < DEPTH) {
        consume(i + D);
        drain_ring<D + 1, DEPTH, PER_STAGE>(consume, consume_last, i);
    } else {
        consume_last(i + D);
    }
}


// One 256-byte K block of a stage: weights at w (16*RG rows, 4 KB per 16-row tile), activations
// at x (4 KB per 16-row block), both already offset by the lane's read offset.  The four 64-byte
// chunks of the block feed two v_mfma_f32_16x16x128_f8f6f4: lane (r, g)
// supplies its 16-byte pieces of chunks 0,1 to the first and of chunks 2,3 to the second - the
// same pieces for both operands, so the K permutation cancels.  The 128-wide instruction runs at
// the full FP8 rate of gfx950 (measured 4.9 PFLOP/s against 0.8-1.3 for v_mfma_f32_16x16x32_fp8_fp8).
template <int MT, int RG>
__device__ __forceinline__ void mma_block_256(const uint8_t* w, const uint8_t* x, f32x4 (&acc)[RG][MT]) {
    i32x8 xv[MT][2];
#pragma unroll
    for (int mt = 0; mt < MT; mt++)
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const i32x4 lo = *reinterpret_cast<const i32x4*>(x + mt * 4096 + (2 * h) * 256);
            const i32x4 hi = *reinterpret_cast<const i32x4*>(x + mt * 4096 + (2 * h + 1) * 256);
            xv[mt][h] = i32x8{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
        }
#pragma unroll
    for (int rg = 0; rg < RG; rg++)
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const i32x4 lo = *reinterpret_cast<const i32x4*>(w + rg * 4096 + (2 * h) * 256);
            const i32x4 hi = *reinterpret_cast<const i32x4*>(w + rg * 4096 + (2 * h + 1) * 256);
            const i32x8 wv = i32x8{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
#pragma unroll
            for (int mt = 0; mt < MT; mt++)
                acc[rg][mt] = mfma_e4m3_16x16x128(wv, xv[mt][h], acc[rg][mt]);
        }
}

// The last block of a K that is not a multiple of 256 (but of 16, and beyond 256): the stage was loaded from K - 256
// (a window that ends with the row, so nothing past it is read) and its first `old_bytes` = 256 - K % 256 bytes have been
// consumed with the block before.  A v_mfma whose two 64-byte chunks are both old is left out; elsewhere the old part
// of the activation operand is zero - whole chunks, and in the chunk the boundary runs through the 16-byte pieces
// below it: lane (r, g) holds piece g of every chunk (the DMA's rotation and the read offset cancel), so that is a
// per-lane select.  The products vanish whatever the weights are - unless a weight is NaN, which had poisoned its
// column with the block before already.
template <int MT, int RG>
__device__ __forceinline__ void mma_block_tail(const uint8_t* w, const uint8_t* x, f32x4 (&acc)[RG][MT], int old_bytes, int g) {
    const int first_chunk = old_bytes >> 6, first_piece = (old_bytes & 63) >> 4;   // wave-uniform
    const bool piece_old = g < first_piece;                                        // per lane
#pragma unroll
    for (int h = 0; h < 2; h++) {
        if (2 * h + 1 < first_chunk) continue;
        const bool lo_old = 2 * h < first_chunk || (2 * h == first_chunk && piece_old);
        const bool hi_old = 2 * h + 1 == first_chunk && piece_old;
        i32x8 xv[MT];
#pragma unroll
        for (int mt = 0; mt < MT; mt++) {
            i32x4 lo = *reinterpret_cast<const i32x4*>(x + mt * 4096 + (2 * h) * 256);
            i32x4 hi = *reinterpret_cast<const i32x4*>(x + mt * 4096 + (2 * h + 1) * 256);
            if (lo_old) lo = i32x4{0, 0, 0, 0};
            if (hi_old) hi = i32x4{0, 0, 0, 0};
            xv[mt] = i32x8{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
        }
#pragma unroll
        for (int rg = 0; rg < RG; rg++) {
            const i32x4 lo = *reinterpret_cast<const i32x4*>(w + rg * 4096 + (2 * h) * 256);
            const i32x4 hi = *reinterpret_cast<const i32x4*>(w + rg * 4096 + (2 * h + 1) * 256);
            const i32x8 wv = i32x8{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
#pragma unroll
            for (int mt = 0; mt < MT; mt++) acc[rg][mt] = mfma_e4m3_16x16x128(wv, xv[mt], acc[rg][mt]);
        }
    }
}

// Tiles of a persistent workgroup: one contiguous run (not a stride of gridDim.x), runs in XCD order.
struct TileRun { int first, count; };
__device__ __forceinline__ TileRun persistent_tile_run(int total_tiles) {
    const int groups = (int)gridDim.x, b = xcd_order((int)blockIdx.x, (int)gridDim.x);
    const int q = total_tiles / groups, rem = total_tiles % groups;
    return TileRun{b * q + (b < rem ? b : rem), q + (b < rem ? 1 : 0)};
}

constexpr int lds_stage_bytes(int RG, int XU) { return (RG * 4 + XU) * 1024; }
// Eight or more accumulator fragments per wave need more than the 128 VGPRs a 16-wave workgroup
// leaves each wave; those instantiations accept at most 8 waves per workgroup.
constexpr int lds_launch_bound(int MT, int RG) { return RG * MT >= 8 ? 512 : 1024; }
// The persistent kernels recompute their DMA addresses per stage instead of keeping one pointer
// per instruction, which costs temporaries: four fragments already overflow 128 VGPRs there.
constexpr int lds_persistent_launch_bound(int MT, int RG) { return RG * MT >= 4 ? 512 : 1024; }

// XU = activation DMA instructions per stage (4 rows each): ceil(min(m, 16*MT) / 4)
// HALF2 (RG == 2 only): 24-row tiles - the second 16-row fragment holds 8 weight rows, its other 8 are never fetched
// (the MFMA reads whatever lies there) and never stored.  6144 rows are 256 tiles of 24 where they are 384 of 16: one
// workgroup per CU instead of one and a half.
// TAIL: k not a multiple of 256 - the last K block is loaded from k - 256 and only its new bytes multiplied (a build of
// its own, so that the loop for whole blocks stays as it is).
template <int MT, int RG, int XU, int DEPTH, bool NT, bool HALF2 = false, bool TAIL = false>
__global__ void __launch_bounds__(lds_launch_bound(MT, RG)) lds_gemm_kernel(const StreamArgs a) {
    extern __shared__ __attribute__((aligned(1024))) uint8_t ring[];  // [wave][DEPTH][stage]
    __shared__ unsigned arrival;

    static_assert(!HALF2 || RG == 2, "24-row tiles are two fragments");
    constexpr int W_INSTR = HALF2 ? 6 : RG * 4;    // weight DMA instructions per stage (4 rows each)
    constexpr int TILE_ROWS = HALF2 ? 24 : 16 * RG;
    constexpr int PER_STAGE = W_INSTR + XU;        // DMA instructions per stage
    constexpr int STAGE_BYTES = PER_STAGE * 1024;
    static_assert((DEPTH - 1) * PER_STAGE <= 63, "ring deeper than vmcnt can count");
    static_assert(XU <= 4 * MT, "more activation rows than the tile has");

    Stamps stamps;
    stamps.begin();
    const int lane = lane_id();
    const int wave = wave_id();
    const int waves = a.waves;

    int tile_n, split, tile_m;
    decode_tile(a, xcd_order((int)blockIdx.x, (int)gridDim.x), tile_n, split, tile_m);
    const int n0 = tile_n * TILE_ROWS;
    const int m0 = tile_m * (16 * MT);

    // K range of this workgroup in 256-byte blocks; the last split takes the remainder
    // (k need not be a multiple of 256: the last block is then loaded from k - 256 and partly used)
    int b_begin, b_end;
    const int blocks_total = (a.k + 255) >> 8;
    split_range(a, blocks_total, split, b_begin, b_end);
    const int mine = blocks_of_wave(a, b_end - b_begin, wave);
    int tail_i = -1;                  // which of this wave's stages is the half block, if any: its last one
    if constexpr (TAIL) {
        if (b_end == blocks_total && mine > 0 && b_begin + wave + (mine - 1) * waves == blocks_total - 1) tail_i = mine - 1;
    }

    // ---- DMA sources: a wave-uniform base per operand (the tile's first row, advanced along K with scalar
    // adds) plus a 32-bit offset per lane and instruction (the host keeps 64 rows of either operand below 2 GB)
    const int q = lane >> 2, p = lane & 3;
    const int src_row = q & 3;        // row inside the 4-row instruction
    const int src_kc = q >> 2;        // 64-byte run inside the 256-byte block
    const uint8_t* w_base = a.B + (size_t)n0 * a.b_stride + ((size_t)(b_begin + wave) << 8);
    const uint8_t* x_base = a.A + (size_t)m0 * a.k + ((size_t)(b_begin + wave) << 8);
    const int w_last = a.n - 1 - n0, x_last = a.m - 1 - m0;   // rows past the edge re-read the last row, never stored
    unsigned woff[RG][4];
#pragma unroll
    for (int rg = 0; rg < RG; rg++)
#pragma unroll
        for (int u = 0; u < 4; u++) {
            int row = rg * 16 + 4 * u + src_row;
            row = row < w_last ? row : w_last;
            woff[rg][u] = (unsigned)row * (unsigned)a.b_stride + src_kc * 64 + ((p + u) & 3) * 16;
        }
    unsigned xoff[XU];
#pragma unroll
    for (int u = 0; u < XU; u++) {
        int row = 4 * u + src_row;
        row = row < x_last ? row : x_last;
        xoff[u] = (unsigned)row * (unsigned)a.k + src_kc * 64 + ((p + (u & 3)) & 3) * 16;
    }

    // ---- LDS read offsets (per lane) ------------------------------------------------------
    const int r = lane & 15, g = lane >> 4;
    const int rd_off = 1024 * (r >> 2) + 64 * (r & 3) + 16 * ((g - (r >> 2)) & 3);
    const uint8_t* my_ring = ring + (size_t)wave * (DEPTH * STAGE_BYTES);
    const unsigned my_ring_lds = lds_addr(my_ring);

    const size_t k_step = (size_t)waves << 8;
    auto issue = [&](int i) __attribute__((always_inline)) {  // i-th stage of this wave -> slot i % DEPTH
        const size_t koff = (size_t)i * k_step - ((TAIL && i == tail_i) ? (size_t)(256 - (a.k & 255)) : 0);
        const unsigned slot = my_ring_lds + (unsigned)(i % DEPTH) * STAGE_BYTES;
#pragma unroll
        for (int rg = 0; rg < RG; rg++)
#pragma unroll
            for (int u = 0; u < 4; u++) {
                if (rg * 4 + u >= W_INSTR) continue;
                if (NT) dma_1kb_stream_at(w_base + koff, woff[rg][u], slot + (rg * 4 + u) * 1024);
                else dma_1kb_at(w_base + koff, woff[rg][u], slot + (rg * 4 + u) * 1024);
            }
#pragma unroll
        for (int u = 0; u < XU; u++) dma_1kb_at(x_base + koff, xoff[u], slot + (W_INSTR + u) * 1024);
    };

    f32x4 acc[RG][MT];
#pragma unroll
    for (int rg = 0; rg < RG; rg++)
#pragma unroll
        for (int mt = 0; mt < MT; mt++) acc[rg][mt] = f32x4{0.f, 0.f, 0.f, 0.f};

    auto consume = [&](int i) __attribute__((always_inline)) {
        const uint8_t* slot = my_ring + (size_t)(i % DEPTH) * STAGE_BYTES + rd_off;
        mma_block_256<MT, RG>(slot, slot + W_INSTR * 1024, acc);
    };
    auto consume_last = [&](int i) __attribute__((always_inline)) {   // this wave's last stage: whole or half
        const uint8_t* slot = my_ring + (size_t)(i % DEPTH) * STAGE_BYTES + rd_off;
        if (TAIL && i == tail_i) mma_block_tail<MT, RG>(slot, slot + W_INSTR * 1024, acc, 256 - (a.k & 255), g);
        else mma_block_256<MT, RG>(slot, slot + W_INSTR * 1024, acc);
    };

    if (mine >= DEPTH) {
#pragma unroll
        for (int d = 0; d < DEPTH; d++) issue(d);
        stamps.mark(1);
        int i = 0;
        for (; i + DEPTH < mine; i++) {
            wait_vmcnt<(DEPTH - 1) * PER_STAGE>();   // stage i has landed; DEPTH-1 stages still in flight
            if (i == 0) stamps.mark(2);
            consume(i);
            // the slot is refilled only after its reads have returned: the MFMAs above need the
            // data, and this wait keeps the DMA behind them
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            __builtin_amdgcn_sched_barrier(0);
            issue(i + DEPTH);
            __builtin_amdgcn_sched_barrier(0);
        }
        if constexpr (TAIL) drain_ring<0, DEPTH, PER_STAGE>(consume, consume_last, i);
        else drain_ring<0, DEPTH, PER_STAGE>(consume, i);
    } else {
        for (int i = 0; i < mine; i++) issue(i);
        stamps.mark(1);
        wait_vmcnt<0>();
        stamps.mark(2);
        if constexpr (TAIL) {
            for (int i = 0; i + 1 < mine; i++) consume(i);
            if (mine > 0) consume_last(mine - 1);
        } else {
            for (int i = 0; i < mine; i++) consume(i);
        }
    }

    // the ring is reused for the cross-wave reduction: every wave must be done reading it
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    stamps.mark(3);
    __syncthreads();
    finish_tile<RG, MT>(a, acc, reinterpret_cast<f32x4*>(ring), &arrival, tile_m, tile_n, split, m0, n0, n0 + TILE_ROWS);
    stamps.end(a);
}

// bf16 activations -> E4M3 codes in the resident-activation layout of the persistent kernel, quantised per row
// exactly as sg_fp8_encode_rows does (same arithmetic, sg_quant.h), by the workgroup that is about to use them.
// Replaces the activation DMA of the resident kernel: K block kb is handled by wave kb % waves (the only wave that
// will read it), and lane l of "instruction" u produces the 16 bytes the DMA would have put at (kb*XU + u) KB + 16*l:
// row 4u + (l/4)%4, k = 256 kb + 64 (l/16) + 16 ((l + u) % 4) .. +15.
//
// Order of events: the wave loads its share of the bf16 activations and takes the row maxima of it (load_and_max);
// the caller then issues the prologue DMAs of the weight ring; finish() combines the maxima of all waves (one
// barrier), derives the scales and writes the codes - while the weights are arriving.  A wave keeps at most 8 chunks
// of 16 values in registers between the two steps (64 registers); a larger share - long K - is read a second time
// (from L2).  Every wave of the workgroup calls both steps exactly once; the caller's next barrier publishes the
// codes and `xscale`.
template <int XU>
struct ActivationQuantizer {
    static constexpr int KB_MAX = XU >= 8 ? 1 : 8 / XU;   // K blocks of a wave whose chunks fit 64 registers
    u32x4 raw[KB_MAX][XU][2];
    float pm[XU];
    int row[XU];
    unsigned koff[XU];
    int kb0, nkb, rr;

    __device__ __forceinline__ const u32x4* chunk(const StreamArgs& a, int kb, int u) const {
        return reinterpret_cast<const u32x4*>(a.A16 + (size_t)row[u] * a.k + ((size_t)kb << 8) + koff[u]);
    }

    __device__ __forceinline__ void load_and_max(const StreamArgs& a, int blocks, int waves, int wave, int lane) {
        rr = (lane >> 2) & 3;
        const int col = (lane >> 4) * 64;
#pragma unroll
        for (int u = 0; u < XU; u++) {
            const int r = 4 * u + rr;
            row[u] = r < a.m ? r : a.m - 1;          // rows past the edge repeat the last row, as the DMA does
            koff[u] = col + (((lane & 3) + (u & 3)) & 3) * 16;
            pm[u] = 0.0f;
        }
        kb0 = wave < waves ? wave : blocks;
        nkb = kb0 < blocks ? (blocks - kb0 + waves - 1) / waves : 0;
        if (nkb <= KB_MAX) {
#pragma unroll
            for (int i = 0; i < KB_MAX; i++)
#pragma unroll
                for (int u = 0; u < XU; u++) {
                    raw[i][u][0] = raw[i][u][1] = u32x4{0u, 0u, 0u, 0u};
                    if (i < nkb) {
                        const u32x4* src = chunk(a, kb0 + i * waves, u);
                        raw[i][u][0] = src[0];
                        raw[i][u][1] = src[1];
                    }
                }
#pragma unroll
            for (int i = 0; i < KB_MAX; i++)
#pragma unroll
                for (int u = 0; u < XU; u++) pm[u] = absmax8_bf16(raw[i][u][1], absmax8_bf16(raw[i][u][0], pm[u]));
        } else {
            for (int kb = kb0; kb < blocks; kb += waves)
#pragma unroll
                for (int u = 0; u < XU; u++) {
                    const u32x4* src = chunk(a, kb, u);
                    pm[u] = absmax8_bf16(src[1], absmax8_bf16(src[0], pm[u]));
                }
        }
    }

    __device__ __forceinline__ void finish(const StreamArgs& a, uint8_t* xres, float* wmax, float* xscale, int blocks, int waves,
                                           int wave, int lane) {
        // lanes that share a row for a given u differ in lane bits 0, 1, 4, 5
#pragma unroll
        for (int u = 0; u < XU; u++) {
            pm[u] = fmaxf(pm[u], __shfl_xor(pm[u], 1));
            pm[u] = fmaxf(pm[u], __shfl_xor(pm[u], 2));
            pm[u] = fmaxf(pm[u], __shfl_xor(pm[u], 16));
            pm[u] = fmaxf(pm[u], __shfl_xor(pm[u], 32));
        }
        if (wave < waves && (lane & 0x33) == 0) {
#pragma unroll
            for (int u = 0; u < XU; u++) wmax[wave * 32 + 4 * u + rr] = pm[u];
        }
        __syncthreads();
        RowQuant rq[XU];
#pragma unroll
        for (int u = 0; u < XU; u++) {
            float amax = 0.0f;
            for (int w = 0; w < waves; w++) amax = fmaxf(amax, wmax[w * 32 + 4 * u + rr]);
            rq[u] = row_quant(amax);
        }
        if (wave == 0 && (lane & 0x33) == 0) {
#pragma unroll
            for (int u = 0; u < XU; u++) {
                xscale[4 * u + rr] = rq[u].s;
                if (a.row_scale_out && blockIdx.x == 0 && 4 * u + rr < a.m) a.row_scale_out[4 * u + rr] = rq[u].s;
            }
        }
        if (nkb <= KB_MAX) {
#pragma unroll
            for (int i = 0; i < KB_MAX; i++) {
                if (i < nkb) {
#pragma unroll
                    for (int u = 0; u < XU; u++) {
                        const u32x2 lo = quantize8_bf16(raw[i][u][0], rq[u]), hi = quantize8_bf16(raw[i][u][1], rq[u]);
                        *reinterpret_cast<u32x4*>(xres + (size_t)((kb0 + i * waves) * XU + u) * 1024 + 16 * lane) =
                            u32x4{lo.x, lo.y, hi.x, hi.y};
                    }
                }
            }
        } else {
            for (int kb = kb0; kb < blocks; kb += waves)
#pragma unroll
                for (int u = 0; u < XU; u++) {
                    const u32x4* src = chunk(a, kb, u);
                    const u32x2 lo = quantize8_bf16(src[0], rq[u]), hi = quantize8_bf16(src[1], rq[u]);
                    *reinterpret_cast<u32x4*>(xres + (size_t)(kb * XU + u) * 1024 + 16 * lane) = u32x4{lo.x, lo.y, hi.x, hi.y};
                }
        }
    }
};

// ---------------------------------------------------------------------------------------------
// Persistent variant for shapes with many more tiles than CUs.  A workgroup walks a contiguous
// run of tiles (persistent_tile_run) and every wave's ring simply continues across the
// tile boundary: while the waves meet to reduce and store tile j, the DMAs of tile j+1 are
// already in flight, so HBM never sees the ramp-down / ramp-up of a workgroup hand-over.
// (The reference's kernel is persistent for the same reason: skinny_gemm_kernel.cu:44-51.)
// The reduction scratch is double-buffered by tile parity, which leaves one barrier per tile.
// No cross-workgroup split-K in this variant.
// QUANT: the activations arrive as bf16 (a.A16) and the workgroup quantises them itself (ActivationQuantizer); a separate
// instantiation with room for 9 waves of 168 registers (the chunks it holds between its two steps), so that the
// ordinary kernel keeps its registers.
constexpr int kQuantThreads = 576;
template <int MT, int RG, int XU, int DEPTH, bool NT, bool XRES, bool QUANT = false>
__global__ void __launch_bounds__(QUANT ? kQuantThreads : lds_persistent_launch_bound(MT, RG))
lds_gemm_persistent_kernel(const StreamArgs a) {
    static_assert(!QUANT || XRES, "in-kernel quantisation writes the resident-activation layout");
    // XRES: [X blocks][XU KB] | [wave][DEPTH][RG*4 KB] | red;  else: [wave][DEPTH][(RG*4 + XU) KB] | red[2][FRAGS][wave][64]
    extern __shared__ __attribute__((aligned(1024))) uint8_t ring[];

    constexpr int PER_STAGE = XRES ? RG * 4 : RG * 4 + XU;
    constexpr int STAGE_BYTES = PER_STAGE * 1024;
    constexpr int FRAGS = RG * MT;
    static_assert((DEPTH - 1) * PER_STAGE <= 63, "ring deeper than vmcnt can count");

    Stamps stamps;
    stamps.begin();
    const int lane = lane_id();
    const int wave = wave_id();
    const int waves = a.waves;
    const int r = lane & 15, g = lane >> 4;

    const int total_tiles = a.n_tiles * a.m_tiles;
    const TileRun run = persistent_tile_run(total_tiles);
    const int my_tiles = run.count;
    const int blocks = a.k >> 8;
    // a workgroup launched with one wave more than a.waves has a dedicated epilogue wave: it
    // streams nothing and does every reduction and store, so that the streaming waves never have
    // a store in their vmcnt queue (a store younger than the ring's DMAs makes every later
    // vmcnt(n) wait for one DMA more than needed until the store is acknowledged)
    const bool epilogue_wave = blockDim.x > (unsigned)waves * 64;
    const int per_tile = wave < waves ? blocks_of_wave(a, blocks, wave) : 0;
    const int total = per_tile * my_tiles;

    const int q = lane >> 2, p = lane & 3;
    const int src_row = q & 3;
    const int src_col = (q >> 2) * 64;
    const int rd_off = 1024 * (r >> 2) + 64 * (r & 3) + 16 * ((g - (r >> 2)) & 3);
    const int x_bytes = XRES ? blocks * XU * 1024 : 0;   // resident activations (needs m_tiles == 1)
    const uint8_t* my_ring = ring + x_bytes + (size_t)wave * (DEPTH * STAGE_BYTES);
    const unsigned my_ring_lds = lds_addr(my_ring);
    f32x4* red = reinterpret_cast<f32x4*>(ring + x_bytes + (size_t)waves * (DEPTH * STAGE_BYTES));
    // bf16 activations quantised here (resident kernel only): the row scales live behind the reduction scratch
    constexpr bool quant = QUANT;
    float* xscale = reinterpret_cast<float*>(red + (size_t)2 * FRAGS * waves * 64);
    const float* row_factors = quant ? xscale : nullptr;

    // Tiles are walked n fastest.  Both the issuing and the finishing side keep their tile's (n, m) coordinates as
    // counters that are stepped when a tile ends: dividing by run-time values per stage (tile index, tile
    // coordinates) cost about 0.8 us in front of the first DMA and delayed every refill.
    const unsigned first_m = fast_div((unsigned)run.first, (unsigned)a.n_tiles, a.inv_n_tiles);
    const int first_n = run.first - (int)first_m * a.n_tiles;
    int iss_tn = first_n, iss_tm = (int)first_m, iss_r = 0;     // tile and stage-in-tile of the next stage to issue
    int fin_tn = first_n, fin_tm = (int)first_m;                // tile the next tile_done() finishes

    // per-lane parts of the DMA addresses: row inside the tile and byte offset inside the 256-byte K block; the rest
    // of an address (tile origin, K block) is wave-uniform and travels in scalar registers
    int wrow[RG][4];
    unsigned wcol[4];
#pragma unroll
    for (int u = 0; u < 4; u++) {
        wcol[u] = src_col + ((p + u) & 3) * 16;
#pragma unroll
        for (int rg = 0; rg < RG; rg++) wrow[rg][u] = rg * 16 + 4 * u + src_row;
    }

    auto issue = [&](int i) __attribute__((always_inline)) {   // called for i = 0, 1, 2, ... in order
        const int kb = wave + iss_r * waves;
        const int n0 = iss_tn * (16 * RG), m0 = iss_tm * (16 * MT);
        const unsigned slot = my_ring_lds + (unsigned)(i % DEPTH) * STAGE_BYTES;
        const uint8_t* w_base = a.B + (size_t)n0 * a.b_stride + ((size_t)kb << 8);
        const int w_last = a.n - 1 - n0;     // rows past the edge re-read the last row, never stored
#pragma unroll
        for (int rg = 0; rg < RG; rg++)
#pragma unroll
            for (int u = 0; u < 4; u++) {
                const int row = wrow[rg][u] < w_last ? wrow[rg][u] : w_last;
                const unsigned voff = (unsigned)row * (unsigned)a.b_stride + wcol[u];
                if (NT) dma_1kb_stream_at(w_base, voff, slot + (rg * 4 + u) * 1024);
                else dma_1kb_at(w_base, voff, slot + (rg * 4 + u) * 1024);
            }
        if (!XRES) {
            const uint8_t* x_base = a.A + (size_t)m0 * a.k + ((size_t)kb << 8);
            const int x_last = a.m - 1 - m0;
#pragma unroll
            for (int u = 0; u < XU; u++) {
                int row = 4 * u + src_row;
                row = row < x_last ? row : x_last;
                dma_1kb_at(x_base, (unsigned)row * (unsigned)a.k + wcol[u & 3], slot + (RG * 4 + u) * 1024);
            }
        }
        if (++iss_r == per_tile) {
            iss_r = 0;
            if (++iss_tn == a.n_tiles) {
                iss_tn = 0;
                iss_tm++;
            }
        }
    };

    f32x4 acc[RG][MT];
#pragma unroll
    for (int rg = 0; rg < RG; rg++)
#pragma unroll
        for (int mt = 0; mt < MT; mt++) acc[rg][mt] = f32x4{0.f, 0.f, 0.f, 0.f};

    int left_in_tile = per_tile;  // stages of the current tile not yet consumed
    auto consume = [&](int i) __attribute__((always_inline)) {
        const uint8_t* slot = my_ring + (size_t)(i % DEPTH) * STAGE_BYTES + rd_off;
        // activations: in the stage, or in the resident copy at this stage's K block
        const uint8_t* xs = XRES ? ring + (size_t)(wave + (per_tile - left_in_tile) * waves) * (XU * 1024) + rd_off
                                 : slot + RG * 4096;
        mma_block_256<MT, RG>(slot, xs, acc);
    };

    const float scale = a.scale ? a.scale[0] : 1.0f;
    int red_turn = 0;
    // Reduce the waves' partial tiles of the j-th tile in wave order, scale, round, store.
    auto tile_done = [&](int j) __attribute__((always_inline)) {
        const int n0 = fin_tn * (16 * RG), m0 = fin_tm * (16 * MT);
        if (++fin_tn == a.n_tiles) {
            fin_tn = 0;
            fin_tm++;
        }
        if (waves == 1 && !epilogue_wave) {
#pragma unroll
            for (int f = 0; f < FRAGS; f++)
                store_fragment(a, acc[f / MT][f % MT], scale, m0 + (f % MT) * 16 + r, n0 + (f / MT) * 16 + 4 * g, row_factors);
        } else {
            f32x4* buf = red + (size_t)(j & 1) * (FRAGS * waves * 64);
            if (wave < waves) {
#pragma unroll
                for (int f = 0; f < FRAGS; f++) buf[(f * waves + wave) * 64 + lane] = acc[f / MT][f % MT];
            }
            // per-column factors of this tile, requested before the barrier: fetched when needed, their memory
            // latency (a different line per tile) would be paid once per tile by the wave that stores
            f32x4 colf[RG];
#pragma unroll
            for (int rg = 0; rg < RG; rg++) colf[rg] = col_scale_ahead(a, n0 + rg * 16 + 4 * g);
            __syncthreads();
            // without an epilogue wave the reducing wave rotates with the tile, so that the cost is
            // spread over the waves
            int first = wave - red_turn, step = waves;        // red_turn = j % waves, kept as a counter
            first = first < 0 ? first + waves : first;
            red_turn = red_turn + 1 == waves ? 0 : red_turn + 1;
            if (epilogue_wave) {
                first = wave == waves ? 0 : FRAGS;
                step = 1;
            }
            for (int f = first; f < FRAGS; f += step) {
                f32x4 v = buf[(f * waves) * 64 + lane];
                for (int w = 1; w < waves; w++) v += buf[(f * waves + w) * 64 + lane];
                f32x4 cf = colf[0];    // colf[f / MT] without indexing registers by a run-time value
#pragma unroll
                for (int rg = 1; rg < RG; rg++)
                    if (f / MT == rg) cf = colf[rg];
                store_fragment(a, v, scale, m0 + (f % MT) * 16 + r, n0 + (f / MT) * 16 + 4 * g, row_factors, &cf);
            }
        }
#pragma unroll
        for (int rg = 0; rg < RG; rg++)
#pragma unroll
            for (int mt = 0; mt < MT; mt++) acc[rg][mt] = f32x4{0.f, 0.f, 0.f, 0.f};
    };

    ActivationQuantizer<QUANT ? XU : 1> aq;
    if constexpr (quant) aq.load_and_max(a, blocks, waves, wave, lane);   // before the weight prologue: see ActivationQuantizer
    if (XRES && !quant) {
        // K block kb of the activations is fetched by wave kb % waves; every wave then starts its
        // weight ring, waits for its own share (older than the ring's DMAs) and meets the others
        const unsigned x_lds = lds_addr(ring);
        int x_issued = 0;
        for (int kb = wave < waves ? wave : blocks; kb < blocks; kb += waves) {
#pragma unroll
            for (int u = 0; u < XU; u++) {
                int row = 4 * u + src_row;
                row = row < a.m ? row : a.m - 1;
                dma_1kb(a.A + (size_t)row * a.k + ((size_t)kb << 8) + src_col + ((p + (u & 3)) & 3) * 16,
                        x_lds + (unsigned)(kb * XU + u) * 1024);
            }
            x_issued += XU;
        }
        (void)x_issued;
    }

    if (per_tile == 0) {  // more waves than K blocks: this wave only takes part in the reductions
        if constexpr (quant) aq.finish(a, ring, reinterpret_cast<float*>(red), xscale, blocks, waves, wave, lane);
        if (XRES) {
            wait_vmcnt<0>();
            __syncthreads();
        }
        for (int j = 0; j < my_tiles; j++) tile_done(j);
        return;
    }

    // stage i ends a tile when it is this wave's last K block of that tile
    int tile_j = 0;
    auto after_consume = [&]() __attribute__((always_inline)) {
        if (--left_in_tile == 0) {
            tile_done(tile_j++);
            left_in_tile = per_tile;
        }
    };

    if (total >= DEPTH) {
#pragma unroll
        for (int d = 0; d < DEPTH; d++) issue(d);
        stamps.mark(1);
        // the weights are on their way; meanwhile the workgroup quantises its copy of the activations
        if constexpr (quant) aq.finish(a, ring, reinterpret_cast<float*>(red), xscale, blocks, waves, wave, lane);
        if (XRES) {
            wait_vmcnt_upto(DEPTH * PER_STAGE);   // this wave's activation blocks are older than its DEPTH stages
            __syncthreads();
        }
        int i = 0;
        for (; i + DEPTH < total; i++) {
            wait_vmcnt<(DEPTH - 1) * PER_STAGE>();
            if (i == 0) stamps.mark(2);
            consume(i);
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            __builtin_amdgcn_sched_barrier(0);
            issue(i + DEPTH);
            __builtin_amdgcn_sched_barrier(0);
            after_consume();
        }
        auto consume_and_close = [&](int ii) __attribute__((always_inline)) {
            consume(ii);
            after_consume();
        };
        drain_ring<0, DEPTH, PER_STAGE>(consume_and_close, i);
    } else {
        for (int i = 0; i < total; i++) issue(i);
        if constexpr (quant) aq.finish(a, ring, reinterpret_cast<float*>(red), xscale, blocks, waves, wave, lane);
        wait_vmcnt<0>();
        if (XRES) __syncthreads();
        for (int i = 0; i < total; i++) {
            consume(i);
            after_consume();
        }
    }
    stamps.mark(3);   // here the last tile's reduction is part of [3]: the streaming waves run into it
    stamps.end(a);
}

// ---------------------------------------------------------------------------------------------
// Wave-per-tile variant with the activations resident in LDS, for shapes with many tiles and a
// short K (the MLP up-projection): every wave owns whole 16*RG-row tiles over the full K range,
// so there is no cross-wave reduction and no barrier after the prologue.  The whole activation
// matrix (ceil(m/4) KB per 256-byte K block) is fetched once per workgroup and shared by its
// waves, which removes a third of the DMA instructions and of the L2 traffic at m = 8.  Wave
// (workgroup b, wave w) walks tiles b + G*w, + total waves, ...; its weight ring runs across
// tile boundaries.
// TAIL: k not a multiple of 256 - K block `blocks - 1` of both operands is loaded from k - 256 and only its new bytes
// multiplied (mma_block_tail), as in lds_gemm_kernel.
template <int MT, int RG, int XU, int DEPTH, bool NT, bool TAIL = false>
__global__ void __launch_bounds__(lds_persistent_launch_bound(MT, RG)) lds_gemm_wavetile_kernel(const StreamArgs a) {
    extern __shared__ __attribute__((aligned(1024))) uint8_t ring[];  // X[blocks][XU KB] | [wave][DEPTH][RG*4 KB]

    constexpr int PER_STAGE = RG * 4;
    constexpr int STAGE_BYTES = PER_STAGE * 1024;
    constexpr int FRAGS = RG * MT;
    static_assert((DEPTH - 1) * PER_STAGE <= 63, "ring deeper than vmcnt can count");
    static_assert(MT == 1 || XU > 4, "two activation blocks need more than four DMA instructions");

    const int lane = lane_id();
    const int wave = wave_id();
    const int waves = a.waves;
    const int r = lane & 15, g = lane >> 4;

    const int blocks = (a.k + 255) >> 8;
    const size_t tail_shift = TAIL ? (size_t)(256 - (a.k & 255)) : 0;   // how far the last block's window starts early
    const int total_tiles = a.n_tiles * a.m_tiles;
    // tiles are dealt to workgroups first (wave w of workgroup b owns tiles b + G*w, b + G*(w + W), ...), so that a
    // few tiles per CU still put a stream on every CU
    const int total_waves = (int)gridDim.x * waves;
    const int first = (int)blockIdx.x + (int)gridDim.x * wave;
    const int my_tiles = first < total_tiles ? (total_tiles - first + total_waves - 1) / total_waves : 0;
    const int total = blocks * my_tiles;
    const int gw = (int)blockIdx.x * waves + wave;   // for the K rotation: neighbours in a workgroup start one block apart
    // Every wave starts its tiles at a different K block and wraps around.  Here all waves of the chip would
    // otherwise ask for block kb of their rows at the same moment, and row pitches are multiples of 4 KB: in step,
    // 8 x 28672 x 4096 takes 24.6 us, spread over all K offsets 19.6 us (eight waves, same process, interleaved).
    // The persistent K-split kernel above already has its waves at different K offsets and measured 1 % slower
    // with a shift per workgroup on top; it keeps plain K order.
    const int k_rot = (int)((unsigned)gw % (unsigned)blocks);

    const int q = lane >> 2, p = lane & 3;
    const int src_row = q & 3;
    const int src_col = (q >> 2) * 64;
    const int rd_off = 1024 * (r >> 2) + 64 * (r & 3) + 16 * ((g - (r >> 2)) & 3);
    const int x_bytes = blocks * XU * 1024;
    const uint8_t* my_ring = ring + x_bytes + (size_t)wave * (DEPTH * STAGE_BYTES);
    const unsigned my_ring_lds = lds_addr(my_ring);
    const unsigned x_lds = lds_addr(ring);

    // ---- resident activations: K block kb is fetched by wave kb % waves (m_tiles == 1) ----------
    int x_issued = 0;
    for (int kb = wave; kb < blocks; kb += waves) {
#pragma unroll
        for (int u = 0; u < XU; u++) {
            int row = 4 * u + src_row;
            row = row < a.m ? row : a.m - 1;
            dma_1kb(a.A + (size_t)row * a.k + ((size_t)kb << 8) - ((TAIL && kb == blocks - 1) ? tail_shift : 0) + src_col +
                        ((p + (u & 3)) & 3) * 16,
                    x_lds + (unsigned)(kb * XU + u) * 1024);
        }
        x_issued += XU;
    }

    auto issue = [&](int i) __attribute__((always_inline)) {
        const int j = i / blocks;
        int kb = i - j * blocks + k_rot;
        kb = kb >= blocks ? kb - blocks : kb;
        const int n0 = ((first + j * total_waves) % a.n_tiles) * (16 * RG);
        const unsigned slot = my_ring_lds + (unsigned)(i % DEPTH) * STAGE_BYTES;
        const size_t koff = ((size_t)kb << 8) - ((TAIL && kb == blocks - 1) ? tail_shift : 0) + src_col;
#pragma unroll
        for (int rg = 0; rg < RG; rg++)
#pragma unroll
            for (int u = 0; u < 4; u++) {
                int row = n0 + rg * 16 + 4 * u + src_row;
                row = row < a.n ? row : a.n - 1;
                const uint8_t* src = a.B + (size_t)row * a.b_stride + koff + ((p + u) & 3) * 16;
                if (NT) dma_1kb_stream(src, slot + (rg * 4 + u) * 1024);
                else dma_1kb(src, slot + (rg * 4 + u) * 1024);
            }
    };

    f32x4 acc[RG][MT];
#pragma unroll
    for (int rg = 0; rg < RG; rg++)
#pragma unroll
        for (int mt = 0; mt < MT; mt++) acc[rg][mt] = f32x4{0.f, 0.f, 0.f, 0.f};

    int kb_cur = 0;  // stages of the current tile already consumed
    auto consume = [&](int i) __attribute__((always_inline)) {
        const uint8_t* slot = my_ring + (size_t)(i % DEPTH) * STAGE_BYTES + rd_off;
        const int kb = kb_cur + k_rot >= blocks ? kb_cur + k_rot - blocks : kb_cur + k_rot;   // the K block it holds
        if (TAIL && kb == blocks - 1) mma_block_tail<MT, RG>(slot, ring + (size_t)kb * (XU * 1024) + rd_off, acc, (int)tail_shift, g);
        else mma_block_256<MT, RG>(slot, ring + (size_t)kb * (XU * 1024) + rd_off, acc);
    };

    const float scale = a.scale ? a.scale[0] : 1.0f;
    int tile_j = 0;
    auto after_consume = [&]() __attribute__((always_inline)) {
        if (++kb_cur == blocks) {   // the tile is complete: scale, round, store, start the next one
            kb_cur = 0;
            const int n0 = ((first + tile_j * total_waves) % a.n_tiles) * (16 * RG);
            tile_j++;
#pragma unroll
            for (int f = 0; f < FRAGS; f++) {
                store_fragment(a, acc[f / MT][f % MT], scale, (f % MT) * 16 + r, n0 + (f / MT) * 16 + 4 * g);
                acc[f / MT][f % MT] = f32x4{0.f, 0.f, 0.f, 0.f};
            }
        }
    };

    // weight prologue first, so that HBM is busy while the activations arrive from L2
    const int pro = total < DEPTH ? total : DEPTH;
    for (int d = 0; d < pro; d++) issue(d);
    // this wave's share of the activations was issued before its weight stages: once at most
    // pro * PER_STAGE DMAs are outstanding it has landed; the barrier publishes everyone's share
    if (x_issued > 0) wait_vmcnt_upto(pro * PER_STAGE);
    __syncthreads();

    if (total >= DEPTH) {
        int i = 0;
        for (; i + DEPTH < total; i++) {
            wait_vmcnt<(DEPTH - 1) * PER_STAGE>();
            consume(i);
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            __builtin_amdgcn_sched_barrier(0);
            issue(i + DEPTH);
            __builtin_amdgcn_sched_barrier(0);
            after_consume();
        }
        auto consume_and_close = [&](int ii) __attribute__((always_inline)) {
            consume(ii);
            after_consume();
        };
        drain_ring<0, DEPTH, PER_STAGE>(consume_and_close, i);
    } else {
        wait_vmcnt<0>();
        for (int i = 0; i < total; i++) {
            consume(i);
            after_consume();
        }
    }
}

}  // namespace sg
