// 2:4 structured-sparse FP8 skinny GEMM for gfx950:
//     D[m,n] = scale * sum_k A[m,k] * Bdense[n,k],   Bdense = decompress(vals, meta)
// with the weights stored compressed: vals[n][k/2] (the two kept E4M3 codes of every group of
// four consecutive k) and meta[n][k/8] (one nibble per group: low two bits = position of the
// first kept value, high two bits = position of the second; group 2u in the low nibble of
// byte u).  No counterpart in the reference: its "sparse" kernels feed a DENSE activation tile
// through the sparse instruction (skinny_gemm/consumers/smfma_16x16x64_consumer.cu:86-92);
// here the compressed WEIGHTS are the sparse operand, which is what the instruction is for.
//
// v_smfmac_f32_16x16x64_fp8_fp8: first operand 16 sparse rows (weight rows n) x 64 dense k,
// of which lane (r = l%16, g = l/16) supplies the 8 stored bytes of its 16-k window plus 16
// index bits; second operand 16 columns (activation rows m) x 64 k, lane (c, g) supplying the
// 16 dense bytes of the same window.  The window a lane works on is free as long as both
// operands agree, so per 512-k stage lane g owns k range [128 g, 128 g + 128): 64 contiguous
// stored bytes, 16 contiguous metadata bytes and 128 contiguous activation bytes, consumed in
// eight steps of 16 k.  Per step the index bits are two metadata bytes, already in the order
// the instruction wants (group j of the window in bits 4j..4j+3).
//
// Streaming: same direct-to-LDS ring as the dense kernel (sg_lds_kernel.h) - 4 rows x 256
// contiguous bytes per DMA instruction for values and activations, 16 rows x 64 bytes for the
// metadata - with the 16-byte pieces of each row XOR-swizzled by the row number so that all
// LDS reads are conflict-free.  HBM traffic per weight row is 0.625 bytes per dense k.
//
// Metadata by whole cache lines (builds with PAIRS; K a multiple of 1024): 64 bytes per row and stage are half a
// 128-byte line, so every metadata line is requested twice by the CU's L1, the second time as an L2 hit that waits
// behind the misses around it - 48 requests per stage for 40 lines.  Asking once takes 10 % of the L1's requests away
// and 0-5 % of the time on the 4096 x 14336 and 14336 x 4096 shapes (most at 16 rows on K = 14336).  A PAIRS
// build takes its stages two at a time, (2P, 2P + 1), whose metadata is one aligned line per row: stage i carries,
// next to its own values, the lines of rows 8h..8h+7 (h = i % 2) for the pair after its own, P = i / 2 + 1, into a ring of
// DEPTH / 2 + 2 pair slots of its own; the first pair's lines go ahead of everything.  DMAs complete in order, so when
// the values of stage 2P have landed so have both halves of pair P's metadata; a pair slot is refilled only after the
// pair DEPTH / 2 + 2 before it has been multiplied.  Every stage still issues the same number of DMA instructions (past
// the last pair the line of the last pair is fetched again into a free slot), so the vmcnt arithmetic is unchanged.
//
// K that 512 does not divide (any multiple of 128 from 512 on; builds with TAIL): the last stage is loaded from the
// window [k - 512, k), which ends with the row, so nothing past a row is read and all three streams stay 16-byte
// aligned.  The 128-k pieces at the front of that window were already multiplied in the stage before; the lanes that
// own them (g < 4 - (k % 512) / 128) replace their activation bytes by zeros for that stage.
#pragma once

#include "sg_device.h"
#include "sg_epilogue.h"
#include "sg_lds_kernel.h"

namespace sg {

struct SparseArgs {
    StreamArgs g;          // g.B = vals (row stride k/2); shapes as for the dense kernels
    const uint8_t* meta;   // [n][k/8]
};

// A stage's activation fragments alone take 32*MT registers; two activation blocks or four row
// tiles per wave do not fit the 128 VGPRs a 16-wave workgroup leaves each wave.
constexpr int sparse_launch_bound(int MT, int RG) { return (MT == 2 || RG == 4) ? 512 : 1024; }

// LDS of one wave: DEPTH stages of RG x (4 KB of values + 1 KB of metadata) [+ XU2 KB of activations]; with PAIRS the
// metadata lives in its own ring of DEPTH / 2 + 2 pair slots of RG x 2 KB instead.
constexpr int sparse_meta_pairs(int DEPTH) { return DEPTH / 2 + 2; }
constexpr int sparse_stage_bytes(int RG, int XU2, bool PAIRS) { return (RG * (PAIRS ? 4 : 5) + XU2) * 1024; }
constexpr int sparse_wave_bytes(int RG, int XU2, int DEPTH, bool PAIRS) {
    return DEPTH * sparse_stage_bytes(RG, XU2, PAIRS) + (PAIRS ? sparse_meta_pairs(DEPTH) * RG * 2048 : 0);
}

// XU2 = activation DMA instructions per stage: 2 halves x ceil(rows/4)
template <int MT, int RG, int XU2, int DEPTH, bool TAIL, bool PAIRS>
__global__ void __launch_bounds__(sparse_launch_bound(MT, RG)) sparse24_gemm_kernel(const SparseArgs sa) {
    extern __shared__ __attribute__((aligned(1024))) uint8_t ring[];  // [wave][DEPTH][stage] (PAIRS: + [pair slot][rg][2 KB])
    __shared__ unsigned arrival;
    const StreamArgs& a = sa.g;
    Stamps stamps;
    stamps.begin();

    constexpr int PER_STAGE = RG * 5 + XU2;   // DMA instructions per stage
    constexpr int W_TILE = PAIRS ? 4096 : 5120;   // a row tile's part of a stage: 4 KB values [| 1 KB metadata]
    constexpr int STAGE_BYTES = sparse_stage_bytes(RG, XU2, PAIRS);
    constexpr int X_OFF = RG * W_TILE;        // stage: row tiles ... | activations
    constexpr int NP = sparse_meta_pairs(DEPTH);
    constexpr int WAVE_BYTES = sparse_wave_bytes(RG, XU2, DEPTH, PAIRS);
    static_assert((DEPTH - 1) * PER_STAGE <= 63, "ring deeper than vmcnt can count");
    static_assert(XU2 <= 8 * MT, "more activation rows than the tile has");
    static_assert(!(TAIL && PAIRS), "whole metadata lines need K in whole pairs of stages");

    const int lane = lane_id();
    const int wave = wave_id();
    const int waves = a.waves;

    int tile_n, split, tile_m;
    decode_tile(a, xcd_order((int)blockIdx.x, (int)gridDim.x), tile_n, split, tile_m);
    const int n0 = tile_n * (16 * RG);
    const int m0 = tile_m * (16 * MT);

    int b_begin, b_end;                                 // in stages; PAIRS: in pairs of stages
    const int full = a.k >> 9;                          // whole 512-k stages
    split_range(a, PAIRS ? full >> 1 : (TAIL ? full + 1 : full), split, b_begin, b_end);
    const int mine = blocks_of_wave(a, b_end - b_begin, wave) << (PAIRS ? 1 : 0);
    const int old_pieces = 4 - ((a.k & 511) >> 7);      // TAIL: 128-k pieces of the last window that belong to the stage before
    // K stage of this wave's i-th stage: the waves take stages (PAIRS: pairs of stages) round-robin
    auto stage_kb = [&](int i) __attribute__((always_inline)) {
        return PAIRS ? 2 * (b_begin + wave + (i >> 1) * waves) + (i & 1) : b_begin + wave + i * waves;
    };

    // ---- DMA sources ------------------------------------------------------------------------
    const int v_row = lane >> 4, v_pp = lane & 15;     // values / activations: 4 rows x 16 pieces
    const int t_row = lane >> 2, t_pp = lane & 3;      // metadata: 16 rows x 4 pieces
    const size_t v_stride = (size_t)(a.k >> 1), t_stride = (size_t)(a.k >> 3);
    const int l_row = lane >> 3, l_pp = lane & 7;      // PAIRS metadata: 8 rows x 8 pieces (one 128-byte line per row)
    const uint8_t* vsrc[RG][4];
    const uint8_t* tsrc[RG];                           // PAIRS: rows 0..7 of the tile ...
    int tsrc_hi[RG];                                   // ... and how far behind them the same lane's piece of rows 8..15 is
#pragma unroll
    for (int rg = 0; rg < RG; rg++) {
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int row16 = 4 * u + v_row;
            int row = n0 + rg * 16 + row16;
            row = row < a.n ? row : a.n - 1;
            vsrc[rg][u] = a.B + (size_t)row * v_stride + ((v_pp ^ row16) << 4);
        }
        if constexpr (PAIRS) {
            int row = n0 + rg * 16 + l_row, row_hi = row + 8;
            row = row < a.n ? row : a.n - 1;
            row_hi = row_hi < a.n ? row_hi : a.n - 1;
            tsrc[rg] = sa.meta + (size_t)row * t_stride + ((l_pp ^ l_row) << 4);
            // (the host keeps 16 metadata rows below 2 GB)
            tsrc_hi[rg] = (row_hi - row) * (int)t_stride + (((l_pp ^ l_row ^ 1) - (l_pp ^ l_row)) << 4);
        } else {
            int row = n0 + rg * 16 + t_row;
            row = row < a.n ? row : a.n - 1;
            tsrc[rg] = sa.meta + (size_t)row * t_stride + ((t_pp ^ (t_row >> 2)) << 4);
            tsrc_hi[rg] = 0;
        }
    }
    const uint8_t* xsrc[XU2];
#pragma unroll
    for (int i = 0; i < XU2; i++) {
        const int row_l = 4 * (i >> 1) + v_row;          // row inside the activation tile
        int row = m0 + row_l;
        row = row < a.m ? row : a.m - 1;
        xsrc[i] = a.A + (size_t)row * a.k + (i & 1) * 256 + ((v_pp ^ (row_l & 15)) << 4);
    }

    const uint8_t* my_ring = ring + (size_t)wave * WAVE_BYTES;
    const unsigned my_ring_lds = lds_addr(my_ring);
    const uint8_t* my_meta = my_ring + DEPTH * STAGE_BYTES;   // PAIRS: [pair slot][rg][rows 0..7 | rows 8..15][8 x 128 B]
    const unsigned my_meta_lds = my_ring_lds + DEPTH * STAGE_BYTES;
    // PAIRS: half h of pair P's metadata lines (the last pair's again past the end) into pair slot P % NP
    auto issue_meta = [&](int P, int h) __attribute__((always_inline)) {
        const int last = (mine >> 1) - 1;
        const size_t off = (size_t)stage_kb(2 * (P < last ? P : last)) << 6;   // 64 metadata bytes per stage and row
#pragma unroll
        for (int rg = 0; rg < RG; rg++)
            dma_1kb_stream(tsrc[rg] + off + h * tsrc_hi[rg], my_meta_lds + (unsigned)(((P % NP) * RG + rg) * 2 + h) * 1024);
    };
    auto issue = [&](int i) __attribute__((always_inline)) {
        const int kb = stage_kb(i);
        // first k of the stage: the last stage of a TAIL build starts at k - 512
        const size_t k0 = (TAIL && kb == full) ? (size_t)a.k - 512 : (size_t)kb << 9;
        const unsigned slot = my_ring_lds + (unsigned)(i % DEPTH) * STAGE_BYTES;
#pragma unroll
        for (int rg = 0; rg < RG; rg++) {
#pragma unroll
            for (int u = 0; u < 4; u++) dma_1kb_stream(vsrc[rg][u] + (k0 >> 1), slot + rg * W_TILE + u * 1024);
            if constexpr (!PAIRS) dma_1kb_stream(tsrc[rg] + (k0 >> 3), slot + rg * W_TILE + 4096);
        }
        if constexpr (PAIRS) issue_meta((i >> 1) + 1, i & 1);
#pragma unroll
        for (int i2 = 0; i2 < XU2; i2++) dma_1kb(xsrc[i2] + k0, slot + X_OFF + i2 * 1024);
    };

    // ---- LDS read offsets ---------------------------------------------------------------------
    const int r = lane & 15, g = lane >> 4;
    const int v_rd = (r >> 2) * 1024 + (r & 3) * 256;                               // + ((4g + i) ^ r) * 16
    const int t_rd = 4096 + r * 64 + ((g ^ (r >> 2)) << 4);
    // PAIRS: row r's line sits in half r / 8 of the pair slot; stage h of the pair owns its pieces 4h .. 4h + 3
    const int t_rd_pair = (r >> 3) * 1024 + (r & 7) * 128;                          // + ((4h + g) ^ (r & 7) ^ (r >> 3)) * 16
    const int t_swz = (r & 7) ^ (r >> 3);
    const int x_rd = ((r >> 2) * 2 + (g >> 1)) * 1024 + (r & 3) * 256;              // + ((8(g&1) + t) ^ r) * 16

    f32x4 acc[RG][MT];
#pragma unroll
    for (int rg = 0; rg < RG; rg++)
#pragma unroll
        for (int mt = 0; mt < MT; mt++) acc[rg][mt] = f32x4{0.f, 0.f, 0.f, 0.f};

    auto consume = [&](int i) __attribute__((always_inline)) {
        const uint8_t* slot = my_ring + (size_t)(i % DEPTH) * STAGE_BYTES;
        i32x4 x[MT][8];
#pragma unroll
        for (int mt = 0; mt < MT; mt++)
#pragma unroll
            for (int t = 0; t < 8; t++)
                x[mt][t] = *reinterpret_cast<const i32x4*>(slot + X_OFF + mt * 8192 + x_rd + (((8 * (g & 1) + t) ^ r) << 4));
        if constexpr (TAIL) {
            if (stage_kb(i) == full && g < old_pieces) {
#pragma unroll
                for (int mt = 0; mt < MT; mt++)
#pragma unroll
                    for (int t = 0; t < 8; t++) x[mt][t] = i32x4{0, 0, 0, 0};
            }
        }
#pragma unroll
        for (int rg = 0; rg < RG; rg++) {
            const uint8_t* w = slot + rg * W_TILE;
            const uint8_t* t = PAIRS ? my_meta + (((i >> 1) % NP) * RG + rg) * 2048 + t_rd_pair + (((4 * (i & 1) + g) ^ t_swz) << 4)
                                     : w + t_rd;
            const i32x4 idx = *reinterpret_cast<const i32x4*>(t);
#pragma unroll
            for (int p = 0; p < 4; p++) {
                const i32x4 v = *reinterpret_cast<const i32x4*>(w + v_rd + (((4 * g + p) ^ r) << 4));
                const i32x2 v_lo = {v.x, v.y}, v_hi = {v.z, v.w};
                const int id_lo = idx[p] & 0xffff, id_hi = (unsigned)idx[p] >> 16;
#pragma unroll
                for (int mt = 0; mt < MT; mt++) {
                    acc[rg][mt] = __builtin_amdgcn_smfmac_f32_16x16x64_fp8_fp8(v_lo, x[mt][2 * p], acc[rg][mt], id_lo, 0, 0);
                    acc[rg][mt] = __builtin_amdgcn_smfmac_f32_16x16x64_fp8_fp8(v_hi, x[mt][2 * p + 1], acc[rg][mt], id_hi, 0, 0);
                }
            }
        }
    };

    if constexpr (PAIRS) {
        if (mine > 0) {   // the first pair's metadata ahead of everything
            issue_meta(0, 0);
            issue_meta(0, 1);
        }
    }
    if (mine >= DEPTH) {
#pragma unroll
        for (int d = 0; d < DEPTH; d++) issue(d);
        stamps.mark(1);
        int i = 0;
        for (; i + DEPTH < mine; i++) {
            wait_vmcnt<(DEPTH - 1) * PER_STAGE>();
            if (i == 0) stamps.mark(2);
            consume(i);
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            __builtin_amdgcn_sched_barrier(0);
            issue(i + DEPTH);
            __builtin_amdgcn_sched_barrier(0);
        }
        drain_ring<0, DEPTH, PER_STAGE>(consume, i);
    } else {
        for (int i = 0; i < mine; i++) issue(i);
        stamps.mark(1);
        wait_vmcnt<0>();
        stamps.mark(2);
        for (int i = 0; i < mine; i++) consume(i);
    }
    stamps.mark(3);

    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __syncthreads();
    finish_tile<RG, MT>(a, acc, reinterpret_cast<f32x4*>(ring), &arrival, tile_m, tile_n, split, m0, n0);
    stamps.end(a);
}

// ---------------------------------------------------------------------------------------------
// Wave-per-tile variant with the activations resident in LDS, for many weight rows and at most 16
// activation rows (the up-projection of a sparse MLP at decode batch sizes).  Next to a 16-row stage of
// compressed weights (5 KB) the activations of the same 512 k are 2-8 KB, so in the kernel above up to
// 60 % of what a workgroup pulls through L2 is the same activation matrix over and over.  Here a workgroup
// fetches the activation matrix once, every wave owns whole 16*RG-row tiles over the full K range - no
// cross-wave reduction, no barrier after the prologue - and its ring carries weights only and runs on across
// tile boundaries.  Tiles are dealt to workgroups first (wave w of workgroup b owns tiles b + G*w,
// b + G*(w + W), ...), so that with three or four tiles per CU every CU streams; every wave starts its
// tiles at a K stage of its own and wraps (waves in step at one K offset load the memory channels unevenly).
template <int RG, int XU2, int DEPTH, bool TAIL, bool PAIRS>
__global__ void __launch_bounds__(RG == 4 ? 512 : 1024) sparse24_gemm_wavetile_kernel(const SparseArgs sa) {
    extern __shared__ __attribute__((aligned(1024))) uint8_t ring[];  // X[stages][XU2 KB] | [wave][sparse_wave_bytes] | 8 KB
    const StreamArgs& a = sa.g;
    Stamps stamps;
    stamps.begin();

    constexpr int PER_STAGE = RG * 5;
    constexpr int W_TILE = PAIRS ? 4096 : 5120;
    constexpr int STAGE_BYTES = sparse_stage_bytes(RG, 0, PAIRS);
    constexpr int NP = sparse_meta_pairs(DEPTH);
    constexpr int WAVE_BYTES = sparse_wave_bytes(RG, 0, DEPTH, PAIRS);
    static_assert((DEPTH - 1) * PER_STAGE <= 63, "ring deeper than vmcnt can count");
    static_assert(!(TAIL && PAIRS), "whole metadata lines need K in whole pairs of stages");

    const int lane = lane_id();
    const int wave = wave_id();
    const int waves = a.waves;
    const int full = a.k >> 9;                       // whole 512-k stages
    const int blocks = TAIL ? full + 1 : full;       // TAIL: one more, loaded from k - 512 and partly used
    const int old_pieces = 4 - ((a.k & 511) >> 7);
    auto first_k = [&](int kb) __attribute__((always_inline)) { return (TAIL && kb == full) ? (size_t)a.k - 512 : (size_t)kb << 9; };
    const int first = (int)blockIdx.x + (int)gridDim.x * wave;
    const int stride = (int)gridDim.x * waves;
    const int my_tiles = first < a.n_tiles ? (a.n_tiles - first + stride - 1) / stride : 0;
    const int total = blocks * my_tiles;
    // (PAIRS: an even stage, so that stages 2P and 2P + 1 of the wave's sequence share their metadata lines)
    const unsigned wave_no = (unsigned)blockIdx.x * (unsigned)waves + (unsigned)wave;
    const int k_rot = PAIRS ? 2 * (int)(wave_no % (unsigned)(blocks >> 1)) : (int)(wave_no % (unsigned)blocks);
    auto rotated = [&](int kb) __attribute__((always_inline)) { return kb + k_rot >= blocks ? kb + k_rot - blocks : kb + k_rot; };

    const int v_row = lane >> 4, v_pp = lane & 15;     // values / activations: 4 rows x 16 pieces
    const int t_row = lane >> 2, t_pp = lane & 3;      // metadata: 16 rows x 4 pieces
    const size_t v_stride = (size_t)(a.k >> 1), t_stride = (size_t)(a.k >> 3);
    const int l_row = lane >> 3, l_pp = lane & 7;      // PAIRS metadata: 8 rows x 8 pieces (one 128-byte line per row)
    const int x_bytes = blocks * XU2 * 1024;
    const uint8_t* my_ring = ring + x_bytes + (size_t)wave * WAVE_BYTES;
    const unsigned my_ring_lds = lds_addr(my_ring);
    const uint8_t* my_meta = my_ring + DEPTH * STAGE_BYTES;   // PAIRS: [pair slot][rg][rows 0..7 | rows 8..15][8 x 128 B]
    const unsigned my_meta_lds = my_ring_lds + DEPTH * STAGE_BYTES;
    const unsigned x_lds = lds_addr(ring);

    // ---- resident activations: stage kb is fetched by wave kb % waves, in the layout of a stage's activation part
    int x_issued = 0;
    for (int kb = wave; kb < blocks; kb += waves) {
#pragma unroll
        for (int i = 0; i < XU2; i++) {
            const int row_l = 4 * (i >> 1) + v_row;
            const int row = row_l < a.m ? row_l : a.m - 1;
            dma_1kb(a.A + (size_t)row * a.k + first_k(kb) + (i & 1) * 256 + ((v_pp ^ (row_l & 15)) << 4),
                    x_lds + (unsigned)(kb * XU2 + i) * 1024);
        }
        x_issued += XU2;
    }

    // PAIRS: half h of the metadata lines of the pair that starts at stage i2 of this wave's sequence (tile j2) into
    // pair slot P % NP
    auto issue_meta = [&](int P, int h, int i2, int j2) __attribute__((always_inline)) {
        const size_t off = (size_t)rotated(i2 - j2 * blocks) << 6;   // 64 metadata bytes per stage and row
        const int n0 = (first + j2 * stride) * (16 * RG);
#pragma unroll
        for (int rg = 0; rg < RG; rg++) {
            int row = n0 + rg * 16 + 8 * h + l_row;
            row = row < a.n ? row : a.n - 1;
            dma_1kb_stream(sa.meta + (size_t)row * t_stride + ((l_pp ^ l_row ^ h) << 4) + off,
                           my_meta_lds + (unsigned)(((P % NP) * RG + rg) * 2 + h) * 1024);
        }
    };
    auto issue = [&](int i) __attribute__((always_inline)) {
        const int j = i / blocks;
        const size_t k0 = first_k(rotated(i - j * blocks));
        const int n0 = (first + j * stride) * (16 * RG);
        const unsigned slot = my_ring_lds + (unsigned)(i % DEPTH) * STAGE_BYTES;
#pragma unroll
        for (int rg = 0; rg < RG; rg++) {
#pragma unroll
            for (int u = 0; u < 4; u++) {
                const int row16 = 4 * u + v_row;
                int row = n0 + rg * 16 + row16;
                row = row < a.n ? row : a.n - 1;   // past the edge: re-read the last row, never stored
                dma_1kb_stream(a.B + (size_t)row * v_stride + ((v_pp ^ row16) << 4) + (k0 >> 1), slot + rg * W_TILE + u * 1024);
            }
            if constexpr (!PAIRS) {
                int row = n0 + rg * 16 + t_row;
                row = row < a.n ? row : a.n - 1;
                dma_1kb_stream(sa.meta + (size_t)row * t_stride + ((t_pp ^ (t_row >> 2)) << 4) + (k0 >> 3), slot + rg * W_TILE + 4096);
            }
        }
        if constexpr (PAIRS) {
            // the pair after the one stage i belongs to (past the end: the last pair again); it starts in this tile
            // or in the next one
            const int P = (i >> 1) + 1;
            int i2 = 2 * P;
            if (i2 >= total) i2 = total - 2;
            issue_meta(P, i & 1, i2, i2 - j * blocks >= blocks ? j + 1 : j);
        }
    };

    const int r = lane & 15, g = lane >> 4;
    const int v_rd = (r >> 2) * 1024 + (r & 3) * 256;
    const int t_rd = 4096 + r * 64 + ((g ^ (r >> 2)) << 4);
    const int t_rd_pair = (r >> 3) * 1024 + (r & 7) * 128;   // + ((4h + g) ^ (r & 7) ^ (r >> 3)) * 16, h = stage % 2
    const int t_swz = (r & 7) ^ (r >> 3);
    const int x_rd = ((r >> 2) * 2 + (g >> 1)) * 1024 + (r & 3) * 256;

    f32x4 acc[RG];
#pragma unroll
    for (int rg = 0; rg < RG; rg++) acc[rg] = f32x4{0.f, 0.f, 0.f, 0.f};

    int kb_cur = 0;   // stages of the current tile already consumed
    auto consume = [&](int i) __attribute__((always_inline)) {
        const uint8_t* slot = my_ring + (size_t)(i % DEPTH) * STAGE_BYTES;
        const int kb = rotated(kb_cur);
        const uint8_t* xs = ring + (size_t)kb * (XU2 * 1024);
        i32x4 x[8];
#pragma unroll
        for (int t = 0; t < 8; t++) x[t] = *reinterpret_cast<const i32x4*>(xs + x_rd + (((8 * (g & 1) + t) ^ r) << 4));
        if constexpr (TAIL) {
            if (kb == full && g < old_pieces) {
#pragma unroll
                for (int t = 0; t < 8; t++) x[t] = i32x4{0, 0, 0, 0};
            }
        }
#pragma unroll
        for (int rg = 0; rg < RG; rg++) {
            const uint8_t* w = slot + rg * W_TILE;
            const uint8_t* t = PAIRS ? my_meta + (((i >> 1) % NP) * RG + rg) * 2048 + t_rd_pair + (((4 * (i & 1) + g) ^ t_swz) << 4)
                                     : w + t_rd;
            const i32x4 idx = *reinterpret_cast<const i32x4*>(t);
#pragma unroll
            for (int p = 0; p < 4; p++) {
                const i32x4 v = *reinterpret_cast<const i32x4*>(w + v_rd + (((4 * g + p) ^ r) << 4));
                const i32x2 v_lo = {v.x, v.y}, v_hi = {v.z, v.w};
                const int id_lo = idx[p] & 0xffff, id_hi = (unsigned)idx[p] >> 16;
                acc[rg] = __builtin_amdgcn_smfmac_f32_16x16x64_fp8_fp8(v_lo, x[2 * p], acc[rg], id_lo, 0, 0);
                acc[rg] = __builtin_amdgcn_smfmac_f32_16x16x64_fp8_fp8(v_hi, x[2 * p + 1], acc[rg], id_hi, 0, 0);
            }
        }
    };

    const float scale = a.scale ? a.scale[0] : 1.0f;
    int tile_j = 0;
    auto after_consume = [&]() __attribute__((always_inline)) {
        if (++kb_cur == blocks) {   // the tile is complete: scale, round, store, start the next one
            kb_cur = 0;
            const int n0 = (first + tile_j * stride) * (16 * RG);
            tile_j++;
#pragma unroll
            for (int rg = 0; rg < RG; rg++) {
                store_fragment(a, acc[rg], scale, r, n0 + rg * 16 + 4 * g);
                acc[rg] = f32x4{0.f, 0.f, 0.f, 0.f};
            }
        }
    };

    // weight prologue behind the activations; once at most pro * PER_STAGE DMAs are outstanding this wave's share of
    // the activations has landed, and the barrier publishes everyone's
    const int pro = total < DEPTH ? total : DEPTH;
    if constexpr (PAIRS) {
        if (total > 0) {   // the first pair's metadata ahead of the weights
            issue_meta(0, 0, 0, 0);
            issue_meta(0, 1, 0, 0);
        }
    }
    for (int d = 0; d < pro; d++) issue(d);
    stamps.mark(1);
    if (x_issued > 0) wait_vmcnt_upto(pro * PER_STAGE);
    __syncthreads();

    if (total >= DEPTH) {
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
        wait_vmcnt<0>();
        stamps.mark(2);
        for (int i = 0; i < total; i++) {
            consume(i);
            after_consume();
        }
    }
    stamps.mark(3);   // (the tiles' stores are part of the streaming phase here: every wave stores as it goes)
    stamps.end(a);
}


}  // namespace sg
