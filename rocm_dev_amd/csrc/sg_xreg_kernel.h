// Persistent LDS-ring skinny GEMM with the activations resident in REGISTERS.
//
// In the persistent K-split kernel (sg_lds_kernel.h) wave w of a workgroup always works on K
// blocks w, w + waves, ... of whatever tile the workgroup is at.  When the K range is short enough
// that this is PT <= 4 blocks per wave, the activation fragments of exactly those blocks - the
// same for every tile - fit in the wave's registers (16*PT*MT VGPRs): they are loaded once
// (through LDS, in the weights' own load pattern, see the prologue), and for the rest of the kernel
// the ring carries weights only and no activation byte crosses L2 or LDS again.  That removes what makes
// M = 17..32 slow in the other variants (an 8 KB activation stage next to every 16 KB weight
// stage) and frees the LDS the resident-in-LDS variant spends on the activations.
//
// Lane (r, g) of the MFMA reads from the weight stage the 16-byte piece g of the 64-byte runs 2h
// and 2h+1 of row r for MFMA h of a 256-byte K block (sg_lds_kernel.h: DMA layout and rd_off), so
// the activation operand held in registers is the same two pieces of activation row r.
//
// Everything else - ring, per-tile reduction through LDS in wave order, optional epilogue wave -
// is the persistent kernel's; the results are bit-identical to it.
#pragma once

#include "sg_device.h"
#include "sg_epilogue.h"
#include "sg_lds_kernel.h"

namespace sg {

// registers a wave needs: the activation fragments, the accumulators, the weight fragments of a stage, ~40 others
// and the addresses of the PT unrolled stages' refills
constexpr int xreg_regs(int MT, int RG, int PT) { return 16 * PT * MT + 4 * RG * MT + 8 * RG + 40 + 16 * PT * RG; }
// 16 waves leave each 128 VGPRs, 9 waves (8 streaming + the epilogue wave) 168, 8 waves 256
constexpr int xreg_launch_bound(int MT, int RG, int PT) { return xreg_regs(MT, RG, PT) <= 100 ? 1024 : (xreg_regs(MT, RG, PT) <= 160 ? 576 : 512); }

// PT: 256-byte K blocks per wave and tile (k = 256 * PT * waves exactly)
template <int MT, int RG, int PT, int DEPTH, bool NT>
__global__ void __launch_bounds__(xreg_launch_bound(MT, RG, PT)) lds_gemm_xreg_kernel(const StreamArgs a) {
    // [wave][DEPTH][RG*4 KB] | red[2][FRAGS][wave][64] f32x4
    extern __shared__ __attribute__((aligned(1024))) uint8_t ring[];
    Stamps stamps;
    stamps.begin();

    constexpr int PER_STAGE = RG * 4;
    constexpr int STAGE_BYTES = PER_STAGE * 1024;
    constexpr int FRAGS = RG * MT;
    static_assert((DEPTH - 1) * PER_STAGE + 4 <= 63, "ring deeper than vmcnt can count");
    static_assert(PT * MT <= 4, "activation fragments must fit in registers");

    const int lane = lane_id();
    const int wave = wave_id();
    const int waves = a.waves;                                   // streaming waves; one more = epilogue wave
    const bool epilogue_wave = blockDim.x > (unsigned)waves * 64;
    const bool streaming = wave < waves;
    const int r = lane & 15, g = lane >> 4;

    const int total_tiles = a.n_tiles;                           // one activation tile (host checks m <= 16*MT)
    const TileRun run = persistent_tile_run(total_tiles);
    const int my_tiles = run.count;
    const int total = streaming ? PT * my_tiles : 0;             // stages of this wave
    // wave w works on K blocks w, w + waves, ... shifted by an amount that differs from workgroup to workgroup
    // (and wrapped), so that the workgroups of the chip are spread over all K offsets at any moment
    // (1 % on 32 x 28672 x 4096, interleaved same-process runs)
    const int blocks = PT * waves;
    const int k_rot = (int)(((unsigned)blockIdx.x * 3u) % (unsigned)blocks);
    auto k_block = [&](int t) __attribute__((always_inline)) {
        const int kb = wave + t * waves + k_rot;
        return kb >= blocks ? kb - blocks : kb;
    };

    // ---- weight ring ------------------------------------------------------------------------------
    const int q = lane >> 2, p = lane & 3;
    const int src_row = q & 3;
    const int src_col = (q >> 2) * 64;
    const int rd_off = 1024 * (r >> 2) + 64 * (r & 3) + 16 * ((g - (r >> 2)) & 3);
    const uint8_t* my_ring = ring + (size_t)(streaming ? wave : 0) * (DEPTH * STAGE_BYTES);
    const unsigned my_ring_lds = lds_addr(my_ring);
    f32x4* red = reinterpret_cast<f32x4*>(ring + (size_t)waves * (DEPTH * STAGE_BYTES));

    auto issue = [&](int i) __attribute__((always_inline)) {   // stage i = tile i / PT, K block k_block(i % PT)
        const int j = i / PT, t = i % PT;
        const int n0 = (run.first + j) * (16 * RG);
        const unsigned slot = my_ring_lds + (unsigned)(i % DEPTH) * STAGE_BYTES;
        const size_t koff = ((size_t)k_block(t) << 8) + src_col;
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

    // one 256-byte K block: two 128-wide MFMAs per (weight tile, activation block)
    auto consume = [&](int i, const i32x8 (&x)[MT][2]) __attribute__((always_inline)) {
        const uint8_t* w = my_ring + (size_t)(i % DEPTH) * STAGE_BYTES + rd_off;
#pragma unroll
        for (int rg = 0; rg < RG; rg++)
#pragma unroll
            for (int h = 0; h < 2; h++) {
                const i32x4 lo = *reinterpret_cast<const i32x4*>(w + rg * 4096 + (2 * h) * 256);
                const i32x4 hi = *reinterpret_cast<const i32x4*>(w + rg * 4096 + (2 * h + 1) * 256);
                const i32x8 wv = i32x8{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
#pragma unroll
                for (int mt = 0; mt < MT; mt++)
                    acc[rg][mt] = mfma_e4m3_16x16x128(wv, x[mt][h], acc[rg][mt]);
            }
    };

    const float scale = a.scale ? a.scale[0] : 1.0f;
    // Reduce the waves' partial tiles of the j-th tile in wave order, scale, round, store.
    auto tile_done = [&](int j) __attribute__((always_inline)) {
        const int n0 = (run.first + j) * (16 * RG);
        if (waves == 1 && !epilogue_wave) {
#pragma unroll
            for (int f = 0; f < FRAGS; f++) store_fragment(a, acc[f / MT][f % MT], scale, (f % MT) * 16 + r, n0 + (f / MT) * 16 + 4 * g);
        } else {
            f32x4* buf = red + (size_t)(j & 1) * (FRAGS * waves * 64);
            if (streaming) {
#pragma unroll
                for (int f = 0; f < FRAGS; f++) buf[(f * waves + wave) * 64 + lane] = acc[f / MT][f % MT];
            }
            __syncthreads();
            int first = wave - j % waves, step = waves;   // no epilogue wave: the reducer rotates with the tile
            first = first < 0 ? first + waves : first;
            if (epilogue_wave) {
                first = streaming ? FRAGS : 0;
                step = 1;
            }
            for (int f = first; f < FRAGS; f += step) {
                f32x4 v = buf[(f * waves) * 64 + lane];
                for (int w = 1; w < waves; w++) v += buf[(f * waves + w) * 64 + lane];
                store_fragment(a, v, scale, (f % MT) * 16 + r, n0 + (f / MT) * 16 + 4 * g);
            }
        }
#pragma unroll
        for (int rg = 0; rg < RG; rg++)
#pragma unroll
            for (int mt = 0; mt < MT; mt++) acc[rg][mt] = f32x4{0.f, 0.f, 0.f, 0.f};
    };

    if (!streaming) {   // epilogue wave: takes part in every barrier, reduces and stores
        __syncthreads();   // the reduction scratch is free (it staged activations, see below)
        for (int j = 0; j < my_tiles; j++) tile_done(j);
        return;
    }

    // ---- activations: once, into registers, through LDS -------------------------------------------
    // A lane-per-row load straight into the operand layout touches 16 rows x 64 B per instruction, and the
    // 16*PT*MT of them a wave needs cost the CU's address unit about 2.6 us in front of the first MFMA
    // (gate_up at 32 rows: first stage consumed 4.6 us after entry against 1.9 us at 8 rows).  The fragments
    // therefore take the weights' way: direct-to-LDS loads in the wide pattern (4 rows x 256 B per
    // instruction), read back with the weight stage's own offsets - which is the operand layout.
    //
    // Staging areas of 4 KB (one 16-row block of one K block) per wave: its last ring slot (filled with weights
    // only afterwards), its share of the reduction scratch (first used at the end of the first tile, behind the
    // barrier below) and, where the launch has the LDS for it (a.x_extra), one more block behind the scratch.
    static_assert(MT <= 2, "two staging areas per pass");
    const unsigned area_lds[3] = {my_ring_lds + (unsigned)(DEPTH - 1) * STAGE_BYTES,
                                  lds_addr(red) + (unsigned)wave * (2 * FRAGS * 1024),
                                  lds_addr(red) + (unsigned)(2 * FRAGS * waves + 4 * wave) * 1024};
    const uint8_t* area_ptr[3] = {my_ring + (size_t)(DEPTH - 1) * STAGE_BYTES,
                                  reinterpret_cast<const uint8_t*>(red) + (size_t)wave * (2 * FRAGS * 1024),
                                  reinterpret_cast<const uint8_t*>(red) + (size_t)(2 * FRAGS * waves + 4 * wave) * 1024};
    auto issue_x = [&](int t, int mt, int area) __attribute__((always_inline)) {
        const size_t koff = ((size_t)k_block(t) << 8) + src_col;
#pragma unroll
        for (int u = 0; u < 4; u++) {
            int row = mt * 16 + 4 * u + src_row;
            row = row < a.m ? row : a.m - 1;   // rows past the edge repeat the last one; never stored
            dma_1kb(a.A + (size_t)row * a.k + koff + ((p + u) & 3) * 16, area_lds[area] + u * 1024);
        }
    };
    i32x8 xr[PT][MT][2];
    auto read_x = [&](int t, int mt, int area) __attribute__((always_inline)) {
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const i32x4 lo = *reinterpret_cast<const i32x4*>(area_ptr[area] + rd_off + (2 * h) * 256);
            const i32x4 hi = *reinterpret_cast<const i32x4*>(area_ptr[area] + rd_off + (2 * h + 1) * 256);
            xr[t][mt][h] = i32x8{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
        }
    };
    constexpr int FIRST = DEPTH - 1;   // weight stages issued before the activations are in registers
    // Four blocks, three areas: three blocks go in front of the weights, so that their wait leaves the weights in
    // flight; the fourth - second row block of the wave's second K block - follows as soon as an area is free and
    // is read in the first tile's second step, which has to wait for the weights issued before it anyway.
    const bool late_block = MT == 2 && PT == 2 && a.x_extra != 0 && total >= DEPTH + 2;   // wave-uniform
    int issued = 0;
    if (late_block) {
        issue_x(0, 0, 0);
        issue_x(0, 1 % MT, 1);
        issue_x(1 % PT, 0, 2);
        for (; issued < FIRST; issued++) issue(issued);
        stamps.mark(1);
        wait_vmcnt<FIRST * PER_STAGE>();
        read_x(0, 0, 0);
        read_x(0, 1 % MT, 1);
        read_x(1 % PT, 0, 2);
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // in registers before the areas are written again
        __syncthreads();   // every wave has what it staged in the reduction scratch
        issue_x(1 % PT, 1 % MT, 2);
        issue(issued);
        issued++;
    } else {
        // one K block per pass: the first pass in front of the weights, the others behind them in the queue
#pragma unroll
        for (int mt = 0; mt < MT; mt++) issue_x(0, mt, mt);
        for (; issued < FIRST && issued < total; issued++) issue(issued);
        stamps.mark(1);
        if (issued == FIRST) wait_vmcnt<FIRST * PER_STAGE>();
        else wait_vmcnt<0>();
#pragma unroll
        for (int mt = 0; mt < MT; mt++) read_x(0, mt, mt);
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
        for (int t = 1; t < PT; t++) {
#pragma unroll
            for (int mt = 0; mt < MT; mt++) issue_x(t, mt, mt);
            wait_vmcnt<0>();
#pragma unroll
            for (int mt = 0; mt < MT; mt++) read_x(t, mt, mt);
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        }
        __syncthreads();   // every wave has its fragments: the reduction scratch may be written
        if (issued < total) {
            issue(issued);
            issued++;
        }
    }
    stamps.mark(2);

    for (int j = 0; j < my_tiles; j++) {
#pragma unroll
        for (int t = 0; t < PT; t++) {
            const int i = j * PT + t;
            const int behind = total - 1 - i;   // stages issued after this one, if fewer than DEPTH - 1
            if (late_block && j == 0) {
                // behind stage 0: stages 1 .. DEPTH-1 and the late block; behind the late block: stage DEPTH-1 and
                // the refill of step 0 (total >= DEPTH + 2, so both exist) - with two slots stage 1 is that stage
                // DEPTH-1, so it is the one to wait for, with only the refill behind it
                if (t == 0) wait_vmcnt<(DEPTH - 1) * PER_STAGE + 4>();
                else {
                    wait_vmcnt<(DEPTH >= 3 ? 2 : 1) * PER_STAGE>();
                    if (t == 1) {
                        read_x(1 % PT, 1 % MT, 2);
                        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                    }
                }
            } else if (behind >= DEPTH - 1) wait_vmcnt<(DEPTH - 1) * PER_STAGE>();
            else wait_vmcnt_upto(behind * PER_STAGE);
            consume(i, xr[t]);
            // the slot is refilled only after its reads have returned
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            __builtin_amdgcn_sched_barrier(0);
            if (i + DEPTH < total) issue(i + DEPTH);
            __builtin_amdgcn_sched_barrier(0);
        }
        if (j == my_tiles - 1) stamps.mark(3);
        tile_done(j);
    }
    stamps.end(a);
}

}  // namespace sg
