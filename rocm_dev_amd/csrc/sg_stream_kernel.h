// Direct-streaming FP8 skinny GEMM for gfx950:  D[m,n] = scale * sum_k A[m,k] * B[n,k].
//
// Role of the MFMA operands.  v_mfma_f32_16x16x32_fp8_fp8 takes, per lane l, 8 K-bytes of
// "row" l%16 for its first operand and 8 K-bytes of "column" l%16 for the second, the
// K-bytes being 8*(l/16)..+7 of a 32-wide window; lane l then owns column l%16 and rows
// 4*(l/16)..+3 of the 16x16 fp32 result.  Here the WEIGHT rows (N) are the first operand
// and the ACTIVATION rows (M <= 16 per block) the second, so a lane ends up with four
// consecutive n for one m: one 8-byte bf16 store.
//
// A dot product does not care in which order K is visited as long as both operands agree,
// so lane (r = l%16, g = l/16) simply loads the 16 contiguous bytes  row r, K offset
// chunk*64 + g*16  of BOTH operands with one 128-bit load each and feeds the low and the
// high 8 bytes to two consecutive MFMAs.  Per load instruction the wave touches 16 rows x
// 64 contiguous bytes (one full 64-byte memory request per row); KU such chunks per stage
// make KU*64 contiguous bytes per row.  The weights never pass through LDS.
//
// Work split.  A workgroup owns 16*RG weight rows and a K range; its waves take the stages
// of that range round-robin (wave w: stage w, w+waves, ...), each keeping DEPTH stages in
// flight in registers.  The waves' fp32 partial tiles meet in LDS and are summed in wave
// order.  With split_k > 1 several workgroups share a tile: each writes its fp32 partial
// to the workspace, and the last one to arrive (an arrival counter per tile) sums the
// partials in split order, so the result does not depend on arrival order.
//
// Reference behaviour restated: tile -> (m, n, k-split) decode with the last split taking
// the remainder (skinny_gemm/skinny_gemm_kernel.cu:54-64); activations through the cache,
// weights streamed (skinny_gemm/producers/producers.cuh:22,41); scale applied once to the
// fp32 sum, rounding last (skinny_gemm/consumers/mfma_16x16x32_consumer.cu:119-127).
#pragma once

#include "sg_device.h"
#include "sg_epilogue.h"

namespace sg {

constexpr int stream_regs(int MT, int RG, int KU, int DEPTH) {
    return DEPTH * KU * (RG + MT) * 4 + RG * MT * 4 + 28;
}
constexpr int stream_launch_bound(int MT, int RG, int KU, int DEPTH) {
    return stream_regs(MT, RG, KU, DEPTH) <= 128 ? 1024 : (stream_regs(MT, RG, KU, DEPTH) <= 256 ? 512 : 256);
}

template <int MT, int RG, int KU>
struct Stage {
    i64x2 w[RG][KU];
    i64x2 x[MT][KU];
};

template <int MT, int RG, int KU, bool TAIL>
__device__ __forceinline__ void load_stage(Stage<MT, RG, KU>& st, const uint8_t* const (&wrow)[RG],
                                           const uint8_t* const (&xrow)[MT], int koff0, int k_lane) {
#pragma unroll
    for (int u = 0; u < KU; u++) {
        const int koff = koff0 + u * 64;
        if (!TAIL || koff < k_lane) {
#pragma unroll
            for (int rg = 0; rg < RG; rg++) st.w[rg][u] = load16_stream(wrow[rg] + koff);
#pragma unroll
            for (int mt = 0; mt < MT; mt++) st.x[mt][u] = load16(xrow[mt] + koff);
        } else {
#pragma unroll
            for (int rg = 0; rg < RG; rg++) st.w[rg][u] = i64x2{0, 0};
#pragma unroll
            for (int mt = 0; mt < MT; mt++) st.x[mt][u] = i64x2{0, 0};
        }
    }
}

template <int MT, int RG, int KU>
__device__ __forceinline__ void mma_stage(const Stage<MT, RG, KU>& st, f32x4 (&acc)[RG][MT]) {
#pragma unroll
    for (int u = 0; u < KU; u++) {
#pragma unroll
        for (int rg = 0; rg < RG; rg++) {
#pragma unroll
            for (int mt = 0; mt < MT; mt++) {
                acc[rg][mt] = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(st.w[rg][u].x, st.x[mt][u].x, acc[rg][mt], 0, 0, 0);
                acc[rg][mt] = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(st.w[rg][u].y, st.x[mt][u].y, acc[rg][mt], 0, 0, 0);
            }
        }
    }
}

template <int MT, int RG, int KU, int DEPTH>
__global__ void __launch_bounds__(stream_launch_bound(MT, RG, KU, DEPTH))
stream_gemm_kernel(const StreamArgs a) {
    extern __shared__ f32x4 red[];  // [frag][wave][64]
    __shared__ unsigned arrival;

    constexpr int FRAGS = RG * MT;
    constexpr int STAGE_K = KU * 64;

    const int lane = lane_id();
    const int wave = wave_id();
    const int waves = a.waves;
    const int r = lane & 15, g = lane >> 4;

    int tile_n, split, tile_m;
    decode_tile(a, xcd_order((int)blockIdx.x, (int)gridDim.x), tile_n, split, tile_m);
    const int n0 = tile_n * (16 * RG);
    const int m0 = tile_m * (16 * MT);

    // K range of this workgroup in stages of STAGE_K bytes; the last split takes the remainder,
    // including a final partial stage when k is not a multiple of STAGE_K
    const int full_stages = a.k / STAGE_K;
    int s_begin, s_end_full;
    split_range(a, full_stages, split, s_begin, s_end_full);
    const bool last_split = split == a.split_k - 1;
    const bool has_tail = last_split && (a.k % STAGE_K) != 0;

    // Rows past the edge of either operand re-read the last valid row: the MFMA keeps result
    // columns (and rows) independent, and those results are never stored.
    const uint8_t* wrow[RG];
    const uint8_t* xrow[MT];
#pragma unroll
    for (int rg = 0; rg < RG; rg++) {
        int row = n0 + rg * 16 + r;
        row = row < a.n ? row : a.n - 1;
        wrow[rg] = a.B + (size_t)row * a.b_stride + g * 16;
    }
#pragma unroll
    for (int mt = 0; mt < MT; mt++) {
        int row = m0 + mt * 16 + r;
        row = row < a.m ? row : a.m - 1;
        xrow[mt] = a.A + (size_t)row * a.k + g * 16;
    }

    f32x4 acc[RG][MT];
#pragma unroll
    for (int rg = 0; rg < RG; rg++)
#pragma unroll
        for (int mt = 0; mt < MT; mt++) acc[rg][mt] = f32x4{0.f, 0.f, 0.f, 0.f};

    // This wave's full stages are  first, first + waves, ...  (mine of them).  The steady-state
    // loop is branch-free so that the compiler can keep DEPTH stages of loads in flight.
    const int n_full = s_end_full - s_begin;
    const int mine = blocks_of_wave(a, n_full, wave);
    const int first_off = (s_begin + wave) * STAGE_K;
    const int step_off = waves * STAGE_K;

    Stage<MT, RG, KU> st[DEPTH];
    int i = 0;
    if (mine >= 2 * DEPTH) {
        // long K range: unconditional prologue, so that the waits inside the loop are exact
#pragma unroll
        for (int d = 0; d < DEPTH; d++) {
            load_stage<MT, RG, KU, false>(st[d], wrow, xrow, first_off + d * step_off, 0);
            __builtin_amdgcn_sched_barrier(0);
        }
        for (; i + 2 * DEPTH <= mine; i += DEPTH) {
#pragma unroll
            for (int d = 0; d < DEPTH; d++) {
                // keep the compiler from sinking the reloads below the next stage's MFMAs: the
                // point of the ring is that DEPTH-1 stages of loads stay in flight behind each wait
                mma_stage<MT, RG, KU>(st[d], acc);
                __builtin_amdgcn_sched_barrier(0);
                load_stage<MT, RG, KU, false>(st[d], wrow, xrow, first_off + (i + DEPTH + d) * step_off, 0);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    } else {
#pragma unroll
        for (int d = 0; d < DEPTH; d++)
            if (d < mine) load_stage<MT, RG, KU, false>(st[d], wrow, xrow, first_off + d * step_off, 0);
    }
#pragma unroll
    for (int d = 0; d < DEPTH; d++) {
        if (i + d < mine) {
            mma_stage<MT, RG, KU>(st[d], acc);
            if (i + DEPTH + d < mine)
                load_stage<MT, RG, KU, false>(st[d], wrow, xrow, first_off + (i + DEPTH + d) * step_off, 0);
        }
    }
#pragma unroll
    for (int d = 0; d < DEPTH; d++)
        if (i + DEPTH + d < mine) mma_stage<MT, RG, KU>(st[d], acc);

    // ragged last stage (k not a multiple of the stage width): one wave of the last split
    if (has_tail && wave == n_full % waves) {
        load_stage<MT, RG, KU, true>(st[0], wrow, xrow, s_end_full * STAGE_K, a.k - g * 16);
        mma_stage<MT, RG, KU>(st[0], acc);
    }

    finish_tile<RG, MT>(a, acc, red, &arrival, tile_m, tile_n, split, m0, n0);
}

}  // namespace sg
