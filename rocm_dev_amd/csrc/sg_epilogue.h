// Arguments and epilogue shared by the dense GEMM kernels: cross-wave reduction through LDS,
// cross-workgroup split-K through the fp32 workspace, scale, bf16 rounding and the store.
//
// Fragment convention (both kernels): acc[rg][mt] is the 16 x 16 fp32 tile of weight rows
// n0 + 16*rg .. +15 against activation rows m0 + 16*mt .. +15 in the MFMA result layout:
// lane l owns activation row (l % 16) and weight rows 4*(l / 16) .. +3, i.e. four
// consecutive n of one output row.
//
// Reference behaviour restated: every partial of every consumer wave and of every K split
// is added into D (skinny_gemm/consumers/mfma_16x16x32_consumer.cu:119-162 does it with
// fp16 atomics into a pre-zeroed D).  Here the partials are summed in fp32 in a fixed
// order - waves in wave order through LDS, K splits in split order through the workspace
// by the last workgroup to arrive - then scaled and rounded to bf16 once, and D is
// overwritten.
#pragma once

#include "sg_device.h"

namespace sg {

struct StreamArgs {
    const uint8_t* A;       // E4M3 activations [m, k] ...
    const uint16_t* A16;    // ... or bf16 activations that the kernel quantises per row itself (resident-activation kernel only; A unused)
    float* row_scale_out;   // with A16: optional [m] output of the row scales the kernel derived, or nullptr
    const uint8_t* B;
    void* D;                // bf16 or fp32, [m, n]
    const float* scale;     // device scalar, or nullptr for 1.0f
    const float* row_scale; // [m] per-activation-row factors, or nullptr
    const float* col_scale; // [n] per-weight-row (output column) factors, or nullptr
    float* ws;              // split-K partials (fp32)
    unsigned* counters;     // one arrival counter per output tile, zero between launches
    int m, n, k, b_stride;
    int split_k, waves;
    int n_tiles, m_tiles;
    int out_f32;
    unsigned inv_n_tiles, inv_split_k, inv_waves;  // div_reciprocal() of n_tiles, split_k, waves (set_reciprocals)
    unsigned long long* stamps;  // profiling aid, normally nullptr: kStampWords time stamps per workgroup (sg_debug_stamps)
    int x_extra;            // register-resident kernel: 1 = the launch's LDS has one more 4 KB staging block per wave behind the reduction scratch
    int defer_reduce;       // mid-batch kernel with split_k > 1: 1 = store the fp32 partials only; a second launch (mid_reduce_kernel) sums them
};

// Time stamps a workgroup leaves when a.stamps is set (wave 0 writes them when it is done):
//   [0] kernel entry (first instruction)  [1] prologue DMAs issued  [2] first stage landed  [3] last stage consumed
//   [4] outputs stored and acknowledged   - all five from the 100 MHz constant clock (10 ns units) -
//   [5] shader clock at entry  [6] shader clock at the end  [7] hardware id: XCC_ID << 32 | HW_ID
// The clock reads are unconditional (one scalar instruction each); only the final wait and the stores depend on
// a.stamps, so a launch without stamps does not wait for that argument before it requests the others.
constexpr int kStampWords = 8;
struct Stamps {
    unsigned long long t[kStampWords];
    __device__ __forceinline__ void begin() {
        t[0] = __builtin_amdgcn_s_memrealtime();
        t[5] = __builtin_amdgcn_s_memtime();
    }
    // mark(1) also presets [2] for the paths on which no stage is waited for separately
    __device__ __forceinline__ void mark(int i) {
        t[i] = __builtin_amdgcn_s_memrealtime();
        if (i == 1) t[2] = t[1];
    }
    __device__ __forceinline__ void end(const StreamArgs& a) {
        if (a.stamps == nullptr) return;
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        t[4] = __builtin_amdgcn_s_memrealtime();
        t[6] = __builtin_amdgcn_s_memtime();
        const unsigned hw = __builtin_amdgcn_s_getreg((31 << 11) | 4), xcc = __builtin_amdgcn_s_getreg((31 << 11) | 20);
        t[7] = ((unsigned long long)xcc << 32) | hw;
        if (threadIdx.x == 0) {
            unsigned long long* out = a.stamps + (size_t)blockIdx.x * kStampWords;
#pragma unroll
            for (int i = 0; i < kStampWords; i++) out[i] = t[i];
        }
    }
};

inline void set_reciprocals(StreamArgs& a) {
    a.inv_n_tiles = div_reciprocal((unsigned)a.n_tiles);
    a.inv_split_k = div_reciprocal((unsigned)a.split_k);
    a.inv_waves = div_reciprocal((unsigned)a.waves);
}

// Position `bid` in tile order -> (tile_n, split, tile_m): the activation tiles of a weight tile fastest (their
// workgroups are neighbours in position, hence - after xcd_order - on one XCD, whose L2 then fetches the weight tile
// once for all of them), then the n tiles, then the K splits.  With one activation tile this is n tiles fastest.
__device__ __forceinline__ void decode_tile(const StreamArgs& a, int bid, int& tile_n, int& split, int& tile_m) {
    unsigned rest = (unsigned)bid;
    tile_m = 0;
    if (a.m_tiles > 1) {
        rest = (unsigned)bid / (unsigned)a.m_tiles;
        tile_m = bid - (int)rest * a.m_tiles;
    }
    const unsigned q = fast_div(rest, (unsigned)a.n_tiles, a.inv_n_tiles);
    tile_n = (int)rest - (int)q * a.n_tiles;
    split = (int)q;
}

// K range [b_begin, b_end) of split `split` out of `blocks` stage-sized blocks; the last split takes the remainder.
__device__ __forceinline__ void split_range(const StreamArgs& a, int blocks, int split, int& b_begin, int& b_end) {
    const int per_split = (int)fast_div((unsigned)blocks, (unsigned)a.split_k, a.inv_split_k);
    b_begin = split * per_split;
    b_end = (split == a.split_k - 1) ? blocks : b_begin + per_split;
}

// Blocks wave `wave` takes when `waves` waves share n_blk blocks round-robin: ceil((n_blk - wave) / waves).
__device__ __forceinline__ int blocks_of_wave(const StreamArgs& a, int n_blk, int wave) {
    return wave < n_blk ? (int)fast_div((unsigned)(n_blk - wave + a.waves - 1), (unsigned)a.waves, a.inv_waves) : 0;
}

// Writes one finished 16(n) x 16(m) fragment: lane owns m = m_base + l%16, n = n_base + 4*(l/16)..+3.
// `lds_row_scale`, when given, is a per-row factor table in LDS (the scales of activations quantised in the kernel)
// that takes the place of a.row_scale.
// `col_factors`, when given, holds a.col_scale[n_idx .. n_idx + 3] fetched ahead of time (col_scale_ahead).
__device__ __forceinline__ f32x4 col_scale_ahead(const StreamArgs& a, int n_idx) {
    f32x4 c = {1.0f, 1.0f, 1.0f, 1.0f};
    if (a.col_scale) {
#pragma unroll
        for (int e = 0; e < 4; e++)
            if (n_idx + e < a.n) c[e] = a.col_scale[n_idx + e];
    }
    return c;
}
// Columns from `n_limit` on belong to another tile (24-row tiles computed with two 16-row fragments) and are not written.
__device__ __forceinline__ void store_fragment(const StreamArgs& a, f32x4 v, float scale, int m_idx, int n_idx,
                                               const float* lds_row_scale = nullptr, const f32x4* col_factors = nullptr,
                                               int n_limit = 0x7fffffff) {
    // Pin the fragment before the lane-divergent exit below.  An MFMA needs every lane of the wave
    // (it reads all lanes' operand registers), but the compiler is free to sink the loads and the
    // MFMA that produce `v` into the region where only lanes with m_idx < m are active - it did so
    // with the 16x16x128 instruction - and the operand rows supplied by the masked lanes are then garbage.
    asm volatile("" : "+v"(v));
    if (m_idx >= a.m || n_idx >= n_limit) return;
    // scale, then the row factor, then the column factors: three separately rounded fp32 products
    v *= scale;
    if (lds_row_scale) v *= lds_row_scale[m_idx];
    else if (a.row_scale) v *= a.row_scale[m_idx];
    if (a.col_scale) {
#pragma unroll
        for (int e = 0; e < 4; e++)
            if (n_idx + e < a.n) v[e] *= col_factors ? (*col_factors)[e] : a.col_scale[n_idx + e];
    }
    const size_t off = (size_t)m_idx * a.n + n_idx;
    if (a.out_f32) {
        float* d = reinterpret_cast<float*>(a.D) + off;
        if (n_idx + 3 < a.n && (a.n & 3) == 0) {
            *reinterpret_cast<f32x4*>(d) = v;
        } else {
#pragma unroll
            for (int e = 0; e < 4; e++)
                if (n_idx + e < a.n) d[e] = v[e];
        }
    } else {
        uint16_t* d = reinterpret_cast<uint16_t*>(a.D) + off;
        if (n_idx + 3 < a.n && (a.n & 3) == 0) {
            u32x2 p = {pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
            *reinterpret_cast<u32x2*>(d) = p;
        } else {
#pragma unroll
            for (int e = 0; e < 4; e++)
                if (n_idx + e < a.n) d[e] = (uint16_t)bf16_bits(v[e]);
        }
    }
}

template <int RG, int MT>
__device__ __forceinline__ void finish_tile(const StreamArgs& a, f32x4 (&acc)[RG][MT], f32x4* red, unsigned* arrival_lds,
                                            int tile_m, int tile_n, int split, int m0, int n0, int n_limit = 0x7fffffff) {
    constexpr int FRAGS = RG * MT;
    const int lane = lane_id();
    const int wave = wave_id();
    const int waves = a.waves;
    const int r = lane & 15, g = lane >> 4;
    unsigned& arrival = *arrival_lds;
    const float scale = a.scale ? a.scale[0] : 1.0f;
    const int tile_id = tile_m * a.n_tiles + tile_n;
    float* ws_tile = a.ws + ((size_t)tile_id * a.split_k) * (FRAGS * 256);

    auto finish = [&](int f, f32x4 v) __attribute__((always_inline)) {
        const int rg = f / MT, mt = f % MT;
        if (a.split_k == 1) {
            store_fragment(a, v, scale, m0 + mt * 16 + r, n0 + rg * 16 + 4 * g, nullptr, nullptr, n_limit);
        } else {
            // agent-scope stores go through to memory, past this XCD's L2, so that a workgroup on
            // another XCD can read them without any cache-wide write-back or invalidate
            float* p = ws_tile + ((size_t)split * FRAGS + f) * 256 + lane;
#pragma unroll
            for (int e = 0; e < 4; e++) __hip_atomic_store(p + e * 64, v[e], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    };

    if (waves == 1) {
#pragma unroll
        for (int f = 0; f < FRAGS; f++) finish(f, acc[f / MT][f % MT]);
    } else {
#pragma unroll
        for (int f = 0; f < FRAGS; f++) red[(f * waves + wave) * 64 + lane] = acc[f / MT][f % MT];
        __syncthreads();
        for (int f = wave; f < FRAGS; f += waves) {
            f32x4 v = red[(f * waves) * 64 + lane];
            for (int w = 1; w < waves; w++) v += red[(f * waves + w) * 64 + lane];
            finish(f, v);
        }
    }

    if (a.split_k == 1) return;

    // ---- cross-workgroup split-K: last arrival sums the partials in split order --------
    // Order without cache-wide fences: the partial stores above are agent-scope (write-through);
    // each wave waits until its stores are acknowledged, the workgroup barrier collects all
    // waves, then one thread bumps the tile's arrival counter.  The workgroup that observes
    // split_k - 1 earlier arrivals reads every partial with agent-scope loads.
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (threadIdx.x == 0)
        arrival = __hip_atomic_fetch_add(&a.counters[tile_id], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    if (arrival != (unsigned)(a.split_k - 1)) return;
    for (int f = wave; f < FRAGS; f += waves) {
        const float* p = ws_tile + (size_t)f * 256 + lane;
        f32x4 v;
#pragma unroll
        for (int e = 0; e < 4; e++) v[e] = __hip_atomic_load(p + e * 64, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        for (int sp = 1; sp < a.split_k; sp++) {
            const float* q = p + (size_t)sp * FRAGS * 256;
#pragma unroll
            for (int e = 0; e < 4; e++) v[e] += __hip_atomic_load(q + e * 64, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        const int rg = f / MT, mt = f % MT;
        store_fragment(a, v, scale, m0 + mt * 16 + r, n0 + rg * 16 + 4 * g, nullptr, nullptr, n_limit);
    }
    if (threadIdx.x == 0)  // ready for the next launch
        __hip_atomic_store(&a.counters[tile_id], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

}  // namespace sg
