// Mid-batch FP8 GEMM for gfx950 (32 < M <= 256 per tile):  D[m,n] = scale * sum_k A[m,k] * B[n,k].
//
// The skinny kernels cover M <= 32 per pass; the reference handles larger M by looping
// 32-row tiles, each re-streaming B (skinny_gemm/skinny_gemm_kernel.cu:44-46,54).  Here B is
// streamed once: a workgroup owns BN = 32*RGW weight rows and ALL activation rows, and both
// operands of a 128-byte K block are staged in LDS for its four waves.
//
// Waves form a 2 x 2 grid over the tile: wave (wn, wm) owns 16*RGW weight rows and 16*MH
// activation rows, so each weight fragment it reads from LDS feeds MH MFMAs and each
// activation fragment RGW MFMAs - the register-level reuse that keeps LDS bandwidth (128
// B/clk/CU) under the MFMA rate.  The MFMA is gfx950's v_mfma_f32_16x16x128_f8f6f4
// (no block scales): 128 bytes of K per instruction, i.e. one instruction per stage and
// fragment pair.  Lane (r = l%16, g = l/16) supplies 32 bytes of row r; which 32 bytes is
// free as long as both operands agree, so both take 16-byte pieces g and g+4 of the block.
//
// LDS stage layout: row-major, 128 bytes per row, filled by direct-to-LDS loads of 8 rows x
// 128 contiguous bytes per instruction.  The 16-byte pieces of a row are XOR-swizzled with
// (row/2) & 7 - a permutation that keeps every aligned 64-byte run intact for the memory
// system - so the sixteen lanes of a ds_read_b128 pass land in sixteen different bank groups.
//
// Pipeline: the weights have DEPTH ring slots and the activations DX <= DEPTH; per K block each wave
// waits for its own DMAs of that block (s_waitcnt vmcnt), one workgroup barrier publishes the stage
// and retires the previous one, the freed slots are refilled (activations first, so that the newest
// weight stage may stay in flight behind them), the stage is consumed.
//
// K is split across workgroups when there are few tiles; partials meet in the fp32 workspace
// and the last workgroup to arrive sums them in split order (same scheme as the skinny path).
// With large tiles that sum is a long serial tail in one workgroup (a 256 x 128 tile split four ways:
// 512 KB read back by one CU while the others have left), so a launch may instead store its partials
// only (StreamArgs::defer_reduce) and leave the sum to mid_reduce_kernel, a second launch that spreads
// it over the whole device, one wave per 16 x 16 fragment; same split order, same result bits.
// Inside its K range a workgroup starts at a block that depends on its weight tile and wraps
// around, so the fp32 sum of an output element is taken in a rotated - still fixed - K order.
#pragma once

#include "sg_device.h"
#include "sg_epilogue.h"
#include "sg_lds_kernel.h"

namespace sg {

// RGW: 16-row weight fragments per wave (2 or 4)  -> BN = 16*RGW*WN rows per workgroup
// MH : 16-row activation fragments per wave (2, 4, 8) -> up to 32*MH activation rows per tile
// WN : waves along N (2, 4 or 7); the workgroup has WN x 2 waves.  WN = 7 makes 224-row tiles: 57344 = 256 x 224,
//      one tile for each of the 256 CUs where 256-row tiles leave 32 CUs idle
// DX : ring slots of the activations (<= DEPTH, the weights' ring slots).  The weights come from HBM,
//      the activations from L2 with about half the latency; with DX < DEPTH the LDS a shallower
//      activation ring frees buys the weights one more stage in flight.
// waves that load the activation rows of a stage: the largest divisor of their `instr` DMA instructions <= waves
constexpr int mid_activation_waves(int instr, int waves) {
    int best = 1;
    for (int d = 1; d <= waves; d++)
        if (instr % d == 0) best = d;
    return best;
}

// TAIL: k is not a multiple of 128 (but of 16, and beyond 128).  The last 128-byte K block of both operands is loaded
//      from k - 128 - a window that ends with the row, nothing past it is read - and the activation fragments of that
//      stage are zero in the 16-byte pieces the block before has already multiplied: lane (r, g) holds pieces g and
//      g + 4 of a row, so that is a per-lane select.  (A build of its own: the loop for whole blocks stays as it is.)
// Workgroup `bid` of a grid of `grid` -> the weight tile it works on and its position p (0 .. per_tile-1) among the
// per_tile workgroups of that tile, in the order described in the kernel below: the weight tiles of XCD 0 (tile_n = 0,
// 8, 16 ...) with all their workgroups, then XCD 1's, XCD x starting where its share of the grid starts.  Both
// launches of a GEMM with a deferred split-K sum use it, so that the workgroups that sum a tile's partials run on the
// XCD whose L2 the partials were last written through.
__device__ __forceinline__ int xcd_weight_tile(int bid, int grid, int per_tile, int n_tiles, int& p) {
    const int xcd = bid & 7, qs = grid >> 3, rs = grid & 7;
    const int j = xcd * qs + (xcd < rs ? xcd : rs) + (bid >> 3);
    const int r = j / per_tile;
    p = j - r * per_tile;
    const int qn = n_tiles >> 3, rn = n_tiles & 7;
    int g, i;
    if (r < rn * (qn + 1)) {
        g = r / (qn + 1);
        i = r - g * (qn + 1);
    } else {                                 // (reached only with qn > 0: otherwise every r is below rn)
        const int r2 = r - rn * (qn + 1);
        g = rn + r2 / qn;
        i = r2 - (g - rn) * qn;
    }
    return g + 8 * i;
}

template <int RGW, int MH, int DEPTH, int WN, int DX = DEPTH, bool TAIL = false>
__global__ void __launch_bounds__(WN * 128) mid_gemm_kernel(const StreamArgs a) {
    // [DEPTH][W rows][128] | [DX][X rows][128], then (split-K only) 16 bytes for the arrival broadcast; no
    // static LDS, so that two workgroups of exactly half the CU's LDS can share a CU
    extern __shared__ __attribute__((aligned(1024))) uint8_t ring[];
    Stamps stamps;      // profiling aid: written out only when a.stamps is set (sg_debug_stamps)
    stamps.begin();

    constexpr int WAVES = 2 * WN;
    constexpr int BN = 16 * RGW * WN;
    constexpr int BM = 32 * MH;
    // The weight rows of a stage split evenly over all waves' DMA instructions (8 rows each); the activation rows
    // over the first XW waves, XW = the largest divisor of their instruction count that is at most WAVES (all
    // waves, except in fourteen-wave workgroups, where 32 or 16 or 8 instructions go to the first eight waves).
    constexpr int XW = mid_activation_waves(BM / 8, WAVES);
    constexpr int W_INSTR = BN / 8 / WAVES;   // DMA instructions per wave per stage for the weights
    constexpr int X_INSTR = BM / 8 / XW;      // ... and for the activations, in the waves that load them
    static_assert(BN % (8 * WAVES) == 0 && BM % (8 * XW) == 0, "stage rows must split evenly over the waves' DMA instructions");
    constexpr int PER_STAGE = W_INSTR + X_INSTR;
    constexpr int W_BYTES = BN * 128, X_BYTES = BM * 128;   // one ring slot of each operand
    constexpr int RING_BYTES = DEPTH * W_BYTES + DX * X_BYTES;
    static_assert(DX >= 2 && DX <= DEPTH, "activation ring between two slots and the weight ring's depth");
    // Per iteration the activations of stage s+DX-1 are issued before the weights of stage s+DEPTH-1, so
    // behind the last instruction of X(s) and W(s) the queue holds at least this many younger ones:
    constexpr int IN_FLIGHT_X = W_INSTR + (DX - 2) * PER_STAGE, IN_FLIGHT_W = (DEPTH - 2) * PER_STAGE;
    constexpr int IN_FLIGHT = IN_FLIGHT_X < IN_FLIGHT_W ? IN_FLIGHT_X : IN_FLIGHT_W;
    static_assert(IN_FLIGHT <= 63, "ring deeper than vmcnt can count");
    // ... and in a wave that loads weights only, behind W(s) the weights of stages s+1 .. s+DEPTH-2:
    constexpr int IN_FLIGHT_W_ONLY = (DEPTH - 2) * W_INSTR;

    const int lane = lane_id();
    const int wave = wave_id();
    const int wn = wave % WN, wm = wave / WN;
    const bool loads_x = XW == WAVES || wave < XW;   // wave-uniform

    // Workgroups go to the eight XCDs round-robin by id, and each XCD has its own L2.  The workgroups that share a
    // weight tile (its activation tiles and K splits) take consecutive slots of ONE XCD, so the tile crosses the
    // fabric once and its readers run side by side: position j in an order that lists the weight tiles of XCD 0
    // (tile_n = 0, 8, 16 ...), then XCD 1's, each with all of its workgroups, and XCD x starting where its
    // share of the grid starts.  Tile counts that 8 does not divide put at most a few tiles on two XCDs.
    int tile_n, split, tile_m;
    {
        const int per_tile = a.split_k * a.m_tiles;
        int p;
        tile_n = xcd_weight_tile((int)blockIdx.x, (int)gridDim.x, per_tile, a.n_tiles, p);
        split = p / a.m_tiles;
        tile_m = p - split * a.m_tiles;
    }
    const int n0 = tile_n * BN;
    const int m0 = tile_m * BM;

    int b_begin, b_end;
    const int blocks_total = (a.k + 127) >> 7;         // 128-byte K blocks, the last of them partial in a TAIL build
    split_range(a, blocks_total, split, b_begin, b_end);
    const int n_blk = b_end - b_begin;
    const int old_pieces = TAIL ? (128 - (a.k & 127)) >> 4 : 0;   // 16-byte pieces of the last window that are not new
    // Every workgroup walks its K range from a different starting block (and wraps): workgroups that start
    // together would otherwise ask one L2 for the same activation lines at the same moment, block after
    // block, and queue up at one channel.  The start depends on the weight tile only, so the workgroups that
    // share weight rows (other activation tiles) still read them together and HBM serves them once.
    const int k_rot = (int)((((unsigned)tile_n >> 3) * 5u) % (unsigned)n_blk);
    auto k_block = [&](int s) __attribute__((always_inline)) {
        const int b = s + k_rot;
        return b_begin + (b >= n_blk ? b - n_blk : b);
    };

    // ---- DMA sources: instruction i of this wave covers stage rows 8*(4*i + wave) .. +7 ------
    const int d_row = lane >> 3;                 // row inside the 8-row instruction
    const int d_pp = lane & 7;                   // physical 16-byte piece inside the 128-byte row
    const uint8_t* wsrc[W_INSTR];
    const uint8_t* xsrc[X_INSTR];
#pragma unroll
    for (int i = 0; i < W_INSTR; i++) {
        const int row_l = 8 * (WAVES * i + wave) + d_row;       // row inside the weight part of the stage
        int row = n0 + row_l;
        row = row < a.n ? row : a.n - 1;
        wsrc[i] = a.B + (size_t)row * a.b_stride + ((d_pp ^ ((row_l >> 1) & 7)) << 4);
    }
#pragma unroll
    for (int i = 0; i < X_INSTR; i++) {
        const int row_l = 8 * (XW * i + (loads_x ? wave : 0)) + d_row;
        int row = m0 + row_l;
        row = row < a.m ? row : a.m - 1;
        xsrc[i] = a.A + (size_t)row * a.k + ((d_pp ^ ((row_l >> 1) & 7)) << 4);
    }
    const unsigned ring_lds = lds_addr(ring);
    // DMA instruction i of a stage's refill: the activation instructions come first, then the weights'
    auto issue_one = [&](int i, int sx, int sw) __attribute__((always_inline)) {
        // byte offset of K block kb inside a row: the last block of a TAIL build starts early, so that it ends with the row
        auto k_offset = [&](int kb) __attribute__((always_inline)) {
            return ((size_t)kb << 7) - ((TAIL && kb == blocks_total - 1) ? (size_t)(old_pieces << 4) : 0);
        };
        if (i < X_INSTR) {
            if (loads_x && sx < n_blk)
                dma_1kb(xsrc[i] + k_offset(k_block(sx)),
                        ring_lds + DEPTH * W_BYTES + (unsigned)(sx % DX) * X_BYTES + (XW * i + wave) * 1024);
        } else {
            if (sw < n_blk)
                dma_1kb_stream(wsrc[i - X_INSTR] + k_offset(k_block(sw)),
                               ring_lds + (unsigned)(sw % DEPTH) * W_BYTES + (WAVES * (i - X_INSTR) + wave) * 1024);
        }
    };
    auto issue_x = [&](int s) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < X_INSTR; i++) issue_one(i, s, 0);
    };
    auto issue_w = [&](int s) __attribute__((always_inline)) {
#pragma unroll
        for (int i = X_INSTR; i < PER_STAGE; i++) issue_one(i, 0, s);
    };

    // ---- LDS read offsets: lane (r, g) reads pieces g and g+4 of row r of a 16-row fragment ------
    const int r = lane & 15, g = lane >> 4;
    // pieces g and g + 4, not 2g and 2g + 1: with the row swizzle above the first choice is free of bank
    // conflicts at the LDS's full 256 B/clk, the second runs every ds_read_b128 at half rate (measured)
    const int piece0 = (g ^ ((r >> 1) & 7)) << 4;
    const int rd0 = r * 128 + piece0;
    const int rd1 = r * 128 + (piece0 ^ 64);
    const int w_base = (wn * RGW * 16) * 128;                   // this wave's weight rows inside a weight slot
    const int x_base = (wm * MH * 16) * 128;                    // this wave's activation rows inside an activation slot

    f32x4 acc[RGW][MH];
#pragma unroll
    for (int rg = 0; rg < RGW; rg++)
#pragma unroll
        for (int mb = 0; mb < MH; mb++) acc[rg][mb] = f32x4{0.f, 0.f, 0.f, 0.f};

    // Consumes stage s and, between the MFMA groups, issues the refill of the slots that stage s-1 left
    // (activations of stage sx, weights of stage sw).  Issued in one burst after the barrier the eight waves'
    // DMA instructions queue up at the CU's one texture-address unit and every wave stalls at issue, in
    // order, in front of its MFMAs; spread over the stage they are absorbed while the matrix cores work.
    auto consume = [&](int s, int sx, int sw) __attribute__((always_inline)) {
        const uint8_t* wslot = ring + (size_t)(s % DEPTH) * W_BYTES + w_base;
        const uint8_t* xslot = ring + (size_t)DEPTH * W_BYTES + (size_t)(s % DX) * X_BYTES + x_base;
        auto read_frag = [&](const uint8_t* p) __attribute__((always_inline)) {
            const i32x4 lo = *reinterpret_cast<const i32x4*>(p + rd0);
            const i32x4 hi = *reinterpret_cast<const i32x4*>(p + rd1);
            return i32x8{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
        };
        // TAIL: the stage that holds the last window - its activation pieces below the boundary are zero
        const bool last_window = TAIL && k_block(s) == blocks_total - 1;
        const bool zero_lo = last_window && g < old_pieces, zero_hi = last_window && g + 4 < old_pieces;
        auto read_x_frag = [&](const uint8_t* p) __attribute__((always_inline)) {
            i32x4 lo = *reinterpret_cast<const i32x4*>(p + rd0);
            i32x4 hi = *reinterpret_cast<const i32x4*>(p + rd1);
            if constexpr (TAIL) {
                if (zero_lo) lo = i32x4{0, 0, 0, 0};
                if (zero_hi) hi = i32x4{0, 0, 0, 0};
            }
            return i32x8{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
        };
        // the wave's weight fragments stay in registers for the stage; its activation fragments are
        // streamed one ahead of the MFMAs that use them, so that only the first reads of a stage are
        // exposed and the rest of the LDS traffic runs under the matrix cores
        i32x8 w[RGW];
#pragma unroll
        for (int rg = 0; rg < RGW; rg++) w[rg] = read_frag(wslot + rg * 2048);
        i32x8 x[2];
        x[0] = read_x_frag(xslot);
#pragma unroll
        for (int mb = 0; mb < MH; mb++) {
            if (mb + 1 < MH) x[(mb + 1) & 1] = read_x_frag(xslot + (mb + 1) * 2048);
#pragma unroll
            for (int i = mb * PER_STAGE / MH; i < (mb + 1) * PER_STAGE / MH; i++) issue_one(i, sx, sw);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int rg = 0; rg < RGW; rg++)
                acc[rg][mb] = mfma_e4m3_16x16x128(w[rg], x[mb & 1], acc[rg][mb]);
            // an MFMA has no side effects and its result is not read before the next stage, so the
            // optimizer would sink the group behind the reads and (conditional) refills that follow, and
            // hoist every read to the top; naming the accumulators as operands of an asm with a memory
            // clobber keeps each group, and the reads around it, where they are written
#pragma unroll
            for (int rg = 0; rg < RGW; rg++) asm volatile("" : "+v"(acc[rg][mb])::"memory");
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    // Four-wave workgroups (one wave per SIMD) measure faster the plain way: refill in one burst after the
    // barrier, all activation fragments read up front, weight fragments one by one.
    auto consume_burst = [&](int s, int sx, int sw) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < PER_STAGE; i++) issue_one(i, sx, sw);
        __builtin_amdgcn_sched_barrier(0);
        const uint8_t* wslot = ring + (size_t)(s % DEPTH) * W_BYTES + w_base;
        const uint8_t* xslot = ring + (size_t)DEPTH * W_BYTES + (size_t)(s % DX) * X_BYTES + x_base;
        const bool last_window = TAIL && k_block(s) == blocks_total - 1;
        const bool zero_lo = last_window && g < old_pieces, zero_hi = last_window && g + 4 < old_pieces;
        i32x8 x[MH];
#pragma unroll
        for (int mb = 0; mb < MH; mb++) {
            i32x4 lo = *reinterpret_cast<const i32x4*>(xslot + mb * 2048 + rd0);
            i32x4 hi = *reinterpret_cast<const i32x4*>(xslot + mb * 2048 + rd1);
            if constexpr (TAIL) {
                if (zero_lo) lo = i32x4{0, 0, 0, 0};
                if (zero_hi) hi = i32x4{0, 0, 0, 0};
            }
            x[mb] = i32x8{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
        }
#pragma unroll
        for (int rg = 0; rg < RGW; rg++) {
            const i32x4 lo = *reinterpret_cast<const i32x4*>(wslot + rg * 2048 + rd0);
            const i32x4 hi = *reinterpret_cast<const i32x4*>(wslot + rg * 2048 + rd1);
            const i32x8 w = i32x8{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
#pragma unroll
            for (int mb = 0; mb < MH; mb++)
                acc[rg][mb] = mfma_e4m3_16x16x128(w, x[mb], acc[rg][mb]);
        }
    };

    // ---- pipeline ------------------------------------------------------------------------------
    for (int i = 0; i < DEPTH - 1; i++) {
        if (i < DX - 1 && i < n_blk) issue_x(i);
        if (i < n_blk) issue_w(i);
    }
    stamps.mark(1);
    for (int s = 0; s < n_blk; s++) {
        // wait for this wave's part of stage s; everything issued after it may stay in flight.  Near the
        // end of the K range fewer stages follow, and the count is no longer known at compile time.
        if (s + DEPTH - 2 >= n_blk) wait_vmcnt<0>();
        else if (loads_x) wait_vmcnt<IN_FLIGHT>();
        else wait_vmcnt<IN_FLIGHT_W_ONLY>();
        __syncthreads();        // stage s is complete for every wave; stage s-1 has been consumed by every wave
        if (s == 0) stamps.mark(2);
        __builtin_amdgcn_sched_barrier(0);
        // refills the slots of X(s-1) and W(s-1) on the way
        if constexpr (WN == 2) consume_burst(s, s + DX - 1, s + DEPTH - 1);
        else consume(s, s + DX - 1, s + DEPTH - 1);
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    }

    stamps.mark(3);

    // ---- epilogue --------------------------------------------------------------------------------
    const float scale = a.scale ? a.scale[0] : 1.0f;
    auto store_all = [&](auto&& get) __attribute__((always_inline)) {
#pragma unroll
        for (int rg = 0; rg < RGW; rg++)
#pragma unroll
            for (int mb = 0; mb < MH; mb++)
                store_fragment(a, get(rg, mb), scale, m0 + (wm * MH + mb) * 16 + r, n0 + (wn * RGW + rg) * 16 + 4 * g);
    };
    if (a.split_k == 1) {
        store_all([&](int rg, int mb) { return acc[rg][mb]; });
        stamps.end(a);
        return;
    }

    // split-K: agent-scope partial stores, arrival counter, last workgroup sums in split order
    constexpr int FRAGS_WG = WAVES * RGW * MH;   // fragments of one workgroup tile
    const int tile_id = tile_m * a.n_tiles + tile_n;
    float* ws_tile = a.ws + ((size_t)tile_id * a.split_k) * (FRAGS_WG * 256);
    if (a.defer_reduce) {
        // partials only: [tile][split][wave][fragment][lane] as one 16-byte store per lane and fragment
        f32x4* mine = reinterpret_cast<f32x4*>(ws_tile + (size_t)split * (FRAGS_WG * 256) + (size_t)wave * (RGW * MH * 256)) + lane;
#pragma unroll
        for (int rg = 0; rg < RGW; rg++)
#pragma unroll
            for (int mb = 0; mb < MH; mb++) mine[(rg * MH + mb) * 64] = acc[rg][mb];
        stamps.end(a);
        return;
    }
    {
        float* mine = ws_tile + (size_t)split * (FRAGS_WG * 256) + (size_t)wave * (RGW * MH * 256) + lane;
#pragma unroll
        for (int rg = 0; rg < RGW; rg++)
#pragma unroll
            for (int mb = 0; mb < MH; mb++)
#pragma unroll
                for (int e = 0; e < 4; e++)
                    __hip_atomic_store(mine + (rg * MH + mb) * 256 + e * 64, acc[rg][mb][e], __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_AGENT);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    volatile unsigned* arrival = reinterpret_cast<volatile unsigned*>(ring + (size_t)RING_BYTES);
    if (threadIdx.x == 0)
        *arrival = __hip_atomic_fetch_add(&a.counters[tile_id], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    if (*arrival != (unsigned)(a.split_k - 1)) {
        stamps.end(a);
        return;
    }
    store_all([&](int rg, int mb) {
        const float* p = ws_tile + (size_t)wave * (RGW * MH * 256) + (rg * MH + mb) * 256 + lane;
        f32x4 v = {0.f, 0.f, 0.f, 0.f};
        for (int sp = 0; sp < a.split_k; sp++) {
            const float* q = p + (size_t)sp * (FRAGS_WG * 256);
#pragma unroll
            for (int e = 0; e < 4; e++) v[e] += __hip_atomic_load(q + e * 64, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        return v;
    });
    if (threadIdx.x == 0) __hip_atomic_store(&a.counters[tile_id], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    stamps.end(a);
}


// Second launch of a mid-batch GEMM whose split-K sum was deferred: every wave adds the split_k partials of
// kReduceFrags 16 x 16 fragments of the output in split order - what the last workgroup to arrive does in the single
// launch, so the result bits are the same - and applies scale, row and column factors and the rounding.  A wave's
// work is a chain of round trips (partials, scale, store), so it takes several fragments at once and requests all
// their partials of a split before it adds any: with one fragment per wave the launch took 7-12 us for 8-33 MB of
// partials that the GEMM had just left in the caches.  The tile geometry comes as run-time values: rgw x mh
// fragments per wave of the GEMM, wn x 2 waves per tile.
constexpr int kReduceFrags = 4;
__global__ void __launch_bounds__(256) mid_reduce_kernel(const StreamArgs a, int rgw, int mh, int wn) {
    const int fr = rgw * mh, frags_wg = 2 * wn * fr;      // fr is a multiple of kReduceFrags (rgw, mh are 2, 4 or 8)
    const int lane = lane_id();
    // a workgroup takes 4 * kReduceFrags consecutive fragments of one tile; the workgroups of a weight tile sit on the
    // XCD that computed it (the grid is n_tiles * m_tiles * chunks workgroups, chunks per tile)
    const int chunks = (frags_wg + 4 * kReduceFrags - 1) / (4 * kReduceFrags);   // (the last one may have idle waves)
    int pos;
    const int tile_n = xcd_weight_tile((int)blockIdx.x, (int)gridDim.x, a.m_tiles * chunks, a.n_tiles, pos);
    const int tile_m = pos / chunks, chunk = pos - tile_m * chunks;
    if (tile_n >= a.n_tiles || tile_m >= a.m_tiles) return;
    const unsigned tile_id = (unsigned)(tile_m * a.n_tiles + tile_n);
    const unsigned rem = (unsigned)((chunk * 4 + wave_id()) * kReduceFrags);     // (wave of the tile, fragment of the wave)
    if (rem >= (unsigned)frags_wg) return;
    const float scale = a.scale ? a.scale[0] : 1.0f;
    const int wave = (int)rem / fr, f0 = (int)rem - wave * fr;
    const int wq = wave % wn, wm = wave / wn;
    const f32x4* p = reinterpret_cast<const f32x4*>(a.ws + ((size_t)tile_id * a.split_k) * ((size_t)frags_wg * 256) +
                                                    (size_t)wave * (fr * 256) + (size_t)f0 * 256) + lane;
    const size_t split_stride = (size_t)frags_wg * 64;
    f32x4 v[kReduceFrags];
#pragma unroll
    for (int j = 0; j < kReduceFrags; j++) v[j] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll 2
    for (int sp = 0; sp < a.split_k; sp++) {
        f32x4 t[kReduceFrags];
#pragma unroll
        for (int j = 0; j < kReduceFrags; j++) t[j] = p[(size_t)sp * split_stride + j * 64];
#pragma unroll
        for (int j = 0; j < kReduceFrags; j++) v[j] += t[j];
    }
    const int r = lane & 15, g = lane >> 4;
#pragma unroll
    for (int j = 0; j < kReduceFrags; j++) {
        const int f = f0 + j, rg = f / mh, mb = f - rg * mh;
        store_fragment(a, v[j], scale, tile_m * (32 * mh) + (wm * mh + mb) * 16 + r, tile_n * (16 * rgw * wn) + (wq * rgw + rg) * 16 + 4 * g);
    }
}

}  // namespace sg
