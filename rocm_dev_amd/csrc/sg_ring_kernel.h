// Producer/consumer LDS-ring FP8 skinny GEMM for gfx950 - the warp-specialised pipeline of the
// reference (skinny_gemm/skinny_gemm_kernel.cu:6-110 and its async_gemm_* ancestors), rebuilt
// on gfx950's direct-to-LDS loads and with an explicitly ordered flag protocol.
//
// Roles inside one workgroup (wave index order, as skinny_gemm_kernel.cu:37-41):
//   A producers   fetch the activation tile of a K block (256 bytes of K) into the ring slot
//   B producers   fetch one 16-row weight tile ("lane") of a K block into the ring slot
//   consumers     own whole K blocks: read the activation tile, then every weight tile of the
//                 block, and issue the MFMAs; each consumer keeps its own fp32 partial tile
// The grid is persistent: workgroup w walks work items w, w + grid, ... and the ring, its flags and
// every role's position simply continue from one item to the next.  A work item is one K split of
// one output tile (skinny_gemm_kernel.cu:44-64 decodes the same triple from its tile counter): the
// items of a tile may run on different workgroups, their fp32 partials meet in the split-K
// workspace, one arrival counter per 16 x 16 fragment, and the wave that arrives last adds them in
// split order - no barrier that a producer wave would have to join.
//
// Ring and flags (layout of skinny_gemm_kernel.cu:27-30).  Block g of the workgroup's running
// block count lives in slot g % QSIZE.  queue[2*BL*slot] guards the slot's activation tile,
// queue[2*(BL*slot + lane) + 1] guards weight tile `lane`.  A flag only ever counts up: for
// the n-th use of a slot (n = g / QSIZE) the producer waits for 2n, fills, stores 2n + 1; the
// consumer waits for 2n + 1, reads, stores 2n + 2.  Nothing is ever reset, which is the
// reference's "p_state += 2 on wrap" (n_full_tiles.cu:118-120) stated on the block counter.
//
// Ordering, where the reference relies on luck (plain LDS reads in a spin loop, no waits
// between data and flag):
//   producer  DMA ... s_waitcnt vmcnt(n)  -> the data of the oldest item is in LDS
//             flag store (volatile LDS store behind a compiler barrier)
//   consumer  flag load (volatile) ... data ds_reads: LDS operations of one wave execute in
//             order, the compiler barrier keeps the data reads behind the flag read
//             s_waitcnt lgkmcnt(0) -> data is in registers -> flag store releases the slot
// A producer never blocks on a full slot while it still owes a signal: it first retires its
// outstanding DMAs, so the consumer that must free the slot can always make progress.
#pragma once

#include "sg_device.h"
#include "sg_epilogue.h"
#include "sg_lds_kernel.h"

namespace sg {

struct RingArgs {
    StreamArgs g;       // operands and shape; g.waves = consumers; g.counters holds one word per fragment of every tile
    int a_producers;
    int b_producers;
    int consumers;
    int qsize;
};

// Every lane reads the same word; readfirstlane makes the value (and the control flow that
// depends on it) wave-uniform for the compiler as well.
__device__ __forceinline__ int flag_load(const volatile int* f) {
    const int v = __builtin_amdgcn_readfirstlane(*f);
    asm volatile("" ::: "memory");
    return v;
}
__device__ __forceinline__ void flag_store(volatile int* f, int v) {
    asm volatile("" ::: "memory");
    *f = v;
}
__device__ __forceinline__ void flag_wait(const volatile int* f, int want) {
    while (flag_load(f) != want) __builtin_amdgcn_s_sleep(1);
}

// waits until at most `n` vector-memory operations of this wave are outstanding (n <= 28)
__device__ __forceinline__ void wait_vmcnt_rt(int n) {
    switch (n) {
#define SG_W(N) case N: wait_vmcnt<N>(); break;
        SG_W(0) SG_W(1) SG_W(2) SG_W(3) SG_W(4) SG_W(5) SG_W(6) SG_W(7) SG_W(8) SG_W(9) SG_W(10) SG_W(11) SG_W(12)
        SG_W(13) SG_W(14) SG_W(15) SG_W(16) SG_W(17) SG_W(18) SG_W(19) SG_W(20) SG_W(21) SG_W(22) SG_W(23) SG_W(24)
        SG_W(25) SG_W(26) SG_W(27) SG_W(28)
#undef SG_W
        default: wait_vmcnt<0>(); break;
    }
}

constexpr int kRingMaxPending = 4;  // DMA items a producer keeps in flight before it signals the oldest

// BL = weight tiles ("lanes") per K block, XU = activation DMA instructions per K block
template <int MT, int BL, int XU, bool NT>
__global__ void __launch_bounds__(1024) ring_gemm_kernel(const RingArgs ra) {
    extern __shared__ __attribute__((aligned(1024))) uint8_t ring[];  // [QSIZE][slot] | red[2][FRAGS][consumers][64] | queue[2*BL*QSIZE] | arrivals[2]
    const StreamArgs& a = ra.g;

    constexpr int SLOT_BYTES = (BL * 4 + XU) * 1024;
    constexpr int FRAGS = BL * MT;

    const int lane = lane_id();
    const int wave = wave_id();
    const int PA = ra.a_producers, PB = ra.b_producers, C = ra.consumers, Q = ra.qsize;
    const int r = lane & 15, g16 = lane >> 4;

    f32x4* red = reinterpret_cast<f32x4*>(ring + (size_t)Q * SLOT_BYTES);
    volatile int* queue = reinterpret_cast<volatile int*>(ring + (size_t)Q * SLOT_BYTES + 2u * FRAGS * C * 1024);
    for (int i = threadIdx.x; i < 2 * BL * Q + 2; i += blockDim.x) queue[i] = 0;  // flags + two arrival counters
    __syncthreads();

    const int total_items = a.n_tiles * a.m_tiles * a.split_k;
    const int my_items = ((int)blockIdx.x < total_items) ? (total_items - (int)blockIdx.x + (int)gridDim.x - 1) / (int)gridDim.x : 0;
    const int blocks = a.k >> 8;                 // K blocks per tile
    const unsigned ring_lds = lds_addr(ring);

    // The j-th work item of this workgroup: its tile, K split and K range.  Items are numbered as decode_tile orders
    // them - the activation (m) tiles of a weight tile fastest, then the n tiles, then the K splits; the last split
    // takes the remainder of K, so items differ
    // in length and every role walks them with a cursor over the workgroup's running block count.
    struct Item { int n0, m0, tile_id, split, kb0, cnt; };
    auto item_at = [&](int j) __attribute__((always_inline)) {
        Item it;
        int tile_n, tile_m, b_begin, b_end;
        decode_tile(a, (int)blockIdx.x + j * (int)gridDim.x, tile_n, it.split, tile_m);
        split_range(a, blocks, it.split, b_begin, b_end);
        it.n0 = tile_n * (16 * BL);
        it.m0 = tile_m * (16 * MT);
        it.tile_id = tile_m * a.n_tiles + tile_n;
        it.kb0 = b_begin;
        it.cnt = b_end - b_begin;
        return it;
    };
    int total_blocks = 0;                        // running block count of this workgroup over all its items
    for (int j = 0; j < my_items; j++) total_blocks += item_at(j).cnt;

    const int q4 = lane >> 2, p4 = lane & 3;
    const int src_row = q4 & 3;
    const int src_col = (q4 >> 2) * 64;

    if (wave < PA + PB) {
        // ------------------------------ producers ------------------------------------------
        const bool is_a = wave < PA;
        const int me = is_a ? wave : wave - PA;
        const int P = is_a ? PA : PB;
        const int n_items = is_a ? total_blocks : total_blocks * BL;   // B items: (block, lane) pairs
        const int per_item = is_a ? XU : 4;                            // DMA instructions per item

        auto flag_of = [&](int item) __attribute__((always_inline)) -> volatile int* {
            const int gb = is_a ? item : item / BL;
            const int slot = gb % Q;
            return is_a ? &queue[2 * BL * slot] : &queue[2 * (BL * slot + (item - gb * BL)) + 1];
        };
        auto phase_of = [&](int item) __attribute__((always_inline)) { return 2 * ((is_a ? item : item / BL) / Q); };
        // cursor of the issue side: the work item that holds running block gb (gb only ever grows)
        int cur_j = 0, cur_base = 0;
        Item cur = my_items > 0 ? item_at(0) : Item{0, 0, 0, 0, 0, 1};
        auto issue = [&](int item) __attribute__((always_inline)) {
            const int gb = is_a ? item : item / BL;
            const int ln = is_a ? 0 : item - gb * BL;
            while (gb >= cur_base + cur.cnt) {
                cur_base += cur.cnt;
                cur = item_at(++cur_j);
            }
            const int kb = cur.kb0 + (gb - cur_base);
            const int m0 = cur.m0, n0 = cur.n0;
            const unsigned slot = ring_lds + (unsigned)(gb % Q) * SLOT_BYTES;
            const size_t koff = ((size_t)kb << 8) + src_col;
            if (is_a) {
#pragma unroll
                for (int u = 0; u < XU; u++) {
                    int row = m0 + 4 * u + src_row;
                    row = row < a.m ? row : a.m - 1;
                    dma_1kb(a.A + (size_t)row * a.k + koff + ((p4 + (u & 3)) & 3) * 16, slot + (BL * 4 + u) * 1024);
                }
            } else {
#pragma unroll
                for (int u = 0; u < 4; u++) {
                    int row = n0 + ln * 16 + 4 * u + src_row;
                    row = row < a.n ? row : a.n - 1;
                    const uint8_t* src = a.B + (size_t)row * a.b_stride + koff + ((p4 + u) & 3) * 16;
                    if (NT) dma_1kb_stream(src, slot + (ln * 4 + u) * 1024);
                    else dma_1kb(src, slot + (ln * 4 + u) * 1024);
                }
            }
        };

        int next = me, retire = me, pending = 0;
        while (retire < n_items) {
            const bool can_issue =
                next < n_items && pending < kRingMaxPending && flag_load(flag_of(next)) == phase_of(next);
            if (can_issue) {
                issue(next);
                next += P;
                pending++;
            } else if (pending > 0) {
                wait_vmcnt_rt((pending - 1) * per_item);   // the oldest item's data has landed
                flag_store(flag_of(retire), phase_of(retire) + 1);
                retire += P;
                pending--;
            } else {
                __builtin_amdgcn_s_sleep(1);               // nothing in flight and the slot is still being read
            }
        }
        return;  // the consumers' reductions synchronise among consumers only
    }

    // ---------------------------------- consumers ----------------------------------------------
    const int c = wave - PA - PB;
    const int rd_off = 1024 * (r >> 2) + 64 * (r & 3) + 16 * ((g16 - (r >> 2)) & 3);
    const float scale = a.scale ? a.scale[0] : 1.0f;

    f32x4 acc[BL][MT];
#pragma unroll
    for (int ln = 0; ln < BL; ln++)
#pragma unroll
        for (int mt = 0; mt < MT; mt++) acc[ln][mt] = f32x4{0.f, 0.f, 0.f, 0.f};

    // One finished fragment of work item `it` (already summed over this workgroup's consumers).  Unsplit: scale,
    // round, store.  Split: the partial goes to the workspace with agent-scope stores (past this XCD's L2), the wave
    // waits for their acknowledgement and then bumps the fragment's arrival counter; the wave that finds split_k - 1
    // earlier arrivals reads all partials back in split order, stores the result and zeroes the counter again.
    auto finish = [&](const Item& it, int f, f32x4 v) __attribute__((always_inline)) {
        const int m_idx = it.m0 + (f % MT) * 16 + r, n_idx = it.n0 + (f / MT) * 16 + 4 * g16;
        if (a.split_k == 1) {
            store_fragment(a, v, scale, m_idx, n_idx);
            return;
        }
        float* tile_ws = a.ws + ((size_t)it.tile_id * a.split_k) * (FRAGS * 256);
        float* p = tile_ws + ((size_t)it.split * FRAGS + f) * 256 + lane;
#pragma unroll
        for (int e = 0; e < 4; e++) __hip_atomic_store(p + e * 64, v[e], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        unsigned* counter = a.counters + (size_t)it.tile_id * FRAGS + f;
        unsigned arrived = 0;
        if (lane == 0) arrived = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        arrived = __builtin_amdgcn_readfirstlane(arrived);
        if (arrived != (unsigned)(a.split_k - 1)) return;
        const float* q = tile_ws + (size_t)f * 256 + lane;
        f32x4 sum;
#pragma unroll
        for (int e = 0; e < 4; e++) sum[e] = __hip_atomic_load(q + e * 64, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        for (int sp = 1; sp < a.split_k; sp++) {
            const float* qs = q + (size_t)sp * FRAGS * 256;
#pragma unroll
            for (int e = 0; e < 4; e++) sum[e] += __hip_atomic_load(qs + e * 64, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        store_fragment(a, sum, scale, m_idx, n_idx);
        if (lane == 0) __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // ready for the next launch
    };

    int gb_lo = 0;   // running block index at which item j starts
    for (int j = 0; j < my_items; j++) {
        const Item it = item_at(j);
        // blocks of item j: running indices gb_lo .. gb_lo + cnt - 1; mine are those = c (mod C)
        const int gb_hi = gb_lo + it.cnt;
        int gb = gb_lo + ((c - gb_lo % C) + C) % C;
        for (; gb < gb_hi; gb += C) {
            const int slot = gb % Q;
            const int full = 2 * (gb / Q) + 1;
            const uint8_t* base = ring + (size_t)slot * SLOT_BYTES + rd_off;
            volatile int* fa = &queue[2 * BL * slot];
            flag_wait(fa, full);
            // the lane's 16-byte pieces of the block's four 64-byte chunks: chunks 0,1 feed the first
            // 128-byte MFMA, chunks 2,3 the second (same pieces for both operands, as in mma_block_256)
            i32x8 x[MT][2];
#pragma unroll
            for (int mt = 0; mt < MT; mt++)
#pragma unroll
                for (int h = 0; h < 2; h++) {
                    const i32x4 lo = *reinterpret_cast<const i32x4*>(base + (BL * 4 + mt * 4) * 1024 + (2 * h) * 256);
                    const i32x4 hi = *reinterpret_cast<const i32x4*>(base + (BL * 4 + mt * 4) * 1024 + (2 * h + 1) * 256);
                    x[mt][h] = i32x8{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
                }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            flag_store(fa, full + 1);
#pragma unroll
            for (int ln = 0; ln < BL; ln++) {
                volatile int* fb = &queue[2 * (BL * slot + ln) + 1];
                flag_wait(fb, full);
                i32x8 w[2];
#pragma unroll
                for (int h = 0; h < 2; h++) {
                    const i32x4 lo = *reinterpret_cast<const i32x4*>(base + ln * 4096 + (2 * h) * 256);
                    const i32x4 hi = *reinterpret_cast<const i32x4*>(base + ln * 4096 + (2 * h + 1) * 256);
                    w[h] = i32x8{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
                }
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                flag_store(fb, full + 1);
#pragma unroll
                for (int h = 0; h < 2; h++)
#pragma unroll
                    for (int mt = 0; mt < MT; mt++) acc[ln][mt] = mfma_e4m3_16x16x128(w[h], x[mt][h], acc[ln][mt]);
            }
        }
        gb_lo = gb_hi;

        // item j is complete for this consumer: sum the consumers' partials in consumer order
        if (C == 1) {
#pragma unroll
            for (int f = 0; f < FRAGS; f++) finish(it, f, acc[f / MT][f % MT]);
        } else {
            // Consumer-only rendezvous (producers are busy with the next items and must not be
            // stalled by a workgroup barrier): each consumer publishes its partial, then bumps an
            // arrival counter that only ever counts up; buffer and counter alternate by item parity.
            f32x4* buf = red + (size_t)(j & 1) * (FRAGS * C * 64);
#pragma unroll
            for (int f = 0; f < FRAGS; f++) buf[(f * C + c) * 64 + lane] = acc[f / MT][f % MT];
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            int* arrive = const_cast<int*>(&queue[2 * BL * Q + (j & 1)]);
            if (lane == 0) __hip_atomic_fetch_add(arrive, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            flag_wait(arrive, C * ((j >> 1) + 1));
            for (int f = c; f < FRAGS; f += C) {
                f32x4 v = buf[(f * C) * 64 + lane];
                for (int w = 1; w < C; w++) v += buf[(f * C + w) * 64 + lane];
                finish(it, f, v);
            }
        }
#pragma unroll
        for (int ln = 0; ln < BL; ln++)
#pragma unroll
            for (int mt = 0; mt < MT; mt++) acc[ln][mt] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
}

}  // namespace sg
