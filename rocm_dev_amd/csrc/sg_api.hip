// C ABI of libsgemm.so: argument validation, configuration choice and launches.
// The contract of every entry point is documented in include/sgemm.h.
#include <dlfcn.h>

#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <tuple>
#include <vector>

#include "sg_host.h"
#include "sg_stream_kernel.h"
#include "sg_ring_kernel.h"
#include "sg_sparse_kernel.h"
#include "sg_debug_kernel.h"
#include <string>

namespace sg {

int launch_fp8_encode_rows(const void* X, uint8_t* Q, float* scales, int rows, int cols, hipStream_t stream);
int launch_fp8_decode_rows(const uint8_t* Q, const float* scales, void* Y, int rows, int cols, hipStream_t stream);
int launch_fp8_reduce_rows(const uint8_t* Q, const float* scales, void* Y, int nbuf, size_t q_buf_stride, int rows,
                           int cols, hipStream_t stream);
int launch_tiled_sum_reduce(const float* A, const float* B, float* D, int b, int m, int n, hipStream_t stream);
int launch_tiled_sum_reduce_ring(const float* A, const float* B, float* D, int b, int m, int n, hipStream_t stream);
int launch_sparse24_compress(const uint8_t* B, uint8_t* vals, uint8_t* meta, int n, int k, int b_stride, hipStream_t stream);

// ---- per-device state -------------------------------------------------------------------
constexpr int kMaxDevices = 16;
constexpr size_t kDefaultPartialBytes = 64u << 20;  // what sg_init() sets up for the default stream
constexpr size_t kMinPartialBytes = 4u << 20;       // smallest partials buffer created on demand
constexpr size_t kMaxPartialBytes = 512u << 20;     // one launch may not ask for more
constexpr size_t kMinCounters = 1u << 14;           // arrival counters (one per output tile)
constexpr size_t kMaxCounters = 1u << 22;

static std::mutex g_mutex;
// Split-K workspaces, one per (device, stream).  Launches on one stream run in order and may share
// their partials and arrival counters; launches on different streams may overlap and must not.
static std::map<hipStream_t, Workspace> g_ws[kMaxDevices];
static size_t g_ws_bytes[kMaxDevices];   // device memory held by the workspaces of a device (retired buffers included)
// Buffers a workspace has outgrown: launches already enqueued may still use them, so they are only freed by
// sg_release_workspaces / sg_release_stream, behind a synchronisation.
struct Retired { hipStream_t stream; void* p; size_t bytes; };
static std::vector<Retired> g_retired[kMaxDevices];
static DeviceInfo g_dev[kMaxDevices];
static bool g_dev_known[kMaxDevices];

hipError_t report_hip(const char* what, hipError_t e) {
    if (e != hipSuccess && getenv("SG_VERBOSE")) fprintf(stderr, "libsgemm: %s: %s\n", what, hipGetErrorString(e));
    return e;
}

static int current_device(int* dev) {
    if (hipGetDevice(dev) != hipSuccess || *dev < 0 || *dev >= kMaxDevices) {
        (void)hipGetLastError();
        return SG_NO_DEVICE;
    }
    return SG_SUCCESS;
}

int get_device_info(DeviceInfo** out) {
    int dev;
    if (int rc = current_device(&dev)) return rc;
    std::lock_guard<std::mutex> lock(g_mutex);
    if (!g_dev_known[dev]) {
        hipDeviceProp_t prop;
        if (hipGetDeviceProperties(&prop, dev) != hipSuccess) {
            (void)hipGetLastError();
            return SG_NO_DEVICE;
        }
        g_dev[dev].cu_count = prop.multiProcessorCount;
        g_dev[dev].lds_per_block = (int)prop.sharedMemPerBlock;
        g_dev[dev].is_gfx950 = std::string(prop.gcnArchName).rfind("gfx950", 0) == 0;
        g_dev_known[dev] = true;
    }
    *out = &g_dev[dev];
    return g_dev[dev].is_gfx950 ? SG_SUCCESS : SG_NO_DEVICE;
}

static size_t round_up_pow2(size_t v, size_t floor) {
    size_t r = floor;
    while (r < v) r <<= 1;
    return r;
}

// Device memory for a workspace.  A stream under capture in the default (global) capture mode refuses
// allocation calls made by its thread; the mode is relaxed for the duration of the call, which
// records nothing into the graph.
static void* workspace_alloc(size_t bytes) {
    hipStreamCaptureMode mode = hipStreamCaptureModeRelaxed;
    const bool exchanged = hipThreadExchangeStreamCaptureMode(&mode) == hipSuccess;
    void* p = nullptr;
    if (hipMalloc(&p, bytes) != hipSuccess) {
        (void)hipGetLastError();
        p = nullptr;
    }
    if (exchanged) (void)hipThreadExchangeStreamCaptureMode(&mode);
    return p;
}

__global__ void fill_zero_kernel(unsigned* p, size_t n) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) p[i] = 0u;
}

// Zeroes n words on `stream` with a kernel (not a memset: a memset node recorded into a captured
// graph is not reliable on replays), so that every later launch on that stream finds them zero.
static int fill_zero(unsigned* p, size_t n, hipStream_t stream) {
    const unsigned grid = (unsigned)((n + 255) / 256 < 1024 ? (n + 255) / 256 : 1024);
    hipLaunchKernelGGL(fill_zero_kernel, dim3(grid), dim3(256), 0, stream, p, n);
    if (report_hip("fill_zero_kernel", hipGetLastError()) != hipSuccess) return SG_LAUNCH_FAILED;
    return SG_SUCCESS;
}

// Zeroes n words of a buffer that nothing uses yet, now: on a stream of the library's own (non-blocking, so it
// neither joins nor disturbs a capture in progress on the caller's stream), waited for before returning.
static int fill_zero_now(unsigned* p, size_t n) {
    hipStreamCaptureMode mode = hipStreamCaptureModeRelaxed;
    const bool exchanged = hipThreadExchangeStreamCaptureMode(&mode) == hipSuccess;
    hipStream_t own = nullptr;
    int rc = SG_LAUNCH_FAILED;
    if (report_hip("hipStreamCreateWithFlags", hipStreamCreateWithFlags(&own, hipStreamNonBlocking)) == hipSuccess) {
        rc = fill_zero(p, n, own);
        if (rc == SG_SUCCESS && report_hip("hipStreamSynchronize", hipStreamSynchronize(own)) != hipSuccess) rc = SG_LAUNCH_FAILED;
        (void)hipStreamDestroy(own);
    } else {
        (void)hipGetLastError();
    }
    if (exchanged) (void)hipThreadExchangeStreamCaptureMode(&mode);
    return rc;
}

static bool stream_is_capturing(hipStream_t stream) {
    hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &status) != hipSuccess) {
        (void)hipGetLastError();
        return false;
    }
    return status != hipStreamCaptureStatusNone;
}

// The workspace of `stream` on the current device, grown to hold partial_bytes of fp32 partials and
// n_counters arrival counters.  A buffer that is outgrown is kept until the process ends (launches
// already enqueued may still use it); sizes double, so what is kept is less than what is in use.
int get_workspace(hipStream_t stream, size_t partial_bytes, size_t n_counters, Workspace* out) {
    if (partial_bytes > kMaxPartialBytes || n_counters > kMaxCounters) return SG_WORKSPACE_TOO_SMALL;
    int dev;
    if (int rc = current_device(&dev)) return rc;
    std::lock_guard<std::mutex> lock(g_mutex);
    Workspace& w = g_ws[dev][stream];
    if (w.partial_bytes < partial_bytes) {
        const size_t bytes = round_up_pow2(partial_bytes, kMinPartialBytes);
        void* p = workspace_alloc(bytes);
        if (!p) return SG_NO_DEVICE;
        if (w.partials) g_retired[dev].push_back({stream, w.partials, w.partial_bytes});
        w.partials = static_cast<float*>(p);
        w.partial_bytes = bytes;
        g_ws_bytes[dev] += bytes;
    }
    if (w.n_counters < n_counters) {
        const size_t n = round_up_pow2(n_counters, kMinCounters);
        void* c = workspace_alloc(n * sizeof(unsigned));
        if (!c) return SG_NO_DEVICE;
        // Zero before the launch that asked for them (and every later one on this stream): in stream order - unless the
        // stream is being captured, where a kernel launched on it would only be recorded: then at once, outside the
        // graph, so that the graph's replays and eager launches on the stream alike find the counters zero.
        const int rc = stream_is_capturing(stream) ? fill_zero_now(static_cast<unsigned*>(c), n)
                                                   : fill_zero(static_cast<unsigned*>(c), n, stream);
        if (rc) {
            (void)hipFree(c);
            return rc;
        }
        if (w.counters) g_retired[dev].push_back({stream, w.counters, w.n_counters * sizeof(unsigned)});
        w.counters = static_cast<unsigned*>(c);
        w.n_counters = n;
        g_ws_bytes[dev] += n * sizeof(unsigned);
    }
    *out = w;
    return SG_SUCCESS;
}

// ---- scratch for the entry point that allocates nothing -------------------------------------------
// Split-K partials and arrival counters of sg_skinny_gemm_tuned_noalloc live in this array instead of a
// workspace from hipMalloc.  Every device the library runs on holds its own copy at its own address; in host
// code the name below is only a handle for hipGetSymbolAddress, never a device address.
constexpr size_t kStaticPartialBytes = 8u << 20;
constexpr size_t kStaticCounters = 4096;
static __device__ __align__(256) unsigned char scratch[kStaticPartialBytes + kStaticCounters * sizeof(unsigned)];
static unsigned char* g_scratch_ptr[kMaxDevices];   // device address of `scratch` per device, looked up once

// *first_use is set when this call looked the address up (the first call on the device).
static int static_workspace(Workspace* out, bool* first_use) {
    int dev;
    if (int rc = current_device(&dev)) return rc;
    std::lock_guard<std::mutex> lock(g_mutex);
    *first_use = false;
    if (!g_scratch_ptr[dev]) {
        void* ptr = nullptr;
        if (report_hip("hipGetSymbolAddress", hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch))) != hipSuccess || !ptr) {
            (void)hipGetLastError();
            return SG_NO_DEVICE;
        }
        g_scratch_ptr[dev] = static_cast<unsigned char*>(ptr);
        *first_use = true;
    }
    out->partials = reinterpret_cast<float*>(g_scratch_ptr[dev]);
    out->partial_bytes = kStaticPartialBytes;
    out->counters = reinterpret_cast<unsigned*>(g_scratch_ptr[dev] + kStaticPartialBytes);
    out->n_counters = kStaticCounters;
    return SG_SUCCESS;
}

// ---- time stamps (profiling aid) -------------------------------------------------------------------
static unsigned long long* g_stamp_buf = nullptr;
static size_t g_stamp_words = 0, g_stamp_cursor = 0;
static std::atomic<bool> g_stamps_on{false};   // the launch path takes the lock below only while a buffer is set

// Room for one launch of `grid` workgroups, or nullptr when stamps are off or the buffer is full.
static unsigned long long* take_stamps(unsigned grid) {
    if (!g_stamps_on.load(std::memory_order_relaxed)) return nullptr;
    std::lock_guard<std::mutex> lock(g_mutex);
    const size_t need = (size_t)grid * kStampWords;
    if (!g_stamp_buf || g_stamp_cursor + need > g_stamp_words) return nullptr;
    unsigned long long* p = g_stamp_buf + g_stamp_cursor;
    g_stamp_cursor += need;
    return p;
}

// ---- kernel dispatch ------------------------------------------------------------------------
enum Engine { ENGINE_AUTO = 0, ENGINE_DIRECT = 1, ENGINE_LDS = 2, ENGINE_RING = 3, ENGINE_MID = 4 };

struct Config {
    int engine;   // ENGINE_DIRECT: global -> VGPR -> MFMA;  ENGINE_LDS: global -> LDS ring (DMA) -> MFMA
    int mt;       // 16-row activation blocks per tile (1 or 2)
    int rg;       // 16-row weight tiles per wave
    int ku;       // direct engine: 64-byte K chunks per stage (the LDS engine's stage is 256 bytes);
                  // mid-batch engine: ring slots of the activations (0 = depth)
    int depth;    // stages in flight per wave
    int waves;    // waves per workgroup, splitting K among themselves
    int split_k;  // workgroups per tile, splitting K among themselves
    int nt;       // weights loaded with the non-temporal hint
    int persist;  // LDS engine: 0 = one workgroup per tile; n > 0 = n persistent workgroups per CU walking the tiles
    const Workspace* fixed_ws = nullptr;   // split-K partials and counters to use instead of the stream's own workspace
    int wavetile; // LDS engine, bits 0-1: 1 = every wave owns whole tiles, activations resident in LDS (persist = workgroups per CU);
                  //             2 = persistent K-split workgroups with the activations resident in LDS
                  //             3 = ... resident in the waves' registers (k = 256 * waves * {1, 2, 4});  bit 2: epilogue wave
};

// Split-K partials (fp32) and arrival counters for `tiles` output tiles of per_tile_bytes each: the caller's
// fixed workspace if the configuration names one, the launch stream's own otherwise.
static int attach_workspace(const Config& c, StreamArgs& a, size_t tiles, size_t per_tile_bytes, hipStream_t stream) {
    a.ws = nullptr;
    a.counters = nullptr;
    if (c.split_k <= 1) return SG_SUCCESS;
    const size_t need = tiles * c.split_k * per_tile_bytes;
    Workspace w;
    if (c.fixed_ws) {
        w = *c.fixed_ws;
        if (tiles > w.n_counters || need > w.partial_bytes) return SG_WORKSPACE_TOO_SMALL;
    } else if (int rc = get_workspace(stream, need, tiles, &w)) {
        return rc;
    }
    a.ws = w.partials;
    a.counters = w.counters;
    return SG_SUCCESS;
}

static int prepare(const Config& c, StreamArgs& a, int stage_bytes_k, size_t* tiles_out, hipStream_t stream, int tile_rows = 0) {
    const int frags = c.rg * c.mt;
    if (c.waves < 1 || c.waves > 16 || c.depth < 1 || c.rg < 1 || c.mt < 1 || stage_bytes_k < 16) return SG_INVALID_CONFIG;
    if (tile_rows <= 0) tile_rows = 16 * c.rg;
    a.waves = c.waves;
    a.split_k = c.split_k;
    a.n_tiles = (a.n + tile_rows - 1) / tile_rows;
    a.m_tiles = (a.m + 16 * c.mt - 1) / (16 * c.mt);
    const int total_stages = a.k / stage_bytes_k > 0 ? a.k / stage_bytes_k : 1;
    if (c.split_k < 1 || c.split_k > total_stages) return SG_INVALID_CONFIG;
    const size_t tiles = (size_t)a.n_tiles * a.m_tiles;
    if (tiles * c.split_k > 0x7fffffffu) return SG_BAD_ARGUMENT;
    if (int rc = attach_workspace(c, a, tiles, (size_t)frags * 1024, stream)) return rc;
    set_reciprocals(a);
    *tiles_out = tiles;
    return SG_SUCCESS;
}

static int launch_stream(const Config& c, StreamArgs a, hipStream_t stream) {
    size_t tiles;
    if (int rc = prepare(c, a, c.ku * 64, &tiles, stream)) return rc;
    const size_t lds = c.waves > 1 ? (size_t)c.waves * c.rg * c.mt * 1024 : 0;
    if (lds > 64 * 1024) return SG_INVALID_CONFIG;
    const unsigned grid = (unsigned)(tiles * c.split_k);
    const unsigned threads = (unsigned)c.waves * 64;
#define SG_GO(MT, RG) \
    if (c.mt == MT && c.rg == RG) return SG_STREAM_LAUNCHER(MT, RG)(c.ku, c.depth, a, grid, threads, lds, stream);
    SG_GO(1, 1) SG_GO(1, 2) SG_GO(1, 3) SG_GO(1, 4) SG_GO(2, 1) SG_GO(2, 2) SG_GO(2, 3) SG_GO(2, 4)
#undef SG_GO
    return SG_INVALID_CONFIG;
}

// Persistent workgroups for `tiles` tiles when at most `most` fit the device: the launch lasts as long as the
// workgroup with the most tiles, ceil(tiles / most) of them, so no more workgroups are started than it takes to give
// every one that many (896 tiles on 256 CUs: 224 workgroups of 4 instead of 128 of 4 and 128 of 3 - the same
// critical path with fewer streams competing for memory, 8 x 14336 x 4096 12.35 -> 11.54 us).
static unsigned level_persistent_grid(unsigned tiles, size_t most) {
    if (most >= tiles) return tiles;
    const size_t rounds = (tiles + most - 1) / most;
    return (unsigned)((tiles + rounds - 1) / rounds);
}

// Any k beyond 256 (a multiple of 16, like every k the library takes) also runs on the per-tile ring and on the
// wave-per-tile kernel: the last block is loaded from k - 256 and partly used (the K-split persistent kernels take
// multiples of 256 only).
static bool lds_half_block_k(int k) { return k % 256 != 0 && k % 16 == 0 && k > 256; }

static int launch_lds(const Config& c, StreamArgs a, hipStream_t stream) {
    if (a.k % 256 != 0 && !(lds_half_block_k(a.k) && !a.A16 && ((c.persist == 0 && (c.wavetile & 7) == 0) || c.wavetile == 1)))
        return SG_K_NOT_DIVISIBLE_BY_WARPTILE_K;
    // wave_tiles bit 3: 24-row tiles (two fragments, the second half used), one workgroup per tile
    const bool rows24 = (c.wavetile & 8) != 0;
    if (rows24 && (c.rg != 2 || c.persist != 0 || (c.wavetile & 7) != 0)) return SG_INVALID_CONFIG;
    size_t tiles;
    if (int rc = prepare(c, a, 256, &tiles, stream, rows24 ? 24 : 0)) return rc;
    // activation DMA instructions per stage: 4 rows each, rounded up to a compiled count
    int xu = 8;
    if (c.mt == 1) {
        const int need = (a.m + 3) / 4;
        xu = need <= 1 ? 1 : (need <= 2 ? 2 : 4);
    }
    const size_t stage = (size_t)((rows24 ? 6 : c.rg * 4) + xu) * 1024;
    // + 4 KB: lanes of activation rows that are not loaded read past the last slot
    size_t lds = (size_t)c.waves * c.depth * stage + 4096;
    unsigned grid = (unsigned)(tiles * c.split_k);
    int mode = rows24 ? 5 : 0, extra_wave = 0;
    if (a.A16 && !(c.persist > 0 && (c.wavetile & 3) == 2)) return SG_INVALID_CONFIG;
    if (c.wavetile == 1) {
        // whole activation matrix resident: one tile row of activations only, no K split
        if (c.split_k != 1 || a.m_tiles != 1 || c.persist < 1) return SG_INVALID_CONFIG;
        mode = 2;
        lds = (size_t)((a.k + 255) / 256) * xu * 1024 + (size_t)c.waves * c.depth * c.rg * 4096 + 4096;
        DeviceInfo* dev;
        if (int rc = get_device_info(&dev)) return rc;
        size_t want = (size_t)dev->cu_count * c.persist;
        if (want > tiles) want = tiles;
        grid = (unsigned)want;
    } else if (c.persist > 0 && (c.wavetile & 3) == 3) {
        // activations resident in registers: every wave keeps the fragments of its own K blocks
        if (c.split_k != 1 || a.m_tiles != 1) return SG_INVALID_CONFIG;
        const int blocks = a.k / 256;
        if (blocks % c.waves != 0) return SG_INVALID_CONFIG;
        const int pt = blocks / c.waves;
        if (pt * c.mt > 4) return SG_INVALID_CONFIG;
        DeviceInfo* dev;
        if (int rc = get_device_info(&dev)) return rc;
        grid = level_persistent_grid(grid, (size_t)dev->cu_count * c.persist);
        const unsigned threads = (unsigned)(c.waves + ((c.wavetile & 4) ? 1 : 0)) * 64;
        if (threads > 1024) return SG_TOO_MANY_WARPS;
        size_t lds_x = (size_t)c.waves * c.depth * c.rg * 4096 + 2u * c.waves * c.rg * c.mt * 1024;
        if (lds_x > 159 * 1024) return SG_INVALID_CONFIG;
        // room for one more 4 KB staging block per wave (the kernel has no static LDS: all 160 KB may be asked for):
        // the activation fragments then reach the registers without the first weight stages being waited for
        a.x_extra = (c.mt == 2 && pt == 2 && lds_x + (size_t)c.waves * 4096 <= 160 * 1024) ? 1 : 0;
        if (a.x_extra) lds_x += (size_t)c.waves * 4096;
        a.stamps = take_stamps(grid);
        return launch_xreg(c.mt, c.rg, pt, c.depth, a, grid, threads, lds_x, stream);
    } else if (c.persist > 0) {
        if (c.split_k != 1) return SG_INVALID_CONFIG;
        mode = 1;
        if (c.wavetile & 4) extra_wave = 1;   // dedicated epilogue wave
        if ((c.wavetile & 3) == 2) {   // activations resident: stages hold weights only
            if (a.m_tiles != 1) return SG_INVALID_CONFIG;
            mode = 3;
            lds = (size_t)(a.k / 256) * xu * 1024 + (size_t)c.waves * c.depth * c.rg * 4096 + 4096;
        }
        lds += 2u * c.waves * c.rg * c.mt * 1024;   // double-buffered reduction scratch
        DeviceInfo* dev;
        if (int rc = get_device_info(&dev)) return rc;
        grid = level_persistent_grid(grid, (size_t)dev->cu_count * c.persist);
    }
    if (lds > 159 * 1024) return SG_INVALID_CONFIG;  // 160 KB per CU, minus the kernel's static LDS
    if (a.A16) {   // only the resident-activation kernel quantises bf16 activations itself
        if (mode != 3) return SG_INVALID_CONFIG;
        mode = 4;
    }
    const unsigned threads = (unsigned)(c.waves + extra_wave) * 64;
    if (threads > 1024) return SG_TOO_MANY_WARPS;
    if (mode != 2) a.stamps = take_stamps(grid);
#define SG_GO(MT, RG)                                                                                          \
    if (c.mt == MT && c.rg == RG)                                                                              \
        return SG_LDS_LAUNCHER(MT, RG)(xu, c.depth, c.nt, mode, a, grid, threads, lds, stream);
    SG_GO(1, 1) SG_GO(1, 2) SG_GO(1, 4) SG_GO(2, 1) SG_GO(2, 2) SG_GO(2, 4)
#undef SG_GO
    return SG_INVALID_CONFIG;
}

// Producer/consumer ring: a_producers + b_producers + consumers waves per persistent workgroup.
struct RingConfig {
    int mt, b_lanes, qsize, a_producers, b_producers, consumers, nt;
    int split_k = 1;                       // work items per output tile, splitting K among themselves
    const Workspace* fixed_ws = nullptr;   // split-K partials and counters to use instead of the stream's own workspace
};

static int launch_ring(const RingConfig& c, StreamArgs a, hipStream_t stream) {
    if (a.k % 256 != 0) return SG_K_NOT_DIVISIBLE_BY_WARPTILE_K;
    if (c.a_producers < 1 || c.b_producers < 1 || c.consumers < 1 || c.qsize < 1) return SG_INVALID_CONFIG;
    if (c.a_producers + c.b_producers + c.consumers > 16) return SG_TOO_MANY_WARPS;
    if (c.b_lanes < 1 || c.b_lanes > 6 || (c.mt != 1 && c.mt != 2)) return SG_INVALID_CONFIG;
    if (c.split_k < 1 || c.split_k > a.k / 256) return SG_INVALID_CONFIG;
    a.waves = c.consumers;
    a.split_k = c.split_k;
    a.n_tiles = (a.n + 16 * c.b_lanes - 1) / (16 * c.b_lanes);
    a.m_tiles = (a.m + 16 * c.mt - 1) / (16 * c.mt);
    a.ws = nullptr;
    a.counters = nullptr;
    set_reciprocals(a);
    const size_t tiles = (size_t)a.n_tiles * a.m_tiles * c.split_k;   // work items: one K split of one output tile
    if (tiles > 0x7fffffffu) return SG_BAD_ARGUMENT;
    if (c.split_k > 1) {
        // fp32 partials [tile][split][fragment][256] and one arrival counter per fragment of every tile
        const size_t frags = (size_t)c.b_lanes * c.mt, out_tiles = (size_t)a.n_tiles * a.m_tiles;
        Workspace w;
        if (c.fixed_ws) {
            w = *c.fixed_ws;
            if (out_tiles * frags > w.n_counters || tiles * frags * 1024 > w.partial_bytes) return SG_WORKSPACE_TOO_SMALL;
        } else if (int rc = get_workspace(stream, tiles * frags * 1024, out_tiles * frags, &w)) {
            return rc;
        }
        a.ws = w.partials;
        a.counters = w.counters;
    }
    int xu = 8;
    if (c.mt == 1) {
        const int need = (a.m + 3) / 4;
        xu = need <= 1 ? 1 : (need <= 2 ? 2 : 4);
    }
    const size_t slot = (size_t)(c.b_lanes * 4 + xu) * 1024;
    const size_t flags = ((size_t)(2 * c.b_lanes * c.qsize + 2) * sizeof(int) + 1023) & ~(size_t)1023;
    // ring | double-buffered reduction scratch | flags | 4 KB slack for activation rows that are not loaded
    const size_t lds = (size_t)c.qsize * slot + 2u * c.b_lanes * c.mt * c.consumers * 1024 + flags + 4096;
    if (lds > 159 * 1024) return SG_INVALID_CONFIG;
    DeviceInfo* dev;
    if (int rc = get_device_info(&dev)) return rc;
    size_t per_cu = (159 * 1024) / lds;
    if (per_cu < 1) per_cu = 1;
    if (per_cu > 4) per_cu = 4;
    size_t grid = (size_t)dev->cu_count * per_cu;
    if (grid > tiles) grid = tiles;
    RingArgs ra;
    ra.g = a;
    ra.a_producers = c.a_producers;
    ra.b_producers = c.b_producers;
    ra.consumers = c.consumers;
    ra.qsize = c.qsize;
    const unsigned threads = (unsigned)(c.a_producers + c.b_producers + c.consumers) * 64;
    if (c.mt == 1) return SG_RING_LAUNCHER(1)(c.b_lanes, xu, c.nt, ra, (unsigned)grid, threads, lds, stream);
    return SG_RING_LAUNCHER(2)(c.b_lanes, xu, c.nt, ra, (unsigned)grid, threads, lds, stream);
}

// Mid-batch engine: c.rg = 16-row weight fragments per wave (2 or 4), c.mt = 16-row activation
// fragments per wave (2, 4 or 8); a workgroup tile is 16*c.rg*(waves/2) weight rows x 32*c.mt activation rows.
// The mid-batch kernel's stage is 128 bytes of K; a k beyond 128 that is only a multiple of 16 runs in the builds with a
// partial last block, which exist for the tiles and rings pick_mid chooses.
static bool mid_partial_block_k(int k) { return k % 128 != 0 && k % 16 == 0 && k > 128; }

static int launch_mid_engine(const Config& c, StreamArgs a, hipStream_t stream) {
    if (a.k % 128 != 0 && !mid_partial_block_k(a.k)) return SG_K_NOT_DIVISIBLE_BY_WARPTILE_K;
    if ((c.rg != 2 && c.rg != 4) || (c.mt != 2 && c.mt != 4 && c.mt != 8) || c.depth < 2) return SG_INVALID_CONFIG;
    if (c.waves != 4 && c.waves != 8 && c.waves != 14) return SG_INVALID_CONFIG;
    const int wn = c.waves / 2;                   // waves = wn (along n) x 2 (along m)
    const int bn = 16 * c.rg * wn, bm = 32 * c.mt;
    // stage rows split evenly over the waves' 8-row DMA instructions (fourteen waves: the kernel gives the
    // activation rows to the first eight)
    if (bn % (16 * wn) != 0 || (wn != 7 && bm % (16 * wn) != 0)) return SG_INVALID_CONFIG;
    a.waves = c.waves;
    a.split_k = c.split_k;
    a.n_tiles = (a.n + bn - 1) / bn;
    a.m_tiles = (a.m + bm - 1) / bm;
    const int blocks = a.k / 128;
    if (c.split_k < 1 || c.split_k > blocks) return SG_INVALID_CONFIG;
    const size_t tiles = (size_t)a.n_tiles * a.m_tiles;
    if (tiles * c.split_k > 0x7fffffffu) return SG_BAD_ARGUMENT;
    // fp32 fragments of one workgroup tile
    if (int rc = attach_workspace(c, a, tiles, (size_t)c.waves * c.rg * c.mt * 1024, stream)) return rc;
    set_reciprocals(a);
    // c.ku: ring slots of the activations (0 or out of range = as many as the weights')
    const int dx = (c.ku >= 2 && c.ku < c.depth) ? c.ku : c.depth;
    // c.wavetile = 1: the split-K partials are summed by a second launch over the whole device instead of by the last
    // workgroup of every tile to arrive (no arrival word in LDS, no counters touched)
    if (c.wavetile != 0 && c.wavetile != 1) return SG_INVALID_CONFIG;
    a.defer_reduce = (c.wavetile == 1 && c.split_k > 1) ? 1 : 0;
    const size_t lds = ((size_t)c.depth * bn + (size_t)dx * bm) * 128 + ((c.split_k > 1 && !a.defer_reduce) ? 16 : 0);
    if (lds > 160 * 1024) return SG_INVALID_CONFIG;
    a.stamps = take_stamps((unsigned)(tiles * c.split_k));
    if (int rc = launch_mid(c.rg, c.mt, c.depth, dx, wn, a, (unsigned)(tiles * c.split_k), lds, stream)) return rc;
    return a.defer_reduce ? launch_mid_reduce(c.rg, c.mt, wn, a, stream) : SG_SUCCESS;
}

// Microseconds of a mid-batch launch of bn x bm tiles with K split sk ways, from what the ingest probe measured
// (sg_debug_cu_ingest) rather than from named shapes: a CU takes in operand bytes - L2 misses and hits in turn - at
// about 55 GB/s with this kernel's mix, the chip serves misses at 6.9 TB/s, the matrix cores sustain about
// 2 PFLOP/s on real data, and a split adds its partials to every workgroup's stores (27 GB/s per CU), a second launch
// (4 us) and the partials once more as that launch's reads.
static double mid_model_us(int m, int n, int k, int bn, int bm, int sk, int cu_count) {
    const double n_tiles = (n + bn - 1) / bn, m_tiles = (m + bm - 1) / bm;
    const double wgs = n_tiles * m_tiles * sk;
    const double rounds = (double)(((long)wgs + cu_count - 1) / cu_count);
    const double per_wg = (double)(bn + bm) * k / sk / 55e9 + (sk > 1 ? (double)bn * bm * 4 / 27e9 : 0.0);
    const double hbm = (n_tiles * bn + 8 * m_tiles * bm) * k / 6.9e12;
    const double mfma = 2.0 * n_tiles * bn * m_tiles * bm * k / 2.0e15;
    double t = rounds * per_wg;
    if (hbm > t) t = hbm;
    if (mfma > t) t = mfma;
    t += 3.5e-6;
    if (sk > 1) t += 4.0e-6 + sk * m_tiles * bm * n_tiles * bn * 4 / 6.9e12;
    return t * 1e6;
}

// Mid-batch heuristic, fitted to timings of the Llama-3-70B projection shapes at M = 64..256:
// what matters first is that one round of workgroups covers the device (a second, partly
// filled round costs more than any tile-shape effect), then that the round is as full as
// possible, then the tile: 128x128 and 128x64 tiles on eight waves beat both smaller tiles
// (more operand traffic per flop) and 256-wide ones (one workgroup per CU and a two-slot ring),
// which only pay off when nothing else fits in one round.  K may be split up to four ways as
// long as every split keeps 32 K blocks (three ways: 16, for m <= 64).
static Config pick_mid(int m, int n, int k, int cu_count) {
    struct Tile { int bn, bm, waves; };
    // {224, *, 14}: fourteen waves; 57344 = 256 x 224 gives every CU a tile where 256-row tiles fill 224 of 256
    // (5-10 % at M = 128 and 256 on N(0,1)-quantised operands, 4 % at M = 64 over two co-resident 128 x 64 tiles)
    // The 64 x 128 tile on four waves only where it covers all of m and K is beyond 4096 - up to 96 rows at any such K
    // that is not a power of two (with rows 8192 bytes apart the eight-wave tile is 3-5 % ahead: 72 x 12288 x 8192 30.5
    // against 31.8), at 97..128 rows below K = 8192 (stacked - 129..192 or more than 256 rows on a narrow weight matrix, where its padded
    // rows look like a fuller round - 128 x 64 on eight waves measured 6-12 % faster, ten shapes; at K = 8192 and more
    // and 96..128 rows 2-8 % faster, nine shapes).
    static const Tile order[] = {{128, 128, 8}, {128, 64, 8}, {64, 64, 4}, {64, 128, 4}, {256, 128, 8}, {224, 128, 14},
                                 {256, 64, 8}, {224, 64, 14}, {128, 256, 8}, {256, 256, 8}, {224, 256, 14}};
    const int bm_max = m <= 64 ? 64 : (m <= 128 ? 128 : 256);
    const int blocks = (k + 127) / 128;
    Config best;
    long best_rounds = -1, best_wgs = 0;
    const Tile* best_tile = nullptr;
    for (const Tile& t : order) {
        if (t.bm > bm_max) continue;
        const bool tall4 = t.bn == 64 && t.bm == 128;
        if (tall4 && (m > 128 || blocks <= 32 || (blocks >= 64 && (m > 96 || (k & (k - 1)) == 0)))) continue;
        const long m_tiles = (m + t.bm - 1) / t.bm;
        const long tiles = (long)((n + t.bn - 1) / t.bn) * m_tiles;
        for (int sk = 1; sk <= 4; sk++) {
            // a three-way split only up to 64 activation rows, where the partials are small against the weights
            // (64 x 10240 x 8192: 80 tiles -> 240 workgroups, 24.5 -> 22.5 us); two and four ways keep 32 K blocks
            if (sk == 3 ? (m > 64 || blocks / sk < 16) : (sk > 1 && blocks / sk < 32)) continue;
            // the fp32 partials of a split are written and read back: no split whose partials (padded rows x 4 bytes x
            // splits per weight row) exceed a third of the weight row's k bytes (320 x 8192 x 8192: 256-row tiles split
            // in two 51.9 us, 128-row tiles unsplit 39.3)
            if (sk > 1 && m_tiles * t.bm * 4 * sk * 3 > k) continue;
            const long wgs = tiles * sk;
            const long rounds = (wgs + cu_count - 1) / cu_count;
            // the fourteen-wave tile only where it is known to pay: unsplit, filling at least 70 % of its rounds, and all
            // of m in one tile or tiles of at least 128 rows (the weights streamed at most a few times: 144..256 x 28672 x
            // 4096 on two 224 x 128 tiles 3-4 % ahead of 256 x 128, 320 and 448 rows on 224 x 256 11-15 % ahead of
            // 256 x 256; 448 x 13824 x 5120, 62 tiles x 4, 52.3 -> 47.4)
            if (t.waves == 14 && (sk > 1 || (m > t.bm && t.bm < 128) || wgs * 10 < rounds * cu_count * 7)) continue;
            bool better = best_rounds < 0 || rounds < best_rounds ||
                          (rounds == best_rounds && wgs * 16 > best_wgs * 17) ||   // clearly fuller round
                          // as full with less splitting, when the splits had become short
                          (rounds == best_rounds && wgs == best_wgs && sk < best.split_k &&
                           blocks / best.split_k < 40);
            if (best_rounds >= 0 && rounds == best_rounds && blocks < 80 && m > 64) {
                // above 64 rows and below K = 10240 an unsplit launch that fills 70 % of its rounds beats a split one
                // that fills them all (144 x 8192 x 8192: 192 workgroups unsplit 29.1 us, 256 split in two 31.7);
                // with a longer K the split wins (448 x 4096 x 14336: 46.2 against 50.4, 200 x 6144 x 11008: 37.9 against 42.9)
                if (sk == 1 && best.split_k > 1 && wgs * 10 >= rounds * cu_count * 7) better = true;
                if (sk > 1 && best.split_k == 1 && best_wgs * 10 >= rounds * cu_count * 7) better = false;
            }
            // 65..128 rows, K beyond 4096 (from 97 rows on: below 8192): against 128 x 64 on eight waves and two activation tiles, one 64 x 128 tile
            // over all of m on four waves - as many workgroups, the weights pass each CU once (72 x 13824 x 5120
            // 29.6 -> 23.5 us, 100 rows 28.6 -> 26.1, 72 x 14336 x 5120 28.3 -> 23.7, 72 x 12288 x 5120 28.0 -> 23.0,
            // 72 x 16384 x 11008 59.5 -> 44.1, 72 x 16384 x 14336 73.1 -> 54.1, 72 x 12288 x 10240 52.0 -> 42.4; level at
            // K = 4096 - the second 64-row activation tile of a 72-row problem re-reads all weights for 8 rows)
            if (tall4 && sk == 1 && rounds == best_rounds && best_tile && best_tile->bn == 128 && best_tile->bm == 64 &&
                best.split_k == 1 && wgs * 16 >= best_wgs * 15)
                better = true;
            if (!better) continue;
            best_rounds = rounds;
            best_wgs = wgs;
            best_tile = &t;
            best.waves = t.waves;
            best.rg = t.bn / (t.waves * 8);      // 16-row tiles per wave: bn = 16 * rg * (waves / 2)
            best.mt = t.bm / 32;
            best.split_k = sk;
        }
    }
    Config c = best;
    // Second opinion of the cost model: a K split over tiles of 128 or 256 weight rows (its sum in a second launch) where
    // the model puts it at least 8 % ahead of the choice above.  On 72 shapes (64..256 rows x twelve weight shapes) every
    // override the margin lets through measured level or faster (-27 % ... +0 %: 128 x 5120 x 13824 32.1 -> 23.6 us,
    // 96 x 9216 x 8192 29.1 -> 23.8, 256 x 8192 x 28672 86.6 -> 77.5), and every choice the model would have made worse
    // (+4 ... +15 %, all of them ties or within 5 % in the model) stays with the rules.
    if (k % 128 == 0 && c.waves != 14) {
        struct Alt { int waves, rg, mt; };
        static const Alt alts[] = {{4, 2, 2}, {4, 4, 4}, {8, 2, 2}, {8, 2, 4}, {8, 4, 2}, {8, 4, 4}, {8, 2, 8}, {8, 4, 8}};
        const double own = mid_model_us(m, n, k, 8 * c.rg * c.waves, 32 * c.mt, c.split_k, cu_count);
        double alt_us = own;
        for (const Alt& t : alts) {
            if (32 * t.mt >= 2 * m && t.mt > 2) continue;   // tile more than twice as tall as the problem
            for (int sk = 2; sk <= 8 && blocks / sk >= 16; sk++) {
                const double us = mid_model_us(m, n, k, 8 * t.rg * t.waves, 32 * t.mt, sk, cu_count);
                if (us < alt_us && us <= 0.92 * own) {
                    alt_us = us;
                    c.waves = t.waves; c.rg = t.rg; c.mt = t.mt; c.split_k = sk;
                }
            }
        }
    }
    bool co_resident = false;
    if (m <= 64 && c.waves != 14 && (long)((n + 127) / 128) * 2 >= 3L * cu_count) {
        // memory-bound and many tiles: several small two-slot workgroups per CU hide the DMA
        // latency better than one deep ring
        c.waves = 8; c.rg = 2; c.mt = 2; c.split_k = 1;
        co_resident = true;
    }
    c.engine = ENGINE_MID;
    c.nt = 1;
    c.persist = 0;
    // a K split leaves its sum to a second launch over the whole device: level or ahead of the last workgroup's serial
    // sum on every split record of the Llama-3-70B shapes (128 x 128 tiles split three ways at 128 x 10240 x 8192
    // 32.1 -> 26.6 us, 128 x 64 split four ways at 64 x 8192 x 28672 46.8 -> 43.6, 64 x 64 split in two 19.1 -> 18.5)
    c.wavetile = c.split_k > 1 ? 1 : 0;
    const int bn = 8 * c.rg * c.waves, bm = 32 * c.mt;
    const int per_wave_w = bn / (8 * c.waves), per_wave_x = bm / (8 * c.waves);   // DMA instructions per wave and stage
    // (weight slots, activation slots; 0 = as many): the deepest ring that fits 160 KB.  A shallower
    // activation ring (activations come from L2, weights from HBM) is what lets the 256 x 256 tile keep
    // two weight stages in flight, and the 224 x 128 tile three (86 -> 80 us at 128 x 57344 x 8192).
    static const int rings[][2] = {{4, 0}, {4, 3}, {3, 0}, {3, 2}, {2, 0}};
    c.depth = 2;
    c.ku = 0;
    if (co_resident) {
        c.depth = 4;
        c.ku = 2;
    } else {
        for (const auto& r : rings) {
            const int dw = r[0], dx = r[1] ? r[1] : r[0];
            if (dw == 4 && dx == 3 && c.waves != 14) continue;   // compiled for the 224 x 128 tile, which it fills to 160 KB
            const int in_flight_x = per_wave_w + (dx - 2) * (per_wave_w + per_wave_x);
            const int in_flight_w = (dw - 2) * (per_wave_w + per_wave_x);
            const size_t lds = ((size_t)dw * bn + (size_t)dx * bm) * 128;   // (a split's sum is a second launch: no arrival word)
            if (lds > 160 * 1024) continue;
            if ((in_flight_x < in_flight_w ? in_flight_x : in_flight_w) > 63) continue;
            c.depth = dw;
            c.ku = r[1];
            break;
        }
    }
    return c;
}

// K the 2:4 kernels take: whole 128-k pieces (one lane's share of a 512-k stage; keeps the rows of all three streams
// 16-byte aligned), at least one whole stage.
static bool sparse_k_ok(int k) { return k >= 512 && k % 128 == 0; }

// 2:4 sparse engine: c.rg row tiles per wave, c.waves waves splitting K, c.depth ring slots.
static int launch_sparse_engine(const Config& c, StreamArgs a, const uint8_t* meta, hipStream_t stream) {
    if (!sparse_k_ok(a.k)) return SG_K_NOT_DIVISIBLE_BY_WARPTILE_K;
    const int blocks = (a.k + 511) / 512;   // 512-k stages, the last one partly used when 512 does not divide k
    size_t tiles;
    if (int rc = prepare(c, a, 512, &tiles, stream)) return rc;
    int xu2 = 16;
    if (c.mt == 1) {
        const int need = (a.m + 3) / 4;
        xu2 = need <= 1 ? 2 : (need <= 2 ? 4 : 8);
    }
    SparseArgs sa;
    sa.meta = meta;
    // Metadata by whole 128-byte lines (two stages' worth per row and request) where K is a multiple of 1024, every K
    // split holds whole pairs of stages and the pair ring still fits the LDS; by 64-byte pieces per stage otherwise, or
    // when the record asks for that (k_chunks = 1).
    const size_t pair_ring = (size_t)(c.depth / 2 + 2) * c.rg * 2048;   // per wave, in place of depth x rg KB
    bool pairs = c.ku != 1 && a.k % 1024 == 0 && c.split_k <= a.k / 1024;
    if (c.wavetile == 1) {
        // every wave owns whole tiles, the activation matrix is resident in LDS: one activation tile of at most 16
        // rows, no K split, c.persist workgroups per CU at most
        if (c.mt != 1 || a.m_tiles != 1 || c.split_k != 1 || c.persist < 1 || (c.rg != 1 && c.rg != 2)) return SG_INVALID_CONFIG;
        if (c.waves * 64 > 1024) return SG_TOO_MANY_WARPS;
        size_t lds_wt = (size_t)blocks * xu2 * 1024 + (size_t)c.waves * c.depth * c.rg * 5120 + 8192;
        if (lds_wt > 159 * 1024) return SG_INVALID_CONFIG;
        const size_t lds_pairs = (size_t)blocks * xu2 * 1024 + (size_t)c.waves * (c.depth * c.rg * 4096 + pair_ring) + 8192;
        pairs = pairs && lds_pairs <= 159 * 1024;
        if (pairs) lds_wt = lds_pairs;
        DeviceInfo* dev;
        if (int rc = get_device_info(&dev)) return rc;
        size_t grid = (size_t)dev->cu_count * c.persist;
        if (grid > tiles) grid = tiles;
        a.stamps = take_stamps((unsigned)grid);
        sa.g = a;
        return launch_sparse_wavetile(c.rg, xu2, c.depth, pairs, sa, (unsigned)grid, (unsigned)c.waves * 64, lds_wt, stream);
    }
    const size_t stage = (size_t)(c.rg * 5 + xu2) * 1024;
    // + 8 KB: lanes of activation rows that are not loaded read past the last slot
    size_t lds = (size_t)c.waves * c.depth * stage + 8192;
    if (lds > 159 * 1024) return SG_INVALID_CONFIG;
    const size_t lds_pairs = (size_t)c.waves * (c.depth * (stage - (size_t)c.rg * 1024) + pair_ring) + 8192;
    pairs = pairs && lds_pairs <= 159 * 1024;
    if (pairs) lds = lds_pairs;
    a.stamps = take_stamps((unsigned)(tiles * c.split_k));
    sa.g = a;
    return launch_sparse(c.mt, c.rg, xu2, c.depth, pairs, sa, (unsigned)(tiles * c.split_k), (unsigned)c.waves * 64, lds, stream);
}

static Config pick_sparse(int m, int n, int k, int cu_count) {
    Config c;
    c.engine = ENGINE_LDS;
    c.nt = 1;
    c.persist = 0;
    c.wavetile = 0;
    c.ku = 8;
    c.split_k = 1;
    c.mt = m <= 16 ? 1 : 2;
    const int tiles16 = (n + 15) / 16;
    const int blocks = (k + 511) / 512;
    // above 8 activation rows the activation stage outweighs a 16-row weight stage: share it between two row tiles
    c.rg = (tiles16 >= 4 * cu_count || (m > 8 && tiles16 >= 2 * cu_count)) ? 2 : 1;
    c.waves = blocks >= 16 ? 2 : 1;
    // many tiles per CU: shallow rings so that several workgroups share a CU
    c.depth = (c.rg == 2 || tiles16 / c.rg >= 2 * cu_count) ? 2 : 4;
    const int xu2 = c.mt == 2 ? 16 : ((m + 3) / 4 <= 1 ? 2 : ((m + 3) / 4 <= 2 ? 4 : 8));
    while (c.depth > 2 && ((c.depth - 1) * (c.rg * 5 + xu2) > 63 ||
                           (size_t)c.waves * c.depth * (c.rg * 5 + xu2) * 1024 + 8192 > 159 * 1024))
        c.depth--;
    if (c.mt == 1 && m > 4 && tiles16 * 4 >= cu_count * 5) {
        // 5..16 activation rows and more than one tile per CU: the activation matrix stays resident in LDS and
        // four waves per CU each stream whole tiles (4-33 % faster on ten shapes than refetching 4-8 KB of
        // activations with every 5 KB weight stage; at four rows and below the two are level)
        // (a K of whole 1024s gets its metadata by lines, which takes a pair ring next to the stages: at 9..16 rows and
        // K = 4096 three slots with it rather than four without - level to 2 % ahead on 16 x 14336 x 4096)
        const size_t x_res = (size_t)blocks * xu2 * 1024;
        for (int depth = 4; depth >= 2; depth--) {
            const size_t wave_bytes = k % 1024 == 0 ? (size_t)depth * 4096 + (size_t)(depth / 2 + 2) * 2048 : (size_t)depth * 5120;
            if (x_res + 4 * wave_bytes + 8192 > 159 * 1024) continue;
            c.rg = 1;
            c.waves = 4;
            c.depth = depth;
            c.persist = 1;
            c.wavetile = 1;
            break;
        }
    }
    // Metadata by whole lines (launch_sparse_engine) costs a wave 4 KB of LDS more: with one-wave workgroups on
    // two-slot rings that is one workgroup less per CU, and up to 4 activation rows it does not pay (1 x 14336 x 4096
    // 7.85 -> 7.83-8.0 us, where 32 x 14336 x 4096 on the same ring goes 12.3 -> 11.9 and 16 x 4096 x 14336 10.6 -> 10.1)
    if (m <= 4 && c.depth == 2 && c.waves == 1) c.ku = 1;
    return c;
}

// Split-K partial bytes and arrival counters the launch of `c` on an m x n x k problem takes from its workspace
// (zero without a K split): the arithmetic of prepare() / launch_mid_engine() without the launch.
static void workspace_need(const Config& c, int m, int n, size_t* partial_bytes, size_t* counters) {
    *partial_bytes = 0;
    *counters = 0;
    if (c.split_k <= 1) return;
    size_t tiles, per_tile;
    if (c.engine == ENGINE_MID) {
        const int wn = c.waves / 2;
        const int bn = 16 * c.rg * (wn > 0 ? wn : 1), bm = 32 * c.mt;
        tiles = (size_t)((n + bn - 1) / bn) * ((m + bm - 1) / bm);
        per_tile = (size_t)c.waves * c.rg * c.mt * 1024;
    } else {
        const int tile_rows = (c.engine == ENGINE_LDS && (c.wavetile & 8)) ? 24 : 16 * c.rg;
        tiles = (size_t)((n + tile_rows - 1) / tile_rows) * ((m + 16 * c.mt - 1) / (16 * c.mt));
        per_tile = (size_t)c.rg * c.mt * 1024;
    }
    *partial_bytes = tiles * c.split_k * per_tile;
    *counters = tiles;
}

static int launch_config(const Config& c, const StreamArgs& a, hipStream_t stream) {
    if (c.engine == ENGINE_DIRECT) return launch_stream(c, a, stream);
    if (c.engine == ENGINE_LDS) return launch_lds(c, a, stream);
    if (c.engine == ENGINE_MID) return launch_mid_engine(c, a, stream);
    return SG_INVALID_CONFIG;
}

static int check_pointers(const void* A, const void* B, const void* D, int m, int n, int k, int b_stride) {
    if (!A || !B || !D || m <= 0 || n <= 0 || k <= 0 || b_stride < k) return SG_BAD_ARGUMENT;
    if ((reinterpret_cast<uintptr_t>(A) | reinterpret_cast<uintptr_t>(B)) & 15u) return SG_BAD_ALIGNMENT;
    if ((reinterpret_cast<uintptr_t>(D) & 7u) || (b_stride & 15)) return SG_BAD_ALIGNMENT;
    // the kernels address a tile's rows with 32-bit offsets from the tile's first row: 64 rows must stay below 2 GB
    if ((size_t)b_stride * 64 > 0x7fffffffu || (size_t)k * 64 > 0x7fffffffu) return SG_BAD_ARGUMENT;
    return SG_SUCCESS;
}

// Register-streaming engine: any k that is a multiple of 16.
static Config direct_config(int m, int n, int k, int cu_count) {
    Config c;
    c.mt = m <= 16 ? 1 : 2;
    c.nt = 1;
    c.split_k = 1;
    c.persist = 0;
    c.wavetile = 0;
    const int tiles16 = (n + 15) / 16;
    c.engine = ENGINE_DIRECT;
    c.ku = (k % 256 == 0) ? 4 : ((k % 128 == 0) ? 2 : 1);
    const int stages = (k + c.ku * 64 - 1) / (c.ku * 64);
    c.rg = tiles16 >= 8 * cu_count ? 2 : 1;
    const int n_tiles = (n + 16 * c.rg - 1) / (16 * c.rg);
    const int m_tiles = (m + 16 * c.mt - 1) / (16 * c.mt);
    c.waves = stages >= 16 ? 8 : (stages >= 4 ? 4 : (stages >= 2 ? 2 : 1));
    // few tiles: spread K over more workgroups until half the CUs have one
    while ((long)n_tiles * m_tiles * c.split_k < cu_count / 2 && stages / (c.split_k * 2) >= 2 * c.waves &&
           c.split_k < 16)
        c.split_k *= 2;
    const int per_wave = stages / (c.split_k * c.waves);
    c.depth = per_wave >= 4 ? 4 : (per_wave >= 2 ? 2 : 1);
    while (stream_regs(c.mt, c.rg, c.ku, c.depth) > 128 && c.depth > 1) c.depth--;
    if (c.depth == 3 && c.ku == 8) c.depth = 2;
    return c;
}

// Shape -> configuration.  Weights are streamed once, so the only goals are (1) enough
// loads in flight on every CU to cover HBM latency and (2) long contiguous runs per weight
// row.  The LDS ring wins wherever it applies (k a multiple of 256); the register-streaming
// engine covers every other k.  The constants come from sweeps on one MI355X.
static Config pick_config(int m, int n, int k, int cu_count) {
    Config c;
    c.mt = m <= 16 ? 1 : 2;
    c.nt = 1;
    c.split_k = 1;
    c.persist = 0;
    c.wavetile = 0;
    const int tiles16 = (n + 15) / 16;
    // (a K that is not a multiple of 256 on the per-tile ring: against the register-streaming engine, us:
    // 8 x 8192 x 29568 58.1 -> 37, 32 x 8192 x 29568 87.9 -> 45, 8 x 2048 x 1408 4.2 -> 3.2)
    if (k % 256 == 0 || (lds_half_block_k(k) && m <= 32)) {
        c.engine = ENGINE_LDS;
        c.ku = 4;
        const int blocks = (k + 255) / 256;
        const int xu0 = c.mt == 2 ? 8 : ((m + 3) / 4 <= 1 ? 1 : ((m + 3) / 4 <= 2 ? 2 : 4));
        // Fewer 16-row tiles than half the CUs and K of 7168 or more: the idle CUs take K splits, up to four, of at least
        // 14 K blocks (8 at 17..32 rows) each.  Against one workgroup per tile, us: 8 x 2048 x 14336 10.9 -> 8.6,
        // 8 x 1024 x 14336 10.6 -> 7.6, 8 x 512 x 28672 18.6 -> 8.9, 16 x 1024 x 8192 7.7 -> 6.8, 8 x 2048 x 8192 7.3 -> 6.9;
        // 32 x 1024 x 14336 13.1 -> 8.9, 32 x 2048 x 14336 13.8 -> 10.9, 32 x 512 x 28672 20.1 -> 10.9, 32 x 512 x 8192 8.8 -> 7.0.
        // (At K = 4096 the unsplit launch is ahead: 24 x 2048 x 4096 6.2 against 6.6.)
        int few_tiles_split = 1;
        if (tiles16 * 2 <= cu_count && blocks >= 28) {
            const int per_split = c.mt == 2 ? 8 : 14;
            few_tiles_split = std::min(std::min(cu_count / tiles16, blocks / per_split), 4);
            if (few_tiles_split < 2) few_tiles_split = 1;
        }
        if (tiles16 > 2 * cu_count && k % 256 != 0) {
            // many tiles and a K the persistent kernels do not take: still one workgroup per tile.  Against the
            // register-streaming engine, us: 8 x 28672 x 4224 33.3 -> 23.5, 8 x 151936 x 896 33.5 -> 29.5, 8 x 14336 x 4112
            // 21.9 -> 14.7, 8 x 57344 x 8320 108 -> 79, 16 x 28672 x 2176 19.8 -> 15.0; 32 x 28672 x 4224 45.8 -> 27.1,
            // 32 x 151936 x 1152 54.9 -> 56.0
            c.rg = 1;
            c.waves = 1;
            c.depth = 4;
            if (c.mt == 2) {
                if (blocks >= 8) {
                    c.rg = 4;
                    c.waves = 2;
                    c.depth = 2;
                } else {
                    c.rg = 2;
                }
            }
            // ... or, where the whole activation matrix fits LDS beside the rings, whole tiles per wave on a persistent
            // workgroup per CU (the kernel of the short-K rule below, which takes any k); up to four tiles per CU only
            // at 17..32 rows, as there
            const bool fits8 = (size_t)blocks * xu0 * 1024 + 8 * 2 * 4096 + 4096 <= 159 * 1024;
            const bool fits4 = (size_t)blocks * xu0 * 1024 + 4 * 4 * 4096 + 4096 <= 159 * 1024;
            if (tiles16 > 4 * cu_count ? fits8 : (c.mt == 2 && fits4)) {
                c.rg = 1;
                c.persist = 1;
                c.wavetile = 1;
                c.waves = tiles16 > 4 * cu_count ? 8 : 4;
                c.depth = tiles16 > 4 * cu_count ? 2 : 4;
            }
            return c;
        }
        if (tiles16 > 2 * cu_count) {
            // more than two tiles per CU (at exactly two, one-wave workgroups are still 2-3 % ahead up to 16 rows;
            // at 2.25 they are 20 % behind): one persistent workgroup per CU walks them with continuous rings;
            // when one activation tile covers all of m, it stays resident in LDS and the stages
            // carry weights only
            c.rg = 1;
            c.persist = 1;
            const size_t x_res = (size_t)blocks * xu0 * 1024;
            if (blocks <= 10) {
                // a short K: every wave owns whole tiles over all of K - no reduction across waves in front of the
                // store - next to the whole activation matrix in LDS (at most 80 KB), eight waves x two slots.  Against
                // one wave per K block with its activation fragments in registers, us, cold weights: 8 x 28672 x 256
                // 8.5 -> 3.8, x 512 7.2 -> 4.9, x 1024 8.4 -> 7.3, x 2048 13.1 -> 11.7, x 2560 15.0 -> 14.0;
                // 16 x 57344 x 1024 13.5 -> 12.4, 32 x 28672 x 1024 9.8 -> 8.1, x 2048 14.4 -> 12.7, x 2560 17.1 -> 15.0,
                // 24 x 28672 x 512 8.8 -> 5.5.  (From 12 K blocks on the K-split waves below are level or ahead.)
                c.waves = 8;
                c.depth = 2;
                c.wavetile = 1;
                if (tiles16 <= 4 * cu_count) {
                    // up to four tiles per CU eight waves do not all find a tile: four waves x four slots at 17..32 rows
                    // (32 x 10240 x 2048 7.75 -> 6.67, 32 x 9216 x 2560 8.74 -> 7.36, 24 x 16384 x 2560 10.9 -> 10.1),
                    // and one-wave workgroups per tile up to 16 rows from 1024 columns of K on, 2-5 % ahead of that
                    // (8 x 16384 x 1024 5.29 -> 5.03, x 2048 7.71 -> 7.29, 16 x 16384 x 2048 7.73 -> 7.57)
                    if (c.mt == 2) {
                        c.waves = 4;
                        c.depth = 4;
                    } else if (blocks >= 4) {
                        c.persist = 0;
                        c.wavetile = 0;
                        c.waves = 1;
                        c.depth = 3;
                    }
                }
                return c;
            }
            // as many waves (at most eight) as divide the K blocks evenly, so that none idles through part of every
            // tile: 12 blocks on six waves 16.3 -> 15.9 us (8 x 28672 x 3072), 10 on five 14.9 -> 14.1 (x 2560)
            c.waves = 8;
            for (int w = 8; w >= 4; w--)
                if (blocks % w == 0) {
                    c.waves = w;
                    break;
                }
            c.depth = 2;
            if (m <= 16 * c.mt && x_res + (size_t)c.waves * (c.depth * 4 + 2 * c.mt) * 1024 + 4096 <= 159 * 1024) {
                c.wavetile = 2 | 4;   // resident activations + a dedicated epilogue wave (0.3-0.9 us on gate_up)
                return c;
            }
            c.waves = m <= 8 ? 8 : 6;
            // The activations do not fit LDS next to the rings (17..32 rows, or a long K): up to eight waves keep the
            // fragments of their own K blocks in registers - K = 256 * waves * blocks per wave, at most 4 / m_blocks of
            // them.  Against what ran before, us: 32 x 28672 x 3072 19.4 -> 17.6 (six waves), x 3584 20.9 -> 19.7;
            // 16 x 28672 x 8192 41.5 -> 38.3, 16 x 28672 x 6144 33.0 -> 29.1, 16 x 14336 x 8192 25.3 -> 24.1.
            for (int w = 8; w >= 2; w--) {
                const int pt = blocks / w;   // compiled for 1, 2 and 4 blocks per wave
                if (blocks % w != 0 || pt * c.mt > 4 || pt == 3) continue;
                c.waves = w;
                c.depth = blocks / w == 1 ? (w <= 2 ? 4 : 2) : 3;
                c.wavetile = 3;
                return c;
            }
            if (c.mt == 2) {
                // 17..32 rows, activations neither in LDS nor in registers: one workgroup per tile.  Up to three tiles
                // per CU one-wave workgroups on 16-row tiles (32 x 10240 x 8192 26.5 -> 20.4 us, 32 x 12288 x 5120
                // 18.0 -> 15.6), above that 64-row tiles, which share an activation stage among four weight tiles, on
                // three waves (32 x 13824 x 5120 18.3 -> 16.5, 32 x 12288 x 12288 41.7 -> 36.0; 16-row tiles fall off
                // a cliff there: 26.4)
                c.persist = 0;
                if (tiles16 <= 3 * cu_count) {
                    c.rg = 1;
                    c.waves = 1;
                    c.depth = 3;
                } else {
                    c.rg = 4;
                    c.waves = 3;
                    c.depth = 2;
                }
                return c;
            }
            // Up to 16 rows, the activations neither in LDS nor in registers (a long K that the waves cannot divide):
            // 9..16 rows share an activation stage among four weight tiles, 64-row tiles on two waves (16 x 14336 x 14336
            // 41.2 -> 32.5 us, 16 x 28672 x 10240 57.2 -> 47.4 against six waves on 16-row tiles); up to 8 rows one
            // workgroup of four waves per 16-row tile (8 x 28672 x 14336 63.8 -> 60.4, 4 x 57344 x 14336 120 -> 115).
            if (m > 8) {
                c.rg = 4;
                c.waves = 2;
                c.depth = 2;
            } else {
                c.persist = 0;
                c.waves = 4;
                c.depth = 3;
            }
        } else if (c.mt == 2) {                 // 17..32 activation rows: the activation traffic rivals the weights'
            // (exactly two 16-row tiles per CU belong here: 32-row tiles, one per CU - 32 x 8192 x 8192 23.8 -> 15.0 us
            // against 64-row tiles on half the CUs, 32 x 8192 x 4096 9.95 -> 9.50 against the register-resident kernel.
            // A long K is split in two only where that fills the device: with more than one tile per CU the unsplit
            // 32-row tiles win, 32 x 5120 x 13824 25.5 -> 20.6, 20 x 8192 x 14336 27.9 -> 23.3)
            if (few_tiles_split > 1) {          // fewer tiles than half the CUs and a long K: see below
                c.rg = 1;
                c.waves = 2;
                c.depth = 3;
                c.split_k = few_tiles_split;
            } else if (blocks >= 48 && tiles16 <= cu_count) {
                c.rg = 2;
                c.waves = 2;
                c.depth = 3;
                c.split_k = 2;
            } else if (tiles16 * 4 >= cu_count * 5) {
                c.rg = 2;
                c.waves = 2;
                c.depth = 2;
            } else {                            // (two waves x three slots beat three x two by 2-5 % on nine shapes)
                c.rg = 1;
                c.waves = 2;
                c.depth = 3;
            }
        } else {                                // about one tile per CU: few waves, deep rings
            // (one wave x eight slots also for long K: 4096 x 14336 at 1, 4, 8, 16 rows 0.5-2.3 % ahead of two waves
            // x four slots in the tuner's alternating rounds - no cross-wave reduction in front of the store)
            c.rg = 1;
            c.waves = 1;
            c.depth = 8;
            c.split_k = few_tiles_split;
            // between one and two 16-row tiles per CU half of the CUs stream twice what the others do (all
            // workgroups are resident at once); 24-row tiles that give every CU one workgroup level that.  Measured
            // on 6144 x 4096: level with 16-row tiles up to 8 activation rows (6.75 against 6.70 us - the launch is
            // bound by its fixed costs and the stream rate, not by the imbalance), 3-5 % ahead at 9..16 rows
            // (7.00 against 7.23-7.40 us), where the activation stage is shared by more weight rows.  With a longer K
            // a tile is worth more against the fixed costs and the levelling pays at any row count: 8 x 5120 x 5120
            // 7.8 -> 7.3, 8 x 6144 x 8192 11.1 -> 10.6, 8 x 5120 x 13824 16.7 -> 14.8, 8 x 6144 x 14336 18.7 -> 16.9.
            const int tiles24 = (n + 23) / 24;
            if ((m > 8 || blocks > 16) &&
                ((tiles24 + cu_count - 1) / cu_count) * 24 < ((tiles16 + cu_count - 1) / cu_count) * 16) {
                c.rg = 2;
                c.wavetile = 8;
                c.waves = 2;
                c.depth = 4;
            }
        }
        const int xu = c.mt == 2 ? 8 : ((m + 3) / 4 <= 1 ? 1 : ((m + 3) / 4 <= 2 ? 2 : 4));
        const int w_instr = (c.wavetile & 8) ? 6 : c.rg * 4;
        while (c.depth > 2 && ((c.depth - 1) * (w_instr + xu) > 63 ||
                               (size_t)c.waves * c.depth * (w_instr + xu) * 1024 + 4096 > 159 * 1024))
            c.depth--;
        if (!c.persist && c.depth > blocks / c.waves && blocks / c.waves >= 2) c.depth = blocks / c.waves;
        if (c.depth == 5 || c.depth == 7) c.depth--;
        return c;
    }
    return direct_config(m, n, k, cu_count);
}

// bf16 activations -> the GEMM quantises them itself: the persistent kernel with the activations resident in LDS
// (every workgroup derives the row scales and the codes of its own copy).  fused_config: what the kernel can run -
// one activation tile covers all of m and the codes fit LDS next to the rings of at least four waves.
static bool fused_config(int m, int k, Config* out) {
    if (k % 256 != 0 || m > 32) return false;
    Config c;
    c.engine = ENGINE_LDS;
    c.mt = m <= 16 ? 1 : 2;
    c.rg = 1;
    c.ku = 4;
    c.depth = 2;
    c.split_k = 1;
    c.nt = 1;
    c.persist = 1;
    c.wavetile = 2 | 4;          // resident activations + epilogue wave
    const int blocks = k / 256;
    const int xu = c.mt == 2 ? 8 : ((m + 3) / 4 <= 1 ? 1 : ((m + 3) / 4 <= 2 ? 2 : 4));
    const size_t x_res = (size_t)blocks * xu * 1024;
    // at least four streaming waves: fewer keep too little in flight per CU
    for (int waves : {8, 6, 4}) {
        if (x_res + (size_t)waves * (c.depth * 4 + 2 * c.mt) * 1024 + 4096 > 159 * 1024) continue;
        c.waves = waves;
        *out = c;
        return true;
    }
    return false;
}

// ... and where it pays.  Every workgroup repeats the quantisation of all m x k activations (about 2.4 us of vector
// work per workgroup at m = 8, k = 4096), which is only hidden where the workgroup goes on to stream several tiles:
// 8 x 28672 x 4096 takes 26.9 us fused against 29.0 us for the two launches, 8 x 4096 x 4096 8.5 against 8.4,
// 8 x 6144 x 4096 10.8 against 9.9, and at 16 rows or with a share too long for registers the two launches win.
static bool pick_bf16act(int m, int n, int k, int cu_count, Config* out) {
    Config c;
    if (!fused_config(m, k, &c)) return false;
    const int tiles = (n + 15) / 16, blocks = k / 256;
    const int xu = c.mt == 2 ? 8 : ((m + 3) / 4 <= 1 ? 1 : ((m + 3) / 4 <= 2 ? 2 : 4));
    if (m > 8 || tiles < 3 * cu_count || ((blocks + c.waves - 1) / c.waves) * xu > 8) return false;
    *out = c;
    return true;
}

// Scratch for the two-launch form of sg_skinny_gemm_bf16act (shapes the fused kernel does not take): the E4M3 codes
// and row scales of the activations, one buffer per (device, stream), grown on demand and kept.
struct ActScratch { uint8_t* p = nullptr; size_t bytes = 0; };
static std::map<hipStream_t, ActScratch> g_act[kMaxDevices];

static int get_act_scratch(hipStream_t stream, size_t bytes, uint8_t** out) {
    int dev;
    if (int rc = current_device(&dev)) return rc;
    std::lock_guard<std::mutex> lock(g_mutex);
    ActScratch& sc = g_act[dev][stream];
    if (sc.bytes < bytes) {
        const size_t want = round_up_pow2(bytes, 1u << 20);
        void* p = workspace_alloc(want);    // an outgrown buffer is kept: launches already enqueued may still read it
        if (!p) return SG_NO_DEVICE;
        if (sc.p) g_retired[dev].push_back({stream, sc.p, sc.bytes});
        sc.p = static_cast<uint8_t*>(p);
        sc.bytes = want;
        g_ws_bytes[dev] += want;
    }
    *out = sc.p;
    return SG_SUCCESS;
}

static Config config_from_tuning(const SgTuning& t) {
    Config c;
    c.engine = t.engine;
    c.mt = t.m_blocks;
    c.rg = t.row_tiles;
    c.ku = t.k_chunks;
    c.depth = t.depth;
    c.waves = t.waves;
    c.split_k = t.split_k;
    c.nt = t.non_temporal;
    c.persist = t.persistent_wgs_per_cu;
    c.wavetile = t.wave_tiles;
    return c;
}

// 33..256 activation rows on a small weight matrix: the skinny ring over several 32-row activation tiles beats the
// mid-batch tiles, which leave most CUs without work or split K to fill them, as long as one round of workgroups
// covers every (weight tile, activation tile) pair.  The activation tiles of a weight tile are neighbours in tile
// order, i.e. on one XCD, whose L2 fetches the weight tile once for all of them.  The smallest weight tile - 16, 32 or
// 64 rows - that fits the round; 64-row tiles only below K = 8192 (224 x 1536 x 6144 16.1 -> 12.6; level at 8192, behind
// at 14336).  Same-process
// medians, us, cold weights, against the mid-batch choice: 64 x 1024 x 4096 12.7 -> 5.9, 128 x 2048 x 4096 12.8 -> 7.2,
// 256 x 1024 x 4096 12.4 -> 6.7, 64 x 4096 x 4096 13.3 -> 8.0, 128 x 4096 x 4096 13.1 -> 10.9, 256 x 2048 x 4096
// 12.7 -> 10.2, 64 x 8192 x 4096 14.2 -> 12.2, 128 x 4096 x 2048 8.7 -> 7.4, 96 x 5120 x 5120 16.1 -> 13.5,
// 128 x 2048 x 8192 16.6 -> 10.7, 64 x 4096 x 8192 16.6 -> 12.6, 128 x 2048 x 14336 23.8 -> 17.1, 64 x 2048 x 14336
// 20.4 -> 13.5.  Up to 64 rows one-wave workgroups on 16-row tiles still win at up to one and a half tiles per CU
// (64 x 6144 x 4096 13.6 -> 11.0, 64 x 5120 x 5120 18.1 -> 13.4); beyond (64 x 10240 x 4096, 96 x 6144 x 4096,
// 192 x 4096 x 4096) the mid-batch engine is 10-25 % ahead.
static bool two_pass_config(int m, int n, int k, int cu_count, Config* out) {
    if (m <= 32 || m > 256 || (k % 256 != 0 && !lds_half_block_k(k))) return false;
    const long tiles16 = (n + 15) / 16, tiles32 = (n + 31) / 32, tiles64 = (n + 63) / 64;
    const int blocks = (k + 255) / 256, m_tiles = (m + 31) / 32;
    Config c;
    c.engine = ENGINE_LDS;
    c.mt = 2;
    c.nt = 1;
    c.ku = 4;
    c.split_k = 1;
    c.persist = 0;
    c.wavetile = 0;
    c.depth = 2;
    if (blocks >= 64) {
        // K of 16384 or more: two K splits on the tile that still fits the round with them, or the mid-batch engine
        // (which splits up to four ways).  us: 40 x 1024 x 28672 20.9 unsplit -> 14.3 (mid-batch 24.6), 128 x 1024 x 28672
        // 23.7 -> 18.8 (26.5), 64 x 2048 x 28672 25.7 -> 21.2 (28.2), 64 x 2048 x 20480 19.7 -> 16.9 (23.5); 48 x 3072 x 28672
        // and 64 x 4096 x 28672, where only the unsplit ring fits, 34.9 and 36.1 against 28.5 and 31.7 for the mid-batch engine
        c.split_k = 2;
        if (tiles16 * m_tiles * 2 <= cu_count) {
            c.rg = 1;
            c.waves = 2;
            c.depth = 3;
        } else if (tiles32 * m_tiles * 2 <= cu_count) {
            c.rg = 2;
            c.waves = 3;
        } else {
            return false;
        }
        *out = c;
        return true;
    }
    if (tiles16 * m_tiles <= cu_count) {           // 16-row tiles: every (tile, activation tile) pair gets a CU
        c.rg = 1;
        c.waves = 2;
        c.depth = 3;
    } else if (tiles32 * m_tiles <= cu_count) {    // 32-row tiles
        c.rg = 2;
        c.waves = blocks > 32 ? 3 : 4;
    } else if (m <= 64 && tiles16 * 2 <= cu_count * 3 && blocks <= 20) {
        c.rg = 1;                                  // (2-4 % ahead of 64-row tiles there: 64 x 6144 x 4096 11.0 against 11.5)
        c.waves = 1;
        c.depth = 3;
    } else if (tiles64 * m_tiles <= cu_count && blocks < 32) {
        c.rg = 4;
        c.waves = 3;
    } else {
        return false;
    }
    *out = c;
    return true;
}

static Config heuristic_config(int m, int n, int k, int cu_count) {
    Config two;
    if (two_pass_config(m, n, k, cu_count, &two)) return two;
    // (a k that is not a multiple of 128 runs in the mid-batch kernel's builds with a partial last block: against the
    // skinny ring over 64-row weight tiles, which took such k before, us: 128 x 4096 x 7392 19.9 -> see the design notes)
    if (m > 32 && (k % 128 == 0 || mid_partial_block_k(k))) return pick_mid(m, n, k, cu_count);
    return pick_config(m, n, k, cu_count);
}

// ---- per-shape tuning table ---------------------------------------------------------------
// What a tuning driver measured to be the best record for a shape; consulted before the
// heuristics by the launchers that choose their own configuration.  Process-wide, any thread.
static std::mutex g_table_mutex;
static std::map<std::tuple<int, int, int>, SgTuning> g_table;
static std::atomic<int> g_table_entries{0};   // an empty table costs the launch path one relaxed load
static int sg_tuning_load_file(const char* path);   // what sg_tuning_load does, without the default table first

// The table the library ships: tuning/mi355x.tbl beside the package's csrc directory (the records its tuning driver
// found for the benchmark shapes), merged into the table once, before the table is first read or changed.  The
// environment variable SGEMM_TUNING_TABLE names another file to load instead; empty or "none" loads nothing.
static std::once_flag g_default_table_once;
static void load_default_table() {
    const char* env = std::getenv("SGEMM_TUNING_TABLE");
    if (env) {
        if (*env && std::strcmp(env, "none") != 0 && sg_tuning_load_file(env) != SG_SUCCESS && std::getenv("SG_VERBOSE"))
            std::fprintf(stderr, "libsgemm: cannot load the tuning table %s\n", env);
        return;
    }
    Dl_info info;
    if (!dladdr(reinterpret_cast<const void*>(&load_default_table), &info) || !info.dli_fname) return;
    std::string path(info.dli_fname);
    const size_t slash = path.rfind('/');
    path = (slash == std::string::npos ? std::string(".") : path.substr(0, slash)) + "/../tuning/mi355x.tbl";
    if (FILE* f = std::fopen(path.c_str(), "r")) {
        std::fclose(f);
        if (sg_tuning_load_file(path.c_str()) != SG_SUCCESS && std::getenv("SG_VERBOSE"))
            std::fprintf(stderr, "libsgemm: malformed tuning table %s\n", path.c_str());
    }
}
static void ensure_default_table() { std::call_once(g_default_table_once, load_default_table); }

static bool table_lookup(int m, int n, int k, SgTuning* out) {
    ensure_default_table();
    if (g_table_entries.load(std::memory_order_relaxed) == 0) return false;
    std::lock_guard<std::mutex> lock(g_table_mutex);
    const auto it = g_table.find(std::make_tuple(m, n, k));
    if (it == g_table.end()) return false;
    *out = it->second;
    return true;
}

// A record is rejected by the launch functions before anything is enqueued with one of these codes
// (no kernel for it, ring does not fit LDS, k not a multiple of the engine's stage, ...).
static bool rejected_before_launch(int rc) {
    return rc == SG_INVALID_CONFIG || rc == SG_K_NOT_DIVISIBLE_BY_WARPTILE_K || rc == SG_TOO_MANY_WARPS ||
           rc == SG_WORKSPACE_TOO_SMALL;
}

// The table's record for the shape if it has a usable one, the heuristics' otherwise.  Should a launch
// function refuse the heuristics' own record before anything is enqueued (split-K partials beyond the
// workspace limit, a combination nothing is compiled for), the same record without the K split and then
// the register-streaming engine, which takes every legal shape, are tried.
static int launch_chosen(const StreamArgs& a, int cu_count, hipStream_t stream, const Workspace* fixed_ws = nullptr) {
    SgTuning t;
    if (table_lookup(a.m, a.n, a.k, &t) && t.engine != ENGINE_AUTO) {
        Config c = config_from_tuning(t);
        c.fixed_ws = fixed_ws;
        if (c.engine == ENGINE_MID || c.mt == 1 || c.mt == 2) {
            const int rc = launch_config(c, a, stream);
            if (!rejected_before_launch(rc)) return rc;
        }
    }
    Config c = heuristic_config(a.m, a.n, a.k, cu_count);
    c.fixed_ws = fixed_ws;
    int rc = launch_config(c, a, stream);
    if (rejected_before_launch(rc) && c.split_k > 1) {
        c.split_k = 1;
        rc = launch_config(c, a, stream);
    }
    if (rejected_before_launch(rc)) {
        c = direct_config(a.m, a.n, a.k, cu_count);
        c.fixed_ws = fixed_ws;
        c.split_k = 1;
        rc = launch_config(c, a, stream);
    }
    return rc;
}

}  // namespace sg

using namespace sg;

extern "C" {

const char* sg_strerror(int code) {
    switch (code) {
        case SG_SUCCESS: return "success";
        case SG_M_ABOVE_WARPTILE_M: return "m is greater than WARPTILE_M";
        case SG_N_NOT_EVEN: return "n is not even";
        case SG_K_NOT_DIVISIBLE_BY_WARPTILE_K: return "k is not divisible by WARPTILE_K";
        case SG_TOO_MANY_WARPS: return "A_producers + B_producers + consumers is greater than 16";
        case SG_QSIZE_TOO_SMALL: return "qsize is less than A_producers, B_producers / b_lanes, or consumers";
        case SG_INVALID_CONFIG: return "no kernel is compiled for this configuration";
        case SG_LAUNCH_FAILED: return "the HIP runtime refused the launch";
        case SG_BAD_ALIGNMENT: return "pointer or stride is not sufficiently aligned";
        case SG_BAD_ARGUMENT: return "null pointer or size out of range";
        case SG_WORKSPACE_TOO_SMALL: return "split-K partials do not fit the workspace";
        case SG_NO_DEVICE: return "no usable gfx950 device";
        default: return "unknown code";
    }
}

int sg_init(void) { return sg_init_stream(nullptr, kDefaultPartialBytes); }

int sg_init_stream(void* stream, size_t partial_bytes) {
    DeviceInfo* d;
    if (int rc = get_device_info(&d)) return rc;
    Workspace w;
    return get_workspace(static_cast<hipStream_t>(stream), partial_bytes, kMinCounters, &w);
}

size_t sg_workspace_bytes(void) {
    int dev;
    if (current_device(&dev)) return 0;
    std::lock_guard<std::mutex> lock(g_mutex);
    return g_ws_bytes[dev];
}

// Frees the buffers of g_ws / g_act / g_retired that belong to `stream` (all streams with every == true); the caller
// has synchronised.  g_mutex held.
static void free_owned(int dev, hipStream_t stream, bool every) {
    for (auto it = g_ws[dev].begin(); it != g_ws[dev].end();) {
        if (every || it->first == stream) {
            if (it->second.partials) { (void)hipFree(it->second.partials); g_ws_bytes[dev] -= it->second.partial_bytes; }
            if (it->second.counters) { (void)hipFree(it->second.counters); g_ws_bytes[dev] -= it->second.n_counters * sizeof(unsigned); }
            it = g_ws[dev].erase(it);
        } else {
            ++it;
        }
    }
    for (auto it = g_act[dev].begin(); it != g_act[dev].end();) {
        if (every || it->first == stream) {
            if (it->second.p) { (void)hipFree(it->second.p); g_ws_bytes[dev] -= it->second.bytes; }
            it = g_act[dev].erase(it);
        } else {
            ++it;
        }
    }
    std::vector<Retired> keep;
    for (const Retired& r : g_retired[dev]) {
        if (every || r.stream == stream) { (void)hipFree(r.p); g_ws_bytes[dev] -= r.bytes; }
        else keep.push_back(r);
    }
    g_retired[dev].swap(keep);
}

int sg_release_stream(void* stream) {
    int dev;
    if (int rc = current_device(&dev)) return rc;
    if (report_hip("hipStreamSynchronize", hipStreamSynchronize(static_cast<hipStream_t>(stream))) != hipSuccess) {
        (void)hipGetLastError();
        return SG_LAUNCH_FAILED;
    }
    std::lock_guard<std::mutex> lock(g_mutex);
    free_owned(dev, static_cast<hipStream_t>(stream), false);
    return SG_SUCCESS;
}

int sg_release_workspaces(void) {
    int dev;
    if (int rc = current_device(&dev)) return rc;
    if (report_hip("hipDeviceSynchronize", hipDeviceSynchronize()) != hipSuccess) {
        (void)hipGetLastError();
        return SG_LAUNCH_FAILED;
    }
    std::lock_guard<std::mutex> lock(g_mutex);
    free_owned(dev, nullptr, true);
    return SG_SUCCESS;
}

// Caller-owned workspace: [kCallerCounters arrival counters][fp32 partials].  The counter region has one size for
// every shape, so that one buffer serves launches of different shapes one after the other.
constexpr size_t kCallerCounters = 16384;
constexpr size_t kCallerCounterBytes = kCallerCounters * sizeof(unsigned);

int sg_workspace_query(int m, int n, int k, size_t* bytes) {
    if (!bytes || m <= 0 || n <= 0 || k <= 0) return SG_BAD_ARGUMENT;
    DeviceInfo* dev;
    int cu = 256;
    if (get_device_info(&dev) == SG_SUCCESS) cu = dev->cu_count;
    SgTuning t;
    Config c = (table_lookup(m, n, k, &t) && t.engine != ENGINE_AUTO) ? config_from_tuning(t) : heuristic_config(m, n, k, cu);
    size_t partial, counters;
    workspace_need(c, m, n, &partial, &counters);
    // (should the table's record be refused at launch, the heuristics' record runs: it must fit as well)
    const Config h = heuristic_config(m, n, k, cu);
    size_t partial_h, counters_h;
    workspace_need(h, m, n, &partial_h, &counters_h);
    if (partial_h > partial) partial = partial_h;
    *bytes = partial ? kCallerCounterBytes + partial : 0;
    return SG_SUCCESS;
}

int sg_workspace_init(void* workspace, size_t bytes, void* stream) {
    if (!workspace || bytes < kCallerCounterBytes || (reinterpret_cast<uintptr_t>(workspace) & 255u)) return SG_BAD_ARGUMENT;
    return fill_zero(static_cast<unsigned*>(workspace), kCallerCounters, static_cast<hipStream_t>(stream));
}

int sg_skinny_gemm_auto_ws(const uint8_t* A, const uint8_t* B, void* D, const float* scale_tensor, int m, int n, int k,
                           int b_stride, void* workspace, size_t workspace_bytes, void* stream) {
    if (n % 2 != 0) return SG_N_NOT_EVEN;
    if (k % 16 != 0) return SG_K_NOT_DIVISIBLE_BY_WARPTILE_K;
    if (int rc = check_pointers(A, B, D, m, n, k, b_stride)) return rc;
    if (!scale_tensor) return SG_BAD_ARGUMENT;
    if (workspace && (reinterpret_cast<uintptr_t>(workspace) & 255u)) return SG_BAD_ALIGNMENT;
    DeviceInfo* dev;
    if (int rc = get_device_info(&dev)) return rc;
    size_t need = 0;
    if (int rc = sg_workspace_query(m, n, k, &need)) return rc;
    if (need > 0 && (!workspace || workspace_bytes < need)) return SG_WORKSPACE_TOO_SMALL;
    // a launch without a K split gets a workspace nothing fits into: whatever would want one is refused, never allocated
    Workspace w;
    if (need > 0) {
        w.counters = static_cast<unsigned*>(workspace);
        w.n_counters = kCallerCounters;
        w.partials = reinterpret_cast<float*>(static_cast<unsigned char*>(workspace) + kCallerCounterBytes);
        w.partial_bytes = workspace_bytes - kCallerCounterBytes;
    }
    StreamArgs a{};
    a.A = A; a.B = B; a.D = D; a.scale = scale_tensor;
    a.m = m; a.n = n; a.k = k; a.b_stride = b_stride;
    a.out_f32 = 0;
    return launch_chosen(a, dev->cu_count, static_cast<hipStream_t>(stream), &w);
}

int sg_debug_stamps(unsigned long long* device_buffer, size_t n_words) {
    std::lock_guard<std::mutex> lock(g_mutex);
    g_stamp_buf = n_words ? device_buffer : nullptr;
    g_stamp_words = device_buffer ? n_words : 0;
    g_stamp_cursor = 0;
    g_stamps_on.store(g_stamp_buf != nullptr && g_stamp_words > 0, std::memory_order_relaxed);
    return SG_SUCCESS;
}

int sg_debug_read_stream(const uint8_t* B, int n, int k, int b_stride, int segment_bytes, void* stream) {
    if (!B || n <= 0 || k <= 0 || k % 1024 != 0 || b_stride < k || (b_stride & 15) || (reinterpret_cast<uintptr_t>(B) & 15u))
        return SG_BAD_ARGUMENT;
    if (segment_bytes != 256 && segment_bytes != 512 && segment_bytes != 1024) return SG_BAD_ARGUMENT;
    DeviceInfo* dev;
    if (int rc = get_device_info(&dev)) return rc;
    const int tile_rows = 4 * (1024 / segment_bytes);
    const int tiles = (n + tile_rows - 1) / tile_rows;
    const unsigned grid = (unsigned)(tiles < dev->cu_count ? tiles : dev->cu_count);
    auto kernel = segment_bytes == 256 ? read_stream_kernel<256> : (segment_bytes == 512 ? read_stream_kernel<512> : read_stream_kernel<1024>);
    kernel<<<dim3(grid), dim3(512), 8 * 2 * 4096, static_cast<hipStream_t>(stream)>>>(B, n, k, b_stride, nullptr);
    return report_hip("read_stream_kernel launch", hipGetLastError()) == hipSuccess ? SG_SUCCESS : SG_LAUNCH_FAILED;
}

int sg_debug_cu_ingest(const uint8_t* cold, size_t cold_bytes, const uint8_t* hot, size_t hot_bytes, int workgroups, int waves,
                       int cold_waves, int hot_per_cold, int depth, int ticks, unsigned long long* counts, void* stream) {
    if (!cold || !hot || !counts || workgroups < 1 || workgroups > 4096 || ticks < 1 || ticks > 1000000) return SG_BAD_ARGUMENT;
    if (waves != 1 && waves != 2 && waves != 4 && waves != 8 && waves != 16) return SG_BAD_ARGUMENT;
    if (cold_waves > waves || (cold_waves < 0 && hot_per_cold < 1) || (depth != 4 && depth != 8 && depth != 16)) return SG_BAD_ARGUMENT;
    if (depth > 128 / waves) return SG_BAD_ARGUMENT;
    if ((reinterpret_cast<uintptr_t>(cold) | reinterpret_cast<uintptr_t>(hot)) & 15u) return SG_BAD_ALIGNMENT;
    // largest powers of two that fit: a region per wave of the cold buffer, one window per XCD of the hot one; a load
    // instruction spans 8 rows of 8 KB
    auto floor_pow2 = [](size_t v) { size_t p = 1; while (p * 2 <= v) p *= 2; return p; };
    const size_t region = floor_pow2(cold_bytes / ((size_t)workgroups * waves)), window = floor_pow2(hot_bytes / 8);
    if (region < 65536 || window < 65536 || region > 0x80000000u || window > 0x80000000u) return SG_BAD_ARGUMENT;
    DeviceInfo* dev;
    if (int rc = get_device_info(&dev)) return rc;
    auto kernel = depth == 4 ? cu_ingest_kernel<4> : (depth == 8 ? cu_ingest_kernel<8> : cu_ingest_kernel<16>);
    static LdsGranted granted[3];
    if (int rc = request_dynamic_lds(reinterpret_cast<const void*>(kernel), 128 * 1024, granted[depth == 4 ? 0 : (depth == 8 ? 1 : 2)])) return rc;
    kernel<<<dim3((unsigned)workgroups), dim3((unsigned)waves * 64), 128 * 1024, static_cast<hipStream_t>(stream)>>>(
        cold, (unsigned)region, hot, (unsigned)window, ticks, cold_waves, hot_per_cold, counts);
    return report_hip("cu_ingest_kernel launch", hipGetLastError()) == hipSuccess ? SG_SUCCESS : SG_LAUNCH_FAILED;
}

int sg_skinny_gemm(const uint8_t* A, const uint8_t* B, void* D, const float* scale_tensor, int m, int n, int k,
                   int b_stride, int split_k, int A_producers, int B_producers, int consumers, int b_lanes, int qsize,
                   int op_m, int ops, void* stream) {
    if (op_m != 8 && op_m != 16 && op_m != 32) return SG_INVALID_CONFIG;
    if (ops <= 0 || b_lanes <= 0 || qsize <= 0 || split_k <= 0 || A_producers < 0 || B_producers < 0 || consumers <= 0)
        return SG_INVALID_CONFIG;
    const int warptile_k = (512 / op_m) * ops;
    // same order as skinny_gemm/skinny_gemm_caller.cu:55-75
    if (n % 2 != 0) return SG_N_NOT_EVEN;
    if (k % warptile_k != 0) return SG_K_NOT_DIVISIBLE_BY_WARPTILE_K;
    if (A_producers + B_producers + consumers > 16) return SG_TOO_MANY_WARPS;
    const bool ring = A_producers > 0 || B_producers > 0;
    if (ring && (qsize < A_producers || qsize < (B_producers / b_lanes) || qsize < consumers)) return SG_QSIZE_TOO_SMALL;
    if (int rc = check_pointers(A, B, D, m, n, k, b_stride)) return rc;
    if (!scale_tensor) return SG_BAD_ARGUMENT;
    DeviceInfo* dev;
    if (int rc = get_device_info(&dev)) return rc;

    if (ring) {
        // the ring's stage is one 256-byte K block; both operands need a producer
        if (warptile_k != 256 || A_producers < 1 || B_producers < 1) return SG_INVALID_CONFIG;
        RingConfig rc;
        rc.mt = op_m == 32 ? 2 : 1;
        rc.b_lanes = b_lanes;
        rc.qsize = qsize;
        rc.a_producers = A_producers;
        rc.b_producers = B_producers;
        rc.consumers = consumers;
        rc.nt = 1;
        rc.split_k = split_k;
        StreamArgs ar{};
        ar.A = A; ar.B = B; ar.D = D; ar.scale = scale_tensor;
        ar.m = m; ar.n = n; ar.k = k; ar.b_stride = b_stride;
        ar.out_f32 = 0;
        return launch_ring(rc, ar, static_cast<hipStream_t>(stream));
    }

    if (warptile_k % 64 != 0) return SG_INVALID_CONFIG;
    Config c;
    c.mt = op_m == 32 ? 2 : 1;
    c.rg = b_lanes;
    c.ku = warptile_k / 64;
    c.depth = qsize;
    c.waves = consumers;
    c.split_k = split_k;
    c.nt = 1;
    c.persist = 0;
    c.wavetile = 0;
    // a 256-byte stage with at least two ring slots is the LDS ring's shape; everything else
    // streams straight into registers
    StreamArgs a{};
    a.A = A; a.B = B; a.D = D; a.scale = scale_tensor;
    a.m = m; a.n = n; a.k = k; a.b_stride = b_stride;
    a.out_f32 = 0;
    if (warptile_k == 256 && qsize >= 2 && k % 256 == 0 && (b_lanes == 1 || b_lanes == 2 || b_lanes == 4)) {
        c.engine = ENGINE_LDS;
        const int rc = launch_config(c, a, static_cast<hipStream_t>(stream));
        if (rc != SG_INVALID_CONFIG) return rc;   // ring does not fit LDS: stream through registers instead
    }
    c.engine = ENGINE_DIRECT;
    return launch_config(c, a, static_cast<hipStream_t>(stream));
}

int sg_skinny_gemm_tuned(const uint8_t* A, const uint8_t* B, void* D, const float* scale_tensor, int m, int n, int k,
                         int b_stride, const SgTuning* t, void* stream) {
    if (!t) return SG_BAD_ARGUMENT;
    if (n % 2 != 0) return SG_N_NOT_EVEN;
    if (k % 16 != 0) return SG_K_NOT_DIVISIBLE_BY_WARPTILE_K;
    if (int rc = check_pointers(A, B, D, m, n, k, b_stride)) return rc;
    if (!scale_tensor) return SG_BAD_ARGUMENT;
    DeviceInfo* dev;
    if (int rc = get_device_info(&dev)) return rc;
    Config c = config_from_tuning(*t);
    if (c.engine == ENGINE_AUTO) c = heuristic_config(m, n, k, dev->cu_count);
    if (c.engine != ENGINE_MID && c.mt != 1 && c.mt != 2) return SG_INVALID_CONFIG;
    StreamArgs a{};
    a.A = A; a.B = B; a.D = D; a.scale = scale_tensor;
    a.m = m; a.n = n; a.k = k; a.b_stride = b_stride;
    a.out_f32 = 0;
    return launch_config(c, a, static_cast<hipStream_t>(stream));
}

int sg_skinny_gemm_tuned_noalloc(const uint8_t* A, const uint8_t* B, void* D, const float* scale_tensor, int m, int n,
                                 int k, int b_stride, const SgTuning* t, void* stream) {
    if (!t) return SG_BAD_ARGUMENT;
    if (n % 2 != 0) return SG_N_NOT_EVEN;
    if (k % 16 != 0) return SG_K_NOT_DIVISIBLE_BY_WARPTILE_K;
    if (int rc = check_pointers(A, B, D, m, n, k, b_stride)) return rc;
    if (!scale_tensor) return SG_BAD_ARGUMENT;
    DeviceInfo* dev;
    if (int rc = get_device_info(&dev)) return rc;
    Workspace w;
    bool first_use = false;
    if (int rc = static_workspace(&w, &first_use)) return rc;
    Config c = config_from_tuning(*t);
    if (c.engine == ENGINE_AUTO) {
        c = heuristic_config(m, n, k, dev->cu_count);
        // the library's own choice is made to fit the array: a K split whose partials or counters do not, is not taken
        size_t partial_bytes, counters;
        workspace_need(c, m, n, &partial_bytes, &counters);
        if (partial_bytes > w.partial_bytes || counters > w.n_counters) {
            c.split_k = 1;
            if (c.engine == ENGINE_MID) c.wavetile = 0;
        }
    }
    if (c.engine != ENGINE_MID && c.mt != 1 && c.mt != 2) return SG_INVALID_CONFIG;
    c.fixed_ws = &w;
    StreamArgs a{};
    a.A = A; a.B = B; a.D = D; a.scale = scale_tensor;
    a.m = m; a.n = n; a.k = k; a.b_stride = b_stride;
    a.out_f32 = 0;
    // The array keeps whatever the last call left.  The partials are written before they are read.  The arrival
    // counters must start at zero: the array is zero when the device image is loaded and every launch that completes
    // leaves its counters at zero, so they are cleared once, with the first call on the device (by a kernel, at once:
    // under capture a launch on the stream would only be recorded), and not again before every launch.
    if (first_use)
        if (int rc = fill_zero_now(w.counters, w.n_counters)) return rc;
    return launch_config(c, a, static_cast<hipStream_t>(stream));
}

int sg_skinny_gemm_pick(int m, int n, int k, int out[8]) {
    if (!out || m <= 0 || n <= 0 || k <= 0) return SG_BAD_ARGUMENT;
    DeviceInfo* dev;
    int cu = 256;
    if (get_device_info(&dev) == SG_SUCCESS) cu = dev->cu_count;
    const Config c = pick_config(m, n, k, cu);
    const int op_m = c.mt == 2 ? 32 : (m <= 8 ? 8 : 16);
    out[0] = c.split_k; out[1] = 0; out[2] = 0; out[3] = c.waves;
    out[4] = c.rg; out[5] = c.depth; out[6] = op_m; out[7] = c.ku * 64 / (512 / op_m);
    return SG_SUCCESS;
}

int sg_skinny_gemm_choice(int m, int n, int k, SgTuning* out, int* from_table) {
    if (!out || m <= 0 || n <= 0 || k <= 0) return SG_BAD_ARGUMENT;
    if (table_lookup(m, n, k, out)) {
        if (from_table) *from_table = 1;
        return SG_SUCCESS;
    }
    DeviceInfo* dev;
    int cu = 256;
    if (get_device_info(&dev) == SG_SUCCESS) cu = dev->cu_count;
    const Config c = heuristic_config(m, n, k, cu);
    out->engine = c.engine; out->split_k = c.split_k; out->waves = c.waves; out->row_tiles = c.rg; out->m_blocks = c.mt;
    out->depth = c.depth; out->k_chunks = c.ku; out->non_temporal = c.nt; out->persistent_wgs_per_cu = c.persist;
    out->wave_tiles = c.wavetile;
    if (from_table) *from_table = 0;
    return SG_SUCCESS;
}

int sg_skinny_gemm_auto(const uint8_t* A, const uint8_t* B, void* D, const float* scale_tensor, int m, int n, int k,
                        int b_stride, void* stream) {
    if (n % 2 != 0) return SG_N_NOT_EVEN;
    if (k % 16 != 0) return SG_K_NOT_DIVISIBLE_BY_WARPTILE_K;
    if (int rc = check_pointers(A, B, D, m, n, k, b_stride)) return rc;
    if (!scale_tensor) return SG_BAD_ARGUMENT;
    DeviceInfo* dev;
    if (int rc = get_device_info(&dev)) return rc;
    StreamArgs a{};
    a.A = A; a.B = B; a.D = D; a.scale = scale_tensor;
    a.m = m; a.n = n; a.k = k; a.b_stride = b_stride;
    a.out_f32 = 0;
    return launch_chosen(a, dev->cu_count, static_cast<hipStream_t>(stream));
}

int sg_skinny_gemm_rowcol(const uint8_t* A, const uint8_t* B, void* D, const float* scale_tensor, const float* row_scales,
                          const float* col_scales, int m, int n, int k, int b_stride, void* stream) {
    if (n % 2 != 0) return SG_N_NOT_EVEN;
    if (k % 16 != 0) return SG_K_NOT_DIVISIBLE_BY_WARPTILE_K;
    if (int rc = check_pointers(A, B, D, m, n, k, b_stride)) return rc;
    if ((reinterpret_cast<uintptr_t>(row_scales) | reinterpret_cast<uintptr_t>(col_scales)) & 3u) return SG_BAD_ALIGNMENT;
    DeviceInfo* dev;
    if (int rc = get_device_info(&dev)) return rc;
    StreamArgs a{};
    a.A = A; a.B = B; a.D = D; a.scale = scale_tensor;   // nullptr = 1.0f
    a.row_scale = row_scales;
    a.col_scale = col_scales;
    a.m = m; a.n = n; a.k = k; a.b_stride = b_stride;
    a.out_f32 = 0;
    return launch_chosen(a, dev->cu_count, static_cast<hipStream_t>(stream));
}

static void config_to_tuning(const Config& c, SgTuning* out) {
    out->engine = c.engine; out->split_k = c.split_k; out->waves = c.waves; out->row_tiles = c.rg; out->m_blocks = c.mt;
    out->depth = c.depth; out->k_chunks = c.ku; out->non_temporal = c.nt; out->persistent_wgs_per_cu = c.persist;
    out->wave_tiles = c.wavetile;
}

int sg_skinny_gemm_bf16act(const void* X_bf16, const uint8_t* B, void* D, const float* scale_tensor, const float* col_scales,
                           float* row_scales_out, int m, int n, int k, int b_stride, void* stream) {
    if (n % 2 != 0) return SG_N_NOT_EVEN;
    if (k % 16 != 0) return SG_K_NOT_DIVISIBLE_BY_WARPTILE_K;
    if (int rc = check_pointers(X_bf16, B, D, m, n, k, b_stride)) return rc;
    if ((reinterpret_cast<uintptr_t>(row_scales_out) | reinterpret_cast<uintptr_t>(col_scales)) & 3u) return SG_BAD_ALIGNMENT;
    DeviceInfo* dev;
    if (int rc = get_device_info(&dev)) return rc;
    hipStream_t st = static_cast<hipStream_t>(stream);
    StreamArgs a{};
    a.B = B; a.D = D; a.scale = scale_tensor;   // nullptr = 1.0f
    a.col_scale = col_scales;
    a.m = m; a.n = n; a.k = k; a.b_stride = b_stride;
    a.out_f32 = 0;
    Config c;
    if (pick_bf16act(m, n, k, dev->cu_count, &c)) {
        a.A16 = static_cast<const uint16_t*>(X_bf16);
        a.row_scale_out = row_scales_out;
        const int rc = launch_config(c, a, st);
        if (!rejected_before_launch(rc)) return rc;
        a.A16 = nullptr;
        a.row_scale_out = nullptr;
    }
    // two launches: the row encoder into the stream's scratch, then the GEMM with its scales in the epilogue
    uint8_t* scratch = nullptr;
    const size_t q_bytes = ((size_t)m * k + 255) & ~(size_t)255;
    if (int rc = get_act_scratch(st, q_bytes + (size_t)m * sizeof(float), &scratch)) return rc;
    float* scales = row_scales_out ? row_scales_out : reinterpret_cast<float*>(scratch + q_bytes);
    if (int rc = launch_fp8_encode_rows(X_bf16, scratch, scales, m, k, st)) return rc;
    a.A = scratch;
    a.row_scale = scales;
    return launch_chosen(a, dev->cu_count, st);
}

int sg_skinny_gemm_bf16act_tuned(const void* X_bf16, const uint8_t* B, void* D, const float* scale_tensor,
                                 const float* col_scales, float* row_scales_out, int m, int n, int k, int b_stride,
                                 const SgTuning* t, void* stream) {
    if (!t) return SG_BAD_ARGUMENT;
    if (n % 2 != 0) return SG_N_NOT_EVEN;
    if (k % 256 != 0) return SG_K_NOT_DIVISIBLE_BY_WARPTILE_K;
    if (int rc = check_pointers(X_bf16, B, D, m, n, k, b_stride)) return rc;
    if ((reinterpret_cast<uintptr_t>(row_scales_out) | reinterpret_cast<uintptr_t>(col_scales)) & 3u) return SG_BAD_ALIGNMENT;
    DeviceInfo* dev;
    if (int rc = get_device_info(&dev)) return rc;
    Config c;
    if (t->engine == ENGINE_AUTO) {
        if (!fused_config(m, k, &c)) return SG_INVALID_CONFIG;
    } else {
        c = config_from_tuning(*t);
        if (c.engine != ENGINE_LDS || (c.mt != 1 && c.mt != 2)) return SG_INVALID_CONFIG;
    }
    StreamArgs a{};
    a.A16 = static_cast<const uint16_t*>(X_bf16);
    a.row_scale_out = row_scales_out;
    a.B = B; a.D = D; a.scale = scale_tensor;
    a.col_scale = col_scales;
    a.m = m; a.n = n; a.k = k; a.b_stride = b_stride;
    a.out_f32 = 0;
    return launch_config(c, a, static_cast<hipStream_t>(stream));
}

int sg_skinny_gemm_bf16act_choice(int m, int n, int k, SgTuning* out, int* fused) {
    if (!out || m <= 0 || n <= 0 || k <= 0) return SG_BAD_ARGUMENT;
    DeviceInfo* dev;
    int cu = 256;
    if (get_device_info(&dev) == SG_SUCCESS) cu = dev->cu_count;
    Config c;
    if (pick_bf16act(m, n, k, cu, &c)) {
        config_to_tuning(c, out);
        if (fused) *fused = 1;
        return SG_SUCCESS;
    }
    if (fused) *fused = 0;
    return sg_skinny_gemm_choice(m, n, k, out, nullptr);
}

int sg_tuning_set(int m, int n, int k, const SgTuning* t) {
    if (m <= 0 || n <= 0 || k <= 0) return SG_BAD_ARGUMENT;
    ensure_default_table();
    std::lock_guard<std::mutex> lock(g_table_mutex);
    if (t) {
        if (t->engine != ENGINE_DIRECT && t->engine != ENGINE_LDS && t->engine != ENGINE_MID) return SG_INVALID_CONFIG;
        g_table[std::make_tuple(m, n, k)] = *t;
    } else {
        g_table.erase(std::make_tuple(m, n, k));
    }
    g_table_entries.store((int)g_table.size(), std::memory_order_relaxed);
    return SG_SUCCESS;
}

int sg_tuning_get(int m, int n, int k, SgTuning* out) {
    if (!out) return SG_BAD_ARGUMENT;
    return table_lookup(m, n, k, out) ? SG_SUCCESS : SG_INVALID_CONFIG;
}

int sg_tuning_count(void) {
    ensure_default_table();
    return g_table_entries.load(std::memory_order_relaxed);
}

int sg_tuning_clear(void) {
    ensure_default_table();
    std::lock_guard<std::mutex> lock(g_table_mutex);
    g_table.clear();
    g_table_entries.store(0, std::memory_order_relaxed);
    return SG_SUCCESS;
}

// File: first line "sgemm-tuning 1"; then one record per line, thirteen integers
//   m n k engine split_k waves row_tiles m_blocks depth k_chunks non_temporal persistent_wgs_per_cu wave_tiles
// '#' starts a comment; blank lines are skipped.
int sg_tuning_load(const char* path) {
    ensure_default_table();
    return sg_tuning_load_file(path);
}

}  // extern "C"

namespace sg {
static int sg_tuning_load_file(const char* path) {
    if (!path) return SG_BAD_ARGUMENT;
    FILE* f = std::fopen(path, "r");
    if (!f) return SG_BAD_ARGUMENT;
    std::map<std::tuple<int, int, int>, SgTuning> parsed;
    char line[512];
    bool header = false, ok = true;
    while (ok && std::fgets(line, sizeof line, f)) {
        char* hash = std::strchr(line, '#');
        if (hash) *hash = 0;
        char* p = line;
        while (*p == ' ' || *p == '\t' || *p == '\r' || *p == '\n') p++;
        if (!*p) continue;
        if (!header) {
            int version = 0;
            char tail = 0;
            ok = std::sscanf(p, "sgemm-tuning %d %c", &version, &tail) == 1 && version == 1;
            header = true;
            continue;
        }
        int v[13];
        char tail = 0;
        const int got = std::sscanf(p, "%d %d %d %d %d %d %d %d %d %d %d %d %d %c", &v[0], &v[1], &v[2], &v[3], &v[4], &v[5],
                                    &v[6], &v[7], &v[8], &v[9], &v[10], &v[11], &v[12], &tail);
        if (got != 13 || v[0] <= 0 || v[1] <= 0 || v[2] <= 0 ||
            (v[3] != ENGINE_DIRECT && v[3] != ENGINE_LDS && v[3] != ENGINE_MID)) {
            ok = false;
            break;
        }
        SgTuning t;
        t.engine = v[3]; t.split_k = v[4]; t.waves = v[5]; t.row_tiles = v[6]; t.m_blocks = v[7]; t.depth = v[8];
        t.k_chunks = v[9]; t.non_temporal = v[10]; t.persistent_wgs_per_cu = v[11]; t.wave_tiles = v[12];
        parsed[std::make_tuple(v[0], v[1], v[2])] = t;
    }
    std::fclose(f);
    if (!ok || !header) return SG_BAD_ARGUMENT;   // the table is left as it was
    std::lock_guard<std::mutex> lock(g_table_mutex);
    for (const auto& e : parsed) g_table[e.first] = e.second;
    g_table_entries.store((int)g_table.size(), std::memory_order_relaxed);
    return SG_SUCCESS;
}
}  // namespace sg

extern "C" {

int sg_tuning_save(const char* path) {
    if (!path) return SG_BAD_ARGUMENT;
    ensure_default_table();
    FILE* f = std::fopen(path, "w");
    if (!f) return SG_BAD_ARGUMENT;
    std::fprintf(f, "sgemm-tuning 1\n# m n k engine split_k waves row_tiles m_blocks depth k_chunks non_temporal "
                    "persistent_wgs_per_cu wave_tiles\n");
    {
        std::lock_guard<std::mutex> lock(g_table_mutex);
        for (const auto& e : g_table) {
            const SgTuning& t = e.second;
            std::fprintf(f, "%d %d %d %d %d %d %d %d %d %d %d %d %d\n", std::get<0>(e.first), std::get<1>(e.first),
                         std::get<2>(e.first), t.engine, t.split_k, t.waves, t.row_tiles, t.m_blocks, t.depth, t.k_chunks,
                         t.non_temporal, t.persistent_wgs_per_cu, t.wave_tiles);
        }
    }
    return std::fclose(f) == 0 ? SG_SUCCESS : SG_BAD_ARGUMENT;
}

int sg_skinny_gemm_fastpath(const uint8_t* A, const uint8_t* B, void* D, const float* scale_tensor, int m, int n,
                            int k) {
    return sg_skinny_gemm_auto(A, B, D, scale_tensor, m, n, k, k, nullptr);
}

// async_gemm: the producer/consumer ring with a fixed role split (as the reference's
// async_gemm_* launchers fix theirs in core.cu); shapes the ring cannot take stream directly.
static int async_gemm_common(const uint8_t* A, const uint8_t* B, void* D, int m, int n, int k, int out_f32) {
    if (k % 64 != 0) return SG_K_NOT_DIVISIBLE_BY_WARPTILE_K;
    if (int rc = check_pointers(A, B, D, m, n, k, k)) return rc;
    DeviceInfo* dev;
    if (int rc = get_device_info(&dev)) return rc;
    StreamArgs a{};
    a.A = A; a.B = B; a.D = D; a.scale = nullptr;
    a.m = m; a.n = n; a.k = k; a.b_stride = k;
    a.out_f32 = out_f32;
    if (k % 256 == 0) {
        RingConfig rc;
        rc.mt = m <= 16 ? 1 : 2;
        rc.b_lanes = 2;
        rc.qsize = 6;
        rc.a_producers = 1;
        rc.b_producers = 4;
        rc.consumers = 3;
        rc.nt = 1;
        return launch_ring(rc, a, nullptr);
    }
    const Config c = pick_config(m, n, k, dev->cu_count);
    return launch_config(c, a, nullptr);
}

int sg_async_gemm_f32(const uint8_t* A, const uint8_t* B, float* D, int m, int n, int k) {
    if (D && (reinterpret_cast<uintptr_t>(D) & 15u)) return SG_BAD_ALIGNMENT;
    return async_gemm_common(A, B, D, m, n, k, 1);
}

int sg_async_gemm_bf16(const uint8_t* A, const uint8_t* B, void* D, int m, int n, int k) {
    return async_gemm_common(A, B, D, m, n, k, 0);
}

int sg_sparse24_gemm(const uint8_t* A, const uint8_t* B_vals, const uint8_t* B_meta, void* D, const float* scale_tensor,
                     int m, int n, int k, void* stream) {
    if (n % 2 != 0) return SG_N_NOT_EVEN;
    if (!sparse_k_ok(k)) return SG_K_NOT_DIVISIBLE_BY_WARPTILE_K;
    if (!A || !B_vals || !B_meta || !D || !scale_tensor || m <= 0 || n <= 0 || k <= 0) return SG_BAD_ARGUMENT;
    if ((reinterpret_cast<uintptr_t>(A) | reinterpret_cast<uintptr_t>(B_vals) | reinterpret_cast<uintptr_t>(B_meta)) & 15u)
        return SG_BAD_ALIGNMENT;
    if (reinterpret_cast<uintptr_t>(D) & 7u) return SG_BAD_ALIGNMENT;
    DeviceInfo* dev;
    if (int rc = get_device_info(&dev)) return rc;
    const Config c = pick_sparse(m, n, k, dev->cu_count);
    StreamArgs a{};
    a.A = A; a.B = B_vals; a.D = D; a.scale = scale_tensor;
    a.m = m; a.n = n; a.k = k; a.b_stride = k / 2;
    a.out_f32 = 0;
    return launch_sparse_engine(c, a, B_meta, static_cast<hipStream_t>(stream));
}

int sg_sparse24_compress(const uint8_t* B, uint8_t* B_vals, uint8_t* B_meta, int n, int k, int b_stride, void* stream) {
    if (!B || !B_vals || !B_meta || n <= 0 || k <= 0 || b_stride < k) return SG_BAD_ARGUMENT;
    if (k % 16 != 0) return SG_K_NOT_DIVISIBLE_BY_WARPTILE_K;
    if ((reinterpret_cast<uintptr_t>(B) & 15u) || (b_stride & 15) || (reinterpret_cast<uintptr_t>(B_vals) & 7u) ||
        (reinterpret_cast<uintptr_t>(B_meta) & 1u))
        return SG_BAD_ALIGNMENT;
    DeviceInfo* dev;
    if (int rc = get_device_info(&dev)) return rc;
    return launch_sparse24_compress(B, B_vals, B_meta, n, k, b_stride, static_cast<hipStream_t>(stream));
}

int sg_sparse24_gemm_tuned(const uint8_t* A, const uint8_t* B_vals, const uint8_t* B_meta, void* D,
                           const float* scale_tensor, int m, int n, int k, const SgTuning* t, void* stream) {
    if (!t) return SG_BAD_ARGUMENT;
    if (n % 2 != 0) return SG_N_NOT_EVEN;
    if (!sparse_k_ok(k)) return SG_K_NOT_DIVISIBLE_BY_WARPTILE_K;
    if (!A || !B_vals || !B_meta || !D || !scale_tensor || m <= 0 || n <= 0 || k <= 0) return SG_BAD_ARGUMENT;
    if ((reinterpret_cast<uintptr_t>(A) | reinterpret_cast<uintptr_t>(B_vals) | reinterpret_cast<uintptr_t>(B_meta)) & 15u)
        return SG_BAD_ALIGNMENT;
    if (reinterpret_cast<uintptr_t>(D) & 7u) return SG_BAD_ALIGNMENT;
    DeviceInfo* dev;
    if (int rc = get_device_info(&dev)) return rc;
    Config c = pick_sparse(m, n, k, dev->cu_count);
    if (t->engine != ENGINE_AUTO) {
        c.rg = t->row_tiles;
        c.waves = t->waves;
        c.depth = t->depth;
        c.split_k = t->split_k;
        c.mt = t->m_blocks;
        c.persist = t->persistent_wgs_per_cu;
        c.wavetile = t->wave_tiles;
        c.ku = t->k_chunks;   // 1: metadata by 64-byte pieces per stage also where whole lines are possible
        if (c.mt != 1 && c.mt != 2) return SG_INVALID_CONFIG;
        if (c.wavetile != 0 && c.wavetile != 1) return SG_INVALID_CONFIG;
    }
    StreamArgs a{};
    a.A = A; a.B = B_vals; a.D = D; a.scale = scale_tensor;
    a.m = m; a.n = n; a.k = k; a.b_stride = k / 2;
    a.out_f32 = 0;
    return launch_sparse_engine(c, a, B_meta, static_cast<hipStream_t>(stream));
}

int sg_tiled_sum_reduce(const float* A, const float* B, float* D, int b, int m, int n, void* stream) {
    return launch_tiled_sum_reduce(A, B, D, b, m, n, static_cast<hipStream_t>(stream));
}

int sg_tiled_sum_reduce_async(const float* A, const float* B, float* D, int b, int m, int n, void* stream) {
    return launch_tiled_sum_reduce_ring(A, B, D, b, m, n, static_cast<hipStream_t>(stream));
}

int sg_fp8_encode_rows(const void* X, uint8_t* Q, float* scales, int rows, int cols, void* stream) {
    return launch_fp8_encode_rows(X, Q, scales, rows, cols, static_cast<hipStream_t>(stream));
}

int sg_fp8_decode_rows(const uint8_t* Q, const float* scales, void* Y, int rows, int cols, void* stream) {
    return launch_fp8_decode_rows(Q, scales, Y, rows, cols, static_cast<hipStream_t>(stream));
}

int sg_fp8_reduce_rows(const uint8_t* Q, const float* scales, void* Y, int nbuf, size_t q_buf_stride, int rows,
                       int cols, void* stream) {
    return launch_fp8_reduce_rows(Q, scales, Y, nbuf, q_buf_stride, rows, cols, static_cast<hipStream_t>(stream));
}

}  // extern "C"
