// Host-side declarations shared by the translation units of libsgemm.so.
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include <atomic>
#include <mutex>

#include "../../include/sgemm.h"

namespace sg {

struct StreamArgs;

#define SG_CAT_(a, b, c) a##b##_##c
#define SG_CAT(a, b, c) SG_CAT_(a, b, c)
#define SG_STREAM_LAUNCHER(MT, RG) SG_CAT(launch_stream_, MT, RG)

#define SG_DECL_STREAM(MT, RG)                                                                       \
    int SG_STREAM_LAUNCHER(MT, RG)(int ku, int depth, const StreamArgs& a, unsigned grid, unsigned threads, \
                                   size_t lds, hipStream_t stream);
SG_DECL_STREAM(1, 1) SG_DECL_STREAM(1, 2) SG_DECL_STREAM(1, 3) SG_DECL_STREAM(1, 4)
SG_DECL_STREAM(2, 1) SG_DECL_STREAM(2, 2) SG_DECL_STREAM(2, 3) SG_DECL_STREAM(2, 4)

#define SG_CAT_LDS_(a, b, c) a##b##_##c
#define SG_CAT_LDS(a, b, c) SG_CAT_LDS_(a, b, c)
#define SG_LDS_LAUNCHER(MT, RG) SG_CAT_LDS(launch_lds_, MT, RG)
#define SG_DECL_LDS(MT, RG)                                                                              \
    int SG_LDS_LAUNCHER(MT, RG)(int xu, int depth, int nt, int mode, const StreamArgs& a, unsigned grid, unsigned threads, \
                                size_t lds, hipStream_t stream);
SG_DECL_LDS(1, 1) SG_DECL_LDS(1, 2) SG_DECL_LDS(1, 4) SG_DECL_LDS(2, 1) SG_DECL_LDS(2, 2) SG_DECL_LDS(2, 4)

struct RingArgs;
#define SG_RING_CAT_(a, b) a##b
#define SG_RING_CAT(a, b) SG_RING_CAT_(a, b)
#define SG_RING_LAUNCHER(MT) SG_RING_CAT(launch_ring_, MT)
int SG_RING_LAUNCHER(1)(int bl, int xu, int nt, const RingArgs& ra, unsigned grid, unsigned threads, size_t lds,
                        hipStream_t stream);
int SG_RING_LAUNCHER(2)(int bl, int xu, int nt, const RingArgs& ra, unsigned grid, unsigned threads, size_t lds,
                        hipStream_t stream);

// persistent LDS ring with the activations resident in registers: pt K blocks per wave and tile
int launch_xreg(int mt, int rg, int pt, int depth, const StreamArgs& a, unsigned grid, unsigned threads, size_t lds,
                hipStream_t stream);
int launch_mid(int rgw, int mh, int depth, int dx, int wn, const StreamArgs& a, unsigned grid, size_t lds, hipStream_t stream);
// second launch of a mid-batch GEMM with StreamArgs::defer_reduce: sums the split-K partials of every output fragment
int launch_mid_reduce(int rgw, int mh, int wn, const StreamArgs& a, hipStream_t stream);

struct SparseArgs;
int launch_sparse(int mt, int rg, int xu2, int depth, bool pairs, const SparseArgs& sa, unsigned grid, unsigned threads,
                  size_t lds, hipStream_t stream);
int launch_sparse_wavetile(int rg, int xu2, int depth, bool pairs, const SparseArgs& sa, unsigned grid, unsigned threads,
                           size_t lds, hipStream_t stream);

// Prints a HIP failure to stderr when the environment variable SG_VERBOSE is set; returns e.
hipError_t report_hip(const char* what, hipError_t e);

// Dynamic LDS above the 48 KB default has to be requested per kernel and device.  `granted` (one array per
// kernel, indexed by device, zero-initialised static storage) remembers the largest request already made, so
// that the launch path normally makes no runtime call here.  Raising the limit is serialised: a smaller request
// that overtook a larger one would otherwise lower the attribute under the larger one's launch.
typedef std::atomic<size_t> LdsGranted[16];
inline int request_dynamic_lds(const void* kernel, size_t lds, LdsGranted& granted) {
    if (lds <= 48 * 1024) return SG_SUCCESS;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 16) return SG_NO_DEVICE;
    if (granted[dev].load(std::memory_order_acquire) >= lds) return SG_SUCCESS;
    static std::mutex raise;
    std::lock_guard<std::mutex> lock(raise);
    if (granted[dev].load(std::memory_order_relaxed) >= lds) return SG_SUCCESS;
    if (report_hip("hipFuncSetAttribute",
                   hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds)) != hipSuccess) {
        (void)hipGetLastError();
        return SG_LAUNCH_FAILED;
    }
    granted[dev].store(lds, std::memory_order_release);
    return SG_SUCCESS;
}

// Split-K workspace: fp32 partial fragments and one arrival counter per output tile.
struct Workspace {
    float* partials = nullptr;
    unsigned* counters = nullptr;
    size_t partial_bytes = 0;
    size_t n_counters = 0;
};
// The workspace of `stream` on the current device, created or grown on demand; *out is a copy.
int get_workspace(hipStream_t stream, size_t partial_bytes, size_t n_counters, Workspace* out);

// Device facts queried once per device.
struct DeviceInfo {
    int cu_count = 0;
    int lds_per_block = 0;
    bool is_gfx950 = false;
};
int get_device_info(DeviceInfo** out);

}  // namespace sg
