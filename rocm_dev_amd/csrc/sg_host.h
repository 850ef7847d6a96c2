// Host-side declarations shared by the translation units of libsgemm.so.
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

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

// Split-K workspace of the current device (created on first use).
struct Workspace {
    float* partials = nullptr;
    unsigned* counters = nullptr;
    size_t partial_bytes = 0;
    size_t n_counters = 0;
};
int get_workspace(Workspace** out);

// Device facts queried once per device.
struct DeviceInfo {
    int cu_count = 0;
    int lds_per_block = 0;
    bool is_gfx950 = false;
};
int get_device_info(DeviceInfo** out);

}  // namespace sg
