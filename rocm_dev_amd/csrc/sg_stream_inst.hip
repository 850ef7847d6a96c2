// One translation unit per (SG_MT, SG_RG): instantiates the streaming kernel for every
// compiled (KU, DEPTH) and exposes a launcher the dispatcher in sg_api.hip calls.
#include "sg_stream_kernel.h"
#include "sg_host.h"

#ifndef SG_MT
#error "compile with -DSG_MT=<1|2> -DSG_RG=<1..4>"
#endif

namespace sg {

template <int KU, int DEPTH>
static int launch_one(const StreamArgs& a, unsigned grid, unsigned threads, size_t lds, hipStream_t stream) {
    if (threads > (unsigned)stream_launch_bound(SG_MT, SG_RG, KU, DEPTH)) return SG_INVALID_CONFIG;
    stream_gemm_kernel<SG_MT, SG_RG, KU, DEPTH><<<dim3(grid), dim3(threads), lds, stream>>>(a);
    return hipGetLastError() == hipSuccess ? SG_SUCCESS : SG_LAUNCH_FAILED;
}

#define SG_CASE(KU_, DEPTH_)                                                              \
    if (ku == KU_ && depth == DEPTH_) {                                                   \
        if constexpr (stream_regs(SG_MT, SG_RG, KU_, DEPTH_) <= 500)                      \
            return launch_one<KU_, DEPTH_>(a, grid, threads, lds, stream);                \
        else                                                                              \
            return SG_INVALID_CONFIG;                                                     \
    }

int SG_STREAM_LAUNCHER(SG_MT, SG_RG)(int ku, int depth, const StreamArgs& a, unsigned grid, unsigned threads,
                                     size_t lds, hipStream_t stream) {
    SG_CASE(1, 1) SG_CASE(1, 2) SG_CASE(1, 3) SG_CASE(1, 4) SG_CASE(1, 6) SG_CASE(1, 8)
    SG_CASE(2, 1) SG_CASE(2, 2) SG_CASE(2, 3) SG_CASE(2, 4) SG_CASE(2, 6)
    SG_CASE(4, 1) SG_CASE(4, 2) SG_CASE(4, 3) SG_CASE(4, 4)
    SG_CASE(8, 1) SG_CASE(8, 2) SG_CASE(8, 3) SG_CASE(8, 4)
    return SG_INVALID_CONFIG;
}

}  // namespace sg
