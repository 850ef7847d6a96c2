// One translation unit per (SG_MT, SG_RG): instantiates the LDS-ring kernel for every
// compiled (XU, DEPTH, NT) and exposes a launcher the dispatcher in sg_api.hip calls.
#include "sg_lds_kernel.h"
#include "sg_host.h"

#ifndef SG_MT
#error "compile with -DSG_MT=<1|2> -DSG_RG=<1|2|4>"
#endif

namespace sg {

template <int XU, int DEPTH, bool NT, int MODE>
static int launch_one(const StreamArgs& a, unsigned grid, unsigned threads, size_t lds, hipStream_t stream) {
    constexpr int bound = MODE == 4 ? kQuantThreads : ((MODE == 0 || MODE == 5) ? lds_launch_bound(SG_MT, SG_RG) : lds_persistent_launch_bound(SG_MT, SG_RG));
    if (threads > (unsigned)bound) return SG_INVALID_CONFIG;
    void (*kernel)(const StreamArgs) = nullptr;
    if constexpr (MODE == 4) kernel = lds_gemm_persistent_kernel<SG_MT, SG_RG, XU, DEPTH, NT, true, true>;
    else if constexpr (MODE == 5) kernel = (a.k & 255) ? lds_gemm_kernel<SG_MT, SG_RG, XU, DEPTH, NT, true, true>
                                                        : lds_gemm_kernel<SG_MT, SG_RG, XU, DEPTH, NT, true>;
    else if constexpr (MODE == 2) kernel = (a.k & 255) ? lds_gemm_wavetile_kernel<SG_MT, SG_RG, XU, DEPTH, NT, true>
                                                        : lds_gemm_wavetile_kernel<SG_MT, SG_RG, XU, DEPTH, NT>;
    else if constexpr (MODE == 3) kernel = lds_gemm_persistent_kernel<SG_MT, SG_RG, XU, DEPTH, NT, true>;
    else if constexpr (MODE == 1) kernel = lds_gemm_persistent_kernel<SG_MT, SG_RG, XU, DEPTH, NT, false>;
    else kernel = (a.k & 255) ? lds_gemm_kernel<SG_MT, SG_RG, XU, DEPTH, NT, false, true>   // half a block at the end of K
                              : lds_gemm_kernel<SG_MT, SG_RG, XU, DEPTH, NT>;
    static LdsGranted granted[2];
    if (int rc = request_dynamic_lds(reinterpret_cast<const void*>(kernel), lds, granted[(a.k & 255) ? 1 : 0])) return rc;
    kernel<<<dim3(grid), dim3(threads), lds, stream>>>(a);
    return report_hip("lds_gemm_kernel launch", hipGetLastError()) == hipSuccess ? SG_SUCCESS : SG_LAUNCH_FAILED;
}

#define SG_CASE(XU_, DEPTH_)                                                                    \
    if (xu == XU_ && depth == DEPTH_) {                                                         \
        if constexpr (XU_ <= 4 * SG_MT && (SG_MT == 1 || XU_ > 4)) {                            \
            if (mode == 5) { /* 24-row tiles: two fragments, six weight instructions per stage */ \
                if constexpr (SG_RG == 2 && (DEPTH_ - 1) * (6 + XU_) <= 63)                     \
                    return nt ? launch_one<XU_, DEPTH_, true, 5>(a, grid, threads, lds, stream) \
                              : launch_one<XU_, DEPTH_, false, 5>(a, grid, threads, lds, stream); \
                else                                                                            \
                    return SG_INVALID_CONFIG;                                                   \
            }                                                                                   \
            if (mode == 4) { /* bf16 activations quantised in the kernel: one row tile per wave, two slots */ \
                if constexpr (SG_RG == 1 && DEPTH_ == 2)                                        \
                    return nt ? launch_one<XU_, DEPTH_, true, 4>(a, grid, threads, lds, stream) \
                              : launch_one<XU_, DEPTH_, false, 4>(a, grid, threads, lds, stream); \
                else                                                                            \
                    return SG_INVALID_CONFIG;                                                   \
            }                                                                                   \
            if (mode == 2 || mode == 3) {                                                       \
                if constexpr ((DEPTH_ - 1) * (SG_RG * 4) <= 63) {                               \
                    if (mode == 3)                                                              \
                        return nt ? launch_one<XU_, DEPTH_, true, 3>(a, grid, threads, lds, stream) \
                                  : launch_one<XU_, DEPTH_, false, 3>(a, grid, threads, lds, stream); \
                    return nt ? launch_one<XU_, DEPTH_, true, 2>(a, grid, threads, lds, stream) \
                              : launch_one<XU_, DEPTH_, false, 2>(a, grid, threads, lds, stream); \
                } else {                                                                        \
                    return SG_INVALID_CONFIG;                                                   \
                }                                                                               \
            }                                                                                   \
            if constexpr ((DEPTH_ - 1) * (SG_RG * 4 + XU_) <= 63) {                             \
                if (mode == 1)                                                                  \
                    return nt ? launch_one<XU_, DEPTH_, true, 1>(a, grid, threads, lds, stream) \
                              : launch_one<XU_, DEPTH_, false, 1>(a, grid, threads, lds, stream); \
                return nt ? launch_one<XU_, DEPTH_, true, 0>(a, grid, threads, lds, stream)     \
                          : launch_one<XU_, DEPTH_, false, 0>(a, grid, threads, lds, stream);   \
            } else {                                                                            \
                return SG_INVALID_CONFIG;                                                       \
            }                                                                                   \
        } else {                                                                                \
            return SG_INVALID_CONFIG;                                                           \
        }                                                                                       \
    }

int SG_LDS_LAUNCHER(SG_MT, SG_RG)(int xu, int depth, int nt, int mode, const StreamArgs& a, unsigned grid, unsigned threads,
                                  size_t lds, hipStream_t stream) {
#if SG_MT == 1
    SG_CASE(1, 2) SG_CASE(1, 3) SG_CASE(1, 4) SG_CASE(1, 6) SG_CASE(1, 8)
    SG_CASE(2, 2) SG_CASE(2, 3) SG_CASE(2, 4) SG_CASE(2, 6) SG_CASE(2, 8)
    SG_CASE(4, 2) SG_CASE(4, 3) SG_CASE(4, 4) SG_CASE(4, 6) SG_CASE(4, 8)
#else
    SG_CASE(8, 2) SG_CASE(8, 3) SG_CASE(8, 4) SG_CASE(8, 6) SG_CASE(8, 8)
#endif
    return SG_INVALID_CONFIG;
}

}  // namespace sg
