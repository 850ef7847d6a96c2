// Instantiates the register-resident-activation persistent kernel and exposes its launcher.
#include "sg_xreg_kernel.h"
#include "sg_host.h"

namespace sg {

template <int MT, int RG, int PT, int DEPTH>
static int launch_one(const StreamArgs& a, unsigned grid, unsigned threads, size_t lds, hipStream_t stream) {
    if (threads > (unsigned)xreg_launch_bound(MT, RG, PT)) return SG_INVALID_CONFIG;
    auto kernel = lds_gemm_xreg_kernel<MT, RG, PT, DEPTH, true>;
    static LdsGranted granted;
    if (int rc = request_dynamic_lds(reinterpret_cast<const void*>(kernel), lds, granted)) return rc;
    kernel<<<dim3(grid), dim3(threads), lds, stream>>>(a);
    return report_hip("lds_gemm_xreg_kernel launch", hipGetLastError()) == hipSuccess ? SG_SUCCESS : SG_LAUNCH_FAILED;
}

#define SG_CASE(MT_, RG_, PT_, DEPTH_) \
    if (mt == MT_ && rg == RG_ && pt == PT_ && depth == DEPTH_) return launch_one<MT_, RG_, PT_, DEPTH_>(a, grid, threads, lds, stream);
#define SG_DEPTHS(MT_, RG_, PT_) SG_CASE(MT_, RG_, PT_, 2) SG_CASE(MT_, RG_, PT_, 3) SG_CASE(MT_, RG_, PT_, 4)

int launch_xreg(int mt, int rg, int pt, int depth, const StreamArgs& a, unsigned grid, unsigned threads, size_t lds,
                hipStream_t stream) {
    SG_DEPTHS(1, 1, 1) SG_DEPTHS(1, 1, 2) SG_DEPTHS(1, 1, 4)
    SG_DEPTHS(1, 2, 1) SG_DEPTHS(1, 2, 2) SG_DEPTHS(1, 2, 4)
    SG_DEPTHS(2, 1, 1) SG_DEPTHS(2, 1, 2)
    SG_DEPTHS(2, 2, 1) SG_DEPTHS(2, 2, 2)
    return SG_INVALID_CONFIG;
}

}  // namespace sg
