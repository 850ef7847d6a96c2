// One translation unit per SG_MT: instantiates the producer/consumer ring kernel for every
// compiled (B_LANES, XU) and exposes a launcher the dispatcher in sg_api.hip calls.
#include "sg_ring_kernel.h"
#include "sg_host.h"

#ifndef SG_MT
#error "compile with -DSG_MT=<1|2>"
#endif

namespace sg {

template <int BL, int XU>
static int launch_one(int nt, const RingArgs& ra, unsigned grid, unsigned threads, size_t lds, hipStream_t stream) {
    auto kernel = nt ? ring_gemm_kernel<SG_MT, BL, XU, true> : ring_gemm_kernel<SG_MT, BL, XU, false>;
    static LdsGranted granted[2];
    if (int rc = request_dynamic_lds(reinterpret_cast<const void*>(kernel), lds, granted[nt ? 1 : 0])) return rc;
    kernel<<<dim3(grid), dim3(threads), lds, stream>>>(ra);
    return report_hip("ring_gemm_kernel launch", hipGetLastError()) == hipSuccess ? SG_SUCCESS : SG_LAUNCH_FAILED;
}

#define SG_CASE(BL_, XU_) \
    if (bl == BL_ && xu == XU_) return launch_one<BL_, XU_>(nt, ra, grid, threads, lds, stream);

int SG_RING_LAUNCHER(SG_MT)(int bl, int xu, int nt, const RingArgs& ra, unsigned grid, unsigned threads, size_t lds,
                            hipStream_t stream) {
#if SG_MT == 1
    SG_CASE(1, 1) SG_CASE(1, 2) SG_CASE(1, 4) SG_CASE(2, 1) SG_CASE(2, 2) SG_CASE(2, 4) SG_CASE(3, 1) SG_CASE(3, 2)
    SG_CASE(3, 4) SG_CASE(4, 1) SG_CASE(4, 2) SG_CASE(4, 4) SG_CASE(5, 1) SG_CASE(5, 2) SG_CASE(5, 4) SG_CASE(6, 1)
    SG_CASE(6, 2) SG_CASE(6, 4)
#else
    SG_CASE(1, 8) SG_CASE(2, 8) SG_CASE(3, 8) SG_CASE(4, 8) SG_CASE(5, 8) SG_CASE(6, 8)
#endif
    return SG_INVALID_CONFIG;
}

}  // namespace sg
