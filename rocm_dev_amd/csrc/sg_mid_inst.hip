// Instantiates the mid-batch kernel for every compiled (RGW, MH, DEPTH) and exposes the
// launcher the dispatcher in sg_api.hip calls.
#include "sg_mid_kernel.h"
#include "sg_host.h"

namespace sg {

template <int RGW, int MH, int DEPTH, int WN, int DX = DEPTH, bool TAIL = false>
static int launch_one(const StreamArgs& a, unsigned grid, size_t lds, hipStream_t stream) {
    auto kernel = mid_gemm_kernel<RGW, MH, DEPTH, WN, DX, TAIL>;
    static LdsGranted granted;
    if (int rc = request_dynamic_lds(reinterpret_cast<const void*>(kernel), lds, granted)) return rc;
    kernel<<<dim3(grid), dim3(WN * 128), lds, stream>>>(a);
    return report_hip("mid_gemm_kernel launch", hipGetLastError()) == hipSuccess ? SG_SUCCESS : SG_LAUNCH_FAILED;
}

#define SG_CASE(RGW_, MH_, DEPTH_)                                                             \
    if (rgw == RGW_ && mh == MH_ && depth == DEPTH_ && dx == DEPTH_) {                         \
        if (wn == 2) {                                                                         \
            if constexpr ((DEPTH_ - 2) * (RGW_ + MH_) <= 63)                                   \
                return launch_one<RGW_, MH_, DEPTH_, 2>(a, grid, lds, stream);                 \
            else                                                                               \
                return SG_INVALID_CONFIG;                                                      \
        }                                                                                      \
        if (wn == 4) return launch_one<RGW_, MH_, DEPTH_, 4>(a, grid, lds, stream);            \
        return SG_INVALID_CONFIG;                                                              \
    }
// eight-wave tiles with a shallower activation ring (dx < depth)
#define SG_CASE_DX(RGW_, MH_, DEPTH_, DX_)                                                     \
    if (rgw == RGW_ && mh == MH_ && depth == DEPTH_ && dx == DX_ && wn == 4)                   \
        return launch_one<RGW_, MH_, DEPTH_, 4, DX_>(a, grid, lds, stream);

// fourteen-wave workgroups (7 along n x 2 along m): 224-row tiles
#define SG_CASE_7(MH_, DEPTH_, DX_)                                                            \
    if (rgw == 2 && mh == MH_ && depth == DEPTH_ && dx == DX_ && wn == 7)                      \
        return launch_one<2, MH_, DEPTH_, 7, DX_>(a, grid, lds, stream);

// k not a multiple of 128: the tiles and rings the heuristics choose (pick_mid), built with the partial last block
#define SG_TAIL(RGW_, MH_, DEPTH_, WN_, DX_)                                                   \
    if (rgw == RGW_ && mh == MH_ && depth == DEPTH_ && dx == DX_ && wn == WN_)                 \
        return launch_one<RGW_, MH_, DEPTH_, WN_, DX_, true>(a, grid, lds, stream);

static int launch_mid_tail(int rgw, int mh, int depth, int dx, int wn, const StreamArgs& a, unsigned grid, size_t lds,
                           hipStream_t stream) {
    SG_TAIL(2, 2, 4, 2, 4) SG_TAIL(2, 4, 4, 2, 4)                          // 64 x 64, 64 x 128 on four waves
    SG_TAIL(2, 2, 4, 4, 4) SG_TAIL(2, 4, 4, 4, 4) SG_TAIL(2, 8, 3, 4, 3)   // 128 x 64, 128 x 128, 128 x 256
    SG_TAIL(2, 2, 4, 4, 2)                                                 // two 128 x 64 workgroups per CU
    SG_TAIL(4, 2, 4, 4, 4) SG_TAIL(4, 2, 3, 4, 3) SG_TAIL(4, 4, 3, 4, 3)   // 256 x 64 (unsplit, split), 256 x 128
    SG_TAIL(4, 8, 3, 4, 2) SG_TAIL(4, 8, 2, 4, 2)                          // 256 x 256 (unsplit, split)
    SG_TAIL(2, 2, 4, 7, 4) SG_TAIL(2, 4, 4, 7, 3) SG_TAIL(2, 8, 3, 7, 2)   // 224 x 64, 224 x 128, 224 x 256
    return SG_K_NOT_DIVISIBLE_BY_WARPTILE_K;
}

int launch_mid_reduce(int rgw, int mh, int wn, const StreamArgs& a, hipStream_t stream) {
    const int frags_wg = 2 * wn * rgw * mh;                    // fragments of a tile; a workgroup of four waves takes 4 * kReduceFrags
    if ((rgw * mh) % kReduceFrags != 0) return SG_INVALID_CONFIG;
    const size_t grid = (size_t)a.n_tiles * a.m_tiles * ((frags_wg + 4 * kReduceFrags - 1) / (4 * kReduceFrags));
    if (grid == 0 || grid > 0x7fffffffu) return SG_BAD_ARGUMENT;
    mid_reduce_kernel<<<dim3((unsigned)grid), dim3(256), 0, stream>>>(a, rgw, mh, wn);
    return report_hip("mid_reduce_kernel launch", hipGetLastError()) == hipSuccess ? SG_SUCCESS : SG_LAUNCH_FAILED;
}

int launch_mid(int rgw, int mh, int depth, int dx, int wn, const StreamArgs& a, unsigned grid, size_t lds, hipStream_t stream) {
    if (a.k & 127) return launch_mid_tail(rgw, mh, depth, dx, wn, a, grid, lds, stream);
    SG_CASE_7(8, 3, 2) SG_CASE_7(8, 2, 2)                                       // 224 x 256: 84 + 64 KB
    SG_CASE_7(4, 4, 2) SG_CASE_7(4, 4, 3) SG_CASE_7(4, 3, 3) SG_CASE_7(4, 3, 2)  // 224 x 128
    SG_CASE_7(2, 4, 2) SG_CASE_7(2, 4, 4) SG_CASE_7(2, 3, 3)                     // 224 x 64
    if (wn == 7) return SG_INVALID_CONFIG;
    SG_CASE(2, 2, 2) SG_CASE(2, 2, 3) SG_CASE(2, 2, 4) SG_CASE(2, 2, 6)
    SG_CASE(2, 4, 2) SG_CASE(2, 4, 3) SG_CASE(2, 4, 4) SG_CASE(2, 4, 6)
    SG_CASE(2, 8, 2) SG_CASE(2, 8, 3) SG_CASE(2, 8, 4)
    SG_CASE(4, 2, 2) SG_CASE(4, 2, 3) SG_CASE(4, 2, 4) SG_CASE(4, 2, 6)
    SG_CASE(4, 4, 2) SG_CASE(4, 4, 3) SG_CASE(4, 4, 4)
    SG_CASE(4, 8, 2) SG_CASE(4, 8, 3)
    SG_CASE_DX(4, 8, 3, 2)                                            // 256 x 256: 96 + 64 KB
    SG_CASE_DX(4, 4, 4, 2) SG_CASE_DX(4, 4, 4, 3) SG_CASE_DX(4, 4, 3, 2)   // 256 x 128
    SG_CASE_DX(4, 2, 4, 2) SG_CASE_DX(4, 2, 4, 3)                     // 256 x 64
    SG_CASE_DX(2, 8, 4, 2) SG_CASE_DX(2, 8, 3, 2) SG_CASE_DX(2, 8, 6, 2)   // 128 x 256
    SG_CASE_DX(2, 4, 6, 2) SG_CASE_DX(2, 4, 6, 3) SG_CASE_DX(2, 4, 4, 2)   // 128 x 128
    SG_CASE_DX(2, 2, 6, 2) SG_CASE_DX(2, 2, 6, 3) SG_CASE_DX(2, 2, 4, 2)   // 128 x 64
    return SG_INVALID_CONFIG;
}

}  // namespace sg
