// Instantiates the 2:4 sparse kernel for every compiled (MT, RG, XU2, DEPTH) and exposes the
// launcher the dispatcher in sg_api.hip calls.
#include "sg_sparse_kernel.h"
#include "sg_host.h"

namespace sg {

template <int MT, int RG, int XU2, int DEPTH, bool TAIL, bool PAIRS>
static int launch_one(const SparseArgs& sa, unsigned grid, unsigned threads, size_t lds, hipStream_t stream) {
    if (threads > (unsigned)sparse_launch_bound(MT, RG)) return SG_INVALID_CONFIG;
    if (lds < (size_t)(threads / 64) * sparse_wave_bytes(RG, XU2, DEPTH, PAIRS)) return SG_INVALID_CONFIG;
    auto kernel = sparse24_gemm_kernel<MT, RG, XU2, DEPTH, TAIL, PAIRS>;
    static LdsGranted granted;
    if (int rc = request_dynamic_lds(reinterpret_cast<const void*>(kernel), lds, granted)) return rc;
    kernel<<<dim3(grid), dim3(threads), lds, stream>>>(sa);
    return report_hip("sparse24_gemm_kernel launch", hipGetLastError()) == hipSuccess ? SG_SUCCESS : SG_LAUNCH_FAILED;
}

#define SG_CASE(MT_, RG_, XU2_, DEPTH_)                                                     \
    if (mt == MT_ && rg == RG_ && xu2 == XU2_ && depth == DEPTH_) {                          \
        if constexpr ((DEPTH_ - 1) * (RG_ * 5 + XU2_) <= 63)                                \
            return tail    ? launch_one<MT_, RG_, XU2_, DEPTH_, true, false>(sa, grid, threads, lds, stream)   \
                   : pairs ? launch_one<MT_, RG_, XU2_, DEPTH_, false, true>(sa, grid, threads, lds, stream)   \
                           : launch_one<MT_, RG_, XU2_, DEPTH_, false, false>(sa, grid, threads, lds, stream); \
        else                                                                                \
            return SG_INVALID_CONFIG;                                                       \
    }
#define SG_DEPTHS(MT_, RG_, XU2_) SG_CASE(MT_, RG_, XU2_, 2) SG_CASE(MT_, RG_, XU2_, 3) SG_CASE(MT_, RG_, XU2_, 4) SG_CASE(MT_, RG_, XU2_, 6)

// k % 512 != 0 (a multiple of 128 beyond 512) runs the builds with a partly used last stage; `pairs` (k % 1024 == 0,
// at most k / 1024 K splits, `lds` sized with sparse_wave_bytes(..., true)) the builds that fetch the metadata by whole
// cache lines
int launch_sparse(int mt, int rg, int xu2, int depth, bool pairs, const SparseArgs& sa, unsigned grid, unsigned threads,
                  size_t lds, hipStream_t stream) {
    const bool tail = (sa.g.k & 511) != 0;
    if (pairs && ((sa.g.k & 1023) != 0 || sa.g.split_k > (sa.g.k >> 10))) return SG_INVALID_CONFIG;
    SG_DEPTHS(1, 1, 2) SG_DEPTHS(1, 1, 4) SG_DEPTHS(1, 1, 8)
    SG_DEPTHS(1, 2, 2) SG_DEPTHS(1, 2, 4) SG_DEPTHS(1, 2, 8)
    SG_DEPTHS(1, 4, 2) SG_DEPTHS(1, 4, 4) SG_DEPTHS(1, 4, 8)
    SG_DEPTHS(2, 1, 16) SG_DEPTHS(2, 2, 16) SG_DEPTHS(2, 4, 16)
    return SG_INVALID_CONFIG;
}

template <int RG, int XU2, int DEPTH, bool TAIL, bool PAIRS>
static int launch_wavetile(const SparseArgs& sa, unsigned grid, unsigned threads, size_t lds, hipStream_t stream) {
    if (threads > (RG == 4 ? 512u : 1024u)) return SG_INVALID_CONFIG;
    const size_t stages = (size_t)((sa.g.k + 511) >> 9);
    if (lds < stages * XU2 * 1024 + (size_t)(threads / 64) * sparse_wave_bytes(RG, 0, DEPTH, PAIRS)) return SG_INVALID_CONFIG;
    auto kernel = sparse24_gemm_wavetile_kernel<RG, XU2, DEPTH, TAIL, PAIRS>;
    static LdsGranted granted;
    if (int rc = request_dynamic_lds(reinterpret_cast<const void*>(kernel), lds, granted)) return rc;
    kernel<<<dim3(grid), dim3(threads), lds, stream>>>(sa);
    return report_hip("sparse24_gemm_wavetile_kernel launch", hipGetLastError()) == hipSuccess ? SG_SUCCESS : SG_LAUNCH_FAILED;
}

#define SG_WT_CASE(RG_, XU2_, DEPTH_)                                                                  \
    if (rg == RG_ && xu2 == XU2_ && depth == DEPTH_)                                                   \
        return tail    ? launch_wavetile<RG_, XU2_, DEPTH_, true, false>(sa, grid, threads, lds, stream)   \
               : pairs ? launch_wavetile<RG_, XU2_, DEPTH_, false, true>(sa, grid, threads, lds, stream)   \
                       : launch_wavetile<RG_, XU2_, DEPTH_, false, false>(sa, grid, threads, lds, stream);
#define SG_WT_DEPTHS(RG_, XU2_) SG_WT_CASE(RG_, XU2_, 2) SG_WT_CASE(RG_, XU2_, 3) SG_WT_CASE(RG_, XU2_, 4) SG_WT_CASE(RG_, XU2_, 6)

// wave-per-tile kernel with the activations resident in LDS (at most 16 activation rows)
int launch_sparse_wavetile(int rg, int xu2, int depth, bool pairs, const SparseArgs& sa, unsigned grid, unsigned threads,
                           size_t lds, hipStream_t stream) {
    const bool tail = (sa.g.k & 511) != 0;
    if (pairs && (sa.g.k & 1023) != 0) return SG_INVALID_CONFIG;
    SG_WT_DEPTHS(1, 2) SG_WT_DEPTHS(1, 4) SG_WT_DEPTHS(1, 8)
    SG_WT_DEPTHS(2, 2) SG_WT_DEPTHS(2, 4) SG_WT_DEPTHS(2, 8)
    return SG_INVALID_CONFIG;
}

}  // namespace sg
