// Instantiations of the LDS-tiled kernel: per-tensor scales, dense rows.
#include "fp8_gemm_tile.h"
#include "fp8_gemm_tile_deep.h"
#include "tg_host.h"

namespace tg {

hipError_t run_tile_per_tensor(int bm, int bn, bool split, const GemmParams& p, int gx, int gy, hipStream_t s) {
#define TG_CASE(BM, BN, WGM, WGN)                                                               \
    if (bm == BM && bn == BN) {                                                                  \
        return split ? launch_tile<BM, BN, WGM, WGN, false, GROUP_DENSE, true>(p, gx, gy, s)     \
                     : launch_tile<BM, BN, WGM, WGN, false, GROUP_DENSE, false>(p, gx, gy, s);   \
    }
    TG_CASE(256, 256, 4, 2)
    TG_CASE(128, 128, 2, 2)
    TG_CASE(128, 256, 2, 4)
    TG_CASE(64, 128, 1, 4)
#undef TG_CASE
    return hipErrorInvalidConfiguration;
}

hipError_t run_tile_deep(bool split, const GemmParams& p, int gx, int gy, hipStream_t s) {
    return split ? launch_tile_deep<true>(p, gx, gy, s) : launch_tile_deep<false>(p, gx, gy, s);
}

}  // namespace tg
