// Instantiations of the LDS-tiled kernel: block scales, expert-grouped rows (ragged segments or
// token gather).
#include "fp8_gemm_tile.h"
#include "tg_host.h"

namespace tg {

hipError_t run_tile_block_grouped(int bm, int bn, int group, const GemmParams& p, int gx, hipStream_t s) {
#define TG_CASE(BM, BN, WGM, WGN)                                                               \
    if (bm == BM && bn == BN) {                                                                  \
        return group == GROUP_RAGGED                                                             \
                   ? launch_tile<BM, BN, WGM, WGN, true, GROUP_RAGGED, false>(p, gx, 1, s)       \
                   : launch_tile<BM, BN, WGM, WGN, true, GROUP_GATHER, false>(p, gx, 1, s);      \
    }
    TG_CASE(256, 256, 4, 2)
    TG_CASE(128, 128, 2, 2)
    TG_CASE(128, 256, 2, 4)
    TG_CASE(64, 128, 1, 4)
#undef TG_CASE
    return hipErrorInvalidConfiguration;
}

// Gate/up MoE GEMM with the SiLU-multiply-quantize epilogue (a tile is 128 gate + 128 up columns; 256 or 128 rows).
hipError_t run_tile_moe_act(int bm, const GemmParams& p, int gx, hipStream_t s) {
    if (bm == 256) return launch_tile<256, 256, 4, 2, true, GROUP_GATHER_ACT, false>(p, gx, 1, s);
    if (bm == 128) return launch_tile<128, 256, 2, 4, true, GROUP_GATHER_ACT, false>(p, gx, 1, s);
    return hipErrorInvalidConfiguration;
}

}  // namespace tg
