// Instantiations of the list form of the LDS-tiled kernel (tilegym.ops.group_gemm in one launch).
#include "fp8_gemm_tile.h"
#include "tg_host.h"

namespace tg {

hipError_t run_tile_list(int bm, int bn, const GemmList& gl, int gx, hipStream_t s) {
    if (bm == 256 && bn == 256) return launch_tile_list<256, 256, 4, 2>(gl, gx, s);
    if (bm == 128 && bn == 128) return launch_tile_list<128, 128, 2, 2>(gl, gx, s);
    if (bm == 64 && bn == 128) return launch_tile_list<64, 128, 1, 4>(gl, gx, s);
    return hipErrorInvalidConfiguration;
}

}  // namespace tg
