// Instantiations of the hand-ordered 256x256 per-tensor tile kernel and of the narrow tiles with in-workgroup split-K.
#include "fp8_gemm_tile256.h"
#include "fp8_gemm_tile_mid.h"
#include "tg_host.h"

namespace tg {

hipError_t run_tile256(const GemmParams& p, int gx, hipStream_t s) { return launch_tile256(p, gx, s); }
hipError_t run_tile_mid(int bm, int bn, const GemmParams& p, hipStream_t s) {
    if (bn == 64) return launch_tile_mid<64, 64, 2>(p, s);
    return bm == 32 ? launch_tile_mid<32, 32, 4>(p, s) : launch_tile_mid<64, 32, 3>(p, s);
}

}  // namespace tg
