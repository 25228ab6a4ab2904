// Instantiations of the persistent 256x256 block-scaled tile kernel (dense rows and ragged expert segments).
#include "fp8_gemm_tile_bs256.h"
#include "tg_host.h"

namespace tg {

hipError_t run_bs256(int group, const GemmParams& p, int tiles_bound, hipStream_t s) {
    const int cus = compute_units();
    if (group == GROUP_DENSE) return launch_bs256<GROUP_DENSE>(p, tiles_bound, cus, s);
    if (group == GROUP_RAGGED) return launch_bs256<GROUP_RAGGED>(p, tiles_bound, cus, s);
    return hipErrorInvalidConfiguration;
}

}  // namespace tg
