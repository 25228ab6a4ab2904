// Instantiations of the weight-streaming skinny-M kernel.
#include "fp8_gemm_skinny.h"
#include "tg_host.h"

namespace tg {

hipError_t run_skinny(int mt, int rg, bool bs, const GemmParams& p, int gx, int gy, hipStream_t s) {
#define TG_CASE(MT, RG)                                                       \
    if (mt == MT && rg == RG) {                                               \
        return bs ? launch_skinny<MT, RG, true>(p, gx, gy, s)                 \
                  : launch_skinny<MT, RG, false>(p, gx, gy, s);               \
    }
    TG_CASE(1, 1) TG_CASE(1, 2) TG_CASE(1, 4)
    TG_CASE(2, 1) TG_CASE(2, 2) TG_CASE(2, 4)
    TG_CASE(4, 1) TG_CASE(4, 2) TG_CASE(4, 4)
#undef TG_CASE
    return hipErrorInvalidConfiguration;
}

}  // namespace tg
