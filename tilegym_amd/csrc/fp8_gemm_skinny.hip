// Instantiations of the weight-streaming skinny-M kernel.
#include "fp8_gemm_skinny.h"
#include "tg_host.h"

namespace tg {

template <int MT, int RG>
static hipError_t run_skinny_nw(int nw, bool bs, const GemmParams& p, int gx, int gy, hipStream_t s) {
    switch (nw) {
        case 4: return bs ? launch_skinny<MT, RG, 4, true>(p, gx, gy, s) : launch_skinny<MT, RG, 4, false>(p, gx, gy, s);
        case 8: return bs ? launch_skinny<MT, RG, 8, true>(p, gx, gy, s) : launch_skinny<MT, RG, 8, false>(p, gx, gy, s);
        case 16: return bs ? launch_skinny<MT, RG, 16, true>(p, gx, gy, s) : launch_skinny<MT, RG, 16, false>(p, gx, gy, s);
        default: return hipErrorInvalidConfiguration;
    }
}

hipError_t run_skinny(int mt, int rg, int nw, bool bs, const GemmParams& p, int gx, int gy, hipStream_t s) {
#define TG_CASE(MT, RG) \
    if (mt == MT && rg == RG) return run_skinny_nw<MT, RG>(nw, bs, p, gx, gy, s);
    TG_CASE(1, 1) TG_CASE(1, 2) TG_CASE(1, 4)
    TG_CASE(2, 1) TG_CASE(2, 2)
    TG_CASE(4, 1) TG_CASE(4, 2)
#undef TG_CASE
    return hipErrorInvalidConfiguration;
}

}  // namespace tg
