// Instantiation of the hand-ordered 256x256 per-tensor tile kernel.
#include "fp8_gemm_tile256.h"
#include "tg_host.h"

namespace tg {

hipError_t run_tile256(const GemmParams& p, int gx, hipStream_t s) { return launch_tile256(p, gx, s); }

}  // namespace tg
