// Instantiation unit of the register-pipelined 256x256 per-tensor kernel.
#include "fp8_gemm_pipe.h"
#include "tg_host.h"

namespace tg {

hipError_t run_pipe(int waves, int loaders, const GemmParams& p, int gx, hipStream_t s) {
    if (waves == 8 && loaders == 4) return launch_pipe<8, 4>(p, gx, s);
    if (waves == 8 && loaders == 8) return launch_pipe<8, 8>(p, gx, s);
    return hipErrorInvalidConfiguration;
}

}  // namespace tg
