// Instantiations of the hand-ordered 256x256 per-tensor tile kernel and of the narrow tiles with in-workgroup split-K.
#include "fp8_gemm_tile256.h"
#include "fp8_gemm_tile_mid.h"
#include "tg_host.h"

namespace tg {

// Compute units of the current device: the persistent 256x256 kernel runs one workgroup on each.
int compute_units() {
    static int cached[64];  // by device ordinal; 0 = not asked yet (racing first calls write the same value)
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
    if (cached[dev] == 0) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        cached[dev] = n;
    }
    return cached[dev];
}

hipError_t run_tile256(const GemmParams& p, int gx, hipStream_t s) { return launch_tile256(p, gx, compute_units(), s); }
hipError_t run_tile_mid(int bm, int bn, const GemmParams& p, hipStream_t s) {
    if (bn == 64) return launch_tile_mid<64, 64, 2>(p, s);
    return bm == 32 ? launch_tile_mid<32, 32, 4>(p, s) : launch_tile_mid<64, 32, 3>(p, s);
}

}  // namespace tg
