// Instantiations of the second-generation weight-streaming skinny-M kernel.
#include "fp8_gemm_stream.h"
#include "tg_host.h"

namespace tg {

hipError_t run_stream(int mt, int nbuf, int waves, bool bs, const GemmParams& p, int gx, int gy, hipStream_t s) {
    // rows per workgroup: 1 .. 16; with block scales a workgroup's rows share one weight scale
    if (p.wave_rows < 0 || p.wave_rows > 16 || (bs && p.wave_rows > 0 && 128 % p.wave_rows != 0)) return hipErrorInvalidValue;
    // eight waves per workgroup (one 16 KiB buffer each, one workgroup per compute unit): long K over few weight rows
    if (waves == 8 && mt == 1 && nbuf == 1)
        return bs ? launch_stream<1, 1, true, 8>(p, gx, gy, s) : launch_stream<1, 1, false, 8>(p, gx, gy, s);
#define TG_CASE(MT, NBUF)                                                   \
    if (mt == MT && nbuf == NBUF)                                           \
        return bs ? launch_stream<MT, NBUF, true>(p, gx, gy, s) : launch_stream<MT, NBUF, false>(p, gx, gy, s);
    TG_CASE(1, 1) TG_CASE(1, 2) TG_CASE(2, 1) TG_CASE(2, 2) TG_CASE(4, 1) TG_CASE(4, 2)
#undef TG_CASE
    return hipErrorInvalidConfiguration;
}

hipError_t run_stream_ragged(const GemmParams& p, int waves, hipStream_t s) {
    switch (waves) {
        case 4: return launch_stream_ragged<4>(p, s);
        case 6: return launch_stream_ragged<6>(p, s);
        case 8: return launch_stream_ragged<8>(p, s);
        default: return hipErrorInvalidConfiguration;
    }
}

hipError_t run_stream_wide(bool bs, const GemmParams& p, int gy, hipStream_t s, bool two_buffers, int mt) {
    int gx = (p.N + 63) / 64;
    if (two_buffers && p.K % 128 == 0) {
        if (p.wave_rows > 0) gx = (p.N + 4 * p.wave_rows - 1) / (4 * p.wave_rows);
        if (mt == 1) return bs ? launch_stream_wide_db<true, 1>(p, gx, gy, s) : launch_stream_wide_db<false, 1>(p, gx, gy, s);
        if (mt == 2) return bs ? launch_stream_wide_db<true, 2>(p, gx, gy, s) : launch_stream_wide_db<false, 2>(p, gx, gy, s);
        return hipErrorInvalidConfiguration;
    }
    if (mt != 1 || (p.wave_rows != 0 && p.wave_rows != 16)) return hipErrorInvalidConfiguration;
    return bs ? launch_stream_wide<true>(p, gx, gy, s) : launch_stream_wide<false>(p, gx, gy, s);
}

}  // namespace tg
