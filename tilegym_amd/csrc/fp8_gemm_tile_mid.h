// 64 x 64, 64 x 32 and 32 x 32 per-tensor tiles whose four waves split K inside the workgroup (16 < M <= 256 against
// small weights, one launch): C[m,n] = sum_k A[m,k] * B[n,k].
//
// These M are weight-streaming problems with too few output tiles to fill the chip: M = 64 against a 4096 x 4096
// weight is 32 tiles of 64 x 128.  Splitting K across workgroups fills it, but the partial sums then need a second
// launch that costs more than the GEMM's own roofline time.  Here the tile is narrow (128 - 400 workgroups on the
// Llama shapes) and K is split across the four waves of the workgroup instead: every wave owns a contiguous quarter
// of the K steps and runs its own ring of LDS stages ((BM + BN) rows x 128 bytes each; two stages of 16 KiB at
// 64 x 64, three of 12 KiB at 64 x 32, four of 8 KiB at 32 x 32: 128 - 144 KiB per workgroup).  There is no barrier
// in the loop -- a wave only waits for its own loads -- and ALL stages of a ring are in flight: a wave reads the
// fragments of step i into registers, waits for those reads, requests step i + STAGES into the same stage at once
// and only then runs the MFMAs of step i.  What bounds these launches is the number of bytes a compute unit has in
// flight against the latency of HBM, not the matrix pipe (16 - 64 MFMAs per step): keeping a stage idle while its
// step is multiplied cost 20 % (4096 x 4096 weight, M = 256: 15.5 -> 12.5 us).  The four partial tiles are added
// through LDS at the end, in a fixed order.
// The price is activation traffic: every workgroup reads all K of its activation rows (L2 hits), one or two bytes per
// weight byte, and those bytes take LDS that would otherwise hold weights in flight from HBM.  It pays while one round
// of workgroups covers the problem and the weights are small (measured: 4096 x 4096 and 6144 x 4096 at M <= 256); for
// larger weights the 64 x 128 tile with split-K across workgroups stays faster.
// Measured and not kept: the same K partition with both operands streamed through a ring of register sets instead of
// LDS (3 - 8 steps in flight per wave, bit-identical): 20 - 40 % slower at every depth -- a fragment load fetches 64
// bytes of 16 rows where a direct load fetches 128 bytes of 8; eight waves per workgroup splitting K eight ways with
// half the stages each: 2 - 8 % slower.
// Slab layout, swizzles and fragment addressing are those of fp8_gemm_tile.h.
#pragma once

#include "fp8_gemm_tile.h"

namespace tg {

template <int BM, int BN, int STAGES>
__global__ void __launch_bounds__(256, 1) fp8_gemm_tile_mid_kernel(const GemmParams p) {
#if defined(__HIP_DEVICE_COMPILE__)
    constexpr int NW = 4;
    constexpr int TM = BM / 16, TN = BN / 16;
    constexpr int A_IT = BM / 8, B_IT = BN / 8;               // BM / 8 + 4 direct loads per wave and K step
    constexpr int STAGE_BYTES = (BM + BN) * kKBlock;
    constexpr int PER_STEP = A_IT + B_IT;
    static_assert(TN == 2 || TN == 4, "one or two column-tile pairs");

    constexpr int RED_BYTES = NW * TN * TM * 1024;
    constexpr int RING_BYTES = NW * STAGES * STAGE_BYTES;
    __shared__ __align__(1024) uint8_t lds[RING_BYTES > RED_BYTES ? RING_BYTES : RED_BYTES];  // <= 160 KiB; reused for the reduction

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int K = p.K;
    const int n0 = (int)blockIdx.x * BN, m0 = (int)blockIdx.y * BM;
    const int rows_valid = min(BM, p.M - m0);
    // this wave's K steps: a contiguous share
    const int ks = (int)((int64_t)p.kblocks * wave / NW), ks_end = (int)((int64_t)p.kblocks * (wave + 1) / NW);
    const int nsteps = ks_end - ks;

    const int lrow = lane >> 3;
    const int lj = (lane & 7) ^ swz16(lrow);
    uint32_t a_off[A_IT], b_off[B_IT];
#pragma unroll
    for (int i = 0; i < A_IT; ++i) {
        const int r = i * 8 + lrow;
        a_off[i] = (uint32_t)(m0 + min(r, rows_valid - 1)) * (uint32_t)K + lj * 16;
    }
#pragma unroll
    for (int i = 0; i < B_IT; ++i) {
        const int br = i * 8 + lrow;
        const int ljb = (lane & 7) ^ swz_w(((i & 1) << 3) | lrow);
        b_off[i] = (uint32_t)min(n0 + br, p.N - 1) * (uint32_t)K + ljb * 16;
    }
    const v4i rsrc_a = make_rsrc(p.A), rsrc_b = make_rsrc(p.B);
    uint8_t* my = lds + wave * STAGES * STAGE_BYTES;
    const uint32_t lds0 = lds_address(my);
    auto issue = [&](int kstep, int stage) {
        const int k0 = kstep * kKBlock;
        const uint32_t dst = lds0 + stage * STAGE_BYTES;
#pragma unroll
        for (int i = 0; i < B_IT; ++i) direct_load_b128_nt(rsrc_b, dst + BM * kKBlock + i * 1024, b_off[i], k0);
#pragma unroll
        for (int i = 0; i < A_IT; ++i) direct_load_b128(rsrc_a, dst + i * 1024, a_off[i], k0);
    };

    const int li = lane & 15, lg = lane >> 4;
    const uint32_t frag0 = li * kKBlock + ((lg ^ swz16(li)) << 4), frag1 = frag0 ^ 64;
    const int wrow = ((li >> 2) << 3) | (li & 3);
    const uint32_t wfrag0 = BM * kKBlock + wrow * kKBlock + ((lg ^ swz_w(wrow)) << 4), wfrag1 = wfrag0 ^ 64;

    v4f acc[TN][TM];
#pragma unroll
    for (int tn = 0; tn < TN; ++tn)
#pragma unroll
        for (int tm = 0; tm < TM; ++tm) acc[tn][tm] = v4f{0.f, 0.f, 0.f, 0.f};

    // All STAGES steps of the ring are in flight: step i's fragments are read into registers, and as soon as those
    // reads have returned the same stage is requested again for step i + STAGES; the MFMAs of step i run behind that.
    constexpr int kKeep = (STAGES - 1) * PER_STEP;  // the later stages may still be in flight
    constexpr int kWaitStep = 0x0F70 | (kKeep & 15) | ((kKeep >> 4) << 14);
    constexpr int kWaitAll = 0x0F70, kWaitLds = 0xC07F;

#pragma unroll
    for (int s = 0; s < STAGES; ++s)
        if (s < nsteps) issue(ks + s, s);
    for (int i = 0; i < nsteps; ++i) {
        const int stage = i % STAGES;
        // step i has landed: all but the STAGES - 1 later steps, if that many were requested
        if (i + STAGES <= nsteps) __builtin_amdgcn_s_waitcnt(kWaitStep);
        else __builtin_amdgcn_s_waitcnt(kWaitAll);
        const uint8_t* base = my + stage * STAGE_BYTES;
        v8i af[TM], wf[TN];
#pragma unroll
        for (int tn = 0; tn < TN; ++tn) {
            const uint8_t* b = base + ((tn >> 1) * 32 + (tn & 1) * 4) * kKBlock;
            wf[tn] = join(*reinterpret_cast<const v4i*>(b + wfrag0), *reinterpret_cast<const v4i*>(b + wfrag1));
        }
#pragma unroll
        for (int tm = 0; tm < TM; ++tm) {
            const uint8_t* a = base + tm * 16 * kKBlock;
            af[tm] = join(*reinterpret_cast<const v4i*>(a + frag0), *reinterpret_cast<const v4i*>(a + frag1));
        }
        if (i + STAGES < nsteps) {
            __builtin_amdgcn_s_waitcnt(kWaitLds);  // the fragments are in registers: the stage is free
#pragma unroll
            for (int tn = 0; tn < TN; ++tn) asm volatile("" : "+v"(wf[tn]));
#pragma unroll
            for (int tm = 0; tm < TM; ++tm) asm volatile("" : "+v"(af[tm]));
            issue(ks + i + STAGES, stage);
        }
#pragma unroll
        for (int tn = 0; tn < TN; ++tn)
#pragma unroll
            for (int tm = 0; tm < TM; ++tm) acc[tn][tm] = mfma_e4m3(wf[tn], af[tm], acc[tn][tm]);
    }
    __builtin_amdgcn_s_waitcnt(kWaitLds);
    __syncthreads();

    // ---- add the four partial tiles through LDS: wave w writes its 8 accumulator tiles, then every wave sums
    // column-tile-pair rows tm = w (fixed order over the waves) and stores them
    v4f* red = reinterpret_cast<v4f*>(lds);
#pragma unroll
    for (int tn = 0; tn < TN; ++tn)
#pragma unroll
        for (int tm = 0; tm < TM; ++tm) red[((wave * TN + tn) * TM + tm) * 64 + lane] = acc[tn][tm];
    __syncthreads();
    float scale = p.alpha;
    if (p.As) scale *= p.As[0];
    if (p.Bs) scale *= p.Bs[0];
    const bool vec_ok = p.vec_store != 0 && (p.N % 8) == 0;
    const int col = n0 + lg * 8;
    // every wave finishes (row group, column-tile pair) units wave, wave + NW, ...: the partial sums in wave order
    for (int u = wave; u < TM * (TN / 2); u += NW) {
        const int tm = u / (TN / 2), tp = u % (TN / 2);
        const int rt = tm * 16 + li;
        v4f s0 = red[((0 * TN + 2 * tp) * TM + tm) * 64 + lane], s1 = red[((0 * TN + 2 * tp + 1) * TM + tm) * 64 + lane];
#pragma unroll
        for (int w = 1; w < NW; ++w) {
            s0 += red[((w * TN + 2 * tp) * TM + tm) * 64 + lane];
            s1 += red[((w * TN + 2 * tp + 1) * TM + tm) * 64 + lane];
        }
        const int c = col + tp * 32;
        if (rt < rows_valid && c < p.N) store8(p.C, p.out_type, m0 + rt, c, p.N, p.ldc, s0 * scale, s1 * scale, p.beta, vec_ok);
    }
#endif
}

template <int BM, int BN, int STAGES>
inline hipError_t launch_tile_mid(const GemmParams& p, hipStream_t stream) {
    hipLaunchKernelGGL((fp8_gemm_tile_mid_kernel<BM, BN, STAGES>), dim3((p.N + BN - 1) / BN, (p.M + BM - 1) / BM, 1), dim3(256, 1, 1), 0, stream, p);
    return hipGetLastError();
}

}  // namespace tg
