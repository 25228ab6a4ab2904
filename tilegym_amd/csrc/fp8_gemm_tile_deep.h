// Deep-pipelined form of the 64x128 per-tensor tile (16 < M <= 512 while its tiles fit one round of the chip,
// usually with split-K): three LDS stages of one K step each (3 x 24 KiB), loads requested up to three steps
// ahead, one barrier per step, and a software-pipelined step (see the loop).
// These launches are weight-streaming: a workgroup runs 8-32 K steps of 8 MFMAs per wave, mostly alone on its
// compute unit.  With the two stages of fp8_gemm_tile.h (weights one step ahead) every step waited for a full trip
// to HBM (1.3-2.2 k clocks per step measured, against 0.4 k of load issue and 0.26 k of MFMA); with three stages
// but load issue, fragment reads and MFMAs one after the other inside a step, a step still took ~1 k clocks.
//
// Same slab layout, swizzles, fragment addressing, MFMA order per accumulator and epilogue arithmetic
// as fp8_gemm_tile_kernel<64, 128, 1, 4, false, GROUP_DENSE, SPLIT>: identical results.
// Steps past the end re-fetch the last one, which keeps the wait counts uniform.
// A tile may cover fewer than 128 weight rows (p.tile_cols, a multiple of 8): the slab rows beyond them are requested from
// beyond the buffer descriptor's range (no memory traffic, zeros) and their columns are not stored.  With 28672 weight
// rows at M = 64, tiles of 112 are one per compute unit where tiles of 128 leave an eighth of the chip idle.
#pragma once

#include "fp8_gemm_tile.h"

namespace tg {

template <bool SPLIT>
__global__ void __launch_bounds__(256, 2) fp8_gemm_tile_deep_kernel(const GemmParams p) {
#if defined(__HIP_DEVICE_COMPILE__)
    constexpr int BM = 64, BN = 128, WGN = 4, NW = 4, NL = 4, STAGES = 3;  // (six stages, one workgroup per compute unit: 5-10 % slower)
    constexpr int WTN = BN / WGN;            // 32 columns per wave, all 64 rows
    constexpr int TM = BM / 16, TN = WTN / 16;
    constexpr int RPP = 8 * NL;
    constexpr int A_IT = BM / RPP, B_IT = BN / RPP;
    constexpr int STAGE_BYTES = (BM + BN) * kKBlock;
    static_assert(TN == 2 && A_IT == 2 && B_IT == 4 && NW == WGN, "shape");

    __shared__ __align__(1024) uint8_t lds[STAGES * STAGE_BYTES];  // stage s: A slab (8 KiB), then B slab (16 KiB)

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wn = wave;
    const int K = p.K;
    const int cols = p.tile_cols > 0 ? p.tile_cols : BN;   // weight rows (output columns) this tile covers
    const int tiles_n = (p.N + cols - 1) / cols, tiles_m = (p.M + BM - 1) / BM;
    const int pid = xcd_remap((int)blockIdx.x, tiles_m * tiles_n);
    constexpr int GM = 8;
    const int width = GM * tiles_n;
    const int group = pid / width, first_m = group * GM;
    const int gsz = min(tiles_m - first_m, GM);
    const int tile_m = first_m + (pid % width) % gsz, tile_n = (pid % width) / gsz;
    const int m0 = tile_m * BM, n0 = tile_n * cols;
    const int n_end = min(n0 + cols, p.N);
    const int rows_valid = min(BM, p.M - m0);

    int ks = 0, ks_end = p.kblocks;
    if constexpr (SPLIT) {
        ks = blockIdx.y * p.ksteps_per_split;
        ks_end = min(ks + p.ksteps_per_split, p.kblocks);
    }
    const int nsteps = ks_end - ks, last = ks_end - 1;
    if (nsteps <= 0) return;

    const int lrow = lane >> 3;
    const int lj = (lane & 7) ^ swz16(lrow);
    const int ljb = (lane & 7) ^ swz_w(((wave & 1) << 3) | lrow);
    uint32_t a_off[A_IT], b_off[B_IT];
#pragma unroll
    for (int i = 0; i < A_IT; ++i) {
        const int r = (i * NL + wave) * 8 + lrow;
        a_off[i] = (uint32_t)(m0 + min(r, rows_valid - 1)) * (uint32_t)K + lj * 16;
    }
#pragma unroll
    for (int i = 0; i < B_IT; ++i) {
        const int br = (i * NL + wave) * 8 + lrow;
        b_off[i] = n0 + br < n_end ? (uint32_t)(n0 + br) * (uint32_t)K + ljb * 16 : 0x80000000u;  // (>= the descriptor's 2^31 - 1 bytes)
    }
    const v4i rsrc_a = make_rsrc(p.A), rsrc_b = make_rsrc(p.B);
    const uint32_t lds0 = lds_address(lds) + wave * 1024;
    auto issue = [&](int kstep, int stage) {  // this wave's share of one K step: 2 + 4 direct loads
        const int k0 = min(kstep, last) * kKBlock;
        const uint32_t dst = lds0 + stage * STAGE_BYTES;
#pragma unroll
        for (int i = 0; i < A_IT; ++i) direct_load_b128(rsrc_a, dst + i * NL * 1024, a_off[i], k0);
#pragma unroll
        for (int i = 0; i < B_IT; ++i) direct_load_b128_nt(rsrc_b, dst + BM * kKBlock + i * NL * 1024, b_off[i], k0);
    };

    const int li = lane & 15, lg = lane >> 4;
    const uint32_t frag0 = li * kKBlock + ((lg ^ swz16(li)) << 4), frag1 = frag0 ^ 64;
    const int wrow = ((li >> 2) << 3) | (li & 3);
    const uint32_t wfrag0 = BM * kKBlock + wn * WTN * kKBlock + wrow * kKBlock + ((lg ^ swz_w(wrow)) << 4), wfrag1 = wfrag0 ^ 64;

    v4f acc[TN][TM];
#pragma unroll
    for (int tn = 0; tn < TN; ++tn)
#pragma unroll
        for (int tm = 0; tm < TM; ++tm) acc[tn][tm] = v4f{0.f, 0.f, 0.f, 0.f};

    // vmcnt(n): all of this wave's direct loads except the n most recent have landed
    constexpr int PER_STEP = A_IT + B_IT;
    constexpr int kPro = (STAGES - 1) * PER_STEP, kLoop = (STAGES - 2) * PER_STEP;  // loads that may stay in flight
    constexpr int kWaitBut2 = 0x0F70 | (kPro & 15) | ((kPro >> 4) << 14);
    constexpr int kWaitBut1 = 0x0F70 | (kLoop & 15) | ((kLoop >> 4) << 14);
    constexpr int kWaitAll = 0x0F70;
    constexpr int kWaitLds = 0xC07F;
#define TG_FENCE() __builtin_amdgcn_sched_barrier(0)

    // Software-pipelined loop.  The fragments of step i are in registers when iteration i starts (read during iteration
    // i-1), so iteration i runs its MFMAs while the fragments of step i+1 are read and the loads of step i+3 are issued,
    // one direct load and one fragment behind each MFMA: with one workgroup per compute unit (these launches rarely have
    // more) nothing else would hide the LDS latency and the load issue time.  One barrier per step: behind it every
    // wave's share of step i+1 is visible and stage i is free (everyone holds its fragments).
    v8i af[2][TM], wf[2][TN];
    auto read_frag = [&](int f, int set, const uint8_t* base) {  // fragment f of a step: 0..TM-1 activations, then weights
        if (f < TM) {
            const uint8_t* a = base + f * 16 * kKBlock;
            af[set][f] = join(*reinterpret_cast<const v4i*>(a + frag0), *reinterpret_cast<const v4i*>(a + frag1));
        } else {
            const int tn = f - TM;
            const uint8_t* b = base + ((tn >> 1) * 32 + (tn & 1) * 4) * kKBlock;
            wf[set][tn] = join(*reinterpret_cast<const v4i*>(b + wfrag0), *reinterpret_cast<const v4i*>(b + wfrag1));
        }
    };
    auto issue1 = [&](int q, int kstep, int stage) {  // direct load q of a step (activations first)
        const int k0 = min(kstep, last) * kKBlock;
        const uint32_t dst = lds0 + stage * STAGE_BYTES;
        if (q < A_IT) direct_load_b128(rsrc_a, dst + q * NL * 1024, a_off[q], k0);
        else direct_load_b128_nt(rsrc_b, dst + BM * kKBlock + (q - A_IT) * NL * 1024, b_off[q - A_IT], k0);
    };
#pragma unroll
    for (int s = 0; s < STAGES; ++s) issue(ks + s, s);
    __builtin_amdgcn_s_waitcnt(kWaitBut2);  // step 0 has landed
    __builtin_amdgcn_s_barrier();
#pragma unroll
    for (int f = 0; f < TM + TN; ++f) read_frag(f, 0, lds);
    auto body = [&](int i, auto cur_tag) {
        constexpr int CUR = decltype(cur_tag)::value, NXT = CUR ^ 1;
        const int stage_n = (i + 1) % STAGES, stage_free = i % STAGES;
        __builtin_amdgcn_s_waitcnt(kWaitBut1);  // step i+1 has landed (steps past the end re-fetch the last one)
        __builtin_amdgcn_s_waitcnt(kWaitLds);   // my fragments of step i are in registers
        __builtin_amdgcn_s_barrier();
        TG_FENCE();
        const uint8_t* nbase = lds + stage_n * STAGE_BYTES;
        int j = 0;
#pragma unroll
        for (int tn = 0; tn < TN; ++tn)
#pragma unroll
            for (int tm = 0; tm < TM; ++tm, ++j) {
                acc[tn][tm] = mfma_e4m3(wf[CUR][tn], af[CUR][tm], acc[tn][tm]);
                TG_FENCE();
                if (j < PER_STEP) issue1(j, ks + i + STAGES, stage_free);
                if (j < TM + TN) read_frag(j, NXT, nbase);
                TG_FENCE();
            }
    };
    static_assert(TM * TN >= PER_STEP && TM * TN >= TM + TN, "one load and one fragment behind each MFMA");
    int i = 0;
    for (; i + 1 < nsteps; i += 2) {
        body(i, std::integral_constant<int, 0>{});
        body(i + 1, std::integral_constant<int, 1>{});
    }
    if (i < nsteps) body(i, std::integral_constant<int, 0>{});
#undef TG_FENCE
    __builtin_amdgcn_s_waitcnt(kWaitAll);  // the re-fetches past the end must land before the workgroup's LDS is released
    __builtin_amdgcn_s_waitcnt(kWaitLds);

    // epilogue, straight from the accumulators (row 16*tm + li, eight consecutive columns per lane)
    float scale = p.alpha;
    if (p.As) scale *= p.As[0];
    if (p.Bs) scale *= p.Bs[0];
    const bool vec_ok = p.vec_store != 0 && (p.N % 8) == 0;
    const int64_t MN = (int64_t)p.M * p.N;
    const int col = n0 + wn * WTN + lg * 8;
    auto emit = [&](auto type_tag) {
        constexpr int OT = decltype(type_tag)::value;
#pragma unroll
        for (int tm = 0; tm < TM; ++tm) {
            const int rt = tm * 16 + li;
            if (rt >= rows_valid || col >= n_end) continue;
            if constexpr (SPLIT)
                store8(p.partials + (int64_t)blockIdx.y * MN, OUT_F32, m0 + rt, col, n_end, p.N, acc[0][tm], acc[1][tm], 0.f, vec_ok);
            else
                store8(p.C, OT, m0 + rt, col, n_end, p.ldc, acc[0][tm] * scale, acc[1][tm] * scale, p.beta, vec_ok);
        }
    };
    if (SPLIT || p.out_type == OUT_BF16) emit(std::integral_constant<int, OUT_BF16>{});
    else if (p.out_type == OUT_F32) emit(std::integral_constant<int, OUT_F32>{});
    else if (p.out_type == OUT_F8) emit(std::integral_constant<int, OUT_F8>{});
    else emit(std::integral_constant<int, OUT_F16>{});
#endif
}

template <bool SPLIT>
inline hipError_t launch_tile_deep(const GemmParams& p, int grid_x, int grid_y, hipStream_t stream) {
    if (p.tile_cols != 0 && (p.tile_cols < 8 || p.tile_cols > 128 || (p.tile_cols % 8) != 0)) return hipErrorInvalidValue;
    hipLaunchKernelGGL(fp8_gemm_tile_deep_kernel<SPLIT>, dim3(grid_x, grid_y, 1), dim3(256, 1, 1), 0, stream, p);
    return hipGetLastError();
}

}  // namespace tg
