// 256x256 per-tensor tile, persistent, with a hand-ordered K loop (prefill shapes): C[m,n] = sum_k A[m,k] * B[n,k].
//
// Same slab layout, swizzles, fragment addressing, per-accumulator MFMA order and epilogue arithmetic as
// fp8_gemm_tile_kernel<256, 256, 4, 2, false, GROUP_DENSE, false>: identical results.  What differs:
//   * Four waves, one per SIMD, each with a 128 x 128 part of the tile (8 x 8 MFMA tiles; the 256 accumulator
//     registers of a lane live in the accumulation half of the register file).  A K step reads 128 + 128 fragment
//     rows per wave from LDS for 64 MFMAs; eight waves of 64 x 128 read 64 + 128 rows for 32.  A third fewer LDS
//     bytes per MFMA is less energy per FLOP, and this path is limited by power: the same loop at the same number of
//     clocks per step runs at a 3 - 5 % higher clock (measured against the eight-wave form of this kernel).
//   * Persistent: one workgroup per compute unit walks tiles b, b + grid, b + 2 grid, ... of the rastered tile
//     sequence, and the slab rings run on across tiles.  The last two K steps of a tile request steps 0 and 1 of the
//     workgroup's next tile, so those land while this tile's results are converted and stored; a workgroup per tile
//     paid 5 - 7 k clocks of first-load latency per tile (of ~92 k) plus the gap between two workgroups on a
//     compute unit (8192 x 28672 x 4096: 677 -> 646 us).
//   * All waves load (sixteen 1 KiB loads per wave and step), one load behind every group of four MFMAs in the
//     first half of a step (weights) and one behind every pair in its tail (activations): while a wave waits for
//     room in the address path (about 14 clocks per 1 KiB load for the whole compute unit) it issues no MFMAs, so
//     bursts of loads put load time and MFMA time in series.
//   * Two activation slabs and three weight slabs (160 KiB, all of LDS) let one barrier per step do:
//     a step requests B(k+2) between its first MFMAs and, after its barrier, A(k+2), always into slabs
//     nobody reads any more.  The weights get the long lead (1.25 - 2 steps): on the big projections
//     they stream from HBM, while the activation panel of a tile row is re-read by every tile of that
//     row and sits in the L2 / memory-side cache.
//   * The barrier sits in front of the last sixteen MFMAs of a step, which are ordered by row group so
//     that the activation fragments of step k+1 are read into the registers those MFMAs release:
//     the matrix pipe has work while the fragment reads of the next step are in flight.
// The order is pinned with scheduling fences: the direct loads are inline assembly (see
// direct_load_b128), which the compiler's own interleaving hints cannot see.
// K must be at least two steps (256): the switch to the next tile's addresses happens two steps before a tile's end.
#pragma once

#include "fp8_gemm_tile.h"

namespace tg {

__global__ void __launch_bounds__(256, 1) fp8_gemm_tile256_kernel(const GemmParams p) {
#if defined(__HIP_DEVICE_COMPILE__)
    constexpr int BM = 256, BN = 256, WGM = 2, WGN = 2, NW = 4;
    constexpr int WTN = BN / WGN;                 // 128 columns per wave
    constexpr int TM = 8, TN = WTN / 16;          // 8 row groups x 8 column tiles per wave
    constexpr int SLAB = 256 * kKBlock;           // 32 KiB
    constexpr int A_STAGES = 2, B_STAGES = 3;
    constexpr int IT = 256 / (8 * NW);            // 8 loads per wave, slab and step
    static_assert(TN == 8 && IT == 8 && TM == 8, "schedule below is written for 8 x 8 MFMA tiles and 8 + 8 loads per wave");

    __shared__ __align__(1024) uint8_t sA[A_STAGES * SLAB];
    __shared__ __align__(1024) uint8_t sB[B_STAGES * SLAB];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave % WGM, wn = wave / WGM;
    const int K = p.K;
    const int tiles_n = (p.N + BN - 1) / BN, tiles_m = (p.M + BM - 1) / BM;
    // Persistent: workgroup b computes tiles b, b + gridDim.x, b + 2 gridDim.x, ... of the rastered tile sequence
    // (with a grid that is a multiple of 8 -- the 256 compute units -- a workgroup's tiles all belong to its XCD's range of
    // the sequence; any other grid computes the same tiles with less reuse in the L2s).
    const int total = tiles_m * tiles_n, stride = (int)gridDim.x;
    auto origin = [&](int v, int& om0, int& on0) {
        const int pid = xcd_remap(v, total);
        constexpr int GM = 8;
        const int width = GM * tiles_n;
        const int group = pid / width, first_m = group * GM;
        const int gsz = min(tiles_m - first_m, GM);
        om0 = (first_m + (pid % width) % gsz) * BM;
        on0 = ((pid % width) / gsz) * BN;
    };
    int vt = (int)blockIdx.x;  // position of the current tile in the sequence
    int m0, n0;
    origin(vt, m0, n0);
    const int nsteps = p.kblocks, last = nsteps - 1;

    // ---- direct loads: pass i of wave w fills slab rows 8*(i*4 + w) .. +7 (lane l: row + l/8, chunk position l%8)
    const int lrow = lane >> 3;
    const int lj = (lane & 7) ^ swz16(lrow);
    const int ljb = (lane & 7) ^ swz_w(((wave & 1) << 3) | lrow);
    uint32_t a_off[IT], b_off[IT];
    auto set_offsets = [&](int om0, int on0) {
        const int rv = min(BM, p.M - om0);
#pragma unroll
        for (int i = 0; i < IT; ++i) {
            const int r = (i * NW + wave) * 8 + lrow;
            a_off[i] = (uint32_t)(om0 + min(r, rv - 1)) * (uint32_t)K + lj * 16;
            b_off[i] = (uint32_t)min(on0 + r, p.N - 1) * (uint32_t)K + ljb * 16;
        }
    };
    set_offsets(m0, n0);
    const v4i rsrc_a = make_rsrc(p.A), rsrc_b = make_rsrc(p.B);
    // (the loads of this kernel go without the wait states of direct_load_b128: their scalar operands are the two
    // descriptors, these two settled addresses and the loop's own scalar counters)
    const uint32_t ldsA = settle(lds_address(sA) + wave * 1024), ldsB = settle(lds_address(sB) + wave * 1024);
    auto load_a = [&](int i, int kstep, int stage) {
        direct_load_b128_settled(rsrc_a, ldsA + stage * SLAB + i * NW * 1024, a_off[i], kstep * kKBlock);
    };
    auto load_b = [&](int i, int kstep, int stage) {
        direct_load_b128_settled(rsrc_b, ldsB + stage * SLAB + i * NW * 1024, b_off[i], kstep * kKBlock);
    };

    // ---- fragment addresses (see fp8_gemm_tile.h)
    const int li = lane & 15, lg = lane >> 4;
    const uint32_t frag0 = wm * 16 * kKBlock + li * kKBlock + ((lg ^ swz16(li)) << 4), frag1 = frag0 ^ 64;
    const int wrow = ((li >> 2) << 3) | (li & 3);
    const uint32_t wfrag0 = wn * WTN * kKBlock + wrow * kKBlock + ((lg ^ swz_w(wrow)) << 4), wfrag1 = wfrag0 ^ 64;
    auto read_a = [&](int tm, const uint8_t* cA) {
        const uint8_t* base = cA + tm * (WGM * 16 * kKBlock);
        return join(*reinterpret_cast<const v4i*>(base + frag0), *reinterpret_cast<const v4i*>(base + frag1));
    };
    auto read_w = [&](int tn, const uint8_t* cB) {
        const uint8_t* base = cB + ((tn >> 1) * 32 + (tn & 1) * 4) * kKBlock;
        return join(*reinterpret_cast<const v4i*>(base + wfrag0), *reinterpret_cast<const v4i*>(base + wfrag1));
    };

    v4f acc[TN][TM];
#pragma unroll
    for (int tn = 0; tn < TN; ++tn)
#pragma unroll
        for (int tm = 0; tm < TM; ++tm) acc[tn][tm] = v4f{0.f, 0.f, 0.f, 0.f};

    constexpr int kWaitBut16 = 0x4F70 | 0, kWaitBut8 = 0x0F70 | 8, kWaitAll = 0x0F70;
    constexpr int kWaitLds = 0xC07F;  // lgkmcnt(0)
#define TG_FENCE() __builtin_amdgcn_sched_barrier(0)

    // ---- prologue: A(0), B(0), B(1), A(1); the first two must have landed
#pragma unroll
    for (int i = 0; i < IT; ++i) load_a(i, 0, 0);
#pragma unroll
    for (int i = 0; i < IT; ++i) load_b(i, 0, 0);
#pragma unroll
    for (int i = 0; i < IT; ++i) load_b(i, min(1, last), 1);
#pragma unroll
    for (int i = 0; i < IT; ++i) load_a(i, min(1, last), 1);
    __builtin_amdgcn_s_waitcnt(kWaitBut16);   // B(1), A(1) may be in flight
    __builtin_amdgcn_s_barrier();
    v8i af[TM], wf[4];
    wf[0] = read_w(0, sB);
    wf[1] = read_w(1, sB);
#pragma unroll
    for (int tm = 0; tm < TM; ++tm) af[tm] = read_a(tm, sA);

    // ---- main loop.  On entry to step k: A(k) and B(k) are in LDS and visible to every wave; the reads of af (fragments
    // of A(k)) and wf[0], wf[1] (column tiles 0, 1 of B(k)) are issued; B(k+1) and A(k+1) are requested.
    // Requests of a wave in order: ... B(k+1) x8 | A(k+1) x8 | B(k+2) x8 |: at the wait of step k all but the last eight
    // have landed, i.e. B(k+1) and A(k+1).  (The stores of a tile's results sit in that sequence like loads: the wait of
    // the next tile's first step also waits for them.)
    // The slab rings run on across tiles: the last two steps of a tile request steps 0 and 1 of the workgroup's next
    // tile (in place of re-fetches past the end), so the next tile's first operands land while this tile's results
    // are converted and stored, and its first step finds them in LDS.
    int sa = 0, sb = 0;  // slabs that hold A(k) and B(k)
    for (;;) {  // tiles of this workgroup
        const int cm0 = m0, cn0 = n0;  // this tile's origin (the offsets move on to the next tile two steps before the end)
        bool more = false;
        for (int k = 0; k < nsteps; ++k) {
            if (k == nsteps - 2) {
                more = vt + stride < total;
                if (more) {
                    vt += stride;
                    origin(vt, m0, n0);
                    set_offsets(m0, n0);
                }
            }
            int k2 = k + 2;                       // step the requests of this step are for
            if (k2 >= nsteps) k2 = more ? k2 - nsteps : last;
            const int sa1 = sa ^ 1;                              // holds/receives A(k+1)
            const int sb1 = sb == B_STAGES - 1 ? 0 : sb + 1;     // holds B(k+1)
            const int sb2 = sb1 == B_STAGES - 1 ? 0 : sb1 + 1;   // receives B(k+2)  (free: held B(k-1))
            const uint8_t* cB = sB + sb * SLAB;
            TG_FENCE();
            // column tiles 0 .. 5 in halves of four MFMAs; behind each half of the first four a direct load (B(k+2) goes to
            // the slab B(k-1) had), behind each first half the weight fragment of the column tile after next
#pragma unroll
            for (int tn = 0; tn < 6; ++tn) {
#pragma unroll
                for (int h = 0; h < 2; ++h) {
#pragma unroll
                    for (int j = 0; j < 4; ++j) acc[tn][4 * h + j] = mfma_e4m3(wf[tn & 3], af[4 * h + j], acc[tn][4 * h + j]);
                    TG_FENCE();
                    if (2 * tn + h < IT) load_b(2 * tn + h, k2, sb2);
                    if (h == 0) wf[(tn + 2) & 3] = read_w(tn + 2, cB);
                    TG_FENCE();
                }
            }
            // B(k+1) and A(k+1) have landed (all but the eight requests of B(k+2)); all my reads of B(k) are done
            __builtin_amdgcn_s_waitcnt(kWaitBut8);
            __builtin_amdgcn_s_waitcnt(kWaitLds);
            __builtin_amdgcn_s_barrier();
            TG_FENCE();
            // column tiles 6 and 7 by row group: each pair of MFMAs releases one activation fragment, which is refilled from
            // A(k+1) at once; the first two weight fragments of step k+1 are read first.  A(k)'s slab is free (every wave
            // read its fragments before this barrier) and receives A(k+2).
            const uint8_t* nA = sA + sa1 * SLAB;
            const uint8_t* nB = sB + sb1 * SLAB;
            wf[0] = read_w(0, nB);
            wf[1] = read_w(1, nB);
            TG_FENCE();
#pragma unroll
            for (int tm = 0; tm < TM; ++tm) {
                acc[6][tm] = mfma_e4m3(wf[2], af[tm], acc[6][tm]);
                acc[7][tm] = mfma_e4m3(wf[3], af[tm], acc[7][tm]);
                TG_FENCE();
                af[tm] = read_a(tm, nA);
                load_a(tm, k2, sa);
                TG_FENCE();
            }
            sa = sa1;
            sb = sb1;
        }
        // the fragment reads issued for the step after the last one are never used; keep the compiler from deleting the
        // loop-carried registers' last assignment in a way that changes the loop body
#pragma unroll
        for (int tm = 0; tm < TM; ++tm) asm volatile("" : : "v"(af[tm]));
        asm volatile("" : : "v"(wf[0]), "v"(wf[1]));

        // ---- epilogue, straight from the accumulators (as fp8_gemm_tile.h)
        const int rows_valid = min(BM, p.M - cm0);
        float scale = p.alpha;
        if (p.As) scale *= p.As[0];
        if (p.Bs) scale *= p.Bs[0];
        const bool vec_ok = p.vec_store != 0 && (p.N % 8) == 0;
        int dsts[TM];
#pragma unroll
        for (int tm = 0; tm < TM; ++tm) {
            const int rt = (tm * WGM + wm) * 16 + li;
            dsts[tm] = rt < rows_valid ? cm0 + rt : -1;
        }
        auto emit = [&](auto type_tag) __attribute__((always_inline)) {
            constexpr int OT = decltype(type_tag)::value;
            // (one call per row group instead of a loop: the body is too large for the unroller's budget, and a loop that
            // stays a loop would index the accumulators at run time, i.e. put them in scratch memory)
            auto rows = [&](auto tm_tag) __attribute__((always_inline)) {
                constexpr int tm = decltype(tm_tag)::value;
#pragma unroll
                for (int tp = 0; tp < TN / 2; ++tp) {
                    const int col = cn0 + wn * WTN + tp * 32 + lg * 8;
                    if (dsts[tm] < 0 || col >= p.N) continue;
                    store8(p.C, OT, dsts[tm], col, p.N, p.ldc, acc[2 * tp][tm] * scale, acc[2 * tp + 1][tm] * scale, p.beta, vec_ok);
                }
            };
            rows(std::integral_constant<int, 0>{}); rows(std::integral_constant<int, 1>{});
            rows(std::integral_constant<int, 2>{}); rows(std::integral_constant<int, 3>{});
            rows(std::integral_constant<int, 4>{}); rows(std::integral_constant<int, 5>{});
            rows(std::integral_constant<int, 6>{}); rows(std::integral_constant<int, 7>{});
        };
        if (p.out_type == OUT_BF16) emit(std::integral_constant<int, OUT_BF16>{});
        else if (p.out_type == OUT_F32) emit(std::integral_constant<int, OUT_F32>{});
        else if (p.out_type == OUT_F8) emit(std::integral_constant<int, OUT_F8>{});
        else emit(std::integral_constant<int, OUT_F16>{});
        if (!more) break;
#pragma unroll
        for (int tn = 0; tn < TN; ++tn)
#pragma unroll
            for (int tm = 0; tm < TM; ++tm) acc[tn][tm] = v4f{0.f, 0.f, 0.f, 0.f};
    }
#undef TG_FENCE
    __builtin_amdgcn_s_waitcnt(kWaitAll);  // the re-fetches past the end must land before the workgroup's LDS is released
#endif
}

// `tiles` 256x256 tiles on at most `max_workgroups` workgroups (the device's compute units).
inline hipError_t launch_tile256(const GemmParams& p, int tiles, int max_workgroups, hipStream_t stream) {
    if (p.kblocks < 2) return hipErrorInvalidValue;
    const int grid = tiles < max_workgroups ? tiles : max_workgroups;
    hipLaunchKernelGGL(fp8_gemm_tile256_kernel, dim3(grid, 1, 1), dim3(256, 1, 1), 0, stream, p);
    return hipGetLastError();
}

}  // namespace tg
