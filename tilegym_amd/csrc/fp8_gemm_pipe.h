// Persistent, register-pipelined 256x256 FP8 GEMM for gfx950, per-tensor scales, 2-byte output:
//   C[m,n] = scale * sum_k A[m,k] * B[n,k]      (both operands K-contiguous, K % 128 == 0)
//
// Same staging idea as fp8_gemm_tile_kernel (direct global->LDS loads, swizzle applied on the
// global side, MFMA "row" operand from the weights) but built around the 32x32x64 MFMA so
// that one K half-step (64 bytes of K) is a unit of its own:
//   * a wave's operand fragments for a half-step are 48 registers (64x64 + 128x64 bytes), so
//     two sets fit beside the 128 accumulator registers: the fragments of half-step s+1 are
//     read from LDS while the eight MFMAs of half-step s run;
//   * LDS holds four half-stages (A 256x64 + B 256x64 bytes each).  As soon as every wave has
//     its registers filled from a half-stage (one barrier per half-step) that half-stage is
//     refilled with the data of four half-steps later, so three half-stages (96 KiB per
//     compute unit) are always in flight;
//   * one workgroup per compute unit walks over its tiles (persistent grid) and the stream of
//     half-steps runs on across tile boundaries: while a tile's last MFMAs execute, the loads
//     of the next tile are already in flight, and the tile's output (accumulators regrouped
//     with v_permlane32_swap so that a lane owns 8 consecutive columns, scaled, rounded, one
//     16-byte store per lane) drains to memory while the next tile is being computed.  A
//     non-persistent grid leaves the matrix pipe idle for the whole write-out of every tile,
//     because all compute units reach it at the same time.
// A half-stage row is 64 bytes (four 16-byte chunks); chunk c of row r sits at chunk position
// c ^ ((r >> 2) & 3), which makes ds_read_b128 of 32 consecutive rows conflict free
// (measured: 4.0 clocks per wave-read).
#pragma once
#include "fp8_gemm_tile.h"

typedef float v16f __attribute__((ext_vector_type(16)));
typedef unsigned v2u __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float v8f __attribute__((ext_vector_type(8)));

namespace tg {

// 32x32x64 e4m3 MFMA, fp32 accumulation.  `w` supplies 32 rows of the result (lane l: row
// l%32, K bytes of K-group l/32), `x` the 32 columns; lane l receives column l%32 and rows
// 8*(v/4) + 4*(l/32) + v%4 for v = 0..15 (checked on hardware against an integer reference).
__device__ __forceinline__ v16f mfma32_e4m3(v8i w, v8i x, v16f acc) {
    return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(w, x, acc, 0, 0, 0, 0, 0, 0);
}

constexpr int kPipeBM = 256, kPipeBN = 256;
constexpr int kPipeHalf = 64;               // bytes of K per half-step
constexpr int kPipeSlab = 256 * kPipeHalf;  // one operand of one half-stage: 16 KiB
constexpr int kPipeStages = 4;              // half-stages in LDS

// NW waves per workgroup: 8 (wave tile 64x128, two waves per SIMD).  A four-wave layout (wave tile
// 128x128, 256 accumulator registers in the AGPR half of the file) is expressible with the same
// code but is not instantiated: the compiler spills it.  NL of the waves issue the direct loads.
template <int NW, int NL>
__global__ void __launch_bounds__(64 * NW, 1) fp8_gemm_pipe_kernel(const GemmParams p) {
#if defined(__HIP_DEVICE_COMPILE__)
    constexpr int BM = kPipeBM, BN = kPipeBN, WGM = NW / 2, WTM = BM / WGM, WTN = 128;
    constexpr int MB = WTM / 32, NB = WTN / 32;  // 32x32 blocks per wave tile
    constexpr int NMF = MB * NB;                 // MFMAs per wave and half-step
    constexpr int GPW = 16 / NL;                 // 16-row groups per loader wave and operand
    constexpr int LPB = 2 * GPW;                 // direct loads per loader wave and half-stage
    constexpr int NSTORE = NMF * 2;              // 16-byte stores per wave and full tile
    static_assert((NW == 8 && (NL == 8 || NL == 4)) || (NW == 4 && NL == 4), "wave layout");

    __shared__ __align__(1024) uint8_t smem[kPipeStages * 2 * kPipeSlab];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave % WGM, wn = wave / WGM;
    const int K = p.K;
    const int tiles_n = (p.N + BN - 1) / BN, tiles_m = (p.M + BM - 1) / BM;
    const int ntiles = tiles_m * tiles_n, G = gridDim.x;

    // Tile q of the persistent sequence (workgroup b takes q = b, b + G, ...).  With G a multiple
    // of 8 the workgroups of one XCD work, in every round, on 32 consecutive tiles of the
    // grouped order (8 row tiles x 4 column tiles): they share their A and B slabs in that L2.
    auto decode = [&](int q, int& m0, int& n0) {
        const int pid = xcd_remap(q, ntiles);
        constexpr int GM = 8;
        const int width = GM * tiles_n;
        const int first_m = (pid / width) * GM;
        const int gsz = min(tiles_m - first_m, GM);
        m0 = (first_m + (pid % width) % gsz) * BM;
        n0 = ((pid % width) / gsz) * BN;
    };

    // ---------------------------------------------------------------- load cursor
    // One direct load fills 16 slab rows: lane l lands at row l/4, chunk position l%4, and so
    // fetches logical chunk (l%4) ^ ((row >> 2) & 3) = (l%4) ^ (l >> 4).
    const bool loader = wave < NL;
    const int lrow = lane >> 2, lchunk = (lane & 3) ^ (lane >> 4);
    const int T = 2 * p.kblocks;  // half-steps per tile
    uint32_t a_off[GPW], b_off[GPW];
    auto set_offsets = [&](int q) {
        int m0, n0;
        decode(q, m0, n0);
        const int rows_valid = min(BM, p.M - m0);
#pragma unroll
        for (int i = 0; i < GPW; ++i) {
            const int r = ((wave % NL) * GPW + i) * 16 + lrow;
            a_off[i] = (uint32_t)(m0 + min(r, rows_valid - 1)) * (uint32_t)K + lchunk * 16;
            b_off[i] = (uint32_t)min(n0 + r, p.N - 1) * (uint32_t)K + lchunk * 16;
        }
    };
    int ld_q = blockIdx.x, ld_t = 0;
    bool ld_more = true;
    set_offsets(ld_q);
    const v4i rsrc_a = make_rsrc(p.A), rsrc_b = make_rsrc(p.B);
    const uint32_t smem_addr = lds_address(smem);
    // Issue the loads of the cursor's half-step into half-stage h and advance the cursor.  Past
    // the last half-step of the last tile the same data is fetched again into an idle
    // half-stage, which keeps the count of loads in flight (and so the waits below) uniform.
    // Direct load i (0 .. LPB-1; the first GPW fill the A slab, the others the B slab) of the
    // cursor's half-step into half-stage h.
    auto dma = [&](int h, int i) {
        if (loader) {
            const int k0 = ld_t * kPipeHalf;
            const uint32_t dst = smem_addr + h * (2 * kPipeSlab) + (wave % NL) * GPW * 1024;
            if (i < GPW) direct_load_b128(rsrc_a, dst + i * 1024, a_off[i], k0);
            else direct_load_b128(rsrc_b, dst + kPipeSlab + (i - GPW) * 1024, b_off[i - GPW], k0);
        }
    };
    auto issue_loads = [&](int h) {
#pragma unroll
        for (int i = 0; i < LPB; ++i) dma(h, i);
    };
    auto advance_cursor = [&]() {
        if (ld_more) {
            if (++ld_t == T) {
                if (ld_q + G < ntiles) {
                    ld_q += G;
                    ld_t = 0;
                    set_offsets(ld_q);
                } else {
                    ld_more = false;
                    ld_t = T - 1;
                }
            }
        }
    };
    auto issue_next = [&](int h) {
        issue_loads(h);
        advance_cursor();
    };

    // ---------------------------------------------------------------- fragment reads
    const int lr = lane & 31, lg = lane >> 5;
    const uint32_t frag0 = lr * kPipeHalf + (((2 * lg) ^ ((lr >> 2) & 3)) << 4);
    const uint32_t a_base = wm * WTM * kPipeHalf, b_base = kPipeSlab + wn * WTN * kPipeHalf;
    v8i fa[2][MB], fb[2][NB];
    auto read_fb = [&](int set, int h, int nb) {
        const uint8_t* s0 = smem + h * (2 * kPipeSlab) + frag0 + b_base + nb * 32 * kPipeHalf;
        const uint8_t* s1 = smem + h * (2 * kPipeSlab) + (frag0 ^ 16) + b_base + nb * 32 * kPipeHalf;
        fb[set][nb] = join(*reinterpret_cast<const v4i*>(s0), *reinterpret_cast<const v4i*>(s1));
    };
    auto read_fa = [&](int set, int h, int mb) {
        const uint8_t* s0 = smem + h * (2 * kPipeSlab) + frag0 + a_base + mb * 32 * kPipeHalf;
        const uint8_t* s1 = smem + h * (2 * kPipeSlab) + (frag0 ^ 16) + a_base + mb * 32 * kPipeHalf;
        fa[set][mb] = join(*reinterpret_cast<const v4i*>(s0), *reinterpret_cast<const v4i*>(s1));
    };
    auto read_frags = [&](int set, int h) {
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) read_fb(set, h, nb);
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) read_fa(set, h, mb);
    };

    v16f acc[NB][MB];
    auto zero_acc = [&]() {
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[nb][mb][v] = 0.f;
    };
    auto mma1 = [&](int set, int nb, int mb) { acc[nb][mb] = mfma32_e4m3(fb[set][nb], fa[set][mb], acc[nb][mb]); };

    // vmcnt(n): of this wave's vector memory operations all but the n most recent are complete
    // (loads complete in issue order).
    auto vm = [](int n) constexpr { return 0x0F70 | (n & 15) | ((n >> 4) << 14); };
    constexpr int kWait3 = vm(3 * LPB), kWait2 = vm(2 * LPB), kWait2Stores = vm(2 * LPB + NSTORE);
    static_assert(2 * LPB + NSTORE < 64, "vmcnt is a 6-bit counter");
    constexpr int kWaitAll = 0x0F70, kWaitLds = 0xC07F;

    // ---------------------------------------------------------------- epilogue of one tile
    float scale = p.alpha;
    if (p.As) scale *= p.As[0];
    if (p.Bs) scale *= p.Bs[0];
    // have the value in a scalar register now, not at its first use inside the tile loop
    scale = __uint_as_float(__builtin_amdgcn_readfirstlane(__float_as_uint(scale)));
    const bool is_bf16 = p.out_type == OUT_BF16;
    const bool vec_ok = p.vec_store != 0 && (p.N % 8) == 0;
    uint16_t* const Cout = reinterpret_cast<uint16_t*>(p.C);
    // A lane holds, per 32x32 block, row m = lr and columns 8*qd + 4*lg + j (qd, j = 0..3).
    // v_permlane32_swap of the registers of qd = 2*pr and 2*pr + 1 gives lanes 0..31 the eight
    // columns 16*pr .. 16*pr + 7 and lanes 32..63 the eight columns 16*pr + 8 .. 16*pr + 15.
    auto write_tile = [&](int m0, int n0) {
        const int rows_valid = min(BM, p.M - m0);
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                for (int pr = 0; pr < 2; ++pr) {
                    v8f x;
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const v2u r = __builtin_amdgcn_permlane32_swap(__float_as_uint(acc[nb][mb][8 * pr + j]),
                                                                       __float_as_uint(acc[nb][mb][8 * pr + 4 + j]), false, false);
                        x[j] = __uint_as_float(r[0]) * scale;
                        x[4 + j] = __uint_as_float(r[1]) * scale;
                    }
                    const int rt = wm * WTM + mb * 32 + lr;
                    const int col = n0 + wn * WTN + nb * 32 + 16 * pr + 8 * lg;
                    if (rt >= rows_valid || col >= p.N) continue;
                    v4i packed;
                    if (is_bf16) packed = __builtin_bit_cast(v4i, __builtin_convertvector(x, bf16x8));
                    else packed = __builtin_bit_cast(v4i, __builtin_convertvector(x, f16x8));
                    uint16_t* out = Cout + (int64_t)(m0 + rt) * p.N + col;
                    if (vec_ok && col + 7 < p.N) {
                        *reinterpret_cast<v4i*>(out) = packed;
                    } else {
                        for (int j = 0; j < 8 && col + j < p.N; ++j)
                            out[j] = (uint16_t)((uint32_t)packed[j >> 1] >> ((j & 1) * 16));
                    }
                }
    };

    // ---------------------------------------------------------------- pipeline
    // At the top of half-step s (every wave past the barrier): registers (set s%2) hold the
    // fragments of s; half-stage s%4 is free (all waves hold s); half-stage (s+1)%4 holds s+1
    // (landed); s+2 and s+3 are in flight.
    //   body s:  8 MFMAs of s, and between them: the loads of s+4 into half-stage s%4, the
    //            fragment reads of s+1 into the other register set, the cursor update -- a wave's
    //            memory instructions issue while the matrix pipe works on the MFMAs of the two
    //            waves of its SIMD
    //            wait: own reads done, own loads of s+2 landed;  barrier
    issue_next(0);
    issue_next(1);
    issue_next(2);
    issue_next(3);
    if (loader) __builtin_amdgcn_s_waitcnt(kWait3);
    __builtin_amdgcn_s_barrier();
    read_frags(0, 0);
    __builtin_amdgcn_s_waitcnt(kWaitLds);
    if (loader) __builtin_amdgcn_s_waitcnt(kWait2);
    __builtin_amdgcn_s_barrier();

    // `stores_behind`: the 16 output stores of the previous tile were issued after the loads of
    // that tile's last body; in the next two bodies they sit between the loads being waited for
    // and the most recent ones and are allowed to stay in flight.
#define TG_FENCE __builtin_amdgcn_sched_barrier(0)
    auto body = [&](int set, int h_free, int h_read, bool stores_behind) {
        const int o = set ^ 1;
        // One memory instruction group behind every MFMA: first the fragment reads of s+1 (one
        // 32-row fragment = two ds_read_b128), then the direct loads of s+4 (a direct load blocks
        // the wave for ~40 clocks while the texture unit takes its 64 addresses; an MFMA occupies
        // the matrix pipe for 64).
        constexpr int DMA0 = NMF - LPB;  // first MFMA slot that carries a direct load
#pragma unroll
        for (int i = 0; i < NMF; ++i) {
            // Two waves share a SIMD and the older one wins every tie for the matrix pipe: left
            // alone, it would issue all its MFMAs first and the younger one would then run with
            // nothing to cover its memory-instruction stalls.  The older wave therefore alternates
            // between a higher and a lower priority than the younger one's constant 1.
            if constexpr (NW == 8) {
                if (wave < 4) {
                    if (i & 1) __builtin_amdgcn_s_setprio(0);
                    else __builtin_amdgcn_s_setprio(2);
                }
            }
            mma1(set, i / MB, i % MB);
            if (i < NB) read_fb(o, h_read, i);
            else if (i < NB + MB) read_fa(o, h_read, i - NB);
            if (i >= DMA0) {
                TG_FENCE;
                dma(h_free, i - DMA0);
            }
            TG_FENCE;
        }
        advance_cursor();
        TG_FENCE;
        __builtin_amdgcn_s_waitcnt(kWaitLds);
        if (loader) {
            if (stores_behind) __builtin_amdgcn_s_waitcnt(kWait2Stores);
            else __builtin_amdgcn_s_waitcnt(kWait2);
        }
        __builtin_amdgcn_s_barrier();
    };
#undef TG_FENCE

    if (NW == 8 && wave >= 4) __builtin_amdgcn_s_setprio(1);
    int cur_q = blockIdx.x, m0, n0;
    decode(cur_q, m0, n0);
    zero_acc();
    bool prev_full = false;  // the previous tile of this workgroup issued exactly NSTORE stores per wave
    int s = 0, t = 0;
    for (;;) {
        body(0, s & 3, (s + 1) & 3, prev_full && t < 2);
        body(1, (s + 1) & 3, (s + 2) & 3, prev_full && t + 1 < 2);
        s += 2;
        t += 2;
        if (t == T) {
            write_tile(m0, n0);
            prev_full = vec_ok && T >= 4 && m0 + BM <= p.M && n0 + BN <= p.N;
            cur_q += G;
            if (cur_q >= ntiles) break;
            decode(cur_q, m0, n0);
            zero_acc();
            t = 0;
        }
    }
    __builtin_amdgcn_s_waitcnt(kWaitAll);  // the re-fetched loads still target this workgroup's LDS
#endif
}

template <int NW, int NL>
inline hipError_t launch_pipe(const GemmParams& p, int grid_x, hipStream_t stream) {
    auto kern = fp8_gemm_pipe_kernel<NW, NL>;
    hipLaunchKernelGGL(kern, dim3(grid_x, 1, 1), dim3(64 * NW, 1, 1), 0, stream, p);
    return hipGetLastError();
}

}  // namespace tg
