// Weight-streaming FP8 GEMM for skinny activations (M <= 64): C[m,n] = sum_k A[m,k] * B[n,k].
//
// The problem is bound by reading B once from HBM, so B never goes through LDS: every wave
// streams 16*RG rows of B straight from global memory into MFMA "row" operands (two 16-byte
// loads per lane and K step, non-temporal), multiplies them with the activation rows held as
// the MFMA "column" operand, and keeps 16x16 fp32 accumulators.  The NW (4, 8 or 16) waves of
// a workgroup take interleaved K steps of the same rows -- the workgroup reads NW*128
// contiguous bytes of each row per round -- and their accumulators are added through LDS, so
// that a 4096-wide layer still puts 16 waves with all their loads in flight on every CU
// without any traffic between workgroups.  For the rare shape where even that leaves the chip
// idle, K is also split across workgroups (grid.y): each writes raw fp32 sums to the
// workspace and a separate reduction kernel adds them in a fixed order.  The reference has no
// split-K schedule at all (wiki/cutile-knowledge-wiki/kernels/kernel-gemm.md:55-66).
#pragma once
#include "tg_device.h"

namespace tg {

template <int MT, int RG, int NW, bool BLOCKSCALE>
__global__ void __launch_bounds__(64 * NW) fp8_gemm_skinny_kernel(const GemmParams p) {
    __shared__ v4f s_red[NW - 1][RG * MT][64];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li = lane & 15, lg = lane >> 4;
    const int K = p.K, N = p.N, M = p.M;
    const int n_base = blockIdx.x * (16 * RG);

    int ks_begin = 0, ks_end = p.kblocks;
    if (p.split_k > 1) {
        ks_begin = blockIdx.y * p.ksteps_per_split;
        ks_end = min(ks_begin + p.ksteps_per_split, p.kblocks);
    }

    const uint8_t* wptr[RG];
#pragma unroll
    for (int rg = 0; rg < RG; ++rg) {
        const int n = min(n_base + rg * 16 + li, N - 1);
        wptr[rg] = p.B + (int64_t)n * K + lg * 16;
    }
    const uint8_t* aptr[MT];
    bool aok[MT];
    int arow[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int m = mt * 16 + li;
        aok[mt] = m < M;
        arow[mt] = min(m, M - 1);
        aptr[mt] = p.A + (int64_t)arow[mt] * K + lg * 16;
    }
    const float* bs_ptr[RG];
    if constexpr (BLOCKSCALE) {
#pragma unroll
        for (int rg = 0; rg < RG; ++rg) {
            const int nb = min((n_base + rg * 16) / 128, p.nblocks - 1);
            bs_ptr[rg] = p.Bs ? p.Bs + (int64_t)nb * p.kblocks : nullptr;
        }
    }

    v4f acc[RG][MT];
#pragma unroll
    for (int rg = 0; rg < RG; ++rg)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[rg][mt] = v4f{0.f, 0.f, 0.f, 0.f};

    v4i w_lo[RG], w_hi[RG], a_lo[MT], a_hi[MT];
    float sa[MT], sb[RG];
    auto load = [&](int kstep) {
        const int k0 = kstep * kKBlock;
        const bool ok0 = (k0 + lg * 16) < K, ok1 = (k0 + 64 + lg * 16) < K;
        const v4i zero = v4i{0, 0, 0, 0};
#pragma unroll
        for (int rg = 0; rg < RG; ++rg) {
            w_lo[rg] = ok0 ? __builtin_nontemporal_load(reinterpret_cast<const v4i*>(wptr[rg] + k0)) : zero;
            w_hi[rg] = ok1 ? __builtin_nontemporal_load(reinterpret_cast<const v4i*>(wptr[rg] + k0 + 64)) : zero;
        }
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            a_lo[mt] = (aok[mt] && ok0) ? *reinterpret_cast<const v4i*>(aptr[mt] + k0) : zero;
            a_hi[mt] = (aok[mt] && ok1) ? *reinterpret_cast<const v4i*>(aptr[mt] + k0 + 64) : zero;
        }
        if constexpr (BLOCKSCALE) {
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
                sa[mt] = p.As ? p.As[(int64_t)arow[mt] * p.kblocks + kstep] : 1.0f;
#pragma unroll
            for (int rg = 0; rg < RG; ++rg) sb[rg] = bs_ptr[rg] ? bs_ptr[rg][kstep] : 1.0f;
        }
    };

    int ks = ks_begin + wave;
    if (ks < ks_end) load(ks);
    while (ks < ks_end) {
        v8i wf[RG], af[MT];
        float sc[RG][MT];
#pragma unroll
        for (int rg = 0; rg < RG; ++rg) wf[rg] = join(w_lo[rg], w_hi[rg]);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) af[mt] = join(a_lo[mt], a_hi[mt]);
        if constexpr (BLOCKSCALE) {
#pragma unroll
            for (int rg = 0; rg < RG; ++rg)
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) sc[rg][mt] = sa[mt] * sb[rg];
        }
        const int nxt = ks + NW;
        if (nxt < ks_end) load(nxt);
#pragma unroll
        for (int rg = 0; rg < RG; ++rg)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                if constexpr (BLOCKSCALE) {
                    const v4f part = mfma_e4m3(wf[rg], af[mt], v4f{0.f, 0.f, 0.f, 0.f});
                    acc[rg][mt] += part * sc[rg][mt];
                } else {
                    acc[rg][mt] = mfma_e4m3(wf[rg], af[mt], acc[rg][mt]);
                }
            }
        ks = nxt;
    }

    // ---- add the waves' accumulators (wave 0 keeps the sum, in wave order)
    if (wave > 0) {
#pragma unroll
        for (int rg = 0; rg < RG; ++rg)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) s_red[wave - 1][rg * MT + mt][lane] = acc[rg][mt];
    }
    __syncthreads();
    if (wave != 0) return;
#pragma unroll
    for (int rg = 0; rg < RG; ++rg)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int w = 0; w < NW - 1; ++w) acc[rg][mt] += s_red[w][rg * MT + mt][lane];

    const bool vec_ok = p.vec_store != 0;
    if (p.split_k > 1) {
        float* mine = p.partials + (int64_t)blockIdx.y * M * N;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const int m = mt * 16 + li;
            if (m >= M) continue;
#pragma unroll
            for (int rg = 0; rg < RG; ++rg) {
                const int col = n_base + rg * 16 + lg * 4;
                if (col < N) store4(mine, OUT_F32, m, col, N, N, acc[rg][mt], 0.f, vec_ok);
            }
        }
        return;
    }
    float scale = p.alpha;
    if constexpr (!BLOCKSCALE) {
        if (p.As) scale *= p.As[0];
        if (p.Bs) scale *= p.Bs[0];
    }
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int m = mt * 16 + li;
        if (m >= M) continue;
#pragma unroll
        for (int rg = 0; rg < RG; ++rg) {
            const int col = n_base + rg * 16 + lg * 4;
            if (col < N) store4(p.C, p.out_type, m, col, N, p.ldc, acc[rg][mt] * scale, p.beta, vec_ok);
        }
    }
}

template <int MT, int RG, int NW, bool BLOCKSCALE>
inline hipError_t launch_skinny(const GemmParams& p, int grid_x, int grid_y, hipStream_t stream) {
    auto kern = fp8_gemm_skinny_kernel<MT, RG, NW, BLOCKSCALE>;
    hipLaunchKernelGGL(kern, dim3(grid_x, grid_y, 1), dim3(64 * NW, 1, 1), 0, stream, p);
    return hipGetLastError();
}

}  // namespace tg
