// Weight-streaming FP8 GEMM for skinny activations (M <= 64), second generation:
// C[m,n] = sum_k A[m,k] * B[n,k], bound by reading B once from HBM.
//
// Measured on MI355X: a wave-wide load whose 64 lanes cover 1 KiB of ONE weight row streams at
// ~6.5 TB/s, while loads shaped like the MFMA operand (16 rows x 64 bytes per instruction) stay
// near 4.5 TB/s.  So the weights are fetched with direct global->LDS loads of one row x 1 KiB per
// instruction and LDS does the transposition into the MFMA operand layout: a wave owns a
// private 16-row x 1 KiB LDS buffer (or two, double buffered), fills it with 16 such loads,
// waits for its own loads only (no workgroup barrier in the loop) and runs 8 K steps of
// 16x16x128 MFMAs from it.  Lane l of the load for row r fetches 16-byte chunk l ^ r of the
// 1 KiB piece, which makes the later fragment reads (16 rows, same logical chunk) bank-conflict
// free.  The 4 waves of a workgroup take interleaved 1 KiB pieces of the same 16 rows; their
// accumulators are added through LDS at the end.  K can additionally be split across
// workgroups (grid.y) into fp32 partial sums reduced by a second kernel.
#pragma once
#include "fp8_gemm_tile.h"

namespace tg {

constexpr int kStreamChunk = 1024;  // bytes of one row fetched by one load instruction

template <int MT, int NBUF, bool BLOCKSCALE, int NW = 4>
__global__ void __launch_bounds__(64 * NW) fp8_gemm_stream_kernel(const GemmParams p) {
#if defined(__HIP_DEVICE_COMPILE__)
    constexpr int BUF = 16 * kStreamChunk;
    __shared__ __align__(1024) uint8_t sW[NW * NBUF * BUF];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li = lane & 15, lg = lane >> 4;
    const int K = p.K, N = p.N, M = p.M;
    // weight rows per workgroup: 16, or fewer so that the workgroups come out even over the compute units (6144 rows:
    // 384 workgroups of 16 rows put two on half of the compute units and one on the others, 512 of 12 rows two on each).
    // The rows a workgroup does not own are requested from beyond the descriptor's range (no memory request) and not stored.
    const int R = p.wave_rows > 0 ? p.wave_rows : 16;
    const int n_base = blockIdx.x * R;
    const int n_end = min(n_base + R, N);
    const int nchunks_total = (K + kStreamChunk - 1) / kStreamChunk;

    int c_begin = 0, c_end = nchunks_total;
    if (p.split_k > 1) {  // ksteps_per_split counts 1 KiB pieces here
        c_begin = blockIdx.y * p.ksteps_per_split;
        c_end = min(c_begin + p.ksteps_per_split, nchunks_total);
    }

    // per-row byte offsets of this lane's 16-byte chunk: row r, logical chunk lane ^ r
    const v4i rsrc_b = make_rsrc(p.B);
    uint8_t* my_buf = sW + wave * NBUF * BUF;
    const uint32_t my_lds = lds_address(my_buf);

    auto issue_chunk = [&](int c, int buf) {
        const int k0 = c * kStreamChunk;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int n = min(n_base + r, N - 1);
            const int j = lane ^ r;
            const uint32_t voff = n_base + r < n_end ? (uint32_t)n * (uint32_t)K + j * 16 : 0x80000000u;
            const uint32_t dst = my_lds + buf * BUF + r * kStreamChunk;
            if (k0 + j * 16 < K) {
                direct_load_b128_nt(rsrc_b, dst, voff, k0);
            } else {  // past the end of K: zeros
                *reinterpret_cast<v4i*>(my_buf + buf * BUF + r * kStreamChunk + lane * 16) = v4i{0, 0, 0, 0};
            }
        }
    };

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
    const float* bs_ptr = nullptr;
    if constexpr (BLOCKSCALE) {
        const int nb = min(n_base / 128, p.nblocks - 1);
        bs_ptr = p.Bs ? p.Bs + (int64_t)nb * p.kblocks : nullptr;
    }

    v4f acc[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[mt] = v4f{0.f, 0.f, 0.f, 0.f};

    auto load_act = [&](int kstep, v4i* lo, v4i* hi) {
        const int k0 = kstep * kKBlock;
        const bool ok0 = (k0 + lg * 16) < K, ok1 = (k0 + 64 + lg * 16) < K;
        const v4i zero = v4i{0, 0, 0, 0};
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            lo[mt] = (aok[mt] && ok0) ? *reinterpret_cast<const v4i*>(aptr[mt] + k0) : zero;
            hi[mt] = (aok[mt] && ok1) ? *reinterpret_cast<const v4i*>(aptr[mt] + k0 + 64) : zero;
        }
    };

    constexpr int SPC = kStreamChunk / kKBlock;  // K steps per 1 KiB piece
    // M <= 16: the activation fragments of a whole piece are fetched up front (before the piece
    // after it is requested: loads complete in order, so an activation load issued behind the
    // next piece's direct loads would have to wait for them).  Larger M: one K step ahead.
    constexpr bool PRELOAD = MT == 1;
    v4i pa_lo[PRELOAD ? SPC : 1], pa_hi[PRELOAD ? SPC : 1];
    // block scales of a whole piece travel with the preloaded activations: fetched before the wait
    // for the weights, not between the MFMAs
    float psc[(PRELOAD && BLOCKSCALE) ? SPC : 1];
    auto preload_act = [&](int c) {
        if constexpr (PRELOAD) {
#pragma unroll
            for (int s = 0; s < SPC; ++s) load_act(c * SPC + s, &pa_lo[s], &pa_hi[s]);
            if constexpr (BLOCKSCALE) {
#pragma unroll
                for (int s = 0; s < SPC; ++s) {
                    const int ks = min(c * SPC + s, p.kblocks - 1);
                    const float sb = bs_ptr ? bs_ptr[ks] : 1.0f;
                    psc[s] = (p.As ? p.As[(int64_t)arow[0] * p.kblocks + ks] : 1.0f) * sb;
                }
            }
        }
    };
    auto mma_step = [&](int ks, v8i wf, const v8i* af, int s_in_piece) {
        float sc[MT];
        if constexpr (BLOCKSCALE && PRELOAD) {
            sc[0] = psc[s_in_piece];
        } else if constexpr (BLOCKSCALE) {
            const float sb = bs_ptr ? bs_ptr[ks] : 1.0f;
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
                sc[mt] = (p.As ? p.As[(int64_t)arow[mt] * p.kblocks + ks] : 1.0f) * sb;
        }
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            if constexpr (BLOCKSCALE) {
                const v4f part = mfma_e4m3(wf, af[mt], v4f{0.f, 0.f, 0.f, 0.f});
                acc[mt] += part * sc[mt];
            } else {
                acc[mt] = mfma_e4m3(wf, af[mt], acc[mt]);
            }
        }
    };
    auto compute_chunk = [&](int c, int buf) {
        const uint8_t* base = my_buf + buf * BUF + li * kStreamChunk;
        const int ks0 = c * SPC;
        const int nks = min(SPC, p.kblocks - ks0);
        if constexpr (PRELOAD) {
#pragma unroll
            for (int s = 0; s < SPC; ++s) {
                if (s < nks) {
                    const int j0 = s * 8 + lg, j1 = j0 + 4;
                    const v8i wf = join(*reinterpret_cast<const v4i*>(base + ((j0 ^ li) << 4)),
                                        *reinterpret_cast<const v4i*>(base + ((j1 ^ li) << 4)));
                    const v8i af = join(pa_lo[s], pa_hi[s]);
                    mma_step(ks0 + s, wf, &af, s);
                }
            }
        } else {
            v4i a_lo[MT], a_hi[MT];
            load_act(ks0, a_lo, a_hi);
            for (int s = 0; s < nks; ++s) {
                v8i af[MT];
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) af[mt] = join(a_lo[mt], a_hi[mt]);
                if (s + 1 < nks) load_act(ks0 + s + 1, a_lo, a_hi);
                const int j0 = s * 8 + lg, j1 = j0 + 4;
                const v8i wf = join(*reinterpret_cast<const v4i*>(base + ((j0 ^ li) << 4)),
                                    *reinterpret_cast<const v4i*>(base + ((j1 ^ li) << 4)));
                mma_step(ks0 + s, wf, af, 0);
            }
        }
    };

    // ---- stream this wave's 1 KiB pieces
    constexpr int kWaitMine = 0x0070;                                   // vmcnt(0) lgkmcnt(0)
    constexpr int kWaitAllBut16 = 0x0F70 | (16 & 15) | ((16 >> 4) << 14);  // vmcnt(16)
    constexpr int kWaitLds = 0xC07F;                                    // lgkmcnt(0)
    int c = c_begin + wave;
    if constexpr (NBUF == 1) {
        for (; c < c_end; c += NW) {
            preload_act(c);
            issue_chunk(c, 0);
            __builtin_amdgcn_s_waitcnt(kWaitMine);  // my loads and zero fills have landed
            compute_chunk(c, 0);
            __builtin_amdgcn_s_waitcnt(kWaitLds);   // my LDS reads are done before the refill
        }
    } else {
        int buf = 0;
        if (c < c_end) issue_chunk(c, 0);
        for (; c < c_end; c += NW) {
            const int nxt = c + NW;
            preload_act(c);
            if (nxt < c_end) {
                issue_chunk(nxt, buf ^ 1);
                __builtin_amdgcn_s_waitcnt(kWaitAllBut16);  // everything older than the next piece
                __builtin_amdgcn_s_waitcnt(kWaitLds);
            } else {
                __builtin_amdgcn_s_waitcnt(kWaitMine);
            }
            compute_chunk(c, buf);
            __builtin_amdgcn_s_waitcnt(kWaitLds);
            buf ^= 1;
        }
    }

    // ---- add the four waves' accumulators through LDS (each wave's buffer is its own until here)
    __syncthreads();
    v4f* red = reinterpret_cast<v4f*>(sW);
    if (wave > 0) {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) red[((wave - 1) * MT + mt) * 64 + lane] = acc[mt];
    }
    __syncthreads();
    if (wave != 0) return;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int w = 0; w < NW - 1; ++w) acc[mt] += red[(w * MT + mt) * 64 + lane];

    const bool vec_ok = p.vec_store != 0 && (R & 3) == 0;  // (a lane's four outputs are all the workgroup's, or with R % 4 != 0 some of them)
    const int col = n_base + lg * 4;
    if (p.split_k > 1) {
        float* mine = p.partials + (int64_t)blockIdx.y * M * N;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const int m = mt * 16 + li;
            if (m < M && col < n_end) store4(mine, OUT_F32, m, col, n_end, N, acc[mt], 0.f, vec_ok);
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
        if (m < M && col < n_end) store4(p.C, p.out_type, m, col, n_end, p.ldc, acc[mt] * scale, p.beta, vec_ok);
    }
#endif
}

// Wide variant for M <= 16 and many weight rows: a workgroup owns 64 weight
// rows, wave w the rows 16w .. 16w+15 over the workgroup's whole K range, so no cross-wave
// reduction is needed -- and all four waves multiply the SAME activation piece, which is fetched
// once per workgroup into a shared 16 KiB LDS buffer with the same row-wise direct loads as the
// weights.  In the kernel above every wave loads its own activation fragments in MFMA layout: 16
// rows x 64 bytes per instruction, i.e. 16 half-used cache lines, as many load instructions as for
// the weights themselves (measured: 33 us instead of 26 us at M = 16 on the 28672 x 4096 layer).
// Here the activations cost a quarter of the weights' load instructions, each over full lines.
// Only rows < M of the activation buffer are filled; the other columns of the MFMA result are
// never stored.
template <bool BLOCKSCALE>
__global__ void __launch_bounds__(256) fp8_gemm_stream_wide_kernel(const GemmParams p) {
#if defined(__HIP_DEVICE_COMPILE__)
    constexpr int NW = 4;
    constexpr int BUF = 16 * kStreamChunk;
    constexpr int SPC = kStreamChunk / kKBlock;
    __shared__ __align__(1024) uint8_t sW[NW * BUF];
    __shared__ __align__(1024) uint8_t sA[BUF];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li = lane & 15, lg = lane >> 4;
    const int K = p.K, N = p.N, M = p.M;
    const int n_base = blockIdx.x * 64 + wave * 16;
    const int nchunks_total = (K + kStreamChunk - 1) / kStreamChunk;
    int c_begin = 0, c_end = nchunks_total;
    if (p.split_k > 1) {  // ksteps_per_split counts 1 KiB pieces here
        c_begin = blockIdx.y * p.ksteps_per_split;
        c_end = min(c_begin + p.ksteps_per_split, nchunks_total);
    }
    const v4i rsrc_b = make_rsrc(p.B), rsrc_a = make_rsrc(p.A);
    uint8_t* my_buf = sW + wave * BUF;
    const uint32_t my_lds = lds_address(my_buf), a_lds = lds_address(sA);
    const int rows_a = min(M, 16);

    auto issue = [&](int c) {
        const int k0 = c * kStreamChunk;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int n = min(n_base + r, N - 1);
            const int j = lane ^ r;
            if (k0 + j * 16 < K) direct_load_b128_nt(rsrc_b, my_lds + r * kStreamChunk, (uint32_t)n * (uint32_t)K + j * 16, k0);
            else *reinterpret_cast<v4i*>(my_buf + r * kStreamChunk + lane * 16) = v4i{0, 0, 0, 0};
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int r = wave * 4 + i;  // wave-uniform
            if (r < rows_a) {
                const int j = lane ^ r;
                if (k0 + j * 16 < K) direct_load_b128(rsrc_a, a_lds + r * kStreamChunk, (uint32_t)r * (uint32_t)K + j * 16, k0);
                else *reinterpret_cast<v4i*>(sA + r * kStreamChunk + lane * 16) = v4i{0, 0, 0, 0};
            }
        }
    };

    // block scales: the wave's 16 weight rows lie in one 128-row block (one scalar per K step), the
    // activation scale belongs to the lane's column (row li of A); both are fetched per piece
    // before the wait for the weights
    const float* bs_ptr = nullptr;
    const float* as_ptr = nullptr;
    if constexpr (BLOCKSCALE) {
        bs_ptr = p.Bs ? p.Bs + (int64_t)min(n_base / 128, p.nblocks - 1) * p.kblocks : nullptr;
        as_ptr = p.As ? p.As + (int64_t)min(li, M - 1) * p.kblocks : nullptr;
    }
    v4f acc = v4f{0.f, 0.f, 0.f, 0.f};
    constexpr int kWaitMine = 0x0070;  // vmcnt(0) lgkmcnt(0)
    constexpr int kWaitLds = 0xC07F;   // lgkmcnt(0)
    // All of a piece's fragments go to registers first; the buffers are then requested again for the next piece and the
    // MFMAs of this piece run while those loads are in flight (2 - 3 % shorter launches than refilling after the MFMAs).
    if (c_begin < c_end) issue(c_begin);
    for (int c = c_begin; c < c_end; ++c) {
        float psc[BLOCKSCALE ? SPC : 1];
        if constexpr (BLOCKSCALE) {
#pragma unroll
            for (int s = 0; s < SPC; ++s) {
                const int ks = min(c * SPC + s, p.kblocks - 1);
                psc[s] = (as_ptr ? as_ptr[ks] : 1.0f) * (bs_ptr ? bs_ptr[ks] : 1.0f);
            }
        }
        __builtin_amdgcn_s_waitcnt(kWaitMine);
        __builtin_amdgcn_s_barrier();  // every wave's share of the activation piece has landed
        const uint8_t* wb = my_buf + li * kStreamChunk;
        const uint8_t* ab = sA + li * kStreamChunk;
        v8i wf[SPC], af[SPC];
#pragma unroll
        for (int s = 0; s < SPC; ++s) {
            const int j0 = ((s * 8 + lg) ^ li) << 4, j1 = ((s * 8 + 4 + lg) ^ li) << 4;
            wf[s] = join(*reinterpret_cast<const v4i*>(wb + j0), *reinterpret_cast<const v4i*>(wb + j1));
            af[s] = join(*reinterpret_cast<const v4i*>(ab + j0), *reinterpret_cast<const v4i*>(ab + j1));
        }
        __builtin_amdgcn_s_waitcnt(kWaitLds);
#pragma unroll
        for (int s = 0; s < SPC; ++s) asm volatile("" : "+v"(wf[s]), "+v"(af[s]));
        __builtin_amdgcn_s_barrier();  // every wave holds its fragments: the buffers may be refilled
        if (c + 1 < c_end) issue(c + 1);
        const int nks = min(SPC, p.kblocks - c * SPC);
#pragma unroll
        for (int s = 0; s < SPC; ++s) {
            if (s < nks) {
                if constexpr (BLOCKSCALE) acc += mfma_e4m3(wf[s], af[s], v4f{0.f, 0.f, 0.f, 0.f}) * psc[s];
                else acc = mfma_e4m3(wf[s], af[s], acc);
            }
        }
    }
    const bool vec_ok = p.vec_store != 0;
    const int col = n_base + lg * 4, m = li;
    if (m >= M || col >= N) return;
    if (p.split_k > 1) {
        store4(p.partials + (int64_t)blockIdx.y * M * N, OUT_F32, m, col, N, N, acc, 0.f, vec_ok);
        return;
    }
    float scale = p.alpha;
    if constexpr (!BLOCKSCALE) {
        if (p.As) scale *= p.As[0];
        if (p.Bs) scale *= p.Bs[0];
    }
    store4(p.C, p.out_type, m, col, N, p.ldc, acc * scale, p.beta, vec_ok);
#endif
}

// One float at a wave-uniform address: a scalar load.
__device__ __forceinline__ float stream_uniform_f32(const float* p) {
    return *(const __attribute__((address_space(4))) float*)(uintptr_t)p;
}

// The wide variant with two half-size buffers per wave: pieces of 512 bytes of K (four K steps), piece c+1 in flight
// while piece c is multiplied, piece c+2 requested as soon as piece c's fragments are in registers.  A load instruction
// covers two rows x 512 bytes (lanes 0 - 31 one row, lanes 32 - 63 the next).  Needs K % 128 == 0 (a last piece of one to
// three K steps is loaded with the same number of instructions and multiplied over its valid steps): every wave issues a
// fixed number of loads per piece (eight for its weight rows, two per 16 activation rows for its share of those, one per
// 16 activation rows for their block scales), which the vmcnt waits count.
// Workgroup b starts at piece b % (pieces) of its K range and wraps around: with all workgroups at the same K offset of
// rows that lie a power of two apart (K = 4096, 8192) the requests of one moment fall on few memory channels
// (28672 x 4096 at M = 1: 22.1 us in step, 20.6 us staggered; 8192 x 8192: 17.1 and 15.7).  The sum over K is the same
// set of products added in a rotated order.
// Four waves per workgroup (64 weight rows).  Measured with 4 .. 8: four is the fastest everywhere (28672 x 4096:
// 22.1 / 26.0 / 29.3 / 24.6 / 25.4 us for 4 / 5 / 6 / 7 / 8 waves, although seven waves make exactly one workgroup per
// compute unit).
// MT tiles of 16 activation rows (M <= 16 MT): the activation piece in LDS grows to 16 MT rows, every wave multiplies
// its weight fragments with all of them.  Built for MT = 1 and 2; MT = 4 works and is slower than the tile kernels.
// The wide kernel's LDS table of activation scales: none at all for per-tensor scales, so that the per-tensor kernel's
// 64 + 16 KiB of buffers are exactly half of a compute unit's 160 KiB and two workgroups share one.
template <bool BLOCKSCALE, int FLOATS>
struct StreamScaleTable {
    __device__ static __forceinline__ float* get() {
        __shared__ __align__(16) float table[FLOATS];
        return table;
    }
};
template <int FLOATS>
struct StreamScaleTable<false, FLOATS> {
    __device__ static __forceinline__ float* get() { return nullptr; }
};

template <bool BLOCKSCALE, int MT>
__global__ void __launch_bounds__(256) fp8_gemm_stream_wide_db_kernel(const GemmParams p) {
#if defined(__HIP_DEVICE_COMPILE__)
    constexpr int NW = 4;
    constexpr int PIECE = 512;                 // bytes of K per piece and row
    constexpr int BUF = 16 * PIECE;            // 8 KiB: a wave's 16 weight rows
    constexpr int ABUF = MT * BUF;             // the activation piece
    constexpr int SPC = PIECE / kKBlock;       // 4 K steps per piece
    constexpr int A_LOADS = 2 * MT;            // per wave and piece: the piece is 8 MT loads of two rows, dealt over four waves
    __shared__ __align__(1024) uint8_t sW[NW * 2 * BUF];
    __shared__ __align__(1024) uint8_t sA[2 * ABUF];
    // block scales: every wave's own copy of the piece's 16 MT rows x 4 steps of activation scales, fetched by MT more direct
    // loads of the piece so that they are counted by the same vmcnt wait.  (An ordinary load here would make the compiler
    // wait for vmcnt(0) before its first use, i.e. for the next piece's loads as well: no overlap left.)
    float* const sS = StreamScaleTable<BLOCKSCALE, NW * 2 * MT * 64>::get();

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li = lane & 15, lg = lane >> 4;
    const int K = p.K, N = p.N, M = p.M;
    // weight rows per wave: 16, or fewer so that the workgroups (4 R rows each) come out as a whole number per compute unit
    // (28672 rows: 448 workgroups of 64 rows are 1.75 per compute unit, 512 of 56 rows are two).  The rows a wave does
    // not own are loaded from beyond the descriptor's range (no memory request, zeros) and never stored.
    const int R = p.wave_rows > 0 ? p.wave_rows : 16;
    const int n_base = (blockIdx.x * NW + wave) * R;
    const int npieces = (K + PIECE - 1) / PIECE;
    const int tail_steps = (K % PIECE) / kKBlock;  // K steps of the last piece when K is no multiple of 512 (0: every piece is whole)
    constexpr uint32_t kOutOfRange = 0x80000000u;  // >= the descriptor's 2^31 - 1 bytes
    int c_begin = 0, c_end = npieces;
    if (p.split_k > 1) {  // ksteps_per_split counts 1 KiB of K: two pieces
        c_begin = blockIdx.y * p.ksteps_per_split * 2;
        c_end = min(c_begin + p.ksteps_per_split * 2, npieces);
    }
    const v4i rsrc_b = make_rsrc(p.B), rsrc_a = make_rsrc(p.A);
    const uint32_t my_lds = lds_address(sW) + wave * 2 * BUF, a_lds = lds_address(sA);
    const uint8_t* my_buf = sW + wave * 2 * BUF;
    const int rows_a = min(M, 16 * MT);

    // lane l of a load: row 2i + l/32, LDS position l%32 of the row's 32 chunks, which holds logical chunk (l%32) ^ (row % 16)
    const int half = lane >> 5, pos = lane & 31;
    // (the *_tail offsets are those of the short last piece: a load that would pass the end of its row fetches the piece's
    // first chunk again instead; the MFMAs of that piece stop at its valid steps)
    uint32_t w_off[8], a_off[A_LOADS], w_tail[8], a_tail[A_LOADS];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int r = 2 * i + half, chunk = pos ^ r;
        const bool mine = r < R && n_base + r < N;
        const uint32_t row = (uint32_t)min(n_base + r, N - 1) * (uint32_t)K;
        w_off[i] = mine ? row + (uint32_t)(chunk << 4) : kOutOfRange;
        w_tail[i] = mine ? row + (uint32_t)((chunk < tail_steps * 8 ? chunk : 0) << 4) : kOutOfRange;
    }
    // wave w issues loads w, w + 4, w + 8, ... of the activation piece
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i) {
        const int r = 2 * (wave + i * NW) + half, chunk = pos ^ (r & 15);
        const uint32_t row = (uint32_t)min(r, rows_a - 1) * (uint32_t)K;  // (rows past M: a copy of the last row, never stored)
        a_off[i] = row + (uint32_t)(chunk << 4);
        a_tail[i] = row + (uint32_t)((chunk < tail_steps * 8 ? chunk : 0) << 4);
    }
    // lane l of scale load mt: activation row 16 mt + l / 4, K step l % 4 of the piece
    const bool has_as = BLOCKSCALE && p.As != nullptr;
    const float* bs_ptr = BLOCKSCALE && p.Bs ? p.Bs + (int64_t)min(n_base / 128, p.nblocks - 1) * p.kblocks : nullptr;
    // with fewer than 16 rows per wave its rows may lie on both sides of a 128-row boundary of the weight scales: the scales of
    // the next block row are fetched as well (scalar loads), and every lane picks per output which of the two is its own
    const float* bs_ptr2 = BLOCKSCALE && p.Bs ? p.Bs + (int64_t)min(n_base / 128 + 1, p.nblocks - 1) * p.kblocks : nullptr;
    bool next_block[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) next_block[q] = BLOCKSCALE && (n_base + lg * 4 + q) / 128 != n_base / 128;
    const v4i rsrc_as = make_rsrc(p.As);
    const uint32_t s_lds = lds_address(sS) + (BLOCKSCALE ? wave * (2 * MT * 256) : 0);
    uint32_t as_off[MT], as_tail[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const uint32_t row = (uint32_t)min(mt * 16 + (lane >> 2), rows_a - 1) * (uint32_t)p.kblocks;
        as_off[mt] = (row + (lane & 3)) * 4u;
        as_tail[mt] = (row + ((lane & 3) < tail_steps ? (lane & 3) : 0)) * 4u;
    }
    auto issue = [&](int c, int buf) {
        const int k0 = c * PIECE;
        if (tail_steps != 0 && c == npieces - 1) {
#pragma unroll
            for (int i = 0; i < 8; ++i) direct_load_b128_nt(rsrc_b, my_lds + buf * BUF + i * 1024, w_tail[i], k0);
#pragma unroll
            for (int i = 0; i < A_LOADS; ++i) direct_load_b128(rsrc_a, a_lds + buf * ABUF + (wave + i * NW) * 1024, a_tail[i], k0);
            if constexpr (BLOCKSCALE) {
                if (has_as) {
#pragma unroll
                    for (int mt = 0; mt < MT; ++mt) direct_load_b32(rsrc_as, s_lds + (buf * MT + mt) * 256, as_tail[mt], c * (SPC * 4));
                }
            }
            return;
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) direct_load_b128_nt(rsrc_b, my_lds + buf * BUF + i * 1024, w_off[i], k0);
#pragma unroll
        for (int i = 0; i < A_LOADS; ++i) direct_load_b128(rsrc_a, a_lds + buf * ABUF + (wave + i * NW) * 1024, a_off[i], k0);
        if constexpr (BLOCKSCALE) {
            if (has_as) {
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) direct_load_b32(rsrc_as, s_lds + (buf * MT + mt) * 256, as_off[mt], c * (SPC * 4));
            }
        }
    };

    v4f acc[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[mt] = v4f{0.f, 0.f, 0.f, 0.f};
    // all but the loads of one piece: 8 + 2 MT, and MT more with block scales of the activations
    constexpr int kPlain = 8 + A_LOADS, kScaled = 8 + A_LOADS + MT;
    constexpr int kWaitButPlain = 0x0F70 | (kPlain & 15) | ((kPlain >> 4) << 14);
    constexpr int kWaitButScaled = 0x0F70 | (kScaled & 15) | ((kScaled >> 4) << 14);
    constexpr int kWaitAll = 0x0F70, kWaitLds = 0xC07F;
    const int n_pieces = max(c_end - c_begin, 0);
    const int rot = n_pieces > 0 ? (int)(blockIdx.x % (unsigned)n_pieces) : 0;  // staggered start, see above
    auto piece = [&](int i) { const int c = c_begin + i + rot; return c >= c_end ? c - n_pieces : c; };
    if (0 < n_pieces) issue(piece(0), 0);
    if (1 < n_pieces) issue(piece(1), 1);
    for (int it = 0; it < n_pieces; ++it) {
        const int c = piece(it);
        const int buf = it & 1;
        const int steps = (tail_steps != 0 && c == npieces - 1) ? tail_steps : SPC;
        float bsc[BLOCKSCALE ? SPC : 1], bsc2[BLOCKSCALE ? SPC : 1];
        if constexpr (BLOCKSCALE) {  // the weight scales are the same in every lane: scalar loads, not counted by vmcnt
#pragma unroll
            for (int s = 0; s < SPC; ++s) {
                bsc[s] = bs_ptr ? stream_uniform_f32(bs_ptr + min(c * SPC + s, p.kblocks - 1)) : 1.0f;
                bsc2[s] = bs_ptr2 ? stream_uniform_f32(bs_ptr2 + min(c * SPC + s, p.kblocks - 1)) : 1.0f;
            }
        }
        // my loads of piece c have landed (those of piece c+1 may be in flight) ...
        if (it + 1 >= n_pieces) __builtin_amdgcn_s_waitcnt(kWaitAll);
        else if (has_as) __builtin_amdgcn_s_waitcnt(kWaitButScaled);
        else __builtin_amdgcn_s_waitcnt(kWaitButPlain);
        __builtin_amdgcn_s_barrier();  // ... and so has every other wave's share of the activation piece
        const uint8_t* wb = my_buf + buf * BUF + li * PIECE;
        const uint8_t* ab = sA + buf * ABUF + li * PIECE;
        v8i wf[SPC], af[MT][SPC];
#pragma unroll
        for (int s = 0; s < SPC; ++s) {
            const int j0 = ((s * 8 + lg) ^ li) << 4, j1 = ((s * 8 + 4 + lg) ^ li) << 4;
            wf[s] = join(*reinterpret_cast<const v4i*>(wb + j0), *reinterpret_cast<const v4i*>(wb + j1));
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
                af[mt][s] = join(*reinterpret_cast<const v4i*>(ab + mt * BUF + j0), *reinterpret_cast<const v4i*>(ab + mt * BUF + j1));
        }
        v4f as4[MT];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            as4[mt] = v4f{1.f, 1.f, 1.f, 1.f};
            if constexpr (BLOCKSCALE)
                if (has_as) as4[mt] = *reinterpret_cast<const v4f*>(sS + wave * (2 * MT * 64) + (buf * MT + mt) * 64 + li * 4);
        }
        __builtin_amdgcn_s_waitcnt(kWaitLds);
#pragma unroll
        for (int s = 0; s < SPC; ++s) {
            asm volatile("" : "+v"(wf[s]));
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) asm volatile("" : "+v"(af[mt][s]));
        }
        if constexpr (BLOCKSCALE) {
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) asm volatile("" : "+v"(as4[mt]));
        }
        __builtin_amdgcn_s_barrier();  // every wave holds its fragments: this buffer may be refilled
        if (it + 2 < n_pieces) issue(piece(it + 2), buf);
#pragma unroll
        for (int s = 0; s < SPC; ++s) {
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                if (s >= steps) continue;
                if constexpr (BLOCKSCALE) {
                    // (the same product of the two scales as with one scale per wave, then one multiply-add per output)
                    const float lo = as4[mt][s] * bsc[s], hi = as4[mt][s] * bsc2[s];
                    const v4f sc = v4f{next_block[0] ? hi : lo, next_block[1] ? hi : lo, next_block[2] ? hi : lo, next_block[3] ? hi : lo};
                    acc[mt] += mfma_e4m3(wf[s], af[mt][s], v4f{0.f, 0.f, 0.f, 0.f}) * sc;
                } else {
                    acc[mt] = mfma_e4m3(wf[s], af[mt][s], acc[mt]);
                }
            }
        }
    }
    // a lane holds four consecutive weight rows' results: all of them, or (R % 4 != 0) only the first R - 4 lg, are the wave's
    const bool vec_ok = p.vec_store != 0 && (R & 3) == 0;
    const int col = n_base + lg * 4;
    const int n_end = min(n_base + R, N);  // (store4 writes single elements up to its N argument when four would pass it)
    float scale = p.alpha;
    if constexpr (!BLOCKSCALE) {
        if (p.As) scale *= p.As[0];
        if (p.Bs) scale *= p.Bs[0];
    }
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int m = mt * 16 + li;
        if (m >= M || col >= n_end) continue;
        if (p.split_k > 1) store4(p.partials + (int64_t)blockIdx.y * M * N, OUT_F32, m, col, n_end, N, acc[mt], 0.f, vec_ok);
        else store4(p.C, p.out_type, m, col, n_end, p.ldc, acc[mt] * scale, p.beta, vec_ok);
    }
#endif
}

// grid_x = ceil(N / (4 R)) with R = p.wave_rows weight rows per wave (0: 16); M <= 16 MT
template <bool BLOCKSCALE, int MT>
inline hipError_t launch_stream_wide_db(const GemmParams& p, int grid_x, int grid_y, hipStream_t stream) {
    if (p.K % kKBlock != 0 || p.K <= 0 || p.M > 16 * MT || p.wave_rows < 0 || p.wave_rows > 16) return hipErrorInvalidValue;
    hipLaunchKernelGGL((fp8_gemm_stream_wide_db_kernel<BLOCKSCALE, MT>), dim3(grid_x, grid_y, 1), dim3(256, 1, 1), 0, stream, p);
    return hipGetLastError();
}

// Ragged (expert-grouped) block-scaled GEMM for a handful of rows per expert: the decode regime of a MoE layer, where most
// experts receive no row and the others one to a dozen.  The wide two-piece form above, one grid row per expert:
// workgroup (x, e) streams weight rows 64 x .. 64 x + 63 of expert e once per 16 rows that m_indptr gives that expert and
// leaves at once when it has none.  K % 128 == 0: the last piece of a K that is no multiple of 512 has one to three K
// steps; its loads are redirected to the piece's first step where they would pass the end of a row, and its MFMAs stop
// at the valid steps.  N * K < 2^31 per expert (32-bit offsets inside an expert's weight), total rows * K < 2^32.
// NW waves per workgroup (16 NW weight rows): four, or more when that brings the workgroups that find rows (at most one
// grid row per routed row) down to one per compute unit -- a launch of this kernel takes a "round" per 256 workgroups
// (one token of config 5, six experts of 2816 weight rows: 264 workgroups of 64 rows take 11.5 us, 180 of 96 rows 9.7 us).
template <int NW>
__global__ void __launch_bounds__(64 * NW) fp8_gemm_stream_ragged_kernel(const GemmParams p) {
#if defined(__HIP_DEVICE_COMPILE__)
    constexpr int PIECE = 512, BUF = 16 * PIECE, SPC = PIECE / kKBlock;
    __shared__ __align__(1024) uint8_t sW[NW * 2 * BUF];
    __shared__ __align__(1024) uint8_t sA[2 * BUF];
    __shared__ __align__(16) float sS[NW * 2 * 64];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li = lane & 15, lg = lane >> 4;
    const int K = p.K, N = p.N;
    const int e = blockIdx.y;
    const int row_lo = __builtin_amdgcn_readfirstlane(p.m_indptr[e]), row_hi = __builtin_amdgcn_readfirstlane(p.m_indptr[e + 1]);
    if (row_hi <= row_lo) return;
    const int n_base = blockIdx.x * (16 * NW) + wave * 16;
    const int npieces = (K + PIECE - 1) / PIECE;
    const int tail_steps = (K % PIECE) / kKBlock;  // 0: every piece is whole
    const v4i rsrc_b = make_rsrc(p.B + (int64_t)e * N * K), rsrc_a = make_rsrc(p.A), rsrc_as = make_rsrc(p.As);
    const float* bs_ptr = p.Bs + ((int64_t)e * p.nblocks + min(n_base / 128, p.nblocks - 1)) * p.kblocks;
    const uint32_t my_lds = lds_address(sW) + wave * 2 * BUF, a_lds = lds_address(sA), s_lds = lds_address(sS) + wave * 512;
    const uint8_t* my_buf = sW + wave * 2 * BUF;

    // lane l of a load: row 2i + l/32, LDS position l%32 of the row's 32 chunks, which holds logical chunk (l%32) ^ row
    const int half = lane >> 5, pos = lane & 31;
    uint32_t w_off[8], w_tail[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int r = 2 * i + half, chunk = pos ^ r;
        const uint32_t row = (uint32_t)min(n_base + r, N - 1) * (uint32_t)K;
        w_off[i] = row + (uint32_t)(chunk << 4);
        w_tail[i] = row + (uint32_t)((chunk < tail_steps * 8 ? chunk : 0) << 4);
    }
    constexpr int kWaitBut11 = 0x0F70 | 11, kWaitAll = 0x0F70, kWaitLds = 0xC07F;
    const int rot = (int)(blockIdx.x % (unsigned)npieces);  // staggered start over K, as in the dense form
    auto piece = [&](int i) { const int c = i + rot; return c >= npieces ? c - npieces : c; };
    const bool vec_ok = p.vec_store != 0;
    const int col = n_base + lg * 4;

    for (int row0 = row_lo; row0 < row_hi; row0 += 16) {
        const int rows_a = min(16, row_hi - row0);
        uint32_t a_off[2], a_tail[2];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            // (eight loads of two rows make the piece; with more than four waves the surplus loads repeat the last one)
            const int r = 2 * min(wave + i * NW, 7) + half, chunk = pos ^ r;
            const uint32_t row = (uint32_t)(row0 + min(r, rows_a - 1)) * (uint32_t)K;  // (rows past the tile: a copy of its last row, never stored)
            a_off[i] = row + (uint32_t)(chunk << 4);
            a_tail[i] = row + (uint32_t)((chunk < tail_steps * 8 ? chunk : 0) << 4);
        }
        // lane l of the scale load: activation row l / 4, K step l % 4 of the piece
        const uint32_t as_row = (uint32_t)(row0 + min(lane >> 2, rows_a - 1)) * (uint32_t)p.kblocks;
        const uint32_t as_off = (as_row + (lane & 3)) * 4u, as_tail = (as_row + ((lane & 3) < tail_steps ? (lane & 3) : 0)) * 4u;
        auto issue = [&](int c, int buf) {
            const int k0 = c * PIECE;
            if (tail_steps != 0 && c == npieces - 1) {
#pragma unroll
                for (int i = 0; i < 8; ++i) direct_load_b128_nt(rsrc_b, my_lds + buf * BUF + i * 1024, w_tail[i], k0);
                direct_load_b128(rsrc_a, a_lds + buf * BUF + min(wave, 7) * 1024, a_tail[0], k0);
                direct_load_b128(rsrc_a, a_lds + buf * BUF + min(wave + NW, 7) * 1024, a_tail[1], k0);
                direct_load_b32(rsrc_as, s_lds + buf * 256, as_tail, c * (SPC * 4));
            } else {
#pragma unroll
                for (int i = 0; i < 8; ++i) direct_load_b128_nt(rsrc_b, my_lds + buf * BUF + i * 1024, w_off[i], k0);
                direct_load_b128(rsrc_a, a_lds + buf * BUF + min(wave, 7) * 1024, a_off[0], k0);
                direct_load_b128(rsrc_a, a_lds + buf * BUF + min(wave + NW, 7) * 1024, a_off[1], k0);
                direct_load_b32(rsrc_as, s_lds + buf * 256, as_off, c * (SPC * 4));
            }
        };
        v4f acc = v4f{0.f, 0.f, 0.f, 0.f};
        issue(piece(0), 0);
        if (1 < npieces) issue(piece(1), 1);
        for (int it = 0; it < npieces; ++it) {
            const int c = piece(it);
            const int buf = it & 1;
            const int steps = (tail_steps != 0 && c == npieces - 1) ? tail_steps : SPC;
            float bsc[SPC];
#pragma unroll
            for (int s = 0; s < SPC; ++s) bsc[s] = stream_uniform_f32(bs_ptr + min(c * SPC + s, p.kblocks - 1));
            if (it + 1 >= npieces) __builtin_amdgcn_s_waitcnt(kWaitAll);
            else __builtin_amdgcn_s_waitcnt(kWaitBut11);
            __builtin_amdgcn_s_barrier();
            const uint8_t* wb = my_buf + buf * BUF + li * PIECE;
            const uint8_t* ab = sA + buf * BUF + li * PIECE;
            v8i wf[SPC], af[SPC];
#pragma unroll
            for (int s = 0; s < SPC; ++s) {
                const int j0 = ((s * 8 + lg) ^ li) << 4, j1 = ((s * 8 + 4 + lg) ^ li) << 4;
                wf[s] = join(*reinterpret_cast<const v4i*>(wb + j0), *reinterpret_cast<const v4i*>(wb + j1));
                af[s] = join(*reinterpret_cast<const v4i*>(ab + j0), *reinterpret_cast<const v4i*>(ab + j1));
            }
            v4f as4 = *reinterpret_cast<const v4f*>(sS + wave * 128 + buf * 64 + li * 4);
            __builtin_amdgcn_s_waitcnt(kWaitLds);
#pragma unroll
            for (int s = 0; s < SPC; ++s) asm volatile("" : "+v"(wf[s]), "+v"(af[s]));
            asm volatile("" : "+v"(as4));
            __builtin_amdgcn_s_barrier();  // every wave holds its fragments: this buffer may be refilled
            if (it + 2 < npieces) issue(piece(it + 2), buf);
#pragma unroll
            for (int s = 0; s < SPC; ++s)
                if (s < steps) acc += mfma_e4m3(wf[s], af[s], v4f{0.f, 0.f, 0.f, 0.f}) * (as4[s] * bsc[s]);
        }
        if (li < rows_a && col < N) store4(p.C, p.out_type, row0 + li, col, N, p.ldc, acc * p.alpha, p.beta, vec_ok);
    }
#endif
}

// one grid row per expert; needs both scale tensors, K % 128 == 0, N * K < 2^31
template <int NW>
inline hipError_t launch_stream_ragged(const GemmParams& p, hipStream_t stream) {
    if (p.K % kKBlock != 0 || p.K <= 0 || !p.As || !p.Bs || !p.m_indptr || (int64_t)p.N * p.K >= ((int64_t)1 << 31)) return hipErrorInvalidValue;
    hipLaunchKernelGGL(fp8_gemm_stream_ragged_kernel<NW>, dim3((p.N + 16 * NW - 1) / (16 * NW), p.E, 1), dim3(64 * NW, 1, 1), 0, stream, p);
    return hipGetLastError();
}

template <bool BLOCKSCALE>
inline hipError_t launch_stream_wide(const GemmParams& p, int grid_x, int grid_y, hipStream_t stream) {
    hipLaunchKernelGGL(fp8_gemm_stream_wide_kernel<BLOCKSCALE>, dim3(grid_x, grid_y, 1), dim3(256, 1, 1), 0, stream, p);
    return hipGetLastError();
}

template <int MT, int NBUF, bool BLOCKSCALE, int NW = 4>
inline hipError_t launch_stream(const GemmParams& p, int grid_x, int grid_y, hipStream_t stream) {
    auto kern = fp8_gemm_stream_kernel<MT, NBUF, BLOCKSCALE, NW>;
    hipLaunchKernelGGL(kern, dim3(grid_x, grid_y, 1), dim3(64 * NW, 1, 1), 0, stream, p);
    return hipGetLastError();
}

}  // namespace tg
