// LDS-tiled FP8 GEMM for gfx950: C[m,n] = sum_k A[m,k] * B[n,k]  (both operands K-contiguous).
//
// One workgroup (4 or 8 waves) computes a BM x BN tile of C.  Per K step of 128 bytes it stages a
// BM x 128 slab of A and a BN x 128 slab of B in LDS with direct global->LDS loads (16 bytes
// per lane, no staging registers, double buffered), and every wave runs 16x16x128 e4m3 MFMAs
// over its (BM/WGM) x (BN/WGN) sub-tile with fp32 accumulators.  A direct load writes lane l
// of a wave to LDS byte 16*l of the wave's 1 KiB destination, so the XOR swizzle that keeps
// the fragment reads bank-conflict free is applied on the global side: each lane fetches the
// 16-byte chunk that belongs at its LDS position.  The two stages are separate LDS objects so
// that the compiler can tell a load into one from a read of the other.
//
// The MFMA "row" operand is fed from B (weights) and the "column" operand from A
// (activations): a lane then owns, for one activation row m, four consecutive n, so a
// per-token scale is one register per lane.  The weight rows of a column-tile pair are
// permuted so that those four-column runs of the two tiles join into eight consecutive columns.
//
// Epilogue: straight from the accumulators, one 16-byte store (8 bf16/f16 outputs) per lane and
// column-tile pair; scaling, beta, routed weights and the output cast happen there.  The gate/up
// form of the MoE layer computes SiLU(gate) * up and its 1 x 128 e4m3 quantization instead.
//
// Rows are dealt to the wave rows in interleaved 16-row groups, and the grouped forms run the K
// loop specialised on how many of a wave's row groups hold valid rows: padding rows cost no MFMAs.
//
// Scale modes:  per-tensor (one multiply in the epilogue) or block-scaled (every K step's
// 16x16 product is multiplied by As[m,kb] * Bs[n/128,kb] while it is added to the
// accumulator, the arithmetic of src/tilegym/suites/unsloth/cutile/fp8.py:282-323).
// Row modes: dense, ragged (expert segments from m_indptr, the schedule of
// src/tilegym/suites/flashinfer/cutile/gemm/ragged_block_scaled_bmm.py:71-91) and gather
// (sorted_token_ids / expert_ids, the contract of src/tilegym/ops/tilecpp/moe.cuh:72-225).
#pragma once
#include <type_traits>

#include "tg_device.h"

namespace tg {

constexpr int kMaxKBlocks = 512;  // K <= 65536 for the block-scaled tiled kernels (host checks)

// Raw buffer descriptor over [base, base + 2 GiB): byte offsets, no format conversion.
__device__ __forceinline__ v4i make_rsrc(const void* base) {
    // the base is the same in every lane; say so, so that the descriptor lives in scalar registers
    const uintptr_t a = reinterpret_cast<uintptr_t>(base);
    const int lo = __builtin_amdgcn_readfirstlane((int)(uint32_t)a);
    const int hi = __builtin_amdgcn_readfirstlane((int)((uint32_t)(a >> 32) & 0xFFFFu));
    return v4i{lo, hi, 0x7FFFFFFF, 0x00020000};
}

// One direct global->LDS load: every lane fetches 16 bytes at rsrc.base + voffset + soffset and
// the wave's 64 x 16 bytes land at LDS address lds_addr + 16 * lane.  Written as inline assembly
// on purpose: the compiler's wait-count insertion treats a builtin direct load that is still in
// flight as possibly aliasing every later LDS read and drains the whole memory pipeline
// (vmcnt(0)) in front of it, which would undo the multi-step prefetch.  Completion is tracked by
// hand with the vmcnt waits in the kernel; the "memory" clobber keeps LDS reads from being
// cached across it.  The compiler's hazard recognizer does not look into inline assembly either:
// a scalar operand that a vector instruction has just written (v_readfirstlane, when the
// compiler keeps a wave-uniform offset in a vector register) must not be read by a memory
// instruction within five wait states, or the instruction sees the register's old value.  The
// M0 write and the s_nop in front of each load are those five.
__device__ __forceinline__ void direct_load_b128(v4i rsrc, uint32_t lds_addr, uint32_t voffset, int soffset) {
    lds_addr = __builtin_amdgcn_readfirstlane(lds_addr);  // wave-uniform by construction
    soffset = __builtin_amdgcn_readfirstlane(soffset);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 3\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                 :
                 : "s"(lds_addr), "v"(voffset), "s"(rsrc), "s"(soffset)
                 : "memory");
}

// The same load without those wait states, for the one loop where they cost measurable time (a 256 x 256 tile's
// sixteen loads per K step: 2-3% of the launch).  Only for scalar operands that no vector instruction can have written
// shortly before: values that come out of settle() below and scalar arithmetic on them, in a kernel that spills no
// scalar register (a spilled one comes back through v_readlane).  check_hazards.py verifies both on the kernel's assembly.
__device__ __forceinline__ void direct_load_b128_settled(v4i rsrc, uint32_t lds_addr, uint32_t voffset, int soffset) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                 :
                 : "s"(lds_addr), "v"(voffset), "s"(rsrc), "s"(soffset)
                 : "memory");
}
// A wave-uniform value in a scalar register written by a scalar instruction: what the compiler derives from it with
// scalar arithmetic is never produced by v_readfirstlane right in front of its use.
__device__ __forceinline__ int settle(int x) {
    int r;
    x = __builtin_amdgcn_readfirstlane(x);
    asm volatile("s_mov_b32 %0, %1" : "=s"(r) : "s"(x));
    return r;
}

// The same load marked non-temporal: for data a launch reads exactly once (the weights of a
// skinny-M GEMM).  The lines are the first to be replaced in the caches instead of displacing
// what is reused; measured 5-11% shorter weight-streaming launches.
__device__ __forceinline__ void direct_load_b128_nt(v4i rsrc, uint32_t lds_addr, uint32_t voffset, int soffset) {
    lds_addr = __builtin_amdgcn_readfirstlane(lds_addr);
    soffset = __builtin_amdgcn_readfirstlane(soffset);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 3\n\tbuffer_load_dwordx4 %1, %2, %3 offen nt lds"
                 :
                 : "s"(lds_addr), "v"(voffset), "s"(rsrc), "s"(soffset)
                 : "memory");
}

// Same for 4 bytes per lane (the wave's 64 x 4 bytes land at lds_addr + 4 * lane).
__device__ __forceinline__ void direct_load_b32(v4i rsrc, uint32_t lds_addr, uint32_t voffset, int soffset) {
    lds_addr = __builtin_amdgcn_readfirstlane(lds_addr);
    soffset = __builtin_amdgcn_readfirstlane(soffset);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 3\n\tbuffer_load_dword %1, %2, %3 offen lds"
                 :
                 : "s"(lds_addr), "v"(voffset), "s"(rsrc), "s"(soffset)
                 : "memory");
}

__device__ __forceinline__ uint32_t lds_address(const void* p) {
    return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const void*)p;
}

// Chunk swizzle of a 128-byte slab row: 16-byte chunk j of row r sits at chunk position j ^ (r % 8).
// Measured on gfx950 (128 B/clk LDS): ds_read_b128 of 16 consecutive rows at one logical chunk is
// conflict free with this XOR (8 clocks per 1 KiB wave-read, the LDS's full rate); additive
// variants are 2-way conflicted.
__device__ __forceinline__ int swz16(int r) { return r & 7; }
constexpr int kScaleChunk = 8;  // K steps per chunk of the activation-scale table
// chunk swizzle of the weight slab: row bits 0, 1 and 3
__device__ __forceinline__ int swz_w(int r) { return (r & 3) | ((r >> 1) & 4); }

// Number of BM-row tiles over all experts (every lane returns the same value).
__device__ __forceinline__ int ragged_count_tiles(const int* indptr, int E, int BM, int lane) {
    int total = 0;
    for (int e0 = 0; e0 < E; e0 += 64) {
        int e = e0 + lane, cnt = 0;
        if (e < E) {
            int rows = indptr[e + 1] - indptr[e];
            cnt = rows > 0 ? (rows + BM - 1) / BM : 0;
        }
#pragma unroll
        for (int d = 32; d >= 1; d >>= 1) cnt += __shfl_xor(cnt, d);
        total += cnt;
    }
    return total;
}

// Expert that owns m-tile `mt`, and the index of that tile inside the expert.
__device__ __forceinline__ void ragged_find(const int* indptr, int E, int BM, int lane, int mt,
                                            int& expert, int& tile_in_expert) {
    int base = 0;
    expert = -1;
    tile_in_expert = 0;
    for (int e0 = 0; e0 < E; e0 += 64) {
        int e = e0 + lane, cnt = 0;
        if (e < E) {
            int rows = indptr[e + 1] - indptr[e];
            cnt = rows > 0 ? (rows + BM - 1) / BM : 0;
        }
        int incl = cnt;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            int t = __shfl_up(incl, d);
            if (lane >= d) incl += t;
        }
        int excl = base + incl - cnt;
        unsigned long long hit = __ballot(mt >= excl && mt < excl + cnt);
        if (hit) {
            int src = __ffsll((long long)hit) - 1;
            expert = e0 + src;
            tile_in_expert = mt - __shfl(excl, src);
            return;
        }
        base += __shfl(incl, 63);
    }
}

// Write 8 consecutive outputs C[row][col..col+7] = v (+ beta * old), masked against N columns; ld = row stride.
__device__ __forceinline__ void store8(void* C, int out_type, int64_t row, int col, int N, int ld,
                                       v4f lo, v4f hi, float beta, bool vec_ok) {
    const int64_t base = row * (int64_t)ld + col;
    if (vec_ok && col + 7 < N) {
        if (out_type == OUT_F32) {
            v4f* p = reinterpret_cast<v4f*>(reinterpret_cast<float*>(C) + base);
            if (beta != 0.0f) {
                lo += beta * p[0];
                hi += beta * p[1];
            }
            p[0] = lo;
            p[1] = hi;
        } else if (out_type == OUT_F8) {
            uint8_t* p = reinterpret_cast<uint8_t*>(C) + base;
            if (beta != 0.0f) {
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    lo[q] += beta * e4m3_to_f32(p[q]);
                    hi[q] += beta * e4m3_to_f32(p[4 + q]);
                }
            }
            *reinterpret_cast<v2i*>(p) = v2i{pack_e4m3x4(lo[0], lo[1], lo[2], lo[3]), pack_e4m3x4(hi[0], hi[1], hi[2], hi[3])};
        } else if (out_type == OUT_BF16) {
            typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
            typedef float v8f __attribute__((ext_vector_type(8)));
            bf16x8* p = reinterpret_cast<bf16x8*>(reinterpret_cast<__bf16*>(C) + base);
            v8f v = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
            if (beta != 0.0f) v += beta * __builtin_convertvector(*p, v8f);
            *p = __builtin_convertvector(v, bf16x8);
        } else {
            typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
            typedef float v8f __attribute__((ext_vector_type(8)));
            f16x8* p = reinterpret_cast<f16x8*>(reinterpret_cast<_Float16*>(C) + base);
            v8f v = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
            if (beta != 0.0f) v += beta * __builtin_convertvector(*p, v8f);
            *p = __builtin_convertvector(v, f16x8);
        }
        return;
    }
    for (int q = 0; q < 8; ++q) {
        if (col + q >= N) break;
        float x = q < 4 ? lo[q & 3] : hi[q & 3];
        if (out_type == OUT_BF16) {
            __bf16* p = reinterpret_cast<__bf16*>(C) + base + q;
            if (beta != 0.0f) x += beta * (float)(*p);
            *p = (__bf16)x;
        } else if (out_type == OUT_F32) {
            float* p = reinterpret_cast<float*>(C) + base + q;
            if (beta != 0.0f) x += beta * (*p);
            *p = x;
        } else if (out_type == OUT_F8) {
            uint8_t* p = reinterpret_cast<uint8_t*>(C) + base + q;
            if (beta != 0.0f) x += beta * e4m3_to_f32(*p);
            *p = f32_to_e4m3(x);
        } else {
            _Float16* p = reinterpret_cast<_Float16*>(C) + base + q;
            if (beta != 0.0f) x += beta * (float)(*p);
            *p = (_Float16)x;
        }
    }
}

// Body of the tiled kernel for workgroup `bid` of problem `p` (the kernels below only differ in
// how a workgroup finds its problem).
template <int BM, int BN, int WGM, int WGN, bool BLOCKSCALE, int GROUP, bool SPLIT>
__device__ __forceinline__ void fp8_gemm_tile_body(const GemmParams& p, const int bid) {
#if defined(__HIP_DEVICE_COMPILE__)  // the body is device-only assembly; the host pass only needs the stub
    constexpr int NT = 64 * WGM * WGN;
    constexpr int NW = WGM * WGN;
    constexpr int WTM = BM / WGM, WTN = BN / WGN;
    constexpr int TM = WTM / 16, TN = WTN / 16;
    constexpr int NL = NW;                // every wave issues its share of the direct global->LDS loads
    constexpr int RPP = 8 * NL;           // slab rows filled per pass of the waves
    constexpr int A_IT = BM / RPP, B_IT = BN / RPP;
    static_assert(NW == 4 || NW == 8, "wave grid");
    static_assert(BM % RPP == 0 && BN % RPP == 0 && NL % 2 == 0, "loader shape");
    static_assert(WTM % 16 == 0 && WTN % 32 == 0, "wave tile: column tiles are taken in pairs");
    static_assert(!BLOCKSCALE || (WTN <= 128 && 128 % WTN == 0), "one weight scale per wave");
    static_assert(!SPLIT || GROUP == GROUP_DENSE, "split-K is dense only");
    // fused activation epilogue (MoE gate/up GEMM): a tile is 128 gate columns + the 128 matching up columns
    constexpr bool ACT = GROUP == GROUP_GATHER_ACT;
    static_assert(!ACT || (BLOCKSCALE && BN == 256 && WTN % 64 == 0 && WGN * BM <= 2 * BM * kScaleChunk),
                  "fused activation: block-scaled, 128 gate + 128 up columns per tile, each wave with as many gate as up column tiles");

    __shared__ __align__(1024) uint8_t sA0[BM * kKBlock];
    __shared__ __align__(1024) uint8_t sA1[BM * kKBlock];
    __shared__ __align__(1024) uint8_t sB0[BN * kKBlock];
    __shared__ __align__(1024) uint8_t sB1[BN * kKBlock];
    // activation scales of the tile rows, two chunks of kScaleChunk K steps (block-scaled kernels only)
    __shared__ __align__(256) float sTab[BLOCKSCALE ? 2 * BM * kScaleChunk : 1];
    // weight block scales of this tile's column blocks for every K step (fetched once)
    __shared__ float sBs[BLOCKSCALE ? (BN + 127) / 128 : 1][BLOCKSCALE ? kMaxKBlocks : 1];
    __shared__ int s_src[GROUP == GROUP_DENSE ? 1 : BM];
    __shared__ int s_dst[GROUP == GROUP_DENSE ? 1 : BM];
    // routed weight of each tile row (gather GEMM with mul_routed_weight), fetched once per tile: a load
    // inside the epilogue's row loop would put a global-memory latency on every iteration
    __shared__ float s_w[GROUP == GROUP_GATHER ? BM : 1];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave % WGM, wn = wave / WGM;
    const int tiles_n = ACT ? p.inter / 128 : (p.N + BN - 1) / BN;
    const int K = p.K;

    // ---------------------------------------------------------------- which tile
    int tile_m = 0, tile_n = 0, m0 = 0, rows_valid = BM;
    const uint8_t* Bbase = p.B;
    const float* Bsbase = p.Bs;
    int post_pad = 0;
    if constexpr (GROUP == GROUP_DENSE) {
        const int tiles_m = (p.M + BM - 1) / BM;
        const int pid = xcd_remap(bid, tiles_m * tiles_n);
        constexpr int GM = 8;
        const int width = GM * tiles_n;
        const int group = pid / width, first_m = group * GM;
        const int gsz = min(tiles_m - first_m, GM);
        tile_m = first_m + (pid % width) % gsz;
        tile_n = (pid % width) / gsz;
        m0 = tile_m * BM;
        rows_valid = min(BM, p.M - m0);
    } else if constexpr (GROUP == GROUP_RAGGED) {
        const int total_mt = ragged_count_tiles(p.m_indptr, p.E, BM, lane);
        const int nblk = total_mt * tiles_n;
        if (bid >= nblk) return;
        const int pid = xcd_remap(bid, nblk);
        tile_m = pid / tiles_n;
        tile_n = pid % tiles_n;
        int e, t_in_e;
        ragged_find(p.m_indptr, p.E, BM, lane, tile_m, e, t_in_e);
        e = __builtin_amdgcn_readfirstlane(e);
        t_in_e = __builtin_amdgcn_readfirstlane(t_in_e);
        if (e < 0) return;
        const int lo = p.m_indptr[e], hi = min(p.m_indptr[e + 1], p.M);
        m0 = lo + t_in_e * BM;
        rows_valid = min(BM, hi - m0);
        if (rows_valid <= 0 || lo < 0) return;
        Bbase += (int64_t)e * p.N * K;
        if (Bsbase) Bsbase += (int64_t)e * p.nblocks * p.kblocks;
    } else {
        post_pad = min(p.num_post_pad[0], p.em_capacity);
        const int total_mt = (post_pad + BM - 1) / BM;
        const int nblk = total_mt * tiles_n;
        if (bid >= nblk) return;
        const int pid = xcd_remap(bid, nblk);
        tile_m = pid / tiles_n;
        tile_n = pid % tiles_n;
        m0 = tile_m * BM;  // position in the sorted slot sequence
        const int e = p.expert_ids[m0 / p.block_m];
        if (e < 0 || e >= p.E) return;
        Bbase += (int64_t)e * p.N * K;
        if (Bsbase) Bsbase += (int64_t)e * p.nblocks * p.kblocks;
    }
    const int n0 = ACT ? tile_n * 128 : tile_n * BN;  // ACT: first gate column of the tile

    int ks = 0, ks_end = p.kblocks;
    if constexpr (SPLIT) {
        ks = blockIdx.y * p.ksteps_per_split;
        ks_end = min(ks + p.ksteps_per_split, p.kblocks);
    }

    // ---------------------------------------------------------------- weight slab of the first K step
    // Requested before anything else: it needs only the tile's column and expert, so its trip to memory
    // overlaps the row maps and scale tables fetched below (which the activation loads must wait for).
    const int lrow = lane >> 3;
    // weight slab: its own swizzle (see the fragment addresses below).  Row 8g + lrow with g = i*NL + wave:
    // NL is even, so bit 3 of the row is the parity of the wave.
    const int ljb = (lane & 7) ^ swz_w(((wave & 1) << 3) | lrow);
    // (with NL == NW every wave loads: no test, and so no branch inside the K loop)
    uint32_t b_off[B_IT];
#pragma unroll
    for (int i = 0; i < B_IT; ++i) {
        const int br = (i * NL + (wave % NL)) * 8 + lrow;  // slab row
        int n;
        // fused activation: wave column wn owns slab rows WTN*wn .. +WTN-1 = WTN/2 gate rows, then the WTN/2 up rows of the same columns
        if constexpr (ACT) n = ((br % WTN) / (WTN / 2)) * p.inter + n0 + (br / WTN) * (WTN / 2) + br % (WTN / 2);
        else n = min(n0 + br, p.N - 1);
        b_off[i] = (uint32_t)n * (uint32_t)K + ljb * 16;
    }
    const v4i rsrc_b = make_rsrc(Bbase);
    auto issue_b1 = [&](int i, int kstep, uint8_t* dB) {  // piece i of this wave's share of a weight slab
        const int k0 = kstep * kKBlock;
        const uint32_t dst = lds_address(dB) + wave * 1024;
        // the 64-row tile serves M <= 64: one row tile, every weight byte is read once
        if constexpr (BM == 64) direct_load_b128_nt(rsrc_b, dst + i * NL * 1024, b_off[i], k0);
        else direct_load_b128(rsrc_b, dst + i * NL * 1024, b_off[i], k0);
    };
    auto issue_b = [&](int kstep, uint8_t* dB) {
#pragma unroll
        for (int i = 0; i < B_IT; ++i) issue_b1(i, kstep, dB);
    };
    issue_b(ks, sB0);

    // ---------------------------------------------------------------- row maps and scale tables
    // Both come from global memory; the slot ids are requested first and used last, so that the two
    // round trips (and the weight slab's) overlap.  One barrier publishes all of it.
    static_assert(BM <= NT, "one tile row per thread");
    int slot_id = 0;
    if constexpr (GROUP == GROUP_GATHER || GROUP == GROUP_GATHER_ACT) {
        const int idx = m0 + tid;
        slot_id = (tid < BM && idx < post_pad) ? p.sorted_ids[idx] : p.num_valid;
    }
    if constexpr (BLOCKSCALE) {
        // weight block scales of this tile's column blocks for every K step
        constexpr int NBT = (BN + 127) / 128;
        for (int idx = tid; idx < NBT * p.kblocks; idx += NT) {
            const int j = idx / p.kblocks, kb = idx % p.kblocks;
            const int nb = ACT ? (j == 0 ? n0 / 128 : (p.inter + n0) / 128) : min(n0 / 128 + j, p.nblocks - 1);
            sBs[j][kb] = Bsbase ? Bsbase[(int64_t)nb * p.kblocks + kb] : 1.0f;
        }
        if (!p.As) {  // no activation scales: ones
            for (int r2 = tid; r2 < 2 * BM * kScaleChunk; r2 += NT) sTab[r2] = 1.0f;
        }
    }
    if constexpr (GROUP != GROUP_DENSE) {
        if (tid < BM) {
            const int r = tid;
            int src, dst;
            if constexpr (GROUP == GROUP_RAGGED) {
                src = m0 + min(r, rows_valid - 1);
                dst = r < rows_valid ? m0 + r : -1;
            } else {
                const bool ok = slot_id >= 0 && slot_id < p.num_valid;
                src = ok ? slot_id / p.top_k : 0;
                dst = ok ? slot_id : -1;
            }
            s_src[r] = src;
            s_dst[r] = dst;
        }
    }
    if constexpr (BLOCKSCALE || GROUP != GROUP_DENSE) __syncthreads();

    // ---------------------------------------------------------------- loader set-up
    // Every wave issues its share of the direct loads, one or two behind each column tile's MFMAs (see the
    // main loop): the address path takes ~14 clocks per 1 KiB load for the whole compute unit, whoever
    // issues it, and a wave that waits for room there issues no MFMAs, so bursts of loads from a few
    // loader waves put load time and MFMA time of those waves in series.  Pass i of wave w fills the 8-row group
    // g = i*NL + w: lane l lands at row 8g + l/8, chunk position l%8, and therefore fetches
    // logical chunk (l%8) ^ swz16(row) = (l%8) ^ (l/8).
    const int lj = (lane & 7) ^ swz16(lrow);
    uint32_t a_off[A_IT];
#pragma unroll
    for (int i = 0; i < A_IT; ++i) {
        const int r = (i * NL + (wave % NL)) * 8 + lrow;
        int src;
        if constexpr (GROUP == GROUP_DENSE) src = m0 + min(r, rows_valid - 1);
        else src = s_src[r];
        a_off[i] = (uint32_t)src * (uint32_t)K + lj * 16;
    }

    const int li = lane & 15, lg = lane >> 4;
    const uint32_t frag0 = li * kKBlock + ((lg ^ swz16(li)) << 4);
    const uint32_t frag1 = frag0 ^ 64;
    // Weight fragments.  Row r of column tile tn (the MFMA's 16 output columns) is slab row
    //   (tn/2)*32 + (r/4)*8 + (tn%2)*4 + r%4
    // instead of tn*16 + r: a lane's four accumulator columns 4*lg .. 4*lg+3 of tiles 2t and 2t+1 are then
    // the eight CONSECUTIVE output columns 32t + 8*lg .. +7, which the epilogue stores straight from
    // registers as one 16-byte write.  The slab's chunk swizzle uses row bits 0, 1 and 3 (the bits that
    // vary over a fragment's sixteen rows besides the repeated one), so the reads stay conflict-free.
    const int wrow = ((li >> 2) << 3) | (li & 3);
    const uint32_t wfrag0 = wrow * kKBlock + ((lg ^ swz_w(wrow)) << 4);
    const uint32_t wfrag1 = wfrag0 ^ 64;
    auto w_tile_row = [](int tn) { return (tn >> 1) * 32 + (tn & 1) * 4; };
    // Rows: wave row wm owns the 16-row groups wm, wm + WGM, wm + 2*WGM, ... of the tile (not a contiguous
    // block of rows), so that a tile whose valid rows are a prefix -- the last row tile of an expert or
    // of the problem -- spreads them evenly over the waves and every wave can skip the same share of
    // its MFMAs (see `n_tm` below).
    auto tile_row = [&](int tm) { return (tm * WGM + wm) * 16; };
    const uint32_t a_frag_base = wm * 16 * kKBlock, b_frag_base = wn * WTN * kKBlock;

    // Block scales.  The weight scale is one scalar per wave and K step (table sBs).  The activation
    // scales (one per tile row and K step) come in chunks of kScaleChunk = 8 K steps through a
    // double-buffered LDS table: one 4-byte direct load covers 8 rows x 8 consecutive K steps, i.e. 8
    // runs of 32 contiguous bytes -- fetching one K step for 64 rows would touch 64 cache lines per
    // instruction, eight times what a slab load does.  Chunk c+1 is requested while chunk c is in use,
    // one 8-row group per wave and K step.  Lane l of the load for row group g lands at float
    // 64*g + l of the chunk's buffer; it fetches row 8g + l/8 at chunk step (l%8 - l/8) % 8, so step s of
    // row r sits at position (s + r) % 8 of the row's eight floats and the 16 rows a fragment's lanes
    // read in one K step spread over the banks.
    constexpr int S_GROUPS = BM / 8;                     // 8-row groups of the tile
    constexpr int S_PHASES = (S_GROUPS + NL - 1) / NL;   // K steps a chunk's loads are spread over
    static_assert(S_PHASES <= kScaleChunk, "a chunk is fetched within the chunk before it");
    const int s_kbi = ((lane & 7) - (lane >> 3)) & 7;    // chunk step this lane fetches
    v4f acc[TN][TM];
#pragma unroll
    for (int tn = 0; tn < TN; ++tn)
#pragma unroll
        for (int tm = 0; tm < TM; ++tm) acc[tn][tm] = v4f{0.f, 0.f, 0.f, 0.f};

    // Direct global->LDS loads of one K step, as buffer loads: 32-bit per-lane offset + scalar
    // K offset, no 64-bit address arithmetic in the loop.  K is a multiple of 128 here (the host
    // sends other K to the fallback kernel), so every lane's 16 bytes are in range.
    const v4i rsrc_a = make_rsrc(p.A);
    auto issue_a1 = [&](int i, int kstep, uint8_t* dA) {
        direct_load_b128(rsrc_a, lds_address(dA) + wave * 1024 + i * NL * 1024, a_off[i], kstep * kKBlock);
    };
    auto issue_a = [&](int kstep, uint8_t* dA) {
#pragma unroll
        for (int i = 0; i < A_IT; ++i) issue_a1(i, kstep, dA);
    };
    const v4i rsrc_s = make_rsrc(p.As);
    // direct load of row group ph*NL + wave of chunk `chunk` (K steps ks + 8*chunk ..), if this wave has one
    auto issue_s = [&](int chunk, int ph) {
        if constexpr (BLOCKSCALE) {
            const int g = ph * NL + wave;
            if (p.As && g < S_GROUPS) {
                const int r = g * 8 + (lane >> 3);
                int src;
                if constexpr (GROUP == GROUP_DENSE) src = m0 + min(r, rows_valid - 1);
                else src = s_src[r];
                const int kb = min(ks + chunk * kScaleChunk + s_kbi, p.kblocks - 1);
                const uint32_t off = ((uint32_t)src * (uint32_t)p.kblocks + (uint32_t)kb) * 4u;
                direct_load_b32(rsrc_s, lds_address(sTab) + ((chunk & 1) * BM * kScaleChunk + g * 64) * 4, off, 0);
            }
        }
    };
    float sc[TM];
    float sc_up[ACT ? TM : 1];  // fused activation: column tiles TN/2 .. TN-1 are up columns, with their own weight block
    // position of row tile_row(0) + li in a chunk buffer, without the step rotation (see above)
    const int s_rbase = (wm * 2 + (li >> 3)) * 64 + (li & 7) * 8;
    auto read_scales = [&](auto ntm_tag, int kstep) {
        constexpr int NTM = decltype(ntm_tag)::value;
        if constexpr (BLOCKSCALE && NTM > 0) {
            const int kk = kstep - ks;
            const float* cS = sTab + ((kk / kScaleChunk) & 1) * (BM * kScaleChunk) + s_rbase + (((kk % kScaleChunk) + li) & 7);
            const float bs = sBs[ACT ? 0 : (wn * WTN) / 128][kstep];
#pragma unroll
            for (int tm = 0; tm < NTM; ++tm) {
                const float as = cS[tm * (WGM * 128)];
                sc[tm] = as * bs;
                if constexpr (ACT) sc_up[tm] = as * sBs[1][kstep];
            }
        }
    };
    auto scale_of = [&](int tn, int tm) -> float {
        if constexpr (ACT) return tn >= TN / 2 ? sc_up[tm] : sc[tm];
        else return sc[tm];
    };
    v8i af[TM];
    auto read_a = [&](auto ntm_tag, const uint8_t* cA) {
        constexpr int NTM = decltype(ntm_tag)::value;
#pragma unroll
        for (int tm = 0; tm < NTM; ++tm) {
            const uint8_t* base = cA + a_frag_base + tm * (WGM * 16 * kKBlock);
            af[tm] = join(*reinterpret_cast<const v4i*>(base + frag0),
                          *reinterpret_cast<const v4i*>(base + frag1));
        }
    };
    // `after_tile(tn)` runs behind the MFMAs of column tile tn (the step's direct loads are issued there)
    auto mma = [&](auto ntm_tag, const uint8_t* cB, auto&& after_tile) {
        constexpr int NTM = decltype(ntm_tag)::value;  // this wave's row groups that hold valid rows
        if constexpr (NTM == 0) {
#pragma unroll
            for (int tn = 0; tn < TN; ++tn) after_tile(tn);
            return;
        } else if constexpr (BLOCKSCALE) {
            // One MFMA (into a zeroed 16x16 product), then the four scale-and-add operations of the
            // product issued two MFMAs earlier: the matrix pipe works on the MFMA for 32 clocks while
            // the wave issues 16 clocks of VALU work behind it, and a product is complete (two MFMA
            // slots old) when it is read.  Three product registers rotate.  The scheduling fence after
            // every such pair keeps the compiler from collecting the VALU work behind the last MFMA
            // (where the matrix pipe would idle); the weight fragment of column tile tn+1 is fetched
            // during column tile tn.
            constexpr int NJ = TN * NTM;
            v4f part[3];
            v8i wf[2];
            auto read_w = [&](int tn) {
                const uint8_t* base = cB + b_frag_base + w_tile_row(tn) * kKBlock;
                wf[tn & 1] = join(*reinterpret_cast<const v4i*>(base + wfrag0), *reinterpret_cast<const v4i*>(base + wfrag1));
            };
            read_w(0);
#pragma unroll
            for (int j = 0; j < NJ; ++j) {
                const int tn = j / NTM, tm = j % NTM;
                part[j % 3] = mfma_e4m3(wf[tn & 1], af[tm], v4f{0.f, 0.f, 0.f, 0.f});
                if (tm == 0 && tn + 1 < TN) read_w(tn + 1);
                if (j >= 2) acc[(j - 2) / NTM][(j - 2) % NTM] += part[(j - 2) % 3] * scale_of((j - 2) / NTM, (j - 2) % NTM);
                __builtin_amdgcn_sched_barrier(0);
                if (tm == NTM - 1) {
                    after_tile(tn);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
#pragma unroll
            for (int j = NJ - 2; j < NJ; ++j) acc[j / NTM][j % NTM] += part[j % 3] * scale_of(j / NTM, j % NTM);
            // Pin the scale-and-add results here: without a use in this block the compiler sinks the
            // whole VALU chain behind the next conditional (a later K step's loader test), keeps every
            // 16x16 product alive until then and spills.  No instruction is emitted.
#pragma unroll
            for (int tn = 0; tn < TN; ++tn)
#pragma unroll
                for (int tm = 0; tm < NTM; ++tm) asm volatile("" : "+v"(acc[tn][tm]));
        } else {
            // weight fragments two column tiles ahead; the order is pinned (the direct loads are inline assembly, which
            // the compiler's own interleaving hints cannot place)
            v8i wf[2];
            auto read_w = [&](int tn) {
                const uint8_t* base = cB + b_frag_base + w_tile_row(tn) * kKBlock;
                wf[tn & 1] = join(*reinterpret_cast<const v4i*>(base + wfrag0), *reinterpret_cast<const v4i*>(base + wfrag1));
            };
            read_w(0);
            read_w(1);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int tn = 0; tn < TN; ++tn) {
#pragma unroll
                for (int tm = 0; tm < NTM; ++tm) acc[tn][tm] = mfma_e4m3(wf[tn & 1], af[tm], acc[tn][tm]);
                __builtin_amdgcn_sched_barrier(0);
                after_tile(tn);
                if (tn + 2 < TN) read_w(tn + 2);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    };
    // vmcnt(n): this wave's direct loads, except the n most recent, have landed in LDS.
    constexpr int kWaitAllButA = 0x0F70 | (A_IT & 15) | ((A_IT >> 4) << 14);
    constexpr int kWaitAll = 0x0F70;
    constexpr int kWaitLds = 0xC07F;  // lgkmcnt(0) only
    // Workgroup barrier without the memory fence of __syncthreads(): that fence would also wait
    // for every direct load in flight (vmcnt(0)), which is exactly what the deeper prefetch must
    // not do.  LDS reads are ordered with lgkmcnt, direct loads with the vmcnt waits below.
    auto lds_barrier = [&]() {
        __builtin_amdgcn_s_waitcnt(kWaitLds);
        __builtin_amdgcn_s_barrier();
    };

    // ---------------------------------------------------------------- main loop
    // Stage buffers (sA0,sB0) and (sA1,sB1); step k computes from stage k%2.  The B slab of a stage
    // is read throughout the step, the A slab only at its start (the A fragments stay in
    // registers), so A is prefetched two steps ahead and B one:
    //   top of step k : issue B(k+1) -> other stage (and one row group of the next chunk of activation
    //                   scales);  read A fragments (and scales) of stage k%2;  barrier
    //                   (every wave holds its A fragments: that A slab is free)
    //   then          : MFMAs with B fragments streamed from LDS; behind each of the first column tiles' MFMAs one
    //                   or two of the direct loads of A(k+2) -> this stage's A slab
    //   end of step k : wait for all direct loads except A(k+2);  barrier
    // (Measured on the block-scaled and grouped forms: dealing B(k+1) over the column tiles as well, so that no load
    // is issued in a burst, leaves the weights half a step to land and is 5-15 % slower.)
    // Steps past the end are clamped to the last step: they re-fetch it into an idle slab, which
    // keeps the loop body free of branches.
    const int nsteps = ks_end - ks, last = ks_end - 1;
    // Routed weight of each tile row (thread t holds row t's): needed by the epilogue only, so it is
    // requested now, rides through the K loop in a register and goes to LDS after the loop.
    float row_w = 1.0f;
    if constexpr (GROUP == GROUP_GATHER) {
        if (tid < BM && p.row_weight) {
            const int dst = s_dst[tid];
            if (dst >= 0) row_w = p.row_weight[dst];
        }
    }
    issue_a(ks, sA0);  // (the weight slab of this step is in flight since the top of the kernel)
#pragma unroll
    for (int ph = 0; ph < S_PHASES; ++ph) issue_s(0, ph);
    issue_a(min(ks + 1, last), sA1);
    __builtin_amdgcn_s_waitcnt(kWaitAllButA);  // a wave without loads in flight passes at once
    lds_barrier();
    // The loop exists once per number of row groups a wave may have to compute (NTM = 0 .. TM): the
    // waves of a workgroup can run different copies, every copy issues the same loads and barriers.
    auto k_loop = [&](auto ntm_tag) {
        auto step = [&](int k, uint8_t* cA, uint8_t* cB, uint8_t* oB) {
            // the weight slab of step k+1 is requested first: it has this whole step to land
            issue_b(min(k + 1, last), oB);
            issue_s((k - ks) / kScaleChunk + 1, (k - ks) % kScaleChunk);
            read_a(ntm_tag, cA);
            read_scales(ntm_tag, k);
            lds_barrier();
            // the activation slab of step k+2 goes into the slab whose fragments every wave holds in registers since the
            // barrier above, one or two loads behind each of the first column tiles' MFMAs
            constexpr int PER = (A_IT + TN - 1) / TN;
            const int ka2 = min(k + 2, last);
            mma(ntm_tag, cB, [&](int tn) {
#pragma unroll
                for (int q = 0; q < PER; ++q) {
                    const int idx = tn * PER + q;
                    if (idx < A_IT) issue_a1(idx, ka2, cA);
                }
            });
            __builtin_amdgcn_s_waitcnt(kWaitAllButA);
            lds_barrier();
        };
        int i = 0;
        for (; i + 1 < nsteps; i += 2) {
            step(ks + i, sA0, sB0, sB1);
            step(ks + i + 1, sA1, sB1, sB0);
        }
        if (i < nsteps) step(ks + i, sA0, sB0, sB1);
    };
    // Row groups of this wave that hold at least one valid row, counted up to the last such group (the
    // valid rows of a tile are a prefix wherever the row maps come from this library's own alignment;
    // any other map only costs the skipped work).  Dense problems skip nothing: one copy of the loop.
    int n_tm = TM;
    if constexpr (GROUP == GROUP_DENSE) {
        k_loop(std::integral_constant<int, TM>{});
    } else {
        static_assert(TM == 4, "dispatch below");
        n_tm = 0;
#pragma unroll
        for (int tm = 0; tm < TM; ++tm)
            if (__ballot(s_dst[tile_row(tm) + li] >= 0) != 0) n_tm = tm + 1;
        n_tm = __builtin_amdgcn_readfirstlane(n_tm);
        if (n_tm == 4) k_loop(std::integral_constant<int, 4>{});
        else if (n_tm == 3) k_loop(std::integral_constant<int, 3>{});
        else if (n_tm == 2) k_loop(std::integral_constant<int, 2>{});
        else if (n_tm == 1) k_loop(std::integral_constant<int, 1>{});
        else k_loop(std::integral_constant<int, 0>{});
    }
    __builtin_amdgcn_s_waitcnt(kWaitAll);
    if constexpr (GROUP == GROUP_GATHER) {
        if (tid < BM) s_w[tid] = row_w;
    }
    __syncthreads();

    // ---------------------------------------------------------------- fused activation epilogue
    // Wave (wm, wn) holds, for its 16-row groups, gate columns (WTN/2)*wn .. of the tile in its first
    // TN/2 column tiles and the matching up columns in the other TN/2: a lane has gate and up of the same
    // elements of each of its rows in registers and computes, exactly as the stand-alone kernel
    // does on the stored GEMM output,
    //   g = T(acc_gate), u = T(acc_up), act = T(g * sigmoid(g) * u)          (T = the 16-bit type)
    // The maximum of a row's 128 activations (4 lanes x WGN waves) goes through two shuffles and one LDS
    // exchange; then scale = amax / 448 (1 for an all-zero group), codes = e4m3(act / scale), written
    // 8 bytes per lane and column-tile pair.
    if constexpr (ACT) {
        float actv[TM][TN / 4][8];
        float* const amax_mine = sTab + wn * BM;  // (the scale table is idle now) one row of maxima per wave column
        // (one branch on the type around all 64 elements of the lane, so that their chains interleave)
        auto activate = [&](auto type_tag) {
            using T = decltype(type_tag);
#pragma unroll
            for (int tm = 0; tm < TM; ++tm) {
                if (tm < n_tm) {  // wave-uniform: row groups without a valid row were not computed and are not stored
#pragma unroll
                    for (int tp = 0; tp < TN / 4; ++tp)
#pragma unroll
                        for (int q = 0; q < 8; ++q) {
                            const float ga = acc[2 * tp + (q >> 2)][tm][q & 3], ua = acc[TN / 2 + 2 * tp + (q >> 2)][tm][q & 3];
                            actv[tm][tp][q] = silu_mul_round<T>((float)(T)ga, (float)(T)ua);
                        }
                } else {
#pragma unroll
                    for (int tp = 0; tp < TN / 4; ++tp)
#pragma unroll
                        for (int q = 0; q < 8; ++q) actv[tm][tp][q] = 0.f;
                }
            }
        };
        if (p.act_is_bf16) activate(__bf16{});
        else activate(_Float16{});
#pragma unroll
        for (int tm = 0; tm < TM; ++tm) {
            float amax = 0.f;
#pragma unroll
            for (int tp = 0; tp < TN / 4; ++tp)
#pragma unroll
                for (int q = 0; q < 8; ++q) amax = fmaxf(amax, fabsf(actv[tm][tp][q]));
            amax = fmaxf(amax, __shfl_xor(amax, 16));
            amax = fmaxf(amax, __shfl_xor(amax, 32));
            if (lg == 0) amax_mine[tile_row(tm) + li] = amax;
        }
        __syncthreads();
        uint8_t* const qout = reinterpret_cast<uint8_t*>(p.C);
        const int groups_per_row = p.inter / 128;
#pragma unroll
        for (int tm = 0; tm < TM; ++tm) {
            const int rt = tile_row(tm) + li;
            float amax = sTab[rt];
#pragma unroll
            for (int w = 1; w < WGN; ++w) amax = fmaxf(amax, sTab[w * BM + rt]);
            const float sc1 = amax == 0.f ? 1.0f : amax / 448.0f;
            const int dst = s_dst[rt];
            if (dst < 0) continue;
            const ScaleDivider div(sc1);
            if (div.fast) {
#pragma unroll
                for (int tp = 0; tp < TN / 4; ++tp)
#pragma unroll
                    for (int q = 0; q < 8; ++q) actv[tm][tp][q] = div.quotient(actv[tm][tp][q]);
            } else {
#pragma unroll
                for (int tp = 0; tp < TN / 4; ++tp)
#pragma unroll
                    for (int q = 0; q < 8; ++q) actv[tm][tp][q] = actv[tm][tp][q] / sc1;
            }
#pragma unroll
            for (int tp = 0; tp < TN / 4; ++tp) {
                int packed[2];
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    float c[4];
#pragma unroll
                    for (int i = 0; i < 4; ++i) c[i] = fminf(fmaxf(actv[tm][tp][4 * h + i], -448.0f), 448.0f);
                    int w = 0;
                    w = __builtin_amdgcn_cvt_pk_fp8_f32(c[0], c[1], w, false);
                    w = __builtin_amdgcn_cvt_pk_fp8_f32(c[2], c[3], w, true);
                    packed[h] = w;
                }
                *reinterpret_cast<v2i*>(qout + (int64_t)dst * p.inter + n0 + wn * (WTN / 2) + tp * 32 + lg * 8) = v2i{packed[0], packed[1]};
            }
            if (wn == 0 && lg == 0) p.act_scales[(int64_t)dst * groups_per_row + tile_n] = sc1;
        }
        return;
    }

    // ---------------------------------------------------------------- epilogue
    // Straight from the accumulators: for every pair of column tiles a lane holds eight consecutive
    // output columns of row 16*tm + li (see the weight fragment addresses), i.e. one 16-byte store of
    // bf16/f16 or two of fp32; the four lanes of a row cover 32 consecutive columns.
    float scale = p.alpha;
    if constexpr (!BLOCKSCALE) {
        if (p.As) scale *= p.As[0];
        if (p.Bs) scale *= p.Bs[0];
    }
    const bool vec_ok = p.vec_store != 0 && (p.N % 8) == 0;  // 8-wide rows stay 16-byte aligned
    const int64_t MN = (int64_t)p.M * p.N;
    int dsts[TM];
    float rws[TM];
#pragma unroll
    for (int tm = 0; tm < TM; ++tm) {
        const int rt = tile_row(tm) + li;  // row inside the workgroup tile
        if constexpr (GROUP == GROUP_DENSE) dsts[tm] = rt < rows_valid ? m0 + rt : -1;
        else dsts[tm] = s_dst[rt];
        rws[tm] = scale;
        if constexpr (GROUP == GROUP_GATHER) rws[tm] *= s_w[rt];
    }
    auto emit = [&](auto type_tag) {
        constexpr int OT = decltype(type_tag)::value;
        // (row group outermost: the two 64-byte halves of an output line are written back to back)
#pragma unroll
        for (int tm = 0; tm < TM; ++tm) {
#pragma unroll
            for (int tp = 0; tp < TN / 2; ++tp) {
                const int col = n0 + wn * WTN + tp * 32 + lg * 8;
                if (dsts[tm] < 0 || col >= p.N) continue;
                if constexpr (SPLIT)
                    store8(p.partials + (int64_t)blockIdx.y * MN, OUT_F32, dsts[tm], col, p.N, p.N, acc[2 * tp][tm], acc[2 * tp + 1][tm], 0.f, vec_ok);
                else
                    store8(p.C, OT, dsts[tm], col, p.N, p.ldc, acc[2 * tp][tm] * rws[tm], acc[2 * tp + 1][tm] * rws[tm], p.beta, vec_ok);
            }
        }
    };
    if (SPLIT || p.out_type == OUT_BF16) emit(std::integral_constant<int, OUT_BF16>{});
    else if (p.out_type == OUT_F32) emit(std::integral_constant<int, OUT_F32>{});
    else if (p.out_type == OUT_F8) emit(std::integral_constant<int, OUT_F8>{});
    else emit(std::integral_constant<int, OUT_F16>{});

#endif
}

template <int BM, int BN, int WGM, int WGN, bool BLOCKSCALE, int GROUP, bool SPLIT>
__global__ void __launch_bounds__(64 * WGM * WGN, (WGM * WGN == 4 ? 2 : 1)) fp8_gemm_tile_kernel(const GemmParams p) {
    fp8_gemm_tile_body<BM, BN, WGM, WGN, BLOCKSCALE, GROUP, SPLIT>(p, (int)blockIdx.x);
}

// A list of independent per-tensor-scaled GEMMs in one launch (tilegym.ops.group_gemm,
// src/tilegym/ops/cutile/group_gemm.py:170-197).  The problems travel in the kernel arguments;
// a workgroup finds the problem that owns its tile with a scan over the tile prefix and then runs
// the dense body on it.
template <int BM, int BN, int WGM, int WGN>
__global__ void __launch_bounds__(64 * WGM * WGN, (WGM * WGN == 4 ? 2 : 1)) fp8_gemm_tile_list_kernel(const GemmList gl) {
    const int bid = (int)blockIdx.x;
    int i = 0, start = 0;
    while (i + 1 < gl.count && bid >= gl.prob[i].tile_end) {
        start = gl.prob[i].tile_end;
        ++i;
    }
    GemmParams p{};
    p.A = gl.prob[i].A; p.B = gl.prob[i].B; p.C = gl.prob[i].C;
    p.As = gl.prob[i].As; p.Bs = gl.prob[i].Bs;
    p.M = gl.prob[i].M; p.N = gl.prob[i].N; p.K = gl.prob[i].K; p.ldc = p.N;
    p.kblocks = p.K / kKBlock; p.nblocks = (p.N + 127) / 128;
    p.alpha = gl.alpha; p.beta = 0.f;
    p.out_type = gl.out_type;
    p.vec_store = gl.prob[i].vec_store;
    p.split_k = 1; p.ksteps_per_split = p.kblocks;
    p.E = 1; p.top_k = 1;
    fp8_gemm_tile_body<BM, BN, WGM, WGN, false, GROUP_DENSE, false>(p, bid - start);
}

template <int BM, int BN, int WGM, int WGN>
inline hipError_t launch_tile_list(const GemmList& gl, int grid_x, hipStream_t stream) {
    auto kern = fp8_gemm_tile_list_kernel<BM, BN, WGM, WGN>;
    hipLaunchKernelGGL(kern, dim3(grid_x, 1, 1), dim3(64 * WGM * WGN, 1, 1), 0, stream, gl);
    return hipGetLastError();
}

template <int BM, int BN, int WGM, int WGN, bool BLOCKSCALE, int GROUP, bool SPLIT>
inline hipError_t launch_tile(const GemmParams& p, int grid_x, int grid_y, hipStream_t stream) {
    auto kern = fp8_gemm_tile_kernel<BM, BN, WGM, WGN, BLOCKSCALE, GROUP, SPLIT>;
    hipLaunchKernelGGL(kern, dim3(grid_x, grid_y, 1), dim3(64 * WGM * WGN, 1, 1), 0, stream, p);
    return hipGetLastError();
}

}  // namespace tg
