// Device side of moe_align_block_size (see moe_align.hip for the algorithm): the body of one workgroup, shared by the
// stand-alone kernel and by the kernel that runs it beside the activation quantizer (moe_prepare.hip).
#pragma once
#include "tg_host.h"

namespace tg {

constexpr int kAlignWaves = 16;
constexpr int kAlignMaxGrid = 32;
constexpr int kAlignMaxExperts = 512;   // LDS: (16 + 5) rows x E counters stay under 48 KiB

// Work of workgroup g of G (64 * kAlignWaves threads; `lds`: (kAlignWaves + 4) * E + 1 + kAlignWaves ints of dynamic LDS).
template <typename IdT>
__device__ __forceinline__ void moe_align_body(const IdT* __restrict__ ids, int numel, int E,
                                               int block_size, int* __restrict__ sorted_ids, int cap,
                                               int* __restrict__ expert_ids, int nblk,
                                               int* __restrict__ num_post_pad, int* __restrict__ cumsum,
                                               int* __restrict__ max_cnt, int* lds, const int G, const int g) {
    int* cnt = lds;                         // [kAlignWaves][E]: per-wave counts, later per-wave write cursors
    int* before = cnt + kAlignWaves * E;    // [E]: ids of the expert in earlier workgroups' slices
    int* after = before + E;                // [E]: ... in later workgroups' slices
    int* tot = after + E;                   // [E]: unpadded group sizes
    int* pad_start = tot + E;               // [E + 1]: padded prefix
    int* scan_tmp = pad_start + E + 1;      // [kAlignWaves]: wave totals of the scan
    __shared__ int s_max;

    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int NT = 64 * kAlignWaves;
    for (int i = tid; i < (kAlignWaves + 2) * E; i += NT) cnt[i] = 0;  // cnt, before, after
    if (tid == 0) s_max = 0;
    __syncthreads();

    // Both passes fetch kBatch x 64 ids before they use the first one: the loads of a batch are in
    // flight together, so a pass pays the memory latency once per batch and not once per 64 ids.
    constexpr int kBatch = 8;
    const int per_wave = ((numel + G * kAlignWaves - 1) / (G * kAlignWaves) + 63) / 64 * 64;
    const int wg_lo = min(g * kAlignWaves * per_wave, numel), wg_hi = min(wg_lo + kAlignWaves * per_wave, numel);
    constexpr int kBatch1 = 12;  // pass 1 holds nothing else in registers: deeper batches
    for (int i0 = wave * 64 * kBatch1; i0 < numel; i0 += NT * kBatch1) {
        IdT ev[kBatch1];
#pragma unroll
        for (int u = 0; u < kBatch1; ++u) {
            const int i = i0 + u * 64 + lane;
            ev[u] = i < numel ? ids[i] : (IdT)-1;
        }
#pragma unroll
        for (int u = 0; u < kBatch1; ++u) {
            // slice bounds are multiples of 64 (or the end of the sequence): the 64 ids of a load share their owner
            const int c = i0 + u * 64;
            int* row = c < wg_lo ? before : c >= wg_hi ? after : cnt + ((c - wg_lo) / per_wave) * E;
            if (ev[u] >= 0 && ev[u] < E) atomicAdd(&row[(int)ev[u]], 1);
        }
    }
    __syncthreads();

    // per expert: per-wave exclusive offsets inside the expert's group (kept in cnt), total, padded size.
    // 16 lanes per expert, lane w holding the row of wave w: a 16-wide shuffle scan instead of a
    // serial walk over the rows.
    for (int idx = tid; idx < E * kAlignWaves; idx += NT) {
        const int e = idx / kAlignWaves, w = idx % kAlignWaves;
        const int c = cnt[w * E + e];
        int incl_w = c;
#pragma unroll
        for (int d = 1; d < kAlignWaves; d <<= 1) {
            const int t = __shfl_up(incl_w, d, kAlignWaves);
            if (w >= d) incl_w += t;
        }
        const int b = before[e];
        cnt[w * E + e] = b + incl_w - c;
        if (w == kAlignWaves - 1) {
            const int total = b + incl_w + after[e];
            atomicMax(&s_max, total);
            tot[e] = total;
        }
    }
    __syncthreads();
    int padded = 0;
    if (tid < E) padded = (tot[tid] + block_size - 1) / block_size * block_size;  // E <= 512 < NT
    // inclusive scan of the padded sizes over the experts (thread e holds expert e, E <= 512 = 8 waves):
    // shuffle scan inside each wave, wave totals through LDS
    int incl = padded;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const int t = __shfl_up(incl, d);
        if (lane >= d) incl += t;
    }
    if (lane == 63) scan_tmp[wave] = incl;
    __syncthreads();
    int wave_base = 0, total_padded = 0;
    for (int w = 0; w < kAlignWaves; ++w) {
        const int t = scan_tmp[w];
        if (w < wave) wave_base += t;
        total_padded += t;
    }
    if (tid < E) {
        const int my_start = wave_base + incl - padded;  // exclusive
        pad_start[tid] = my_start;
        if (g == 0) cumsum[tid] = my_start;
    }
    if (tid == 0) pad_start[E] = total_padded;
    if (tid == 0 && g == 0) {
        cumsum[E] = total_padded;
        num_post_pad[0] = total_padded;
        max_cnt[0] = s_max;
    }
    for (int i = total_padded + g * NT + tid; i < cap; i += G * NT) sorted_ids[i] = numel;
    for (int b = total_padded / block_size + g * NT + tid; b < nblk; b += G * NT) expert_ids[b] = 0;
    __syncthreads();
    // sentinel tail of every group and the block -> expert table: one wave of the grid per expert at a time
    for (int e = g * kAlignWaves + wave; e < E; e += G * kAlignWaves) {
        const int start = pad_start[e], end = pad_start[e + 1];
        for (int i = start + tot[e] + lane; i < end; i += 64) sorted_ids[i] = numel;
        for (int b = start / block_size + lane; b < end / block_size; b += 64) expert_ids[b] = e;
    }

    // pass 2: stable scatter.  `mine[e]` is this wave's next free rank inside expert e's group.
    // Lanes holding the same expert are found without a loop over the distinct experts: one ballot
    // per bit of the expert label, combined into the mask of lanes that agree with this lane on
    // every bit.  The lowest lane of each such set advances the cursor.
    int* mine = cnt + wave * E;
    const int lo = min(wg_lo + wave * per_wave, wg_hi), hi = min(lo + per_wave, wg_hi);
    int nbits = 0;
    while ((1 << nbits) < E) ++nbits;
    const unsigned long long below = (1ull << lane) - 1ull;
    for (int i0 = lo; i0 < hi; i0 += 64 * kBatch) {
        long long ev[kBatch];
#pragma unroll
        for (int u = 0; u < kBatch; ++u) {
            const int i = i0 + u * 64 + lane;
            ev[u] = i < hi ? (long long)ids[i] : -1;
        }
#pragma unroll
        for (int u = 0; u < kBatch; ++u) {
            if (i0 + u * 64 >= hi) break;  // wave-uniform
            const int i = i0 + u * 64 + lane;
            const bool valid = ev[u] >= 0 && ev[u] < E;
            const int e = valid ? (int)ev[u] : 0;
            unsigned long long same = __ballot(valid);
            for (int b = 0; b < nbits; ++b) {
                const unsigned long long m = __ballot((e >> b) & 1);
                same &= ((e >> b) & 1) ? m : ~m;
            }
            if (valid) {
                const int base = mine[e];
                const int rank = __popcll(same & below);
                sorted_ids[pad_start[e] + base + rank] = i;
                // every lane of the set has read the cursor before its first lane rewrites it: the
                // read and the write below are separate LDS instructions of one wave, executed in order
                if (rank == 0) mine[e] = base + __popcll(same);
            }
        }
    }
}

inline size_t moe_align_lds_bytes(int E) { return (size_t)((kAlignWaves + 4) * E + 1 + kAlignWaves) * sizeof(int); }
inline int moe_align_grid(int numel) {
    // one workgroup per 1024 ids (every workgroup reads all ids, so a larger grid only pays while the
    // scattered stores of a slice outweigh that read)
    int grid = (numel + 1023) / 1024;
    return grid < 1 ? 1 : grid > kAlignMaxGrid ? kAlignMaxGrid : grid;
}

}  // namespace tg
