// moe_align_block_size on the device, one launch: groups the (token, slot) pairs of a top-k
// routing by expert, pads every expert's group to a multiple of block_size and emits the
// block -> expert table the gather GEMM walks.  Output contract of
// src/tilegym/ops/cutile/moe_align_block.py:205-268 (torch statement: src/tilegym/ops/moe_interface.py:30-79):
//   sorted_ids[cap]   flat pair indices grouped by expert, ascending inside an expert (stable),
//                     every other position = numel (the sentinel), cap = numel + E * (block_size - 1)
//   expert_ids[nblk]  expert of each block of block_size positions (0 past the padded total)
//   num_post_pad[1]   padded total;  cumsum[E + 1] padded prefix;  max_cnt[1] largest expert count
//
// One workgroup of 16 waves.  Wave w owns the contiguous slice w of the flat id sequence.
//   pass 1: every wave histograms its slice into its own LDS row (LDS atomics; order-free)
//   scan  : thread e adds the rows of expert e (giving each wave its start inside the expert's
//           group) and the padded group sizes are prefix-summed over the experts
//   pass 2: every wave walks its slice 64 ids at a time; lanes with equal experts are ranked by
//           lane order with ballots, so the result does not depend on any atomic's timing
#include "tg_host.h"

namespace tg {

constexpr int kAlignWaves = 16;
constexpr int kAlignMaxExperts = 512;   // LDS: 16 rows x E counters + scan space stays under 48 KiB

template <typename IdT>
__global__ void __launch_bounds__(64 * kAlignWaves) moe_align_kernel(const IdT* __restrict__ ids, int numel, int E,
                                                                    int block_size, int* __restrict__ sorted_ids, int cap,
                                                                    int* __restrict__ expert_ids, int nblk,
                                                                    int* __restrict__ num_post_pad, int* __restrict__ cumsum,
                                                                    int* __restrict__ max_cnt) {
    extern __shared__ int lds[];
    int* cnt = lds;                         // [kAlignWaves][E]: per-wave counts, later per-wave write cursors
    int* pad_start = lds + kAlignWaves * E; // [E + 1]: padded prefix
    int* scan_tmp = pad_start + E + 1;      // [1024]
    __shared__ int s_max;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int NT = 64 * kAlignWaves;
    for (int i = tid; i < kAlignWaves * E; i += NT) cnt[i] = 0;
    if (tid == 0) s_max = 0;
    __syncthreads();

    const int per_wave = ((numel + kAlignWaves - 1) / kAlignWaves + 63) / 64 * 64;
    const int lo = min(wave * per_wave, numel), hi = min(lo + per_wave, numel);
    int* mine = cnt + wave * E;
    for (int i = lo + lane; i < hi; i += 64) {
        const long long e = (long long)ids[i];
        if (e >= 0 && e < E) atomicAdd(&mine[(int)e], 1);
    }
    __syncthreads();

    // per expert: total, per-wave exclusive offsets (kept in cnt), padded size
    int padded = 0;
    for (int e = tid; e < E; e += NT) {  // E <= NT: at most one expert per thread
        int total = 0;
        for (int w = 0; w < kAlignWaves; ++w) {
            const int c = cnt[w * E + e];
            cnt[w * E + e] = total;
            total += c;
        }
        padded = (total + block_size - 1) / block_size * block_size;
        atomicMax(&s_max, total);
        scan_tmp[e] = padded;
        pad_start[e] = total;  // temporarily: unpadded total
    }
    for (int e = E + tid; e < 1024; e += NT) scan_tmp[e] = 0;
    __syncthreads();
    // inclusive scan of scan_tmp[0..1023] (Hillis-Steele, one element per thread)
    for (int d = 1; d < 1024; d <<= 1) {
        const int v = (tid >= d) ? scan_tmp[tid - d] : 0;
        __syncthreads();
        scan_tmp[tid] += v;
        __syncthreads();
    }
    const int total_padded = scan_tmp[1023];
    int my_total = 0, my_start = 0;
    if (tid < E) {
        my_total = pad_start[tid];
        my_start = scan_tmp[tid] - padded;  // exclusive
    }
    __syncthreads();
    if (tid < E) {
        pad_start[tid] = my_start;
        cumsum[tid] = my_start;
        for (int i = my_start + my_total; i < my_start + padded; ++i) sorted_ids[i] = numel;
        for (int b = my_start / block_size; b < (my_start + padded) / block_size; ++b) expert_ids[b] = tid;
    }
    if (tid == 0) {
        pad_start[E] = total_padded;
        cumsum[E] = total_padded;
        num_post_pad[0] = total_padded;
        max_cnt[0] = s_max;
    }
    for (int i = total_padded + tid; i < cap; i += NT) sorted_ids[i] = numel;
    for (int b = total_padded / block_size + tid; b < nblk; b += NT) expert_ids[b] = 0;
    __syncthreads();

    // pass 2: stable scatter.  `mine[e]` is this wave's next free rank inside expert e's group.
    // Lanes holding the same expert are found without a loop over the distinct experts: one ballot
    // per bit of the expert label, combined into the mask of lanes that agree with this lane on
    // every bit.  The lowest lane of each such set advances the cursor.
    int nbits = 0;
    while ((1 << nbits) < E) ++nbits;
    const unsigned long long below = (1ull << lane) - 1ull;
    for (int i0 = lo; i0 < hi; i0 += 64) {
        const int i = i0 + lane;
        long long e64 = -1;
        if (i < hi) e64 = (long long)ids[i];
        const bool valid = e64 >= 0 && e64 < E;
        const int e = valid ? (int)e64 : 0;
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

hipError_t run_moe_align(const void* ids, int ids_are_i64, int numel, int E, int block_size, int* sorted_ids, int cap,
                         int* expert_ids, int nblk, int* num_post_pad, int* cumsum, int* max_cnt, hipStream_t s) {
    if (E < 1 || E > kAlignMaxExperts) return hipErrorInvalidConfiguration;
    const size_t lds = (size_t)(kAlignWaves * E + E + 1 + 1024) * sizeof(int);
    if (ids_are_i64)
        hipLaunchKernelGGL(moe_align_kernel<long long>, dim3(1), dim3(64 * kAlignWaves), lds, s, (const long long*)ids, numel, E,
                           block_size, sorted_ids, cap, expert_ids, nblk, num_post_pad, cumsum, max_cnt);
    else
        hipLaunchKernelGGL(moe_align_kernel<int>, dim3(1), dim3(64 * kAlignWaves), lds, s, (const int*)ids, numel, E, block_size,
                           sorted_ids, cap, expert_ids, nblk, num_post_pad, cumsum, max_cnt);
    return hipGetLastError();
}

}  // namespace tg
