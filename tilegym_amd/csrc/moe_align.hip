// moe_align_block_size on the device, one launch: groups the (token, slot) pairs of a top-k
// routing by expert, pads every expert's group to a multiple of block_size and emits the
// block -> expert table the gather GEMM walks.  Output contract of
// src/tilegym/ops/cutile/moe_align_block.py:205-268 (torch statement: src/tilegym/ops/moe_interface.py:30-79):
//   sorted_ids[cap]   flat pair indices grouped by expert, ascending inside an expert (stable),
//                     every other position = numel (the sentinel), cap = numel + E * (block_size - 1)
//   expert_ids[nblk]  expert of each block of block_size positions (0 past the padded total)
//   num_post_pad[1]   padded total;  cumsum[E + 1] padded prefix;  max_cnt[1] largest expert count
//
// One launch of G <= 32 workgroups of 16 waves, no communication between them.  Workgroup g owns
// the contiguous slice g of the flat id sequence, wave w of it the sub-slice w of that slice.
//   pass 1: every workgroup histograms the WHOLE sequence (it comes from L2 after the first
//           reader) into LDS counters, split three ways per expert: ids before its slice, ids
//           after it, and one counter row per owning wave for the ids inside it (LDS atomics;
//           order-free).  Every workgroup thus knows all group sizes and where its own ids start
//           inside each group, without waiting for any other workgroup.
//   scan  : thread e turns the rows of expert e into each wave's start inside the expert's group;
//           the padded group sizes are prefix-summed over the experts (shuffle scan)
//   fill  : sentinels and the block -> expert table, spread over all waves of the grid
//   pass 2: every wave walks its sub-slice 64 ids at a time; lanes with equal experts are ranked by
//           lane order with ballots, so the result does not depend on any atomic's timing.  The
//           scattered 4-byte stores of this pass are what a single workgroup would spend most of
//           its time on (one compute unit issues one such request per clock): hence the grid.
#include "moe_align_device.h"

namespace tg {

template <typename IdT>
__global__ void __launch_bounds__(64 * kAlignWaves) moe_align_kernel(const IdT* __restrict__ ids, int numel, int E,
                                                                    int block_size, int* __restrict__ sorted_ids, int cap,
                                                                    int* __restrict__ expert_ids, int nblk,
                                                                    int* __restrict__ num_post_pad, int* __restrict__ cumsum,
                                                                    int* __restrict__ max_cnt) {
    extern __shared__ int lds[];
    moe_align_body<IdT>(ids, numel, E, block_size, sorted_ids, cap, expert_ids, nblk, num_post_pad, cumsum, max_cnt, lds,
                        (int)gridDim.x, (int)blockIdx.x);
}

hipError_t run_moe_align(const void* ids, int ids_are_i64, int numel, int E, int block_size, int* sorted_ids, int cap,
                         int* expert_ids, int nblk, int* num_post_pad, int* cumsum, int* max_cnt, hipStream_t s) {
    if (E < 1 || E > kAlignMaxExperts) return hipErrorInvalidConfiguration;
    const size_t lds = moe_align_lds_bytes(E);
    const int grid = moe_align_grid(numel);
    if (ids_are_i64)
        hipLaunchKernelGGL(moe_align_kernel<long long>, dim3(grid), dim3(64 * kAlignWaves), lds, s, (const long long*)ids, numel, E,
                           block_size, sorted_ids, cap, expert_ids, nblk, num_post_pad, cumsum, max_cnt);
    else
        hipLaunchKernelGGL(moe_align_kernel<int>, dim3(grid), dim3(64 * kAlignWaves), lds, s, (const int*)ids, numel, E, block_size,
                           sorted_ids, cap, expert_ids, nblk, num_post_pad, cumsum, max_cnt);
    return hipGetLastError();
}

}  // namespace tg
