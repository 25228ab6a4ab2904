// The two launches in front of the first MoE GEMM as one: moe_align_block_size over the routing ids
// (src/tilegym/ops/moe_interface.py:246-248) and the 1 x 128 activation quantizer over the hidden states that the FP8
// GEMM needs.  They share no data -- one reads the top-k ids, the other the activations -- and both are short,
// latency-bound launches (about 10 us each at 4096 tokens), so they run side by side in one grid: the first
// workgroups do the alignment (its own algorithm, untouched: moe_align_device.h), the others quantize, four
// 256-thread quantizer blocks per 1024-thread workgroup (quant_device.h).  Outputs are bit-identical to the
// two stand-alone kernels.
#include "moe_align_device.h"
#include "quant_device.h"

namespace tg {

template <typename IdT, typename T>
__global__ void __launch_bounds__(64 * kAlignWaves) moe_prepare_kernel(const IdT* __restrict__ ids, int numel, int E, int block_size,
                                                                      int* __restrict__ sorted_ids, int cap,
                                                                      int* __restrict__ expert_ids, int nblk,
                                                                      int* __restrict__ num_post_pad, int* __restrict__ cumsum,
                                                                      int* __restrict__ max_cnt, int align_wgs,
                                                                      const T* __restrict__ x, uint8_t* __restrict__ q,
                                                                      float* __restrict__ scales, int64_t groups) {
    extern __shared__ int lds[];
    if ((int)blockIdx.x < align_wgs) {  // (uniform over the workgroup: the barriers inside are met by all its waves)
        moe_align_body<IdT>(ids, numel, E, block_size, sorted_ids, cap, expert_ids, nblk, num_post_pad, cumsum, max_cnt, lds,
                            align_wgs, (int)blockIdx.x);
    } else {
        const int64_t block = ((int64_t)blockIdx.x - align_wgs) * (kAlignWaves / 4) + (threadIdx.x >> 8);
        act_quant_group_body<T, 16, false, false>(x, q, scales, groups, 0.0f, QUANT_ZERO_TO_ONE, 1u, 0, 0, block, (int)(threadIdx.x & 255));
    }
}

// ids: (numel) int32 or int64 top-k expert ids; x: (groups * 128) bf16 (x_is_bf16) or f16 activations, q / scales their
// e4m3 codes and one fp32 scale per 128 elements (all-zero group -> 1: the rule of unsloth's act_quant).
hipError_t run_moe_align_quant(const void* ids, int ids_are_i64, int numel, int E, int block_size, int* sorted_ids, int cap,
                               int* expert_ids, int nblk, int* num_post_pad, int* cumsum, int* max_cnt, const void* x,
                               int x_is_bf16, uint8_t* q, float* scales, int64_t groups, hipStream_t s) {
    if (E < 1 || E > kAlignMaxExperts) return hipErrorInvalidConfiguration;
    const size_t lds = moe_align_lds_bytes(E);
    const int align_wgs = moe_align_grid(numel);
    constexpr int per_wg = (kAlignWaves / 4) * (256 / 16) * kQuantGroupsPerLane;   // groups of 128 per 1024-thread workgroup
    const int64_t quant_wgs = (groups + per_wg - 1) / per_wg;
    if (quant_wgs + align_wgs > INT32_MAX) return hipErrorInvalidValue;
    const dim3 grid((unsigned)(align_wgs + quant_wgs)), block(64 * kAlignWaves);
#define TG_LAUNCH_PREPARE(IDT, XT)                                                                                             \
    hipLaunchKernelGGL((moe_prepare_kernel<IDT, XT>), grid, block, lds, s, (const IDT*)ids, numel, E, block_size, sorted_ids,  \
                       cap, expert_ids, nblk, num_post_pad, cumsum, max_cnt, align_wgs, (const XT*)x, q, scales, groups)
    if (ids_are_i64 && x_is_bf16) TG_LAUNCH_PREPARE(long long, __bf16);
    else if (ids_are_i64) TG_LAUNCH_PREPARE(long long, _Float16);
    else if (x_is_bf16) TG_LAUNCH_PREPARE(int, __bf16);
    else TG_LAUNCH_PREPARE(int, _Float16);
#undef TG_LAUNCH_PREPARE
    return hipGetLastError();
}

}  // namespace tg
