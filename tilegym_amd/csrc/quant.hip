// Per-token 1 x 128 FP8 (e4m3fn) activation quantizer: the producer of the (M, K/128) scale
// layout the block-scaled GEMMs consume.
//   amax over each group of 128 consecutive elements of a row
//   scale = amax / 448                      (all-zero group -> 1.0)        unsloth rule
//           max(amax, eps) / 448                                           flashinfer rule
//   q     = rne_e4m3(clamp(x / scale, -448, 448))
// Arithmetic of src/tilegym/suites/unsloth/cutile/fp8.py:92-120 and
// src/tilegym/suites/flashinfer/cutile/per_token_group_quant_8bit.py:22-66; both divisions are
// IEEE divisions (a reciprocal multiply moves values across rounding boundaries).
//
// HBM-bound: 16 lanes own one group (8 elements = one 16-byte load of bf16/f16 per lane, two for
// fp32), the maximum is reduced over the 16 lanes with cross-lane shuffles, every lane writes 8
// bytes of codes and lane 0 of the group the scale.
#include "tg_host.h"

typedef float v8f_q __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8_q __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8_q __attribute__((ext_vector_type(8)));

namespace tg {

template <typename T>
__device__ __forceinline__ v8f_q load8(const T* p);
template <>
__device__ __forceinline__ v8f_q load8<__bf16>(const __bf16* p) {
    return __builtin_convertvector(*reinterpret_cast<const bf16x8_q*>(p), v8f_q);
}
template <>
__device__ __forceinline__ v8f_q load8<_Float16>(const _Float16* p) {
    return __builtin_convertvector(*reinterpret_cast<const f16x8_q*>(p), v8f_q);
}
template <>
__device__ __forceinline__ v8f_q load8<float>(const float* p) {
    const v4f lo = reinterpret_cast<const v4f*>(p)[0], hi = reinterpret_cast<const v4f*>(p)[1];
    return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
}

template <typename T>
__global__ void __launch_bounds__(256) act_quant_1x128_kernel(const T* __restrict__ x, uint8_t* __restrict__ q,
                                                             float* __restrict__ scales, int64_t groups, float eps,
                                                             int flashinfer_rule) {
    const int64_t g = (int64_t)blockIdx.x * 16 + (threadIdx.x >> 4);
    if (g >= groups) return;  // whole 16-lane groups leave together: the shuffles below stay inside a group
    const int sub = threadIdx.x & 15;
    const int64_t base = g * 128 + sub * 8;
    const v8f_q v = load8<T>(x + base);
    float amax = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) amax = fmaxf(amax, fabsf(v[i]));
#pragma unroll
    for (int d = 1; d < 16; d <<= 1) amax = fmaxf(amax, __shfl_xor(amax, d));
    float s;
    if (flashinfer_rule) s = fmaxf(amax, eps) / 448.0f;
    else s = amax == 0.f ? 1.0f : amax / 448.0f;
    int packed[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        float c[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) c[i] = fminf(fmaxf(v[4 * h + i] / s, -448.0f), 448.0f);
        int w = 0;
        w = __builtin_amdgcn_cvt_pk_fp8_f32(c[0], c[1], w, false);
        w = __builtin_amdgcn_cvt_pk_fp8_f32(c[2], c[3], w, true);
        packed[h] = w;
    }
    *reinterpret_cast<v2i*>(q + base) = v2i{packed[0], packed[1]};
    if (sub == 0) scales[g] = s;
}

hipError_t run_act_quant_1x128(const void* x, int x_type, uint8_t* q, float* scales, int64_t groups, float eps,
                               int flashinfer_rule, hipStream_t s) {
    if (groups <= 0) return hipSuccess;
    const dim3 grid((unsigned)((groups + 15) / 16)), block(256);
    if (x_type == OUT_BF16)
        hipLaunchKernelGGL(act_quant_1x128_kernel<__bf16>, grid, block, 0, s, (const __bf16*)x, q, scales, groups, eps, flashinfer_rule);
    else if (x_type == OUT_F16)
        hipLaunchKernelGGL(act_quant_1x128_kernel<_Float16>, grid, block, 0, s, (const _Float16*)x, q, scales, groups, eps, flashinfer_rule);
    else if (x_type == OUT_F32)
        hipLaunchKernelGGL(act_quant_1x128_kernel<float>, grid, block, 0, s, (const float*)x, q, scales, groups, eps, flashinfer_rule);
    else
        return hipErrorInvalidValue;
    return hipGetLastError();
}

}  // namespace tg
