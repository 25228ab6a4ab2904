// Elementwise producers around the FP8 GEMMs: the per-token 1 x 128 activation quantizer, the
// SiLU-and-multiply + requantization between the two MoE GEMMs, and the top-k combine.
//
// Per-token 1 x 128 FP8 (e4m3fn) activation quantizer: the producer of the (M, K/128) scale
// layout the block-scaled GEMMs consume.
//   amax over each group of 128 consecutive elements of a row
//   scale = amax / 448                      (all-zero group -> 1.0)        unsloth rule
//           max(amax, eps) / 448                                           flashinfer rule
//   q     = rne_e4m3(clamp(x / scale, -448, 448))
// Arithmetic of src/tilegym/suites/unsloth/cutile/fp8.py:92-120 and
// src/tilegym/suites/flashinfer/cutile/per_token_group_quant_8bit.py:22-66; both divisions are
// correctly rounded (IEEE) divisions (a plain reciprocal multiply moves values across rounding boundaries).
//
// HBM-bound: 16 lanes own one group at a time (8 elements = one 16-byte load of bf16/f16 per lane,
// two for fp32) and four groups in all, whose loads are issued together; the maximum is reduced over
// the 16 lanes with cross-lane shuffles, every lane writes 8 bytes of codes and lane 0 of the group
// the scale.  The divisions go through ScaleDivider (bit-equal to the IEEE division).
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

// kGroupsPerLane groups per 16 lanes, all loads issued before the first use (one 16-byte load per lane
// leaves too few bytes in flight per wave for an HBM-bound kernel).
constexpr int kQuantGroupsPerLane = 4;

template <typename T>
__global__ void __launch_bounds__(256) act_quant_1x128_kernel(const T* __restrict__ x, uint8_t* __restrict__ q,
                                                             float* __restrict__ scales, int64_t groups, float eps,
                                                             int flashinfer_rule) {
    constexpr int G = kQuantGroupsPerLane;
    const int sub = threadIdx.x & 15;
    const int64_t g0 = (int64_t)blockIdx.x * (16 * G) + (threadIdx.x >> 4);
    v8f_q v[G];
#pragma unroll
    for (int j = 0; j < G; ++j) {
        const int64_t g = g0 + j * 16;
        // whole 16-lane groups are in or out together: the shuffles below stay inside a group
        if (g < groups) v[j] = load8<T>(x + g * 128 + sub * 8);
        else {
#pragma unroll
            for (int i = 0; i < 8; ++i) v[j][i] = 0.f;
        }
    }
#pragma unroll
    for (int j = 0; j < G; ++j) {
        const int64_t g = g0 + j * 16;
        float amax = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) amax = fmaxf(amax, fabsf(v[j][i]));
#pragma unroll
        for (int d = 1; d < 16; d <<= 1) amax = fmaxf(amax, __shfl_xor(amax, d));
        float s;
        if (flashinfer_rule) s = fmaxf(amax, eps) / 448.0f;
        else s = amax == 0.f ? 1.0f : amax / 448.0f;
        if (g >= groups) continue;
        const ScaleDivider div(s);
        float c[8];
        if (div.fast) {
#pragma unroll
            for (int i = 0; i < 8; ++i) c[i] = div.quotient(v[j][i]);
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i) c[i] = v[j][i] / s;
        }
        int packed[2];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            int w = 0;
            w = __builtin_amdgcn_cvt_pk_fp8_f32(fminf(fmaxf(c[4 * h], -448.0f), 448.0f), fminf(fmaxf(c[4 * h + 1], -448.0f), 448.0f), w, false);
            w = __builtin_amdgcn_cvt_pk_fp8_f32(fminf(fmaxf(c[4 * h + 2], -448.0f), 448.0f), fminf(fmaxf(c[4 * h + 3], -448.0f), 448.0f), w, true);
            packed[h] = w;
        }
        *reinterpret_cast<v2i*>(q + g * 128 + sub * 8) = v2i{packed[0], packed[1]};
        if (sub == 0) scales[g] = s;
    }
}

// Between the two MoE GEMMs: act = silu(gate) * up of a (R, 2*I) bf16/f16 GEMM output (gate =
// first I columns, src/tilegym/ops/ops.py:172-193), rounded to the input's 16-bit type as the
// reference's intermediate cache is (src/tilegym/ops/moe_interface.py:206-210,272-277), then
// quantized 1 x 128 with the all-zero -> 1.0 rule: the second GEMM gets a real per-group
// activation scale instead of the reference's all-ones one.  I % 8 == 0; the last group of a row
// may be partial.
template <typename T>
__global__ void __launch_bounds__(256) silu_mul_quant_kernel(const T* __restrict__ x, uint8_t* __restrict__ q,
                                                            float* __restrict__ scales, int64_t rows, int I, int groups_per_row) {
    const int64_t g = (int64_t)blockIdx.x * 16 + (threadIdx.x >> 4);
    if (g >= rows * groups_per_row) return;
    const int sub = threadIdx.x & 15;
    const int64_t row = g / groups_per_row;
    const int col = (int)(g % groups_per_row) * 128 + sub * 8;
    const bool live = col < I;  // I % 8 == 0: a lane's eight elements are all inside or all outside
    v8f_q act;
#pragma unroll
    for (int i = 0; i < 8; ++i) act[i] = 0.f;
    if (live) {
        const v8f_q gate = load8<T>(x + row * (2 * (int64_t)I) + col);
        const v8f_q up = load8<T>(x + row * (2 * (int64_t)I) + I + col);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            act[i] = silu_mul_round<T>(gate[i], up[i]);  // the quantization below keeps its IEEE divisions
        }
    }
    float amax = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) amax = fmaxf(amax, fabsf(act[i]));
#pragma unroll
    for (int d = 1; d < 16; d <<= 1) amax = fmaxf(amax, __shfl_xor(amax, d));
    const float s = amax == 0.f ? 1.0f : amax / 448.0f;
    if (live) {
        int packed[2];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            float c[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) c[i] = fminf(fmaxf(act[4 * h + i] / s, -448.0f), 448.0f);
            int w = 0;
            w = __builtin_amdgcn_cvt_pk_fp8_f32(c[0], c[1], w, false);
            w = __builtin_amdgcn_cvt_pk_fp8_f32(c[2], c[3], w, true);
            packed[h] = w;
        }
        *reinterpret_cast<v2i*>(q + row * (int64_t)I + col) = v2i{packed[0], packed[1]};
    }
    if (sub == 0) scales[g] = s;
}

// out[t, :] = sum_j x[t, j, :]  (fp32 sum in slot order, rounded once), the top-k combine of
// src/tilegym/ops/moe_interface.py:308-321.  H % 8 == 0.
template <typename T>
__global__ void __launch_bounds__(256) moe_sum_kernel(const T* __restrict__ x, T* __restrict__ out, int64_t tokens, int top_k, int H) {
    typedef T vecT __attribute__((ext_vector_type(8)));
    const int64_t idx = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 8;
    if (idx >= tokens * H) return;
    const int64_t t = idx / H;
    const int h = (int)(idx % H);
    v8f_q acc = load8<T>(x + (t * top_k) * (int64_t)H + h);
    for (int j = 1; j < top_k; ++j) acc += load8<T>(x + (t * top_k + j) * (int64_t)H + h);
    *reinterpret_cast<vecT*>(out + idx) = __builtin_convertvector(acc, vecT);
}

hipError_t run_act_quant_1x128(const void* x, int x_type, uint8_t* q, float* scales, int64_t groups, float eps,
                               int flashinfer_rule, hipStream_t s) {
    if (groups <= 0) return hipSuccess;
    constexpr int per_wg = 16 * kQuantGroupsPerLane;
    const dim3 grid((unsigned)((groups + per_wg - 1) / per_wg)), block(256);
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

hipError_t run_silu_mul_quant(const void* x, int x_type, uint8_t* q, float* scales, int64_t rows, int I, hipStream_t s) {
    const int gpr = (I + 127) / 128;
    const int64_t groups = rows * gpr;
    if (groups <= 0) return hipSuccess;
    const dim3 grid((unsigned)((groups + 15) / 16)), block(256);
    if (x_type == OUT_BF16)
        hipLaunchKernelGGL(silu_mul_quant_kernel<__bf16>, grid, block, 0, s, (const __bf16*)x, q, scales, rows, I, gpr);
    else if (x_type == OUT_F16)
        hipLaunchKernelGGL(silu_mul_quant_kernel<_Float16>, grid, block, 0, s, (const _Float16*)x, q, scales, rows, I, gpr);
    else
        return hipErrorInvalidValue;
    return hipGetLastError();
}

hipError_t run_moe_sum(const void* x, void* out, int x_type, int64_t tokens, int top_k, int H, hipStream_t s) {
    const int64_t n = tokens * H / 8;
    if (n <= 0) return hipSuccess;
    const dim3 grid((unsigned)((n + 255) / 256)), block(256);
    if (x_type == OUT_BF16)
        hipLaunchKernelGGL(moe_sum_kernel<__bf16>, grid, block, 0, s, (const __bf16*)x, (__bf16*)out, tokens, top_k, H);
    else if (x_type == OUT_F16)
        hipLaunchKernelGGL(moe_sum_kernel<_Float16>, grid, block, 0, s, (const _Float16*)x, (_Float16*)out, tokens, top_k, H);
    else
        return hipErrorInvalidValue;
    return hipGetLastError();
}

}  // namespace tg
