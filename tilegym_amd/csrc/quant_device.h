// Device side of the per-token group quantizer (see quant.hip): shared by the stand-alone kernel and by the kernel that
// runs it beside moe_align_block_size (moe_prepare.hip).
#pragma once
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

// kQuantGroupsPerLane groups per lane, all loads issued before the first use (one 16-byte load per lane
// leaves too few bytes in flight per wave for an HBM-bound kernel).
constexpr int kQuantGroupsPerLane = 4;

enum QuantRule { QUANT_ZERO_TO_ONE = 0, QUANT_EPS = 1, QUANT_EPS_POW2 = 2 };

// LPG lanes per group (group size 8 * LPG).  STRIDED: the scale of group j of row r goes to
// scales[r * s_row + j * s_col] (groups < 2^31); otherwise to scales[g].
// I8: the destination is int8 instead of e4m3 (per_token_group_quant_8bit with dst_dtype=torch.int8,
// tests/suites/flashinfer/test_per_token_group_quant_8bit.py:41-68): scale = amax / 127, q = the quotient clamped to
// [-128, 127] and converted as a float -> integer cast does (toward zero).
// (body of 256-thread block `block`, thread `tid` of it: the kernel below runs it as such, the MoE preparation kernel
// runs four such blocks per 1024-thread workgroup)
template <typename T, int LPG, bool STRIDED, bool I8>
__device__ __forceinline__ void act_quant_group_body(const T* __restrict__ x, uint8_t* __restrict__ q,
                                                     float* __restrict__ scales, int64_t groups, float eps,
                                                     int rule, uint32_t groups_per_row, int64_t s_row, int64_t s_col,
                                                     const int64_t block, const int tid) {
    constexpr int G = kQuantGroupsPerLane, GS = 8 * LPG, PASS = 256 / LPG;
    constexpr float QMAX = I8 ? 127.0f : 448.0f, QMIN = I8 ? -128.0f : -448.0f;
    const int sub = tid & (LPG - 1);
    const int64_t g0 = block * (PASS * G) + (tid / LPG);
    v8f_q v[G];
#pragma unroll
    for (int j = 0; j < G; ++j) {
        const int64_t g = g0 + j * PASS;
        // the LPG lanes of a group are in or out together: the shuffles below stay inside a group
        if (g < groups) v[j] = load8<T>(x + g * GS + sub * 8);
        else {
#pragma unroll
            for (int i = 0; i < 8; ++i) v[j][i] = 0.f;
        }
    }
#pragma unroll
    for (int j = 0; j < G; ++j) {
        const int64_t g = g0 + j * PASS;
        float amax = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) amax = fmaxf(amax, fabsf(v[j][i]));
#pragma unroll
        for (int d = 1; d < LPG; d <<= 1) amax = fmaxf(amax, __shfl_xor(amax, d));
        float s;
        if (rule == QUANT_ZERO_TO_ONE) s = amax == 0.f ? 1.0f : amax / QMAX;
        else s = fmaxf(amax, eps) / QMAX;
        if (rule == QUANT_EPS_POW2) s = exp2f(ceilf(log2f(fmaxf(fabsf(s), 1e-10f))));
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
            float cc[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) cc[i] = fminf(fmaxf(c[4 * h + i], QMIN), QMAX);
            int w = 0;
            if constexpr (I8) {
#pragma unroll
                for (int i = 0; i < 4; ++i) w |= ((int)cc[i] & 0xFF) << (8 * i);
            } else {
                w = __builtin_amdgcn_cvt_pk_fp8_f32(cc[0], cc[1], w, false);
                w = __builtin_amdgcn_cvt_pk_fp8_f32(cc[2], cc[3], w, true);
            }
            packed[h] = w;
        }
        *reinterpret_cast<v2i*>(q + g * GS + sub * 8) = v2i{packed[0], packed[1]};
        if (sub == 0) {
            if constexpr (STRIDED) {
                const uint32_t row = (uint32_t)g / groups_per_row, col = (uint32_t)g - row * groups_per_row;
                scales[row * s_row + col * s_col] = s;
            } else {
                scales[g] = s;
            }
        }
    }
}

}  // namespace tg
