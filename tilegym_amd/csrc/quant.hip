// Elementwise producers and consumers around the FP8 GEMMs: the per-token group quantizer, the block
// dequantizer of a weight, the SiLU-and-multiply + requantization between the two MoE GEMMs, and the
// top-k combine.
//
// Per-token group FP8 (e4m3fn) activation quantizer (groups of 16, 32, 64 or 128 consecutive elements
// of a row; 128 gives the (M, K/128) scale layout the block-scaled GEMMs consume):
//   amax over the group
//   scale = amax / 448                      (all-zero group -> 1.0)        rule 0, unsloth
//           max(amax, eps) / 448                                           rule 1, flashinfer
//           2^ceil(log2(max(that, 1e-10)))                                 rule 2, flashinfer with power-of-two scales
//   q     = rne_e4m3(clamp(x / scale, -448, 448))
// Arithmetic of src/tilegym/suites/unsloth/cutile/fp8.py:92-120, of the column-major kernel of
// src/tilegym/suites/flashinfer/cutile/per_token_group_quant_8bit.py:78-145 and of the reference's
// test oracle for that operator (x / scale); both divisions are correctly rounded (IEEE) divisions.
// The reference's row-major kernel (per_token_group_quant_8bit.py:57-63) multiplies by 1.0 / scale
// instead, which can land one e4m3 code away at rounding boundaries: rule 1 with row-major scales
// follows the test oracle's x / scale here, not that kernel's reciprocal form.
// The scale of group j of row r is written to scales[r * row_stride + j * col_stride], which covers the
// row-major layout and the column-major ones of per_token_group_quant_8bit.py:185-204.
//
// HBM-bound: group_size / 8 lanes own one group at a time (8 elements = one 16-byte load of bf16/f16 per
// lane, two for fp32) and four groups in all, whose loads are issued together; the maximum is reduced over
// those lanes with cross-lane shuffles, every lane writes 8 bytes of codes and the first lane of the group
// the scale.  The divisions go through ScaleDivider (bit-equal to the IEEE division).
#include "quant_device.h"

namespace tg {

template <typename T, int LPG, bool STRIDED, bool I8>
__global__ void __launch_bounds__(256) act_quant_group_kernel(const T* __restrict__ x, uint8_t* __restrict__ q,
                                                             float* __restrict__ scales, int64_t groups, float eps,
                                                             int rule, uint32_t groups_per_row, int64_t s_row, int64_t s_col) {
    act_quant_group_body<T, LPG, STRIDED, I8>(x, q, scales, groups, eps, rule, groups_per_row, s_row, s_col, (int64_t)blockIdx.x,
                                              (int)threadIdx.x);
}

// y = float(x) * s[i / bs][j / bs] for an (M, N) e4m3 weight with one fp32 scale per bs x bs block
// (src/tilegym/suites/unsloth/cutile/fp8.py:36-71,348-367): fp32 product, rounded once to the output
// type.  HBM-bound (1 byte in, 2 or 4 out per element).  VEC: a lane converts 16 consecutive
// elements of one row (N % 16 == 0, bs % 16 == 0, 16-byte aligned rows); otherwise one element.
template <typename OT, bool VEC>
__global__ void __launch_bounds__(256) weight_dequant_kernel(const uint8_t* __restrict__ x, const float* __restrict__ s,
                                                            OT* __restrict__ y, int64_t M, int64_t N, int bs, int64_t s_cols) {
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if constexpr (VEC) {
        const int64_t chunks = N / 16;
        if (idx >= M * chunks) return;
        const int64_t row = idx / chunks, col = (idx - row * chunks) * 16;
        const float scale = s[(row / bs) * s_cols + col / bs];
        const v4i raw = *reinterpret_cast<const v4i*>(x + row * N + col);
        typedef OT vecT __attribute__((ext_vector_type(8)));
        typedef float v2f_q __attribute__((ext_vector_type(2)));
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            v8f_q f;
#pragma unroll
            for (int w = 0; w < 2; ++w) {
                const v2f_q lo = __builtin_amdgcn_cvt_pk_f32_fp8(raw[2 * h + w], false);
                const v2f_q hi = __builtin_amdgcn_cvt_pk_f32_fp8(raw[2 * h + w], true);
                f[4 * w] = lo[0] * scale, f[4 * w + 1] = lo[1] * scale, f[4 * w + 2] = hi[0] * scale, f[4 * w + 3] = hi[1] * scale;
            }
            // the fp32 products are rounded on their own before the conversion (no single-rounding mixed-precision FMA)
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                float t = f[i];
                asm("" : "+v"(t));
                f[i] = t;
            }
            *reinterpret_cast<vecT*>(y + row * N + col + 8 * h) = __builtin_convertvector(f, vecT);
        }
    } else {
        if (idx >= M * N) return;
        const int64_t row = idx / N, col = idx - row * N;
        float t = e4m3_to_f32(x[idx]) * s[(row / bs) * s_cols + col / bs];
        asm("" : "+v"(t));
        y[idx] = (OT)t;
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

template <typename T, int LPG>
static void launch_act_quant(const T* x, uint8_t* q, bool i8, float* scales, int64_t groups, float eps, int rule, bool strided,
                             uint32_t groups_per_row, int64_t s_row, int64_t s_col, hipStream_t s) {
    constexpr int per_wg = (256 / LPG) * kQuantGroupsPerLane;
    const dim3 grid((unsigned)((groups + per_wg - 1) / per_wg)), block(256);
    if (strided && i8)
        hipLaunchKernelGGL((act_quant_group_kernel<T, LPG, true, true>), grid, block, 0, s, x, q, scales, groups, eps, rule, groups_per_row, s_row, s_col);
    else if (strided)
        hipLaunchKernelGGL((act_quant_group_kernel<T, LPG, true, false>), grid, block, 0, s, x, q, scales, groups, eps, rule, groups_per_row, s_row, s_col);
    else if (i8)
        hipLaunchKernelGGL((act_quant_group_kernel<T, LPG, false, true>), grid, block, 0, s, x, q, scales, groups, eps, rule, groups_per_row, s_row, s_col);
    else
        hipLaunchKernelGGL((act_quant_group_kernel<T, LPG, false, false>), grid, block, 0, s, x, q, scales, groups, eps, rule, groups_per_row, s_row, s_col);
}

template <typename T>
static hipError_t dispatch_act_quant(const T* x, uint8_t* q, bool i8, float* scales, int64_t groups, int group_size, float eps, int rule,
                                     bool strided, uint32_t groups_per_row, int64_t s_row, int64_t s_col, hipStream_t s) {
    switch (group_size) {
        case 128: launch_act_quant<T, 16>(x, q, i8, scales, groups, eps, rule, strided, groups_per_row, s_row, s_col, s); break;
        case 64: launch_act_quant<T, 8>(x, q, i8, scales, groups, eps, rule, strided, groups_per_row, s_row, s_col, s); break;
        case 32: launch_act_quant<T, 4>(x, q, i8, scales, groups, eps, rule, strided, groups_per_row, s_row, s_col, s); break;
        case 16: launch_act_quant<T, 2>(x, q, i8, scales, groups, eps, rule, strided, groups_per_row, s_row, s_col, s); break;
        default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

// groups of group_size (16, 32, 64, 128) elements; with `strided` the scale of group j of row r (groups_per_row
// groups in a row) is written to scales[r * s_row + j * s_col], otherwise to scales[r * groups_per_row + j]
hipError_t run_act_quant_group(const void* x, int x_type, uint8_t* q, bool q_is_int8, float* scales, int64_t groups, int group_size, float eps,
                               int rule, bool strided, int64_t groups_per_row, int64_t s_row, int64_t s_col, hipStream_t s) {
    if (groups <= 0) return hipSuccess;
    if (strided && (groups > INT32_MAX || groups_per_row <= 0)) return hipErrorInvalidValue;
    const uint32_t gpr = (uint32_t)groups_per_row;
    if (x_type == OUT_BF16) return dispatch_act_quant((const __bf16*)x, q, q_is_int8, scales, groups, group_size, eps, rule, strided, gpr, s_row, s_col, s);
    if (x_type == OUT_F16) return dispatch_act_quant((const _Float16*)x, q, q_is_int8, scales, groups, group_size, eps, rule, strided, gpr, s_row, s_col, s);
    if (x_type == OUT_F32) return dispatch_act_quant((const float*)x, q, q_is_int8, scales, groups, group_size, eps, rule, strided, gpr, s_row, s_col, s);
    return hipErrorInvalidValue;
}

template <typename OT>
static hipError_t launch_weight_dequant(const uint8_t* x, const float* sc, OT* y, int64_t M, int64_t N, int bs, int64_t s_cols,
                                        bool vec, hipStream_t s) {
    const int64_t work = vec ? M * (N / 16) : M * N;
    const dim3 grid((unsigned)((work + 255) / 256)), block(256);
    if (vec) hipLaunchKernelGGL((weight_dequant_kernel<OT, true>), grid, block, 0, s, x, sc, y, M, N, bs, s_cols);
    else hipLaunchKernelGGL((weight_dequant_kernel<OT, false>), grid, block, 0, s, x, sc, y, M, N, bs, s_cols);
    return hipGetLastError();
}

hipError_t run_weight_dequant(const uint8_t* x, const float* sc, void* y, int y_type, int64_t M, int64_t N, int bs, int64_t s_cols,
                              bool vec, hipStream_t s) {
    if (M <= 0 || N <= 0) return hipSuccess;
    if (y_type == OUT_BF16) return launch_weight_dequant(x, sc, (__bf16*)y, M, N, bs, s_cols, vec, s);
    if (y_type == OUT_F16) return launch_weight_dequant(x, sc, (_Float16*)y, M, N, bs, s_cols, vec, s);
    if (y_type == OUT_F32) return launch_weight_dequant(x, sc, (float*)y, M, N, bs, s_cols, vec, s);
    return hipErrorInvalidValue;
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
