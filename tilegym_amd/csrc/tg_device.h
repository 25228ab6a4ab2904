// Device-side building blocks shared by the FP8 GEMM kernels (gfx950 / CDNA4 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));

namespace tg {

constexpr int kKBlock = 128;    // bytes of K consumed by one 16x16x128 MFMA = the quant block

enum OutType { OUT_F32 = 0, OUT_F16 = 1, OUT_BF16 = 2, OUT_F8 = 7 };  // same numbering as the ABI dtype codes (7: e4m3fn)

// How rows of the activation operand are found.
// GROUP_GATHER_ACT: the gather form for a (E, 2I, K) gate/up weight whose epilogue produces
// act = silu(gate) * up, quantized 1 x 128 to e4m3, instead of the GEMM output.
enum GroupMode { GROUP_DENSE = 0, GROUP_RAGGED = 1, GROUP_GATHER = 2, GROUP_GATHER_ACT = 3 };

struct GemmParams {
    const uint8_t* A;   // activations, (M,K) row-major, e4m3
    const uint8_t* B;   // weights, (N,K) row-major (or (E,N,K)), e4m3
    void* C;            // (M,N) row-major
    const float* As;    // per-tensor: 1 float or null.  block: (M, kblocks)
    const float* Bs;    // per-tensor: 1 float or null.  block: ([E,] nblocks, kblocks)
    int M, N, K;
    int ldc;               // row stride of C in elements (N, or the full width when the columns are computed in chunks)
    int kblocks, nblocks;  // ceil(K/128), ceil(N/128)
    float alpha, beta;
    int out_type;
    int vec_store;      // 1 when N % 4 == 0 and C is 16-byte aligned: 4-wide stores allowed
    // split-K: grid.y partitions of the K steps; each writes raw fp32 sums to partials[z][M][N]
    // and a separate reduction kernel adds them in z order and applies the epilogue
    int split_k;        // >= 1
    int ksteps_per_split;
    float* partials;
    // grouped forms
    const int* m_indptr;   // ragged: (E+1)
    int E;
    const int* sorted_ids; // gather: (EM)
    const int* expert_ids; // gather: (EM / block_m)
    const int* num_post_pad;  // gather: (1)
    const float* row_weight;  // gather: (num_valid) or null
    int top_k, num_valid, block_m, em_capacity;
    // GROUP_GATHER_ACT: I (gate rows are B[e][0:I], up rows B[e][I:2I]); C is then the (num_valid, I)
    // e4m3 activation and act_scales its (num_valid, I/128) fp32 scales; act_is_bf16 says which
    // 16-bit type the GEMM output and the activation are rounded to on the way
    int inter;
    float* act_scales;
    int act_is_bf16;
    // wide streaming form: weight rows per wave (1 .. 16; 0 means 16).  Fewer than 16 make more, smaller workgroups
    int wave_rows;
    // deep 64 x 128 tile kernel: weight rows a tile covers (a multiple of 8, 72 .. 128; 0 means 128).  Fewer make more tiles
    int tile_cols;
};

// A list of independent per-tensor-scaled NT GEMMs handed to one launch in the kernel arguments.
constexpr int kListMax = 40;
struct ListProblem {
    const uint8_t* A;
    const uint8_t* B;
    void* C;
    const float* As;
    const float* Bs;
    int M, N, K;
    int tile_end;   // exclusive prefix of BM x BN tiles over the list
    int vec_store;
    int pad;
};
struct GemmList {
    int count, out_type;
    float alpha;
    int pad;
    ListProblem prob[kListMax];
};

// One 16x16x128 e4m3 x e4m3 MFMA with fp32 accumulation.  `w` supplies the 16 rows of the
// result (lane l: row l%16, K bytes of K-group l/16), `x` supplies the 16 columns; lane l
// receives column l%16, rows 4*(l/16)..+3.  With both scale operands zero the compiler
// selects the unscaled instruction.
__device__ __forceinline__ v4f mfma_e4m3(v8i w, v8i x, v4f acc) {
    return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(w, x, acc, 0, 0, 0, 0, 0, 0);
}

__device__ __forceinline__ v8i join(v4i lo, v4i hi) {
    return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
}

// Exact software decode of one e4m3fn code (used only by the generic fallback kernel).
__device__ __forceinline__ float e4m3_to_f32(uint8_t c) {
    uint32_t s = (uint32_t)(c & 0x80) << 24;
    uint32_t e = (c >> 3) & 0xF, m = c & 7;
    if (e == 0xF && m == 7) return __uint_as_float(s | 0x7FC00000u);
    if (e == 0) {
        float v = (float)m * 0.001953125f;  // m * 2^-9
        return __uint_as_float(__float_as_uint(v) | s);
    }
    return __uint_as_float(s | ((e + 120u) << 23) | (m << 20));
}

// One fp32 value -> e4m3fn code, round to nearest even, saturating at +-448 (NaN stays NaN).
__device__ __forceinline__ float clamp_e4m3(float x) {
    const float c = fminf(fmaxf(x, -448.0f), 448.0f);
    return x == x ? c : x;
}
// Four values -> four e4m3fn codes packed in one dword (element 0 in the low byte).
__device__ __forceinline__ int pack_e4m3x4(float a, float b, float c, float d) {
    int w = 0;
    w = __builtin_amdgcn_cvt_pk_fp8_f32(clamp_e4m3(a), clamp_e4m3(b), w, false);
    w = __builtin_amdgcn_cvt_pk_fp8_f32(clamp_e4m3(c), clamp_e4m3(d), w, true);
    return w;
}
__device__ __forceinline__ uint8_t f32_to_e4m3(float x) { return (uint8_t)(pack_e4m3x4(x, 0.f, 0.f, 0.f) & 0xFF); }

// Store 4 consecutive outputs C[row][col..col+3] = v (+ beta * old), masked against N columns; ld = row stride.
__device__ __forceinline__ void store4(void* C, int out_type, int64_t row, int col, int N, int ld, v4f v,
                                       float beta, bool vec_ok) {
    int64_t base = row * (int64_t)ld + col;
    if (vec_ok && col + 3 < N) {
        if (out_type == OUT_BF16) {
            bf16x4* p = reinterpret_cast<bf16x4*>(reinterpret_cast<__bf16*>(C) + base);
            if (beta != 0.0f) {
                bf16x4 o = *p;
                v4f of = __builtin_convertvector(o, v4f);
                v = v + beta * of;
            }
            *p = __builtin_convertvector(v, bf16x4);
        } else if (out_type == OUT_F32) {
            v4f* p = reinterpret_cast<v4f*>(reinterpret_cast<float*>(C) + base);
            if (beta != 0.0f) v = v + beta * (*p);
            *p = v;
        } else if (out_type == OUT_F8) {
            uint8_t* p = reinterpret_cast<uint8_t*>(C) + base;
            if (beta != 0.0f) {
#pragma unroll
                for (int r = 0; r < 4; ++r) v[r] += beta * e4m3_to_f32(p[r]);
            }
            *reinterpret_cast<int*>(p) = pack_e4m3x4(v[0], v[1], v[2], v[3]);
        } else {
            f16x4* p = reinterpret_cast<f16x4*>(reinterpret_cast<_Float16*>(C) + base);
            if (beta != 0.0f) {
                f16x4 o = *p;
                v4f of = __builtin_convertvector(o, v4f);
                v = v + beta * of;
            }
            *p = __builtin_convertvector(v, f16x4);
        }
        return;
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        if (col + r >= N) break;
        float x = v[r];
        if (out_type == OUT_BF16) {
            __bf16* p = reinterpret_cast<__bf16*>(C) + base + r;
            if (beta != 0.0f) x += beta * (float)(*p);
            *p = (__bf16)x;
        } else if (out_type == OUT_F32) {
            float* p = reinterpret_cast<float*>(C) + base + r;
            if (beta != 0.0f) x += beta * (*p);
            *p = x;
        } else if (out_type == OUT_F8) {
            uint8_t* p = reinterpret_cast<uint8_t*>(C) + base + r;
            if (beta != 0.0f) x += beta * e4m3_to_f32(*p);
            *p = f32_to_e4m3(x);
        } else {
            _Float16* p = reinterpret_cast<_Float16*>(C) + base + r;
            if (beta != 0.0f) x += beta * (float)(*p);
            *p = (_Float16)x;
        }
    }
}

// Workgroups are handed to the 8 XCDs round-robin by linear id.  Re-number them so that each
// XCD (own L2) works on a contiguous range of the tile sequence.
__device__ __forceinline__ int xcd_remap(int pid, int nblk) {
    constexpr int X = 8;
    int q = nblk / X, r = nblk % X;
    int x = pid % X, idx = pid / X;
    return x * q + (x < r ? x : r) + idx;
}

// silu(gate) * up rounded to the 16-bit type T, with gate and up already values of T.  The sigmoid uses
// the hardware exponential and reciprocal (about 2 ulp in fp32, far below the 16-bit rounding that
// follows).  The fp32 product is rounded on its own and only then converted: the empty asm keeps the
// compiler from folding multiply and conversion into one mixed-precision FMA, which rounds once (and
// gives a zero product the sign of its zero addend), so that every kernel that calls this returns the
// same bits as separate fp32 multiply and conversion steps do.
template <typename T>
__device__ __forceinline__ float silu_mul_round(float gate, float up) {
    const float sl = gate * __builtin_amdgcn_rcpf(1.0f + __expf(-gate));
    float prod = sl * up;
    asm("" : "+v"(prod));  // not volatile: the pins of different elements need no order among themselves
    return (float)(T)prod;
}

// a / s for many a and one s, bit-equal to the IEEE division `a / s`.  For a divisor well inside the
// exponent range this is the compiler's own expansion of a float division without the operand
// pre-scaling and the special-case fix-up, which only act on extreme exponents (reciprocal estimate,
// one Newton step, then two residual corrections of the quotient; the reciprocal is shared by all
// numerators).  The fast form is used for 2^-60 <= s <= 2^60: every numerator whose quotient is not
// far below the smallest e4m3 step (|a / s| >= 2^-30) then has normal residuals, so the corrections
// are exact; smaller quotients may differ in their last bits, and every caller rounds the quotient to
// e4m3, where all such values are zero of the same sign.  For other divisors (zero, subnormal, huge, inf, nan) `fast` is false and the caller
// divides plainly; the test is per divisor so that a caller branches once for all its numerators.
struct ScaleDivider {
    float s, r;
    bool fast;
    __device__ __forceinline__ explicit ScaleDivider(float scale) : s(scale) {
        fast = scale >= 0x1p-60f && scale <= 0x1p60f;
        const float r0 = __builtin_amdgcn_rcpf(scale);
        r = __builtin_fmaf(__builtin_fmaf(-scale, r0, 1.0f), r0, r0);
    }
    // valid while `fast` holds; a zero numerator keeps its sign as in the plain division
    __device__ __forceinline__ float quotient(float a) const {
        const float q0 = a * r;
        const float q1 = __builtin_fmaf(__builtin_fmaf(-s, q0, a), r, q0);
        return __builtin_copysignf(__builtin_fmaf(__builtin_fmaf(-s, q1, a), r, q1), a);
    }
};

}  // namespace tg
