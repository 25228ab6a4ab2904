/*
 * Plain-C restatement of the FP8 (OCP e4m3fn) GEMM arithmetic.  TEST INFRASTRUCTURE ONLY:
 * it is the checker for the HIP kernels and is never linked into the product library.
 *
 * The arithmetic follows the reference's own oracles:
 *   - block-scaled GEMM: tests/suites/unsloth/test_fp8.py:159-191
 *       C[m,n] = sum_k (A[m,k]*As[m,k/bk]) * (B[n,k]*Bs[n/bn,k/bk])
 *   - grouped form: tests/suites/flashinfer/test_flashinfer_ragged_block_scaled_bmm.py:77-136
 *   - token alignment: src/tilegym/ops/moe_interface.py:30-79
 * Products are formed in fp32 exactly as the torch oracle forms them (dequantized
 * operands are fp32), the sum over k is carried in double, then rounded once to fp32
 * and (optionally) once more to bf16 (round to nearest even).
 *
 * Pinned by tests/test_oracle.py: decode table against torch's float8 view, the GEMMs
 * against the torch oracle and against exact integer cases, alignment against the
 * worked example of src/tilegym/ops/cutile/moe_align_block.py:234-250.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* OCP E4M3: 1-4-3, bias 7, no inf, NaN = S.1111.111, subnormals k*2^-9, max 448. */
float orc_e4m3_decode(uint8_t code) {
    int sign = code >> 7, e = (code >> 3) & 0xF, m = code & 7;
    float v;
    if (e == 0xF && m == 7) return NAN;
    if (e == 0) v = ldexpf((float)m, -9);
    else v = ldexpf(1.0f + (float)m / 8.0f, e - 7);
    return sign ? -v : v;
}

/* round-to-nearest-even, saturating at +-448 (callers clamp first, as the reference's
 * quantizers do: src/tilegym/suites/unsloth/cutile/fp8.py:115) */
uint8_t orc_e4m3_encode(float x) {
    uint8_t sign = signbit(x) ? 0x80 : 0;
    double a = fabs((double)x);
    if (isnan(x)) return sign | 0x7F;
    if (a > 448.0) a = 448.0;
    if (a == 0.0) return sign;
    int e = (int)floor(log2(a));
    if (e < -6) e = -6;
    double q = ldexp(1.0, e - 3);
    double k = nearbyint(a / q); /* default rounding mode: to nearest even */
    double v = k * q;
    if (v > 448.0) v = 448.0;
    if (v < ldexp(1.0, -6)) return sign | (uint8_t)(v / ldexp(1.0, -9));
    int e2 = (int)floor(log2(v));
    int man = (int)nearbyint((v / ldexp(1.0, e2) - 1.0) * 8.0);
    return sign | (uint8_t)(((e2 + 7) << 3) | man);
}

void orc_e4m3_decode_table(float* out256) {
    for (int i = 0; i < 256; ++i) out256[i] = orc_e4m3_decode((uint8_t)i);
}

/* fp32 -> bf16 bits, round to nearest even (NaN kept quiet) */
uint16_t orc_bf16_bits(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x40);
    u += 0x7FFFu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

/*
 * Block-scaled NT GEMM.  A (M,K) codes, B (N,K) codes, As (M, ceil(K/bk)) or NULL (ones),
 * Bs (ceil(N/bn), ceil(K/bk)) or NULL (ones).  out (M,N) fp32.  alpha multiplies the result.
 */
void orc_gemm_block_scaled(const uint8_t* A, const uint8_t* B, const float* As, const float* Bs,
                           int64_t M, int64_t N, int64_t K, int64_t bn, int64_t bk, float alpha,
                           float* out) {
    float tab[256];
    orc_e4m3_decode_table(tab);
    int64_t kb = (K + bk - 1) / bk;
#pragma omp parallel for schedule(static)
    for (int64_t m = 0; m < M; ++m) {
        float* arow = (float*)malloc(sizeof(float) * (size_t)K);
        for (int64_t k = 0; k < K; ++k)
            arow[k] = tab[A[m * K + k]] * (As ? As[m * kb + k / bk] : 1.0f);
        for (int64_t n = 0; n < N; ++n) {
            double acc = 0.0;
            for (int64_t k = 0; k < K; ++k) {
                float b = tab[B[n * K + k]] * (Bs ? Bs[(n / bn) * kb + k / bk] : 1.0f);
                acc += (double)(arow[k] * b);
            }
            out[m * N + n] = alpha * (float)acc;
        }
        free(arow);
    }
}

/* Per-tensor NT GEMM: out = (sa*sb) * sum_k A[m,k]*B[n,k] with dequantized fp32 operands. */
void orc_gemm_per_tensor(const uint8_t* A, const uint8_t* B, float sa, float sb, int64_t M,
                         int64_t N, int64_t K, float* out) {
    float tab[256];
    orc_e4m3_decode_table(tab);
#pragma omp parallel for schedule(static)
    for (int64_t m = 0; m < M; ++m)
        for (int64_t n = 0; n < N; ++n) {
            double acc = 0.0;
            for (int64_t k = 0; k < K; ++k)
                acc += (double)((tab[A[m * K + k]] * sa) * (tab[B[n * K + k]] * sb));
            out[m * N + n] = (float)acc;
        }
}

/* Grouped form: expert q owns rows [indptr[q], indptr[q+1]) of A and weight B[q] (N,K). */
void orc_gemm_ragged(const uint8_t* A, const uint8_t* B, const float* As, const float* Bs,
                     const int32_t* indptr, int64_t Q, int64_t N, int64_t K, int64_t bn,
                     int64_t bk, float* out) {
    int64_t kb = (K + bk - 1) / bk, nb = (N + bn - 1) / bn;
    for (int64_t q = 0; q < Q; ++q) {
        int64_t lo = indptr[q], hi = indptr[q + 1];
        if (hi <= lo) continue;
        orc_gemm_block_scaled(A + lo * K, B + q * N * K, As ? As + lo * kb : NULL,
                              Bs ? Bs + q * nb * kb : NULL, hi - lo, N, K, bn, bk, 1.0f,
                              out + lo * N);
    }
}

/*
 * Token alignment for block-wise MoE.  topk_ids: numel flat expert ids.  sorted_ids must hold
 * numel + E*(bs-1) entries, expert_ids ceil(that/bs); cumsum E+1.  Stable within an expert.
 * Returns num_tokens_post_pad; *max_cnt = largest per-expert count before padding.
 */
int32_t orc_moe_align(const int32_t* topk_ids, int64_t numel, int32_t E, int32_t bs,
                      int32_t* sorted_ids, int32_t* expert_ids, int32_t* cumsum,
                      int32_t* max_cnt) {
    int64_t cap = numel + (int64_t)E * (bs - 1);
    int64_t nblk = (cap + bs - 1) / bs;
    for (int64_t i = 0; i < cap; ++i) sorted_ids[i] = (int32_t)numel;
    for (int64_t i = 0; i < nblk; ++i) expert_ids[i] = 0;
    int32_t* cnt = (int32_t*)calloc((size_t)E, sizeof(int32_t));
    for (int64_t i = 0; i < numel; ++i) cnt[topk_ids[i]]++;
    int32_t mx = 0;
    cumsum[0] = 0;
    for (int32_t e = 0; e < E; ++e) {
        if (cnt[e] > mx) mx = cnt[e];
        cumsum[e + 1] = cumsum[e] + (cnt[e] + bs - 1) / bs * bs;
        for (int32_t b = cumsum[e] / bs; b < cumsum[e + 1] / bs; ++b) expert_ids[b] = e;
    }
    int32_t* fill = (int32_t*)calloc((size_t)E, sizeof(int32_t));
    for (int64_t i = 0; i < numel; ++i) {
        int32_t e = topk_ids[i];
        sorted_ids[cumsum[e] + fill[e]++] = (int32_t)i;
    }
    *max_cnt = mx;
    int32_t post = cumsum[E];
    free(cnt);
    free(fill);
    return post;
}
