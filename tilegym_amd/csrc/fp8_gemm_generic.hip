// Layout-agnostic FP8 GEMM fallback (any strides, any K, all row modes) and a byte transpose.
// These are correctness paths for operand layouts the MFMA kernels do not take (K not a
// multiple of 16, unaligned bases, transposed A); they decode e4m3 in software and use no
// matrix instructions.
#include "tg_host.h"

namespace tg {

__device__ void generic_row(const GenericParams& q, int n, int r);

__global__ void __launch_bounds__(256) fp8_gemm_generic_kernel(const GenericParams q) {
    const GemmParams& p = q.g;
    const int n = blockIdx.x * 64 + threadIdx.x;
    if (n >= p.N) return;
    // rows: grid-stride (grid.y is capped at the launch limit)
    for (int r = blockIdx.y * 4 + threadIdx.y; r < q.rows; r += gridDim.y * 4) generic_row(q, n, r);
}

__device__ void generic_row(const GenericParams& q, int n, int r) {
    const GemmParams& p = q.g;
    int arow = r, crow = r, e = 0;
    if (q.group == GROUP_RAGGED) {
        e = -1;
        for (int i = 0; i < p.E; ++i)
            if (r >= p.m_indptr[i] && r < p.m_indptr[i + 1]) { e = i; break; }
        if (e < 0) return;
    } else if (q.group == GROUP_GATHER) {
        const int post = min(p.num_post_pad[0], p.em_capacity);
        if (r >= post) return;
        const int id = p.sorted_ids[r];
        if (id < 0 || id >= p.num_valid) return;
        arow = id / p.top_k;
        crow = id;
        e = p.expert_ids[r / p.block_m];
        if (e < 0 || e >= p.E) return;
    }
    const uint8_t* a = p.A + (int64_t)arow * q.a_sm;
    const uint8_t* b = p.B + (int64_t)e * q.b_se + (int64_t)n * q.b_sn;
    float acc = 0.f;
    // one partial sum per quantization block of K (128 elements unless the caller's blocks differ), scaled, then added
    const int qbk = q.block_scaled ? q.qbk : kKBlock, qbn = q.block_scaled ? q.qbn : 128;
    const int nkq = (p.K + qbk - 1) / qbk, nnq = (p.N + qbn - 1) / qbn;
    for (int kb = 0; kb < nkq; ++kb) {
        const int k_hi = min((kb + 1) * qbk, p.K);
        float part = 0.f;
        for (int k = kb * qbk; k < k_hi; ++k)
            part += e4m3_to_f32(a[(int64_t)k * q.a_sk]) * e4m3_to_f32(b[(int64_t)k * q.b_sk]);
        float s = 1.0f;
        if (q.block_scaled) {
            if (p.As) s *= p.As[(int64_t)arow * nkq + kb];
            if (p.Bs) s *= p.Bs[((int64_t)e * nnq + n / qbn) * nkq + kb];
        }
        acc += part * s;
    }
    float scale = p.alpha;
    if (!q.block_scaled) {
        if (p.As) scale *= p.As[0];
        if (p.Bs) scale *= p.Bs[0];
    }
    if (q.group == GROUP_GATHER && p.row_weight) scale *= p.row_weight[crow];
    float v = acc * scale;
    const int64_t at = (int64_t)crow * p.ldc + n;
    if (p.out_type == OUT_BF16) {
        __bf16* c = reinterpret_cast<__bf16*>(p.C) + at;
        if (p.beta != 0.f) v += p.beta * (float)(*c);
        *c = (__bf16)v;
    } else if (p.out_type == OUT_F32) {
        float* c = reinterpret_cast<float*>(p.C) + at;
        if (p.beta != 0.f) v += p.beta * (*c);
        *c = v;
    } else if (p.out_type == OUT_F8) {
        uint8_t* c = reinterpret_cast<uint8_t*>(p.C) + at;
        if (p.beta != 0.f) v += p.beta * e4m3_to_f32(*c);
        *c = f32_to_e4m3(v);
    } else {
        _Float16* c = reinterpret_cast<_Float16*>(p.C) + at;
        if (p.beta != 0.f) v += p.beta * (float)(*c);
        *c = (_Float16)v;
    }
}

hipError_t run_generic(const GenericParams& q, hipStream_t s) {
    if (q.rows <= 0 || q.g.N <= 0) return hipSuccess;
    const int gy = (q.rows + 3) / 4;
    dim3 grid((q.g.N + 63) / 64, gy < 65535 ? gy : 65535, 1);
    hipLaunchKernelGGL(fp8_gemm_generic_kernel, grid, dim3(64, 4, 1), 0, s, q);
    return hipGetLastError();
}

// dst (cols x ld) = transpose of src (rows x cols); ld >= rows, and dst[c][rows .. ld) = 0.
__global__ void __launch_bounds__(256) transpose_u8_kernel(const uint8_t* __restrict__ src,
                                                           uint8_t* __restrict__ dst, int rows,
                                                           int cols, int ld) {
    __shared__ uint8_t t[64][65];
    const int c0 = blockIdx.x * 64, r0 = blockIdx.y * 64;
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
    for (int i = ty; i < 64; i += 4) {
        const int r = r0 + i, c = c0 + tx;
        t[i][tx] = (r < rows && c < cols) ? src[(int64_t)r * cols + c] : 0;
    }
    __syncthreads();
    for (int i = ty; i < 64; i += 4) {
        const int c = c0 + i, r = r0 + tx;
        if (c < cols && r < ld) dst[(int64_t)c * ld + r] = t[tx][i];
    }
}

// dst (rows x ld) = src (rows x cols) with dst[r][cols .. ld) = 0; ld % 16 == 0, dst 16-byte aligned.  One thread writes
// 16 bytes; it reads them as one vector when the source rows are 16-byte aligned too (cols % 16 == 0), else byte by byte.
__global__ void __launch_bounds__(256) pad_rows_u8_kernel(const uint8_t* __restrict__ src, uint8_t* __restrict__ dst,
                                                          int rows, int cols, int ld, int vec) {
    const int per_row = ld / 16;
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (int64_t)rows * per_row) return;
    const int r = (int)(idx / per_row), c0 = (int)(idx % per_row) * 16;
    v4i out = v4i{0, 0, 0, 0};
    if (vec && c0 + 16 <= cols) {
        out = *reinterpret_cast<const v4i*>(src + (int64_t)r * cols + c0);
    } else if (c0 < cols) {
        uint8_t bytes[16];
#pragma unroll
        for (int q = 0; q < 16; ++q) bytes[q] = c0 + q < cols ? src[(int64_t)r * cols + c0 + q] : (uint8_t)0;
        __builtin_memcpy(&out, bytes, 16);
    }
    *reinterpret_cast<v4i*>(dst + (int64_t)r * ld + c0) = out;
}

// Second pass of the split-K schedules: one thread adds the split_k partial sums of four
// consecutive outputs in z order, then scales, applies beta and casts.
__global__ void __launch_bounds__(256) splitk_reduce_kernel(const GemmParams p, int block_scaled) {
    const int64_t quads_per_row = (p.N + 3) / 4;
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= quads_per_row * p.M) return;
    const int m = (int)(idx / quads_per_row), col = (int)(idx % quads_per_row) * 4;
    const int64_t MN = (int64_t)p.M * p.N, at = (int64_t)m * p.N + col;
    const bool vec_ok = p.vec_store != 0;
    v4f sum = v4f{0.f, 0.f, 0.f, 0.f};
    if (vec_ok && col + 3 < p.N) {
        // four partial sums are fetched before any is added: the kernel is one memory round trip
        // deep per group of four instead of one per split (the z order of the additions is kept)
        int z = 0;
        for (; z + 4 <= p.split_k; z += 4) {
            v4f t[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) t[i] = __builtin_nontemporal_load(reinterpret_cast<const v4f*>(p.partials + (z + i) * MN + at));
#pragma unroll
            for (int i = 0; i < 4; ++i) sum += t[i];
        }
        for (; z < p.split_k; ++z) sum += __builtin_nontemporal_load(reinterpret_cast<const v4f*>(p.partials + z * MN + at));
    } else {
        for (int z = 0; z < p.split_k; ++z) {
            const float* src = p.partials + z * MN + at;
            for (int q = 0; q < 4 && col + q < p.N; ++q) sum[q] += src[q];
        }
    }
    float scale = p.alpha;
    if (!block_scaled) {
        if (p.As) scale *= p.As[0];
        if (p.Bs) scale *= p.Bs[0];
    }
    store4(p.C, p.out_type, m, col, p.N, p.ldc, sum * scale, p.beta, vec_ok);
}

hipError_t run_splitk_reduce(const GemmParams& p, bool block_scaled, hipStream_t s) {
    const int64_t work = (int64_t)((p.N + 3) / 4) * p.M;
    if (work <= 0) return hipSuccess;
    hipLaunchKernelGGL(splitk_reduce_kernel, dim3((unsigned)((work + 255) / 256)), dim3(256), 0, s, p,
                       block_scaled ? 1 : 0);
    return hipGetLastError();
}

// Block scales given per (qbn x qbk) block, qbn and qbk multiples of 128, written out per 128 x 128 block: out[r][kb] =
// in[r / rdiv][kb / kdiv] (rdiv = qbn / 128 for weight scales, 1 for the activations' per-row scales; kdiv = qbk / 128).
__global__ void __launch_bounds__(256) expand_scales_kernel(const float* __restrict__ in, float* __restrict__ out, int rows_out, int cols_out,
                                                            int in_cols, int rdiv, int kdiv) {
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (int64_t)rows_out * cols_out) return;
    const int r = (int)(idx / cols_out), kb = (int)(idx % cols_out);
    out[idx] = in[(int64_t)(r / rdiv) * in_cols + kb / kdiv];
}

hipError_t run_expand_scales(const float* in, float* out, int rows_out, int cols_out, int in_cols, int rdiv, int kdiv, hipStream_t s) {
    const int64_t work = (int64_t)rows_out * cols_out;
    if (work <= 0) return hipSuccess;
    hipLaunchKernelGGL(expand_scales_kernel, dim3((unsigned)((work + 255) / 256)), dim3(256), 0, s, in, out, rows_out, cols_out, in_cols, rdiv, kdiv);
    return hipGetLastError();
}

hipError_t run_transpose_u8(const uint8_t* src, uint8_t* dst, int rows, int cols, int ld, hipStream_t s) {
    if (rows <= 0 || cols <= 0 || ld < rows) return hipSuccess;
    dim3 grid((cols + 63) / 64, (ld + 63) / 64, 1);
    hipLaunchKernelGGL(transpose_u8_kernel, grid, dim3(256, 1, 1), 0, s, src, dst, rows, cols, ld);
    return hipGetLastError();
}

hipError_t run_pad_rows_u8(const uint8_t* src, uint8_t* dst, int rows, int cols, int ld, hipStream_t s) {
    if (rows <= 0 || cols <= 0 || ld < cols || (ld % 16) != 0) return hipSuccess;
    const int64_t threads = (int64_t)rows * (ld / 16);
    const int vec = (cols % 16) == 0 && (reinterpret_cast<uintptr_t>(src) % 16) == 0;
    hipLaunchKernelGGL(pad_rows_u8_kernel, dim3((unsigned)((threads + 255) / 256), 1, 1), dim3(256, 1, 1), 0, s, src, dst, rows, cols, ld, vec);
    return hipGetLastError();
}

}  // namespace tg
