// Yardstick kernels: what this GPU sustains on the two resources the GEMM kernels are bound by, measured by the same
// process that times the GEMMs.  They compute nothing useful.
//   tg_diag_read : a plain read of a buffer (16 bytes per lane, non-temporal, grid-stride) -- the floor of any kernel
//                  that has to read those bytes once (the decode GEMMs: their weights).
//   tg_diag_mfma : e4m3 16x16x128 MFMAs on register operands, eight waves per compute unit, optionally with `fmas`
//                  scale-and-add FMAs behind every MFMA the way the block-scaled kernels issue them: the matrix pipe's
//                  rate on non-zero data, and what is left of it when the VALU issue port is shared with four FMAs per
//                  MFMA (an MFMA holds the port for about as long as four FMAs do, together the MFMA's own time).
#include "../../include/tilegym_hip.h"
#include "tg_device.h"

namespace {

template <int UNROLL>
__global__ void __launch_bounds__(256) diag_read_kernel(const v4i* __restrict__ src, int64_t n16, int* out) {
    const int64_t stride = (int64_t)gridDim.x * 256;
    int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    v4i acc = {0, 0, 0, 0};
    for (; i + (UNROLL - 1) * stride < n16; i += UNROLL * stride) {
        v4i t[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) t[u] = __builtin_nontemporal_load(src + i + u * stride);
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) acc ^= t[u];
    }
    for (; i < n16; i += stride) acc ^= __builtin_nontemporal_load(src + i);
    const int v = acc[0] ^ acc[1] ^ acc[2] ^ acc[3];
    if (v == 0x5A5A1234) out[blockIdx.x] = v;  // (practically never: the loads must not be optimised away)
}

template <int NF>
__global__ void __launch_bounds__(512, 1) diag_mfma_kernel(float* out, int iters, float scale) {
    const int lane = threadIdx.x;
    v8i a, b;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        a[i] = (int)((lane * 2654435761u + i * 40503u) & 0x77777777u);  // finite e4m3 codes, all bit positions in use
        b[i] = (int)((lane * 40503u + i * 2654435761u) & 0x77777777u);
    }
    constexpr int NACC = 32;
    v4f acc[NACC];
#pragma unroll
    for (int i = 0; i < NACC; ++i) acc[i] = v4f{0.f, 0.f, 0.f, 0.f};
    v4f part[3] = {v4f{0.f, 0.f, 0.f, 0.f}, v4f{0.f, 0.f, 0.f, 0.f}, v4f{0.f, 0.f, 0.f, 0.f}};
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int j = 0; j < NACC; ++j) {
            if constexpr (NF == 0) {
                acc[j] = tg::mfma_e4m3(a, b, acc[j]);
            } else {
                asm volatile("" : "+v"(a));  // (the MFMAs must not be merged into one)
                part[j % 3] = tg::mfma_e4m3(a, b, v4f{0.f, 0.f, 0.f, 0.f});
                const int jj = (j + 1) % 3, d = (j + NACC - 2) % NACC;  // the product issued two MFMAs earlier
#pragma unroll
                for (int r = 0; r < NF; ++r) acc[d][r & 3] = __builtin_fmaf(part[jj][r & 3], scale, acc[d][r & 3]);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < NACC; ++i) s += acc[i][0] + acc[i][1] + acc[i][2] + acc[i][3];
    out[(size_t)blockIdx.x * 512 + threadIdx.x] = s;
}

}  // namespace

extern "C" {

int32_t tg_diag_read(const tg_tensor* x, const tg_tensor* out, int32_t workgroups, int32_t loads_in_flight, int32_t device_id,
                     uint64_t hip_stream) {
    if (!x || !out || !x->ptr || !out->ptr) return TG_ERR_NULL;
    int64_t bytes = 1;
    for (int i = 0; i < x->ndim; ++i) bytes *= x->shape[i];
    switch (x->dtype) {
        case TG_F32: case TG_I32: bytes *= 4; break;
        case TG_F16: case TG_BF16: bytes *= 2; break;
        case TG_I64: bytes *= 8; break;
        default: break;
    }
    int64_t slots = 1;
    for (int i = 0; i < out->ndim; ++i) slots *= out->shape[i];
    if (workgroups <= 0) workgroups = 2048;
    if (loads_in_flight <= 0) loads_in_flight = 4;
    if ((x->ptr & 15) != 0 || out->dtype != TG_I32 || workgroups > 65536 || slots < workgroups ||
        (loads_in_flight != 1 && loads_in_flight != 2 && loads_in_flight != 4 && loads_in_flight != 8))
        return TG_ERR_INVALID;
    int prev = -1;
    if (hipGetDevice(&prev) != hipSuccess) return TG_ERR_DEVICE;
    if (prev != device_id && hipSetDevice(device_id) != hipSuccess) return TG_ERR_DEVICE;
    hipStream_t s = reinterpret_cast<hipStream_t>(hip_stream);
    const v4i* src = reinterpret_cast<const v4i*>(x->ptr);
    int* o = reinterpret_cast<int*>(out->ptr);
    const dim3 g(workgroups), b(256);
    switch (loads_in_flight) {
        case 1: hipLaunchKernelGGL(diag_read_kernel<1>, g, b, 0, s, src, bytes / 16, o); break;
        case 2: hipLaunchKernelGGL(diag_read_kernel<2>, g, b, 0, s, src, bytes / 16, o); break;
        case 4: hipLaunchKernelGGL(diag_read_kernel<4>, g, b, 0, s, src, bytes / 16, o); break;
        default: hipLaunchKernelGGL(diag_read_kernel<8>, g, b, 0, s, src, bytes / 16, o); break;
    }
    const hipError_t e = hipGetLastError();
    if (prev != device_id) (void)hipSetDevice(prev);
    return e == hipSuccess ? TG_OK : TG_ERR_LAUNCH;
}

int32_t tg_diag_mfma(int32_t fmas, int32_t iters, int32_t workgroups, const tg_tensor* out, int32_t device_id, uint64_t hip_stream) {
    if (!out || !out->ptr) return TG_ERR_NULL;
    int64_t slots = 1;
    for (int i = 0; i < out->ndim; ++i) slots *= out->shape[i];
    if (out->dtype != TG_F32 || workgroups < 1 || workgroups > 4096 || slots < (int64_t)workgroups * 512 || iters < 1 || iters > (1 << 20))
        return TG_ERR_INVALID;
    if (fmas != 0 && fmas != 2 && fmas != 4 && fmas != 6 && fmas != 8) return TG_ERR_INVALID;
    int prev = -1;
    if (hipGetDevice(&prev) != hipSuccess) return TG_ERR_DEVICE;
    if (prev != device_id && hipSetDevice(device_id) != hipSuccess) return TG_ERR_DEVICE;
    hipStream_t s = reinterpret_cast<hipStream_t>(hip_stream);
    float* o = reinterpret_cast<float*>(out->ptr);
    const dim3 g(workgroups), b(512);
    switch (fmas) {
        case 0: hipLaunchKernelGGL(diag_mfma_kernel<0>, g, b, 0, s, o, iters, 1.5f); break;
        case 2: hipLaunchKernelGGL(diag_mfma_kernel<2>, g, b, 0, s, o, iters, 1.5f); break;
        case 4: hipLaunchKernelGGL(diag_mfma_kernel<4>, g, b, 0, s, o, iters, 1.5f); break;
        case 6: hipLaunchKernelGGL(diag_mfma_kernel<6>, g, b, 0, s, o, iters, 1.5f); break;
        default: hipLaunchKernelGGL(diag_mfma_kernel<8>, g, b, 0, s, o, iters, 1.5f); break;
    }
    const hipError_t e = hipGetLastError();
    if (prev != device_id) (void)hipSetDevice(prev);
    return e == hipSuccess ? TG_OK : TG_ERR_LAUNCH;
}

}  // extern "C"
