// Host-side declarations shared by the C-ABI translation unit and the kernel instantiation units.
#pragma once
#include <hip/hip_runtime.h>
#include "tg_device.h"

namespace tg {

// Arguments of the layout-agnostic fallback kernel: any strides, any K.
struct GenericParams {
    GemmParams g;            // pointers, sizes, scales, grouping (A/B strides below override NT)
    int64_t a_sm, a_sk;      // element strides of A along m and k
    int64_t b_sn, b_sk;      // element strides of B along n and k
    int64_t b_se;            // element stride between experts
    int group;               // GroupMode
    int block_scaled;        // 0 per-tensor, 1 block
    int qbn, qbk;            // block-scaled: weight rows and K elements per scale (128 x 128 on the MFMA kernels; any here)
    int rows;                // row slots to visit (M, or the sorted-slot capacity in gather mode)
};

struct TileShape { int bm, bn; };

// Launchers return hipErrorInvalidConfiguration when the combination is not instantiated.
hipError_t run_tile_per_tensor(int bm, int bn, bool split, const GemmParams& p, int gx, int gy, hipStream_t s);
// 256x256 per-tensor tile with the hand-ordered K loop (dense, no split-K, K % 128 == 0): same results as
// run_tile_per_tensor(256, 256, false, ...)
hipError_t run_tile256(const GemmParams& p, int gx, hipStream_t s);
// 64x32 per-tensor tile, K split across the four waves of a workgroup (one launch; 16 < M <= ~512)
hipError_t run_tile_mid(int bm, int bn, const GemmParams& p, hipStream_t s);
// 64x128 per-tensor tile with four LDS stages (loads three K steps ahead): the 16 < M <= 64 form
hipError_t run_tile_deep(bool split, const GemmParams& p, int gx, int gy, hipStream_t s);
// 256x256 block-scaled tile, persistent (one workgroup per compute unit walks the tiles), dense rows or ragged expert
// segments: same results as the 256 x 256 forms of run_tile_block_dense / run_tile_block_grouped.  Needs K >= 256,
// both scale tensors; tiles_bound = an upper bound of the number of tiles
hipError_t run_bs256(int group, const GemmParams& p, int tiles_bound, hipStream_t s);
// K steps run_bs256 takes: at least two, and not 4c + 1 (a last chunk of scales of a single step); the weights of all
// experts together must also stay below 4 GiB
inline bool bs256_takes_k(int kblocks) { return kblocks >= 2 && kblocks % 4 != 1; }
// compute units of the current device
int compute_units();
hipError_t run_tile_block_dense(int bm, int bn, bool split, const GemmParams& p, int gx, int gy, hipStream_t s);
hipError_t run_tile_moe_act(int bm, const GemmParams& p, int gx, hipStream_t s);
hipError_t run_tile_block_grouped(int bm, int bn, int group, const GemmParams& p, int gx, hipStream_t s);
// up to kListMax per-tensor NT problems in one launch (tile 256x256, 128x128 or 64x128)
hipError_t run_tile_list(int bm, int bn, const GemmList& gl, int gx, hipStream_t s);
hipError_t run_skinny(int mt, int rg, int nw, bool blockscale, const GemmParams& p, int gx, int gy, hipStream_t s);
hipError_t run_stream(int mt, int nbuf, int waves, bool blockscale, const GemmParams& p, int gx, int gy, hipStream_t s);
// 64 weight rows per workgroup, activation piece shared through LDS: M <= 16
// ragged block-scaled GEMM, a handful of rows per expert: one grid row per expert, weights streamed once per 16 rows
hipError_t run_stream_ragged(const GemmParams& p, int waves, hipStream_t s);  // waves per workgroup: 4, 6 or 8 (16 weight rows each)
// two_buffers (needs K % 128 == 0): two 512-byte-per-row pieces per wave in flight, staggered over K; else one 1 KiB piece
// mt = 1, 2: tiles of 16 activation rows (M <= 16 mt; two only with two_buffers)
hipError_t run_stream_wide(bool blockscale, const GemmParams& p, int gy, hipStream_t s, bool two_buffers, int mt);
// C <- epilogue(sum_z partials[z]) for the split-K schedules (fixed z order: bit-reproducible)
hipError_t run_splitk_reduce(const GemmParams& p, bool block_scaled, hipStream_t s);
hipError_t run_generic(const GenericParams& p, hipStream_t s);
// moe_align_block_size in one launch (num_experts <= 512); ids are int32 or int64
hipError_t run_moe_align(const void* ids, int ids_are_i64, int numel, int E, int block_size, int* sorted_ids, int cap,
                         int* expert_ids, int nblk, int* num_post_pad, int* cumsum, int* max_cnt, hipStream_t s);
// moe_align_block_size and the 1 x 128 activation quantizer (all-zero group -> scale 1) side by side in one launch
hipError_t run_moe_align_quant(const void* ids, int ids_are_i64, int numel, int E, int block_size, int* sorted_ids, int cap,
                               int* expert_ids, int nblk, int* num_post_pad, int* cumsum, int* max_cnt, const void* x,
                               int x_is_bf16, uint8_t* q, float* scales, int64_t groups, hipStream_t s);
// per-token group e4m3 quantizer (group_size 16/32/64/128); x_type uses the OutType numbering (f32/f16/bf16);
// rule 0: zero group -> scale 1, 1: amax clamped below by eps, 2: as 1 with the scale rounded up to a power of two;
// strided: scale of group j of row r at scales[r * s_row + j * s_col]
hipError_t run_act_quant_group(const void* x, int x_type, uint8_t* q, bool q_is_int8, float* scales, int64_t groups, int group_size, float eps,
                               int rule, bool strided, int64_t groups_per_row, int64_t s_row, int64_t s_col, hipStream_t s);
// y (M,N) = float(x) * sc[i / bs][j / bs]; vec needs N % 16 == 0, bs % 16 == 0 and 16-byte aligned x and y
hipError_t run_weight_dequant(const uint8_t* x, const float* sc, void* y, int y_type, int64_t M, int64_t N, int bs, int64_t s_cols,
                              bool vec, hipStream_t s);
// q, scales <- quantize_1x128(round16(silu(x[:, :I]) * x[:, I:]));  x (rows, 2I) bf16/f16, I % 8 == 0
hipError_t run_silu_mul_quant(const void* x, int x_type, uint8_t* q, float* scales, int64_t rows, int I, hipStream_t s);
// out (tokens, H) <- sum over the top_k axis of x (tokens, top_k, H); bf16/f16, H % 8 == 0
hipError_t run_moe_sum(const void* x, void* out, int x_type, int64_t tokens, int top_k, int H, hipStream_t s);
// dst (cols, rows) <- transpose of src (rows, cols), one byte per element
// dst (cols x ld) = transpose of src (rows x cols), zero beyond `rows` in every dst row
hipError_t run_transpose_u8(const uint8_t* src, uint8_t* dst, int rows, int cols, int ld, hipStream_t s);
// dst (rows x ld) = src (rows x cols), zero beyond `cols` in every dst row
hipError_t run_pad_rows_u8(const uint8_t* src, uint8_t* dst, int rows, int cols, int ld, hipStream_t s);
// out (rows_out, cols_out) = in[r / rdiv][kb / kdiv] (in has in_cols columns): block scales of coarser blocks per 128 x 128 block
hipError_t run_expand_scales(const float* in, float* out, int rows_out, int cols_out, int in_cols, int rdiv, int kdiv, hipStream_t s);

}  // namespace tg
