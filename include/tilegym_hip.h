/*
 * tilegym_hip.h -- C ABI of libtilegym_hip.so: FP8 (OCP e4m3fn) GEMM for AMD gfx950 (MI355X).
 *
 * One shared library, plain pointers and sizes, no framework types.  Every entry point
 *   - borrows the memory it is given (never frees, never keeps a pointer),
 *   - validates its arguments on the host BEFORE touching the device (so argument errors
 *     are reported without a GPU),
 *   - enqueues its kernels on the given HIP stream and returns without synchronising,
 *   - returns an int32 code: 0 = ok, negative = error (see tg_rc_message).
 *
 * The tensor descriptor and the return codes keep the layout / numbering of the
 * reference's own C-ABI precedent (TensorDesc: src/tilegym/ops/cutile_rs/ffi_util.rs:26-35,
 * rc codes: src/tilegym/ops/cutile_rs/ffi_util.rs:108-122).
 */
#ifndef TILEGYM_HIP_H
#define TILEGYM_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TG_ABI_VERSION 1
#define TG_MAX_DIMS 5

/* dtype codes (src/tilegym/ops/cutile_rs/ffi_util.rs:32-34) */
enum {
    TG_F32 = 0,
    TG_F16 = 1,
    TG_BF16 = 2,
    TG_I32 = 3,
    TG_I64 = 4,
    TG_F8E5M2 = 5,
    TG_F8E4M3FN = 7,
    TG_I8 = 8        /* not in the reference's numbering (0-7): the int8 destination of tg_fp8_quant_group */
};

/* return codes (src/tilegym/ops/cutile_rs/ffi_util.rs:108-122); -1 is reserved as the
 * "auto" sentinel of the cfg array and is never returned. */
enum {
    TG_OK = 0,
    TG_ERR_DTYPE = -2,
    TG_ERR_LAUNCH = -3,
    TG_ERR_DEVICE = -4,
    TG_ERR_NULL = -5,
    TG_ERR_INVALID = -6
};

/* Borrowed view of a device tensor.  Strides are in ELEMENTS. */
typedef struct tg_tensor {
    uint64_t ptr;
    int32_t ndim;
    int64_t shape[TG_MAX_DIMS];
    int64_t strides[TG_MAX_DIMS];
    int32_t dtype;
} tg_tensor;

/* cfg[] slots: tile / schedule overrides, -1 (or a short array) = choose automatically.
 * This is the C form of the reference's per-call `kernel_configs={...}` override
 * (src/tilegym/kernel_utils.py:14-36). */
enum {
    TG_CFG_KERNEL = 0,  /* 0 fallback (no MFMA), 1 LDS-tiled MFMA kernel, 2 skinny (direct weight streaming), 3 stream (weight streaming through LDS) */
    TG_CFG_BLOCK_M = 1, /* tiled kernel: rows of A per workgroup (32/64/128/256; 32x32, 64x32 and 64x64 = in-workgroup K split, per-tensor only) */
    TG_CFG_BLOCK_N = 2, /* tiled kernel: rows of B per workgroup (32/64/128/256; per-tensor with BLOCK_M = 64 also 72 .. 120 in steps of 8); stream kernel, wide form (ROW_GROUPS = 4,
                         * K % 128 == 0): rows of B per workgroup, a multiple of 4 up to 64 (four waves own a quarter each); narrow form: 1 .. 16 */
    TG_CFG_SPLIT_K = 3, /* K partitions reduced through the workspace (1 = none)         */
    TG_CFG_ROW_GROUPS = 4, /* skinny kernel: 16-row groups of B per wave (1/2/4); stream kernel: LDS buffers per wave (1/2);
                            * tiled 256x256 block-scaled kernels (dense and ragged): 1 = the persistent form (one workgroup per
                            * compute unit walks the tiles, three weight slabs in LDS, scales in registers); the ragged GEMM
                            * chooses it by itself for K <= 1536 */
    TG_CFG_WAVES = 5,   /* skinny kernel: waves per workgroup splitting K (4/8/16); stream kernel: 8 = eight waves split K inside a 16-row workgroup, and with ROW_GROUPS = 4 (the wide form) 1 = one 1 KiB piece per wave in flight instead of two half pieces; tiled 256x256 kernels: 8 = the generic eight-wave tile kernel (one workgroup per tile) instead of the persistent one; ragged GEMM, streaming form: 4 / 6 / 8 waves (64 / 96 / 128 weight rows) per workgroup */
    TG_CFG_QUANT_BLOCK_N = 6, /* block-scaled tg_fp8_gemm: weight rows per scale (default 128) */
    TG_CFG_QUANT_BLOCK_K = 7, /* block-scaled tg_fp8_gemm: K elements per scale (default 128): the reference's
                               * block_size=[bn, bk] argument, src/tilegym/suites/unsloth/cutile/fp8.py:388-446.  Blocks that
                               * are multiples of 128 x 128 (256 x 128, 128 x 256, 256 x 256, ...) run on the MFMA kernels: with
                               * a workspace (tg_fp8_gemm_workspace_bytes counts the room) tg_fp8_gemm first writes the scales
                               * out per 128 x 128 block; finer blocks, and coarse ones without that room, run on the fallback
                               * kernel (no MFMA) */
    TG_CFG_PIECES = 8,  /* reported by tg_last_config only: 1, or the number of separately scheduled pieces the call ran as
                         * (column chunks of a weight of 2 GiB and more; the columns or rows that fill whole rounds of the chip
                         * with 256x256 tiles and the rest): the other slots then describe the first piece.  Ignored in cfg[]. */
    TG_CFG_COUNT = 9
};

/*
 * Dense FP8 GEMM:  C <- alpha * (sa * op(A)) @ (sb * op(B)) + beta * C
 *
 * Replaces, for e4m3 inputs, the launch half of
 *   tilegym.ops.matmul                      src/tilegym/ops/cutile/matmul.py:421-455
 *   flashinfer gemm_alpha_beta              src/tilegym/suites/flashinfer/cutile/gemm/gemm_alpha_beta.py:336-504
 *   unsloth w8a8_block_fp8_matmul           src/tilegym/suites/unsloth/cutile/fp8.py:388-446
 *
 * a: (M,K), or (K,M) when trans_a;  b: (K,N), or (N,K) when trans_b;  both e4m3fn, contiguous.
 * c: (M,N) contiguous, dtype bf16 / f32 / f16, or float8_e4m3fn (the fp32 result is rounded to nearest even and
 *    saturates at +-448; NaN stays NaN).  beta != 0 reads c.
 * scale_a / scale_b (f32, device memory):
 *     NULL                     -> 1.0
 *     1 element                -> per-tensor scale
 *     scale_a (M, ceil(K/128)) and scale_b (ceil(N/128), ceil(K/128)) -> block scaled:
 *        C[m,n] = sum_kb scale_a[m,kb] * scale_b[n/128,kb] * sum_{k in kb} A[m,k] * B[n,k]
 *     (both must be of the same kind; block form requires the NT layout.)
 * workspace: NULL, or a 16-byte-aligned scratch buffer (any dtype, contents irrelevant) of at
 *     least tg_fp8_gemm_workspace_bytes() bytes.  It holds split-K partial sums, for
 *     (K,N) weights a K-contiguous copy of b, and for a K that the MFMA kernels cannot step
 *     through (K % 16 != 0; K % 128 != 0 above 64 rows) copies of a and b with every row
 *     zero-padded to the next multiple of 128.  Calls that share a workspace must not overlap
 *     in time (calls on one stream never do).  Without a workspace the split-K schedules, the
 *     (K,N) fast path and the padded copies are not used (such a K then runs on the fallback
 *     kernel).
 */
int32_t tg_fp8_gemm(const tg_tensor* c, const tg_tensor* a, const tg_tensor* b,
                    const tg_tensor* scale_a, const tg_tensor* scale_b, int32_t trans_a,
                    int32_t trans_b, float alpha, float beta, const tg_tensor* workspace,
                    const int32_t* cfg, int32_t ncfg, int32_t device_id, uint64_t hip_stream);

/*
 * tg_fp8_gemm for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.  Same arguments, schedules
 * and results as tg_fp8_gemm, without the workspace argument: split-K partial sums and the K-contiguous copy of
 * a (K,N) weight go to a TG_STATIC_SCRATCH_BYTES array inside the library's device image (one copy per GPU,
 * held until the process ends).  The call allocates nothing and frees nothing.  A problem whose schedule needs
 * more scratch than the array holds returns TG_ERR_INVALID (the text says how much): call tg_fp8_gemm with a
 * caller-owned workspace for it.  All calls on one GPU share that GPU's array, whatever the stream: calls that
 * overlap in time on one GPU race on it; calls on one stream never overlap.  Nothing in the array needs to start
 * at zero (no atomics are used), so nothing is cleared between calls.  The first call on a device looks the
 * array's address up (hipGetSymbolAddress); make that call outside graph capture.
 */
#define TG_STATIC_SCRATCH_BYTES (32 * 1024 * 1024)
int32_t tg_fp8_gemm_static_scratch(const tg_tensor* c, const tg_tensor* a, const tg_tensor* b,
                                   const tg_tensor* scale_a, const tg_tensor* scale_b, int32_t trans_a,
                                   int32_t trans_b, float alpha, float beta, const int32_t* cfg, int32_t ncfg,
                                   int32_t device_id, uint64_t hip_stream);

/* Bytes of workspace that let tg_fp8_gemm use every schedule for this problem
 * (trans_b == 0 adds room for a K-contiguous copy of B; a K that is no multiple of 16, or
 * no multiple of 128 above 64 rows, adds room for zero-padded copies of both operands).
 * Never fails; returns 0 for non-positive sizes. */
int64_t tg_fp8_gemm_workspace_bytes(int64_t M, int64_t N, int64_t K, int32_t trans_b,
                                    const int32_t* cfg, int32_t ncfg);

/*
 * Grouped (expert-offset) block-scaled FP8 GEMM, NT layout:
 *   for q in [0,Q):  C[m_indptr[q]:m_indptr[q+1]] = (A[rows] * a_scale) @ (B[q] * b_scale[q])^T
 *
 * Replaces the launch half of flashinfer ragged_block_scaled_bmm
 *   src/tilegym/suites/flashinfer/cutile/gemm/ragged_block_scaled_bmm.py:497-616
 * a (total_m,K) e4m3; b (Q,N,K) e4m3; a_scale (total_m, ceil(K/128)) f32 or NULL (ones);
 * b_scale (Q, ceil(N/128), ceil(K/128)) f32, or NULL (ones);
 * m_indptr (Q+1) i32 DEVICE memory, non-decreasing, m_indptr[Q] <= total_m; segments need no
 * alignment and may be empty.  Rows at or past m_indptr[Q] are not written.
 * c (total_m,N) bf16/f32/f16 (or float8_e4m3fn, as for tg_fp8_gemm).
 */
int32_t tg_fp8_ragged_gemm(const tg_tensor* c, const tg_tensor* a, const tg_tensor* b,
                           const tg_tensor* a_scale, const tg_tensor* b_scale,
                           const tg_tensor* m_indptr, const int32_t* cfg, int32_t ncfg,
                           int32_t device_id, uint64_t hip_stream);

/*
 * Token-gather MoE GEMM (block-scaled FP8, NT):
 *   for every slot r < num_tokens_post_padded with id = sorted_token_ids[r] < num_valid:
 *       C[id] = (A[id / top_k] * a_scale) @ (B[expert_ids[r / block_m]] * b_scale)^T  (* topk_weights[id])
 *
 * Replaces the launch half of invoke_fused_moe_kernel's use_fp8_w8a8 path
 *   src/tilegym/ops/tilecpp/moe.py:241-310, kernel src/tilegym/ops/tilecpp/moe.cuh:72-225
 * a (T,K) e4m3; b (E,N,K) e4m3; c (num_valid, N) bf16/f32/f16 (the (T,top_k,N) cache, flattened);
 * a_scale (T, ceil(K/128)) or NULL; b_scale (E, ceil(N/128), ceil(K/128)) or NULL;
 * topk_weights (num_valid) f32 or NULL (required when mul_routed_weight != 0);
 * sorted_token_ids (EM) i32, expert_ids (>= EM/block_m) i32, num_tokens_post_padded (1) i32,
 * all DEVICE memory, as produced by moe_align_block_size with block size block_m
 * (src/tilegym/ops/cutile/moe_align_block.py:205-268); block_m must be a multiple of 16.
 */
int32_t tg_fp8_moe_gemm(const tg_tensor* c, const tg_tensor* a, const tg_tensor* b,
                        const tg_tensor* a_scale, const tg_tensor* b_scale,
                        const tg_tensor* topk_weights, const tg_tensor* sorted_token_ids,
                        const tg_tensor* expert_ids, const tg_tensor* num_tokens_post_padded,
                        int32_t mul_routed_weight, int32_t top_k, int32_t block_m,
                        const int32_t* cfg, int32_t ncfg, int32_t device_id, uint64_t hip_stream);

/*
 * First GEMM of the FP8 MoE layer with its activation fused into the epilogue:
 *   for every routed slot id:  h = (A[id / top_k] * a_scale) @ (B[e] * b_scale)^T        (2*I columns, rounded to `act_dtype`)
 *                              act = act_dtype(silu(h[:I]) * h[I:])
 *                              q[id], scales[id] = 1x128 e4m3 quantization of act (all-zero group -> scale 1)
 * i.e. tg_fp8_moe_gemm followed by tg_silu_mul_quant_1x128, bit for bit, without the (T*top_k, 2*I) intermediate.
 * Replaces the GEMM1 + SiLU-and-multiply steps of fused_experts_impl, src/tilegym/ops/moe_interface.py:252-277
 * (activation: src/tilegym/ops/ops.py:172-193).
 * b (E, 2*I, K) e4m3 with I % 128 == 0 and K % 128 == 0; q (num_valid, I) e4m3; scales (num_valid, I/128) f32;
 * act_dtype: TG_BF16 or TG_F16; block_m (the moe_align block size) must be a multiple of 128 (256-row tiles when
 * it is a multiple of 256, else 128-row tiles); the other
 * arguments as for tg_fp8_moe_gemm.  Shapes outside these limits return TG_ERR_INVALID: call the two-step form.
 */
int32_t tg_fp8_moe_gemm_silu_quant(const tg_tensor* q, const tg_tensor* scales, const tg_tensor* a, const tg_tensor* b,
                                   const tg_tensor* a_scale, const tg_tensor* b_scale,
                                   const tg_tensor* sorted_token_ids, const tg_tensor* expert_ids,
                                   const tg_tensor* num_tokens_post_padded, int32_t top_k, int32_t block_m,
                                   int32_t act_dtype, int32_t device_id, uint64_t hip_stream);

/*
 * A list of independent FP8 GEMMs, C_i <- (sa_i * A_i) @ (sb_i * op(B_i)), i < count, in one launch when
 * every problem has (N,K) weights (trans_b != 0), K_i % 128 == 0 and 16-byte aligned operands; any other
 * list is run problem by problem with tg_fp8_gemm's schedules (same results).
 * Replaces the launch half of tilegym.ops.group_gemm, src/tilegym/ops/cutile/group_gemm.py:170-197.
 * c, a, b: arrays of `count` descriptor pointers; scale_a, scale_b: NULL, or arrays whose entries are NULL or
 * one-element f32 tensors.  All c_i share one dtype (bf16 / f16 / f32 / float8_e4m3fn).  workspace: as for tg_fp8_gemm
 * (only used on the problem-by-problem route).
 */
int32_t tg_fp8_group_gemm(const tg_tensor* const* c, const tg_tensor* const* a, const tg_tensor* const* b,
                          const tg_tensor* const* scale_a, const tg_tensor* const* scale_b, int32_t count,
                          int32_t trans_b, const tg_tensor* workspace, const int32_t* cfg, int32_t ncfg,
                          int32_t device_id, uint64_t hip_stream);

/*
 * moe_align_block_size: group the (token, slot) pairs of a top-k routing by expert and pad every
 * group to a multiple of block_size, in one launch and without host synchronisation.
 * Replaces src/tilegym/ops/cutile/moe_align_block.py:205-268 (four launches) and
 * src/tilegym/ops/tilecpp/moe_align_block.py:274-335; arithmetic of src/tilegym/ops/moe_interface.py:30-79.
 * topk_ids: any shape, i32 or i64, numel pairs, expert labels in [0, num_experts) (others are skipped).
 * sorted_token_ids (numel + num_experts * (block_size - 1)) i32: pair indices grouped by expert,
 *   ascending inside an expert; every unused position holds numel.
 * expert_ids (ceil(that / block_size)) i32; num_tokens_post_padded (1) i32; cumsum (num_experts + 1) i32
 * (padded prefix sums); max_expert_count (1) i32.  num_experts <= 512 (rc -6 beyond).
 */
int32_t tg_moe_align_block_size(const tg_tensor* topk_ids, int32_t block_size, int32_t num_experts,
                                const tg_tensor* sorted_token_ids, const tg_tensor* expert_ids,
                                const tg_tensor* num_tokens_post_padded, const tg_tensor* cumsum,
                                const tg_tensor* max_expert_count, int32_t device_id, uint64_t hip_stream);

/*
 * tg_moe_align_block_size and the 1 x 128 activation quantizer (tg_fp8_quant_1x128 with rule 0) as ONE launch: the two
 * launches in front of the first GEMM of the FP8 MoE layer (the layer of src/tilegym/ops/moe_interface.py:116-321 calls
 * moe_align_block_size at :246-248; the FP8 GEMM needs its activations quantized 1 x 128 first).  The two share no data.
 * Arguments and results as for the two entry points; x: bf16 or f16, last dimension a multiple of 128.
 */
int32_t tg_moe_align_quant_1x128(const tg_tensor* topk_ids, int32_t block_size, int32_t num_experts,
                                 const tg_tensor* sorted_token_ids, const tg_tensor* expert_ids,
                                 const tg_tensor* num_tokens_post_padded, const tg_tensor* cumsum,
                                 const tg_tensor* max_expert_count, const tg_tensor* q, const tg_tensor* scales,
                                 const tg_tensor* x, int32_t device_id, uint64_t hip_stream);

/*
 * Per-token 1 x 128 FP8 quantizer (the producer of scale_a for the block-scaled GEMMs):
 *   scales[m, kb] = amax(x[m, 128*kb : 128*kb+128]) / 448      (rule 0: an all-zero group gets 1.0;
 *                                                               rule 1: amax is first clamped below by eps)
 *   q = e4m3fn(clamp(x / scale, -448, 448)), round to nearest even, IEEE divisions.
 * Replaces src/tilegym/suites/unsloth/cutile/fp8.py:370-385 (act_quant, rule 0) and the row-major fp8 case of
 * src/tilegym/suites/flashinfer/cutile/per_token_group_quant_8bit.py:152-272 (rule 1).
 * x (..., K) bf16 / f16 / f32 contiguous, K % 128 == 0, 16-byte aligned; q same shape e4m3fn;
 * scales (..., K/128) f32 contiguous.
 */
int32_t tg_fp8_quant_1x128(const tg_tensor* q, const tg_tensor* scales, const tg_tensor* x, float eps,
                           int32_t rule, int32_t device_id, uint64_t hip_stream);

/*
 * Per-token group FP8 quantizer, the general form of tg_fp8_quant_1x128: groups of group_size = 16, 32, 64 or 128
 * consecutive elements of a row, and a third scale rule,
 *   rule 2: as rule 1, then scale = 2^ceil(log2(max(|scale|, 1e-10)))   (power-of-two "UE8M0" scales).
 * scales is either contiguous with numel(x) / group_size elements (row-major), or a 2-D (rows, K / group_size)
 * descriptor with any element strides - (1, rows) is the column-major layout and (1, ceil4(rows)) the 16-byte
 * aligned one of the reference.  rows = numel(x) / K.
 * Replaces src/tilegym/suites/flashinfer/cutile/per_token_group_quant_8bit.py:22-145 (both kernels) and the host
 * function at :152-272 for dst_dtype float8_e4m3fn.
 * x (..., K) bf16 / f16 / f32 contiguous, K % group_size == 0, 16-byte aligned; q same shape e4m3fn, 8-byte aligned.
 */
int32_t tg_fp8_quant_group(const tg_tensor* q, const tg_tensor* scales, const tg_tensor* x, int32_t group_size,
                           float eps, int32_t rule, int32_t device_id, uint64_t hip_stream);

/*
 * Block dequantization of a weight: y[i, j] = float(x[i, j]) * s[i / block_size, j / block_size], fp32 product
 * rounded once to y's type.  Replaces src/tilegym/suites/unsloth/cutile/fp8.py:36-71 (kernel) and :348-367 (host).
 * x (M, N) e4m3fn contiguous; s (ceil(M / block_size), ceil(N / block_size)) f32 contiguous; y (M, N) bf16 / f16 / f32
 * contiguous; block_size >= 1.
 */
int32_t tg_fp8_weight_dequant(const tg_tensor* y, const tg_tensor* x, const tg_tensor* s, int32_t block_size,
                              int32_t device_id, uint64_t hip_stream);

/*
 * Between the two MoE GEMMs, one launch: act = silu(x[:, :I]) * x[:, I:], rounded to x's 16-bit type
 * (the reference's intermediate cache, src/tilegym/ops/moe_interface.py:206-210,272-277; silu_and_mul:
 * src/tilegym/ops/ops.py:172-193), then quantized 1 x 128 (all-zero group -> scale 1.0).  The reference
 * casts the activation to fp8 with an all-ones scale (moe_interface.py:279-288); this gives the second
 * GEMM a real a2_scale.  x (R, 2I) bf16/f16 contiguous, I % 8 == 0; q (R, I) e4m3fn; scales (R, ceil(I/128)) f32.
 */
int32_t tg_silu_mul_quant_1x128(const tg_tensor* q, const tg_tensor* scales, const tg_tensor* x,
                                int32_t device_id, uint64_t hip_stream);

/*
 * Top-k combine: out[t, :] = sum_j x[t, j, :] (fp32 sum, one rounding), src/tilegym/ops/moe_interface.py:308-321.
 * x (T, top_k, H) and out (T, H) bf16 or f16 (same type), contiguous, H % 8 == 0, 16-byte aligned.
 */
int32_t tg_moe_sum(const tg_tensor* out, const tg_tensor* x, int32_t device_id, uint64_t hip_stream);

/*
 * The FP8 MoE layer in one call: what src/tilegym/ops/moe_interface.py:116-322 (fused_experts_impl, use_fp8_w8a8) does
 * for one chunk of tokens, as the four launches tg_moe_align_quant_1x128 -> tg_fp8_moe_gemm_silu_quant -> tg_fp8_moe_gemm
 * (x routed weight) -> tg_moe_sum on the caller's stream, with every intermediate in `workspace`.  The results are the
 * bits the four calls give one by one; what the call saves is the host time of four bindings and nine allocations, which at
 * one to sixteen tokens is more than the kernels run.
 *   hidden (T, H) bf16 / f16, H % 128 == 0; w1 (E, 2I, H), w2 (E, H, I) e4m3fn with w1_scale (E, 2I/128, H/128) and
 *   w2_scale (E, H/128, ceil(I/128)) f32; topk_weights (T, k) f32 and topk_ids (T, k) int32 / int64, contiguous;
 *   out (T, H) of hidden's type.  E <= 512, 2I % 256 == 0, block_m 128 or 256 (the alignment block = the row tile of the
 *   grouped GEMMs); T * k + E * (block_m - 1) slots must fit int32.
 *   workspace: uint8, 256-byte aligned, at least tg_fp8_fused_moe_workspace_bytes(...) bytes; it needs no initialisation
 *   and holds nothing between calls.
 * Layers outside these limits (more tokens than one chunk, other intermediate sizes, fp8 activations with their own scales)
 * are run call by call, as the Python layer does.
 */
int64_t tg_fp8_fused_moe_workspace_bytes(int64_t tokens, int64_t top_k, int64_t experts, int64_t hidden, int64_t inter,
                                         int32_t block_m);
int32_t tg_fp8_fused_moe(const tg_tensor* out, const tg_tensor* hidden, const tg_tensor* w1, const tg_tensor* w2,
                         const tg_tensor* w1_scale, const tg_tensor* w2_scale, const tg_tensor* topk_weights,
                         const tg_tensor* topk_ids, const tg_tensor* workspace, int32_t block_m, int32_t device_id,
                         uint64_t hip_stream);

/* The schedule the most recent GEMM call on this host thread chose: fills out[0..n) with the
 * TG_CFG_* slots (kernel, BLOCK_M, BLOCK_N, SPLIT_K, ROW_GROUPS, WAVES).  Returns slots written. */
int32_t tg_last_config(int32_t* out, int32_t n);

/* Static message for a return code (src/tilegym/ops/cutile_rs/ffi_util.rs:125-135). */
const char* tg_rc_message(int32_t rc);

/* Detail text of the most recent error on this host thread ("" if none). */
const char* tg_last_error(void);

int32_t tg_abi_version(void);

/*
 * Yardsticks (no counterpart in the reference): kernels that compute nothing useful and exist so that the process that
 * times the GEMMs can also time, on the same GPU and in the same run, what bounds them.
 *
 * tg_diag_read: a plain read of all bytes of x (16-byte aligned; 16 bytes per lane, non-temporal, grid-stride over
 *   `workgroups` workgroups of 256 threads with `loads_in_flight` (1, 2, 4 or 8) loads per lane in flight; 0 = 2048 and 4):
 *   the floor for any kernel that has to read those bytes once.  out: int32, >= workgroups elements (scratch).
 * tg_diag_mfma: `workgroups` workgroups of eight waves issue iters x 32 e4m3 16x16x128 MFMAs per wave on non-zero register
 *   operands (65536 FLOP per MFMA and wave), with `fmas` (0, 2, 4, 6 or 8) scale-and-add FMAs behind every MFMA: the
 *   rate of the matrix pipe, and what is left of it when it shares the issue port with the block-scaled kernels' VALU
 *   work.  out: f32, >= workgroups * 512 elements (scratch).
 */
int32_t tg_diag_read(const tg_tensor* x, const tg_tensor* out, int32_t workgroups, int32_t loads_in_flight, int32_t device_id,
                     uint64_t hip_stream);
int32_t tg_diag_mfma(int32_t fmas, int32_t iters, int32_t workgroups, const tg_tensor* out, int32_t device_id, uint64_t hip_stream);

#ifdef __cplusplus
}
#endif
#endif /* TILEGYM_HIP_H */
