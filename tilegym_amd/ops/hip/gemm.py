""" "hip" implementations of the dense and grouped FP8 GEMM ops.  Each one validates like the
reference implementation it replaces, allocates the output with torch on the inputs' device,
and enqueues the HIP kernels on torch's current stream through the C ABI."""

from __future__ import annotations

import math
from typing import List, Optional, Sequence

import torch

from ... import _lib
from ...backend import register_impl

FP8 = torch.float8_e4m3fn
_OUT_DTYPES = (torch.bfloat16, torch.float16, torch.float32)


def _require_fp8(*tensors):
    for t in tensors:
        if t.dtype != FP8:
            raise NotImplementedError(
                f"the hip backend implements float8_e4m3fn GEMM only (got {t.dtype})")


def _split_scale(scale, alpha: float):
    """float scales fold into alpha; tensors are passed to the kernel (read on the device)."""
    if scale is None:
        return None, alpha
    if isinstance(scale, (int, float)):
        return None, alpha * float(scale)
    if not isinstance(scale, torch.Tensor):
        raise TypeError("scale must be a float or a tensor")
    s = scale
    if s.dtype != torch.float32:
        s = s.float()
    return s.contiguous(), alpha


@register_impl("matmul", backend="hip")
def matmul(a, b, trans_a=None, trans_b=None, static_persistent=None, use_tma=None, **kwargs):
    trans_a = bool(trans_a) if trans_a is not None else False
    trans_b = bool(trans_b) if trans_b is not None else False
    _require_fp8(a, b)
    if a.dim() != 2 or b.dim() != 2:
        raise ValueError("matmul expects 2-D operands")
    if trans_a:
        K, M = a.shape
    else:
        M, K = a.shape
    if trans_b:
        N, KB = b.shape
    else:
        KB, N = b.shape
    assert K == KB, f"Incompatible matrices: K dimension of A is {K}, K dimension of B is {KB}"
    assert a.is_contiguous() and b.is_contiguous(), "operands must be contiguous"

    out_dtype = kwargs.get("out_dtype")
    if out_dtype is None:
        # reference behaviour: result in a.dtype (src/tilegym/ops/cutile/matmul.py:446); the kernel's epilogue casts
        # (round to nearest even, saturating at +-448)
        out_dtype = torch.float8_e4m3fn
    if out_dtype not in _OUT_DTYPES and out_dtype != torch.float8_e4m3fn:
        raise NotImplementedError(f"out_dtype {out_dtype} not supported")
    sa, alpha = _split_scale(kwargs.get("scale_a"), float(kwargs.get("alpha", 1.0)))
    sb, alpha = _split_scale(kwargs.get("scale_b"), alpha)
    c = torch.empty((M, N), device=a.device, dtype=out_dtype)
    _lib.fp8_gemm(c, a, b, sa, sb, trans_a, trans_b, alpha, 0.0, kwargs.get("kernel_configs"))
    return c


@register_impl("flashinfer.gemm.gemm_alpha_beta", backend="hip")
def gemm_alpha_beta(a, b, c, trans_a=False, trans_b=True, alpha=1.0, beta=0.0, num_sms=None, **kwargs):
    """C <- alpha * A @ B(^T) + beta * C, in place
    (src/tilegym/suites/flashinfer/cutile/gemm/gemm_alpha_beta.py:336-504).  ``num_sms`` throttles
    the reference's persistent grid and has no meaning here; it is ignored."""
    _require_fp8(a, b)
    if trans_a:
        K, M = a.shape
    else:
        M, K = a.shape
    if trans_b:
        N, KB = b.shape
    else:
        KB, N = b.shape
    assert K == KB, "incompatible dimensions"
    assert c.shape == (M, N), "C must have shape [M, N]"
    assert a.is_contiguous(), "A matrix must be contiguous"
    assert b.is_contiguous(), "B matrix must be contiguous"
    assert c.is_contiguous(), "C matrix must be contiguous"
    if c.dtype not in _OUT_DTYPES:
        raise NotImplementedError(f"C dtype {c.dtype} not supported")
    _lib.fp8_gemm(c, a, b, None, None, bool(trans_a), bool(trans_b), float(alpha), float(beta),
                  kwargs.get("kernel_configs"))
    return c


@register_impl("unsloth.w8a8_block_fp8_matmul", backend="hip")
def w8a8_block_fp8_matmul(A, B, As, Bs, block_size: Optional[Sequence[int]] = None,
                          output_dtype: torch.dtype = torch.float32, **kwargs):
    """Block-scaled FP8 GEMM (src/tilegym/suites/unsloth/cutile/fp8.py:388-446)."""
    if block_size is None:
        block_n, block_k = 128, 128
    else:
        assert len(block_size) == 2
        block_n, block_k = block_size[0], block_size[1]
    if block_n <= 0 or block_k <= 0:
        raise ValueError(f"block_size must be positive, got {block_size}")
    _require_fp8(A, B)
    N, K = B.shape
    assert A.shape[-1] == B.shape[-1]
    assert A.shape[:-1] == As.shape[:-1] and A.is_contiguous()
    assert math.ceil(A.shape[-1] / block_k) == As.shape[-1]
    assert B.ndim == 2 and B.is_contiguous() and Bs.ndim == 2
    assert math.ceil(N / block_n) == Bs.shape[0]
    assert math.ceil(K / block_k) == Bs.shape[1]
    if output_dtype not in _OUT_DTYPES:
        raise NotImplementedError(f"output_dtype {output_dtype} not supported")
    M = A.numel() // A.shape[-1]
    C = A.new_empty(A.shape[:-1] + (N,), dtype=output_dtype)
    if M == 0:
        return C
    As2 = As.reshape(M, -1).float().contiguous()
    Bs2 = Bs.float().contiguous()
    kc = kwargs.get("kernel_configs")
    if (block_n, block_k) != (128, 128):
        # quantization blocks other than 128 x 128 run on the library's software-decode kernel (correct, no MFMA)
        kc = dict(kc or {}, QUANT_BLOCK_N=block_n, QUANT_BLOCK_K=block_k)
    _lib.fp8_gemm(C.view(M, N), A.view(M, K), B, As2, Bs2, False, True, 1.0, 0.0, kc)
    return C


@register_impl("flashinfer.gemm.ragged_block_scaled_bmm", backend="hip")
def ragged_block_scaled_bmm(a, b, a_scale, b_scale, m_indptr, max_m, max_m_device=None,
                            transpose_a=False, transpose_b=True, out_dtype=None, **kwargs):
    """Grouped block-scaled FP8 GEMM over expert segments
    (src/tilegym/suites/flashinfer/cutile/gemm/ragged_block_scaled_bmm.py:497-616).
    ``max_m`` / ``max_m_device`` bound the reference's uniform tile walk; the expert-offset
    launch here reads the segment sizes on the device, so both are accepted and unused."""
    assert transpose_a == False and transpose_b == True, "Only NT layout is supported"  # noqa: E712
    assert a.is_contiguous(), "A matrix must be contiguous"
    assert b.is_contiguous(), "B matrix must be contiguous"
    assert a_scale is None or a_scale.is_contiguous(), "A scale matrix must be contiguous"
    assert b_scale.is_contiguous(), "B scale matrix must be contiguous"
    assert m_indptr.is_contiguous(), "m_indptr must be contiguous"
    _require_fp8(a, b)
    total_m, K_A = a.shape
    Q, N, K_B = b.shape
    assert K_A == K_B, f"K dimensions must match: {K_A} != {K_B}"
    assert m_indptr.shape[0] == Q + 1, "m_indptr must have Q+1 elements"
    Q_SB, rnb, rkb = b_scale.shape
    # quantization blocks as the reference derives them (ragged_block_scaled_bmm.py:535-537): K elements per scale from the
    # scale tensor's shape; likewise the weight rows per scale
    # (a shape that 128 x 128 blocks explain is read as 128 x 128: ragged edges make the division ambiguous)
    if math.ceil(N / 128) == rnb and math.ceil(K_B / 128) == rkb:
        block_n, block_k = 128, 128
    else:
        block_k, block_n = K_B // rkb, -(-N // rnb)
    assert block_k > 0 and math.ceil(K_B / block_k) == rkb and math.ceil(N / block_n) == rnb, "b_scale shape does not tile (N, K)"
    kc = kwargs.get("kernel_configs")
    if (block_n, block_k) != (128, 128):
        # blocks other than 128 x 128 run on the library's software-decode kernel (correct, no MFMA)
        kc = dict(kc or {}, QUANT_BLOCK_N=block_n, QUANT_BLOCK_K=block_k)
    if a_scale is not None:
        assert a_scale.shape[0] == total_m, "a_scale total_m dimension mismatch"
    assert Q_SB == Q, "b_scale Q dimension mismatch"
    if out_dtype is None:
        out_dtype = torch.bfloat16
    if out_dtype not in _OUT_DTYPES:
        raise NotImplementedError(f"out_dtype {out_dtype} not supported")
    # rows past m_indptr[-1] belong to no segment and are left untouched by the kernel
    c = torch.zeros((total_m, N), device=a.device, dtype=out_dtype) if kwargs.get("zero_init") \
        else torch.empty((total_m, N), device=a.device, dtype=out_dtype)
    ptr = m_indptr if m_indptr.dtype == torch.int32 else m_indptr.to(torch.int32)
    a_s = None if a_scale is None else a_scale.float()
    _lib.fp8_ragged_gemm(c, a, b, a_s, b_scale.float(), ptr, kc)
    return c


@register_impl("group_gemm", backend="hip")
def group_gemm(group_A, group_B, static_persistent=True, use_tma=True, transpose_b=False, **kwargs):
    """List of GEMMs (src/tilegym/ops/cutile/group_gemm.py:170-197) through tg_fp8_group_gemm: one
    launch for (N,K) weights with K % 128 == 0, otherwise problem by problem; all on the current
    stream; outputs in ``A.dtype`` unless ``out_dtype`` is given.  ``scales_a`` / ``scales_b``:
    optional lists of per-tensor scales (one-element tensors, floats or None)."""
    if not group_A or not group_B:
        raise ValueError("group_A and group_B must not be empty")
    if len(group_A) != len(group_B):
        raise ValueError(f"group_A and group_B must have same length, got {len(group_A)} and {len(group_B)}")
    transpose_b = bool(transpose_b)
    out_dtype = kwargs.get("out_dtype")
    if out_dtype is None:
        out_dtype = torch.float8_e4m3fn  # A.dtype, cast in the kernels' epilogue (saturating, round to nearest even)
    if out_dtype not in _OUT_DTYPES and out_dtype != torch.float8_e4m3fn:
        raise NotImplementedError(f"out_dtype {out_dtype} not supported")
    dev = group_A[0].device
    if not group_A[0].is_cuda:
        raise RuntimeError("the hip backend works on device tensors only")
    outs = []
    for A, B in zip(group_A, group_B):
        _require_fp8(A, B)
        if A.dim() != 2 or B.dim() != 2:
            raise ValueError("group_gemm expects 2-D operands")
        N, KB = (B.shape if transpose_b else (B.shape[1], B.shape[0]))
        assert A.shape[1] == KB, f"Incompatible matrices: K dimension of A is {A.shape[1]}, K dimension of B is {KB}"
        assert A.is_contiguous() and B.is_contiguous(), "operands must be contiguous"
        outs.append(torch.empty((A.shape[0], N), device=dev, dtype=out_dtype))

    def as_tensors(scales):
        if scales is None:
            return None
        res = []
        for sc in scales:
            if sc is None:
                res.append(None)
            elif isinstance(sc, torch.Tensor):
                res.append(sc.reshape(-1)[:1].float().contiguous())
            else:
                res.append(torch.full((1,), float(sc), dtype=torch.float32, device=dev))
        return res

    _lib.fp8_group_gemm(outs, list(group_A), list(group_B), as_tensors(kwargs.get("scales_a")),
                        as_tensors(kwargs.get("scales_b")), transpose_b, kwargs.get("kernel_configs"))
    return outs
