"""CPU oracle for the FP8 (OCP e4m3fn) GEMM path: dequantize -> fp32 matmul -> cast.

TEST INFRASTRUCTURE ONLY -- the product never imports this module.  It is the
checker for the HIP kernels (tests, smoke) and the timed CPU baseline of the bench.

Every function restates, in plain torch/numpy on the CPU, the arithmetic that the
reference's own test oracles define for this path; the reference location each one
follows is cited in its docstring.  How each function is pinned (so that a dropped
term, a wrong index or a transposed operand fails a test) is listed here:

=============================  ==================================================
function                       pinned by (tests/test_oracle.py)
=============================  ==================================================
e4m3fn_decode_table            closed form of OCP FP8 E4M3 checked code by code
                               against torch's own uint8->float8_e4m3fn view
e4m3fn_encode_rne              brute force over a dense grid of floats against
                               torch's ``.to(float8_e4m3fn)`` after clamping
quantize_*                     scale*q round trip error bound, amax hits +-448,
                               all-zero block -> scale 1.0 (unsloth) / eps (flashinfer);
                               power-of-two scales against exponent-bit arithmetic;
                               groups of 16/32/64 against a per-group loop
weight_dequant                 element loop with ragged edge blocks
ref_gemm_per_tensor            integer-valued inputs whose product is exact in fp32
                               (compared with an int64 matmul), power-of-two scale
                               linearity, transposed-operand shapes (M != N != K)
ref_gemm_alpha_beta            alpha/beta linearity against ref_gemm_per_tensor
ref_w8a8_block_fp8_matmul      pure-Python triple loop on tiny inputs (block 128 and
                               ragged tails), all-equal scales == per-tensor
ref_ragged_block_scaled_bmm    Q=1 == dense; expert permutation permutes segments;
                               zero-row experts; per-expert loop of the dense oracle
moe_align_block_size_ref       the worked example in the reference docstring
                               (the only known-answer vector on this path)
ref_fused_moe_gemm             per-token Python loops on tiny inputs
=============================  ==================================================
"""

from __future__ import annotations

import math
from typing import List, Optional, Sequence, Tuple

import numpy as np
import torch

FP8_MAX = 448.0  # torch.finfo(torch.float8_e4m3fn).max
FP8 = torch.float8_e4m3fn


# ----------------------------------------------------------------------------
# e4m3fn codec (closed form)
# ----------------------------------------------------------------------------
def e4m3fn_decode_table() -> np.ndarray:
    """All 256 e4m3fn codes as float32.

    OCP 8-bit float, 1-4-3, bias 7, no infinities, NaN = S.1111.111, max 448,
    subnormals k * 2**-9.  The reference keeps this format end to end as
    ``torch.float8_e4m3fn`` (tests/suites/unsloth/test_fp8.py:216-218).
    """
    out = np.empty(256, dtype=np.float32)
    for code in range(256):
        sign = -1.0 if code & 0x80 else 1.0
        exp = (code >> 3) & 0xF
        man = code & 0x7
        if exp == 0xF and man == 0x7:
            val = float("nan")
        elif exp == 0:
            val = sign * man * 2.0 ** (-9)
        else:
            val = sign * (1.0 + man / 8.0) * 2.0 ** (exp - 7)
        out[code] = val
    return out


def e4m3fn_encode_rne(x: np.ndarray) -> np.ndarray:
    """Round-to-nearest-even float32 -> e4m3fn code for inputs already clamped to
    [-448, 448] (every quantizer of the reference clamps first:
    src/tilegym/suites/unsloth/cutile/fp8.py:115,
    src/tilegym/suites/flashinfer/cutile/per_token_group_quant_8bit.py:63)."""
    x = np.asarray(x, dtype=np.float32)
    sign = (np.signbit(x)).astype(np.uint8) << 7
    a = np.abs(x).astype(np.float64)
    # quantum: 2**-9 below 2**-6, else 2**(floor(log2 a) - 3)
    with np.errstate(divide="ignore"):
        e = np.floor(np.log2(np.where(a > 0, a, 1.0)))
    e = np.clip(e, -6, 8)
    q = 2.0 ** (e - 3)
    k = np.rint(a / q)  # numpy rint == round half to even
    v = k * q
    # re-derive exponent/mantissa of the rounded value
    with np.errstate(divide="ignore"):
        e2 = np.floor(np.log2(np.where(v > 0, v, 1.0)))
    e2 = np.clip(e2, -6, 8)
    is_sub = v < 2.0**-6
    man = np.where(is_sub, v / 2.0**-9, (v / 2.0**e2 - 1.0) * 8.0)
    expf = np.where(is_sub, 0, e2 + 7)
    code = (expf.astype(np.int64) << 3) | np.rint(man).astype(np.int64)
    return (code.astype(np.uint8) | sign).astype(np.uint8)


def fp8_bytes(t: torch.Tensor) -> np.ndarray:
    """Raw codes of an e4m3fn tensor."""
    return t.contiguous().view(torch.uint8).numpy()


def fp8_to_f32(t: torch.Tensor) -> torch.Tensor:
    """Decode through the closed-form table (not through torch's cast)."""
    tab = torch.from_numpy(e4m3fn_decode_table())
    return tab[t.contiguous().view(torch.uint8).long()]


# ----------------------------------------------------------------------------
# quantizers
# ----------------------------------------------------------------------------
def quantize_per_tensor(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """scale = amax/448, q = clamp(x/scale, +-448) -> e4m3fn (one fp32 scale).

    Same rule as the reference's block quantizer applied to the whole tensor
    (src/tilegym/suites/unsloth/cutile/fp8.py:105-116)."""
    xf = x.float()
    amax = xf.abs().max()
    scale = torch.where(amax == 0, torch.ones_like(amax), amax / FP8_MAX)
    q = (xf / scale).clamp(-FP8_MAX, FP8_MAX).to(FP8)
    return q, scale.reshape(1)


def quantize_act_1x128(x: torch.Tensor, block: int = 128, eps: Optional[float] = None, ue8m0: bool = False,
                       dst_dtype: torch.dtype = FP8):
    """Per-token 1 x ``block`` quantization; returns (q, scales[..., K/block]).  ``dst_dtype=torch.int8``: the
    integer destination of the flashinfer operator (same test oracle, :52-57): range [-128, 127], scale = amax / 127,
    the quotient converted by torch's float -> int8 cast (toward zero).

    ``eps=None``: the unsloth rule, all-zero block -> scale 1.0
    (tests/suites/unsloth/test_fp8.py:80-97, src/.../unsloth/cutile/fp8.py:105-116).
    ``eps=1e-10``: the flashinfer rule, amax clamped below by eps
    (tests/suites/flashinfer/test_per_token_group_quant_8bit.py:41-68); with ``ue8m0`` the scale is then
    rounded up to a power of two, ``2^ceil(log2(max(|s|, 1e-10)))`` (same file, :61-63)."""
    assert x.shape[-1] % block == 0
    qmin, qmax = (-128.0, 127.0) if dst_dtype == torch.int8 else (-FP8_MAX, FP8_MAX)
    xb = x.float().reshape(-1, block)
    amax = xb.abs().amax(dim=-1, keepdim=True)
    if eps is None:
        assert not ue8m0
        s = amax / qmax
        s = torch.where(s == 0, torch.ones_like(s), s)
    else:
        s = amax.clamp(min=eps) / qmax
        if ue8m0:
            s = torch.exp2(torch.ceil(torch.log2(torch.maximum(s.abs(), torch.tensor(1e-10)))))
    q = (xb / s).clamp(qmin, qmax).to(dst_dtype).reshape(x.shape)
    return q, s.reshape(*x.shape[:-1], x.shape[-1] // block)


def quantize_weight_128x128(w: torch.Tensor, block_n: int = 128, block_k: int = 128):
    """Per (block_n x block_k) block quantization of a (N, K) weight; the layout
    ``Bs (ceil(N/bn), ceil(K/bk))`` is the one the block-scaled GEMM consumes
    (src/tilegym/suites/unsloth/ops.py:254-256); ragged edge blocks allowed."""
    N, K = w.shape
    nb, kb = -(-N // block_n), -(-K // block_k)
    wp = torch.zeros(nb * block_n, kb * block_k, dtype=torch.float32)
    wp[:N, :K] = w.float()
    blocks = wp.reshape(nb, block_n, kb, block_k)
    amax = blocks.abs().amax(dim=(1, 3))
    s = torch.where(amax == 0, torch.ones_like(amax), amax / FP8_MAX)
    q = (blocks / s[:, None, :, None]).clamp(-FP8_MAX, FP8_MAX)
    q = q.reshape(nb * block_n, kb * block_k)[:N, :K].contiguous().to(FP8)
    return q, s


def weight_dequant(x: torch.Tensor, s: torch.Tensor, block_size: int = 128,
                   dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    """y = fp8(x) * s[i // bs, j // bs]  (src/tilegym/suites/unsloth/cutile/fp8.py:36-71)."""
    M, N = x.shape
    se = s.repeat_interleave(block_size, 0)[:M].repeat_interleave(block_size, 1)[:, :N]
    return (fp8_to_f32(x) * se).to(dtype)


# ----------------------------------------------------------------------------
# GEMM oracles
# ----------------------------------------------------------------------------
def _as_scalar(s) -> torch.Tensor:
    if s is None:
        return torch.ones((), dtype=torch.float32)
    if isinstance(s, torch.Tensor):
        return s.float().reshape(())
    return torch.tensor(float(s), dtype=torch.float32)


def cast_output(acc: torch.Tensor, out_dtype, saturate: bool = True) -> torch.Tensor:
    """The one stated rule for a GEMM's output cast.  16- and 32-bit types: torch's cast (nearest even).  e4m3: nearest
    even after clamping to +-448 when ``saturate`` (what the HIP epilogues do); ``saturate=False`` is torch's plain cast,
    which gives NaN from about 465 up -- what the reference gets when it casts an fp32 result with ``.to(float8_e4m3fn)``
    (src/tilegym/ops/cutile/matmul.py:446).  The reference's own tests keep results in range, where the two agree; beyond
    the range parity with the reference is unpinned."""
    if out_dtype == FP8 and saturate:
        return acc.float().clamp(-FP8_MAX, FP8_MAX).to(FP8)
    return acc.to(out_dtype)


def ref_gemm_per_tensor(a, b, scale_a=None, scale_b=None, trans_a=False, trans_b=False,
                        out_dtype=torch.bfloat16) -> torch.Tensor:
    """(dequant(a) @ dequant(b)) in fp32 -> out_dtype.

    Shapes follow ``tilegym.ops.matmul`` (src/tilegym/ops/cutile/matmul.py:435-443):
    a is (M,K) or (K,M) when trans_a; b is (K,N) or (N,K) when trans_b."""
    af = fp8_to_f32(a) if a.dtype == FP8 else a.float()
    bf = fp8_to_f32(b) if b.dtype == FP8 else b.float()
    if trans_a:
        af = af.t()
    if trans_b:
        bf = bf.t()
    af = af * _as_scalar(scale_a)
    bf = bf * _as_scalar(scale_b)
    return cast_output(af @ bf, out_dtype)


def ref_gemm_alpha_beta(a, b, c, trans_a=False, trans_b=True, alpha=1.0, beta=0.0) -> torch.Tensor:
    """c <- alpha * (a @ b) + beta * float(c), cast to c.dtype, fp32 accumulation:
    the epilogue of src/tilegym/suites/flashinfer/cutile/gemm/gemm_alpha_beta.py:161-180
    (the reference *test* multiplies in bf16, test_flashinfer_gemm_alpha_beta.py:17-22;
    the kernel accumulates in fp32, which is what is restated here)."""
    acc = ref_gemm_per_tensor(a, b, None, None, trans_a, trans_b, out_dtype=torch.float32)
    return cast_output(alpha * acc + beta * c.float(), c.dtype)


def expand_block_scales(As: torch.Tensor, Bs: torch.Tensor, N: int, K: int,
                        block_n: int, block_k: int):
    """As (M, kb) -> (M, K); Bs (nb, kb) -> (N, K)."""
    a_e = As.float().repeat_interleave(block_k, dim=1)[:, :K]
    b_e = Bs.float().repeat_interleave(block_n, dim=0)[:N].repeat_interleave(block_k, dim=1)[:, :K]
    return a_e, b_e


def ref_w8a8_block_fp8_matmul(A, B, As, Bs, block_size: Optional[Sequence[int]] = None,
                              output_dtype=torch.float32) -> torch.Tensor:
    """Block-scaled GEMM oracle: dequantize both operands block-wise, ``A_deq @ B_deq.T``.

    Restates Test_Unsloth_W8A8_FP8_Matmul.reference
    (tests/suites/unsloth/test_fp8.py:159-191) with the per-element Python loops
    replaced by repeat_interleave (the loops are kept in tests/ as the pin)."""
    block_n, block_k = (128, 128) if block_size is None else block_size
    N, K = B.shape
    lead = A.shape[:-1]
    A2 = A.reshape(-1, K)
    a_e, b_e = expand_block_scales(As.reshape(A2.shape[0], -1), Bs, N, K, block_n, block_k)
    A_deq = fp8_to_f32(A2) * a_e
    B_deq = fp8_to_f32(B) * b_e
    return (A_deq @ B_deq.t()).to(output_dtype).reshape(*lead, N)


def ref_ragged_block_scaled_bmm(a, b, a_scale, b_scale, m_indptr, block_n=128, block_k=128,
                                out_dtype=torch.bfloat16) -> torch.Tensor:
    """Grouped block-scaled GEMM: rows [m_indptr[q], m_indptr[q+1]) of ``a`` times
    ``b[q].T``; restates Test_FlashInfer_RaggedBlockScaledBMM.reference
    (tests/suites/flashinfer/test_flashinfer_ragged_block_scaled_bmm.py:77-136).
    Unlike that test, empty segments are allowed (they write nothing) and rows past
    m_indptr[-1] stay zero.  ``a_scale=None`` means all-ones activation scales
    (ragged_block_scaled_bmm.py:124-131 HAS_A_SCALE)."""
    total_m, K = a.shape
    Q, N, Kb = b.shape
    assert K == Kb
    c = torch.zeros((total_m, N), dtype=out_dtype)
    ptr = [int(v) for v in m_indptr.tolist()]
    for q in range(Q):
        lo, hi = ptr[q], ptr[q + 1]
        if hi <= lo:
            continue
        a_s = a_scale[lo:hi] if a_scale is not None else torch.ones(hi - lo, -(-K // block_k))
        c[lo:hi] = ref_w8a8_block_fp8_matmul(a[lo:hi], b[q], a_s, b_scale[q],
                                             [block_n, block_k], out_dtype)
    return c


def ref_group_gemm(group_A: List[torch.Tensor], group_B: List[torch.Tensor], transpose_b=False,
                   scales_a=None, scales_b=None, out_dtype=None) -> List[torch.Tensor]:
    """List of independent GEMMs (src/tilegym/ops/cutile/group_gemm.py:170-197;
    oracle tests/ops/test_group_gemm.py:16-27: fp32 ``a @ b`` cast back)."""
    outs = []
    for i, (A, B) in enumerate(zip(group_A, group_B)):
        sa = None if scales_a is None else scales_a[i]
        sb = None if scales_b is None else scales_b[i]
        od = out_dtype or A.dtype
        acc = ref_gemm_per_tensor(A, B, sa, sb, False, transpose_b, out_dtype=torch.float32)
        outs.append(cast_output(acc, od))
    return outs


# ----------------------------------------------------------------------------
# MoE: alignment and token-gather GEMM
# ----------------------------------------------------------------------------
def moe_align_block_size_ref(topk_ids: torch.Tensor, block_size: int, num_experts: int):
    """Sort flat (token, k) slots by expert (stable), pad each expert to a multiple of
    ``block_size`` with the sentinel ``numel``.

    Restates moe_align_block_size_torch (src/tilegym/ops/moe_interface.py:30-79), with
    the buffer sizes of the device version (worst-case, data-independent:
    src/tilegym/ops/cutile/moe_align_block.py:252-268).  Returns
    (sorted_ids[numel + E*(bs-1)], expert_ids[ceil(that/bs)], num_tokens_post_pad[1],
    cumsum[E+1] of padded counts, max_expert_cnt[1])."""
    flat = topk_ids.reshape(-1).to(torch.int64)
    numel = flat.numel()
    max_padded = numel + num_experts * (block_size - 1)
    sorted_ids = torch.full((max_padded,), numel, dtype=torch.int32)
    expert_ids = torch.zeros((-(-max_padded // block_size),), dtype=torch.int32)
    order = torch.argsort(flat, stable=True)
    counts = torch.bincount(flat, minlength=num_experts)
    cumsum = torch.zeros(num_experts + 1, dtype=torch.int32)
    tok = 0
    blk = 0
    for e in range(num_experts):
        n = int(counts[e])
        nb = -(-n // block_size)
        expert_ids[blk:blk + nb] = e
        sorted_ids[blk * block_size: blk * block_size + n] = order[tok:tok + n].to(torch.int32)
        tok += n
        blk += nb
        cumsum[e + 1] = blk * block_size
    post = torch.tensor([blk * block_size], dtype=torch.int32)
    mx = torch.tensor([int(counts.max()) if numel else 0], dtype=torch.int32)
    return sorted_ids, expert_ids, post, cumsum, mx


def ref_fused_moe_gemm(A, B, A_scale, B_scale, topk_weights, topk_ids, mul_routed_weight,
                       top_k, block_shape=(128, 128), out_dtype=torch.bfloat16) -> torch.Tensor:
    """Token-gather MoE GEMM: C[t, j] = dequant(A[(t*topk+j)//top_k]) @ dequant(B[topk_ids[t, j]]).T
    (optionally times topk_weights[t, j]); returns C (T, topk, N).

    Follows the contract of invoke_fused_moe_kernel's FP8 branch
    (src/tilegym/ops/tilecpp/moe.cuh:163-207) and fused_moe_torch
    (src/tilegym/ops/moe_interface.py:82-113).  That branch is exercised by no test of the
    reference: PARITY UNPINNED against the reference there; pinned here against
    per-token Python loops only."""
    E, N, K = B.shape
    T_slots = topk_ids.numel()
    bn, bk = block_shape
    C = torch.zeros(T_slots, N, dtype=torch.float32)
    flat_e = topk_ids.reshape(-1).tolist()
    wts = topk_weights.reshape(-1).float() if topk_weights is not None else None
    for slot in range(T_slots):
        e = flat_e[slot]
        row = slot // top_k
        a_s = A_scale[row:row + 1] if A_scale is not None else torch.ones(1, -(-K // bk))
        b_s = B_scale[e] if B_scale is not None else torch.ones(-(-N // bn), -(-K // bk))
        out = ref_w8a8_block_fp8_matmul(A[row:row + 1], B[e], a_s, b_s, [bn, bk], torch.float32)
        if mul_routed_weight:
            out = out * wts[slot]
        C[slot] = out[0]
    return C.to(out_dtype).reshape(*topk_ids.shape, N)


# ----------------------------------------------------------------------------
# comparison (tolerance "relative to output scale")
# ----------------------------------------------------------------------------
def ref_silu_mul_quant(x: torch.Tensor):
    """act = silu(x[:, :I]) * x[:, I:] in fp32, rounded to x's dtype (the reference's intermediate
    cache, src/tilegym/ops/moe_interface.py:206-210,272-277; silu_and_mul: src/tilegym/ops/ops.py:172-193),
    then 1 x 128 quantization with a possibly partial last group."""
    inter = x.shape[1] // 2
    g, u = x[:, :inter].float(), x[:, inter:].float()
    act = ((g / (1.0 + torch.exp(-g))) * u).to(x.dtype)
    pad = (-inter) % 128
    ap = torch.nn.functional.pad(act.float(), (0, pad))
    q, s = quantize_act_1x128(ap, 128, None)
    return q[:, :inter].contiguous(), s, act


def ref_fused_experts_fp8(hidden, w1, w2, w1_scale, w2_scale, topk_weights, topk_ids, a1_scale=None):
    """The FP8 MoE layer token by token: quantize -> block-scaled GEMM with the token's experts ->
    silu * up -> re-quantize -> block-scaled GEMM x routed weight -> fp32 sum over the slots.
    Order of operations of src/tilegym/ops/moe_interface.py:230-321 and of the torch MoE oracle
    (tests/ops/test_moe.py:19-66); the FP8 branch itself is covered by no reference test
    (PARITY UNPINNED against the reference; pinned here by being a composition of the pinned
    per-op oracles above)."""
    T, H = hidden.shape
    k = topk_ids.shape[1]
    out_dtype = torch.bfloat16 if hidden.dtype == torch.bfloat16 else torch.float16
    if hidden.dtype == FP8:
        xq, xs = hidden, a1_scale
    else:
        xq, xs = quantize_act_1x128(hidden, 128, None)
    h1 = ref_fused_moe_gemm(xq, w1, xs, w1_scale, topk_weights, topk_ids, False, k, out_dtype=out_dtype)
    q2, s2, _ = ref_silu_mul_quant(h1.reshape(T * k, -1))
    h2 = ref_fused_moe_gemm(q2, w2, s2, w2_scale, topk_weights, topk_ids, True, 1, out_dtype=out_dtype)
    return h2.reshape(T, k, H).float().sum(dim=1).to(out_dtype)


def compare_to_oracle(out: torch.Tensor, ref: torch.Tensor, rtol=2e-2, atol=2e-2):
    """|out - ref| <= atol*sigma_ref + rtol*|ref|, sigma_ref = std of the oracle output.
    Returns (ok, report) with the fields the reference's compare_tensors prints
    (tests/common.py:807-820): max abs, max rel, fraction matched."""
    o = out.detach().float().cpu()
    r = ref.detach().float().cpu()
    assert o.shape == r.shape, f"shape {tuple(o.shape)} vs {tuple(r.shape)}"
    sigma = float(r.std()) if r.numel() > 1 else float(r.abs().max())
    if not math.isfinite(sigma) or sigma == 0.0:
        sigma = 1.0
    err = (o - r).abs()
    bound = atol * sigma + rtol * r.abs()
    okmask = err <= bound
    # NaN never matches
    okmask &= ~torch.isnan(o)
    rep = {
        "max_abs": float(err.max()) if err.numel() else 0.0,
        "max_rel_to_sigma": float(err.max() / sigma) if err.numel() else 0.0,
        "matched": float(okmask.float().mean()) if err.numel() else 1.0,
        "sigma": sigma,
    }
    return bool(okmask.all()), rep
