"""Seeded synthetic workloads: the five FP8 GEMM configurations the benchmark and the parity
tests run.  Inputs are drawn on the CPU with ``torch.Generator().manual_seed(seed)`` in fp32 and
quantized on the CPU by the small generators below; callers move them to the device.

LLAMA_SHAPES are the Llama-3.1-8B projection shapes (N, K): QKV, O, gate+up, down.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Tuple

import torch

FP8 = torch.float8_e4m3fn
FP8_MAX = 448.0

LLAMA_SHAPES: Dict[str, Tuple[int, int]] = {
    "qkv": (6144, 4096),
    "o": (4096, 4096),
    "gate_up": (28672, 4096),
    "down": (4096, 14336),
}
DECODE_M = (1, 8, 16, 64)
PREFILL_M = 8192
BLOCK_SCALED_SHAPES = ((12288, 5120), (5120, 12288))
BLOCK_SCALED_M = (16, 4096)
MOE = dict(hidden=2048, inter=1408, experts=64, top_k=6, tokens=4096)


# ---- host-side input generators: fp32 -> e4m3 codes and scales, plain torch on the CPU.  They only make the
# ---- synthetic operands below; the operators of this package run on the device through the HIP library.
def _quantize_per_tensor(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """One fp32 scale for the whole tensor: scale = amax/448 (1.0 for an all-zero tensor)."""
    xf = x.float()
    amax = xf.abs().amax()
    scale = torch.where(amax == 0, torch.ones_like(amax), amax / FP8_MAX)
    q = (xf / scale).clamp(-FP8_MAX, FP8_MAX).to(FP8)
    return q, scale.reshape(1)


def _quantize_1x128(x: torch.Tensor, eps: float = 1e-10) -> Tuple[torch.Tensor, torch.Tensor]:
    """Per (row, 128-group) scale max(amax, eps)/448, row-major scales (..., K/128)."""
    xb = x.float().reshape(-1, 128)
    s = xb.abs().amax(dim=-1, keepdim=True).clamp(min=eps) / FP8_MAX
    q = (xb / s).clamp(-FP8_MAX, FP8_MAX).to(FP8).reshape(x.shape)
    return q, s.reshape(*x.shape[:-1], x.shape[-1] // 128)


def _quantize_weight_128x128(w: torch.Tensor, block_n: int = 128, block_k: int = 128):
    """Per (block_n x block_k) block quantization of a (N, K) weight -> (q, Bs (ceil(N/bn), ceil(K/bk)))."""
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


@dataclass
class DenseCase:
    name: str
    a: torch.Tensor                      # (M,K) e4m3
    b: torch.Tensor                      # (N,K) e4m3  (or (K,N) when not trans_b)
    scale_a: torch.Tensor                # per-tensor (1,) or block (M, K/128)
    scale_b: torch.Tensor                # per-tensor (1,) or block (N/128, K/128)
    trans_b: bool = True
    block_scaled: bool = False

    @property
    def M(self): return self.a.shape[0]
    @property
    def K(self): return self.a.shape[1]
    @property
    def N(self): return self.b.shape[0] if self.trans_b else self.b.shape[1]

    def flops(self) -> float:
        return 2.0 * self.M * self.N * self.K

    def algorithmic_bytes(self) -> float:
        """A, B and C once each plus the scale tensors (tests/benchmark/suites/unsloth/bench_fp8.py:80-82)."""
        return (self.M * self.K + self.N * self.K + 2 * self.M * self.N
                + 4 * self.scale_a.numel() + 4 * self.scale_b.numel())

    def to(self, device):
        return DenseCase(self.name, self.a.to(device), self.b.to(device), self.scale_a.to(device),
                         self.scale_b.to(device), self.trans_b, self.block_scaled)


@dataclass
class GroupedCase:
    name: str
    a: torch.Tensor            # (total_m, K) e4m3, rows sorted by expert
    b: torch.Tensor            # (E, N, K) e4m3
    a_scale: torch.Tensor      # (total_m, K/128)
    b_scale: torch.Tensor      # (E, N/128, K/128)
    m_indptr: torch.Tensor     # (E+1,) int32
    extra: dict = field(default_factory=dict)

    def flops(self) -> float:
        rows = int(self.m_indptr[-1])
        return 2.0 * rows * self.b.shape[1] * self.b.shape[2]

    def algorithmic_bytes(self) -> float:
        rows = int(self.m_indptr[-1])
        E, N, K = self.b.shape
        return rows * K + E * N * K + 2 * rows * N + 4 * self.a_scale.numel() + 4 * self.b_scale.numel()

    def to(self, device):
        return GroupedCase(self.name, self.a.to(device), self.b.to(device), self.a_scale.to(device),
                           self.b_scale.to(device), self.m_indptr.to(device), self.extra)


def _gen(seed: int) -> torch.Generator:
    return torch.Generator().manual_seed(seed)


def per_tensor_case(M: int, N: int, K: int, seed: int = 0, w_std: float = 1.0, outliers: bool = False,
                    trans_b: bool = True, name: Optional[str] = None) -> DenseCase:
    """Activations N(0,1) (optionally 0.1% of entries x20), weights N(0, w_std), amax/448 scales."""
    g = _gen(seed)
    a = torch.randn(M, K, generator=g)
    if outliers:
        mask = torch.rand(M, K, generator=g) < 1e-3
        a = torch.where(mask, a * 20.0, a)
    w = torch.randn(N, K, generator=g) * w_std
    qa, sa = _quantize_per_tensor(a)
    qb, sb = _quantize_per_tensor(w)
    if not trans_b:
        qb = qb.view(torch.uint8).t().contiguous().view(torch.float8_e4m3fn)
    return DenseCase(name or f"pt_{M}x{N}x{K}", qa, qb, sa, sb, trans_b, False)


def config1(seed: int = 0, trans_b: bool = True) -> DenseCase:
    """A[256x4096], B[4096x4096] ~ N(0,1), per-tensor scales."""
    return per_tensor_case(256, 4096, 4096, seed, 1.0, False, trans_b, "c1_256x4096x4096")


def llama_decode_case(M: int, proj: str, seed: int = 0) -> DenseCase:
    N, K = LLAMA_SHAPES[proj]
    return per_tensor_case(M, N, K, seed, 0.02, False, True, f"c2_decode_{proj}_M{M}")


def llama_prefill_case(proj: str, M: int = PREFILL_M, seed: int = 0) -> DenseCase:
    N, K = LLAMA_SHAPES[proj]
    return per_tensor_case(M, N, K, seed, 0.02, True, True, f"c3_prefill_{proj}_M{M}")


def _block_weights(N: int, K: int, g: torch.Generator) -> torch.Tensor:
    """N(0,0.02) weights whose 128x128 blocks have magnitudes varied log-uniformly over 1e-3..1e-1."""
    w = torch.randn(N, K, generator=g) * 0.02
    nb, kb = -(-N // 128), -(-K // 128)
    mag = 10.0 ** (torch.rand(nb, kb, generator=g) * 2.0 - 3.0)
    mag = mag.repeat_interleave(128, 0)[:N].repeat_interleave(128, 1)[:, :K]
    return w * (mag / 0.02)


def block_scaled_case(M: int, N: int, K: int, seed: int = 0, name: Optional[str] = None) -> DenseCase:
    """DeepSeek-style: per-token 1x128 activation scales, 128x128 weight block scales."""
    g = _gen(seed)
    a = torch.randn(M, K, generator=g)
    w = _block_weights(N, K, g)
    qa, sa = _quantize_1x128(a)
    qb, sb = _quantize_weight_128x128(w)
    return DenseCase(name or f"c4_block_{M}x{N}x{K}", qa, qb, sa, sb, True, True)


def moe_routing(tokens: int, experts: int, top_k: int, seed: int = 0):
    """softmax of N(0,1) router logits -> top-k -> (topk_weights, topk_ids)."""
    g = _gen(seed + 1000)
    logits = torch.randn(tokens, experts, generator=g)
    probs = torch.softmax(logits, dim=-1)
    w, ids = torch.topk(probs, top_k, dim=-1)
    w = w / w.sum(dim=-1, keepdim=True)
    return w.float(), ids.to(torch.int32)


def moe_grouped_case(which: str = "gate_up", seed: int = 0, tokens: Optional[int] = None,
                     experts: Optional[int] = None, hidden: Optional[int] = None,
                     inter: Optional[int] = None, top_k: Optional[int] = None) -> GroupedCase:
    """DeepSeek-V2-Lite MoE GEMMs as expert-sorted ragged problems.

    gate_up: A = routed copies of the token activations (24576 x 2048), B (64, 2816, 2048).
    down:    A = N(0,1) stand-in for silu(g)*u (24576 x 1408), B (64, 2048, 1408)."""
    T = tokens or MOE["tokens"]; E = experts or MOE["experts"]; H = hidden or MOE["hidden"]
    I = inter or MOE["inter"]; k = top_k or MOE["top_k"]
    g = _gen(seed)
    tw, ids = moe_routing(T, E, k, seed)
    flat = ids.reshape(-1).long()
    order = torch.argsort(flat, stable=True)
    counts = torch.bincount(flat, minlength=E)
    indptr = torch.zeros(E + 1, dtype=torch.int32)
    indptr[1:] = torch.cumsum(counts, 0).to(torch.int32)
    if which == "gate_up":
        x = torch.randn(T, H, generator=g)
        a = x[order // k]
        N, K = 2 * I, H
    else:
        a = torch.randn(T * k, I, generator=g)
        N, K = H, I
    qa, sa = _quantize_1x128(a.contiguous())
    qb = torch.empty(E, N, K, dtype=torch.float8_e4m3fn)
    sb = torch.empty(E, -(-N // 128), -(-K // 128))
    for e in range(E):
        q, s = _quantize_weight_128x128(_block_weights(N, K, g))
        qb[e], sb[e] = q, s
    return GroupedCase(f"c5_moe_{which}", qa, qb, sa, sb, indptr,
                       {"topk_ids": ids, "topk_weights": tw, "order": order, "top_k": k})


def moe_decode_case(base: GroupedCase, tokens: int) -> GroupedCase:
    """The weights of a full-size grouped case with only `tokens` tokens routed over them (top-k of softmax(N(0,1))
    logits, seed = tokens), expert-sorted: the decode regime of the same layer, where most experts receive no row."""
    E, _, K = base.b.shape
    k = base.extra["top_k"]
    tw, ids = moe_routing(tokens, E, k, seed=tokens)
    flat = ids.reshape(-1).long()
    order = torch.argsort(flat, stable=True)
    counts = torch.bincount(flat, minlength=E)
    indptr = torch.zeros(E + 1, dtype=torch.int32)
    indptr[1:] = torch.cumsum(counts, 0).to(torch.int32)
    a = torch.randn(tokens * k, K, generator=_gen(tokens))
    qa, sa = _quantize_1x128(a)
    return GroupedCase(f"{base.name}_T{tokens}", qa, base.b, sa, base.b_scale, indptr,
                       {"topk_ids": ids, "topk_weights": tw, "order": order, "top_k": k})
