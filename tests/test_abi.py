"""CPU-side checks of the C-ABI library: it loads, exports every symbol the header declares,
and validates arguments before touching a device (no compute calls here)."""

import ctypes
import os
import re

import pytest
import torch

from tilegym_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
FP8 = torch.float8_e4m3fn


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "tilegym_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(tg_[a-z0-9_]+)\s*\(", text)))


def test_library_loads_and_exports_every_declared_symbol():
    L = _lib.load()
    names = _declared_symbols()
    assert {"tg_fp8_gemm", "tg_fp8_ragged_gemm", "tg_fp8_moe_gemm", "tg_fp8_gemm_workspace_bytes",
            "tg_rc_message", "tg_abi_version", "tg_last_config", "tg_last_error"} <= set(names)
    for n in names:
        assert hasattr(L, n), f"{n} declared in include/tilegym_hip.h but not exported"
    assert L.tg_abi_version() == 1


def test_rc_messages():
    L = _lib.load()
    want = {0: b"ok", -2: b"unsupported dtype", -3: b"kernel launch failed", -4: b"device init failed",
            -5: b"null tensor pointer", -6: b"invalid arguments", -99: b"unknown error"}
    for rc, msg in want.items():
        assert L.tg_rc_message(rc) == msg


def test_tensor_desc_layout_matches_header():
    # ptr u64, ndim i32 (+pad), shape i64[5], strides i64[5], dtype i32 (+pad)
    assert ctypes.sizeof(_lib.TgTensor) == 8 + 8 + 40 + 40 + 8
    t = torch.zeros(3, 5, dtype=torch.bfloat16)[:, ::2]
    d = _lib.make_tensor_desc(t)
    assert d.ndim == 2 and list(d.shape[:2]) == [3, 3] and list(d.strides[:2]) == [5, 2]
    assert d.dtype == 2 and d.ptr == t.data_ptr()
    assert _lib.make_tensor_desc(torch.zeros(1).to(FP8)).dtype == 7
    assert _lib.make_tensor_desc(None) is None


def _call_gemm(c, a, b, sa=None, sb=None, ta=0, tb=1, ws=None):
    L = _lib.load()
    ds = [_lib.make_tensor_desc(t) for t in (c, a, b, sa, sb)]
    dws = _lib.make_tensor_desc(ws)
    cfg, n = _lib.make_cfg(None)
    refs = [None if d is None else ctypes.byref(d) for d in ds]
    rc = L.tg_fp8_gemm(*refs, ta, tb, 1.0, 0.0, None if dws is None else ctypes.byref(dws), cfg, n, 0, 0)
    return rc, L.tg_last_error().decode()


def test_gemm_argument_validation_runs_without_a_device():
    a = torch.zeros(4, 128).to(FP8)
    b = torch.zeros(8, 128).to(FP8)
    c = torch.zeros(4, 8, dtype=torch.bfloat16)
    L = _lib.load()
    cfg, n = _lib.make_cfg(None)
    dc, da = _lib.make_tensor_desc(c), _lib.make_tensor_desc(a)
    assert L.tg_fp8_gemm(ctypes.byref(dc), ctypes.byref(da), None, None, None, 0, 1, 1.0, 0.0, None, cfg, n, 0, 0) == -5
    assert _call_gemm(c, a.float(), b)[0] == -2                              # A not fp8
    assert _call_gemm(c.to(torch.int32), a, b)[0] == -2                      # C dtype
    rc, msg = _call_gemm(c, a, torch.zeros(8, 64).to(FP8))
    assert rc == -6 and "K of a is 128" in msg                               # mismatched K
    assert _call_gemm(torch.zeros(4, 9, dtype=torch.bfloat16), a, b)[0] == -6  # C shape
    assert _call_gemm(c, a, b, sa=torch.ones(3))[0] == -6                    # bad scale shape
    assert _call_gemm(c, a, b, sa=torch.ones(1, dtype=torch.float16))[0] == -2
    assert _call_gemm(c, a, b, sa=torch.ones(4, 1), sb=torch.ones(1, 1), tb=0)[0] == -6  # block + NN
    nc = torch.zeros(8, 8, dtype=torch.bfloat16)[::2]
    assert _call_gemm(nc, a, b)[0] == -6                                     # non-contiguous
    # empty problem is a no-op that needs no device
    assert _call_gemm(torch.zeros(0, 8, dtype=torch.bfloat16), torch.zeros(0, 128).to(FP8), b)[0] == 0
    if not torch.cuda.is_available():
        rc, msg = _call_gemm(c, a, b)
        assert rc == -4 and "device" in msg                                  # valid args, no GPU


def test_grouped_argument_validation():
    L = _lib.load()
    cfg, n = _lib.make_cfg(None)
    a = torch.zeros(10, 128).to(FP8)
    b = torch.zeros(2, 16, 128).to(FP8)
    c = torch.zeros(10, 16, dtype=torch.bfloat16)
    ptr = torch.tensor([0, 4, 10], dtype=torch.int32)

    def ragged(c, a, b, a_s, b_s, ptr):
        ds = [_lib.make_tensor_desc(t) for t in (c, a, b, a_s, b_s, ptr)]
        return L.tg_fp8_ragged_gemm(*[None if d is None else ctypes.byref(d) for d in ds], cfg, n, 0, 0)

    assert ragged(c, a, b, None, None, ptr[:2]) == -6             # m_indptr length
    assert ragged(c, a, b, None, None, ptr.long()) == -2          # m_indptr dtype
    assert ragged(c, a, b, torch.ones(10, 2), None, ptr) == -6    # a_scale shape
    assert ragged(c, a, b, None, torch.ones(2, 1, 2), ptr) == -6  # b_scale shape
    assert ragged(c, a, torch.zeros(2, 16, 64).to(FP8), None, None, ptr) == -6
    assert ragged(c, a, b, None, None, None) == -5

    def moe(block_m=16, top_k=2, w=None, mul=0, sorted_ids=None, expert_ids=None):
        sorted_ids = torch.zeros(32, dtype=torch.int32) if sorted_ids is None else sorted_ids
        expert_ids = torch.zeros(2, dtype=torch.int32) if expert_ids is None else expert_ids
        post = torch.tensor([32], dtype=torch.int32)
        a5 = torch.zeros(5, 128).to(FP8)
        ds = [_lib.make_tensor_desc(t) for t in (c, a5, b, None, None, w, sorted_ids, expert_ids, post)]
        return L.tg_fp8_moe_gemm(*[None if d is None else ctypes.byref(d) for d in ds], mul, top_k, block_m, cfg, n, 0, 0)

    assert moe(block_m=24) == -6                                   # block_m % 16
    assert moe(top_k=0) == -6
    assert moe(top_k=1) == -6                                      # 10 output rows > 5 tokens * 1
    assert moe(mul=1) == -5                                        # weights required
    assert moe(expert_ids=torch.zeros(1, dtype=torch.int32)) == -6


def test_moe_gemm_silu_quant_argument_validation():
    L = _lib.load()
    T, K, E, I, top_k = 6, 256, 2, 128, 2

    def call(q=None, scales=None, a=None, b=None, a_s=None, b_s=None, sorted_ids=None, expert_ids=None, block_m=256,
             top_k=top_k, act=_lib._DTYPE_CODES[torch.bfloat16]):
        q = torch.zeros(T * top_k, I).to(FP8) if q is None else q
        scales = torch.zeros(T * top_k, I // 128) if scales is None else scales
        a = torch.zeros(T, K).to(FP8) if a is None else a
        b = torch.zeros(E, 2 * I, K).to(FP8) if b is None else b
        a_s = torch.ones(T, K // 128) if a_s is None else a_s
        b_s = torch.ones(E, 2 * I // 128, K // 128) if b_s is None else b_s
        sorted_ids = torch.zeros(512, dtype=torch.int32) if sorted_ids is None else sorted_ids
        expert_ids = torch.zeros(2, dtype=torch.int32) if expert_ids is None else expert_ids
        post = torch.tensor([512], dtype=torch.int32)
        ds = [_lib.make_tensor_desc(t) for t in (q, scales, a, b, a_s, b_s, sorted_ids, expert_ids, post)]
        return L.tg_fp8_moe_gemm_silu_quant(*[ctypes.byref(d) for d in ds], top_k, block_m, act, 0, 0)

    assert call(block_m=64) == -6                                           # row tile of the fused form
    assert call(top_k=0) == -6
    assert call(act=_lib._DTYPE_CODES[torch.float32]) == -2                 # 16-bit intermediate type only
    assert call(q=torch.zeros(T * top_k, I, dtype=torch.bfloat16)) == -2
    assert call(q=torch.zeros(T * top_k, 2 * I).to(FP8)) == -6              # q holds I columns, not 2I
    assert call(scales=torch.zeros(T * top_k, 2)) == -6
    assert call(b=torch.zeros(E, 2 * I + 128, K).to(FP8)) == -6             # I % 128
    assert call(a_s=torch.ones(T, 1)) == -6
    assert call(b_s=torch.ones(E, 1, K // 128)) == -6
    assert call(expert_ids=torch.zeros(1, dtype=torch.int32)) == -6
    assert call(sorted_ids=torch.zeros(512, dtype=torch.int64)) == -2
    assert call(q=torch.zeros(0, I).to(FP8), scales=torch.zeros(0, 1)) == 0  # nothing to do, no device needed
    assert not _lib.moe_gemm_silu_quant_ok(torch.zeros(E, 2 * I, K), 64)
    assert _lib.moe_gemm_silu_quant_ok(torch.zeros(E, 2 * I, K), 128)
    assert _lib.moe_gemm_silu_quant_ok(torch.zeros(E, 2 * I, K), 256)
    assert not _lib.moe_gemm_silu_quant_ok(torch.zeros(E, 2 * 200, K), 256)


def test_workspace_bytes_count_the_room_for_zero_padded_operands():
    """K that the MFMA kernels cannot step through (no multiple of 128 above 64 rows, no multiple of 16 anywhere) is
    padded into the workspace: room for (M + N) rows of the padded K; none when the kernels take K as it is."""
    L = _lib.load()
    cfg, n = _lib.make_cfg(None)
    for M, N, K, padded in [(200, 264, 4104, True), (200, 264, 4096, False), (16, 264, 4112, False), (16, 264, 4100, True), (65, 264, 4112, True)]:
        got = L.tg_fp8_gemm_workspace_bytes(M, N, K, 1, cfg, n)
        same_with_k_aligned = L.tg_fp8_gemm_workspace_bytes(M, N, -(-K // 128) * 128, 1, cfg, n)
        kp = -(-K // 128) * 128
        assert got - same_with_k_aligned == ((-(-M * kp // 256) * 256 + -(-N * kp // 256) * 256) if padded else 0), (M, N, K)


def test_workspace_bytes_count_the_room_for_coarse_block_scales():
    """Quantization blocks that are multiples of 128 x 128 need room to write the scales out per 128 x 128 block."""
    L = _lib.load()
    M, N, K = 64, 1024, 2048
    base = L.tg_fp8_gemm_workspace_bytes(M, N, K, 1, *_lib.make_cfg(None))
    coarse = L.tg_fp8_gemm_workspace_bytes(M, N, K, 1, *_lib.make_cfg({"QUANT_BLOCK_N": 256, "QUANT_BLOCK_K": 256}))
    fine = L.tg_fp8_gemm_workspace_bytes(M, N, K, 1, *_lib.make_cfg({"QUANT_BLOCK_N": 64, "QUANT_BLOCK_K": 64}))
    assert fine == base and coarse == base + M * (K // 128) * 4 + (N // 128) * (K // 128) * 4


def test_fused_moe_argument_validation():
    """tg_fp8_fused_moe checks shapes, types, block size and workspace before any device call."""
    L = _lib.load()
    T, H, E, I, k = 4, 256, 4, 128, 2
    need = L.tg_fp8_fused_moe_workspace_bytes(T, k, E, H, I, 128)
    assert need > 0 and need % 256 == 0
    assert L.tg_fp8_fused_moe_workspace_bytes(T, k, E, H, I, 256) > need     # larger alignment block: more padded slots
    assert L.tg_fp8_fused_moe_workspace_bytes(T, 0, E, H, I, 128) == 0

    def call(out=None, hidden=None, w1=None, w2=None, s1=None, s2=None, tw=None, ids=None, ws=None, block_m=128):
        hidden = torch.zeros(T, H, dtype=torch.bfloat16) if hidden is None else hidden
        out = torch.zeros(T, H, dtype=torch.bfloat16) if out is None else out
        w1 = torch.zeros(E, 2 * I, H).to(FP8) if w1 is None else w1
        w2 = torch.zeros(E, H, I).to(FP8) if w2 is None else w2
        s1 = torch.ones(E, 2 * I // 128, H // 128) if s1 is None else s1
        s2 = torch.ones(E, H // 128, 1) if s2 is None else s2
        tw = torch.ones(T, k) if tw is None else tw
        ids = torch.zeros(T, k, dtype=torch.int32) if ids is None else ids
        ws = torch.zeros(need, dtype=torch.uint8) if ws is None else ws
        ds = [_lib.make_tensor_desc(t) for t in (out, hidden, w1, w2, s1, s2, tw, ids, ws)]
        return L.tg_fp8_fused_moe(*[ctypes.byref(d) for d in ds], block_m, 0, 0)

    assert call(block_m=64) == -6
    assert call(hidden=torch.zeros(T, H)) == -2                              # 16-bit activations only
    assert call(out=torch.zeros(T, H, dtype=torch.float16)) == -2            # out follows hidden's type
    assert call(out=torch.zeros(T + 1, H, dtype=torch.bfloat16)) == -6
    assert call(tw=torch.ones(T, k, dtype=torch.float16)) == -2
    assert call(tw=torch.ones(T, k + 1)) == -6
    assert call(w2=torch.zeros(E, H, 2 * I).to(FP8)) == -6
    assert call(w1=torch.zeros(E, 2 * I + 128, H).to(FP8), w2=torch.zeros(E, H, I + 64).to(FP8)) == -6   # 2I % 256
    assert call(ws=torch.zeros(need - 256, dtype=torch.uint8)) == -6
    assert call(hidden=torch.zeros(0, H, dtype=torch.bfloat16), out=torch.zeros(0, H, dtype=torch.bfloat16), tw=torch.ones(0, k),
                ids=torch.zeros(0, k, dtype=torch.int32)) == 0                # no tokens: nothing to do, no device needed
    assert _lib.fused_moe_ok(torch.zeros(T, H, dtype=torch.bfloat16), torch.zeros(E, 2 * I, H), torch.zeros(E, H, I), 128)
    assert not _lib.fused_moe_ok(torch.zeros(T, H), torch.zeros(E, 2 * I, H), torch.zeros(E, H, I), 128)
    assert not _lib.fused_moe_ok(torch.zeros(T, H, dtype=torch.bfloat16), torch.zeros(E, 2 * 200, H), torch.zeros(E, H, 200), 128)


def test_moe_align_argument_validation():
    L = _lib.load()

    def align(ids, bs, E, sorted_n=None, cum_n=None, dtype=torch.int32):
        n = ids.numel()
        cap = n + E * (bs - 1) if bs > 0 else n
        outs = [torch.zeros(cap if sorted_n is None else sorted_n, dtype=dtype), torch.zeros(max(1, -(-cap // max(bs, 1))), dtype=torch.int32),
                torch.zeros(1, dtype=torch.int32), torch.zeros(E + 1 if cum_n is None else cum_n, dtype=torch.int32),
                torch.zeros(1, dtype=torch.int32)]
        ds = [_lib.make_tensor_desc(t) for t in [ids] + outs]
        return L.tg_moe_align_block_size(ctypes.byref(ds[0]), bs, E, *[ctypes.byref(d) for d in ds[1:]], 0, 0)

    ids = torch.zeros(4, 3, dtype=torch.int64)
    assert align(ids, 0, 4) == -6                      # block size
    assert align(ids, 4, 0) == -6 and align(ids, 4, 513) == -6
    assert align(ids.float(), 4, 4) == -2              # id dtype
    assert align(ids, 4, 4, dtype=torch.int64) == -2   # output dtype
    assert align(ids, 4, 4, sorted_n=10) == -6         # capacity numel + E*(bs-1)
    assert align(ids, 4, 4, cum_n=4) == -6
    assert b"sorted_token_ids" in L.tg_last_error() or b"cumsum" in L.tg_last_error()


def test_quantizer_argument_validation():
    L = _lib.load()

    def quant(x, q=None, s=None, rule=0):
        q = torch.zeros(x.shape, dtype=FP8) if q is None else q
        s = torch.zeros(x.shape[:-1] + (max(x.shape[-1] // 128, 1),)) if s is None else s
        ds = [_lib.make_tensor_desc(t) for t in (q, s, x)]
        return L.tg_fp8_quant_1x128(*[ctypes.byref(d) for d in ds], 1e-10, rule, 0, 0)

    x = torch.zeros(4, 256, dtype=torch.bfloat16)
    assert quant(torch.zeros(4, 200, dtype=torch.bfloat16)) == -6      # K % 128
    assert quant(x.to(torch.int32)) == -2
    assert quant(x, q=torch.zeros(4, 256, dtype=torch.bfloat16)) == -2
    assert quant(x, s=torch.zeros(4, 3)) == -6
    assert quant(x, rule=2) == -6
    assert quant(torch.zeros(0, 256, dtype=torch.bfloat16)) == 0       # nothing to do, no device needed


def test_group_quantizer_and_weight_dequant_argument_validation():
    L = _lib.load()

    def quant(x, group, q=None, s=None, rule=1):
        q = torch.zeros(x.shape, dtype=FP8) if q is None else q
        s = torch.zeros(x.shape[:-1] + (max(x.shape[-1] // max(group, 1), 1),)) if s is None else s
        ds = [_lib.make_tensor_desc(t) for t in (q, s, x)]
        return L.tg_fp8_quant_group(*[ctypes.byref(d) for d in ds], group, 1e-10, rule, 0, 0)

    x = torch.zeros(6, 256, dtype=torch.float16)
    assert quant(x, 48) == -6 and quant(x, 256) == -6 and quant(x, 0) == -6     # group size
    assert quant(torch.zeros(6, 200, dtype=torch.float16), 64) == -6            # K % group
    assert quant(x, 64, rule=3) == -6
    assert quant(x, 64, s=torch.zeros(6, 3)) == -6
    assert quant(x, 64, s=torch.zeros(6, 4, dtype=torch.int32)) == -2
    assert quant(x, 64, s=torch.zeros(6, 4).t()) == -6                          # strided, but not (rows, groups)
    assert quant(x, 64, s=torch.zeros(4).expand(6, 4)) == -6                    # overlapping elements
    assert quant(torch.zeros(0, 256, dtype=torch.float16), 64, s=torch.zeros(0, 4)) == 0

    def dequant(x, s, y=None, bs=128):
        y = torch.zeros(x.shape, dtype=torch.bfloat16) if y is None else y
        ds = [_lib.make_tensor_desc(t) for t in (y, x, s)]
        return L.tg_fp8_weight_dequant(*[ctypes.byref(d) for d in ds], bs, 0, 0)

    w = torch.zeros(200, 300).to(FP8)
    assert dequant(w, torch.ones(2, 2)) == -6                                   # s must be (2, 3)
    assert dequant(w, torch.ones(2, 3), bs=0) == -6
    assert dequant(w.view(torch.uint8), torch.ones(2, 3)) == -2
    assert dequant(w, torch.ones(2, 3, dtype=torch.int32)) == -2
    assert dequant(w, torch.ones(2, 3), y=torch.zeros(200, 300, dtype=torch.int32)) == -2
    assert dequant(w, torch.ones(2, 3), y=torch.zeros(200, 301, dtype=torch.bfloat16)) == -6
    assert dequant(torch.zeros(0, 300).to(FP8), torch.ones(0, 3)) == 0          # nothing to do, no device needed


def test_workspace_bytes_and_cfg():
    L = _lib.load()
    cfg, n = _lib.make_cfg(None)
    assert L.tg_fp8_gemm_workspace_bytes(0, 10, 10, 1, cfg, n) == 0
    nt = L.tg_fp8_gemm_workspace_bytes(16, 4096, 4096, 1, cfg, n)
    nn = L.tg_fp8_gemm_workspace_bytes(16, 4096, 4096, 0, cfg, n)
    assert nt >= 65536 + 16 * 4096 * 4 and nn >= nt + 4096 * 4096
    cfg2, _ = _lib.make_cfg({"KERNEL": "skinny", "SPLIT_K": 4, "block_m": 128, "num_ctas": 2})
    assert list(cfg2)[:5] == [2, 128, -1, 4, -1]
