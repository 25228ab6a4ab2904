"""Pins of the CPU oracle (oracle/reference.py, oracle/fp8_oracle.c): closed forms, exact integer
cases, brute force on tiny inputs, invariants, and the reference's one known-answer vector."""

import math

import numpy as np
import pytest
import torch

from oracle import c_oracle as C
from oracle import reference as R

FP8 = torch.float8_e4m3fn


def _g(seed):
    return torch.Generator().manual_seed(seed)


# ---------------------------------------------------------------- codec
def test_decode_table_matches_torch_view_and_closed_form():
    torch_tab = torch.arange(256, dtype=torch.uint8).view(FP8).float().numpy()
    for tab in (R.e4m3fn_decode_table(), C.decode_table()):
        assert np.array_equal(np.isnan(tab), np.isnan(torch_tab))
        ok = ~np.isnan(tab)
        assert np.array_equal(tab[ok], torch_tab[ok])
    tab = R.e4m3fn_decode_table()
    assert tab[0x7E] == 448.0 and tab[0xFE] == -448.0          # max finite
    assert tab[0x01] == 2.0 ** -9 and tab[0x08] == 2.0 ** -6   # min subnormal, min normal
    assert np.isnan(tab[0x7F]) and np.isnan(tab[0xFF])
    assert tab[0x38] == 1.0 and tab[0x40] == 2.0 and tab[0x3C] == 1.5


def test_encode_rne_matches_torch_cast_dense_grid():
    x = torch.cat([torch.linspace(-448, 448, 100001), torch.linspace(-0.05, 0.05, 20001),
                   torch.tensor([0.0, -0.0, 2.0 ** -10, 3 * 2.0 ** -10, 2.0 ** -9, 447.9, 448.0])])
    want = x.to(FP8).view(torch.uint8).numpy()
    got = R.e4m3fn_encode_rne(x.numpy())
    assert np.array_equal(got, want)
    L = C.lib()
    sub = x[::53]
    got_c = np.array([L.orc_e4m3_encode(float(v)) for v in sub.tolist()], dtype=np.uint8)
    assert np.array_equal(got_c, sub.to(FP8).view(torch.uint8).numpy())


def test_bf16_rounding_matches_torch():
    x = torch.randn(5000, generator=_g(3)) * 100
    want = x.to(torch.bfloat16).view(torch.int16).numpy().astype(np.uint16)
    L = C.lib()
    got = np.array([L.orc_bf16_bits(float(v)) for v in x.tolist()], dtype=np.uint16)
    assert np.array_equal(got, want)


# ---------------------------------------------------------------- quantizers
def test_quantizers_scale_rule_and_zero_blocks():
    x = torch.randn(7, 256, generator=_g(0))
    x[2, :128] = 0
    q, s = R.quantize_act_1x128(x)                 # unsloth rule
    assert s.shape == (7, 2) and s[2, 0] == 1.0
    assert torch.equal(s[0, 0], x[0, :128].abs().max() / 448.0)
    assert R.fp8_to_f32(q).abs().max() == 448.0    # every non-zero block hits +-448
    q2, s2 = R.quantize_act_1x128(x, eps=1e-10)    # flashinfer rule
    assert s2[2, 0] == pytest.approx(1e-10 / 448.0)
    deq = R.fp8_to_f32(q) * s.repeat_interleave(128, 1)
    assert (deq - x).abs().max() <= x.abs().max() * 2 ** -4   # e4m3 has 3 mantissa bits
    w = torch.randn(200, 300, generator=_g(1)) * 0.02
    qw, sw = R.quantize_weight_128x128(w)
    assert sw.shape == (2, 3)
    assert torch.equal(sw[1, 2], w[128:, 256:].abs().max() / 448.0)
    back = R.weight_dequant(qw, sw, 128, torch.float32)
    assert (back - w).abs().max() <= w.abs().max() * 2 ** -4
    qt, st = R.quantize_per_tensor(w)
    assert st.shape == (1,) and torch.equal(st[0], w.abs().max() / 448.0)


def test_quantizer_power_of_two_scales_and_small_groups():
    """Pins of the remaining quantizer forms: (a) with ue8m0 every scale is the smallest power of two that is
    not below the plain scale (exponent arithmetic on the fp32 bits, no logarithm), (b) groups of 16 / 32 / 64
    against a per-group Python loop, (c) weight_dequant against an element loop with ragged edge blocks."""
    x = torch.randn(9, 256, generator=_g(11)) * 3.0
    x[4, 128:] = 0
    x[5, :128] = 448.0 * 2.0 ** -7                                   # plain scale exactly 2^-7: must stay 2^-7
    for block in (16, 32, 64, 128):
        q, s = R.quantize_act_1x128(x, block, eps=1e-10)
        qp, sp = R.quantize_act_1x128(x, block, eps=1e-10, ue8m0=True)
        bits = sp.view(torch.int32)
        assert torch.all((bits & 0x7FFFFF) == 0) and torch.all(sp > 0)   # powers of two
        floor_pow2 = torch.maximum(s, torch.tensor(1e-10)).view(torch.int32).bitwise_and(0x7F800000).view(torch.float32)
        want = torch.where(floor_pow2 == torch.maximum(s, torch.tensor(1e-10)), floor_pow2, floor_pow2 * 2)
        assert torch.equal(sp, want)
        xb = x.reshape(-1, block)
        for gi in (0, 3, xb.shape[0] - 1):                           # per-group loop
            amax = max(abs(v) for v in xb[gi].tolist())
            sc = np.float32(max(amax, 1e-10)) / np.float32(448.0)
            assert np.float32(s.reshape(-1)[gi].item()) == sc
            codes = (xb[gi] / torch.tensor(sc)).clamp(-448, 448).to(FP8)
            assert torch.equal(codes.view(torch.uint8), q.reshape(-1, block)[gi].view(torch.uint8))
            codes2 = (xb[gi] / sp.reshape(-1)[gi]).clamp(-448, 448).to(FP8)
            assert torch.equal(codes2.view(torch.uint8), qp.reshape(-1, block)[gi].view(torch.uint8))
    assert sp.reshape(9, 2)[5, 0] == 2.0 ** -7 and sp.reshape(9, 2)[4, 1] == 2.0 ** math.ceil(math.log2(1e-10))
    w = (torch.randn(70, 150, generator=_g(12)) * 50).to(FP8)
    sc = torch.rand(3, 5, generator=_g(13)) + 0.5
    y = R.weight_dequant(w, sc, 32, torch.float32)
    wf = R.fp8_to_f32(w)
    for i, j in ((0, 0), (31, 32), (69, 149), (64, 127), (33, 96)):
        assert y[i, j] == wf[i, j] * sc[i // 32, j // 32]
    assert torch.equal(R.weight_dequant(w, sc, 32, torch.bfloat16), y.to(torch.bfloat16))


# ---------------------------------------------------------------- GEMMs
def _int_fp8(shape, g, lo=-8, hi=9):
    return torch.randint(lo, hi, shape, generator=g).float().to(FP8)


def test_per_tensor_gemm_exact_integers_and_layouts():
    g = _g(5)
    M, N, K = 5, 7, 96
    a, b = _int_fp8((M, K), g), _int_fp8((N, K), g)
    want = a.float().long() @ b.float().long().t()          # exact int64
    got = R.ref_gemm_per_tensor(a, b, trans_b=True, out_dtype=torch.float32)
    assert torch.equal(got.long(), want)
    # the same product through the other three layouts
    bt = b.view(torch.uint8).t().contiguous().view(FP8)      # (K,N)
    at = a.view(torch.uint8).t().contiguous().view(FP8)      # (K,M)
    assert torch.equal(R.ref_gemm_per_tensor(a, bt, out_dtype=torch.float32).long(), want)
    assert torch.equal(R.ref_gemm_per_tensor(at, bt, trans_a=True, out_dtype=torch.float32).long(), want)
    assert torch.equal(R.ref_gemm_per_tensor(at, b, trans_a=True, trans_b=True, out_dtype=torch.float32).long(), want)
    # power-of-two scales are exact
    got2 = R.ref_gemm_per_tensor(a, b, 0.5, torch.tensor([4.0]), trans_b=True, out_dtype=torch.float32)
    assert torch.equal(got2, got * 2.0)
    # C restatement
    c = C.gemm_per_tensor(R.fp8_bytes(a), R.fp8_bytes(b), 0.5, 4.0)
    assert np.array_equal(c, got2.numpy())


def test_alpha_beta_is_linear_in_the_per_tensor_oracle():
    g = _g(6)
    a, b = _int_fp8((4, 64), g), _int_fp8((6, 64), g)
    c0 = torch.randn(4, 6, generator=g).to(torch.bfloat16)
    base = R.ref_gemm_per_tensor(a, b, trans_b=True, out_dtype=torch.float32)
    got = R.ref_gemm_alpha_beta(a, b, c0.clone(), False, True, 1.5, 2.0)
    assert got.dtype == torch.bfloat16
    assert torch.equal(got, (1.5 * base + 2.0 * c0.float()).to(torch.bfloat16))
    assert torch.equal(R.ref_gemm_alpha_beta(a, b, c0.clone(), False, True, 1.0, 0.0), base.to(torch.bfloat16))


def _loop_block_gemm(A, B, As, Bs, bn, bk):
    """The reference test's own formulation: per-element loops (tests/suites/unsloth/test_fp8.py:159-191)."""
    Af, Bf = R.fp8_to_f32(A), R.fp8_to_f32(B)
    M, K = Af.shape
    N = Bf.shape[0]
    A_deq = torch.zeros(M, K)
    for m in range(M):
        for k0 in range(0, K, bk):
            A_deq[m, k0:k0 + bk] = Af[m, k0:k0 + bk] * As[m, k0 // bk]
    B_deq = torch.zeros(N, K)
    for n0 in range(0, N, bn):
        for k0 in range(0, K, bk):
            B_deq[n0:n0 + bn, k0:k0 + bk] = Bf[n0:n0 + bn, k0:k0 + bk] * Bs[n0 // bn, k0 // bk]
    return A_deq @ B_deq.t()


def test_int8_group_quantizer_oracle_hand_vector_and_properties():
    """dst_dtype=torch.int8 of per_token_group_quant_8bit (tests/suites/flashinfer/test_per_token_group_quant_8bit.py:41-68):
    a hand-computed group, and what the definition fixes: scale = amax / 127, the largest element maps to +-127 (or
    +-126 when the fp32 quotient falls one ulp short), truncation toward zero (never away), all-zero groups use eps."""
    x = torch.zeros(1, 16)
    x[0, :6] = torch.tensor([12.7, -12.7, 1.0, -0.99, 0.05, 6.36])
    q, s = R.quantize_act_1x128(x, 16, 1e-10, dst_dtype=torch.int8)
    assert q.dtype == torch.int8 and abs(float(s) - 0.1) < 1e-7
    # 12.7/0.1 = 127, 1.0/0.1 = 10 (9.99.. in fp32 -> 9 or 10 by the quotient's rounding), -0.99/0.1 = -9.9 -> -9, 0.05/0.1 -> 0, 63.6 -> 63
    want = torch.tensor([127, -127, int(torch.tensor(1.0) / s.reshape(())), -9, 0, 63], dtype=torch.int8)
    assert torch.equal(q[0, :6], want) and int(q[0, 2]) in (9, 10)
    g = _g(55)
    y = torch.randn(37, 256, generator=g) * torch.exp(torch.randn(37, 1, generator=g))
    y[3] = 0.0
    for group in (16, 64, 128):
        q, s = R.quantize_act_1x128(y, group, 1e-10, dst_dtype=torch.int8)
        yb, qb, sb = y.reshape(-1, group), q.reshape(-1, group).float(), s.reshape(-1, 1)
        amax = yb.abs().amax(dim=1, keepdim=True)
        assert torch.equal(sb, amax.clamp(min=1e-10) / 127.0)
        nz = amax.squeeze(1) > 0
        top = qb.abs().amax(dim=1)[nz]   # amax / (amax / 127) is 127 or one ulp below it in fp32, and the cast truncates
        assert ((top == 127) | (top == 126)).all() and (top == 127).any()
        exact = yb.double() / sb.double()
        assert (qb.abs() <= exact.abs() + 1e-4).all() and ((exact.abs() - qb.abs()) < 1.0 + 1e-4).all()   # toward zero, by less than one step
        assert torch.equal(torch.sign(qb)[qb != 0], torch.sign(yb)[qb != 0])
        assert (qb[~nz] == 0).all()


@pytest.mark.parametrize("M,N,K", [(3, 130, 256), (5, 256, 384), (2, 100, 200)])
def test_block_scaled_oracle_against_loops_and_c(M, N, K):
    g = _g(7)
    A = (torch.randn(M, K, generator=g) * 0.1).to(FP8)
    B = (torch.randn(N, K, generator=g) * 0.1).to(FP8)
    As = torch.rand(M, -(-K // 128), generator=g) + 0.1
    Bs = torch.rand(-(-N // 128), -(-K // 128), generator=g) + 0.1
    want = _loop_block_gemm(A, B, As, Bs, 128, 128)
    got = R.ref_w8a8_block_fp8_matmul(A, B, As, Bs)
    assert torch.allclose(got, want, rtol=1e-6, atol=1e-6)
    c = C.gemm_block_scaled(R.fp8_bytes(A), R.fp8_bytes(B), As.numpy(), Bs.numpy())
    assert np.allclose(c, want.numpy(), rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("bn,bk", [(64, 64), (256, 32), (48, 80)])
def test_block_scaled_oracle_with_other_quantization_blocks_against_loops(bn, bk):
    """block_size=[block_n, block_k] other than 128 x 128 (the reference's general form,
    tests/suites/unsloth/test_fp8.py:159-191): the vectorised oracle against the element-by-element loop."""
    g = _g(70 + bn + bk)
    M, N, K = 5, 150, 200
    A = (torch.randn(M, K, generator=g) * 0.1).to(FP8)
    B = (torch.randn(N, K, generator=g) * 0.1).to(FP8)
    As = torch.rand(M, -(-K // bk), generator=g) + 0.1
    Bs = torch.rand(-(-N // bn), -(-K // bk), generator=g) + 0.1
    want = _loop_block_gemm(A, B, As, Bs, bn, bk)
    got = R.ref_w8a8_block_fp8_matmul(A, B, As, Bs, [bn, bk])
    assert torch.allclose(got, want, rtol=1e-6, atol=1e-6)


def test_block_scaled_invariants():
    g = _g(8)
    M, N, K = 4, 256, 256
    A, B = _int_fp8((M, K), g, -4, 5), _int_fp8((N, K), g, -4, 5)
    ones_a, ones_b = torch.ones(M, 2), torch.ones(2, 2)
    exact = (A.float().long() @ B.float().long().t()).float()
    # all-ones scales == unscaled GEMM (exact for small integers)
    assert torch.equal(R.ref_w8a8_block_fp8_matmul(A, B, ones_a, ones_b), exact)
    # all blocks equal == per-tensor
    assert torch.equal(R.ref_w8a8_block_fp8_matmul(A, B, ones_a * 0.25, ones_b * 2.0),
                       R.ref_gemm_per_tensor(A, B, 0.25, 2.0, trans_b=True, out_dtype=torch.float32))
    # scaling one K block of As by 2^k scales only that block's contribution
    As = ones_a.clone(); As[:, 1] = 4.0
    part1 = (A[:, 128:].float().long() @ B[:, 128:].float().long().t()).float()
    assert torch.equal(R.ref_w8a8_block_fp8_matmul(A, B, As, ones_b), exact + 3.0 * part1)
    # one N block of Bs
    Bs = ones_b.clone(); Bs[1, :] = 0.5
    got = R.ref_w8a8_block_fp8_matmul(A, B, ones_a, Bs)
    assert torch.equal(got[:, :128], exact[:, :128]) and torch.equal(got[:, 128:], 0.5 * exact[:, 128:])


def test_ragged_oracle_properties():
    g = _g(9)
    Q, N, K = 4, 128, 256
    sizes = [5, 0, 9, 3]
    ptr = torch.tensor([0, 5, 5, 14, 17], dtype=torch.int32)
    total = 20  # three rows belong to no segment
    a = (torch.randn(total, K, generator=g) * 0.5).to(FP8)
    b = (torch.randn(Q, N, K, generator=g) * 0.5).to(FP8)
    a_s = torch.rand(total, 2, generator=g) + 0.1
    b_s = torch.rand(Q, 1, 2, generator=g) + 0.1
    out = R.ref_ragged_block_scaled_bmm(a, b, a_s, b_s, ptr, out_dtype=torch.float32)
    assert torch.equal(out[17:], torch.zeros(3, N))
    for q in range(Q):
        lo, hi = int(ptr[q]), int(ptr[q + 1])
        if hi > lo:
            dense = R.ref_w8a8_block_fp8_matmul(a[lo:hi], b[q], a_s[lo:hi], b_s[q])
            assert torch.equal(out[lo:hi], dense)
    # permuting experts permutes the output segments
    perm = [2, 0, 3, 1]
    segs = [(int(ptr[q]), int(ptr[q + 1])) for q in perm]
    a_p = torch.cat([a[lo:hi] for lo, hi in segs] + [a[17:]])
    as_p = torch.cat([a_s[lo:hi] for lo, hi in segs] + [a_s[17:]])
    ptr_p = torch.tensor([0] + list(np.cumsum([sizes[q] for q in perm])), dtype=torch.int32)
    out_p = R.ref_ragged_block_scaled_bmm(a_p, b[perm], as_p, b_s[perm], ptr_p, out_dtype=torch.float32)
    assert torch.equal(out_p[:17], torch.cat([out[lo:hi] for lo, hi in segs]))
    # C restatement
    c = C.gemm_ragged(R.fp8_bytes(a), R.fp8_bytes(b), a_s.numpy(), b_s.numpy(), ptr.numpy())
    assert np.allclose(c, out.numpy(), rtol=1e-5, atol=1e-5)
    # a_scale=None means ones
    o1 = R.ref_ragged_block_scaled_bmm(a, b, None, b_s, ptr, out_dtype=torch.float32)
    o2 = R.ref_ragged_block_scaled_bmm(a, b, torch.ones(total, 2), b_s, ptr, out_dtype=torch.float32)
    assert torch.equal(o1, o2)


def test_group_gemm_oracle_is_a_list_of_gemms():
    g = _g(10)
    As = [_int_fp8((3, 32), g), _int_fp8((5, 64), g)]
    Bs = [_int_fp8((32, 4), g), _int_fp8((64, 6), g)]
    outs = R.ref_group_gemm(As, Bs, out_dtype=torch.float32)
    for A, B, o in zip(As, Bs, outs):
        assert torch.equal(o.long(), A.float().long() @ B.float().long())
    Bt = [b.view(torch.uint8).t().contiguous().view(FP8) for b in Bs]
    outs_t = R.ref_group_gemm(As, Bt, transpose_b=True, out_dtype=torch.float32)
    assert all(torch.equal(x, y) for x, y in zip(outs, outs_t))


# ---------------------------------------------------------------- MoE
def test_moe_align_known_answer_vector():
    """Worked example of src/tilegym/ops/cutile/moe_align_block.py:234-250 (expert labels 1..4 there;
    0-based here)."""
    ids = torch.tensor([[2, 3, 4], [1, 2, 4], [1, 3, 4], [1, 2, 3]]) - 1
    want_sorted = [3, 6, 9, 12, 0, 4, 10, 12, 1, 7, 11, 12, 2, 5, 8, 12]
    s, e, post, cum, mx = R.moe_align_block_size_ref(ids, 4, 4)
    assert s[:16].tolist() == want_sorted and s[16:].tolist() == [12] * 8
    assert s.numel() == 12 + 4 * 3 and e.numel() == 6
    assert e[:4].tolist() == [0, 1, 2, 3]
    assert int(post) == 16 and cum.tolist() == [0, 4, 8, 12, 16] and int(mx) == 3
    cs, ce, cpost, ccum, cmx = C.moe_align(ids.numpy(), 4, 4)
    assert cs[:16].tolist() == want_sorted and cpost == 16 and ccum.tolist() == [0, 4, 8, 12, 16] and cmx == 3
    assert ce[:4].tolist() == [0, 1, 2, 3]


def test_moe_align_random_properties():
    g = _g(11)
    E, bs = 8, 16
    ids = torch.randint(0, E, (50, 3), generator=g)
    ids[ids == 5] = 4  # expert 5 gets no tokens
    s, e, post, cum, mx = R.moe_align_block_size_ref(ids, bs, E)
    flat = ids.reshape(-1)
    post = int(post)
    assert post % bs == 0 and cum[-1] == post
    valid = s[:post][s[:post] < flat.numel()]
    assert sorted(valid.tolist()) == list(range(flat.numel()))          # a permutation of all slots
    for blk in range(post // bs):
        rows = s[blk * bs:(blk + 1) * bs]
        rows = rows[rows < flat.numel()]
        assert (flat[rows.long()] == e[blk]).all()                      # one expert per block
        assert rows.tolist() == sorted(rows.tolist())                   # stable
    assert int(mx) == int(torch.bincount(flat, minlength=E).max())
    cs, ce, cpost, ccum, cmx = C.moe_align(ids.numpy(), bs, E)
    assert np.array_equal(cs, s.numpy()) and cpost == post and np.array_equal(ccum, cum.numpy())
    assert np.array_equal(ce[:post // bs], e[:post // bs].numpy())


def test_fused_moe_gemm_oracle_against_token_loops():
    g = _g(12)
    T, E, N, K, topk = 6, 4, 128, 256, 2
    A = (torch.randn(T, K, generator=g) * 0.3).to(FP8)
    B = (torch.randn(E, N, K, generator=g) * 0.3).to(FP8)
    a_s = torch.rand(T, 2, generator=g) + 0.1
    b_s = torch.rand(E, 1, 2, generator=g) + 0.1
    ids = torch.randint(0, E, (T, topk), generator=g)
    w = torch.rand(T, topk, generator=g)
    got = R.ref_fused_moe_gemm(A, B, a_s, b_s, w, ids, True, topk, out_dtype=torch.float32)
    for t in range(T):
        for j in range(topk):
            e = int(ids[t, j])
            a_deq = R.fp8_to_f32(A[t]) * a_s[t].repeat_interleave(128)
            b_deq = R.fp8_to_f32(B[e]) * b_s[e].repeat_interleave(128, 0).repeat_interleave(128, 1)
            want = (b_deq @ a_deq) * w[t, j]
            assert torch.allclose(got[t, j], want, rtol=1e-5, atol=1e-5)


def test_fused_experts_oracle_is_the_composition_of_its_steps():
    """ref_fused_experts_fp8 against an independent per-token evaluation with dequantized weights:
    a dropped routed weight, a swapped gate/up half or a wrong slot->expert index fails this."""
    g = _g(21)
    T, E, k, H, I = 5, 3, 2, 128, 128
    hidden = torch.randn(T, H, generator=g).to(torch.bfloat16)
    w1q, w1s = R.quantize_weight_128x128(torch.randn(E * 2 * I, H, generator=g) * 0.1)
    w2q, w2s = R.quantize_weight_128x128(torch.randn(E * H, I, generator=g) * 0.1)
    w1q, w1s = w1q.reshape(E, 2 * I, H), w1s.reshape(E, 2, 1)
    w2q, w2s = w2q.reshape(E, H, I), w2s.reshape(E, 1, 1)
    ids = torch.tensor([[0, 2], [1, 0], [2, 1], [0, 1], [2, 0]])
    tw = torch.rand(T, k, generator=g)
    out = R.ref_fused_experts_fp8(hidden, w1q, w2q, w1s, w2s, tw, ids)
    xq, xs = R.quantize_act_1x128(hidden, 128, None)
    x = R.fp8_to_f32(xq) * xs                                   # one group per row
    want = torch.zeros(T, H)
    for t in range(T):
        for j in range(k):
            e = int(ids[t, j])
            W1 = R.fp8_to_f32(w1q[e]) * w1s[e].repeat_interleave(128, 0)
            W2 = R.fp8_to_f32(w2q[e]) * w2s[e, 0, 0]
            h1 = (x[t] @ W1.t()).to(torch.bfloat16).float()
            act = ((h1[:I] / (1 + torch.exp(-h1[:I]))) * h1[I:]).to(torch.bfloat16)
            aq, a_s = R.quantize_act_1x128(act.reshape(1, I), 128, None)
            h2 = ((R.fp8_to_f32(aq) * a_s) @ W2.t() * tw[t, j]).to(torch.bfloat16).float()
            want[t] += h2[0]
    assert torch.equal(out, want.to(torch.bfloat16))
    q, s, act = R.ref_silu_mul_quant(torch.randn(3, 2 * 200, generator=g).to(torch.bfloat16))
    assert q.shape == (3, 200) and s.shape == (3, 2) and act.shape == (3, 200)


def test_silu_mul_quant_oracle_against_library_silu_and_a_hand_computed_vector():
    """ref_silu_mul_quant: its activation against torch.nn.functional.silu (a library routine, not the oracle's own
    formula) and against values worked out by hand; a wrong sign in the exponential, sigmoid instead of SiLU, or
    gate and up swapped fails one of them; then scales and codes from the activation's own amax."""
    F = torch.nn.functional
    g = _g(31)
    for dtype in (torch.bfloat16, torch.float16):
        x = (torch.randn(6, 2 * 256, generator=g) * 3).to(dtype)
        q, s, act = R.ref_silu_mul_quant(x)
        want = (F.silu(x[:, :256].float()) * x[:, 256:].float()).to(dtype)
        assert torch.equal(act, want)
        amax = want.float().reshape(6, 2, 128).abs().amax(-1)
        assert torch.equal(s, amax / 448.0)
        assert torch.equal(R.fp8_to_f32(q), (want.float().reshape(6, 2, 128) / s[..., None]).clamp(-448, 448).to(R.FP8).float().reshape(6, 256))
    # by hand: silu(0) = 0; silu(1) = 1 / (1 + e^-1) = 0.7310586; silu(-1) = -0.2689414; silu(2) = 1.7615942; silu(-20) ~ -4.1e-8
    gate = torch.tensor([[0.0, 1.0, -1.0, 2.0, -20.0, 3.0, 0.5, -0.5]])
    up = torch.tensor([[5.0, 2.0, 4.0, -1.0, 1.0, 0.0, -2.0, 8.0]])
    expect = torch.tensor([[0.0, 1.4621172, -1.0757656, -1.7615942, -4.1223e-08, 0.0, -0.6224593, -1.5101871]])
    _, _, act = R.ref_silu_mul_quant(torch.cat([gate, up], 1).to(torch.float16))
    assert torch.equal(act, expect.to(torch.float16))
    _, _, act_swapped = R.ref_silu_mul_quant(torch.cat([up, gate], 1).to(torch.float16))
    assert not torch.equal(act_swapped, act)


def test_compare_to_oracle_flags_errors():
    ref = torch.randn(64, 64, generator=_g(13))
    ok, _ = R.compare_to_oracle(ref.to(torch.bfloat16), ref)
    assert ok
    bad = ref.clone(); bad[3, 4] += 1.0
    ok, rep = R.compare_to_oracle(bad, ref)
    assert not ok and rep["matched"] < 1.0
    nan = ref.clone(); nan[0, 0] = float("nan")
    assert not R.compare_to_oracle(nan, ref)[0]


def test_output_cast_rule_saturates_e4m3_and_leaves_wider_types_to_torch():
    x = torch.tensor([0.0, 1.0, -447.9, 448.0, 464.0, 465.0, 1e4, -1e9, float("inf")])
    sat = R.cast_output(x, R.FP8).float()
    assert torch.equal(sat, torch.tensor([0.0, 1.0, -448.0, 448.0, 448.0, 448.0, 448.0, -448.0, 448.0]))
    plain = R.cast_output(x, R.FP8, saturate=False).float()
    assert torch.equal(plain[:5], sat[:5]) and torch.isnan(plain[5:]).all()
    for dt in (torch.bfloat16, torch.float16, torch.float32):
        assert torch.equal(R.cast_output(x[:7], dt), x[:7].to(dt))
    # in range the two rules are the same function: all 256 codes round-trip
    codes = torch.arange(256, dtype=torch.uint8).view(R.FP8).float()
    finite = codes[~torch.isnan(codes)]
    assert torch.equal(R.cast_output(finite, R.FP8).float(), finite)
