#!/usr/bin/env python3
"""Writes the golden vectors in this directory (run from the repository root:
``python tests/golden/make_fixtures.py``).  numpy only -- neither the oracle nor the HIP library
is used, so the vectors pin both.

The reference holds no input/output files for its FP8 GEMM tests (they draw inputs at run time
on the CUDA generator, tests/suites/unsloth/test_fp8.py:213-222), and its only known-answer
vector on this path is the worked example in the docstring of
src/tilegym/ops/cutile/moe_align_block.py:234-250; that one is stored here as data
(``moe_align_known_answer.json``).  Everything else is built so that the exact result is known
without any floating-point reasoning:

* operand codes are e4m3 encodings of small integers, scales are powers of two, so every
  product, block sum and scaled sum is an exactly representable fp32 number whatever the order
  of accumulation; the expected output is computed in int64 and rounded to bf16
  (round-to-nearest-even on the fp32 bit pattern) by integer arithmetic;
* the e4m3fn decode table is written from the OCP FP8 definition (1-4-3, bias 7, no infinities,
  0x7F/0xFF = NaN, subnormals m * 2**-9).

Files (all a few KB .. 100 KB):
  e4m3fn_decode_table.npy        256 float32 values (NaN at 0x7F / 0xFF)
  per_tensor_24x144x256.npz      a (M,K) u8 codes, b (N,K) u8 codes, scale_a, scale_b, c_bf16 (u16 bits)
  block_scaled_16x256x384.npz    a, b, a_scale (M,K/128), b_scale (N/128,K/128), c_bf16
  ragged_3experts.npz            a (total_m,K), b (E,N,K), a_scale, b_scale, m_indptr (expert 1 empty), c_bf16
  moe_gather_top2.npz            a (T,K), b (E,N,K), scales, topk_ids, topk_weights (powers of two),
                                 c_bf16 (T,top_k,N) with and without the routed weight
  moe_align_known_answer.json    topk_ids / block_size / num_experts -> sorted ids, padded cumsum
"""

import json
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))


def decode_table():
    out = np.zeros(256, dtype=np.float64)
    for code in range(256):
        sign = -1.0 if code & 0x80 else 1.0
        e, m = (code >> 3) & 0xF, code & 7
        if e == 0xF and m == 7:
            out[code] = np.nan
        elif e == 0:
            out[code] = sign * m * 2.0 ** -9
        else:
            out[code] = sign * (1 + m / 8.0) * 2.0 ** (e - 7)
    return out.astype(np.float32)


def encode_small_int(v):
    """e4m3fn code of an integer in [-16, 16] (all exactly representable)."""
    table = decode_table()
    lut = {}
    for code in range(256):
        x = table[code]
        if not np.isnan(x) and float(x).is_integer() and abs(x) <= 16 and not (code == 0x80):
            lut[int(x)] = code
    return np.vectorize(lambda t: lut[int(t)], otypes=[np.uint8])(v)


def bf16_bits_rne(x32):
    """fp32 array -> bf16 bit patterns (uint16), round to nearest even, by integer arithmetic."""
    u = np.asarray(x32, dtype=np.float32).view(np.uint32).astype(np.uint64)
    rounded = (u + 0x7FFF + ((u >> 16) & 1)) >> 16
    return rounded.astype(np.uint16)


def exact_to_bf16(num, log2_den):
    """num / 2**log2_den with |num| < 2**24 -> bf16 bits; the fp32 value is exact."""
    assert np.abs(num).max() < (1 << 24)
    x = (num.astype(np.float64) / float(1 << log2_den)).astype(np.float32)
    assert np.array_equal(x.astype(np.float64) * float(1 << log2_den), num.astype(np.float64))
    return bf16_bits_rne(x)


def pow2_scales(rng, shape, lo=-2, hi=1):
    """Random powers of two 2**e, e in [lo, hi]; returns (float32 scales, e - lo as int64)."""
    e = rng.integers(lo, hi + 1, size=shape)
    return (2.0 ** e).astype(np.float32), (e - lo).astype(np.int64)


def block_scaled_exact(ai, bi, ea, eb, bn=128, bk=128):
    """sum_kb 2**(ea[m,kb] + eb[n//bn,kb]) * sum_{k in kb} ai[m,k]*bi[n,k], in int64."""
    M, K = ai.shape
    N = bi.shape[0]
    out = np.zeros((M, N), dtype=np.int64)
    for kb in range((K + bk - 1) // bk):
        ks = slice(kb * bk, min(K, (kb + 1) * bk))
        part = ai[:, ks] @ bi[:, ks].T
        w = (1 << ea[:, kb])[:, None] * (1 << eb[np.arange(N) // bn, kb])[None, :]
        out += part * w
    return out


def main():
    rng = np.random.default_rng(20240607)
    np.save(os.path.join(HERE, "e4m3fn_decode_table.npy"), decode_table())

    # ---- per-tensor: C = (sa*sb) * A @ B^T, sa = 2**-3, sb = 2**-1
    M, N, K = 24, 144, 256
    ai = rng.integers(-8, 9, size=(M, K)).astype(np.int64)
    bi = rng.integers(-8, 9, size=(N, K)).astype(np.int64)
    np.savez_compressed(os.path.join(HERE, "per_tensor_24x144x256.npz"),
                        a=encode_small_int(ai), b=encode_small_int(bi),
                        scale_a=np.float32(0.125), scale_b=np.float32(0.5),
                        c_bf16=exact_to_bf16(ai @ bi.T, 4))

    # ---- block scaled, scales 2**[-2..1] (N = 384: three weight-scale rows, K = 256: two K blocks)
    M, N, K = 16, 384, 256
    ai = rng.integers(-8, 9, size=(M, K)).astype(np.int64)
    bi = rng.integers(-8, 9, size=(N, K)).astype(np.int64)
    sa, ea = pow2_scales(rng, (M, K // 128))
    sb, eb = pow2_scales(rng, (N // 128, K // 128))
    np.savez_compressed(os.path.join(HERE, "block_scaled_16x256x384.npz"),
                        a=encode_small_int(ai), b=encode_small_int(bi), a_scale=sa, b_scale=sb,
                        c_bf16=exact_to_bf16(block_scaled_exact(ai, bi, ea, eb), 4))

    # ---- ragged grouped: 3 experts, the middle one owns no rows
    E, N, K = 3, 128, 256
    indptr = np.array([0, 37, 37, 60], dtype=np.int32)
    total = int(indptr[-1])
    ai = rng.integers(-8, 9, size=(total, K)).astype(np.int64)
    bi = rng.integers(-8, 9, size=(E, N, K)).astype(np.int64)
    sa, ea = pow2_scales(rng, (total, K // 128))
    sb, eb = pow2_scales(rng, (E, N // 128, K // 128))
    exact = np.zeros((total, N), dtype=np.int64)
    for e in range(E):
        lo, hi = int(indptr[e]), int(indptr[e + 1])
        if hi > lo:
            exact[lo:hi] = block_scaled_exact(ai[lo:hi], bi[e], ea[lo:hi], eb[e])
    np.savez_compressed(os.path.join(HERE, "ragged_3experts.npz"),
                        a=encode_small_int(ai), b=encode_small_int(bi), a_scale=sa, b_scale=sb,
                        m_indptr=indptr, c_bf16=exact_to_bf16(exact, 4))

    # ---- token-gather MoE form: T tokens, top-2 of 4 experts, routed weights are powers of two
    T, E, N, K, top_k = 10, 4, 128, 128, 2
    ai = rng.integers(-8, 9, size=(T, K)).astype(np.int64)
    bi = rng.integers(-8, 9, size=(E, N, K)).astype(np.int64)
    sa, ea = pow2_scales(rng, (T, 1))
    sb, eb = pow2_scales(rng, (E, 1, 1))
    topk_ids = np.stack([rng.permutation(E)[:top_k] for _ in range(T)]).astype(np.int32)
    tw, ew = pow2_scales(rng, (T, top_k), lo=-2, hi=0)
    plain = np.zeros((T, top_k, N), dtype=np.int64)
    for t in range(T):
        for j in range(top_k):
            e = int(topk_ids[t, j])
            plain[t, j] = block_scaled_exact(ai[t:t + 1], bi[e], ea[t:t + 1], eb[e])[0]
    weighted = plain * (1 << ew)[:, :, None]
    np.savez_compressed(os.path.join(HERE, "moe_gather_top2.npz"),
                        a=encode_small_int(ai), b=encode_small_int(bi), a_scale=sa, b_scale=sb,
                        topk_ids=topk_ids, topk_weights=tw,
                        c_bf16=exact_to_bf16(plain, 4), c_weighted_bf16=exact_to_bf16(weighted, 6))

    # ---- the reference's worked example (expert labels 1..4 there; stored 0-based)
    with open(os.path.join(HERE, "moe_align_known_answer.json"), "w") as f:
        json.dump({
            "source": "src/tilegym/ops/cutile/moe_align_block.py:234-250 (docstring example, labels shifted to 0-based)",
            "topk_ids": [[1, 2, 3], [0, 1, 3], [0, 2, 3], [0, 1, 2]],
            "block_size": 4, "num_experts": 4,
            "sorted_token_ids_first16": [3, 6, 9, 12, 0, 4, 10, 12, 1, 7, 11, 12, 2, 5, 8, 12],
            "sentinel": 12, "expert_ids_first4": [0, 1, 2, 3],
            "num_tokens_post_padded": 16, "padded_cumsum": [0, 4, 8, 12, 16], "max_expert_count": 3,
        }, f, indent=1)
    for name in sorted(os.listdir(HERE)):
        print(f"{name:36s} {os.path.getsize(os.path.join(HERE, name)):8d} bytes")


if __name__ == "__main__":
    main()
