"""Golden vectors (tests/golden/, written by tests/golden/make_fixtures.py with numpy integer
arithmetic only): the expected outputs are exact, so both the CPU oracle (not-gpu tests) and the
HIP path through the C ABI (gpu tests) must reproduce them bit for bit in bf16, on every kernel
family that can run the shape.
"""

import json
import os

import numpy as np
import pytest
import torch

from oracle import c_oracle as C
from oracle import reference as R

HERE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
FP8 = torch.float8_e4m3fn


def _npz(name):
    with np.load(os.path.join(HERE, name), allow_pickle=False) as z:
        return {k: z[k] for k in z.files}


def _fp8(codes):
    return torch.from_numpy(np.ascontiguousarray(codes)).view(FP8)


def _bf16(bits):
    return torch.from_numpy(bits.astype(np.int16)).view(torch.bfloat16)


def _same(out, bits, what):
    want = _bf16(bits)
    got = out.detach().cpu().to(torch.bfloat16)
    assert got.shape == want.shape, what
    bad = (got.view(torch.int16) != want.view(torch.int16))
    assert not bad.any(), f"{what}: {int(bad.sum())} of {bad.numel()} values differ from the golden vector"


# ----------------------------------------------------------------------------- oracle (CPU)
def test_decode_table_fixture():
    want = np.load(os.path.join(HERE, "e4m3fn_decode_table.npy"))
    for got in (R.e4m3fn_decode_table(), C.decode_table()):
        got = np.asarray(got, dtype=np.float32)
        assert np.array_equal(np.isnan(got), np.isnan(want))
        assert np.array_equal(got[~np.isnan(want)].view(np.uint32), want[~np.isnan(want)].view(np.uint32))
    assert np.isnan(want[[0x7F, 0xFF]]).all() and want[0x7E] == 448.0 and want[0x01] == 2.0 ** -9


def test_oracle_per_tensor_fixture():
    z = _npz("per_tensor_24x144x256.npz")
    sa, sb = torch.tensor(float(z["scale_a"])), torch.tensor(float(z["scale_b"]))
    _same(R.ref_gemm_per_tensor(_fp8(z["a"]), _fp8(z["b"]), sa, sb, trans_b=True), z["c_bf16"], "torch oracle")
    bt = _fp8(np.ascontiguousarray(z["b"].T))
    _same(R.ref_gemm_per_tensor(_fp8(z["a"]), bt, sa, sb, trans_b=False), z["c_bf16"], "torch oracle, (K,N) weights")
    c = C.gemm_per_tensor(z["a"], z["b"], float(z["scale_a"]), float(z["scale_b"]))
    _same(torch.from_numpy(np.asarray(c, dtype=np.float32)), z["c_bf16"], "C oracle")


def test_oracle_block_scaled_fixture():
    z = _npz("block_scaled_16x256x384.npz")
    out = R.ref_w8a8_block_fp8_matmul(_fp8(z["a"]), _fp8(z["b"]), torch.from_numpy(z["a_scale"]),
                                      torch.from_numpy(z["b_scale"]), [128, 128], torch.bfloat16)
    _same(out, z["c_bf16"], "torch oracle")
    c = C.gemm_block_scaled(z["a"], z["b"], z["a_scale"], z["b_scale"])
    _same(torch.from_numpy(np.asarray(c, dtype=np.float32)), z["c_bf16"], "C oracle")


def test_oracle_ragged_fixture():
    z = _npz("ragged_3experts.npz")
    out = R.ref_ragged_block_scaled_bmm(_fp8(z["a"]), _fp8(z["b"]), torch.from_numpy(z["a_scale"]),
                                        torch.from_numpy(z["b_scale"]), torch.from_numpy(z["m_indptr"]))
    _same(out, z["c_bf16"], "torch oracle")
    c = C.gemm_ragged(z["a"], z["b"], z["a_scale"], z["b_scale"], z["m_indptr"])
    _same(torch.from_numpy(np.asarray(c, dtype=np.float32)), z["c_bf16"], "C oracle")


@pytest.mark.parametrize("mul", [False, True])
def test_oracle_moe_gather_fixture(mul):
    z = _npz("moe_gather_top2.npz")
    out = R.ref_fused_moe_gemm(_fp8(z["a"]), _fp8(z["b"]), torch.from_numpy(z["a_scale"]), torch.from_numpy(z["b_scale"]),
                               torch.from_numpy(z["topk_weights"]), torch.from_numpy(z["topk_ids"]).long(), mul, 2)
    _same(out, z["c_weighted_bf16" if mul else "c_bf16"], "torch oracle")


def test_oracle_moe_align_fixture():
    with open(os.path.join(HERE, "moe_align_known_answer.json")) as f:
        k = json.load(f)
    ids = torch.tensor(k["topk_ids"])
    s, e, post, cum, mx = R.moe_align_block_size_ref(ids, k["block_size"], k["num_experts"])
    assert s[:16].tolist() == k["sorted_token_ids_first16"] and set(s[16:].tolist()) == {k["sentinel"]}
    assert e[:4].tolist() == k["expert_ids_first4"] and int(post) == k["num_tokens_post_padded"]
    assert cum.tolist() == k["padded_cumsum"] and int(mx) == k["max_expert_count"]


# ----------------------------------------------------------------------------- HIP path (GPU)
DENSE_KERNELS = [None, {"KERNEL": "tiled", "BLOCK_M": 64, "BLOCK_N": 128}, {"KERNEL": "tiled", "BLOCK_M": 64, "BLOCK_N": 32}, {"KERNEL": "tiled", "BLOCK_M": 64, "BLOCK_N": 64},
                 {"KERNEL": "tiled", "BLOCK_M": 32, "BLOCK_N": 32}, {"KERNEL": "tiled", "BLOCK_M": 128, "BLOCK_N": 128},
                 {"KERNEL": "tiled", "BLOCK_M": 128, "BLOCK_N": 128, "SPLIT_K": 2},
                 {"KERNEL": "tiled", "BLOCK_M": 256, "BLOCK_N": 256}, {"KERNEL": "tiled", "BLOCK_M": 256, "BLOCK_N": 256, "WAVES": 8},
                 {"KERNEL": "skinny"}, {"KERNEL": "skinny", "WAVES": 8, "ROW_GROUPS": 2}, {"KERNEL": "stream"},
                 {"KERNEL": "stream", "ROW_GROUPS": 4}, {"KERNEL": "fallback"}]


@pytest.mark.gpu
@pytest.mark.parametrize("kc", DENSE_KERNELS, ids=lambda k: "auto" if k is None else "-".join(str(v) for v in k.values()))
def test_hip_per_tensor_fixture(device, kc):
    from tilegym_amd.ops import matmul

    z = _npz("per_tensor_24x144x256.npz")
    sa = torch.tensor(float(z["scale_a"]), device=device)
    sb = torch.tensor(float(z["scale_b"]), device=device)
    out = matmul(_fp8(z["a"]).to(device), _fp8(z["b"]).to(device), trans_b=True, scale_a=sa, scale_b=sb,
                 out_dtype=torch.bfloat16, kernel_configs=kc)
    _same(out, z["c_bf16"], f"HIP per-tensor {kc}")
    if kc is None:
        bt = _fp8(np.ascontiguousarray(z["b"].T)).to(device)
        out = matmul(_fp8(z["a"]).to(device), bt, scale_a=sa, scale_b=sb, out_dtype=torch.bfloat16)
        _same(out, z["c_bf16"], "HIP per-tensor, (K,N) weights")


@pytest.mark.gpu
@pytest.mark.parametrize("kc", DENSE_KERNELS, ids=lambda k: "auto" if k is None else "-".join(str(v) for v in k.values()))
def test_hip_block_scaled_fixture(device, kc):
    from tilegym_amd.suites.unsloth.ops import w8a8_block_fp8_matmul

    z = _npz("block_scaled_16x256x384.npz")
    out = w8a8_block_fp8_matmul(_fp8(z["a"]).to(device), _fp8(z["b"]).to(device), torch.from_numpy(z["a_scale"]).to(device),
                                torch.from_numpy(z["b_scale"]).to(device), [128, 128], torch.bfloat16, kernel_configs=kc)
    _same(out, z["c_bf16"], f"HIP block-scaled {kc}")


@pytest.mark.gpu
@pytest.mark.parametrize("kc", [None, {"BLOCK_M": 64, "BLOCK_N": 128}, {"BLOCK_M": 128, "BLOCK_N": 128}, {"KERNEL": "fallback"}],
                         ids=["auto", "64x128", "128x128", "fallback"])
def test_hip_ragged_fixture(device, kc):
    from tilegym_amd.suites.flashinfer.ops import ragged_block_scaled_bmm

    z = _npz("ragged_3experts.npz")
    max_m = int(np.diff(z["m_indptr"]).max())
    out = ragged_block_scaled_bmm(_fp8(z["a"]).to(device), _fp8(z["b"]).to(device), torch.from_numpy(z["a_scale"]).to(device),
                                  torch.from_numpy(z["b_scale"]).to(device), torch.from_numpy(z["m_indptr"]).to(device), max_m,
                                  out_dtype=torch.bfloat16, kernel_configs=kc)
    _same(out, z["c_bf16"], f"HIP ragged {kc}")


@pytest.mark.gpu
@pytest.mark.parametrize("mul", [False, True])
@pytest.mark.parametrize("block_m", [16, 64, 128])
def test_hip_moe_gather_fixture(device, mul, block_m):
    from tilegym_amd.ops import moe_align_block_size
    from tilegym_amd.ops.moe_interface import invoke_fused_moe_kernel

    z = _npz("moe_gather_top2.npz")
    ids = torch.from_numpy(z["topk_ids"]).to(device)
    T, top_k = ids.shape
    E, N, _ = z["b"].shape
    sorted_ids, expert_ids, post, _, _ = moe_align_block_size(ids, block_m, E)
    out = torch.zeros(T, top_k, N, dtype=torch.bfloat16, device=device)
    invoke_fused_moe_kernel(_fp8(z["a"]).to(device), _fp8(z["b"]).to(device), out, torch.from_numpy(z["a_scale"]).to(device),
                            torch.from_numpy(z["b_scale"]).to(device), torch.from_numpy(z["topk_weights"]).to(device), ids,
                            sorted_ids, expert_ids, post, mul, top_k, {"BLOCK_SIZE_M": block_m},
                            use_fp8_w8a8=True, block_shape=[128, 128])
    _same(out, z["c_weighted_bf16" if mul else "c_bf16"], f"HIP MoE gather block_m={block_m} mul={mul}")


@pytest.mark.gpu
def test_hip_moe_align_fixture(device):
    from tilegym_amd.ops import moe_align_block_size

    with open(os.path.join(HERE, "moe_align_known_answer.json")) as f:
        k = json.load(f)
    s, e, post, cum, mx = moe_align_block_size(torch.tensor(k["topk_ids"], device=device), k["block_size"], k["num_experts"])
    assert s[:16].tolist() == k["sorted_token_ids_first16"] and set(s[16:].tolist()) == {k["sentinel"]}
    assert e[:4].tolist() == k["expert_ids_first4"] and int(post) == k["num_tokens_post_padded"]
    assert cum.tolist() == k["padded_cumsum"] and int(mx) == k["max_expert_count"]
