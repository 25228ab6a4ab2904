"""Host-layer semantics that need no GPU: registry/dispatch behaviour and the op signatures."""

import inspect

import pytest
import torch

import tilegym_amd
from tilegym_amd import backend
from tilegym_amd.ops import hip as hip_impls  # noqa: F401

FP8 = torch.float8_e4m3fn


def test_registry_holds_the_hot_path_ops():
    info = tilegym_amd.get_registry_info()
    for name in ("matmul", "group_gemm", "unsloth.w8a8_block_fp8_matmul", "flashinfer.gemm.gemm_alpha_beta",
                 "flashinfer.gemm.ragged_block_scaled_bmm", "invoke_fused_moe_kernel", "moe_align_block_size"):
        assert "hip" in info[name] and "default" in info[name]


def test_backend_selection():
    assert tilegym_amd.get_current_backend() == "hip"
    assert tilegym_amd.is_backend_available("hip")
    assert not tilegym_amd.is_backend_available("cutile")
    with pytest.raises(ValueError):
        tilegym_amd.set_backend("cutile")
    tilegym_amd.set_backend("hip")


def test_dispatch_semantics():
    calls = []

    @backend.dispatch("unit.test_op")
    def op(x, y=1, **kwargs):
        raise NotImplementedError("stub")

    with pytest.raises(NotImplementedError):
        op(1)

    @backend.register_impl("unit.test_op", backend="hip")
    def impl(x, y=1, **kwargs):
        calls.append((x, y, kwargs))
        return x + y

    assert op(2, y=3, extra=5) == 5 and calls[-1] == (2, 3, {"extra": 5})
    assert op(2, backend="hip") == 3            # explicit backend kwarg is consumed
    assert "backend" not in calls[-1][2]
    with pytest.raises(NotImplementedError):
        op(2, backend="triton")
    assert op._tilegym_op_name == "unit.test_op"
    assert backend.get_available_backends_for_op("unit.test_op") == ["hip"]


def test_signatures_match_the_reference_stubs():
    from tilegym_amd.ops import group_gemm, matmul
    from tilegym_amd.ops.moe_interface import invoke_fused_moe_kernel
    from tilegym_amd.suites.flashinfer.ops import gemm_alpha_beta, ragged_block_scaled_bmm
    from tilegym_amd.suites.unsloth.ops import w8a8_block_fp8_matmul

    def names(f):
        return list(inspect.signature(f).parameters)

    assert names(matmul) == ["a", "b", "trans_a", "trans_b", "static_persistent", "use_tma", "kwargs"]
    assert names(group_gemm) == ["group_A", "group_B", "static_persistent", "use_tma", "kwargs"]
    assert names(w8a8_block_fp8_matmul) == ["A", "B", "As", "Bs", "block_size", "output_dtype"]
    assert inspect.signature(w8a8_block_fp8_matmul).parameters["output_dtype"].default == torch.float32
    assert names(gemm_alpha_beta) == ["a", "b", "c", "trans_a", "trans_b", "alpha", "beta", "num_sms"]
    assert names(ragged_block_scaled_bmm) == ["a", "b", "a_scale", "b_scale", "m_indptr", "max_m",
                                              "max_m_device", "transpose_a", "transpose_b", "out_dtype"]
    assert names(invoke_fused_moe_kernel)[:12] == ["A", "B", "C", "A_scale", "B_scale", "topk_weights", "topk_ids",
                                                   "sorted_token_ids", "expert_ids", "num_tokens_post_padded",
                                                   "mul_routed_weight", "top_k"]


def test_install_as_tilegym_aliases_import_paths():
    tilegym_amd.install_as_tilegym()
    import tilegym
    from tilegym.suites import flashinfer, unsloth  # noqa: F401
    from tilegym.ops.moe_interface import invoke_fused_moe_kernel  # noqa: F401

    assert tilegym.ops.matmul is tilegym_amd.ops.matmul
    assert unsloth.ops.w8a8_block_fp8_matmul is tilegym_amd.suites.unsloth.ops.w8a8_block_fp8_matmul
    assert hasattr(flashinfer.ops, "ragged_block_scaled_bmm")


def test_host_side_errors_mirror_the_reference():
    from tilegym_amd.ops import group_gemm, matmul
    from tilegym_amd.suites.flashinfer.ops import ragged_block_scaled_bmm
    from tilegym_amd.suites.unsloth.ops import w8a8_block_fp8_matmul

    a = torch.zeros(4, 128).to(FP8)
    b = torch.zeros(8, 64).to(FP8)
    with pytest.raises(AssertionError):
        matmul(a, b, trans_b=True)                      # K mismatch asserts, as in the reference
    with pytest.raises(NotImplementedError):
        matmul(a.float(), a.float())                    # only e4m3 here
    with pytest.raises(ValueError):
        group_gemm([], [])
    with pytest.raises(ValueError):
        group_gemm([a], [a, a])
    with pytest.raises(AssertionError):
        w8a8_block_fp8_matmul(a, torch.zeros(8, 128).to(FP8), torch.ones(4, 2), torch.ones(1, 1))
    with pytest.raises(AssertionError):
        ragged_block_scaled_bmm(a, torch.zeros(2, 128, 128).to(FP8), None, torch.ones(2, 1, 1),
                                torch.zeros(3, dtype=torch.int32), 4, transpose_b=False)
    # a CPU tensor never silently computes: there is no CPU path
    with pytest.raises(RuntimeError, match="no CPU implementation"):
        matmul(a, torch.zeros(8, 128).to(FP8), trans_b=True, out_dtype=torch.bfloat16)


def test_quantizer_operators_have_no_host_path():
    from tilegym_amd.suites.flashinfer.ops import per_token_group_quant_8bit
    from tilegym_amd.suites.unsloth.ops import act_quant, weight_dequant

    x = torch.zeros(4, 256, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="HIP device"):
        act_quant(x, 128)
    with pytest.raises(RuntimeError, match="HIP device"):
        per_token_group_quant_8bit(x, 64)
    with pytest.raises(RuntimeError, match="HIP device"):
        weight_dequant(torch.zeros(128, 128).to(FP8), torch.ones(1, 1))
    with pytest.raises(AssertionError):
        act_quant(x, 96)                                               # last dim not divisible
    with pytest.raises(AssertionError):
        per_token_group_quant_8bit(x, 64, scale_ue8m0=True)            # needs column_major_scales, as in the reference
    with pytest.raises(NotImplementedError):
        per_token_group_quant_8bit(x, 64, dst_dtype=torch.int16)       # e4m3 and int8 destinations only
    with pytest.raises(RuntimeError, match="HIP device"):
        per_token_group_quant_8bit(x, 64, dst_dtype=torch.int8)


def test_moe_align_has_no_cpu_path():
    from tilegym_amd.ops import moe_align_block_size

    ids = torch.tensor([[2, 3, 4], [1, 2, 4], [1, 3, 4], [1, 2, 3]]) - 1
    with pytest.raises(RuntimeError, match="device tensors only"):
        moe_align_block_size(ids, 4, 4)  # no CPU path in the product


def test_ops_are_registered_with_torchs_dispatcher():
    """torch.ops.tilegym_hip.* exist after importing the package, carry schemas, infer output shapes without a GPU
    (fake tensors), and refuse CPU tensors (there is no CPU implementation)."""
    import torch
    from torch._subclasses.fake_tensor import FakeTensorMode

    import tilegym_amd  # noqa: F401
    from tilegym_amd import torch_ops

    assert torch_ops.registered_ops() == [f"tilegym_hip::{n}" for n in torch_ops.OP_NAMES]
    schema = str(torch.ops.tilegym_hip.fp8_gemm.default._schema)
    assert "Tensor? scale_a" in schema and "ScalarType out_dtype" in schema and schema.endswith("-> Tensor")
    assert "Tensor(a0!) c" in str(torch.ops.tilegym_hip.fp8_gemm_out.default._schema)
    fp8 = torch.float8_e4m3fn
    with FakeTensorMode():
        a = torch.empty(8, 256, dtype=fp8, device="cuda")
        b = torch.empty(512, 256, dtype=fp8, device="cuda")
        c = torch.ops.tilegym_hip.fp8_gemm(a, b, None, None, False, True, 1.0, torch.bfloat16)
        assert tuple(c.shape) == (8, 512) and c.dtype == torch.bfloat16
        c = torch.ops.tilegym_hip.fp8_gemm(a.t(), b.t(), None, None, True, False, 1.0, torch.float32)
        assert tuple(c.shape) == (8, 512) and c.dtype == torch.float32
        w = torch.empty(4, 384, 256, dtype=fp8, device="cuda")
        r = torch.ops.tilegym_hip.fp8_ragged_gemm(a, w, None, torch.empty(4, 3, 2, device="cuda"),
                                                  torch.empty(5, dtype=torch.int32, device="cuda"), torch.bfloat16)
        assert tuple(r.shape) == (8, 384)
        q, s = torch.ops.tilegym_hip.fp8_quant_1x128(torch.empty(4, 3, 256, dtype=torch.bfloat16, device="cuda"))
        assert q.dtype == fp8 and tuple(q.shape) == (4, 3, 256) and tuple(s.shape) == (4, 3, 2)
        y = torch.ops.tilegym_hip.fp8_fused_moe(torch.empty(5, 256, dtype=torch.float16, device="cuda"), torch.empty(4, 512, 256, dtype=fp8, device="cuda"),
                                                torch.empty(4, 256, 256, dtype=fp8, device="cuda"), torch.empty(4, 4, 2, device="cuda"),
                                                torch.empty(4, 2, 2, device="cuda"), torch.empty(5, 2, device="cuda"),
                                                torch.empty(5, 2, dtype=torch.int64, device="cuda"))
        assert tuple(y.shape) == (5, 256) and y.dtype == torch.float16
    x = torch.zeros(8, 256).to(fp8)
    import pytest
    with pytest.raises(NotImplementedError):
        torch.ops.tilegym_hip.fp8_gemm(x, x, None, None, False, True, 1.0, torch.bfloat16)


def test_release_workspaces_empties_the_cache():
    from tilegym_amd import _lib
    _lib._workspaces[(0, 0, False)] = [__import__("torch").empty(1024, dtype=__import__("torch").uint8)]
    assert _lib.release_workspaces() == 1024 and not _lib._workspaces


def test_recorded_schedule_table_round_trip(tmp_path):
    """tilegym_amd.tune writes a table, _lib reads it: entries are kernel_configs per (M, N, K, block-scaled?), entries
    whose best schedule is the automatic one are dropped, a later run merges, and an unknown shape gets the automatic cfg."""
    from tilegym_amd import _lib, tune

    path = str(tmp_path / "tune.json")
    tune.write_table([{"M": 16, "N": 5120, "K": 12288, "block_scaled": False, "kernel_configs": {"KERNEL": "stream", "ROW_GROUPS": 4, "SPLIT_K": 6},
                       "us": 14.5, "auto_us": 16.0, "auto_schedule": {}},
                      {"M": 1, "N": 4096, "K": 4096, "block_scaled": True, "kernel_configs": {}, "us": 6.3, "auto_us": 6.3, "auto_schedule": {}}], path)
    tune.write_table([{"M": 8, "N": 4096, "K": 11008, "block_scaled": True, "kernel_configs": {"KERNEL": "stream", "WAVES": 8},
                       "us": 14.0, "auto_us": 14.6, "auto_schedule": {}}], path)
    try:
        table = _lib.load_tune_table(path)
        assert set(table) == {(16, 5120, 12288, False), (8, 4096, 11008, True)}
        cfg, n = _lib._tuned_cfg(16, 5120, 12288, False)
        assert n == _lib.TG_CFG_COUNT and cfg[_lib.CFG_SLOTS["KERNEL"]] == 3 and cfg[_lib.CFG_SLOTS["SPLIT_K"]] == 6
        assert cfg[_lib.CFG_SLOTS["ROW_GROUPS"]] == 4 and cfg[_lib.CFG_SLOTS["WAVES"]] == -1
        auto, _ = _lib._tuned_cfg(16, 5120, 12288, True)   # same shape, other scaling: not in the table
        assert all(auto[i] == -1 for i in range(_lib.TG_CFG_COUNT))
    finally:
        assert _lib.load_tune_table("") == {}
    assert [c for c in tune.candidates(1, 4096, 4096, False) if c["KERNEL"] == "tiled"] == []
    assert {"KERNEL": "tiled", "BLOCK_M": 256, "BLOCK_N": 256, "SPLIT_K": 1} in tune.candidates(4096, 4096, 4096, True)
    assert tune._parse_shape("8,4096,11008,block") == (8, 4096, 11008, True) and tune._parse_shape("8,4096,11008") == (8, 4096, 11008, False)
