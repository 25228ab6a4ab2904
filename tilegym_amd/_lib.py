"""ctypes binding of libtilegym_hip.so: tensor descriptors, return-code checks, workspaces.

This is the only module that touches the shared library.  It never falls back to another
implementation: if the library is missing or a call fails, it raises.

The descriptor / return-code conventions follow the reference's own C-ABI precedent
(src/tilegym/backend/cutile_rs/utils.py:268-290 ``make_tensor_desc``, :353-370 ``check_rc``).
"""

from __future__ import annotations

import ctypes
import struct
import weakref
import os
from typing import Dict, Optional, Sequence, Tuple

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_ENV = "TILEGYM_HIP_LIB"
DEFAULT_LIB_PATH = os.path.join(_HERE, "libtilegym_hip.so")

TG_MAX_DIMS = 5
TG_CFG_COUNT = 9
CFG_SLOTS = {"KERNEL": 0, "BLOCK_M": 1, "BLOCK_N": 2, "SPLIT_K": 3, "ROW_GROUPS": 4, "WAVES": 5,
             "QUANT_BLOCK_N": 6, "QUANT_BLOCK_K": 7, "PIECES": 8}
KERNEL_NAMES = {0: "fallback", 1: "tiled", 2: "skinny", 3: "stream"}

# dtype codes of the ABI (include/tilegym_hip.h)
_DTYPE_CODES = {
    torch.float32: 0,
    torch.float16: 1,
    torch.bfloat16: 2,
    torch.int32: 3,
    torch.int64: 4,
    torch.float8_e5m2: 5,
    torch.uint8: 6,
    torch.float8_e4m3fn: 7,
    torch.int8: 8,
}

_RC_NAMES = {0: "ok", -2: "unsupported dtype", -3: "kernel launch failed", -4: "device init failed",
             -5: "null tensor pointer", -6: "invalid arguments"}


class TgTensor(ctypes.Structure):
    _fields_ = [
        ("ptr", ctypes.c_uint64),
        ("ndim", ctypes.c_int32),
        ("shape", ctypes.c_int64 * TG_MAX_DIMS),
        ("strides", ctypes.c_int64 * TG_MAX_DIMS),
        ("dtype", ctypes.c_int32),
    ]


class TileGymHipError(RuntimeError):
    def __init__(self, rc: int, where: str, detail: str):
        self.rc = rc
        msg = f"{where}: rc={rc} ({_RC_NAMES.get(rc, 'unknown error')})"
        if detail:
            msg += f": {detail}"
        super().__init__(msg)


_lib = None


def lib_path() -> str:
    return os.environ.get(LIB_ENV, DEFAULT_LIB_PATH)


def is_built() -> bool:
    return os.path.exists(lib_path())


def load():
    """Load the shared library (once).  Raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    path = lib_path()
    if not os.path.exists(path):
        raise RuntimeError(
            f"libtilegym_hip.so not found at {path}; build it with "
            f"`python -m tilegym_amd.build` (hipcc, gfx950). There is no fallback implementation.")
    L = ctypes.CDLL(path)
    P = ctypes.c_void_p  # const tg_tensor*: a packed descriptor (bytes, see _desc) or ctypes.byref(TgTensor)
    I32P = ctypes.POINTER(ctypes.c_int32)
    L.tg_abi_version.restype = ctypes.c_int32
    L.tg_rc_message.restype = ctypes.c_char_p
    L.tg_rc_message.argtypes = [ctypes.c_int32]
    L.tg_last_error.restype = ctypes.c_char_p
    L.tg_last_config.restype = ctypes.c_int32
    L.tg_last_config.argtypes = [I32P, ctypes.c_int32]
    L.tg_fp8_gemm_workspace_bytes.restype = ctypes.c_int64
    L.tg_fp8_gemm_workspace_bytes.argtypes = [ctypes.c_int64, ctypes.c_int64, ctypes.c_int64,
                                              ctypes.c_int32, I32P, ctypes.c_int32]
    L.tg_fp8_gemm.restype = ctypes.c_int32
    L.tg_fp8_gemm.argtypes = [P, P, P, P, P, ctypes.c_int32, ctypes.c_int32, ctypes.c_float,
                              ctypes.c_float, P, I32P, ctypes.c_int32, ctypes.c_int32, ctypes.c_uint64]
    L.tg_fp8_gemm_static_scratch.restype = ctypes.c_int32
    L.tg_fp8_gemm_static_scratch.argtypes = [P, P, P, P, P, ctypes.c_int32, ctypes.c_int32, ctypes.c_float,
                                             ctypes.c_float, I32P, ctypes.c_int32, ctypes.c_int32, ctypes.c_uint64]
    L.tg_fp8_ragged_gemm.restype = ctypes.c_int32
    L.tg_fp8_ragged_gemm.argtypes = [P, P, P, P, P, P, I32P, ctypes.c_int32, ctypes.c_int32, ctypes.c_uint64]
    L.tg_fp8_moe_gemm.restype = ctypes.c_int32
    L.tg_fp8_moe_gemm.argtypes = [P, P, P, P, P, P, P, P, P, ctypes.c_int32, ctypes.c_int32,
                                  ctypes.c_int32, I32P, ctypes.c_int32, ctypes.c_int32, ctypes.c_uint64]
    L.tg_fp8_moe_gemm_silu_quant.restype = ctypes.c_int32
    L.tg_fp8_moe_gemm_silu_quant.argtypes = [P, P, P, P, P, P, P, P, P, ctypes.c_int32, ctypes.c_int32, ctypes.c_int32,
                                             ctypes.c_int32, ctypes.c_uint64]
    L.tg_moe_align_block_size.restype = ctypes.c_int32
    L.tg_moe_align_block_size.argtypes = [P, ctypes.c_int32, ctypes.c_int32, P, P, P, P, P, ctypes.c_int32, ctypes.c_uint64]
    L.tg_moe_align_quant_1x128.restype = ctypes.c_int32
    L.tg_moe_align_quant_1x128.argtypes = [P, ctypes.c_int32, ctypes.c_int32, P, P, P, P, P, P, P, P, ctypes.c_int32, ctypes.c_uint64]
    L.tg_fp8_quant_1x128.restype = ctypes.c_int32
    L.tg_fp8_quant_1x128.argtypes = [P, P, P, ctypes.c_float, ctypes.c_int32, ctypes.c_int32, ctypes.c_uint64]
    L.tg_fp8_quant_group.restype = ctypes.c_int32
    L.tg_fp8_quant_group.argtypes = [P, P, P, ctypes.c_int32, ctypes.c_float, ctypes.c_int32, ctypes.c_int32, ctypes.c_uint64]
    L.tg_fp8_weight_dequant.restype = ctypes.c_int32
    L.tg_fp8_weight_dequant.argtypes = [P, P, P, ctypes.c_int32, ctypes.c_int32, ctypes.c_uint64]
    L.tg_silu_mul_quant_1x128.restype = ctypes.c_int32
    L.tg_silu_mul_quant_1x128.argtypes = [P, P, P, ctypes.c_int32, ctypes.c_uint64]
    L.tg_moe_sum.restype = ctypes.c_int32
    L.tg_moe_sum.argtypes = [P, P, ctypes.c_int32, ctypes.c_uint64]
    L.tg_fp8_fused_moe_workspace_bytes.restype = ctypes.c_int64
    L.tg_fp8_fused_moe_workspace_bytes.argtypes = [ctypes.c_int64] * 5 + [ctypes.c_int32]
    L.tg_fp8_fused_moe.restype = ctypes.c_int32
    L.tg_fp8_fused_moe.argtypes = [P] * 9 + [ctypes.c_int32, ctypes.c_int32, ctypes.c_uint64]
    PP = ctypes.POINTER(ctypes.POINTER(TgTensor))
    L.tg_fp8_group_gemm.restype = ctypes.c_int32
    L.tg_fp8_group_gemm.argtypes = [PP, PP, PP, PP, PP, ctypes.c_int32, ctypes.c_int32, P, I32P, ctypes.c_int32,
                                    ctypes.c_int32, ctypes.c_uint64]
    L.tg_diag_read.restype = ctypes.c_int32
    L.tg_diag_read.argtypes = [P, P, ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_uint64]
    L.tg_diag_mfma.restype = ctypes.c_int32
    L.tg_diag_mfma.argtypes = [ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, P, ctypes.c_int32, ctypes.c_uint64]
    if L.tg_abi_version() != 1:
        raise RuntimeError(f"libtilegym_hip.so ABI version {L.tg_abi_version()} != 1")
    _lib = L
    return L


def make_tensor_desc(t: Optional[torch.Tensor]) -> Optional[TgTensor]:
    """Borrowed descriptor of a torch tensor (strides in elements); ``None`` -> ``None``."""
    if t is None:
        return None
    if t.dim() > TG_MAX_DIMS:
        raise ValueError(f"tensor rank {t.dim()} exceeds {TG_MAX_DIMS}")
    code = _DTYPE_CODES.get(t.dtype)
    if code is None:
        raise TypeError(f"dtype {t.dtype} has no ABI code")
    d = TgTensor()
    d.ptr = t.data_ptr()
    d.ndim = t.dim()
    for i, (s, st) in enumerate(zip(t.shape, t.stride())):
        d.shape[i] = s
        d.strides[i] = st
    d.dtype = code
    return d


_DESC_PACK = struct.Struct("=Qi4x5q5qi4x")  # the bytes of a TgTensor: ptr, ndim, pad, shape[5], strides[5], dtype, pad
assert _DESC_PACK.size == ctypes.sizeof(TgTensor)


def _desc(t: Optional[torch.Tensor]) -> Optional[bytes]:
    """make_tensor_desc for the call paths: the same descriptor as packed bytes (ctypes passes a bytes object to a
    ``const tg_tensor*`` parameter as a pointer to its buffer), built in one struct.pack instead of a dozen ctypes field
    assignments -- 0.75 us against 1.9 us, on calls that take up to nine of them."""
    if t is None:
        return None
    code = _DTYPE_CODES.get(t.dtype)
    if code is None:
        raise TypeError(f"dtype {t.dtype} has no ABI code")
    sh, st = t.shape, t.stride()
    nd = len(sh)
    if nd == 2:
        return _DESC_PACK.pack(t.data_ptr(), 2, sh[0], sh[1], 0, 0, 0, st[0], st[1], 0, 0, 0, code)
    if nd == 1:
        return _DESC_PACK.pack(t.data_ptr(), 1, sh[0], 0, 0, 0, 0, st[0], 0, 0, 0, 0, code)
    if nd == 3:
        return _DESC_PACK.pack(t.data_ptr(), 3, sh[0], sh[1], sh[2], 0, 0, st[0], st[1], st[2], 0, 0, code)
    if nd > TG_MAX_DIMS:
        raise ValueError(f"tensor rank {nd} exceeds {TG_MAX_DIMS}")
    pad = (0,) * (TG_MAX_DIMS - nd)
    return _DESC_PACK.pack(t.data_ptr(), nd, *sh, *pad, *st, *pad, code)


def _ref(d):
    """What to hand to a ``const tg_tensor*`` parameter: packed bytes as they are, a TgTensor by reference."""
    return d if d is None or isinstance(d, bytes) else ctypes.byref(d)


def make_cfg(kernel_configs: Optional[dict]):
    """``kernel_configs={...}`` (the reference's per-call override, src/tilegym/kernel_utils.py:14-36)
    -> (int32 array, length).  Keys: KERNEL ('fallback'|'tiled'|'skinny' or 0/1/2), BLOCK_M, BLOCK_N,
    SPLIT_K, ROW_GROUPS, WAVES, QUANT_BLOCK_N, QUANT_BLOCK_K; unknown keys (e.g. num_ctas, occupancy) are ignored."""
    arr = (ctypes.c_int32 * TG_CFG_COUNT)(*([-1] * TG_CFG_COUNT))
    if kernel_configs:
        for key, val in kernel_configs.items():
            slot = CFG_SLOTS.get(str(key).upper())
            if slot is None or val is None:
                continue
            if slot == 0 and isinstance(val, str):
                val = {v: k for k, v in KERNEL_NAMES.items()}[val]
            arr[slot] = int(val)
    return arr, TG_CFG_COUNT


_default_cfg_pair = None


def _cfg(kernel_configs: Optional[dict]):
    """make_cfg, with the all-automatic array built once (the library only reads it)."""
    global _default_cfg_pair
    if kernel_configs:
        return make_cfg(kernel_configs)
    if _default_cfg_pair is None:
        _default_cfg_pair = make_cfg(None)
    return _default_cfg_pair


def check_rc(rc: int, where: str) -> None:
    if rc != 0:
        detail = load().tg_last_error().decode("utf-8", "replace")
        raise TileGymHipError(rc, where, detail)


def last_config() -> Dict[str, int]:
    """Schedule chosen by the most recent GEMM call on this thread."""
    out = (ctypes.c_int32 * TG_CFG_COUNT)()
    load().tg_last_config(out, TG_CFG_COUNT)
    d = {name: int(out[slot]) for name, slot in CFG_SLOTS.items()}
    d["KERNEL_NAME"] = KERNEL_NAMES.get(d["KERNEL"], "?")
    return d


# ---------------------------------------------------------------------------- workspaces
# (device, stream handle, under capture?) -> every scratch tensor ever handed out for that key, newest last.
# tg_fp8_gemm bakes the raw workspace pointer into whatever it enqueues, and a HIP graph captured from such
# a call keeps writing split-K partial sums there on every replay; a buffer that is replaced by a larger
# one is therefore kept alive for the life of the process instead of going back to the allocator (where
# another tensor could receive the block while a graph still writes to it).  Buffers at least double, so a
# key holds a handful.
_workspaces: Dict[Tuple[int, int, bool], list] = {}
_WS_MIN_BYTES = 1 << 20


def _raw_stream(index: int) -> int:
    """Handle of torch's current stream on device `index` (what ``torch.cuda.current_stream(d).cuda_stream`` returns,
    without building a Stream object: this is on the path of every call)."""
    return torch._C._cuda_getCurrentRawStream(index)


def workspace_for(device: torch.device, nbytes: int, index: Optional[int] = None, stream: Optional[int] = None) -> Optional[torch.Tensor]:
    """Scratch buffer for the current stream of ``device`` (grown on demand, never freed).  One live buffer
    per (device, stream): calls on one stream are ordered, so they can share it.  Calls made while the
    stream is being captured get buffers of their own (allocated from the capturing graph's pool and kept
    alive here too), so eager calls and graph replays never share scratch memory."""
    if nbytes <= 0:
        return None
    if index is None:
        index = device.index if device.index is not None else torch.cuda.current_device()
    if stream is None:
        stream = _raw_stream(index)
    key = (index, stream, torch.cuda.is_current_stream_capturing())
    held = _workspaces.get(key)
    if held is None:
        held = _workspaces.setdefault(key, [])
    if held and held[-1].numel() >= nbytes:
        return held[-1]
    size = max(int(nbytes), _WS_MIN_BYTES, 2 * held[-1].numel() if held else 0)
    ws = torch.empty(size, dtype=torch.uint8, device=device)
    held.append(ws)
    return ws


def release_workspaces() -> int:
    """Drop every scratch buffer held for the GEMM calls and return the number of bytes released.  Only for callers who
    know that no HIP graph captured from these calls will be replayed again (a graph keeps writing to the buffer it was
    captured with) and that no call is in flight; the next call allocates afresh."""
    freed = sum(t.numel() for held in _workspaces.values() for t in held)
    _workspaces.clear()
    return freed


def workspace_bytes(M: int, N: int, K: int, trans_b: bool, cfg, ncfg) -> int:
    return int(load().tg_fp8_gemm_workspace_bytes(M, N, K, 1 if trans_b else 0, cfg, ncfg))


def _device_index(t: torch.Tensor) -> int:
    if not t.is_cuda:
        raise RuntimeError("tilegym_amd FP8 GEMM needs tensors on a HIP device (got a CPU tensor); "
                           "there is no CPU implementation")
    return t.device.index if t.device.index is not None else torch.cuda.current_device()


def _stream_handle(t: torch.Tensor) -> int:
    index = t.device.index
    return _raw_stream(index if index is not None else torch.cuda.current_device())


# ---------------------------------------------------------------------------- raw calls
# tg_fp8_gemm is called with the same weights, and often with the same activation and output buffers, over and over by
# a decode loop, and building six descriptors, the cfg array and the workspace size costs more host time (~15 us) than a
# small decode kernel runs (6 - 20 us).  Two caches take most of that away:
#   * per call: the prepared arguments of a call whose five tensors are the very objects of an earlier call, keyed by
#     their identities.  A hit is checked on every use (weak references to the tensors, their data pointers, shapes and strides),
#     so a tensor that was freed, resized or given new storage is described afresh; a key whose entry keeps failing that
#     check (Python hands the address of a freed tensor object to the next one, so fresh outputs repeat ids) is marked
#     volatile and no longer kept;
#   * per weight: the descriptors of b and scale_b, keyed and checked the same way, for calls whose activations and
#     outputs are fresh tensors every time; and the workspace size per (M, N, K, trans_b).
_gemm_calls: Dict[tuple, object] = {}
_weight_descs: Dict[int, tuple] = {}
_ws_bytes: Dict[tuple, int] = {}
_CACHE_MAX = 4096
_VOLATILE = object()


def _same(ref, ptr, t) -> bool:
    return (t is None) if ref is None else (ref() is t and t.data_ptr() == ptr)


def _weight_desc(t):
    """Descriptor of a long-lived tensor (None -> None), cached by identity and checked against the object's current
    storage, shape and strides."""
    if t is None:
        return None
    hit = _weight_descs.get(id(t))
    if hit is not None and hit[0]() is t and t.data_ptr() == hit[1] and t.shape == hit[2] and t.stride() == hit[3]:
        return hit[4]
    d = _desc(t)
    if len(_weight_descs) >= _CACHE_MAX:
        _weight_descs.clear()
    _weight_descs[id(t)] = (weakref.ref(t), t.data_ptr(), t.shape, t.stride(), d)
    return d


# ---- recorded schedules: TILEGYM_HIP_TUNE names a JSON file written by ``python -m tilegym_amd.tune`` that maps
# (M, N, K, block-scaled?) to the kernel_configs that measured fastest on this GPU; a call without kernel_configs of its own
# takes the recorded ones (the reference keeps per-architecture config tables and a search for the same purpose,
# src/tilegym/ops/cutile/matmul.py:47-141,327-418).  Without the variable nothing is looked up.
TUNE_ENV = "TILEGYM_HIP_TUNE"
_tune_table: Optional[Dict[tuple, dict]] = None


def load_tune_table(path: Optional[str] = None) -> Dict[tuple, dict]:
    """(Re)load the schedule table from ``path`` (default: the file TILEGYM_HIP_TUNE names; no file -> empty table) and forget
    the prepared calls that were made under the previous one."""
    global _tune_table
    import json
    path = path if path is not None else os.environ.get(TUNE_ENV)
    table: Dict[tuple, dict] = {}
    if path:
        with open(path) as f:
            doc = json.load(f)
        for e in doc.get("entries", []):
            table[(int(e["M"]), int(e["N"]), int(e["K"]), bool(e.get("block_scaled", False)))] = dict(e["kernel_configs"])
    _tune_table = table
    _gemm_calls.clear()
    _ws_bytes.clear()
    return table


def _tuned_cfg(M: int, N: int, K: int, block_scaled: bool):
    """(cfg array, length) for a dense problem: the recorded schedule if there is one, else all-automatic."""
    table = _tune_table if _tune_table is not None else load_tune_table()
    if table:
        kc = table.get((M, N, K, block_scaled))
        if kc:
            return make_cfg(kc)
    return _cfg(None)


def _gemm_constants(a, b, scale_b, trans_a, trans_b, use_workspace):
    M = a.shape[1] if trans_a else a.shape[0]
    K = a.shape[0] if trans_a else a.shape[1]
    N = b.shape[0] if trans_b else b.shape[1]
    cfg, ncfg = _tuned_cfg(M, N, K, scale_b is not None and scale_b.numel() > 1)
    ws_bytes = 0
    if use_workspace and M > 0 and N > 0 and K > 0:
        key = (M, N, K, trans_b, cfg is _cfg(None)[0])
        ws_bytes = _ws_bytes.get(key) if key[4] else None   # (a recorded schedule may ask for another split)
        if ws_bytes is None:
            if len(_ws_bytes) >= _CACHE_MAX:
                _ws_bytes.clear()
            ws_bytes = workspace_bytes(M, N, K, trans_b, cfg, ncfg)
            if key[4]:
                _ws_bytes[key] = ws_bytes
    return cfg, ncfg, ws_bytes


def _prepared_gemm(c, a, b, scale_a, scale_b, trans_a, trans_b, use_workspace):
    """(argument references, cfg, ncfg, device index, workspace bytes, device, keep-alive) of a call without kernel_configs."""
    key = (id(c), id(a), id(b), id(scale_a), id(scale_b), trans_a, trans_b, use_workspace)
    hit = _gemm_calls.get(key)
    if hit is not None and hit is not _VOLATILE:
        refs, ptrs, shapes = hit[0], hit[1], hit[2]
        if (_same(refs[0], ptrs[0], c) and _same(refs[1], ptrs[1], a) and _same(refs[2], ptrs[2], b)
                and _same(refs[3], ptrs[3], scale_a) and _same(refs[4], ptrs[4], scale_b)
                and c.shape == shapes[0] and a.shape == shapes[1] and b.shape == shapes[2]
                and c.stride() == shapes[3] and a.stride() == shapes[4] and b.stride() == shapes[5]):
            return hit[3]
        hit[4][0] += 1
    dev = _device_index(a)
    cfg, ncfg, ws_bytes = _gemm_constants(a, b, scale_b, trans_a, trans_b, use_workspace)
    if hit is _VOLATILE or (hit is not None and hit[4][0] >= 2):
        _gemm_calls[key] = _VOLATILE
        descs = (_desc(c), _desc(a), _weight_desc(b), _desc(scale_a), _weight_desc(scale_b))
        return tuple(_ref(d) for d in descs), cfg, ncfg, dev, ws_bytes, a.device, descs
    tensors = (c, a, b, scale_a, scale_b)
    descs = (_desc(c), _desc(a), _weight_desc(b), _desc(scale_a), _weight_desc(scale_b))
    prepared = (tuple(_ref(d) for d in descs), cfg, ncfg, dev, ws_bytes, a.device, descs)
    if len(_gemm_calls) >= _CACHE_MAX:
        _gemm_calls.clear()
    _gemm_calls[key] = (tuple(None if t is None else weakref.ref(t) for t in tensors),
                        tuple(0 if t is None else t.data_ptr() for t in tensors),
                        (c.shape, a.shape, b.shape, c.stride(), a.stride(), b.stride()), prepared,
                        hit[4] if hit is not None else [0])
    return prepared


def release_call_caches() -> None:
    """Forget every prepared call and cached descriptor (they hold no tensor alive; this only frees the bookkeeping)."""
    _gemm_calls.clear()
    _weight_descs.clear()
    _ws_bytes.clear()


def fp8_gemm(c, a, b, scale_a=None, scale_b=None, trans_a=False, trans_b=True, alpha=1.0, beta=0.0,
             kernel_configs=None, use_workspace=True) -> None:
    L = _lib if _lib is not None else load()
    if kernel_configs is None:
        refs, cfg, ncfg, dev, ws_bytes, device, _ = _prepared_gemm(c, a, b, scale_a, scale_b, bool(trans_a), bool(trans_b),
                                                                   bool(use_workspace))
        stream = _raw_stream(dev)
        dws = None
        if ws_bytes > 0:
            dws = _ref(_weight_desc(workspace_for(device, ws_bytes, dev, stream)))
        rc = L.tg_fp8_gemm(refs[0], refs[1], refs[2], refs[3], refs[4], 1 if trans_a else 0, 1 if trans_b else 0,
                           alpha if type(alpha) is float else float(alpha), beta if type(beta) is float else float(beta),
                           dws, cfg, ncfg, dev, stream)
        if rc != 0:
            check_rc(rc, "tg_fp8_gemm")
        return
    dev = _device_index(a)
    cfg, ncfg = make_cfg(kernel_configs)
    M = a.shape[1] if trans_a else a.shape[0]
    K = a.shape[0] if trans_a else a.shape[1]
    N = b.shape[0] if trans_b else b.shape[1]
    ws = None
    if use_workspace and M > 0 and N > 0 and K > 0:
        ws = workspace_for(a.device, workspace_bytes(M, N, K, trans_b, cfg, ncfg))
    dc, da, db = _desc(c), _desc(a), _desc(b)
    dsa, dsb, dws = _desc(scale_a), _desc(scale_b), _desc(ws)
    rc = L.tg_fp8_gemm(_ref(dc), _ref(da), _ref(db), _ref(dsa), _ref(dsb), int(bool(trans_a)),
                       int(bool(trans_b)), float(alpha), float(beta), _ref(dws), cfg, ncfg, dev,
                       _stream_handle(a))
    check_rc(rc, "tg_fp8_gemm")


STATIC_SCRATCH_BYTES = 32 * 1024 * 1024


def fp8_gemm_static_scratch(c, a, b, scale_a=None, scale_b=None, trans_a=False, trans_b=True, alpha=1.0, beta=0.0,
                            kernel_configs=None) -> None:
    """tg_fp8_gemm_static_scratch: tg_fp8_gemm whose scratch is an array inside the library (no allocation
    anywhere on the way; problems that need more than STATIC_SCRATCH_BYTES raise)."""
    L = load()
    dev = _device_index(a)
    cfg, ncfg = make_cfg(kernel_configs)
    dc, da, db = _desc(c), _desc(a), _desc(b)
    dsa, dsb = _desc(scale_a), _desc(scale_b)
    rc = L.tg_fp8_gemm_static_scratch(_ref(dc), _ref(da), _ref(db), _ref(dsa), _ref(dsb), int(bool(trans_a)),
                                      int(bool(trans_b)), float(alpha), float(beta), cfg, ncfg, dev, _stream_handle(a))
    check_rc(rc, "tg_fp8_gemm_static_scratch")


def fp8_ragged_gemm(c, a, b, a_scale, b_scale, m_indptr, kernel_configs=None) -> None:
    L = load()
    dev = _device_index(a)
    cfg, ncfg = _cfg(kernel_configs)
    rc = L.tg_fp8_ragged_gemm(_desc(c), _desc(a), _weight_desc(b), _desc(a_scale), _weight_desc(b_scale), _desc(m_indptr),
                              cfg, ncfg, dev, _stream_handle(a))
    check_rc(rc, "tg_fp8_ragged_gemm")


def fp8_moe_gemm(c, a, b, a_scale, b_scale, topk_weights, sorted_token_ids, expert_ids,
                 num_tokens_post_padded, mul_routed_weight, top_k, block_m, kernel_configs=None) -> None:
    L = load()
    dev = _device_index(a)
    cfg, ncfg = _cfg(kernel_configs)
    rc = L.tg_fp8_moe_gemm(_desc(c), _desc(a), _weight_desc(b), _desc(a_scale), _weight_desc(b_scale), _desc(topk_weights),
                           _desc(sorted_token_ids), _desc(expert_ids), _desc(num_tokens_post_padded),
                           int(bool(mul_routed_weight)), int(top_k), int(block_m), cfg, ncfg, dev, _stream_handle(a))
    check_rc(rc, "tg_fp8_moe_gemm")


def moe_gemm_silu_quant_ok(b, block_m) -> bool:
    """Shapes the fused GEMM1 + SiLU-multiply + 1x128 quantization entry point accepts."""
    two_i, k = b.shape[1], b.shape[2]
    return two_i % 256 == 0 and k % 128 == 0 and 128 <= k <= 65536 and block_m % 128 == 0


def fp8_moe_gemm_silu_quant(a, b, a_scale, b_scale, sorted_token_ids, expert_ids, num_tokens_post_padded,
                            top_k, block_m, num_valid, act_dtype):
    """tg_fp8_moe_gemm_silu_quant: returns (q (num_valid, I) e4m3, scales (num_valid, I/128) f32)."""
    import torch
    L = load()
    dev = _device_index(a)
    inter = b.shape[1] // 2
    q = torch.empty((num_valid, inter), dtype=torch.float8_e4m3fn, device=a.device)
    scales = torch.empty((num_valid, inter // 128), dtype=torch.float32, device=a.device)
    rc = L.tg_fp8_moe_gemm_silu_quant(_desc(q), _desc(scales), _desc(a), _weight_desc(b), _desc(a_scale), _weight_desc(b_scale),
                                      _desc(sorted_token_ids), _desc(expert_ids), _desc(num_tokens_post_padded),
                                      int(top_k), int(block_m), _DTYPE_CODES[act_dtype], dev, _stream_handle(a))
    check_rc(rc, "tg_fp8_moe_gemm_silu_quant")
    return q, scales


MOE_ALIGN_MAX_EXPERTS = 512


def moe_align_block_size(topk_ids, block_size: int, num_experts: int):
    """One-launch device alignment (tg_moe_align_block_size); allocates the five outputs with the
    worst-case, data-independent sizes of src/tilegym/ops/cutile/moe_align_block.py:252-268."""
    L = load()
    ids = topk_ids if topk_ids.dtype in (torch.int32, torch.int64) else topk_ids.to(torch.int64)
    ids = ids.contiguous()
    dev = ids.device
    numel = ids.numel()
    cap = numel + num_experts * (block_size - 1)
    nblk = -(-cap // block_size)
    sorted_ids = torch.empty(cap, dtype=torch.int32, device=dev)
    expert_ids = torch.empty(max(nblk, 1), dtype=torch.int32, device=dev)[:nblk]
    post = torch.empty(1, dtype=torch.int32, device=dev)
    cumsum = torch.empty(num_experts + 1, dtype=torch.int32, device=dev)
    mx = torch.empty(1, dtype=torch.int32, device=dev)
    rc = L.tg_moe_align_block_size(_ref(_desc(ids)), int(block_size), int(num_experts),
                                   _ref(_desc(sorted_ids)), _ref(_desc(expert_ids)),
                                   _ref(_desc(post)), _ref(_desc(cumsum)), _ref(_desc(mx)),
                                   _device_index(ids), _stream_handle(ids))
    check_rc(rc, "tg_moe_align_block_size")
    return sorted_ids, expert_ids, post, cumsum, mx


def moe_align_quant_1x128(topk_ids, block_size: int, num_experts: int, x: torch.Tensor):
    """moe_align_block_size(topk_ids, ...) and the 1 x 128 quantization of ``x`` (bf16 / f16, all-zero group -> scale 1)
    in one launch (tg_moe_align_quant_1x128).  Returns (sorted_ids, expert_ids, post, cumsum, max_count, q, scales)."""
    L = load()
    ids = topk_ids if topk_ids.dtype in (torch.int32, torch.int64) else topk_ids.to(torch.int64)
    ids = ids.contiguous()
    x = x.contiguous()
    dev = ids.device
    numel = ids.numel()
    cap = numel + num_experts * (block_size - 1)
    nblk = -(-cap // block_size)
    sorted_ids = torch.empty(cap, dtype=torch.int32, device=dev)
    expert_ids = torch.empty(max(nblk, 1), dtype=torch.int32, device=dev)[:nblk]
    post = torch.empty(1, dtype=torch.int32, device=dev)
    cumsum = torch.empty(num_experts + 1, dtype=torch.int32, device=dev)
    mx = torch.empty(1, dtype=torch.int32, device=dev)
    q = torch.empty(x.shape, dtype=torch.float8_e4m3fn, device=x.device)
    scales = torch.empty(x.shape[:-1] + (x.shape[-1] // 128,), dtype=torch.float32, device=x.device)
    rc = L.tg_moe_align_quant_1x128(_ref(_desc(ids)), int(block_size), int(num_experts),
                                    _ref(_desc(sorted_ids)), _ref(_desc(expert_ids)),
                                    _ref(_desc(post)), _ref(_desc(cumsum)), _ref(_desc(mx)),
                                    _ref(_desc(q)), _ref(_desc(scales)), _ref(_desc(x)),
                                    _device_index(ids), _stream_handle(ids))
    check_rc(rc, "tg_moe_align_quant_1x128")
    return sorted_ids, expert_ids, post, cumsum, mx, q, scales


def fp8_quant_1x128(x: torch.Tensor, eps: float = 0.0, flashinfer_rule: bool = False, q=None, scales=None):
    """(q e4m3fn like x, scales (..., K/128) f32) through tg_fp8_quant_1x128; ``q`` / ``scales`` may be given
    (pre-allocated outputs of those shapes)."""
    L = load()
    x = x.contiguous()
    if q is None:
        q = torch.empty(x.shape, dtype=torch.float8_e4m3fn, device=x.device)
    if scales is None:
        scales = torch.empty(x.shape[:-1] + (x.shape[-1] // 128,), dtype=torch.float32, device=x.device)
    rc = L.tg_fp8_quant_1x128(_ref(_desc(q)), _ref(_desc(scales)), _ref(_desc(x)),
                              float(eps), 1 if flashinfer_rule else 0, _device_index(x), _stream_handle(x))
    check_rc(rc, "tg_fp8_quant_1x128")
    return q, scales


def fp8_quant_group(x: torch.Tensor, group_size: int, eps: float, rule: int, scales: Optional[torch.Tensor] = None,
                    dst_dtype: torch.dtype = torch.float8_e4m3fn):
    """(q like x, scales) through tg_fp8_quant_group; q is e4m3fn or, with ``dst_dtype=torch.int8``, int8 (scale =
    amax / 127, quotient truncated toward zero); rule 0 zero-group -> 1, 1 eps clamp, 2 eps clamp and
    power-of-two scales.  ``scales`` may be a 2-D (rows, K/group_size) f32 tensor with any strides (column-major
    layouts); by default it is allocated row-major with x's leading shape."""
    L = load()
    x = x.contiguous()
    q = torch.empty(x.shape, dtype=dst_dtype, device=x.device)
    if scales is None:
        scales = torch.empty(x.shape[:-1] + (x.shape[-1] // group_size,), dtype=torch.float32, device=x.device)
    rc = L.tg_fp8_quant_group(_ref(_desc(q)), _ref(_desc(scales)), _ref(_desc(x)),
                              int(group_size), float(eps), int(rule), _device_index(x), _stream_handle(x))
    check_rc(rc, "tg_fp8_quant_group")
    return q, scales


def fp8_weight_dequant(x: torch.Tensor, s: torch.Tensor, block_size: int, dtype: torch.dtype, out=None) -> torch.Tensor:
    """y (M, N) of ``dtype`` = float(x) * s[i // block_size, j // block_size] through tg_fp8_weight_dequant
    (``out``: a pre-allocated y)."""
    L = load()
    x, s = x.contiguous(), s.contiguous()
    y = out if out is not None else torch.empty(x.shape, dtype=dtype, device=x.device)
    rc = L.tg_fp8_weight_dequant(_ref(_desc(y)), _ref(_desc(x)), _ref(_desc(s)),
                                 int(block_size), _device_index(x), _stream_handle(x))
    check_rc(rc, "tg_fp8_weight_dequant")
    return y


def silu_mul_quant_1x128(x: torch.Tensor):
    """x (R, 2I) bf16/f16 -> (q (R, I) e4m3fn, scales (R, ceil(I/128)) f32) through tg_silu_mul_quant_1x128."""
    L = load()
    R, two_i = x.shape
    inter = two_i // 2
    q = torch.empty(R, inter, dtype=torch.float8_e4m3fn, device=x.device)
    scales = torch.empty(R, -(-inter // 128), dtype=torch.float32, device=x.device)
    rc = L.tg_silu_mul_quant_1x128(_ref(_desc(q)), _ref(_desc(scales)), _ref(_desc(x)),
                                   _device_index(x), _stream_handle(x))
    check_rc(rc, "tg_silu_mul_quant_1x128")
    return q, scales


def moe_sum(x: torch.Tensor, out: torch.Tensor) -> None:
    """out (T, H) <- sum over axis 1 of x (T, top_k, H) through tg_moe_sum."""
    L = load()
    rc = L.tg_moe_sum(_ref(_desc(out)), _ref(_desc(x)), _device_index(x), _stream_handle(x))
    check_rc(rc, "tg_moe_sum")


def _desc_array(tensors):
    """list of tensors (entries may be None) -> (array of descriptor pointers, keep-alive list)."""
    P = ctypes.POINTER(TgTensor)
    descs = [make_tensor_desc(t) for t in tensors]
    arr = (P * len(tensors))(*[ctypes.pointer(d) if d is not None else P() for d in descs])
    return arr, descs


def fp8_group_gemm(cs, As, Bs, scales_a=None, scales_b=None, trans_b=True, kernel_configs=None) -> None:
    """Lists of problems through tg_fp8_group_gemm (one launch when the list qualifies)."""
    L = load()
    n = len(As)
    cfg, ncfg = make_cfg(kernel_configs)
    dev = _device_index(As[0])
    PP = ctypes.POINTER(ctypes.POINTER(TgTensor))
    c_arr, k1 = _desc_array(cs)
    a_arr, k2 = _desc_array(As)
    b_arr, k3 = _desc_array(Bs)
    sa_arr, k4 = _desc_array(scales_a) if scales_a is not None else (None, None)
    sb_arr, k5 = _desc_array(scales_b) if scales_b is not None else (None, None)
    need = 0
    if not trans_b:
        for a, b in zip(As, Bs):
            need = max(need, workspace_bytes(a.shape[0], b.shape[1], a.shape[1], False, cfg, ncfg))
    ws = workspace_for(As[0].device, need) if need else None
    rc = L.tg_fp8_group_gemm(ctypes.cast(c_arr, PP), ctypes.cast(a_arr, PP), ctypes.cast(b_arr, PP),
                             ctypes.cast(sa_arr, PP) if sa_arr is not None else None,
                             ctypes.cast(sb_arr, PP) if sb_arr is not None else None,
                             n, 1 if trans_b else 0, _ref(_desc(ws)), cfg, ncfg, dev, _stream_handle(As[0]))
    del k1, k2, k3, k4, k5
    check_rc(rc, "tg_fp8_group_gemm")



_moe_ws_bytes: Dict[tuple, int] = {}


def fused_moe_ok(hidden, w1, w2, block_m: int) -> bool:
    """Shapes and types tg_fp8_fused_moe takes (one chunk of 16-bit activations, the fused activation epilogue's limits)."""
    return (hidden.dtype in (torch.bfloat16, torch.float16) and hidden.shape[1] % 128 == 0 and w1.shape[1] % 256 == 0
            and w1.shape[0] <= MOE_ALIGN_MAX_EXPERTS and block_m in (128, 256))


def fp8_fused_moe(out, hidden, w1, w2, w1_scale, w2_scale, topk_weights, topk_ids, block_m: int) -> None:
    """tg_fp8_fused_moe: the whole FP8 MoE layer (align + quantize, GEMM1 with the activation epilogue, GEMM2 x routed
    weight, top-k sum) in one call, intermediates in the stream's scratch buffer."""
    L = _lib if _lib is not None else load()
    dev = _device_index(hidden)
    T, H = hidden.shape
    E, two_i, _ = w1.shape
    k = topk_ids.shape[1]
    key = (T, k, E, H, two_i, block_m)
    need = _moe_ws_bytes.get(key)
    if need is None:
        if len(_moe_ws_bytes) >= _CACHE_MAX:
            _moe_ws_bytes.clear()
        need = _moe_ws_bytes[key] = int(L.tg_fp8_fused_moe_workspace_bytes(T, k, E, H, two_i // 2, block_m))
    stream = _raw_stream(dev)
    ws = workspace_for(hidden.device, need, dev, stream)
    rc = L.tg_fp8_fused_moe(_desc(out), _desc(hidden), _weight_desc(w1), _weight_desc(w2), _weight_desc(w1_scale),
                            _weight_desc(w2_scale), _desc(topk_weights), _desc(topk_ids), _weight_desc(ws), int(block_m), dev, stream)
    if rc != 0:
        check_rc(rc, "tg_fp8_fused_moe")


# ---------------------------------------------------------------------------- yardsticks
def diag_read(x: torch.Tensor, scratch: torch.Tensor, workgroups: int = 0, loads_in_flight: int = 0) -> None:
    """tg_diag_read: enqueue a plain read of all bytes of x (scratch: int32, >= workgroups elements; 0 = the defaults,
    2048 workgroups and 4 loads per lane in flight)."""
    rc = load().tg_diag_read(_ref(_desc(x)), _ref(_desc(scratch)), int(workgroups), int(loads_in_flight),
                             _device_index(x), _stream_handle(x))
    check_rc(rc, "tg_diag_read")


def diag_mfma(fmas: int, iters: int, workgroups: int, scratch: torch.Tensor) -> None:
    """tg_diag_mfma: enqueue the MFMA (+ scale-and-add FMA) issue-rate kernel (scratch: f32, >= workgroups * 512)."""
    rc = load().tg_diag_mfma(int(fmas), int(iters), int(workgroups), _ref(_desc(scratch)), _device_index(scratch),
                             _stream_handle(scratch))
    check_rc(rc, "tg_diag_mfma")
