"""Measure every schedule that can be forced for a dense FP8 GEMM shape and record the fastest.

    python -m tilegym_amd.tune --shape 16,5120,12288 --shape 8,4096,11008,block --out tune.json
    TILEGYM_HIP_TUNE=tune.json python my_decode_loop.py

The library picks its schedules in O(1): fixed rules up to 16 rows, cost models over kernels, tiles and split-K factors
above (``choose_dense`` in csrc/tilegym_hip_api.hip; their constants were fitted to tables this module wrote), and a test
holds the choice within 25 % of the best forced schedule on shapes outside the fit (measured: 1 - 2 % on average).
For a caller who wants the last few percent on the shapes of one model, this module does what the reference's
exhaustive search does (src/tilegym/ops/cutile/matmul.py:327-418): it times the candidates on this GPU -- weights
rotated through more copies than the caches hold, launches replayed from a HIP graph, as in a decode step -- and writes
a JSON table that ``tilegym_amd._lib`` reads when TILEGYM_HIP_TUNE names it.  A recorded entry is only a
``kernel_configs`` dictionary: any call can still pass its own.
"""

from __future__ import annotations

import argparse
import json
import os
from typing import Dict, Iterable, List, Optional, Tuple

import torch

from . import _lib

ROTATE_BYTES = 768 << 20
REPORTED = ("KERNEL_NAME", "BLOCK_M", "BLOCK_N", "SPLIT_K", "ROW_GROUPS", "WAVES")


def candidates(M: int, N: int, K: int, block_scaled: bool) -> List[dict]:
    """kernel_configs worth timing for the shape (the library refuses or replaces what does not apply)."""
    out: List[dict] = []
    if M <= 32:
        out += [{"KERNEL": "stream", "ROW_GROUPS": 4, "SPLIT_K": s} for s in (1, 2, 3, 4, 6, 8)]
        # fewer weight rows per workgroup of the wide form
        out += [{"KERNEL": "stream", "ROW_GROUPS": 4, "SPLIT_K": s, "BLOCK_N": bn} for bn in (56, 48, 40, 32, 24) for s in (1, 2)]
    if M <= 16:
        out += [{"KERNEL": "stream", "ROW_GROUPS": 1, "SPLIT_K": 1, "WAVES": 4}, {"KERNEL": "stream", "WAVES": 8}]
    if M <= 64:
        out += [{"KERNEL": "skinny"}]
    if M > 16 and K % 128 == 0:
        tiles = [(64, 128), (128, 128), (128, 256), (256, 256)] + ([] if block_scaled else [(32, 32), (64, 32), (64, 64)])
        for bm, bn in tiles:
            for s in (1, 2, 4, 8):
                if s > 1 and (bm, bn) in ((32, 32), (64, 32), (64, 64)):
                    continue
                out.append({"KERNEL": "tiled", "BLOCK_M": bm, "BLOCK_N": bn, "SPLIT_K": s})
        if not block_scaled and M <= 512:
            # the 64 x 128 tile kernel over fewer weight rows per tile (more, lighter workgroups)
            out += [{"KERNEL": "tiled", "BLOCK_M": 64, "BLOCK_N": bn, "SPLIT_K": s} for bn in (112, 96, 80) for s in (1, 2, 4, 8)]
    return out


def _fp8(shape, device, gen):
    b = torch.randint(0, 0x78, shape, dtype=torch.uint8, device=device, generator=gen)
    sign = torch.randint(0, 2, shape, dtype=torch.uint8, device=device, generator=gen) << 7
    return (b | sign).view(torch.float8_e4m3fn)


def _graph_us(fn, launches: int) -> float:
    stream = torch.cuda.current_stream()
    side = torch.cuda.Stream()
    side.wait_stream(stream)
    with torch.cuda.stream(side):
        fn(0)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        for i in range(launches):
            fn(i)
    torch.cuda.synchronize()
    graph.replay()
    torch.cuda.synchronize()
    best = float("inf")
    for _ in range(3):
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(4):
            graph.replay()
        end.record()
        torch.cuda.synchronize()
        best = min(best, start.elapsed_time(end) * 1e3 / (4 * launches))
    return best


def tune_shape(M: int, N: int, K: int, block_scaled: bool = False, device: Optional[torch.device] = None,
               keep_timings: bool = False) -> dict:
    """Time the automatic schedule and every candidate; returns a table entry (kernel_configs = {} when automatic wins;
    with keep_timings every candidate's time and the schedule it ran as, under "timings")."""
    device = device or torch.device("cuda", torch.cuda.current_device())
    gen = torch.Generator(device=device)
    gen.manual_seed(M * 7 + N + K)
    copies = max(2, min(16, -(-ROTATE_BYTES // max(1, N * K))))
    a = _fp8((M, K), device, gen)
    bs = [_fp8((N, K), device, gen) for _ in range(copies)]
    cs = [torch.empty(M, N, dtype=torch.bfloat16, device=device) for _ in range(2)]
    if block_scaled:
        sa = torch.rand(M, -(-K // 128), device=device, generator=gen) + 0.5
        sb = torch.rand(-(-N // 128), -(-K // 128), device=device, generator=gen) + 0.5
    else:
        sa = torch.full((1,), 0.01, device=device)
        sb = torch.full((1,), 0.02, device=device)

    def timed(kc):
        def fn(i):
            _lib.fp8_gemm(cs[i % 2], a, bs[i % copies], sa, sb, False, True, 1.0, 0.0, kc)
        try:
            fn(0)
        except _lib.TileGymHipError:
            return None, None
        torch.cuda.synchronize()
        ran = _lib.last_config()
        return _graph_us(fn, copies), ran

    automatic = {"KERNEL": -1}                   # an explicit all-automatic cfg: a loaded table is not consulted
    timed(automatic)                             # clocks and caches settle on the first graph; its time is not used
    auto_us, auto_ran = timed(automatic)
    best_kc, best_us, timings = {}, float("inf"), []
    for kc in candidates(M, N, K, block_scaled):
        us, ran = timed(kc)
        if us is None or ran["KERNEL_NAME"] != kc["KERNEL"]:
            continue
        timings.append([kc, round(us, 2), {k: ran[k] for k in REPORTED}])
        if us < best_us:
            best_kc, best_us = kc, us
    auto_us = min(auto_us, timed(automatic)[0])  # and once more behind the candidates
    if best_kc:
        best_us = min(best_us, timed(best_kc)[0])
    # a forced schedule must beat the automatic one by more than the noise of the measurement to be recorded
    if best_us > 0.97 * auto_us:
        best_kc, best_us = {}, auto_us
    entry = {"M": M, "N": N, "K": K, "block_scaled": bool(block_scaled), "kernel_configs": best_kc, "us": round(best_us, 2),
             "auto_us": round(auto_us, 2), "auto_schedule": {k: auto_ran[k] for k in REPORTED}}
    if keep_timings:
        entry["timings"] = timings
    return entry


def write_table(entries: Iterable[dict], path: str) -> None:
    """Merge `entries` into the table at `path` (entries whose kernel_configs is empty are dropped: automatic is best)."""
    merged: Dict[Tuple[int, int, int, bool], dict] = {}
    if os.path.exists(path):
        with open(path) as f:
            for e in json.load(f).get("entries", []):
                merged[(e["M"], e["N"], e["K"], bool(e.get("block_scaled", False)))] = e
    for e in entries:
        key = (e["M"], e["N"], e["K"], bool(e["block_scaled"]))
        if e["kernel_configs"]:
            merged[key] = e
        else:
            merged.pop(key, None)
    name = torch.cuda.get_device_name(0) if torch.cuda.is_available() else "unknown"
    with open(path, "w") as f:
        json.dump({"version": 1, "device": name, "entries": sorted(merged.values(), key=lambda e: (e["block_scaled"], e["N"], e["K"], e["M"]))}, f, indent=1)


def _parse_shape(text: str) -> Tuple[int, int, int, bool]:
    parts = text.split(",")
    if len(parts) not in (3, 4) or (len(parts) == 4 and parts[3] not in ("block", "tensor")):
        raise argparse.ArgumentTypeError("--shape M,N,K[,block|tensor]")
    return int(parts[0]), int(parts[1]), int(parts[2]), len(parts) == 4 and parts[3] == "block"


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("--shape", type=_parse_shape, action="append", required=True, help="M,N,K[,block|tensor] (repeatable)")
    ap.add_argument("--out", required=True, help="JSON table to create or merge into")
    ap.add_argument("--timings", help="also write every candidate's time per shape to this JSON file")
    args = ap.parse_args(argv)
    if not torch.cuda.is_available():
        raise SystemExit("tilegym_amd.tune measures on the GPU; none is visible")
    _lib.load()
    entries = []
    for M, N, K, bs in args.shape:
        e = tune_shape(M, N, K, bs, keep_timings=bool(args.timings))
        entries.append(e)
        print(f"M={M} N={N} K={K} {'block' if bs else 'tensor'}: automatic {e['auto_us']} us ({e['auto_schedule']}), "
              f"best {e['us']} us {e['kernel_configs'] or '(automatic)'}", flush=True)
    if args.timings:
        with open(args.timings, "w") as f:
            json.dump(entries, f, indent=1)
    write_table([{k: v for k, v in e.items() if k != "timings"} for e in entries], args.out)
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
