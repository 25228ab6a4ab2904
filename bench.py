#!/usr/bin/env python3
"""Benchmark of the FP8 GEMM path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload prefill|decode|block|moe|all]

A "step" is one pass over the workload's GEMMs with inputs already resident in HBM.  The headline
line (one JSON object on stdout) reports the prefill workload -- the four Llama-3.1-8B projection
GEMMs at M=8192, FP8 per-tensor scales, bf16 out -- as whole-step TFLOP/s (sum of 2*M*N*K over the
time of K steps), with:
  roofline      the dominant kernel (the 256x256 LDS-tiled MFMA kernel on the gate+up shape):
                algorithmic FLOPs per launch / its average launch duration, against 5.0 PFLOP/s
  decode        the same for the decode workload (M in {1,8,16,64}; weight streaming), in GB/s of
                algorithmic bytes against 8 TB/s, per shape and aggregated, cold cache (operands
                are rotated through > 512 MB so that launches do not hit the 256 MB memory-side cache)
  cpu_baseline  the torch CPU oracle (dequantize -> fp32 matmul -> bf16) timed on this host's cores
                on a bounded sample of the same workload
Kernel durations are measured with HIP events on the stream the kernels are launched on.  Compute-bound
workloads first run untimed for RAMP_MS milliseconds (see _ramp): the device needs ~30 ms under load to
reach its steady state after idle time, and the timed K steps are meant to measure that state.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_FP8_TFLOPS = 5000.0   # MI355X dense FP8 MFMA
PEAK_HBM_GBS = 8000.0      # MI355X HBM3E
KERNEL_SYMBOLS = {"tiled": "fp8_gemm_tile_kernel", "skinny": "fp8_gemm_skinny_kernel", "stream": "fp8_gemm_stream_kernel",
                  "fallback": "fp8_gemm_generic_kernel"}
ROTATE_BYTES = 640 << 20

# HBM bytes per launch (reads + writes) come from the hardware counters FETCH_SIZE and WRITE_SIZE, collected in two profiler
# passes of this program and scaled by what the same counters read for --calibrate-copy's elementwise add of known size.
# The figures live in profiles/hbm_traffic_per_launch.txt, one line per measured shape together with the kernel and
# schedule they were measured on; a run whose schedule differs from the recorded one reports "traffic": null (the
# recorded figure would describe another kernel).
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "hbm_traffic_per_launch.txt")
TRAFFIC_FIELDS = ("shape", "kernel_symbol", "block_m", "block_n", "split_k", "row_groups", "waves", "fetch_kib", "write_kib",
                  "read_scale", "write_scale")


def load_traffic_table(path=TRAFFIC_FILE):
    table = {}
    try:
        with open(path) as f:
            for line in f:
                line = line.split("#", 1)[0].split()
                if len(line) != len(TRAFFIC_FIELDS):
                    continue
                rec = dict(zip(TRAFFIC_FIELDS, line))
                table[rec["shape"]] = rec
    except OSError:
        pass
    return table


def kernel_symbol(shape):
    """Device function a measured shape ran (the stream kernel's 64-row form and the three-stage 64x128
    per-tensor tile are kernels of their own)."""
    if shape["kernel"] == "stream" and shape["row_groups"] == 4:
        return "fp8_gemm_stream_wide_db_kernel" if shape["waves"] == 4 else "fp8_gemm_stream_wide_kernel"
    if shape["kernel"] == "tiled" and shape["block_m"] == 64 and shape["block_n"] == 128 and not shape.get("block_scaled", False):
        return "fp8_gemm_tile_deep_kernel"
    if shape["kernel"] == "tiled" and (shape["block_n"] == 32 or (shape["block_m"], shape["block_n"]) == (64, 64)):
        return "fp8_gemm_tile_mid_kernel"
    if shape["kernel"] == "tiled" and shape["block_m"] == 256 and shape["split_k"] == 1 and not shape.get("block_scaled", False):
        return "fp8_gemm_tile256_kernel"
    return KERNEL_SYMBOLS[shape["kernel"]]


def measured_traffic(shape, table=None):
    """(bytes per launch, note) for a measured shape: the recorded counter figures if they were taken on the kernel and
    schedule this run used, else (None, why)."""
    table = load_traffic_table() if table is None else table
    rec = table.get(shape["name"])
    if rec is None:
        return None, "no counter pass recorded for this shape"
    ran = {"kernel_symbol": kernel_symbol(shape), "block_m": shape["block_m"], "block_n": shape["block_n"],
           "split_k": shape["split_k"], "row_groups": shape["row_groups"], "waves": shape["waves"]}
    diff = [k for k, v in ran.items() if str(v) != rec[k]]
    if diff:
        return None, "recorded on another schedule (" + ", ".join(f"{k}: recorded {rec[k]}, ran {ran[k]}" for k in diff) + ")"
    nbytes = (float(rec["fetch_kib"]) * float(rec["read_scale"]) + float(rec["write_kib"]) * float(rec["write_scale"])) * 1024
    return int(nbytes), f"FETCH_SIZE x {rec['read_scale']} + WRITE_SIZE x {rec['write_scale']}, {os.path.relpath(TRAFFIC_FILE, ROOT)}"


def _events_ms(fn, iters, stream):
    """Time `iters` calls of fn() with HIP events on `stream`; returns total milliseconds."""
    start = torch.cuda.Event(enable_timing=True)
    end = torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    start.record(stream)
    for i in range(iters):
        fn(i)
    end.record(stream)
    torch.cuda.synchronize()
    return start.elapsed_time(end)


RAMP_MS = 100.0


def _ramp(fn, min_ms=RAMP_MS):
    """Untimed: keep the device under the load of fn(i) for at least `min_ms`.  After idle time an MI355X
    runs MFMA-bound kernels 10-20 % slower for its first ~30 ms under load (a (8192, 6144, 4096) GEMM goes
    192 -> 157 us over ~150 back-to-back launches, and back to 190 us after two idle seconds); HBM-bound
    launches show no such drift.  Compute-bound workloads are therefore measured after this phase, which is
    part of the warm-up, never of the timed region."""
    t0 = time.perf_counter()
    i = 0
    while (time.perf_counter() - t0) * 1e3 < min_ms:
        for _ in range(4):
            fn(i)
            i += 1
        torch.cuda.synchronize()


def _graph_ms(fn, launches, replays, stream):
    """Capture `launches` calls of fn(i) into one HIP graph, replay it `replays` times between two
    events.  Removes host launch overhead from the timed region (needed for microsecond kernels).
    Returns total ms, or None if capture is not possible."""
    try:
        side = torch.cuda.Stream()
        side.wait_stream(stream)
        with torch.cuda.stream(side):
            for i in range(min(launches, 2)):
                fn(i)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            for i in range(launches):
                fn(i)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        start = torch.cuda.Event(enable_timing=True)
        end = torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(replays):
            graph.replay()
        end.record()
        torch.cuda.synchronize()
        return start.elapsed_time(end)
    except Exception as exc:  # capture unsupported: report, fall back to plain launches
        print(f"[bench] graph timing unavailable ({type(exc).__name__}: {exc}); using plain launches", file=sys.stderr)
        torch.cuda.synchronize()
        return None


def _vendor_yardstick(runners, shapes, steps, stream):
    """The same per-tensor prefill GEMMs through the vendor library (torch._scaled_mm -> hipBLASLt) on the same operand
    tensors, same process, each after its own load ramp: a yardstick for what this GPU sustains on the shape, not part
    of the product path and not a baseline of the reference.  Adds `vendor_us` to every prefill shape."""
    try:
        total_us = 0.0
        same = True
        for r, sh in zip(runners, shapes):
            sa, sb = r.sa.reshape(()), r.sb.reshape(())
            fn = lambda i, r=r, sa=sa, sb=sb: torch._scaled_mm(r.a[i % r.copies], r.b[i % r.copies].t(), scale_a=sa, scale_b=sb,  # noqa: E731
                                                               out_dtype=torch.bfloat16)
            _ramp(fn)
            us = _events_ms(fn, steps, stream) * 1e3 / steps
            sh["vendor_us"] = round(us, 2)
            total_us += us
            r(0)
            torch.cuda.synchronize()
            same = same and bool(torch.equal(fn(0), r.c[0]))
        flops = sum(r.case.flops() for r in runners)
        return {"library": "torch._scaled_mm (hipBLASLt), same operands", "sum_us": round(total_us, 1),
                "tflops": round(flops / total_us * 1e-6, 1), "outputs_bit_identical_to_ours": same,
                "ours_sum_us": round(sum(sh["us"] for sh in shapes), 1)}
    except Exception as exc:  # the yardstick must never break the bench line
        return {"library": "torch._scaled_mm", "error": f"{type(exc).__name__}: {exc}"[:200]}


def _read_yardstick_us(runner, steps, stream, use_graph):
    """A plain read (tg_diag_read: 16 bytes per lane, nothing else) of the same rotated weight copies the GEMM shape
    streams, timed the same way (graph replay over whole passes of the copies): the floor of any kernel that has to read
    those bytes once, on this GPU, in this run."""
    from tilegym_amd import _lib
    scratch = torch.zeros(8192, dtype=torch.int32, device=runner.b[0].device)
    best = float("inf")
    # (workgroups, 16-byte loads per lane in flight): the fastest of a few launch shapes is the floor
    for wgs, in_flight in ((2048, 1), (2048, 4), (4096, 8)):
        fn = lambda i: _lib.diag_read(runner.b[i % runner.copies], scratch, wgs, in_flight)  # noqa: E731
        for i in range(2):
            fn(i)
        torch.cuda.synchronize()
        per_graph = runner.copies * max(1, -(-8 // runner.copies))
        replays = max(1, steps // per_graph)
        ms = _graph_ms(fn, per_graph, replays, stream) if use_graph else None
        launches = per_graph * replays
        if ms is None:
            launches = steps
            ms = _events_ms(fn, launches, stream)
        best = min(best, ms * 1e3 / launches)
    return best


def _eager_us(fn, n, stream):
    """Per-call time of `n` back-to-back eager calls (no graph): the larger of the host cost of a call through the binding
    and the kernel time."""
    # one untimed pass of the same length first: when the host issues faster than the kernels run, the first long burst
    # makes the runtime grow its pools once (tens of milliseconds), which is not a per-call cost
    for i in range(n):
        fn(i)
    torch.cuda.synchronize()
    return _events_ms(fn, n, stream) * 1e3 / n


def _issue_yardstick(device, stream):
    """tg_diag_mfma: the e4m3 MFMA rate on non-zero register operands with 0 / 4 / 6 scale-and-add FMAs behind every MFMA,
    eight waves per compute unit on every compute unit: what the matrix pipe sustains here, and what is left of it when
    it shares the VALU issue port with the block-scaled kernels' four FMAs per MFMA (plus a little more)."""
    from tilegym_amd import _lib
    props = torch.cuda.get_device_properties(device)
    wgs = props.multi_processor_count
    scratch = torch.empty(wgs * 512, dtype=torch.float32, device=device)
    iters = 3000
    out = {}
    for fmas in (0, 4, 6):
        fn = lambda i, fmas=fmas: _lib.diag_mfma(fmas, iters, wgs, scratch)  # noqa: E731
        _ramp(fn, 60.0)
        us = _events_ms(fn, 5, stream) * 1e3 / 5
        flops = wgs * 8 * iters * 32 * 65536.0
        out[f"mfma_plus_{fmas}_fma_tflops"] = round(flops / us * 1e-6, 1)
    out["note"] = ("register-only loops of the library's tg_diag_mfma, 8 waves per CU, after 60 ms under their own load; "
                   "a block-scaled K step needs 4 FMAs per MFMA plus its scale, address and conversion work")
    return out


class DenseRunner:
    """One dense problem with its operands replicated `copies` times for cache-cold rotation."""

    def __init__(self, case, device, copies):
        from tilegym_amd import _lib
        self._lib = _lib
        self.case = case
        self.copies = max(1, copies)
        d = case.to(device)
        self.a = [d.a] + [d.a.clone() for _ in range(self.copies - 1)]
        self.b = [d.b] + [d.b.clone() for _ in range(self.copies - 1)]
        self.sa, self.sb = d.scale_a, d.scale_b
        self.c = [torch.empty(case.M, case.N, dtype=torch.bfloat16, device=device) for _ in range(min(self.copies, 4))]

    def __call__(self, i):
        j = i % self.copies
        self._lib.fp8_gemm(self.c[i % len(self.c)], self.a[j], self.b[j], self.sa, self.sb, False, True, 1.0, 0.0)


class RaggedRunner:
    def __init__(self, case, device, copies):
        from tilegym_amd import _lib
        self._lib = _lib
        self.case = case
        self.copies = max(1, copies)
        d = case.to(device)
        self.a = [d.a] + [d.a.clone() for _ in range(self.copies - 1)]
        self.b = [d.b] + [d.b.clone() for _ in range(self.copies - 1)]
        self.d = d
        self.c = torch.empty(d.a.shape[0], d.b.shape[1], dtype=torch.bfloat16, device=device)

    def __call__(self, i):
        j = i % self.copies
        self._lib.fp8_ragged_gemm(self.c, self.a[j], self.b[j], self.d.a_scale, self.d.b_scale, self.d.m_indptr)


def _copies_for(nbytes):
    return max(2, min(64, -(-ROTATE_BYTES // max(1, int(nbytes)))))


def measure_shape(runner, steps, warmup, stream, use_graph, ramp=False):
    from tilegym_amd import _lib
    if ramp:
        _ramp(runner)
    for i in range(max(1, warmup)):
        runner(i)
    torch.cuda.synchronize()
    cfg = _lib.last_config()
    ms = None
    launches = steps
    if use_graph:
        # a whole number of passes over the operand copies: a graph that stopped part-way through the
        # rotation would start its next replay on copies the previous one had just read
        per_graph = runner.copies * max(1, -(-8 // runner.copies))
        replays = max(1, steps // per_graph)
        ms = _graph_ms(runner, per_graph, replays, stream)
        launches = per_graph * replays
    if ms is None:
        launches = steps
        ms = _events_ms(runner, launches, stream)
    us = ms * 1e3 / launches
    case = runner.case
    flops, nbytes = case.flops(), case.algorithmic_bytes()
    return {
        "name": case.name,
        "kernel": cfg["KERNEL_NAME"], "block_m": cfg["BLOCK_M"], "block_n": cfg["BLOCK_N"],
        "split_k": cfg["SPLIT_K"], "row_groups": cfg["ROW_GROUPS"], "waves": cfg["WAVES"],
        "us": round(us, 3), "launches": launches,
        "tflops": round(flops / us * 1e-6, 2), "gbs": round(nbytes / us * 1e-3, 1),
        "flops": flops, "bytes": nbytes,
        "frac_mfma": round(flops / us * 1e-6 / PEAK_FP8_TFLOPS, 4),
        "frac_hbm": round(nbytes / us * 1e-3 / PEAK_HBM_GBS, 4),
    }


def cpu_baseline(target_seconds=12.0):
    """Time the torch CPU oracle on a bounded sample of the headline workload: whole passes over the
    four prefill projections on the first `rows` activation rows, dequantization included.  `rows`
    is doubled from 256 while three passes would still fit in about `target_seconds`."""
    from oracle import reference as R
    from tilegym_amd import workloads as W

    threads = torch.get_num_threads()
    cases = [W.llama_prefill_case(p) for p in W.LLAMA_SHAPES]

    def one_pass(rows):
        t0 = time.perf_counter()
        for c in cases:
            R.ref_gemm_per_tensor(c.a[:rows], c.b, c.scale_a, c.scale_b, trans_b=True)
        return time.perf_counter() - t0

    one_pass(64)                                    # warm-up (thread pool, allocator)
    rows = 256
    t_probe = one_pass(rows)
    while rows < cases[0].M and t_probe * 2 * 3 <= target_seconds:
        rows *= 2
        t_probe = one_pass(rows)
    times = [one_pass(rows) for _ in range(3)]
    t = sorted(times)[1]
    flops = sum(2.0 * rows * c.N * c.K for c in cases)
    cpu_model = "unknown"
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    cpu_model = line.split(":", 1)[1].strip()
                    break
    except OSError:
        pass
    return {
        "value": round(flops / t * 1e-12, 4), "unit": "TFLOP/s", "cores": threads, "kind": "port",
        "sample": f"torch CPU oracle (dequantize -> fp32 matmul -> bf16), the four prefill projections on {rows} of "
                  f"{cases[0].M} rows, three passes of {t:.2f} s (median), {sum(times):.1f} s in all; "
                  f"os.cpu_count()={os.cpu_count()}, cpu='{cpu_model}'",
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-vendor", action="store_true", help="skip the vendor-library yardstick of the prefill shapes")
    ap.add_argument("--workload", default="all", choices=["prefill", "decode", "block", "moe", "quant", "all"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-graph", action="store_true", help="time microsecond kernels with plain launches")
    ap.add_argument("--no-yardsticks", action="store_true",
                    help="skip the plain-read and MFMA-issue yardsticks, the eager per-call costs and the MoE decode regime "
                         "(profiler runs: only the GEMM launches of the workload)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="first run a plain elementwise copy of known size (256 MiB read + 256 MiB written, 3 launches): "
                         "the yardstick that hardware traffic counters are scaled by when this command runs under a profiler")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1).", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py needs a HIP device", file=sys.stderr)
        sys.exit(1)

    from tilegym_amd import _lib, workloads as W

    _lib.load()
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)
    stream = torch.cuda.current_stream()
    props = torch.cuda.get_device_properties(device)
    out = {}
    detail = {}
    if args.calibrate_copy:
        src = torch.zeros(64 << 20, dtype=torch.float32, device=device)
        dst = torch.empty_like(src)
        for _ in range(3):
            torch.add(src, 1.0, out=dst)
        torch.cuda.synchronize()
        del src, dst
        torch.cuda.empty_cache()

    # ------------------------------------------------------------------ prefill (headline)
    if args.workload in ("prefill", "all"):
        runners = [DenseRunner(W.llama_prefill_case(p), device, copies=2) for p in W.LLAMA_SHAPES]

        def step(i):
            for r in runners:
                r(i)

        _ramp(step)
        for w in range(max(1, args.warmup)):
            step(w)
        torch.cuda.synchronize()

        ms = _events_ms(step, args.steps, stream)
        total_flops = sum(r.case.flops() for r in runners)
        ms_per_step = ms / args.steps
        shapes = [measure_shape(r, args.steps, 1, stream, use_graph=False) for r in runners]
        dom = max(shapes, key=lambda s: s["us"])
        traffic, traffic_note = measured_traffic(dom)
        out.update({
            "value": round(total_flops / (ms_per_step * 1e-3) * 1e-12, 2),
            "ms_per_step": round(ms_per_step, 4),
            "roofline": {"bound": "mfma", "achieved": dom["tflops"], "peak": PEAK_FP8_TFLOPS, "unit": "TFLOP/s",
                         "frac": dom["frac_mfma"], "traffic": traffic, "traffic_source": traffic_note,
                         "kernel": f"{kernel_symbol(dom)} ({dom['block_m']}x{dom['block_n']} tile, per-tensor scales)",
                         "shape": dom["name"], "us_per_launch": dom["us"]},
        })
        detail["prefill"] = shapes
        if not args.no_vendor:
            out["vendor_yardstick"] = _vendor_yardstick(runners, shapes, args.steps, stream)
        del runners
        torch.cuda.empty_cache()

    # ------------------------------------------------------------------ config 1 (the reference's CPU-runnable case; a parity case, timed for completeness)
    if args.workload in ("prefill", "all"):
        case = W.config1()
        r = DenseRunner(case, device, copies=_copies_for(case.algorithmic_bytes()))
        detail["config1"] = [measure_shape(r, max(args.steps, 64), args.warmup, stream, use_graph=not args.no_graph)]
        del r
        torch.cuda.empty_cache()

    # ------------------------------------------------------------------ decode
    if args.workload in ("decode", "all"):
        shapes = []
        for proj in W.LLAMA_SHAPES:
            big = W.llama_decode_case(64, proj)
            for M in W.DECODE_M:
                case = W.DenseCase(f"c2_decode_{proj}_M{M}", big.a[:M].contiguous(), big.b, big.scale_a, big.scale_b, True, False)
                r = DenseRunner(case, device, copies=_copies_for(case.algorithmic_bytes()))
                sh = measure_shape(r, max(args.steps, 64), args.warmup, stream, use_graph=not args.no_graph)
                # the floor: a plain read of the same weight copies, same replay (once per projection is enough: M does
                # not change the weights), and the eager per-call cost through the ctypes binding and through torch.ops
                if args.no_yardsticks:
                    shapes.append(sh)
                    del r
                    continue
                if M == W.DECODE_M[0]:
                    read_us = _read_yardstick_us(r, max(args.steps, 64), stream, use_graph=not args.no_graph)
                sh["read_yardstick_us"] = round(read_us, 3)
                sh["eager_us"] = round(_eager_us(r, 200, stream), 2)
                c0 = r.c[0]
                op = torch.ops.tilegym_hip.fp8_gemm_out
                sh["eager_us_torch_op"] = round(_eager_us(lambda i, r=r: op(c0, r.a[i % r.copies], r.b[i % r.copies], r.sa, r.sb,
                                                                             False, True, 1.0, 0.0), 200, stream), 2)
                # through the public op with a fresh output tensor per call (torch.empty included): the prepared-call
                # cache of the binding cannot hit, only its per-weight descriptors do
                from tilegym_amd.ops import matmul as op_matmul
                sh["eager_us_fresh_output"] = round(_eager_us(lambda i, r=r: op_matmul(r.a[i % r.copies], r.b[i % r.copies], trans_b=True,
                                                                                   scale_a=r.sa, scale_b=r.sb, out_dtype=torch.bfloat16),
                                                              200, stream), 2)
                shapes.append(sh)
                del r
            torch.cuda.empty_cache()
        tot_b = sum(s["bytes"] for s in shapes)
        tot_us = sum(s["us"] for s in shapes)
        small = [s for s in shapes if int(s["name"].rsplit("M", 1)[1]) <= 16]
        dom = max(small, key=lambda s: s["us"])
        traffic, traffic_note = measured_traffic(dom)
        dec = {
            "metric": "FP8 GEMM decode GB/s (algorithmic bytes, cold cache)", "value": round(tot_b / tot_us * 1e-3, 1), "unit": "GB/s",
            "us_per_step": round(tot_us, 2),
            "hbm_read_yardstick": None if args.no_yardsticks else {
                "what": "tg_diag_read (plain 16-byte-per-lane read, no LDS, no MFMA; the fastest of three launch shapes) over the same rotated weight copies, same graph replay",
                "us_M_le_16": round(sum(s["read_yardstick_us"] for s in small), 2),
                "gemm_us_M_le_16": round(sum(s["us"] for s in small), 2),
                "frac_hbm_of_the_plain_read": round(sum(s["bytes"] for s in small) / sum(s["read_yardstick_us"] for s in small) * 1e-3 / PEAK_HBM_GBS, 4)},
            "frac_hbm_M_le_16": round(sum(s["bytes"] for s in small) / sum(s["us"] for s in small) * 1e-3 / PEAK_HBM_GBS, 4),
            "roofline": {"bound": "hbm", "achieved": dom["gbs"], "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": dom["frac_hbm"],
                         "traffic": traffic, "traffic_source": traffic_note, "kernel": kernel_symbol(dom) + " per-tensor", "shape": dom["name"], "us_per_launch": dom["us"]},
        }
        detail["decode"] = shapes
        if "value" in out:
            out["decode"] = dec
        else:
            out.update({"value": dec["value"], "ms_per_step": round(tot_us * 1e-3, 5), "roofline": dec["roofline"]})
            out["_metric"], out["_unit"] = dec["metric"], "GB/s"

    # ------------------------------------------------------------------ block scaled / MoE (extra)
    if args.workload in ("block", "all"):
        shapes = []
        for (N, K) in W.BLOCK_SCALED_SHAPES:
            big = W.block_scaled_case(4096, N, K)
            for M in W.BLOCK_SCALED_M:
                case = W.DenseCase(f"c4_block_M{M}_{N}x{K}", big.a[:M].contiguous(), big.b, big.scale_a[:M].contiguous(), big.scale_b, True, True)
                r = DenseRunner(case, device, copies=_copies_for(case.algorithmic_bytes()) if M <= 64 else 2)
                shapes.append(measure_shape(r, args.steps if M > 64 else max(args.steps, 64), args.warmup, stream,
                                            use_graph=(M <= 64 and not args.no_graph), ramp=M > 64))
                del r
            torch.cuda.empty_cache()
        detail["block_scaled"] = shapes
        if not args.no_yardsticks:
            out["issue_yardstick"] = _issue_yardstick(device, stream)
    if args.workload in ("moe", "all"):
        shapes = []
        for which in ("gate_up", "down"):
            r = RaggedRunner(W.moe_grouped_case(which), device, copies=2)
            shapes.append(measure_shape(r, args.steps, args.warmup, stream, use_graph=False, ramp=True))
            del r
            torch.cuda.empty_cache()
        detail["moe_grouped"] = shapes
        # the whole FP8 MoE layer those GEMMs sit in (fused_moe: align, 1x128 activation quantizer, GEMM1 with the
        # SiLU-multiply + re-quantization epilogue, GEMM2 with the routed weights, top-k sum)
        from tilegym_amd.ops import fused_moe
        up, down = W.moe_grouped_case("gate_up"), W.moe_grouped_case("down")
        ids, tw = up.extra["topk_ids"].to(device), up.extra["topk_weights"].to(device)
        T, H, I = ids.shape[0], up.b.shape[2], down.b.shape[2]
        hidden = torch.randn(T, H, device=device).to(torch.bfloat16)
        w1, w2, s1, s2 = up.b.to(device), down.b.to(device), up.b_scale.to(device), down.b_scale.to(device)
        fn = lambda i: fused_moe(hidden, w1, w2, tw, ids, w1_scale=s1, w2_scale=s2)  # noqa: E731
        _ramp(fn)
        for w in range(max(2, args.warmup)):
            fn(w)
        n = max(args.steps, 20)
        us = _events_ms(fn, n, stream) * 1e3 / n
        flops = 2.0 * T * ids.shape[1] * (2 * I * H + H * I)
        detail["moe_layer"] = [{"name": f"c5_fused_moe_T{T}_E{w1.shape[0]}_top{ids.shape[1]}_H{H}_I{I}", "us": round(us, 2),
                                "tflops": round(flops / us * 1e-6, 1), "frac_mfma": round(flops / us * 1e-6 / PEAK_FP8_TFLOPS, 4),
                                "note": "five launches per call, outputs allocated by torch inside the timed region"}]
        # MoE decode regime: T tokens on config 5's weights (the reference has a swap-AB variant for it,
        # src/tilegym/suites/flashinfer/cutile/gemm/ragged_block_scaled_bmm.py:189-322).  Bytes = the touched experts'
        # weights and scales + activations in and out; roofline HBM.  Ragged GEMMs (graph replay) and the whole layer.
        dec_shapes = []
        for T_dec in (() if args.no_yardsticks else (1, 16, 64)):
            for which in ("gate_up", "down"):
                gcase = W.moe_decode_case(up if which == "gate_up" else down, T_dec)
                sizes = (gcase.m_indptr[1:] - gcase.m_indptr[:-1])
                touched = int((sizes > 0).sum())
                E_, N_, K_ = gcase.b.shape
                rows = int(gcase.m_indptr[-1])
                nbytes = touched * (N_ * K_ + (N_ // 128) * (K_ // 128) * 4) + rows * (K_ + (K_ // 128) * 4 + N_ * 2)
                # no cold-cache rotation over copies of the whole 369 MB weight set: only the touched experts' rows are read,
                # and they differ per copy anyway (the rotation is over whole weight tensors)
                r = RaggedRunner(gcase, device, copies=2 if touched * N_ * K_ > (128 << 20) else 4)
                for i in range(3):
                    r(i)
                torch.cuda.synchronize()
                cfg = _lib.last_config()
                per_graph = r.copies * 4
                ms = None if args.no_graph else _graph_ms(r, per_graph, max(1, 64 // per_graph), stream)
                launches = per_graph * max(1, 64 // per_graph)
                if ms is None:
                    launches = 64
                    ms = _events_ms(r, launches, stream)
                us = ms * 1e3 / launches
                dec_shapes.append({"name": f"c5_moe_decode_T{T_dec}_{which}", "kernel": cfg["KERNEL_NAME"], "block_m": cfg["BLOCK_M"],
                                   "block_n": cfg["BLOCK_N"], "touched_experts": touched, "rows": rows, "us": round(us, 3),
                                   "gbs": round(nbytes / us * 1e-3, 1), "frac_hbm": round(nbytes / us * 1e-3 / PEAK_HBM_GBS, 4),
                                   "eager_us": round(_eager_us(r, 100, stream), 2)})
                del r
                torch.cuda.empty_cache()
            ids_d, tw_d = W.moe_routing(T_dec, w1.shape[0], ids.shape[1], seed=T_dec)[1].to(device), W.moe_routing(T_dec, w1.shape[0], ids.shape[1], seed=T_dec)[0].to(device)
            hid_d = torch.randn(T_dec, H, device=device).to(torch.bfloat16)
            fn_d = lambda i: fused_moe(hid_d, w1, w2, tw_d, ids_d, w1_scale=s1, w2_scale=s2)  # noqa: E731
            us = _eager_us(fn_d, 50, stream)
            touched = int(torch.unique(ids_d).numel())
            nbytes = touched * (w1[0].numel() + w2[0].numel() + (s1[0].numel() + s2[0].numel()) * 4) + T_dec * H * 4
            dec_shapes.append({"name": f"c5_fused_moe_decode_T{T_dec}", "touched_experts": touched, "us": round(us, 2),
                               "gbs": round(nbytes / us * 1e-3, 1), "frac_hbm": round(nbytes / us * 1e-3 / PEAK_HBM_GBS, 4),
                               "note": "eager calls of the whole layer (host cost included), weights hot in the memory-side cache"})
        detail["moe_decode"] = dec_shapes
        detail["moe_layer"][0]["eager_us"] = detail["moe_layer"][0]["us"]
        del hidden, w1, w2, s1, s2
        torch.cuda.empty_cache()

    if args.workload in ("quant", "all"):
        # the producers either side of the GEMM: 1x128 activation quantizer (HBM-bound) and moe_align_block_size
        shapes = []
        for (M, K) in ((8192, 4096), (8192, 14336), (24576, 2048)):
            xs = [torch.randn(M, K, device=device, dtype=torch.bfloat16) for _ in range(_copies_for(M * K * 3))]
            fn = lambda i: _lib.fp8_quant_1x128(xs[i % len(xs)], 0.0, False)  # noqa: E731
            for w in range(max(1, args.warmup)):
                fn(w)
            n = max(args.steps, 32)
            us_alloc = _events_ms(fn, n, stream) * 1e3 / n
            q_out, s_out = _lib.fp8_quant_1x128(xs[0], 0.0, False)
            fn = lambda i: _lib.fp8_quant_1x128(xs[i % len(xs)], 0.0, False, q=q_out, scales=s_out)  # noqa: E731
            fn(0)
            us = _events_ms(fn, n, stream) * 1e3 / n
            nbytes = M * K * 3 + M * (K // 128) * 4
            shapes.append({"name": f"act_quant_1x128_bf16_{M}x{K}", "kernel": "act_quant_group_kernel", "us": round(us, 2),
                           "gbs": round(nbytes / us * 1e-3, 1), "frac_hbm": round(nbytes / us * 1e-3 / PEAK_HBM_GBS, 4),
                           "us_with_output_allocation": round(us_alloc, 2),
                           "note": "outputs pre-allocated; us_with_output_allocation includes torch.empty of the two outputs"})
            del xs
            torch.cuda.empty_cache()
        for (N, K) in ((28672, 4096), (12288, 5120)):
            ws = [torch.randint(0, 120, (N, K), device=device, dtype=torch.uint8).view(torch.float8_e4m3fn)
                  for _ in range(_copies_for(N * K * 3))]
            sc = torch.rand(N // 128, K // 128, device=device) + 0.5
            fn = lambda i: _lib.fp8_weight_dequant(ws[i % len(ws)], sc, 128, torch.bfloat16)  # noqa: E731
            for w in range(max(1, args.warmup)):
                fn(w)
            n = max(args.steps, 32)
            us_alloc = _events_ms(fn, n, stream) * 1e3 / n
            y_out = _lib.fp8_weight_dequant(ws[0], sc, 128, torch.bfloat16)
            fn = lambda i: _lib.fp8_weight_dequant(ws[i % len(ws)], sc, 128, torch.bfloat16, out=y_out)  # noqa: E731
            fn(0)
            us = _events_ms(fn, n, stream) * 1e3 / n
            nbytes = N * K * 3 + sc.numel() * 4
            shapes.append({"name": f"weight_dequant_bf16_{N}x{K}", "kernel": "weight_dequant_kernel", "us": round(us, 2),
                           "gbs": round(nbytes / us * 1e-3, 1), "frac_hbm": round(nbytes / us * 1e-3 / PEAK_HBM_GBS, 4),
                           "us_with_output_allocation": round(us_alloc, 2),
                           "note": "output pre-allocated; us_with_output_allocation includes torch.empty of the output"})
            del ws
            torch.cuda.empty_cache()
        ids = W.moe_routing(4096, 64, 6, seed=0)[1].to(device)
        fn = lambda i: _lib.moe_align_block_size(ids, 128, 64)  # noqa: E731
        for w in range(max(1, args.warmup)):
            fn(w)
        n = max(args.steps, 32)
        us = _events_ms(fn, n, stream) * 1e3 / n
        shapes.append({"name": "moe_align_block_size_4096x6_E64_bs128", "kernel": "moe_align_kernel", "us": round(us, 2),
                       "note": "one launch + five torch.empty"})
        detail["producers"] = shapes

    if "value" not in out:  # block / moe / quant only
        first = next(iter(detail.values()))
        dom = max(first, key=lambda s: s["us"])
        dom.setdefault("tflops", 0.0)
        dom.setdefault("frac_mfma", 0.0)
        out.update({"value": dom["tflops"], "ms_per_step": round(dom["us"] * 1e-3, 5),
                    "roofline": {"bound": "mfma", "achieved": dom["tflops"], "peak": PEAK_FP8_TFLOPS, "unit": "TFLOP/s",
                                 "frac": dom["frac_mfma"], "traffic": None, "shape": dom["name"]}})

    line = {
        "metric": out.pop("_metric", "FP8 GEMM TFLOP/s (prefill: Llama-3.1-8B projections, M=8192, e4m3 per-tensor scales, bf16 out)"),
        "value": out.pop("value"),
        "unit": out.pop("_unit", "TFLOP/s"),
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": out.pop("ms_per_step"),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f8e4m3 (fp32 accumulate)", "data": "synthetic",
        "config": {"workload": {"prefill": "config 3: Llama-3.1-8B prefill projections, M=8192, (N,K) in qkv/o/gate_up/down",
                                "decode": "config 2: Llama-3.1-8B decode projections, M in {1,8,16,64}",
                                "block": "config 4: block-scaled 12288x5120 / 5120x12288, M in {16,4096}",
                                "moe": "config 5: DeepSeek-V2-Lite MoE grouped GEMMs",
                                "quant": "producers: 1x128 activation quantizer, moe_align_block_size",
                                "all": "config 3 (headline) + configs 2, 4, 5 + producers"}[args.workload],
                   "device": props.name, "compute_units": props.multi_processor_count,
                   "untimed_load_ramp_ms": RAMP_MS},
    }
    line.update(out)
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline()
    line["shapes"] = {k: [{kk: vv for kk, vv in s.items() if kk not in ("flops", "bytes")} for s in v] for k, v in detail.items()}
    print(json.dumps(line))


if __name__ == "__main__":
    main()
