#!/usr/bin/env python3
"""Build check for one hardware rule that the compiler cannot enforce inside inline assembly.

On gfx9-family hardware a vector-memory instruction must not read a scalar register within five
wait states of a vector instruction writing it (v_readfirstlane, v_readlane, a VALU compare or
carry into a scalar pair): the memory instruction would see the register's old value.  hipcc
inserts the s_nops for the instructions it emits itself; the direct global->LDS loads and the
register scale loads of these kernels are inline assembly, which its hazard recognizer does not
look into.  Most of them carry their own wait states; the ones that do not (direct_load_b128_settled)
rely on this check.

    python3 check_hazards.py file.s [file.s ...]     # assembly from hipcc --cuda-device-only -S
    python3 check_hazards.py --build [name.hip ...]   # compile the sources beside this file first

Walks every kernel's control-flow graph backwards from each buffer_/global_/scratch_/flat_
instruction over all paths, five wait states deep (s_nop N counts N + 1, everything else 1).
Exit status 1 and one line per finding if a scalar operand was written by a vector instruction
inside that window.

Second rule, same reason: the compiler takes the result register of an inline-assembly
buffer_load as written when the statement ends, while the data arrives later (the kernels wait
with s_waitcnt vmcnt by hand).  A register copy that the compiler places between the load and
that wait (at a loop's back edge, say) would copy the old contents.  Walks forwards from every
buffer_load into registers: a finding if any path reads or overwrites the destination before an
s_waitcnt with a vmcnt field.
"""
import os
import re
import subprocess
import sys
import tempfile

WAIT_STATES = 5
VMEM_PREFIXES = ("buffer_", "global_", "scratch_", "flat_")
CARRY_OPS = ("v_div_scale", "v_mad_u64_u32", "v_mad_i64_i32")
HIPCC_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Xclang", "-target-feature", "-Xclang",
               "-packed-fp32-ops", "--cuda-device-only", "-S"]
# Instantiations with a known finding of the second rule on a path that cannot run: the TAIL forms of the persistent
# block-scaled kernel keep a test in front of a chunk's second K step (without it the compiler spills 126-216
# registers), so the code has a path "chunk of one step" on which the scale requests of the first step reach the loop's
# register copies and the epilogue without a wait.  The launcher refuses every K with such a chunk (bs256_takes_k).
# Traced by hand to that path; the first rule applies to them like to every kernel.
EARLY_USE_KNOWN = ("fp8_gemm_bs256_kernelILi0ELb1E", "fp8_gemm_bs256_kernelILi1ELb1E")
# Third check, of speed rather than correctness: vector registers spilled by the kernels whose loops are hand-scheduled.
# A source change that looks harmless can push one of them over the register file (the TAIL forms went from 0 to
# 129 / 216 spilled registers, and 2.7 times the run time, when their second K step was made unconditional).
VGPR_SPILL_LIMITS = {"fp8_gemm_tile256_kernel": 0, "fp8_gemm_bs256_kernelILi0ELb0E": 52, "fp8_gemm_bs256_kernelILi0ELb1E": 0,
                     "fp8_gemm_bs256_kernelILi1ELb0E": 17, "fp8_gemm_bs256_kernelILi1ELb1E": 0}
# translation units with inline-assembly memory instructions
DEFAULT_SOURCES = ["fp8_gemm_tile_pt.hip", "fp8_gemm_tile256.hip", "fp8_gemm_tile_bs.hip", "fp8_gemm_tile_bs256.hip",
                   "fp8_gemm_tile_grouped.hip", "fp8_gemm_tile_list.hip", "fp8_gemm_stream.hip"]


def scalar_regs(tok):
    m = re.fullmatch(r"s\[(\d+):(\d+)\]", tok)
    if m:
        return set(range(int(m.group(1)), int(m.group(2)) + 1))
    m = re.fullmatch(r"s(\d+)", tok)
    if m:
        return {int(m.group(1))}
    if tok in ("vcc", "vcc_lo", "vcc_hi"):
        return {"vcc"}
    return set()


def valu_scalar_writes(op, toks):
    """Scalar registers a vector instruction writes."""
    if not op.startswith("v_") or not toks:
        return set()
    dst = scalar_regs(toks[0])
    if len(toks) > 1 and ("_co_" in op or op.startswith(CARRY_OPS)):
        dst |= scalar_regs(toks[1])
    if op.endswith("_e32") and (op.startswith("v_cmp") or "_co_" in op):
        dst |= {"vcc"}
    return dst


def parse_kernels(path):
    """{kernel: [(op, operand tokens, text)]} plus each kernel's label -> instruction index."""
    kernels, labels, name = {}, {}, None
    for raw in open(path):
        line = raw.split(";")[0].strip()
        if not line:
            continue
        if line.endswith(":"):
            label = line[:-1]
            if label.startswith(".L") or label.startswith("BB") or label.startswith(".BB"):
                if name is not None:
                    labels[name][label] = len(kernels[name])
            else:
                name = label
                kernels[name], labels[name] = [], {}
            continue
        if line.startswith(".") or name is None:
            continue
        op, _, rest = line.partition(" ")
        toks = [t.strip().split()[0] for t in rest.split(",") if t.strip()]
        kernels[name].append((op, toks, line))
    return kernels, labels


def vector_regs(tok):
    m = re.fullmatch(r"[va]\[(\d+):(\d+)\]", tok)
    if m:
        return set(range(int(m.group(1)), int(m.group(2)) + 1))
    m = re.fullmatch(r"[va](\d+)", tok)
    if m:
        return {int(m.group(1))}
    return set()


def successors(insts, labels):
    succs = [[] for _ in insts]
    for i, (op, toks, _) in enumerate(insts):
        if op not in ("s_branch", "s_endpgm", "s_setpc_b64") and i + 1 < len(insts):
            succs[i].append(i + 1)
        if op == "s_branch" or op.startswith("s_cbranch"):
            target = labels.get(toks[-1] if toks else "")
            if target is not None and target < len(insts):
                succs[i].append(target)
    return succs


def scan_early_use(path):
    """buffer loads into registers whose destination is touched before any vmcnt wait."""
    findings = []
    kernels, labels = parse_kernels(path)
    for name, insts in kernels.items():
        if any(known in name for known in EARLY_USE_KNOWN):
            continue
        succs = successors(insts, labels[name])
        for i, (op, toks, text) in enumerate(insts):
            if not op.startswith("buffer_load") or " lds" in text or not toks:
                continue
            dst = vector_regs(toks[0])
            stack, seen = list(succs[i]), set()
            while stack:
                j = stack.pop()
                if j in seen:
                    continue
                seen.add(j)
                jop, jtoks, jtext = insts[j]
                if jop == "s_waitcnt" and "vmcnt(" in jtext:
                    continue
                touched = set()
                for t in jtoks:
                    touched |= vector_regs(t)
                if touched & dst:
                    findings.append(f"{os.path.basename(path)}: {name}: '{text}' then '{jtext}' with no vmcnt wait between")
                    continue
                stack.extend(succs[j])
    return findings


def scan_spills(path):
    """kernels of VGPR_SPILL_LIMITS whose metadata reports more spilled vector registers than recorded."""
    findings, name = [], None
    for raw in open(path):
        line = raw.strip()
        if line.startswith(".name:"):
            name = line.split()[-1]
        elif line.startswith(".vgpr_spill_count:") and name:
            spilled = int(line.split()[-1])
            for key, limit in VGPR_SPILL_LIMITS.items():
                if key in name and spilled > limit:
                    findings.append(f"{os.path.basename(path)}: {name}: {spilled} spilled vector registers (recorded: {limit})")
    return findings


def predecessors(insts, labels):
    preds = [[] for _ in insts]
    for i, (op, toks, _) in enumerate(insts):
        falls = op not in ("s_branch", "s_endpgm", "s_setpc_b64")
        if falls and i + 1 < len(insts):
            preds[i + 1].append(i)
        if op == "s_branch" or op.startswith("s_cbranch"):
            target = labels.get(toks[-1] if toks else "")
            if target is not None and target < len(insts):
                preds[target].append(i)
    return preds


def scan(path):
    findings = []
    kernels, labels = parse_kernels(path)
    for name, insts in kernels.items():
        preds = predecessors(insts, labels[name])
        writes = [valu_scalar_writes(op, toks) for op, toks, _ in insts]
        for i, (op, toks, text) in enumerate(insts):
            if not op.startswith(VMEM_PREFIXES):
                continue
            used = set()
            for t in toks:
                used |= scalar_regs(t)
            if not used:
                continue
            stack, seen = [(j, 0) for j in preds[i]], set()
            while stack:
                j, waited = stack.pop()
                if (j, waited) in seen:
                    continue
                seen.add((j, waited))
                if writes[j] & used:
                    findings.append(f"{os.path.basename(path)}: {name}: '{insts[j][2]}' -> '{text}' after {waited} wait states")
                    continue
                jop, jtoks, _ = insts[j]
                waited += int(jtoks[0], 0) + 1 if jop == "s_nop" and jtoks else 1
                if waited < WAIT_STATES:
                    stack.extend((k, waited) for k in preds[j])
    return findings


def main(argv):
    files = argv
    tmp = None
    if argv and argv[0] == "--build":
        here = os.path.dirname(os.path.abspath(__file__))
        hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
        tmp = tempfile.TemporaryDirectory()
        files, procs = [], []
        for src in argv[1:] or DEFAULT_SOURCES:
            out = os.path.join(tmp.name, os.path.splitext(os.path.basename(src))[0] + ".s")
            procs.append(subprocess.Popen([hipcc, *HIPCC_FLAGS, os.path.join(here, src), "-o", out],
                                          stderr=subprocess.DEVNULL))
            files.append(out)
        if any(p.wait() != 0 for p in procs):
            print("check_hazards: a source did not compile", file=sys.stderr)
            return 2
    findings = []
    for f in files:
        findings += scan(f) + scan_early_use(f) + scan_spills(f)
    for line in findings:
        print(line)
    print(f"check_hazards: {len(files)} file(s), {len(findings)} finding(s)")
    return 1 if findings else 0


if __name__ == "__main__":
    sys.exit(main(sys.argv[1:]))
