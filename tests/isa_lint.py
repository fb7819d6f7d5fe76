"""Checks the gfx950 assembly of the kernels for two scalar-register hazards that the compiler's own
hazard pass cannot see, because the reading instruction sits inside an asm block:

  * a vector-memory instruction reads a scalar register that a vector-ALU instruction (v_readfirstlane,
    v_readlane, a compare with a scalar destination ...) wrote fewer than 5 issue slots earlier: the
    memory instruction then takes the register's OLD value as part of its address (a scalar-ALU
    instruction that rewrites the register in between ends the hazard);
  * a global->LDS copy reads M0 in the slot right after the scalar-ALU instruction that wrote it
    (one idle slot is required).

and for the two matrix-core hazards of the hand-scheduled kernels, whose MFMAs are asm statements
that the compiler does not recognise as MFMAs:

  * a result register of a v_mfma_f32_32x32x16 (8 passes) is read or written by a non-MFMA
    instruction, or read as the A or B operand of another MFMA, fewer than 11 slots after the MFMA
    was issued (accumulating into the same registers, C = D, needs no distance);
  * an MFMA reads a register that a vector-ALU instruction wrote fewer than 2 slots earlier.

  * a non-transcendental vector instruction reads the result of a transcendental one (v_exp, v_log,
    v_rcp, v_rsq, v_sqrt, v_sin, v_cos) in the very next slot.

  * the result of a dot-product instruction (v_dot2*, v_dot4*, v_dot8*) is read by a vector-ALU
    instruction of another opcode fewer than 3 slots later, or overwritten by one fewer than 4 slots
    later (the same opcode accumulating into its own result is forwarded by the hardware).

  * a vector-memory store of more than 8 bytes has its data registers overwritten by a vector-ALU
    instruction in the two slots after it (the store still reads them there).

    python isa_lint.py            # compiles every kernel source to assembly and checks it

It also lists the kernels that spill registers to scratch memory (scratch_ops): the hand-scheduled
kernels must not -- the compiler waits for ALL outstanding memory operations before it uses a reloaded
value, the global->LDS copies in flight included.

Slots are counted as the hardware counts wait states: one per instruction, N+1 for `s_nop N`.
The scan is linear (labels and branches are ignored), which is what the hardware sees on the
fall-through path and is conservative for the others.
"""
from __future__ import annotations

import os
import re
import subprocess
import sys
import tempfile
from concurrent.futures import ThreadPoolExecutor

import build as _build

VMEM = ("global_", "buffer_", "flat_", "scratch_")
VMEM_SGPR_SLOTS = 5
M0_DMA_SLOTS = 1


TRANS = ("v_exp_", "v_log_", "v_rcp_", "v_rsq_", "v_sqrt_", "v_sin_", "v_cos_")
MFMA_RESULT_SLOTS = 11
VALU_TO_MFMA_SLOTS = 2
DOT_READ_SLOTS = 3
DOT_WRITE_SLOTS = 4


def _vregs(text: str) -> set[tuple[str, int]]:
    """Vector and accumulation registers named in an operand string, as (file, index)."""
    out: set[tuple[str, int]] = set()
    for m in re.finditer(r"\b([va])\[(\d+):(\d+)\]", text):
        out |= {(m.group(1), i) for i in range(int(m.group(2)), int(m.group(3)) + 1)}
    for m in re.finditer(r"\b([va])(\d+)\b", text):
        out.add((m.group(1), int(m.group(2))))
    return out


def _sregs(text: str) -> set[int]:
    out: set[int] = set()
    for m in re.finditer(r"\bs\[(\d+):(\d+)\]", text):
        out |= set(range(int(m.group(1)), int(m.group(2)) + 1))
    for m in re.finditer(r"\bs(\d+)\b", text):
        out.add(int(m.group(1)))
    return out


def _instructions(asm: str):
    for n, line in enumerate(asm.split("\n"), 1):
        s = line.split(";")[0].strip()
        if not s or s.startswith(".") or s.endswith(":") or s.startswith("//"):
            continue
        yield n, s


def _dest(s: str) -> str:
    parts = s.split(None, 1)
    return parts[1].split(",")[0] if len(parts) > 1 else ""


def _slots(s: str) -> int:
    m = re.match(r"s_nop\s+(\d+)", s)
    return int(m.group(1)) + 1 if m else 1


def lint(asm: str) -> list[str]:
    """Returns one message per hazard found in a gfx9 assembly listing."""
    ins = list(_instructions(asm))
    hits = []
    for i, (ln, s) in enumerate(ins):
        if not s.startswith(VMEM):
            continue
        need = _sregs(s)
        slots, j = 0, i - 1
        while j >= 0 and slots < VMEM_SGPR_SLOTS and need:
            ln2, s2 = ins[j]
            written = _sregs(_dest(s2))
            if s2.startswith("v_") and written & need:
                hits.append(f"line {ln2}: `{s2}` writes a scalar register that line {ln}: `{s}` reads {slots} slot(s) later")
                break
            if s2.startswith("s_"):
                need -= written  # rewritten by the scalar ALU: no hazard through this register
            slots += _slots(s2)
            j -= 1
        if "_lds_" in s or s.rstrip().endswith(" lds"):
            slots, j = 0, i - 1
            while j >= 0 and slots < M0_DMA_SLOTS:
                ln2, s2 = ins[j]
                if s2.startswith("s_") and re.match(r"m0\b", _dest(s2).strip()):
                    hits.append(f"line {ln2}: `{s2}` writes M0 that line {ln}: `{s}` reads {slots} slot(s) later")
                    break
                slots += _slots(s2)
                j -= 1
    hits += _lint_mfma(ins)
    hits += _lint_dot(ins)
    hits += _lint_wide_store(ins)
    for (ln, s), (ln2, s2) in zip(ins, ins[1:]):
        if s.startswith(TRANS) and s2.startswith("v_") and not s2.startswith(TRANS) and not s2.startswith("v_mfma"):
            rest = s2.split(None, 1)[1].split(",", 1)
            if len(rest) > 1 and _vregs(_dest(s)) & _vregs(rest[1]):
                hits.append(f"line {ln}: `{s}` result read by line {ln2}: `{s2}` in the next slot")
    return hits


WIDE_STORE = re.compile(r"(global|flat|buffer|scratch)_store_dwordx[34]\b")
WIDE_STORE_SLOTS = 2


def _lint_wide_store(ins) -> list[str]:
    """A vector-memory store of more than 8 bytes keeps reading its data registers after it was issued:
    a vector-ALU instruction may not overwrite them in the next two issue slots."""
    hits = []
    for i, (ln, s) in enumerate(ins):
        if not WIDE_STORE.match(s):
            continue
        ops = s.split(None, 1)[1].split(",")
        data = _vregs(ops[0] if s.startswith("buffer_") else ops[1] if len(ops) > 1 else "")
        slots, j = 0, i + 1
        while j < len(ins) and slots < WIDE_STORE_SLOTS:
            ln2, s2 = ins[j]
            if s2.startswith("v_") and _vregs(_dest(s2)) & data:
                hits.append(f"line {ln}: `{s}` data overwritten by line {ln2}: `{s2}` {slots} slot(s) later")
                break
            slots += _slots(s2)
            j += 1
    return hits


def _opcode(s: str) -> str:
    return re.sub(r"_e(32|64)$", "", s.split(None, 1)[0])


def _lint_dot(ins) -> list[str]:
    hits = []
    n = len(ins)
    for i, (ln, s) in enumerate(ins):
        if not re.match(r"v_dot\d", s):
            continue
        dst = _vregs(_dest(s))
        slots, j = 0, i + 1
        while j < n and slots < DOT_WRITE_SLOTS:
            ln2, s2 = ins[j]
            if s2.startswith("v_"):
                ops2 = s2.split(None, 1)[1].split(",") if len(s2.split(None, 1)) > 1 else []
                d2 = _vregs(ops2[0]) if ops2 else set()
                srcs = _vregs(",".join(ops2[1:]))
                same = _opcode(s2) == _opcode(s)
                # the accumulator of the same opcode is the last source (VOP3P) or the destination itself (dot2c)
                acc_only = same and not (_vregs(",".join(ops2[1:3])) & dst)
                reads = (srcs | (d2 if re.match(r"v_dot\dc", s2) else set())) & dst
                if reads and not acc_only and slots < DOT_READ_SLOTS:
                    hits.append(f"line {ln}: `{s}` result read by line {ln2}: `{s2}` {slots} slot(s) later")
                elif d2 & dst and not same:
                    hits.append(f"line {ln}: `{s}` result overwritten by line {ln2}: `{s2}` {slots} slot(s) later")
                if d2 & dst:
                    break  # rewritten: later readers see the new value
            slots += _slots(s2)
            j += 1
    return hits


def _lint_mfma(ins) -> list[str]:
    hits = []
    n = len(ins)
    for i, (ln, s) in enumerate(ins):
        if not s.startswith("v_mfma"):
            continue
        ops = s.split(None, 1)[1].split(",")
        dst = _vregs(ops[0])
        # readers of the result
        slots, j = 0, i + 1
        while j < n and slots < MFMA_RESULT_SLOTS:
            ln2, s2 = ins[j]
            if s2.startswith("v_mfma"):
                o2 = s2.split(None, 1)[1].split(",")
                ab, d2, c2 = _vregs(o2[1]) | _vregs(o2[2]), _vregs(o2[0]), _vregs(o2[3])
                if ab & dst or (d2 & dst and d2 != dst) or (c2 & dst and c2 != dst):
                    hits.append(f"line {ln}: `{s}` result used by line {ln2}: `{s2}` {slots} slot(s) later")
            elif not s2.startswith("s_") and _vregs(s2) & dst:
                hits.append(f"line {ln}: `{s}` result touched by line {ln2}: `{s2}` {slots} slot(s) later")
            slots += _slots(s2)
            j += 1
        # operands written just before
        rd = _vregs(ops[1]) | _vregs(ops[2]) | _vregs(ops[3])
        slots, j = 0, i - 1
        while j >= 0 and slots < VALU_TO_MFMA_SLOTS:
            ln2, s2 = ins[j]
            if s2.startswith("v_") and not s2.startswith("v_mfma") and _vregs(_dest(s2)) & rd:
                hits.append(f"line {ln2}: `{s2}` writes an operand of line {ln}: `{s}` {slots} slot(s) later")
            slots += _slots(s2)
            j -= 1
    return hits


def assembly_of(source: str, out_dir: str) -> str:
    """Compiles one kernel source of csrc/ to gfx950 assembly (device side only); returns the text."""
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    out = os.path.join(out_dir, os.path.splitext(source)[0] + ".s")
    flags = [f for f in _build.FLAGS if f not in ("-shared", "-fPIC")]
    cmd = [hipcc] + flags + ["-I", _build.INCLUDE, "-I", _build.CSRC, "--cuda-device-only", "-S", "-o", out,
                             os.path.join(_build.CSRC, source)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc -S failed for {source}:\n{res.stdout}{res.stderr}")
    return open(out).read()


def scratch_ops(asm: str) -> dict[str, int]:
    """Kernels of a listing that access scratch memory (register spills and reloads), with the number
    of such instructions.  (The scratch size a kernel declares can be non-zero for stack objects whose
    accesses were all optimised away; the instructions are what costs.)"""
    out, name = {}, None
    for line in asm.split("\n"):
        m = re.match(r"(_Z\w+):", line)
        if m:
            name = m.group(1)
        elif name is not None and re.match(r"\s*scratch_(load|store)_", line):
            out[name] = out.get(name, 0) + 1
        elif ".end_amdhsa_kernel" in line:
            name = None
    return out


def analyse_sources(sources=None) -> dict[str, tuple[list[str], dict[str, int]]]:
    """Per kernel source: the hazards of its listing and the kernels in it that spill registers."""
    sources = list(sources or _build.SOURCES)
    with tempfile.TemporaryDirectory() as tmp, ThreadPoolExecutor(max_workers=min(8, len(sources))) as ex:
        texts = list(ex.map(lambda s: assembly_of(s, tmp), sources))
    return {s: (lint(t), scratch_ops(t)) for s, t in zip(sources, texts)}


def lint_sources(sources=None) -> dict[str, list[str]]:
    return {s: hits for s, (hits, _) in analyse_sources(sources).items()}


if __name__ == "__main__":
    bad = 0
    for src, hits in lint_sources().items():
        print(f"{src}: {len(hits)} hazard(s)")
        for h in hits:
            print("   ", h)
        bad += len(hits)
    sys.exit(1 if bad else 0)
