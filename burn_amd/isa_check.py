"""Build-time checks of the prefill q-GEMM's hand-managed global loads and matrix instructions.

qgemm.hip issues its global loads through inline asm, so the compiler does not know that the
destination registers are written asynchronously: only the kernel's own `s_waitcnt vmcnt(N)`
statements make them valid. A register allocator decision (a copy at the loop back-edge, a
spill, the reuse of a register whose load is dead) could touch such a register early and would
silently corrupt data. This module scans the generated ISA of every `qgemm_kernel` instantiation:
it replays the instruction stream (prologue, three trips of the main loop, epilogue) with an
in-order queue of outstanding loads, retires loads at every `s_waitcnt vmcnt(N)`, and reports any
instruction that reads or overwrites a register whose load is still outstanding.

The matrix instructions are inline asm as well, so the compiler's hazard recognizer does not see
them either: a vector instruction may read an accumulator only kMfmaDrain wait states after the
last MFMA that wrote it (the kernel drains with `s_nop`s before it leaves the loop). The same scan
counts the wait states between every MFMA and the first other instruction that reads its result.

    python -m burn_amd.isa_check            # compiles qgemm.hip to ISA and checks it
"""
from __future__ import annotations

import os
import re
import subprocess
import sys
import tempfile

HERE = os.path.dirname(os.path.abspath(__file__))

_REG = re.compile(r"\bv\[(\d+):(\d+)\]|\bv(\d+)\b")
_ACC = re.compile(r"\ba\[(\d+):(\d+)\]|\ba(\d+)\b")
# wait states a 16-pass matrix instruction needs before a vector instruction may read its result
# (one per issued instruction, N + 1 per `s_nop N`); the kernel's drain is 48
kMfmaDrain = 20
_LOADS = ("buffer_load", "global_load", "scratch_load")
_NO_DEST = ("ds_write", "buffer_store", "global_store", "scratch_store", "s_", "v_cmp")


def _regs(text):
    out = set()
    for m in _REG.finditer(text):
        if m.group(1):
            out |= set(range(int(m.group(1)), int(m.group(2)) + 1))
        else:
            out.add(int(m.group(3)))
    return out


def _kernels(lines):
    """(name, body lines) of every qgemm_kernel instantiation in an ISA listing."""
    i = 0
    while i < len(lines):
        m = re.match(r"^(_ZN2bq\S*qgemm_kernel\S*):", lines[i])
        if m:
            end = next(j for j in range(i, len(lines)) if "s_endpgm" in lines[j])
            yield m.group(1), lines[i:end]
            i = end
        i += 1


def _accs(text):
    out = set()
    for m in _ACC.finditer(text):
        if m.group(1):
            out |= set(range(int(m.group(1)), int(m.group(2)) + 1))
        else:
            out.add(int(m.group(3)))
    return out


def check_mfma_drain(seq):
    """Instructions other than MFMAs that read an accumulator register too soon after the MFMA that
    wrote it. `seq`: the instruction stream as it executes (the loop unrolled)."""
    written, hazards = {}, []          # accumulator register -> wait states since its last MFMA
    for line in seq:
        line = line.split(";")[0].strip()
        if not line or line.endswith(":") or line.startswith("."):
            continue
        op, _, rest = line.partition(" ")
        ops = rest.split(",")
        if op.startswith("v_mfma"):
            for r in written:
                written[r] += 1
            for r in _accs(ops[0]):
                written[r] = 0
            continue
        if op == "s_nop":
            step = int(rest.strip()) + 1
        else:
            step = 1
            early = [r for r in _accs(",".join(ops[1:]) if not op.startswith(_NO_DEST) else rest)
                     if written.get(r, kMfmaDrain) < kMfmaDrain]
            if early:
                hazards.append((line, sorted(early)))
        for r in written:
            written[r] += step
    return hazards


def check_kernel(body):
    """Returns (hazards, max outstanding loads) of one kernel body."""
    hdr = next(i for i, l in enumerate(body) if "Inner Loop Header" in l)
    back = next(i for i in range(hdr, len(body)) if re.search(r"s_cbranch_\w+ \.LBB\d+_\d+", body[i]))
    loop = body[hdr:back + 1]

    def without_exit_drain(ls):  # the vmcnt(0) + s_nop drain runs on the last trip only
        return [l for i, l in enumerate(ls)
                if not ("s_waitcnt vmcnt(0)" in l and i + 1 < len(ls) and "s_nop 15" in ls[i + 1])]

    seq = body[:hdr] + without_exit_drain(loop) * 2 + loop + body[back + 1:]
    pending, hazards, max_out = [], [], 0
    for line in seq:
        line = line.split(";")[0].strip()
        if not line or line.endswith(":") or line.startswith("."):
            continue
        op, _, rest = line.partition(" ")
        rest = rest.strip()
        if op == "s_waitcnt":
            m = re.search(r"vmcnt\((\d+)\)", rest)
            if m:
                keep = int(m.group(1))
                pending = pending[len(pending) - keep:] if keep and len(pending) > keep else \
                    (pending if keep else [])
            continue
        ops = rest.split(",")
        is_load = op.startswith(_LOADS)
        if op.startswith(_NO_DEST):
            dst, src = set(), _regs(rest)
        else:
            dst, src = _regs(ops[0]), _regs(",".join(ops[1:]))
            if op.startswith(("v_mfma", "v_fmac")):
                src |= dst
        in_flight = set().union(*pending) if pending else set()
        # a load may target a register that is still in flight (loads return in order)
        hit = (src if is_load else (src | dst)) & in_flight
        # v_mad_u64_u32 reads a 64-bit addend whose high half the compiler leaves undefined: the
        # value read there is never used
        if hit and not (op.startswith("v_mad_u64_u32") and len(hit) == 1):
            hazards.append((line, sorted(hit)))
        if is_load:
            pending.append(dst)
            max_out = max(max_out, len(pending))
    # the matrix instructions' results: the last trip (with its drain) and what follows the loop
    hazards += check_mfma_drain(body[:hdr] + without_exit_drain(loop) + loop + body[back + 1:])
    return hazards, max_out


def check_listing(path):
    lines = open(path).read().split("\n")
    report = {}
    for name, body in _kernels(lines):
        report[name] = check_kernel(body)
    if not report:
        raise RuntimeError(f"no qgemm_kernel instantiation found in {path}")
    return report


def compile_and_check(hipcc=None, flags=None):
    """Compiles csrc/qgemm.hip to ISA with the library's flags and checks it. Raises on a finding."""
    from . import build as b
    src = os.path.join(b.CSRC, "qgemm.hip")
    extra = dict(b.SOURCES)["qgemm.hip"]
    with tempfile.TemporaryDirectory() as tmp:
        asm = os.path.join(tmp, "qgemm.s")
        cmd = [hipcc or b.HIPCC, *[f for f in (flags or b.COMMON) if f != "-fPIC"], *extra,
               "-S", "--cuda-device-only", src, "-o", asm]
        proc = subprocess.run(cmd, capture_output=True, text=True)
        if proc.returncode != 0:
            raise RuntimeError(f"hipcc -S failed for qgemm.hip:\n{proc.stderr}")
        report = check_listing(asm)
    bad = {k: v for k, v in report.items() if v[0]}
    if bad:
        msg = "\n".join(f"{k}: {len(h)} finding(s), first: {h[0][0]} (registers {h[0][1]})"
                        for k, (h, _) in bad.items())
        raise RuntimeError("qgemm.hip: a register is touched before its load's wait, or an accumulator is read "
                           "before its matrix instruction has drained:\n" + msg)
    return report


if __name__ == "__main__":
    rep = compile_and_check()
    for name, (haz, out) in sorted(rep.items()):
        print(f"{name[:90]}: {len(haz)} findings, up to {out} loads outstanding")
    print(f"{len(rep)} instantiations checked")
    sys.exit(0)
