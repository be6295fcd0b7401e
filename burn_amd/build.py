"""Builds libburnq_mi355.so (hipcc, gfx950) next to this file.

    python -m burn_amd.build [--force]

hipcc cross-compiles without a GPU, so this runs anywhere the ROCm toolchain is installed. The
library is built in-tree and loaded from here by ``burn_amd._lib``.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
INCLUDE = os.path.join(os.path.dirname(HERE), "include")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "libburnq_mi355.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
COMMON = [
    "--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17", "-Wall", "-Wno-unused-function",
    # no packed-FP32 instruction selection
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    f"-I{INCLUDE}", f"-I{CSRC}",
]
# (source, extra flags). The quantize/dequantize units must not contract a*b+c into an fma:
# their results are compared bit for bit with a CPU that rounds every operation.
SOURCES = [
    ("runtime.cpp", ["-x", "hip"]),
    ("pack.cpp", ["-x", "hip"]),
    ("quantize.hip", ["-ffp-contract=off"]),
    ("dequantize.hip", ["-ffp-contract=off"]),
    ("qmatmul.hip", ["-ffp-contract=off"]),
    ("qskinny.hip", ["-ffp-contract=off"]),
    ("qsplit.hip", ["-ffp-contract=off"]),
    ("qternary.hip", ["-ffp-contract=off"]),
    ("layout.hip", []),
    # (the GEMM's hand-scheduled stage is one fully unrolled loop of 64 MFMA micro-steps, larger
    # than the default limit for "#pragma unroll")
    ("qgemm.hip", ["-ffp-contract=off", "-mllvm", "-pragma-unroll-threshold=1000000"]),
]


def _compile(item):
    src, extra = item
    obj = os.path.join(OBJ, os.path.splitext(src)[0] + ".o")
    cmd = [HIPCC, *COMMON, *extra, "-c", os.path.join(CSRC, src), "-o", obj]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    # the host pass does not know the packed-fp32 feature name; that warning is expected
    err = "\n".join(l for l in proc.stderr.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build(force: bool = True, jobs: int = 4) -> str:
    os.makedirs(OBJ, exist_ok=True)
    if not force and os.path.exists(LIB):
        newest = max(os.path.getmtime(os.path.join(r, f)) for d in (CSRC, INCLUDE)
                     for r, _, fs in os.walk(d) for f in fs)
        if os.path.getmtime(LIB) >= newest:
            return LIB
    with ThreadPoolExecutor(max_workers=jobs + 1) as pool:
        # alongside the objects: the ISA of the prefill GEMM is scanned for any use of a register
        # whose hand-waited global load is still outstanding (see isa_check.py); a finding fails the build
        from . import isa_check
        scan = pool.submit(isa_check.compile_and_check)
        objs = list(pool.map(_compile, SOURCES))
        scan.result()
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", LIB]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"link failed:\n{proc.stderr}")
    return LIB


if __name__ == "__main__":
    print(build(force="--force" in sys.argv or True))
