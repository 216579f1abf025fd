"""Build libfa_rocm.so (C ABI + gfx950 kernels) in-tree with hipcc.

    python flash-attention-npu_amd/build.py            # compile every translation unit, link
The objects and the library land next to the sources (csrc/build/, csrc/libfa_rocm.so)."""
from __future__ import annotations

import os
import re
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OUT_DIR = os.path.join(CSRC, "build")
LIB = os.path.join(CSRC, "libfa_rocm.so")

SOURCES = [
    "fa_rocm_api.cpp",
    "append_rope.hip",
    "decode_paged.hip",
    "decode_wave.hip",
    "decode_mla_i8.hip",
    "prefill_varlen.hip",
    "ragged_rows.hip",
]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17", "-x", "hip",
    # packed-fp32 VALU forms stay off for every kernel of this library
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
] + ([f"-D{d}" for d in os.environ.get("FA_ROCM_DEFINES", "").split()]) + [
]


# Kernels that keep state in accumulation registers (a0..a255) which they address by number in hand-written
# instructions: the compiler must not place anything of its own there.  Their device assembly is checked after
# compilation: outside the hand-written instruction blocks no instruction may name an accumulation register.
ACC_PINNED = {"decode_mla_i8.hip"}


def _check_acc_registers(src: str) -> None:
    asm = os.path.join(OUT_DIR, os.path.splitext(src)[0] + ".s")
    cmd = [HIPCC] + FLAGS + ["--cuda-device-only", "-S", os.path.join(CSRC, src), "-o", asm]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc -S failed for {src}:\n{r.stdout}\n{r.stderr}")
    inside = False
    for n, line in enumerate(open(asm), 1):
        if "ASMSTART" in line:
            inside = True
        elif "ASMEND" in line:
            inside = False
        elif not inside:
            code = line.split(";")[0]
            if not code.strip().startswith(".") and re.search(r"\ba\d+\b|\ba\[\d+:\d+\]", code):
                raise RuntimeError(f"{src}: the compiler used an accumulation register on its own ({asm}:{n}: {line.strip()}); "
                                   "the kernel's accumulators would be overwritten")


def _compile(src: str) -> str:
    obj = os.path.join(OUT_DIR, os.path.splitext(src)[0] + ".o")
    cmd = [HIPCC] + FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{r.stdout}\n{r.stderr}")
    if src in ACC_PINNED:
        _check_acc_registers(src)
    return obj


def build_all(jobs: int = 8, verbose: bool = True) -> str:
    os.makedirs(OUT_DIR, exist_ok=True)
    with ThreadPoolExecutor(max_workers=min(jobs, len(SOURCES))) as ex:
        objs = list(ex.map(_compile, SOURCES))
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stdout}\n{r.stderr}")
    if verbose:
        print(f"built {LIB}")
    return LIB


if __name__ == "__main__":
    build_all()
    sys.exit(0)
