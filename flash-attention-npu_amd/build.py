"""Build libfa_rocm.so (C ABI + gfx950 kernels) in-tree with hipcc, then the PyTorch extension module over it.

    python flash-attention-npu_amd/build.py            # compile every translation unit, link
The objects and the library land next to the sources (csrc/build/, csrc/libfa_rocm.so); the extension module
(csrc/torch_binding.cpp, host C++ only, linked against the library) lands in the package as flash_attn_npu/_C*.so."""
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


def _flags(src: str):
    # the sources that pin accumulation registers refuse to compile without the mark of the build that checks them
    return FLAGS + (["-DFA_ROCM_ACC_REGISTERS_CHECKED=1"] if src in ACC_PINNED else [])


def _check_acc_registers(src: str) -> None:
    asm = os.path.join(OUT_DIR, os.path.splitext(src)[0] + ".s")
    cmd = [HIPCC] + _flags(src) + ["--cuda-device-only", "-S", os.path.join(CSRC, src), "-o", asm]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc -S failed for {src}:\n{r.stdout}\n{r.stderr}")
    with open(asm) as f:
        scan_assembly(src, asm, f)


def scan_assembly(src: str, asm: str, lines) -> None:
    """The two checks on the device assembly of a source that pins accumulation registers (lines: its text, line by line)."""
    inside = False
    prev = ""          # the instruction in front of the current one
    for n, line in enumerate(lines, 1):
        code = line.split(";")[0].strip()
        if "ASMSTART" in line:
            inside = True
        elif "ASMEND" in line:
            inside = False
        elif not inside:
            if not code.startswith(".") and re.search(r"\ba\d+\b|\ba\[\d+:\d+\]", code):
                raise RuntimeError(f"{src}: the compiler used an accumulation register on its own ({asm}:{n}: {line.strip()}); "
                                   "the kernel's accumulators would be overwritten")
        if not code or code.startswith(".") or code.endswith(":"):
            continue
        # A hand-written matrix instruction is opaque to the compiler's hazard handling: an operand that the vector
        # instruction right in front of it wrote is read before it has arrived (seen with v_mov_b64 in front of the
        # instruction that zeroes the first accumulator tile).  One instruction in between is enough.
        if inside and code.startswith("v_mfma") and prev.startswith("v_") and not prev.startswith("v_mfma"):
            written = _vregs(prev.split(None, 1)[1].split(",")[0])
            read = set().union(*[_vregs(t) for t in code.split(None, 1)[1].split(",")[1:]])
            if written & read:
                raise RuntimeError(f"{src}: a matrix instruction reads what the vector instruction in front of it wrote "
                                   f"({asm}:{n}: {prev}  ->  {code}); put wait states in front of it")
        prev = code


def _vregs(tok: str) -> set:
    """vector registers named by an assembly operand (v7, v[4:7])"""
    tok = tok.strip()
    m = re.match(r"v\[(\d+):(\d+)\]$", tok)
    if m:
        return set(range(int(m.group(1)), int(m.group(2)) + 1))
    m = re.match(r"v(\d+)$", tok)
    return {int(m.group(1))} if m else set()


def _compile(src: str) -> str:
    obj = os.path.join(OUT_DIR, os.path.splitext(src)[0] + ".o")
    cmd = [HIPCC] + _flags(src) + ["-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{r.stdout}\n{r.stderr}")
    return obj


def build_all(jobs: int = 8, verbose: bool = True) -> str:
    os.makedirs(OUT_DIR, exist_ok=True)
    with ThreadPoolExecutor(max_workers=min(jobs, len(SOURCES) + len(ACC_PINNED))) as ex:
        checks = [ex.submit(_check_acc_registers, src) for src in SOURCES if src in ACC_PINNED]   # the long pole: start first
        objs = list(ex.map(_compile, SOURCES))
        for c in checks:
            c.result()
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stdout}\n{r.stderr}")
    if verbose:
        print(f"built {LIB}")
    return LIB


def build_binding(verbose: bool = True) -> str:
    """flash_attn_npu/_C: pybind11 + libtorch operator layer (torch_binding.cpp), host code only, g++."""
    import sysconfig
    from torch.utils import cpp_extension as ce
    out = os.path.join(HERE, "flash_attn_npu", "_C" + sysconfig.get_config_var("EXT_SUFFIX"))
    torch_lib = ce.library_paths()[0]
    cmd = ([os.environ.get("CXX", "g++"), "-O2", "-fPIC", "-shared", "-std=c++17", "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
            "-DTORCH_EXTENSION_NAME=_C", "-DTORCH_API_INCLUDE_EXTENSION_H", "-D_GLIBCXX_USE_CXX11_ABI=1", "-Wno-deprecated-declarations"]
           + [f"-I{p}" for p in ce.include_paths()] + [f"-I{sysconfig.get_paths()['include']}", "-I/opt/rocm/include",
              os.path.join(CSRC, "torch_binding.cpp"), "-o", out,
              f"-L{torch_lib}", "-lc10", "-lc10_hip", "-ltorch_cpu", "-ltorch_hip", "-ltorch", "-ltorch_python",
              f"-L{CSRC}", "-lfa_rocm", "-Wl,-rpath,$ORIGIN/../csrc", f"-Wl,-rpath,{torch_lib}", "-L/opt/rocm/lib", "-lamdhip64"])
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"building the extension module failed:\n{r.stdout}\n{r.stderr}")
    if verbose:
        print(f"built {out}")
    return out


if __name__ == "__main__":
    build_all()
    build_binding()
    sys.exit(0)
