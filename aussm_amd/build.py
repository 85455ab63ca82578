"""Builds libaussm_hip.so (hand-written HIP for gfx950) in-tree with hipcc.

    python -m aussm_amd.build            # compile
    python -m aussm_amd.build --asm DIR  # also keep the compiler's gfx950 assembly in DIR

hipcc cross-compiles without a GPU, so this runs on a CPU-only machine.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")
LIBNAME = "libaussm_hip.so"

SOURCES = ["scan_api.hip"]

# Packed-FP32 instructions are switched off on purpose (see the flag): the kernels are written
# with scalar float arithmetic only.
HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    "-ffp-contract=fast",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def lib_path() -> str:
    return os.path.join(LIBDIR, LIBNAME)


def build(verbose: bool = True, asm_dir: str | None = None) -> str:
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    os.makedirs(LIBDIR, exist_ok=True)
    out = lib_path()
    tmp = out + ".tmp"
    cmd = [hipcc] + HIPCC_FLAGS + [os.path.join(CSRC, s) for s in SOURCES] + ["-o", tmp]
    cwd = LIBDIR
    if asm_dir:
        os.makedirs(asm_dir, exist_ok=True)
        cmd += ["-save-temps"]
        cwd = asm_dir
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True, cwd=cwd)
    os.replace(tmp, out)
    return out


if __name__ == "__main__":
    build(asm_dir=os.path.abspath(sys.argv[sys.argv.index("--asm") + 1]) if "--asm" in sys.argv else None)
    print("built", lib_path())
