"""Builds libaussm_hip.so (hand-written HIP for gfx950) in-tree with hipcc.

    python -m aussm_amd.build                 # compile every translation unit and link
    python -m aussm_amd.build --only k_px     # recompile one unit (the others' objects must exist) and relink
    python -m aussm_amd.build --asm DIR       # also keep the compiler's gfx950 assembly in DIR
    python -m aussm_amd.build --experimental  # also build the measured-and-dropped alternative kernels

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

# One translation unit per kernel family: they compile side by side, and a change in one family
# does not recompile the others' objects by hand (`--only k_px` rebuilds one unit and relinks).
SOURCES = ["scan_api.hip", "k_generic.hip", "k_xdl.hip", "k_px.hip"]

# Packed-FP32 instructions are switched off on purpose (see the flag): the kernels are written
# with scalar float arithmetic only.
HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-ffp-contract=fast",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def lib_path() -> str:
    return os.path.join(LIBDIR, LIBNAME)


def _obj(src: str) -> str:
    return os.path.join(LIBDIR, os.path.splitext(src)[0] + ".o")


def _compile(hipcc: str, src: str, verbose: bool, asm_dir: str | None, extra) -> None:
    cmd = [hipcc] + HIPCC_FLAGS + list(extra) + ["-c", os.path.join(CSRC, src), "-o", _obj(src)]
    cwd = LIBDIR
    if asm_dir:
        cmd += ["-save-temps"]
        cwd = asm_dir
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True, cwd=cwd)


def build(verbose: bool = True, asm_dir: str | None = None, only=None, extra=()) -> str:
    """Compile every translation unit (all of them, every time, unless `only` names a subset whose
    siblings' objects already exist) and link libaussm_hip.so."""
    from concurrent.futures import ThreadPoolExecutor
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    os.makedirs(LIBDIR, exist_ok=True)
    if asm_dir:
        os.makedirs(asm_dir, exist_ok=True)
    todo = [s for s in SOURCES if not only or os.path.splitext(s)[0] in only or not os.path.exists(_obj(s))]
    with ThreadPoolExecutor(max_workers=min(len(todo), 8) or 1) as ex:
        for f in [ex.submit(_compile, hipcc, s, verbose, asm_dir, extra) for s in todo]:
            f.result()
    out = lib_path()
    tmp = out + ".tmp"
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC"] + [_obj(s) for s in SOURCES] + ["-o", tmp]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True, cwd=LIBDIR)
    os.replace(tmp, out)
    return out


if __name__ == "__main__":
    argv = sys.argv[1:]
    only = [argv[i + 1] for i, a in enumerate(argv) if a == "--only"]
    extra = ["-DAUSSM_EXPERIMENTAL_KERNELS"] if "--experimental" in argv else []
    build(asm_dir=os.path.abspath(argv[argv.index("--asm") + 1]) if "--asm" in argv else None, only=only or None,
          extra=extra)
    print("built", lib_path())
