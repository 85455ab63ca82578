"""Builds libaussm_hip.so (hand-written HIP for gfx950) in-tree with hipcc.

    python -m aussm_amd.build                 # compile every translation unit and link
    python -m aussm_amd.build --only k_px     # recompile one unit (the others' objects must exist) and relink
    python -m aussm_amd.build --asm DIR       # also keep the compiler's gfx950 assembly in DIR
    python -m aussm_amd.build --experimental  # also build the measured-and-dropped alternative kernels
    python -m aussm_amd.build --check         # compile k_px.hip to assembly and check its listings (below)

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
SOURCES = ["scan_api.hip", "k_generic.hip", "k_xdl.hip", "k_px.hip", "k_dropin.hip"]

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


# ---- listing check of the kernels that track their own loads ------------------------------------
#
# The kernels of scan_px.h (and the prefetch of scan_bwd_xdl.h, into accumulation registers) issue some
# global loads as hand-written instructions and wait for them by count, so that the compiler neither
# sees a load nor places a wait.  Two things the compiler is
# then free to do would silently break them, and both are visible in the assembly it emits:
#   * spilling vector registers (a register that is the destination of a load in flight would be
#     saved before the data has arrived);
#   * touching a load's destination registers between the load and the wait that retires it
#     (copying them, or - when it considers the value dead - reusing them for something else,
#     which the landing data then overwrites).
# check_px_listing() compiles k_px.hip and k_xdl.hip to assembly and looks for both in every kernel
# of the two units.

def scan_listing(text: str):
    """Findings [(line number, instruction)] of one kernel listing: vector or accumulation registers
    touched while they are the destination of a hand-written (ASMSTART ... ASMEND) global load that no
    s_waitcnt vmcnt has retired yet.  The scan follows the file order, not the control flow."""
    import re

    def regs(tok):
        out = set()
        for m in re.finditer(r"\b([va])\[(\d+):(\d+)\]|\b([va])(\d+)\b", tok):
            if m.group(1):
                out.update((m.group(1), r) for r in range(int(m.group(2)), int(m.group(3)) + 1))
            else:
                out.add((m.group(4), int(m.group(5))))
        return out

    inflight, in_asm, found = {}, False, []
    for i, line in enumerate(text.split("\n")):
        s = line.strip()
        if "ASMSTART" in s:
            in_asm = True
            continue
        if "ASMEND" in s:
            in_asm = False
            continue
        if not s or s[0] in ";.":
            continue
        ins = s.split(";")[0]
        if ins.startswith("s_waitcnt") and "vmcnt" in ins:
            k = int(re.search(r"vmcnt\((\d+)\)", ins).group(1))
            issued = sorted(set(inflight.values()))
            keep = set(issued[len(issued) - k:]) if k > 0 else set()
            inflight = {r: ln for r, ln in inflight.items() if ln in keep}
            continue
        if in_asm and re.match(r"global_load_dwordx[24] ", ins):
            ops = ins.split(None, 1)[1].split(",")
            if any(r in inflight for r in regs(ops[1])):
                found.append((i + 1, ins))
            for r in regs(ops[0]):
                inflight[r] = i + 1
            continue
        if any(r in inflight for r in regs(ins)):
            found.append((i + 1, ins))
    return found


def check_unit_listing(unit: str, verbose: bool = True) -> int:
    """Raises RuntimeError if a kernel of the unit touches registers that are the destination of a
    hand-written load in flight, or spills vector registers while such loads land in vector registers;
    returns the number of kernel listings checked."""
    import re
    import tempfile
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    with tempfile.TemporaryDirectory() as tmp:
        out = os.path.join(tmp, os.path.splitext(unit)[0] + ".s")
        cmd = [hipcc] + HIPCC_FLAGS + ["-S", "--cuda-device-only", os.path.join(CSRC, unit), "-o", out]
        if verbose:
            print(" ".join(cmd), flush=True)
        subprocess.run(cmd, check=True, cwd=tmp)
        text = open(out).read()
    problems = []
    kernels = re.findall(r"^(_ZN5aussm\w+):[^\n]*\n(.*?)s_endpgm", text, flags=re.S | re.M)
    if not kernels:
        raise RuntimeError(f"no kernels found in the listing of {unit}")
    by_hand, by_hand_v = set(), set()    # kernels with hand-written loads; ... whose destinations are v registers
    for name, body in kernels:
        if re.search(r"ASMSTART\s*\n\s*global_load", body):
            by_hand.add(name)
        if re.search(r"ASMSTART\s*\n\s*global_load_dwordx[24]\s+v", body):
            by_hand_v.add(name)
        for ln, ins in scan_listing(body):
            problems.append(f"{name}: line {ln}: `{ins.strip()}` touches registers with a load in flight")
    for name, count in re.findall(r"^\s*\.name:\s+(_ZN5aussm\w+)\n(?:.*\n)*?\s*\.vgpr_spill_count:\s+(\d+)", text, flags=re.M):
        # (a spilled v register cannot be the accumulation-register destination of a load in flight)
        if name in by_hand_v and int(count):
            problems.append(f"{name}: {count} vector registers spilled")
    if problems:
        raise RuntimeError(f"{unit}: " + "; ".join(problems))
    if verbose:
        print(f"{unit}: {len(kernels)} kernel listings checked, {len(by_hand)} of them with hand-written loads", flush=True)
    return len(kernels)


def check_px_listing(verbose: bool = True) -> None:
    """The listing check over the two units whose kernels issue loads by hand."""
    for unit in ("k_px.hip", "k_xdl.hip"):
        check_unit_listing(unit, verbose)


if __name__ == "__main__":
    argv = sys.argv[1:]
    if "--check" in argv:
        check_px_listing()
        sys.exit(0)
    only = [argv[i + 1] for i, a in enumerate(argv) if a == "--only"]
    extra = ["-DAUSSM_EXPERIMENTAL_KERNELS"] if "--experimental" in argv else []
    build(asm_dir=os.path.abspath(argv[argv.index("--asm") + 1]) if "--asm" in argv else None, only=only or None,
          extra=extra)
    print("built", lib_path())
