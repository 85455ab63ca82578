"""Builds libaussm_hip.so (hand-written HIP for gfx950) in-tree with hipcc.

    python -m aussm_amd.build                 # compile every translation unit and link
    python -m aussm_amd.build --only k_px     # recompile one unit (the others' objects must exist) and relink
    python -m aussm_amd.build --asm DIR       # also keep the compiler's gfx950 assembly in DIR
    python -m aussm_amd.build --check         # compile k_px.hip to assembly and check its listings (below)

hipcc cross-compiles without a GPU, so this runs on a CPU-only machine.

The kernels of k_px.hip and k_xdl.hip track some of their loads by hand (see check_unit_listing):
they were validated with the compiler named in VALIDATED_HIPCC, every build checks their listings,
and a build with another compiler says so.
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


# `hipcc --version` line ("HIP version: ...") of the compiler the hand-tracked loads were validated with
VALIDATED_HIPCC = "HIP version: 7.2.26015-fc0010cf6a"
# units whose kernels issue loads as hand-written instructions: their listings are checked by every build
HAND_TRACKED = ("k_px.hip", "k_xdl.hip")


def hipcc_version(hipcc: str) -> str:
    out = subprocess.run([hipcc, "--version"], capture_output=True, text=True).stdout
    for line in out.splitlines():
        if line.startswith("HIP version"):
            return line.strip()
    return out.strip().splitlines()[0] if out.strip() else "unknown"


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
    ver = hipcc_version(hipcc)
    if ver != VALIDATED_HIPCC:
        print(f"aussm_amd.build: WARNING: compiling with `{ver}`; the kernels that track their loads by hand were "
              f"validated with `{VALIDATED_HIPCC}` (their listings are checked below)", file=sys.stderr, flush=True)
    if only:
        # the argument blocks in the headers are shared by every unit: an object older than a header would be
        # linked against kernels with another layout of their arguments
        newest = max(os.path.getmtime(os.path.join(CSRC, f)) for f in os.listdir(CSRC) if f.endswith(".h"))
        incl = os.path.getmtime(os.path.join(os.path.dirname(HERE), "include", "aussm_hip.h"))
        stale = [s for s in SOURCES if os.path.splitext(s)[0] not in only and os.path.exists(_obj(s))
                 and os.path.getmtime(_obj(s)) < max(newest, incl)]
        if stale:
            print(f"aussm_amd.build: a header is newer than the objects of {stale}: rebuilding every unit", flush=True)
            only = None
    todo = [s for s in SOURCES if not only or os.path.splitext(s)[0] in only or not os.path.exists(_obj(s))]
    # the listings of the hand-tracked units among them are checked alongside (same compiler, same flags);
    # a finding fails the build before the library is put in place
    with ThreadPoolExecutor(max_workers=8) as ex:
        jobs = [ex.submit(_compile, hipcc, s, verbose, asm_dir, extra) for s in todo]
        jobs += [ex.submit(check_unit_listing, u, verbose) for u in HAND_TRACKED if u in todo]
        for f in jobs:
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
    s_waitcnt vmcnt has retired yet.  The scan follows the file order; at a branch back to a loop header
    (a label the compiler marks "Loop Header") with loads still in flight it also walks the loop body once
    more from that label with those loads in flight, so a load issued at the end of an iteration and retired
    at the top of the next is followed across the edge.  (Blocks the compiler places out of line, behind the
    loop, also branch back to earlier labels; those are not back-edges and the state the file order has
    there is not the state of their entry, so they are not followed.)"""
    import re

    def regs(tok):
        out = set()
        for m in re.finditer(r"\b([va])\[(\d+):(\d+)\]|\b([va])(\d+)\b", tok):
            if m.group(1):
                out.update((m.group(1), r) for r in range(int(m.group(2)), int(m.group(3)) + 1))
            else:
                out.add((m.group(4), int(m.group(5))))
        return out

    lines = text.split("\n")
    labels = {}
    for i, line in enumerate(lines):
        m = re.match(r"^(\.LBB\w+):(.*)", line.strip())
        if m and ("Loop Header" in m.group(2) or "Loop Header" not in text):
            labels[m.group(1)] = i

    found = []

    def walk(start, end, inflight, follow):
        in_asm = False
        for i in range(start, end):
            s = lines[i].strip()
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
                if not follow and not inflight:
                    return
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
            if follow and inflight and ins.startswith("s_cbranch"):
                tgt = ins.split()[-1]
                if tgt in labels and labels[tgt] < i:
                    # (loads carried over the edge are older than anything the body issues: line numbers below it)
                    walk(labels[tgt], i, {r: ln - len(lines) for r, ln in inflight.items()}, False)

    walk(0, len(lines), {}, True)
    return sorted(set(found))


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
    for unit in HAND_TRACKED:
        check_unit_listing(unit, verbose)


if __name__ == "__main__":
    argv = sys.argv[1:]
    if "--check" in argv:
        check_px_listing()
        sys.exit(0)
    only = [argv[i + 1] for i, a in enumerate(argv) if a == "--only"]
    build(asm_dir=os.path.abspath(argv[argv.index("--asm") + 1]) if "--asm" in argv else None, only=only or None)
    print("built", lib_path())
