#!/usr/bin/env python3
"""Headline benchmark: adaptive-unitary core scan, forward + backward, fp32,
B=32 D=512 N=16 L=2048, on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--shape B,D,N,L]

(--shape runs the same step at another shape, e.g. 4,256,16,16384, the long-sequence case whose
launches are split along L; the default and the contract line are the headline shape.)

One "step" = one forward launch (y, checkpoints) + zero-fill of the accumulated gradients +
one backward launch (du, ddelta, dtheta, dB, dC, dD) on synthetic inputs that are already
resident in HBM.  Prints ONE JSON line.

  value          (b,d,l) samples per second over forward+backward (B*D*L / step time)
  roofline       dominant kernel (the backward scan): algorithmic bytes (28E + 32S + 4D,
                 E = B*D*L, S = B*N*L) / the average duration of one backward call (the scan kernel
                 and the two launches around it that leave at once in a training step), measured here
                 with HIP events on the launch stream, against the 8 TB/s HBM peak.  The operand
                 pre-pass of the step runs inside the forward call, whose figures carry it.  "traffic" is
                 the HBM bytes per call from rocprofv3 FETCH_SIZE / WRITE_SIZE passes over this same
                 script, scaled by what the counters read for the 256 MiB device copy that
                 --copy-probe adds to the run.  It is read from profiles/traffic.json, which
                 `bench.py --summarize-traffic FETCH_DIR WRITE_DIR` writes from the two passes'
                 output; the file records the kernels it saw and a digest of the kernel sources,
                 and the figure is reported as null when either no longer matches this build.
  cpu_baseline   the CPU oracle (sequential-loop PyTorch scan + autograd) timed on this host's
                 cores on a bounded slice of the batch: one warm-up run, then the median of three

Before the W warm-up steps the step is repeated for --prewarm-ms (default 200 ms, reported as
prewarm_ms) so that clocks and caches are where a long run has them.
"""
from __future__ import annotations

import argparse
import glob
import hashlib
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
SHAPE = dict(B=32, D=512, N=16, L=2048)
TRAFFIC_JSON = os.path.join(ROOT, "profiles", "traffic.json")
# kernels of one call, by the kernel family the library reports (aussm_unitary_kernel_mode)
# (family 6: the forward call's pre-pass prepares the operands of both directions; the backward call's instance of
# it - <float, true> - finds them and leaves at once, as does the recomputing kernel launched behind the scan kernel)
FWD_KERNELS = {0: ["core_fwd_kernel<0"], 2: ["unitary_fwd_xdl_kernel<2"], 3: ["unitary_fwd_xdl_kernel<3"],
               6: ["unitary_px_prep_kernel<float, false", "unitary_fwd_px_kernel"]}
BWD_KERNELS = {0: ["unitary_bwd_kernel"], 2: ["unitary_bwd_xdl_kernel<2"], 3: ["unitary_bwd_xdl_kernel<3, 2"],
               5: ["unitary_bwd_xdl_kernel<3, 3"],
               6: ["unitary_bwd_px_kernel", "unitary_px_prep_kernel<float, true", "unitary_bwd_xdl_kernel<3, 2"]}


def source_digest() -> str:
    """Digest of the kernel sources: a traffic record is only valid for the sources it was taken with."""
    h = hashlib.sha256()
    for f in sorted(glob.glob(os.path.join(ROOT, "aussm_amd", "csrc", "*"))):
        h.update(os.path.basename(f).encode())
        h.update(open(f, "rb").read())
    return h.hexdigest()[:16]


def summarize_traffic(fetch_dir: str, write_dir: str) -> None:
    """profiles/traffic.json from the counter_collection.csv files of two rocprofv3 --pmc passes
    (FETCH_SIZE, WRITE_SIZE) over `bench.py --copy-probe`."""
    import csv

    def per_kernel(d, counter):
        files = glob.glob(os.path.join(d, "**", "*counter_collection.csv"), recursive=True)
        if not files:
            sys.exit(f"no counter_collection.csv under {d}")
        acc = {}
        for row in csv.DictReader(open(max(files, key=os.path.getmtime))):
            if row["Counter_Name"] == counter:
                acc.setdefault(row["Kernel_Name"], []).append(float(row["Counter_Value"]))
        return {k: (sum(v) / len(v), len(v)) for k, v in acc.items()}

    fetch, write = per_kernel(fetch_dir, "FETCH_SIZE"), per_kernel(write_dir, "WRITE_SIZE")
    copy = [k for k in fetch if "copyBuffer" in k]
    if not copy or copy[0] not in write:
        sys.exit("the passes do not contain the 256 MiB copy (run bench.py with --copy-probe)")
    copy_kib = 256.0 * 1024
    scale = {"FETCH_SIZE": copy_kib / fetch[copy[0]][0], "WRITE_SIZE": copy_kib / write[copy[0]][0]}
    kernels = {}
    for k in fetch:
        if "aussm::" in k and k in write:
            kernels[k] = {"fetch_KiB": fetch[k][0], "write_KiB": write[k][0], "dispatches": fetch[k][1],
                          "read_bytes": fetch[k][0] * scale["FETCH_SIZE"] * 1024,
                          "written_bytes": write[k][0] * scale["WRITE_SIZE"] * 1024}
    rec = {"shape": SHAPE, "sources": source_digest(), "scale": scale, "copy_kernel": copy[0],
           "copy_KiB": {"FETCH_SIZE": fetch[copy[0]][0], "WRITE_SIZE": write[copy[0]][0]}, "kernels": kernels,
           "command": "rocprofv3 --pmc FETCH_SIZE|WRITE_SIZE --kernel-trace --output-format csv -d <out> -- "
                      "python3 bench.py --steps 3 --warmup 1 --prewarm-ms 0 --no-cpu --copy-probe"}
    json.dump(rec, open(TRAFFIC_JSON, "w"), indent=1)
    print(f"wrote {TRAFFIC_JSON}: {len(kernels)} kernels")


def recorded_traffic(kernel_substrings):
    """(bytes per call, note): sum over the named kernels of read + written bytes in profiles/traffic.json, or
    (None, why) when the record does not cover this build or these kernels."""
    if not os.path.exists(TRAFFIC_JSON):
        return None, "profiles/traffic.json missing"
    rec = json.load(open(TRAFFIC_JSON))
    if rec.get("sources") != source_digest():
        return None, "profiles/traffic.json was taken with other kernel sources"
    if rec.get("shape") != SHAPE:
        return None, "profiles/traffic.json was taken at another shape"
    total = 0.0
    for sub in kernel_substrings:
        hit = [v for k, v in rec["kernels"].items() if sub in k and "float" in k]
        if len(hit) != 1:
            return None, f"profiles/traffic.json has {len(hit)} kernels matching {sub!r}"
        total += hit[0]["read_bytes"] + hit[0]["written_bytes"]
    return total, "profiles/traffic.json"


def cpu_baseline(B_sample: int):
    """Oracle forward+backward on a slice of the batch (same D, N, L)."""
    import torch
    from oracle import scan_oracle as O
    D, N, L = SHAPE["D"], SHAPE["N"], SHAPE["L"]
    cores = os.cpu_count() or 1
    threads = min(cores, 16)
    torch.set_num_threads(threads)
    p = O.make_core_inputs(B_sample, D, N, L, seed=0)
    times = []
    for run in range(4):                      # one warm-up run, three timed
        leaves = [p[k].clone().requires_grad_(True) for k in ("u", "delta", "theta", "Bc", "Cc", "Dskip")]
        t0 = time.perf_counter()
        y, _ = O.unitary_core_loop(*leaves)
        (y * p["dy"]).sum().backward()
        if run:
            times.append(time.perf_counter() - t0)
    dt = sorted(times)[1]
    return {
        "value": B_sample * D * L / dt,
        "unit": "(b,d,l) samples/s, forward+backward",
        "cores": threads,
        "kind": "port",
        "sample": f"B={B_sample} of {SHAPE['B']} batch elements at D={D} N={N} L={L}, one warm-up run then the median of "
                  f"three ({', '.join(f'{t:.1f}' for t in times)} s wall), torch {threads} threads on a host with "
                  f"{cores} cores",
    }


def hbm_probe(rows: int, L: int, dev) -> None:
    """Rates of aussm_hbm_probe over [rows, L] float tensors: three read and two written (the mix of a scan call), and
    read only, for a plain streaming kernel and for the scan kernels' pattern.  HIP events, median of 15 launches
    after 300 ms of load."""
    import torch
    from aussm_amd import scan
    lib = scan._lib.load()
    ptr, stream = scan.ptr, scan._stream()
    a, b, c = (torch.randn(rows, L, device=dev) for _ in range(3))
    o1, o2 = torch.empty_like(a), torch.empty_like(a)

    def launch(pattern, write):
        scan.check(lib.aussm_hbm_probe(ptr(a), ptr(b), ptr(c), ptr(o1), ptr(o2), rows, L, pattern, write, stream), "probe")
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < 0.3:
        launch(0, 1)
        torch.cuda.synchronize()
    out = {"probe": "o1 = a + b c, o2 = 2 o1 over [rows, L] float tensors", "rows": rows, "L": L, "unit": "GB/s",
           "hbm_peak": HBM_PEAK_GBS}
    for pattern, pname in ((0, "stream"), (1, "scan_pattern")):
        for write, wname in ((1, "3_read_2_written"), (0, "3_read")):
            ts = []
            for _ in range(15):
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                launch(pattern, write)
                e1.record()
                torch.cuda.synchronize()
                ts.append(e0.elapsed_time(e1) * 1e-3)
            nbytes = (5 if write else 3) * rows * L * 4
            out[f"{pname}_{wname}"] = round(nbytes / sorted(ts)[7] / 1e9, 1)
    launch(1, 1)
    torch.cuda.synchronize()
    want = a.double() + b.double() * c.double()          # (the kernel fuses the multiply and the add)
    assert (o1.double() - want).abs().max() < 1e-5 and (o2.double() - 2 * want).abs().max() < 2e-5, "probe kernel wrote something else"
    print(json.dumps(out))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--cpu-batch", type=int, default=8)
    ap.add_argument("--prewarm-ms", type=float, default=200.0, help="repeat the step for this long before the warm-up steps")
    ap.add_argument("--summarize-traffic", nargs=2, metavar=("FETCH_DIR", "WRITE_DIR"),
                    help="write profiles/traffic.json from the output of the two counter passes and exit")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also run one 256 MiB device-to-device copy (calibrates FETCH_SIZE / WRITE_SIZE under rocprofv3)")
    ap.add_argument("--shape", default=None, help="B,D,N,L instead of the headline shape (no recorded traffic figure then)")
    ap.add_argument("--hbm-probe", action="store_true",
                    help="instead of the benchmark: what the memory system delivers for a plain streaming kernel and for "
                         "the scan kernels' access pattern at this shape (aussm_hbm_probe), one JSON line")
    args = ap.parse_args()
    headline = args.shape is None
    if not headline:
        SHAPE.update(zip("BDNL", (int(v) for v in args.shape.split(","))))
    if args.summarize_traffic:
        summarize_traffic(*args.summarize_traffic)
        return
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU; --gpus must be 1 (no multi-GPU path exists)", file=sys.stderr)
        sys.exit(2)

    import torch
    from aussm_amd import scan

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    B, D, N, L = SHAPE["B"], SHAPE["D"], SHAPE["N"], SHAPE["L"]
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if args.hbm_probe:
        hbm_probe(B * D, L, dev)
        return
    # synthetic inputs with the benchmark contract's value distributions, generated on the device (the CPU oracle is only
    # used by the cpu_baseline leg): u ~ N(0,1), delta = softplus(N(0,1)), theta ~ N(0, 0.5), B_t and C_t complex
    # with parts ~ N(0, 1/sqrt(N)), D ~ N(0,1), dy ~ N(0,1)
    g = torch.Generator(device=dev).manual_seed(0)
    rn = lambda *shape: torch.randn(*shape, generator=g, device=dev)
    p = {"u": rn(B, D, L), "delta": torch.nn.functional.softplus(rn(B, D, L)), "theta": rn(B, D, L) * 0.5,
         "Bc": torch.complex(rn(B, N, L), rn(B, N, L)) * N ** -0.5, "Cc": torch.complex(rn(B, N, L), rn(B, N, L)) * N ** -0.5,
         "Dskip": rn(D), "dy": rn(B, D, L)}
    Bri = torch.view_as_real(p["Bc"]).contiguous()
    Cri = torch.view_as_real(p["Cc"]).contiguous()
    ck = scan.unitary_ck(B, D, N, L)                       # what the autograd wrapper uses for this shape

    aux = scan.unitary_aux(p["u"], N, ck)                    # what the autograd wrapper hands from forward to backward

    def step():
        y, _, hck = scan.unitary_fwd_raw(p["u"], p["delta"], p["theta"], Bri, Cri, p["Dskip"], None, None,
                                         want_state=False, ck=ck, aux=aux)
        return scan.unitary_bwd_raw(p["dy"], None, p["u"], p["delta"], p["theta"], Bri, Cri, p["Dskip"], hck, ck,
                                    aux=aux)

    t_pre = time.perf_counter()
    while (time.perf_counter() - t_pre) * 1e3 < args.prewarm_ms:
        step()
        torch.cuda.synchronize()
    prewarm_ms = (time.perf_counter() - t_pre) * 1e3
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / args.steps

    # ---- per-kernel durations with HIP events on the launch stream (torch's current stream)
    lib = scan._lib.load()
    ptr, stream = scan.ptr, scan._stream()
    f32 = dict(device=dev, dtype=torch.float32)
    y = torch.empty((B, D, L), **f32)
    hck = torch.empty((B, scan.num_checkpoints(L, ck), N, 2, D), **f32)
    du, ddl, dth = (torch.empty((B, D, L), **f32) for _ in range(3))
    dB, dC, dD = torch.zeros((B, N, L, 2), **f32), torch.zeros((B, N, L, 2), **f32), torch.zeros((D,), **f32)

    def fwd_only():
        scan.check(lib.aussm_unitary_fwd_aux(ptr(p["u"]), ptr(p["delta"]), ptr(p["theta"]), ptr(Bri), ptr(Cri),
                                             ptr(p["Dskip"]), None, None, ptr(y), None, ptr(hck), ptr(aux),
                                             B, D, N, L, ck, 0, 1, stream), "fwd")

    def bwd_only():
        scan.check(lib.aussm_unitary_bwd_aux(ptr(p["dy"]), None, ptr(p["u"]), ptr(p["delta"]), ptr(p["theta"]), ptr(Bri),
                                             ptr(Cri), ptr(p["Dskip"]), ptr(hck), ptr(aux), ptr(du), ptr(ddl), ptr(dth),
                                             ptr(dB), ptr(dC), ptr(dD), None, B, D, N, L, ck, 0, 1, stream), "bwd")

    def kernel_us(fn, reps):
        evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(reps)]
        fn()
        torch.cuda.synchronize()
        for s, e in evs:
            s.record()
            fn()
            e.record()
        torch.cuda.synchronize()
        return sum(s.elapsed_time(e) for s, e in evs) / reps * 1e3

    if args.copy_probe:
        src = torch.empty(64 * 1024 * 1024, **f32).normal_()
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    reps = max(10, min(args.steps, 50))
    t_fwd = kernel_us(fwd_only, reps)
    t_bwd = kernel_us(bwd_only, reps)
    E, S = B * D * L, B * N * L
    bytes_fwd = 16 * E + 16 * S + 4 * D
    bytes_bwd = 28 * E + 32 * S + 4 * D
    ach = bytes_bwd / (t_bwd * 1e-6) / 1e9
    # which kernels these calls ran, and what the counter passes recorded for them
    fmode = lib.aussm_unitary_kernel_mode(0, B, D, N, L, ck, 0, 1, 1)
    bmode = lib.aussm_unitary_kernel_mode(1, B, D, N, L, ck, 0, 1, 1)
    traffic_fwd, note_fwd = recorded_traffic(FWD_KERNELS[fmode])
    traffic_bwd, note_bwd = recorded_traffic(BWD_KERNELS[bmode])

    out = {
        "metric": f"unitary scan fwd+bwd elements/s + achieved HBM GB/s (% peak), B{B} D{D} N{N} L{L}",
        "value": B * D * L / dt,
        "unit": "(b,d,l) samples/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "prewarm_ms": prewarm_ms,
        "ms_per_step": dt * 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": (f"unitary core scan fwd+bwd, B={B} D={D} N={N} L={L}, fp32"
                                + (" (BASELINE configs[3], unitary, fp32)" if headline else "")),
                   "B": B, "D": D, "N": N, "L": L, "checkpoint_interval": ck},
        "state_updates_per_s": B * D * N * L / dt,
        "fwd_bwd_algorithmic_GBps": (bytes_fwd + bytes_bwd) / ((t_fwd + t_bwd) * 1e-6) / 1e9,
        "fwd_bwd_frac_of_hbm_peak": (bytes_fwd + bytes_bwd) / ((t_fwd + t_bwd) * 1e-6) / 1e9 / HBM_PEAK_GBS,
        "kernels_us": {"unitary_fwd": t_fwd, "unitary_bwd": t_bwd},
        "roofline": {"bound": "hbm", "kernel": BWD_KERNELS[bmode][0] + " (one backward call)",
                     "achieved": ach, "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": ach / HBM_PEAK_GBS, "traffic": traffic_bwd, "traffic_source": note_bwd,
                     "algorithmic_bytes": bytes_bwd,
                     "fwd_kernel": {"kernel": " + ".join(FWD_KERNELS[fmode]) + " (one forward call)",
                                    "achieved": bytes_fwd / (t_fwd * 1e-6) / 1e9,
                                    "frac": bytes_fwd / (t_fwd * 1e-6) / 1e9 / HBM_PEAK_GBS,
                                    "traffic": traffic_fwd, "traffic_source": note_fwd,
                                    "algorithmic_bytes": bytes_fwd}},
    }
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(min(args.cpu_batch, B))
    print(json.dumps(out))


if __name__ == "__main__":
    main()
