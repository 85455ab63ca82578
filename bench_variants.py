#!/usr/bin/env python3
"""The three scan variants at the headline shape (B=32 D=512 N=16 L=2048), forward and backward,
once with float32 inputs and once with bfloat16 u / delta / B / C (float32 phases, decay, skip,
states, outputs and gradients): configuration 3 of the benchmark contract.

    python bench_variants.py [--reps R] [--shape B,D,N,L] [--variants real,...] [--gate] [--model | --only-model]
    python bench_variants.py --scaling [--runs 50] [--bdn 16,32,64 --bdn 32,256,16] [--lengths 10,...]

With --model it also times configuration 4 of the contract: one training step (forward, MSE loss,
backward) of SSMTS(d_model=256, input_dim=21, output_dim=21, layers="a|m|a|m") on x ~ N(0,1) of
shape (32, 720, 21), random-init weights, wall clock around synchronised steps.

With --scaling it runs the protocol of the reference's sweep, extension-cpp/test/scaling_benchmark.py:99-189,
instead: for each system and each sequence length (20 log-spaced points in [10, 2048] as there, plus
4096 and 16384), 5 warm-up and --runs timed repetitions of the operator's forward pass and of
`y.sum().backward()`, device time of each (HIP events on the launch stream) and peak device memory after
each (torch.cuda.max_memory_allocated, reset before every repetition; `inputs_MB` is what was allocated at
that moment, i.e. the point's inputs).  Systems (the reference's are
"mamba", "SSMau-cuda", "SSMau-pytorch", :193-216): "SSMau-hip" = ssm_adaptive_interface on the fused
kernels, "SSMau-hip-composite" = the same interface on the composite route (phase tensor materialised),
"mamba-hip" = selective_scan_fn.  Shapes: the reference's default b=16, d=32, n=64 (:259-262) and the training
configuration's b=32, d=256, n=16.  One JSON line per (system, shape, length).

Prints one JSON line per (variant, input dtype): the duration of the forward and of the backward
call (HIP events on the launch stream, mean of R launches after a warm-up long enough for the
clocks to settle) and the algorithmic bytes over that duration against the 8 TB/s HBM peak.
`bench.py` stays the contract line (unitary, float32); this script is the table beside it.

Algorithmic bytes (E = B*D*L, S = B*N*L, w = bytes of an input element: 4 or 2):
  unitary  forward  2wE + 8E  + 4wS       backward 2wE + 20E + 4wS + 16S
  complex  forward  2wE + 12E + 4wS       backward 2wE + 28E + 4wS + 16S
  real     forward  2wE + 4E  + 2wS       backward 2wE + 12E + 2wS + 8S
(reads of u, delta in w bytes; theta / rho / dy and all outputs in float32; B, C complex = two
elements, real = one; gradients of B, C in float32).
"""
from __future__ import annotations

import argparse
import json
import time
import os
import sys

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0


def algorithmic_bytes(variant: str, w: int, E: int, S: int):
    if variant == "unitary":
        return 2 * w * E + 8 * E + 4 * w * S, 2 * w * E + 20 * E + 4 * w * S + 16 * S
    if variant == "complex":
        return 2 * w * E + 12 * E + 4 * w * S, 2 * w * E + 28 * E + 4 * w * S + 16 * S
    return 2 * w * E + 4 * E + 2 * w * S, 2 * w * E + 12 * E + 2 * w * S + 8 * S


def scaling(args):
    """The sweep of extension-cpp/test/scaling_benchmark.py:99-189 on this package's operators."""
    import numpy as np
    import torch
    from aussm_amd import ops, scan
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    lengths = ([int(v) for v in args.lengths.split(",")] if args.lengths else
               [int(v) for v in np.logspace(np.log10(10), np.log10(2048), 20)] + [4096, 16384])
    shapes = [tuple(int(v) for v in s.split(",")) for s in (args.bdn or ["16,32,64", "32,256,16"])]
    systems = args.systems.split(",")
    def point(system, b, d, n, l):
        """One (system, shape, length) point; its tensors die with this frame."""
        g = torch.Generator(device=dev).manual_seed(0)
        rn = lambda *s: torch.randn(*s, generator=g, device=dev)
        leaf = lambda t: t.requires_grad_(True)
        u, dt, z, D = leaf(rn(b, d, l)), leaf(rn(b, d, l)), leaf(rn(b, d, l)), leaf(rn(d))
        if system == "mamba-hip":
            A, Bm, Cm = leaf(-torch.exp(rn(d, n))), leaf(rn(b, n, l)), leaf(rn(b, n, l))
            params = [u, dt, A, Bm, Cm, D, z]
            fn = lambda: scan.selective_scan_fn(u, dt, A, Bm, Cm, D, z=z, delta_softplus=True)
        else:
            x, xb = leaf(rn(d, n, d) * d ** -0.5), leaf(rn(d, n))
            Bp, Cp = leaf(torch.complex(rn(n), rn(n))), leaf(torch.complex(rn(n), rn(n)))
            params = [u, dt, x, xb, Bp, Cp, D, z]
            save = system == "SSMau-hip-composite"
            fn = lambda: ops.ssm_adaptive_interface(u, dt, x, xb, Bp, Cp, D, z, unitary=True, save_intermediates=save)
        tf = tb = mf = mb = 0.0
        ev = lambda: torch.cuda.Event(enable_timing=True)
        for run in range(args.runs + 5):
            for t in params:
                t.grad = None
            torch.cuda.synchronize()
            torch.cuda.reset_peak_memory_stats()
            base = torch.cuda.memory_allocated()          # the inputs (and nothing else of this point)
            e0, e1, e2 = ev(), ev(), ev()
            e0.record()
            y = fn()
            e1.record()
            mem_f = torch.cuda.max_memory_allocated()
            y.sum().backward()
            e2.record()
            torch.cuda.synchronize()
            if run >= 5:
                tf += e0.elapsed_time(e1)
                tb += e1.elapsed_time(e2)
                mf += mem_f
                mb += torch.cuda.max_memory_allocated()
            del y
        r = args.runs
        return {"system": system, "b": b, "d": d, "n": n, "L": l, "runs": r,
                "fwd_us": round(tf / r * 1e3, 1), "bwd_us": round(tb / r * 1e3, 1),
                "inputs_MB": round(base * 1e-6, 2),
                "fwd_peak_MB": round(mf / r * 1e-6, 2), "bwd_peak_MB": round(mb / r * 1e-6, 2)}

    import gc
    import time
    # the clocks of the part ramp up over tens of milliseconds of load: the first points would read slow
    warm = torch.randn(4096, 4096, device=dev)
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < 0.3:
        warm = torch.mm(warm, warm).clamp_(-1, 1)
        torch.cuda.synchronize()
    del warm
    for b, d, n in shapes:
        for system in systems:
            # one-off costs of a system's first use (code objects of its backward kernels loaded on first launch, the
            # autograd engine's thread, first allocations) stay out of the timed repetitions of its first point
            try:
                point(system, b, d, n, lengths[0])
            except RuntimeError:
                pass
            for l in lengths:
                try:
                    rec = point(system, b, d, n, l)
                except RuntimeError as e:               # out of memory, or a shape an operator does not take
                    rec = {"system": system, "b": b, "d": d, "n": n, "L": l, "error": str(e).split("\n")[0][:160]}
                print(json.dumps(rec), flush=True)
                gc.collect()
                torch.cuda.empty_cache()


def fused_operator(args):
    """Forward and backward operator calls at one shape, HIP events, with the roofline that bounds them: the phase
    projection theta[b,i,j,l] = x[i,j,:] . u[b,:,l] and, backward, the two products with the phase adjoints
    (grad_x, grad_u) are matrix work, 2 b d^2 n L flops each in fp32 terms; the kernels run every product as six
    bf16 products on exactly split operands, so the fp32-equivalent rate is held against the fp32 matrix peak and the
    bf16 rate (six times the flops) against the bf16 one."""
    import torch
    import aussm_amd.ops  # noqa: F401
    b, d, n, L = (int(v) for v in args.fused.split(","))
    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev).manual_seed(0)
    rn = lambda *s: torch.randn(*s, generator=g, device=dev)
    sp = torch.nn.functional.softplus
    t = [rn(b, d, L), sp(rn(b, d, L)), rn(d, n, d) * d ** -0.5, rn(d, n), sp(rn(n)), rn(n), sp(rn(n)), rn(n), rn(d),
         rn(b, d, L), rn(b, d, n), rn(b, d, n)]
    grads = [rn(b, d, L), rn(b, d, n), rn(b, d, n)]
    fwd = lambda: torch.ops.extension_cpp.ssm_adaptive_unitary(*t)
    nh = list(fwd()[1:])
    bwd = lambda: torch.ops.aussm_amd.ssm_adaptive_backward_unitary_from_state(*grads, *t, *nh)

    def timed(fn):
        t0 = time.perf_counter()
        while time.perf_counter() - t0 < 0.2:
            fn()
            torch.cuda.synchronize()
        evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.reps)]
        for s_, e_ in evs:
            s_.record()
            fn()
            e_.record()
        torch.cuda.synchronize()
        return sum(s_.elapsed_time(e_) for s_, e_ in evs) / args.reps * 1e3
    t_f, t_b = timed(fwd), timed(bwd)
    unit = 2.0 * b * d * d * n * L

    def roof(flops, us):
        tf = flops / us / 1e6
        return {"bound": "mfma", "achieved": round(tf, 1), "peak": 157.3, "unit": "TFLOP/s (fp32-equivalent)",
                "frac": round(tf / 157.3, 4), "flops": flops,
                "as_bf16_products": {"achieved": round(6 * tf, 1), "peak": 2500.0, "unit": "TFLOP/s", "frac": round(6 * tf / 2500.0, 4)}}
    E = b * d * L
    print(json.dumps({
        "operator": "extension_cpp::ssm_adaptive_unitary (fused kernels)", "shape": {"b": b, "d": d, "n": n, "L": L},
        "fwd_us": round(t_f, 1), "bwd_us": round(t_b, 1), "bwd_over_fwd": round(t_b / t_f, 2),
        "roofline_fwd": roof(unit, t_f), "roofline_bwd": roof(3 * unit, t_b),
        "algorithmic_bytes": {"fwd": 16 * E + 4 * d * n * d, "bwd": 32 * E + 8 * d * n * d},
        "note": "backward flops: the phase projection again (the operator recomputes from its inputs) and the two products "
                "with the phase adjoints; durations include output allocation and the workspace"}), flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--reps", type=int, default=30)
    ap.add_argument("--shape", default="32,512,16,2048")
    ap.add_argument("--model", action="store_true", help="also time the hybrid SSMTS training step (configuration 4)")
    ap.add_argument("--only-model", action="store_true", help="time only the SSMTS training step")
    ap.add_argument("--variants", default="unitary,complex,real", help="comma-separated subset of the variants")
    ap.add_argument("--gate", action="store_true",
                    help="time the complex and real scans with the gate z (y = y_pre silu(z), dz returned); the unitary core "
                         "scan has no gate inside its kernels")
    ap.add_argument("--scaling", action="store_true", help="the sequence-length sweep of the reference's scaling benchmark")
    ap.add_argument("--runs", type=int, default=50, help="timed repetitions per point of the sweep (after 5 warm-ups)")
    ap.add_argument("--bdn", action="append", help="b,d,n of the sweep (repeatable)")
    ap.add_argument("--lengths", default=None, help="comma-separated sequence lengths of the sweep")
    ap.add_argument("--systems", default="SSMau-hip,SSMau-hip-composite,mamba-hip")
    ap.add_argument("--fused", default=None, metavar="b,d,n,L", nargs="?", const="32,256,16,720",
                    help="time the fused operator (extension_cpp::ssm_adaptive_unitary and its backward operator) at a shape, "
                         "default: the hybrid model benchmark's operator shape, with its matrix-pipe roofline")
    args = ap.parse_args()
    B, D, N, L = (int(v) for v in args.shape.split(","))

    import torch
    from aussm_amd import scan

    if not torch.cuda.is_available():
        print("bench_variants.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if args.scaling:
        scaling(args)
        return
    if args.fused:
        fused_operator(args)
        return

    def timed(fn):
        for _ in range(40):
            fn()
        torch.cuda.synchronize()
        evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.reps)]
        for s, e in evs:
            s.record()
            fn()
            e.record()
        torch.cuda.synchronize()
        return sum(s.elapsed_time(e) for s, e in evs) / args.reps * 1e3

    def inputs(variant):
        """The contract's value distributions: u ~ N(0,1), delta = softplus(N(0,1)), theta ~ N(0, 0.5),
        B, C ~ N(0, 1/sqrt(N)) per part, D ~ N(0,1), A = -exp(N(0,1)), rho = -delta exp(N(0,1))[d]."""
        g = torch.Generator(device=dev).manual_seed(0)
        rn = lambda *s: torch.randn(*s, generator=g, device=dev)
        std = N ** -0.5
        out = {"u": rn(B, D, L), "delta": torch.nn.functional.softplus(rn(B, D, L)), "Dskip": rn(D), "dy": rn(B, D, L)}
        out["z"] = rn(B, D, L) if (args.gate and variant != "unitary") else None
        if variant == "real":
            out.update(A=-torch.exp(rn(D, N)), Bm=rn(B, N, L) * std, Cm=rn(B, N, L) * std)
        else:
            out.update(theta=rn(B, D, L) * 0.5, Bc=torch.complex(rn(B, N, L) * std, rn(B, N, L) * std),
                       Cc=torch.complex(rn(B, N, L) * std, rn(B, N, L) * std))
            if variant == "complex":
                out["rho"] = -out["delta"] * torch.exp(rn(D))[None, :, None]
        return out

    E, S = B * D * L, B * N * L
    for variant in (() if args.only_model else tuple(args.variants.split(","))):
        base = inputs(variant)
        for name, dt, w in (("f32", torch.float32, 4), ("bf16", torch.bfloat16, 2)):
            p = dict(base)
            u, delta = p["u"].to(dt), p["delta"].to(dt)
            if variant == "real":
                Bm, Cm = p["Bm"].to(dt).contiguous(), p["Cm"].to(dt).contiguous()
                ck = scan.REC_CK

                def fwd():
                    return scan.real_fwd_raw(u, delta, p["A"], Bm, Cm, p["Dskip"], z=p["z"], ck=ck)

                hck = fwd()[2]

                def bwd():
                    return scan.real_bwd_raw(p["dy"], None, u, delta, p["A"], Bm, Cm, p["Dskip"], None, False, None, hck,
                                             z=p["z"])
            else:
                Bri = torch.view_as_real(p["Bc"]).to(dt).contiguous()
                Cri = torch.view_as_real(p["Cc"]).to(dt).contiguous()
                if variant == "unitary":
                    ck = scan.unitary_ck(B, D, N, L)
                    aux = scan.unitary_aux(u, N, ck)

                    def fwd():
                        return scan.unitary_fwd_raw(u, delta, p["theta"], Bri, Cri, p["Dskip"], ck=ck, aux=aux)

                    hck = fwd()[2]

                    def bwd():
                        return scan.unitary_bwd_raw(p["dy"], None, u, delta, p["theta"], Bri, Cri, p["Dskip"], hck, ck,
                                                    aux=aux)
                else:
                    ck = scan.REC_CK

                    def fwd():
                        return scan.complex_fwd_raw(u, delta, p["rho"], p["theta"], Bri, Cri, p["Dskip"], z=p["z"], ck=ck)

                    hck = fwd()[2]

                    def bwd():
                        return scan.complex_bwd_raw(p["dy"], None, u, delta, p["rho"], p["theta"], Bri, Cri, p["Dskip"],
                                                    None, hck, z=p["z"])
            t_f, t_b = timed(fwd), timed(bwd)
            b_f, b_b = algorithmic_bytes(variant, w, E, S)
            gated = p["z"] is not None
            if gated:                      # z read forward; z read and dz written backward
                b_f, b_b = b_f + 4 * E, b_b + 8 * E
            print(json.dumps({
                "variant": variant + (" (gated)" if gated else ""), "inputs": name, "shape": {"B": B, "D": D, "N": N, "L": L},
                "fwd_us": round(t_f, 1), "bwd_us": round(t_b, 1),
                "fwd_GBps": round(b_f / t_f / 1e3, 1), "bwd_GBps": round(b_b / t_b / 1e3, 1),
                "fwd_bwd_frac_of_hbm_peak": round((b_f + b_b) / (t_f + t_b) / 1e3 / HBM_PEAK_GBS, 4),
                "samples_per_s": round(E / ((t_f + t_b) * 1e-6), 1),
                "note": "durations include the output allocation and the zero-fill of the accumulated gradients",
            }), flush=True)

    if args.model or args.only_model:
        import time
        from aussm_amd import blocks
        torch.manual_seed(0)
        net = blocks.SSMTS(d_model=256, input_dim=21, output_dim=21, layers="a|m|a|m").to(dev)
        x = torch.randn(32, 720, 21, device=dev)
        tgt = torch.randn(32, 720, 21, device=dev)

        def step():
            net.zero_grad(set_to_none=True)
            loss = ((net(x) - tgt) ** 2).mean()
            loss.backward()

        for _ in range(5):
            step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(20):
            step()
        torch.cuda.synchronize()
        dt = (time.perf_counter() - t0) / 20
        print(json.dumps({"model": "SSMTS d_model=256 layers=a|m|a|m, x (32, 720, 21), fp32, forward + MSE + backward",
                          "ms_per_step": round(dt * 1e3, 2), "sequences_per_s": round(32 / dt, 1)}), flush=True)


if __name__ == "__main__":
    main()
