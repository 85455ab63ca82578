"""Writes the small fixtures in this directory from the CPU oracle (float64, stored as float32).

    python tests/golden/make_fixtures.py

The reference ships no golden vectors for the scan path; these are regression fixtures of the
build's own oracle, which is pinned independently in tests/test_oracle.py.  adaptive_seed10 follows
the reference test's input recipe (extension-cpp/test/test_extension.py:31-70)."""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import scan_oracle as O  # noqa: E402


def ri(t):
    return torch.view_as_real(t).numpy() if t.is_complex() else t.numpy()


def main():
    out = {}
    for variant in ("unitary", "complex", "real"):
        p = O.make_core_inputs(2, 6, 4, 40, seed=11, variant=variant, dtype=torch.float64, gate=True)
        if variant == "unitary":
            y, h = O.unitary_core_loop(p["u"], p["delta"], p["theta"], p["Bc"], p["Cc"], p["Dskip"], p["z"])
        elif variant == "complex":
            y, h = O.complex_core_loop(p["u"], p["delta"], p["rho"], p["theta"], p["Bc"], p["Cc"], p["Dskip"], p["z"])
        else:
            y, h = O.real_core_loop(p["u"], p["delta"], p["A"], p["Bm"], p["Cm"], p["Dskip"], p["z"])
        for k, v in p.items():
            out[f"{variant}_{k}"] = ri(v).astype(np.float32)
        out[f"{variant}_y"] = y.numpy().astype(np.float32)
        out[f"{variant}_hL"] = ri(h).astype(np.float32)
    args = O.make_adaptive_inputs(dtype=torch.float64)
    for k, v in zip(("u", "dt", "x", "x_bias", "B", "C", "D", "z"), args):
        out[f"adaptive_{k}"] = ri(v).astype(np.float32)
    out["adaptive_y"] = O.adaptive_unitary_polar(*args).numpy().astype(np.float32)
    # the blocks' depthwise causal convolution (ai-modules/wavesAI/model/aussm.py:762, :863) on (b, l, d)
    g = torch.Generator().manual_seed(21)
    cx = torch.randn(2, 9, 5, generator=g, dtype=torch.float64)
    cw = torch.randn(5, 1, 4, generator=g, dtype=torch.float64)
    cb = torch.randn(5, generator=g, dtype=torch.float64)
    out["conv_x"], out["conv_w"], out["conv_b"] = (v.numpy().astype(np.float32) for v in (cx, cw, cb))
    out["conv_y"] = O.causal_conv1d_bld(cx, cw, cb).numpy().astype(np.float32)
    np.savez_compressed(os.path.join(HERE, "scan_fixtures.npz"), **out)
    print("wrote", len(out), "arrays")


if __name__ == "__main__":
    main()
