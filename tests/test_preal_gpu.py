"""The positive-real adaptive scan of the reference's pure-PyTorch file (extension-cpp/extension_cpp/ops.py:300-357
and :465-510) on the HIP scan kernels, against the float64 oracle: outputs and all gradients,
atol = rtol = 1e-4 of each tensor's largest magnitude.  Upstream the form has no reachable kernel and no test."""
import pytest
import torch
import torch.nn.functional as F

from oracle import scan_oracle as O

pytestmark = pytest.mark.gpu


def _inputs(b, d, n, l, seed):
    g = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64)
    # (the form is unstable where the contracted decay is positive - exp of its running sum overflows float32, here as
    # upstream: the weights are scaled so that it stays moderate over the test lengths)
    return dict(u=r(b, d, l), dt=F.softplus(r(b, d, l)), x=r(d, n, d) * (0.25 / d ** 0.5), xb=r(d, n) * 0.2 - 1.0,
                B=r(b, n, l), C=r(b, n, l), D=r(d), z=r(b, d, l))


def _close(got, want, what):
    scale = max(1e-3, float(want.abs().max()))
    torch.testing.assert_close(got.double().cpu() / scale, want / scale, atol=1e-4, rtol=1e-4, msg=lambda m: f"{what}: {m}")


@pytest.mark.parametrize("b,d,n,l", [(2, 8, 4, 64), (1, 20, 16, 130), (2, 5, 3, 37), (1, 16, 16, 300)])
@pytest.mark.parametrize("step_scaled", [False, True])
def test_preal_forward_and_gradients(b, d, n, l, step_scaled):
    from aussm_amd import ops
    p = _inputs(b, d, n, l, seed=b + d + n + l)
    names = ("u", "dt", "x", "xb", "B", "C", "D", "z") if step_scaled else ("u", "dt", "x", "B", "C", "D", "z")
    print(f"case preal step_scaled={step_scaled} b={b} d={d} n={n} l={l}", flush=True)
    g = torch.Generator().manual_seed(1)
    dy = torch.randn(b, d, l, generator=g, dtype=torch.float64)

    def run(fn, dev, dtype):
        lv = [p[k].to(dtype).clone().to(dev).requires_grad_(True) for k in names]
        y = fn(*lv)
        (y * dy.to(dev).to(dtype)).sum().backward()
        return y.detach(), [t.grad for t in lv]

    if step_scaled:
        oracle = lambda u, dt, x, xb, B, C, D, z: O.adaptive_preal_loop(u, dt, x, B, C, D, z, x_bias=xb, step_scaled=True)
        fn = ops.reference_ssm_adaptive_preal_optimized
    else:
        oracle = O.adaptive_preal_loop
        fn = ops.reference_ssm_adaptive_preal
    want, gw = run(oracle, "cpu", torch.float64)
    got, gg = run(fn, "cuda", torch.float32)
    _close(got, want, "y")
    for k, a, c in zip(names, gg, gw):
        _close(a, c, f"d{k}")


def test_preal_rejects_cpu_tensors():
    from aussm_amd import ops
    p = {k: v.float() for k, v in _inputs(1, 4, 2, 8, seed=0).items()}
    with pytest.raises(RuntimeError):
        ops.reference_ssm_adaptive_preal(p["u"], p["dt"], p["x"], p["B"], p["C"], p["D"], p["z"])
