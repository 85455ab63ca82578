"""The benchmark contract's tolerance applied literally: assert_close(atol=1e-4, rtol=1e-4) of the HIP
outputs against the float64 oracle, element by element and without normalising by the tensor's scale,
for configurations 1, 2 (a slice of the channels) and 3 (two batch elements of the headline shape),
all three variants, float32.

Where the literal bound cannot hold element-wise - at L = 2048 outputs reach |y| ~ 60 and the float32
sequential-loop oracle is itself more than 1e-4 away from the float64 one on some elements - the test
asserts instead that the HIP result is no further from float64 than 1.5 times the float32 oracle is
(largest absolute error), and it prints the measured largest absolute and relative errors of both and
the number of elements outside the literal bound, which is where the published figures come
from.  The fused operator gets the same treatment at its benchmark shape on a two-batch slice, directly
against the loop oracle of the operator (factor 2: its phases are sums over 256 channels before they are
sums over time, and its outputs reach |y| ~ 250 there)."""
import pytest
import torch

from oracle import scan_oracle as O

pytestmark = pytest.mark.gpu

ATOL = RTOL = 1e-4


def _to64(p):
    return {k: (v.to(torch.complex128) if v.is_complex() else v.double()) for k, v in p.items()}


def _report(what, got, ref32, ref64, factor=1.5):
    """got, ref32: float32 results (HIP, float32 oracle); ref64: the float64 oracle.  Literal bound if it
    holds; else the 1.5x bound relative to the float32 oracle's own error.  Returns the printed record."""
    got, ref32, ref64 = got.double().cpu(), ref32.double(), ref64.double()
    bound = ATOL + RTOL * ref64.abs()
    eh, eo = (got - ref64).abs(), (ref32 - ref64).abs()
    rel = lambda e: float((e / ref64.abs().clamp_min(1e-30))[ref64.abs() > 1e-3].max())
    vh, vo = int((eh > bound).sum()), int((eo > bound).sum())
    literal = vh == 0
    print(f"tolerance {what}: max|ref| {float(ref64.abs().max()):.3g}  HIP max abs {float(eh.max()):.3e} max rel {rel(eh):.3e} "
          f"outside 1e-4/1e-4: {vh} of {eh.numel()}  |  float32 oracle max abs {float(eo.max()):.3e} max rel {rel(eo):.3e} "
          f"outside: {vo}  ->  {'literal bound holds' if literal else 'bound relative to the float32 oracle'}", flush=True)
    if literal:
        torch.testing.assert_close(got.float(), ref64.float(), atol=ATOL, rtol=RTOL)
        return
    assert float(eh.max()) <= factor * float(eo.max()) + 1e-7, \
        f"{what}: HIP error {float(eh.max()):.3e} vs float32 oracle {float(eo.max()):.3e}"


CASES = [
    ("config 1", 16, 128, 16, 1024, None),
    ("config 2, 16 channels", 4, 16, 16, 16384, None),
    ("config 3, 2 batch elements", 2, 512, 16, 2048, None),
]


@pytest.mark.parametrize("name,B,D,N,L,_", CASES)
@pytest.mark.parametrize("variant", ["unitary", "complex", "real"])
def test_forward_outputs_literal_tolerance(name, B, D, N, L, _, variant):
    from aussm_amd import scan
    p = O.make_core_inputs(B, D, N, L, seed=11, variant=variant)
    p64 = _to64(p)
    q = {k: v.cuda() for k, v in p.items()}
    print(f"case literal tolerance {variant} {name}", flush=True)
    if variant == "unitary":
        args = ("u", "delta", "theta", "Bc", "Cc", "Dskip")
        loop = O.unitary_core_loop
        y, hL = scan.unitary_scan(*[q[k] for k in args], return_last_state=True)
    elif variant == "complex":
        args = ("u", "delta", "rho", "theta", "Bc", "Cc", "Dskip")
        loop = O.complex_core_loop
        y, hL = scan.complex_scan(*[q[k] for k in args], return_last_state=True)
    else:
        args = ("u", "delta", "A", "Bm", "Cm", "Dskip")
        loop = O.real_core_loop
        y, hL = scan.selective_scan_fn(*[q[k] for k in args], return_last_state=True)
    y32, h32 = loop(*[p[k] for k in args])
    y64, h64 = loop(*[p64[k] for k in args])
    _report(f"{variant} {name} y", y, y32, y64)
    real = lambda t: torch.view_as_real(t) if t.is_complex() else t
    _report(f"{variant} {name} hL", real(hL), real(h32), real(h64))


def test_fused_operator_at_its_benchmark_shape_against_the_loop_oracle():
    """Two batch elements of b=32 d=256 n=16 L=720 (the operator shape of the hybrid model benchmark): the three
    outputs against adaptive_unitary_op_loop in float64, and all twelve gradients against its autograd
    (gradients normalised by the oracle gradient's largest magnitude, as everywhere)."""
    import aussm_amd.ops  # noqa: F401  (registers the operators)
    b, d, n, L = 2, 256, 16, 720
    g = torch.Generator().manual_seed(4)
    rn = lambda *s: torch.randn(*s, generator=g)
    t = {"u": rn(b, d, L), "dt": torch.nn.functional.softplus(rn(b, d, L)), "x": rn(d, n, d) * d ** -0.5,
         "x_bias": (torch.rand(d, n, generator=g) * 2 - 1) * 3.14159, "B_r": torch.nn.functional.softplus(rn(n)),
         "B_theta": rn(n), "C_r": torch.nn.functional.softplus(rn(n)), "C_theta": rn(n), "D": rn(d), "z": rn(b, d, L),
         "h_re": rn(b, d, n), "h_im": rn(b, d, n)}
    names = list(t)
    gy, gr, gi = rn(b, d, L), rn(b, d, n), rn(b, d, n)
    print("case literal tolerance fused operator b=2 d=256 n=16 L=720", flush=True)

    def run(fn, dev, dtype):
        lv = [t[k].to(dtype).clone().to(dev).requires_grad_(True) for k in names]
        y, hr, hi = fn(*lv)
        ((y * gy.to(dev).to(dtype)).sum() + (hr * gr.to(dev).to(dtype)).sum() + (hi * gi.to(dev).to(dtype)).sum()).backward()
        return [o.detach().cpu() for o in (y, hr, hi)], [v.grad.cpu() for v in lv]

    out64, g64 = run(O.adaptive_unitary_op_loop, "cpu", torch.float64)
    out32, _ = run(O.adaptive_unitary_op_loop, "cpu", torch.float32)
    outg, gg = run(torch.ops.extension_cpp.ssm_adaptive_unitary, "cuda", torch.float32)
    for k, a, b32, c in zip(("y", "next_hid_real", "next_hid_imag"), outg, out32, out64):
        _report(f"fused operator {k}", a, b32, c, factor=2.0)
    for k, a, c in zip(names, gg, g64):
        scale = max(1.0, float(c.abs().max()))
        torch.testing.assert_close(a.double() / scale, c / scale, atol=ATOL, rtol=RTOL, msg=lambda m: f"grad {k}: {m}")
