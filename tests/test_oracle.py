"""Pins the CPU oracle: each check is independent of the oracle's own formulae
(scalar brute force with Python complex numbers, closed forms, invariants,
finite-difference gradcheck), so a dropped term, a wrong sign or a transposed
index fails at least one of them."""
import cmath
import math

import pytest
import torch
import torch.nn.functional as F

from oracle import scan_oracle as O

torch.manual_seed(0)


def _silu(v):
    return v / (1.0 + math.exp(-v))


def brute_core(u, delta, a_fn, Bc, Cc, Dskip, z, h0):
    """Scalar loops over (b, d, n, l) with Python complex arithmetic."""
    b, d, l = u.shape
    n = Bc.shape[1]
    y = torch.zeros(b, d, l, dtype=torch.float64)
    hL = torch.zeros(b, d, n, dtype=torch.complex128)
    for ib in range(b):
        for idd in range(d):
            h = [complex(h0[ib, idd, j]) if h0 is not None else 0j for j in range(n)]
            for t in range(l):
                acc = 0.0
                for j in range(n):
                    h[j] = a_fn(ib, idd, j, t) * h[j] + float(delta[ib, idd, t]) * complex(Bc[ib, j, t]) * float(u[ib, idd, t])
                    acc += (complex(Cc[ib, j, t]) * h[j]).real
                if Dskip is not None:
                    acc += float(Dskip[idd]) * float(u[ib, idd, t])
                if z is not None:
                    acc *= _silu(float(z[ib, idd, t]))
                y[ib, idd, t] = acc
            for j in range(n):
                hL[ib, idd, j] = h[j]
    return y, hL


def _inp(variant, gate=True, B=2, D=3, N=2, L=7, seed=1):
    return O.make_core_inputs(B, D, N, L, seed=seed, variant=variant, dtype=torch.float64, gate=gate)


def test_unitary_matches_bruteforce():
    p = _inp("unitary")
    h0 = torch.complex(torch.randn(2, 3, 2, dtype=torch.float64), torch.randn(2, 3, 2, dtype=torch.float64))
    y, hL = O.unitary_core_loop(p["u"], p["delta"], p["theta"], p["Bc"], p["Cc"], p["Dskip"], p["z"], h0)
    a = lambda ib, idd, j, t: cmath.exp(1j * float(p["theta"][ib, idd, t]))
    yb, hb = brute_core(p["u"], p["delta"], a, p["Bc"], p["Cc"], p["Dskip"], p["z"], h0)
    torch.testing.assert_close(y, yb, atol=1e-12, rtol=1e-12)
    torch.testing.assert_close(hL, hb, atol=1e-12, rtol=1e-12)


def test_complex_matches_bruteforce():
    p = _inp("complex")
    y, hL = O.complex_core_loop(p["u"], p["delta"], p["rho"], p["theta"], p["Bc"], p["Cc"], p["Dskip"], p["z"])
    a = lambda ib, idd, j, t: cmath.exp(complex(float(p["rho"][ib, idd, t]), float(p["theta"][ib, idd, t])))
    yb, hb = brute_core(p["u"], p["delta"], a, p["Bc"], p["Cc"], p["Dskip"], p["z"], None)
    torch.testing.assert_close(y, yb, atol=1e-12, rtol=1e-12)
    torch.testing.assert_close(hL, hb, atol=1e-12, rtol=1e-12)


def test_real_matches_bruteforce():
    p = _inp("real")
    bias = torch.randn(3, dtype=torch.float64)
    y, hL = O.real_core_loop(p["u"], p["delta"], p["A"], p["Bm"], p["Cm"], p["Dskip"], p["z"],
                             delta_bias=bias, delta_softplus=True)
    dl = torch.log1p(torch.exp(p["delta"] + bias[None, :, None]))
    a = lambda ib, idd, j, t: math.exp(float(dl[ib, idd, t]) * float(p["A"][idd, j]))
    yb, hb = brute_core(p["u"], dl, a, p["Bm"], p["Cm"], p["Dskip"], p["z"], None)
    torch.testing.assert_close(y, yb, atol=1e-12, rtol=1e-12)
    torch.testing.assert_close(hL, hb.real, atol=1e-12, rtol=1e-12)


def test_unitary_zero_phase_is_cumsum():
    p = _inp("unitary", gate=False, L=33)
    y, hL = O.unitary_core_loop(p["u"], p["delta"], torch.zeros_like(p["theta"]), p["Bc"], p["Cc"])
    w = (p["delta"] * p["u"])
    S = torch.cumsum(w[:, :, None, :] * p["Bc"][:, None, :, :], dim=-1)          # (b,d,n,l)
    torch.testing.assert_close(y, (S * p["Cc"][:, None]).sum(2).real, atol=1e-11, rtol=1e-11)
    torch.testing.assert_close(hL, S[..., -1], atol=1e-11, rtol=1e-11)


def test_unitary_constant_phase_geometric_series():
    # theta = phi, delta*u*B = beta constant  ->  h_l = beta (1 - e^{i phi l}) / (1 - e^{i phi})
    B, D, N, L = 1, 1, 1, 40
    phi, beta = 0.37, 0.8 - 0.3j
    u = torch.ones(B, D, L, dtype=torch.float64)
    Bc = torch.full((B, N, L), beta, dtype=torch.complex128)
    Cc = torch.ones(B, N, L, dtype=torch.complex128)
    y, hL = O.unitary_core_loop(u, u.clone(), torch.full_like(u, phi), Bc, Cc)
    for l in range(1, L + 1):
        h = beta * (1 - cmath.exp(1j * phi * l)) / (1 - cmath.exp(1j * phi))
        assert abs(float(y[0, 0, l - 1]) - h.real) < 1e-11
    assert abs(complex(hL[0, 0, 0]) - h) < 1e-11


def test_unitary_preserves_norm_without_input():
    p = _inp("unitary", gate=False, L=50)
    h0 = torch.complex(torch.randn(2, 3, 2, dtype=torch.float64), torch.randn(2, 3, 2, dtype=torch.float64))
    _, hL = O.unitary_core_loop(torch.zeros_like(p["u"]), p["delta"], p["theta"], p["Bc"], p["Cc"], h0=h0)
    torch.testing.assert_close(hL.abs(), h0.abs(), atol=1e-12, rtol=1e-12)
    G = p["theta"].sum(-1)
    torch.testing.assert_close(hL, h0 * torch.polar(torch.ones_like(G), G)[..., None], atol=1e-11, rtol=1e-11)


@pytest.mark.parametrize("variant", ["unitary", "complex", "real"])
def test_chunk_composition(variant):
    """scan[0:L1] then scan[L1:L] with the carried state == one scan; the
    property the reference's chunk loop relies on (ops.py:76-85)."""
    p = _inp(variant, L=21)
    L1 = 8
    if variant == "real":
        f = lambda sl, h0: O.real_core_loop(p["u"][..., sl], p["delta"][..., sl], p["A"], p["Bm"][..., sl],
                                            p["Cm"][..., sl], p["Dskip"], p["z"][..., sl], h0=h0)
    elif variant == "complex":
        f = lambda sl, h0: O.complex_core_loop(p["u"][..., sl], p["delta"][..., sl], p["rho"][..., sl],
                                               p["theta"][..., sl], p["Bc"][..., sl], p["Cc"][..., sl],
                                               p["Dskip"], p["z"][..., sl], h0=h0)
    else:
        f = lambda sl, h0: O.unitary_core_loop(p["u"][..., sl], p["delta"][..., sl], p["theta"][..., sl],
                                               p["Bc"][..., sl], p["Cc"][..., sl], p["Dskip"], p["z"][..., sl], h0=h0)
    y, hL = f(slice(0, 21), None)
    y1, h1 = f(slice(0, L1), None)
    y2, h2 = f(slice(L1, 21), h1)
    torch.testing.assert_close(torch.cat([y1, y2], -1), y, atol=1e-12, rtol=1e-12)
    torch.testing.assert_close(h2, hL, atol=1e-12, rtol=1e-12)


def test_complex_reduces_to_unitary_and_real():
    p = _inp("complex", gate=False)
    yu, hu = O.unitary_core_loop(p["u"], p["delta"], p["theta"], p["Bc"], p["Cc"], p["Dskip"])
    yc, hc = O.complex_core_loop(p["u"], p["delta"], torch.zeros_like(p["rho"]), p["theta"], p["Bc"], p["Cc"], p["Dskip"])
    torch.testing.assert_close(yc, yu, atol=1e-12, rtol=1e-12)
    torch.testing.assert_close(hc, hu, atol=1e-12, rtol=1e-12)
    # theta = 0, real B/C, rho = delta * A with A constant over n -> S6 with that A
    A = -torch.rand(3, 1, dtype=torch.float64).expand(3, 2).contiguous()
    Br, Cr = p["Bc"].real, p["Cc"].real
    yr, hr = O.real_core_loop(p["u"], p["delta"], A, Br, Cr, p["Dskip"])
    yc, hc = O.complex_core_loop(p["u"], p["delta"], p["delta"] * A[None, :, :1], torch.zeros_like(p["theta"]),
                                 Br.to(torch.complex128), Cr.to(torch.complex128), p["Dskip"])
    torch.testing.assert_close(yc, yr, atol=1e-12, rtol=1e-12)
    torch.testing.assert_close(hc.real, hr, atol=1e-12, rtol=1e-12)


def test_real_small_A_limit_is_cumsum():
    p = _inp("real", gate=False, L=19)
    y, _ = O.real_core_loop(p["u"], p["delta"], torch.zeros_like(p["A"]), p["Bm"], p["Cm"])
    S = torch.cumsum((p["delta"] * p["u"])[:, :, None, :] * p["Bm"][:, None], dim=-1)
    torch.testing.assert_close(y, (S * p["Cm"][:, None]).sum(2), atol=1e-12, rtol=1e-12)


def test_linearity_in_input():
    p = _inp("unitary", gate=False)
    f = lambda u: O.unitary_core_loop(u, p["delta"], p["theta"], p["Bc"], p["Cc"], p["Dskip"])[0]
    u2 = torch.randn_like(p["u"])
    torch.testing.assert_close(f(2.0 * p["u"] - 3.0 * u2), 2.0 * f(p["u"]) - 3.0 * f(u2), atol=1e-11, rtol=1e-11)


# ---- gradients: finite differences in float64 pin the autograd path used as the gradient oracle

def test_gradcheck_unitary():
    p = _inp("unitary", B=1, D=2, N=2, L=5)
    h0 = torch.complex(torch.randn(1, 2, 2, dtype=torch.float64), torch.randn(1, 2, 2, dtype=torch.float64))
    args = [p[k].clone().requires_grad_(True) for k in ("u", "delta", "theta", "Bc", "Cc", "Dskip", "z")] + [h0.requires_grad_(True)]
    assert torch.autograd.gradcheck(lambda *a: O.unitary_core_loop(*a), args, atol=1e-7, rtol=1e-6)


def test_gradcheck_complex():
    p = _inp("complex", B=1, D=2, N=2, L=5)
    args = [p[k].clone().requires_grad_(True) for k in ("u", "delta", "rho", "theta", "Bc", "Cc", "Dskip", "z")]
    assert torch.autograd.gradcheck(lambda *a: O.complex_core_loop(*a), args, atol=1e-7, rtol=1e-6)


def test_gradcheck_real():
    p = _inp("real", B=1, D=2, N=2, L=5)
    bias = torch.randn(2, dtype=torch.float64, requires_grad=True)
    args = [p[k].clone().requires_grad_(True) for k in ("u", "delta", "A", "Bm", "Cm", "Dskip", "z")] + [bias]
    assert torch.autograd.gradcheck(lambda *a: O.real_core_loop(*a, delta_softplus=True), args, atol=1e-7, rtol=1e-6)


# ---- drop-in operator semantics

def _adaptive(dtype=torch.float64, **kw):
    return O.make_adaptive_inputs(dtype=dtype, **kw)


def test_adaptive_loop_equals_polar():
    """Recurrence and cumulative-sum formulations (two independent texts in the
    reference: ssm_adaptive_unitary_forward.cu:113-181 as a recurrence, ops.py:661-764)."""
    args = _adaptive(b=3, d=5, n=4, l=14)
    torch.testing.assert_close(O.adaptive_unitary_loop(*args), O.adaptive_unitary_polar(*args), atol=1e-10, rtol=1e-10)
    args = _adaptive(b=2, d=4, n=3, l=37, binary_u=False, seed=3)
    torch.testing.assert_close(O.adaptive_unitary_loop(*args), O.adaptive_unitary_polar(*args), atol=1e-10, rtol=1e-10)


def test_adaptive_loop_bruteforce():
    u, dt, x, xb, Bp, Cp, D, z = _adaptive(b=2, d=3, n=2, l=6, binary_u=False, seed=5)
    y = O.adaptive_unitary_loop(u, dt, x, xb, Bp, Cp, D, z)
    b, d, l = u.shape
    n = Bp.shape[0]
    sp = lambda v: math.log1p(math.exp(v))
    for ib in range(b):
        for i in range(d):
            h = [0j] * n
            for t in range(l):
                us = _silu(float(u[ib, i, t]))
                acc = 0.0
                for j in range(n):
                    th = sum(float(x[i, j, r]) * float(u[ib, r, t]) for r in range(d)) + float(xb[i, j])
                    Bt = sp(float(Bp[j].real)) * cmath.exp(1j * float(Bp[j].imag))
                    Ct = sp(float(Cp[j].real)) * cmath.exp(1j * float(Cp[j].imag))
                    h[j] = cmath.exp(1j * th) * h[j] + Bt * float(dt[ib, i, t]) * us
                    acc += (Ct * h[j]).real
                val = (acc + float(D[i]) * us) * _silu(float(z[ib, i, t]))
                assert abs(val - float(y[ib, i, t])) < 1e-11


def test_adaptive_op_state_carry():
    """Launch-by-launch chunking with (h_re, h_im) carry equals the single scan (ops.py:72-85)."""
    u, dt, x, xb, Bp, Cp, D, z = _adaptive(b=2, d=3, n=2, l=32, binary_u=False, seed=6)
    full = O.adaptive_unitary_loop(u, dt, x, xb, Bp, Cp, D, z)
    Br, Bt, Cr, Ct = O.polar_params(Bp, Cp)
    hr = torch.zeros(2, 3, 2, dtype=torch.float64)
    hi = torch.zeros_like(hr)
    outs = []
    for s in range(0, 32, 16):
        sl = slice(s, s + 16)
        y, hr, hi = O.adaptive_unitary_op_loop(u[..., sl], dt[..., sl], x, xb, Br, Bt, Cr, Ct, D, z[..., sl], hr, hi)
        outs.append(y)
    torch.testing.assert_close(torch.cat(outs, -1), full, atol=1e-11, rtol=1e-11)


def test_reference_phase_loop_bruteforce():
    g = torch.Generator().manual_seed(2)
    b, d, n, l = 2, 3, 2, 5
    r = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64)
    u, dt, x, xb, Bph, Cph, D, z = r(b, d, l), r(b, d, l), r(d, n, d), r(d, n), r(b, n, l), r(b, n, l), r(d), r(b, d, l)
    y = O.reference_unitary_phase_loop(u, dt, x, xb, Bph, Cph, D, z)
    for ib in range(b):
        for i in range(d):
            h = [0j] * n
            for t in range(l):
                acc = 0.0
                for j in range(n):
                    th = sum(float(x[i, j, q]) * float(u[ib, q, t]) for q in range(d)) + float(xb[i, j])
                    h[j] = cmath.exp(1j * th) * h[j] + float(dt[ib, i, t]) * float(u[ib, i, t]) * cmath.exp(1j * float(Bph[ib, j, t]))
                    acc += (cmath.exp(1j * float(Cph[ib, j, t])) * h[j]).real
                val = (acc + float(u[ib, i, t]) * float(D[i])) * _silu(float(z[ib, i, t]))
                assert abs(val - float(y[ib, i, t])) < 1e-11


def test_causal_conv_bruteforce():
    """The blocks' convolution against the explicit causal sum in Python loops (a wrong shift,
    a flipped kernel or a missing trim fails it)."""
    g = torch.Generator().manual_seed(4)
    b, l, d, k = 2, 7, 3, 4
    x = torch.randn(b, l, d, generator=g, dtype=torch.float64)
    w = torch.randn(d, 1, k, generator=g, dtype=torch.float64)
    bias = torch.randn(d, generator=g, dtype=torch.float64)
    got = O.causal_conv1d_bld(x, w, bias)
    assert got.shape == (b, l, d)
    for bi in range(b):
        for li in range(l):
            for di in range(d):
                want = float(bias[di])
                for j in range(k):
                    ls = li - (k - 1) + j
                    if ls >= 0:
                        want += float(w[di, 0, j]) * float(x[bi, ls, di])
                assert abs(float(got[bi, li, di]) - want) < 1e-12


def _preal_inputs(b, d, n, l, seed):
    g = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64)
    # x small enough that exp(x.u) stays moderate over the sequence (the scan is unstable where x.u > 0)
    return dict(u=r(b, d, l), dt=F.softplus(r(b, d, l)), x=r(d, n, d) * 0.3, xb=r(d, n) * 0.3 - 0.5,
                B=r(b, n, l), C=r(b, n, l), D=r(d), z=r(b, d, l))


@pytest.mark.parametrize("step_scaled", [False, True])
def test_adaptive_preal_bruteforce(step_scaled):
    """The positive-real adaptive scan against scalar Python loops: the decay sees the RAW input through x
    (and, step-scaled, the bias and the step size), the input term silu(u) (plain) or u (step-scaled)."""
    b, d, n, l = 2, 3, 2, 6
    p = _preal_inputs(b, d, n, l, seed=12)
    y = O.adaptive_preal_loop(p["u"], p["dt"], p["x"], p["B"], p["C"], p["D"], p["z"],
                              x_bias=p["xb"] if step_scaled else None, step_scaled=step_scaled)
    for ib in range(b):
        for i in range(d):
            h = [0.0] * n
            for t in range(l):
                ut = float(p["u"][ib, i, t])
                v = ut if step_scaled else _silu(ut)
                acc = 0.0
                for j in range(n):
                    la = sum(float(p["x"][i, j, q]) * float(p["u"][ib, q, t]) for q in range(d))
                    if step_scaled:
                        la = (la + float(p["xb"][i, j])) * float(p["dt"][ib, i, t])
                    h[j] = math.exp(la) * h[j] + float(p["dt"][ib, i, t]) * float(p["B"][ib, j, t]) * v
                    acc += float(p["C"][ib, j, t]) * h[j]
                val = (acc + v * float(p["D"][i])) * _silu(float(p["z"][ib, i, t]))
                assert abs(val - float(y[ib, i, t])) < 1e-10 * max(1.0, abs(val))


def test_adaptive_preal_loop_equals_cumsum():
    """Recurrence against the reference's cumulative-sum formulation of the step-scaled form."""
    p = _preal_inputs(2, 4, 3, 24, seed=13)
    a = O.adaptive_preal_loop(p["u"], p["dt"], p["x"], p["B"], p["C"], p["D"], p["z"], x_bias=p["xb"], step_scaled=True)
    c = O.adaptive_preal_cumsum(p["u"], p["dt"], p["x"], p["xb"], p["B"], p["C"], p["D"], p["z"])
    torch.testing.assert_close(a, c, atol=1e-8, rtol=1e-8)


def test_gradcheck_adaptive_preal():
    p = _preal_inputs(1, 2, 2, 4, seed=14)
    leaves = [p[k].clone().requires_grad_(True) for k in ("u", "dt", "x", "B", "C", "D", "z")]
    assert torch.autograd.gradcheck(lambda *a: O.adaptive_preal_loop(*a), leaves, atol=1e-6, rtol=1e-5)


def test_polar_with_time_varying_phases_bruteforce():
    """The cumulative-sum formulation with B, C given as phases (b, n, l) and without the gate (the reference's
    other branches, ops.py:721-723, :745-746, :759-761) against scalar complex loops: the contraction sees the raw
    input, the recurrence silu(u), the coefficients are unit-modulus."""
    g = torch.Generator().manual_seed(21)
    b, d, n, l = 2, 3, 2, 5
    r = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64)
    u, dt, x, xb, Bph, Cph, D = r(b, d, l), r(b, d, l), r(d, n, d), r(d, n), r(b, n, l), r(b, n, l), r(d)
    y = O.adaptive_unitary_polar(u, dt, x, xb, Bph, Cph, D, None)
    for ib in range(b):
        for i in range(d):
            h = [0j] * n
            for t in range(l):
                acc = 0.0
                us = _silu(float(u[ib, i, t]))
                for j in range(n):
                    th = sum(float(x[i, j, q]) * float(u[ib, q, t]) for q in range(d)) + float(xb[i, j])
                    h[j] = cmath.exp(1j * th) * h[j] + float(dt[ib, i, t]) * us * cmath.exp(1j * float(Bph[ib, j, t]))
                    acc += (cmath.exp(1j * float(Cph[ib, j, t])) * h[j]).real
                val = acc + us * float(D[i])
                assert abs(val - float(y[ib, i, t])) < 1e-10
