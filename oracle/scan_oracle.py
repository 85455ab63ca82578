"""CPU oracle for the selective-scan hot path.  TEST INFRASTRUCTURE ONLY.

This module restates, in plain PyTorch on the CPU, the arithmetic of the
reference's scan operators.  It is the checker that the HIP kernels are
compared against; nothing in the shipped package imports it.  Only the test
suite, the smoke entry point and the CPU-baseline leg of the benchmark may use
it.

Every function walks the sequence with an explicit Python loop over time
(the reference's own "sequential-loop scan",
extension-cpp/extension_cpp/ops.py:215-223) unless its name says otherwise.
All functions are differentiable through torch.autograd and accept float32 or
float64 inputs (float64 is used for gradcheck and as a high-precision truth).

Pinning status (which independent check fixes each function):
  unitary_core_loop      brute-force scalar loop, closed forms (theta == 0 ->
                         cumulative sum; constant phase -> geometric series),
                         norm preservation, chunk composition, float64
                         gradcheck                                     pinned
  complex_core_loop      reduces to unitary_core_loop at rho == 0 and to
                         real_core_loop at theta == 0 with real B, C;
                         brute-force scalar loop; gradcheck            pinned
  real_core_loop         brute-force scalar loop, closed forms (A -> 0 gives a
                         cumulative sum), float64 gradcheck.  The reference
                         holds no test or fixture for the third-party
                         selective_scan_fn it calls
                         (ai-modules/wavesAI/model/aussm.py:791-802), so
                         against THAT package:                  parity unpinned
  adaptive_unitary_loop  agrees with adaptive_unitary_polar (two independent
                         formulations in the reference text: recurrence vs
                         cumulative sums), brute-force scalar loop     pinned
  adaptive_unitary_polar same pair                                     pinned
  reference_unitary_phase_loop
                         brute-force scalar loop                       pinned
  causal_conv1d_bld      torch's conv1d called exactly as the reference's blocks
                         call it; explicit causal sum in Python loops  pinned
  adaptive_preal_loop    brute-force scalar loop; with the decay scaled by
                         the step size it agrees with the reference's own
                         cumulative-sum formulation restated beside it
                         (adaptive_preal_cumsum); float64 gradcheck    pinned
  adaptive_preal_cumsum  same pair                                     pinned
"""
from __future__ import annotations

import math
from typing import Optional, Tuple

import torch
import torch.nn.functional as F

Tensor = torch.Tensor


def _cdtype(real_dtype: torch.dtype) -> torch.dtype:
    return torch.complex128 if real_dtype == torch.float64 else torch.complex64


# --------------------------------------------------------------------------
# Core scans: the form the benchmark measures.
#   h_l[b,d,n] = a_l * h_{l-1}[b,d,n] + delta_l[b,d] * B_l[b,n] * u_l[b,d]
#   y_l[b,d]   = Re sum_n C_l[b,n] h_l[b,d,n] + D[d] u_l[b,d]   (* silu(z_l))
# --------------------------------------------------------------------------

def unitary_core_loop(u: Tensor, delta: Tensor, theta: Tensor, Bc: Tensor, Cc: Tensor,
                      Dskip: Optional[Tensor] = None, z: Optional[Tensor] = None,
                      h0: Optional[Tensor] = None) -> Tuple[Tensor, Tensor]:
    """Adaptive-unitary scan, a_l = exp(i * theta_l[b,d]).

    u, delta, theta: (b, d, l) real.  Bc, Cc: (b, n, l) complex.  Dskip: (d,).
    z: (b, d, l) optional gate.  h0: (b, d, n) complex optional start state.
    Returns y (b, d, l) real and the final state h_L (b, d, n) complex.

    Follows the loop of extension-cpp/extension_cpp/ops.py:215-223 (state update
    then read-out with the same step's C), with the phase given per (b, d, l)
    instead of being contracted from u inside (ops.py:205-206).
    """
    b, d, l = u.shape
    n = Bc.shape[1]
    cd = _cdtype(u.dtype)
    a = torch.polar(torch.ones_like(theta), theta)                       # (b, d, l)
    h = torch.zeros(b, d, n, dtype=cd) if h0 is None else h0.to(cd)
    w = (delta * u).to(cd)                                               # (b, d, l)
    ys = []
    for t in range(l):
        h = a[:, :, t, None] * h + w[:, :, t, None] * Bc[:, None, :, t]
        ys.append((h * Cc[:, None, :, t]).sum(-1).real)
    y = torch.stack(ys, dim=-1)
    if Dskip is not None:
        y = y + u * Dskip[None, :, None]
    if z is not None:
        y = y * F.silu(z)
    return y, h


def complex_core_loop(u: Tensor, delta: Tensor, rho: Tensor, theta: Tensor, Bc: Tensor, Cc: Tensor,
                      Dskip: Optional[Tensor] = None, z: Optional[Tensor] = None,
                      h0: Optional[Tensor] = None) -> Tuple[Tensor, Tensor]:
    """Complex scan, a_l = exp(rho_l[b,d] + i * theta_l[b,d]).

    Same shapes as unitary_core_loop plus rho (b, d, l), the log-modulus.
    Follows extension-cpp/extension_cpp/ops.py:270-288 (A = polar(exp(.), .),
    complex B and C of shape (b, n, l)).
    """
    b, d, l = u.shape
    n = Bc.shape[1]
    cd = _cdtype(u.dtype)
    a = torch.polar(torch.exp(rho), theta)
    h = torch.zeros(b, d, n, dtype=cd) if h0 is None else h0.to(cd)
    w = (delta * u).to(cd)
    ys = []
    for t in range(l):
        h = a[:, :, t, None] * h + w[:, :, t, None] * Bc[:, None, :, t]
        ys.append((h * Cc[:, None, :, t]).sum(-1).real)
    y = torch.stack(ys, dim=-1)
    if Dskip is not None:
        y = y + u * Dskip[None, :, None]
    if z is not None:
        y = y * F.silu(z)
    return y, h


def real_core_loop(u: Tensor, delta: Tensor, A: Tensor, Bm: Tensor, Cm: Tensor,
                   Dskip: Optional[Tensor] = None, z: Optional[Tensor] = None,
                   delta_bias: Optional[Tensor] = None, delta_softplus: bool = False,
                   h0: Optional[Tensor] = None) -> Tuple[Tensor, Tensor]:
    """Real (Mamba S6) selective scan, a_l[d,n] = exp(delta_l[b,d] * A[d,n]).

    u, delta: (b, d, l).  A: (d, n).  Bm, Cm: (b, n, l) real.  Dskip: (d,).
    delta_bias: (d,).  Restates the published selective-scan formula behind the
    call at ai-modules/wavesAI/model/aussm.py:791-802:
        delta = softplus(delta + delta_bias); h = exp(delta A) h + delta B u;
        y = C.h + D u; y *= silu(z).
    The real-state loop itself also matches
    extension-cpp/extension_cpp/ops.py:349-356.
    """
    b, d, l = u.shape
    n = A.shape[1]
    if delta_bias is not None:
        delta = delta + delta_bias[None, :, None]
    if delta_softplus:
        delta = F.softplus(delta)
    h = torch.zeros(b, d, n, dtype=u.dtype) if h0 is None else h0
    ys = []
    for t in range(l):
        dA = torch.exp(delta[:, :, t, None] * A[None])                   # (b, d, n)
        h = dA * h + (delta[:, :, t] * u[:, :, t])[:, :, None] * Bm[:, None, :, t]
        ys.append((h * Cm[:, None, :, t]).sum(-1))
    y = torch.stack(ys, dim=-1)
    if Dskip is not None:
        y = y + u * Dskip[None, :, None]
    if z is not None:
        y = y * F.silu(z)
    return y, h


# --------------------------------------------------------------------------
# Drop-in operator semantics (extension_cpp::ssm_adaptive_unitary)
# --------------------------------------------------------------------------

def adaptive_phase(u: Tensor, x: Tensor, x_bias: Tensor) -> Tensor:
    """theta[b,i,j,l] = sum_r x[i,j,r] u[b,r,l] + x_bias[i,j].

    extension-cpp/extension_cpp/csrc/cuda/ssm_adaptive_unitary_forward.cu:83-110,
    extension-cpp/extension_cpp/ops.py:672,680.
    """
    return torch.einsum("ijr,brl->bijl", x, u) + x_bias[None, :, :, None]


def polar_params(Bp: Tensor, Cp: Tensor) -> Tuple[Tensor, Tensor, Tensor, Tensor]:
    """(B_r, B_theta, C_r, C_theta) = (softplus(Re B), Im B, softplus(Re C), Im C).

    extension-cpp/extension_cpp/ops.py:55-58 and :705-706, :737-738.
    """
    return F.softplus(Bp.real), Bp.imag, F.softplus(Cp.real), Cp.imag


def adaptive_unitary_op_loop(u: Tensor, dt: Tensor, x: Tensor, x_bias: Tensor,
                             B_r: Tensor, B_theta: Tensor, C_r: Tensor, C_theta: Tensor,
                             D: Tensor, z: Tensor, h0_re: Tensor, h0_im: Tensor
                             ) -> Tuple[Tensor, Tensor, Tensor]:
    """Sequential-loop restatement of the dispatcher op
    extension_cpp::ssm_adaptive_unitary (12 inputs, 3 outputs).

    Recurrence equivalent of the cumulative-sum kernel
    (ssm_adaptive_unitary_forward.cu:113-181):
        h_l[b,i,j] = exp(i theta_l[b,i,j]) h_{l-1} + Bt_j dt_l[b,i] silu(u_l[b,i])
        y_l[b,i]   = silu(z_l) * (sum_j Re(Ct_j h_l) + D_i silu(u_l))
    with Bt_j = B_r[j] exp(i B_theta[j]), Ct_j likewise, h_0 = h0_re + i h0_im.
    Returns (y, hL_re, hL_im).
    """
    b, d, l = u.shape
    theta = adaptive_phase(u, x, x_bias)                                 # (b, d, n, l)
    a = torch.polar(torch.ones_like(theta), theta)
    Bt = torch.polar(B_r, B_theta)
    Ct = torch.polar(C_r, C_theta)
    us = F.silu(u)
    w = (dt * us).to(a.dtype)
    h = torch.complex(h0_re, h0_im)
    ys = []
    for t in range(l):
        h = a[:, :, :, t] * h + w[:, :, t, None] * Bt[None, None, :]
        ys.append((h * Ct[None, None, :]).sum(-1).real)
    y = torch.stack(ys, dim=-1)
    y = (y + us * D[None, :, None]) * F.silu(z)
    return y, h.real, h.imag


def adaptive_unitary_loop(u: Tensor, dt: Tensor, x: Tensor, x_bias: Tensor, Bp: Tensor, Cp: Tensor,
                          D: Tensor, z: Tensor) -> Tensor:
    """What ssm_adaptive_interface computes (extension-cpp/extension_cpp/ops.py:28-93)
    for constant complex parameters Bp, Cp of shape (n,), from a zero start state,
    written as one sequential loop over the whole sequence."""
    B_r, B_th, C_r, C_th = polar_params(Bp, Cp)
    b, d, _ = u.shape
    n = Bp.shape[0]
    zero = torch.zeros(b, d, n, dtype=u.dtype)
    return adaptive_unitary_op_loop(u, dt, x, x_bias, B_r, B_th, C_r, C_th, D, z, zero, zero)[0]


def adaptive_unitary_polar(u: Tensor, dt: Tensor, x: Tensor, x_bias: Tensor, Bp: Tensor, Cp: Tensor,
                           D: Tensor, z: Optional[Tensor] = None) -> Tensor:
    """Cumulative-sum ("polar") formulation.

    Restates extension-cpp/extension_cpp/ops.py:661-764 (binary=False):
        G = cumsum(theta) mod 2 pi
        re = cumsum(B_r cos(B_theta - G) dt silu(u)), im likewise with sin
        y  = sum_j C_r (cos(C_theta + G) re - sin(C_theta + G) im) + silu(u) D      (* silu(z) if z is given)
    Bp, Cp: constant complex (n,) - radius softplus(real part), phase the imaginary part (ops.py:705-706,
    :737-738), the branch the reference's tests use - or real phases (b, n, l) of unit-modulus time-varying
    coefficients (ops.py:721-723, :745-746).  z None is the reference's z_prod=False.
    This is a formulation independent of the recurrence in adaptive_unitary_loop; the two must agree.
    """
    theta = adaptive_phase(u, x, x_bias).permute(0, 3, 1, 2)             # (b, l, d, n)
    G = torch.cumsum(theta, dim=1) % (2 * math.pi)

    def polar_of(c):
        if c.dim() == 1:
            return F.softplus(c.real), c.imag
        return torch.ones_like(c).permute(0, 2, 1)[:, :, None, :], c.permute(0, 2, 1)[:, :, None, :]   # (b, l, 1, n)
    B_r, B_th = polar_of(Bp)
    C_r, C_th = polar_of(Cp)
    us = F.silu(u).permute(0, 2, 1)                                      # (b, l, d)
    dtl = dt.permute(0, 2, 1)
    amp = (dtl * us)[..., None]
    re = torch.cumsum(B_r * torch.cos(B_th - G) * amp, dim=1)
    im = torch.cumsum(B_r * torch.sin(B_th - G) * amp, dim=1)
    y = (C_r * (torch.cos(C_th + G) * re - torch.sin(C_th + G) * im)).sum(-1)
    y = y + us * D
    if z is not None:
        y = y * F.silu(z.permute(0, 2, 1))
    return y.permute(0, 2, 1)


def reference_unitary_phase_loop(u: Tensor, dt: Tensor, x: Tensor, x_bias: Tensor, B_phase: Tensor,
                                 C_phase: Tensor, D: Tensor, z: Tensor) -> Tensor:
    """Restatement of reference_ssm_adaptive_unitary
    (extension-cpp/extension_cpp/ops.py:170-230): time-varying unit-modulus
    B, C given as phases (b, n, l), raw u (no silu), zero start state."""
    theta = adaptive_phase(u, x, x_bias)                                 # (b, d, n, l)
    a = torch.polar(torch.ones_like(theta), theta)
    Bc = torch.polar(torch.ones_like(B_phase), B_phase)
    Cc = torch.polar(torch.ones_like(C_phase), C_phase)
    b, d, l = u.shape
    n = x.shape[1]
    h = torch.zeros(b, d, n, dtype=a.dtype)
    ys = []
    for t in range(l):
        h = a[:, :, :, t] * h + (dt[:, :, t] * u[:, :, t])[:, :, None] * Bc[:, None, :, t]
        ys.append((h * Cc[:, None, :, t]).sum(-1).real)
    y = torch.stack(ys, dim=-1)
    return (y + u * D[None, :, None]) * F.silu(z)


# --------------------------------------------------------------------------
# Positive-real adaptive scan of the reference's pure-PyTorch file (no kernel
# of the reference is reachable for it; extension_cpp/ops.py:86-87 raises).
# --------------------------------------------------------------------------

def adaptive_preal_loop(u: Tensor, dt: Tensor, x: Tensor, B: Tensor, C: Tensor, D: Tensor, z: Tensor,
                        x_bias: Optional[Tensor] = None, step_scaled: bool = False) -> Tensor:
    """Real adaptive scan whose decay is contracted from the input,
        log a_l[b,i,j] = sum_r x[i,j,r] u_l[b,r]           (+ x_bias[i,j], times dt_l[b,i] if step_scaled)
        h_l = a_l h_{l-1} + dt_l[b,i] B_l[b,j] v_l[b,i],   y_l = (sum_j C_l[b,j] h_l + D_i v_l) silu(z_l),  h_0 = 0.
    step_scaled=False restates reference_ssm_adaptive_preal (extension-cpp/extension_cpp/ops.py:300-357):
    no bias, and the input enters through v = silu(u) (ops.py:333) while the decay sees the raw u (ops.py:331).
    step_scaled=True restates the recurrence behind reference_ssm_adaptive_preal_optimized (ops.py:465-510):
    log a = (x.u + x_bias) dt (ops.py:491-493) and v = u, the raw input (no silu there).
    u, dt, z: (b, d, l); x: (d, n, d); B, C: (b, n, l) real; D: (d,)."""
    b, d, l = u.shape
    log_a = torch.einsum("ijr,brl->bijl", x, u)
    if x_bias is not None:
        log_a = log_a + x_bias[None, :, :, None]
    if step_scaled:
        log_a = log_a * dt[:, :, None, :]
    v = u if step_scaled else F.silu(u)
    a = torch.exp(log_a)                                                 # (b, d, n, l)
    w = dt * v
    h = torch.zeros(b, d, x.shape[1], dtype=u.dtype)
    ys = []
    for t in range(l):
        h = a[:, :, :, t] * h + w[:, :, t, None] * B[:, None, :, t]
        ys.append((h * C[:, None, :, t]).sum(-1))
    y = torch.stack(ys, dim=-1)
    return (y + v * D[None, :, None]) * F.silu(z)


def adaptive_preal_cumsum(u: Tensor, dt: Tensor, x: Tensor, x_bias: Tensor, B: Tensor, C: Tensor, D: Tensor,
                          z: Tensor) -> Tensor:
    """The cumulative-sum formulation the reference writes for the step-scaled form
    (extension-cpp/extension_cpp/ops.py:491-503): G = cumsum(log a), y = sum_j C exp(G) cumsum(exp(-G) dt B u).
    Independent of the recurrence above (and overflow-prone for long sequences, as upstream)."""
    log_a = (torch.einsum("ijr,brl->bijl", x, u) + x_bias[None, :, :, None]) * dt[:, :, None, :]
    G = torch.cumsum(log_a, dim=-1)
    inner = torch.cumsum(torch.exp(-G) * (dt * u)[:, :, None, :] * B[:, None, :, :], dim=-1)
    y = (C[:, None, :, :] * torch.exp(G) * inner).sum(2)
    return (y + u * D[None, :, None]) * F.silu(z)


# --------------------------------------------------------------------------
# Seeded input recipes shared by tests, smoke and bench (synthetic data).
# --------------------------------------------------------------------------

def causal_conv1d_bld(x: Tensor, weight: Tensor, bias: Optional[Tensor]) -> Tensor:
    """The blocks' depthwise causal convolution on x (b, l, d), exactly as the reference writes it
    (ai-modules/wavesAI/model/aussm.py:762, :863): nn.Conv1d(d, d, k, groups=d, padding=k-1) on
    the transposed tensor, output trimmed to l steps.  Pinned by tests/test_oracle.py against the
    explicit sum  y[b,l,d] = bias[d] + sum_j w[d,j] x[b, l-(k-1)+j, d]  in plain Python loops."""
    b, l, d = x.shape
    k = weight.shape[-1]
    y = F.conv1d(x.transpose(1, 2), weight.reshape(d, 1, k), bias, padding=k - 1, groups=d)
    return y[:, :, :l].transpose(1, 2)


def make_core_inputs(B: int, D: int, N: int, L: int, seed: int = 0, variant: str = "unitary",
                     dtype: torch.dtype = torch.float32, gate: bool = False):
    """Value distributions of the benchmark configurations:
    u ~ N(0,1); delta = softplus(N(0,1)); theta ~ N(0, 0.5) (std 0.5);
    B_t, C_t complex with re/im ~ N(0, 1/sqrt(N)) (std N^-1/2); D ~ N(0,1);
    real variant: A = -exp(N(0,1)) (d, n), real B, C with the same std;
    complex variant: rho = -delta * exp(N(0,1))[d] (non-positive log-modulus);
    dy ~ N(0,1).  Returned as a dict of CPU tensors."""
    g = torch.Generator().manual_seed(seed)
    rn = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64).to(dtype)
    std = N ** -0.5
    out = {
        "u": rn(B, D, L),
        "delta": F.softplus(rn(B, D, L)),
        "Dskip": rn(D),
        "dy": rn(B, D, L),
    }
    if variant == "real":
        out["A"] = -torch.exp(rn(D, N))
        out["Bm"] = rn(B, N, L) * std
        out["Cm"] = rn(B, N, L) * std
    else:
        out["theta"] = rn(B, D, L) * 0.5
        out["Bc"] = torch.complex(rn(B, N, L) * std, rn(B, N, L) * std)
        out["Cc"] = torch.complex(rn(B, N, L) * std, rn(B, N, L) * std)
        if variant == "complex":
            out["rho"] = -out["delta"] * torch.exp(rn(D))[None, :, None]
    if gate:
        out["z"] = rn(B, D, L)
    return out


def make_adaptive_inputs(b: int = 16, d: int = 16, n: int = 16, l: int = 14, seed: int = 10,
                         binary_u: bool = True, dtype: torch.dtype = torch.float32):
    """The reference test's input recipe
    (extension-cpp/test/test_extension.py:31-70): seed 10, b=d=n=16, l=14,
    u in {0,1}, everything else standard normal, B and C complex (n,)."""
    g = torch.Generator().manual_seed(seed)
    rn = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64).to(dtype)
    if binary_u:
        u = torch.randint(0, 2, (b, d, l), generator=g).to(dtype)
    else:
        u = rn(b, d, l)
    dt = rn(b, d, l)
    x = rn(d, n, d)
    x_bias = rn(d, n)
    Bp = torch.complex(rn(n), rn(n))
    Cp = torch.complex(rn(n), rn(n))
    D = rn(d)
    z = rn(b, d, l)
    return u, dt, x, x_bias, Bp, Cp, D, z
