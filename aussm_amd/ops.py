"""Drop-in operator layer: the Python surface and the dispatcher ops of the reference's
extension-cpp/extension_cpp/ops.py, running on the HIP core scan.

    ssm_adaptive_interface(u, dt, x, x_bias, B, C, D, z, unitary=True, ...)     ops.py:28-93
    ssm_adaptive_unitary(12 tensors) -> (y, next_hid_real, next_hid_imag)        ops.py:97-105
    torch.ops.extension_cpp.ssm_adaptive_unitary / ssm_adaptive_backward_unitary
        schemas of extension-cpp/extension_cpp/csrc/cuda/ssm_adaptive_unitary_forward.cu:284-285,
        autograd registration as ops.py:148-154.

Operator semantics (ssm_adaptive_unitary_forward.cu:83-181), per batch b, channel i, state j:

    theta_l[b,i,j] = sum_r x[i,j,r] u_l[b,r] + x_bias[i,j]
    h_l[b,i,j]     = exp(i theta_l) h_{l-1}[b,i,j] + Bt_j dt_l[b,i] silu(u_l[b,i]),   Bt_j = B_r[j] e^{i B_theta[j]}
    y_l[b,i]       = silu(z_l[b,i]) * ( sum_j Re(Ct_j h_l[b,i,j]) + D_i silu(u_l[b,i]) )

The two dispatcher ops run the library's fused kernels (aussm_ssm_adaptive_unitary_fwd / _bwd,
include/aussm_hip.h): the phase tensor theta (b, d, n, l) is formed tile by tile inside the scan
kernel and never stored, and the backward op recomputes from the twelve inputs as the reference's
does.  Shapes beyond the fused kernels' limits (n > 64 or d > 512) take the composite route below.

`_composite` is a second, independent route to the same numbers, kept for the interface's
save_intermediates=True mode and as a cross-check in the tests: every (batch, state) pair becomes
one batch element of a core scan with ONE state per channel - its phase is theta[b, j]
(channels x time), its B_t and C_t are the constants Bt_j and Ct_j - the phase projection is a
BLAS GEMM, and the sum over j is taken afterwards.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch
import torch.nn.functional as F
from torch import Tensor

from . import _lib as L
from . import scan

__all__ = ["ssm_adaptive_unitary", "ssm_adaptive_interface", "pad_to_multiple_of",
           "reference_ssm_adaptive_unitary_optimized_polar", "reference_ssm_adaptive_preal",
           "reference_ssm_adaptive_preal_optimized"]

_NS = "extension_cpp"
_FWD_SCHEMA = ("ssm_adaptive_unitary(Tensor u, Tensor dt, Tensor x, Tensor x_bias, Tensor B_r, Tensor B_theta, "
               "Tensor C_r, Tensor C_theta, Tensor D, Tensor z, Tensor prev_hid_real, "
               "Tensor prev_hidden_state_imag) -> (Tensor, Tensor, Tensor)")
_BWD_SCHEMA = ("ssm_adaptive_backward_unitary(Tensor grad_y, Tensor grad_next_hid_real, Tensor grad_next_hid_imag, "
               "Tensor u, Tensor dt, Tensor x, Tensor x_bias, Tensor B_r, Tensor B_theta, Tensor C_r, "
               "Tensor C_theta, Tensor D, Tensor z, Tensor prev_hid_real, Tensor prev_hidden_state_imag) -> "
               "(Tensor, Tensor, Tensor, Tensor, Tensor, Tensor, Tensor, Tensor, Tensor, Tensor, Tensor, Tensor)")

_INPUT_NAMES = ("u", "dt", "x", "x_bias", "B_r", "B_theta", "C_r", "C_theta", "D", "z",
                "prev_hid_real", "prev_hidden_state_imag")


def _check_op_inputs(args) -> Tuple[int, int, int, int]:
    u, dt, x, x_bias, B_r, B_theta, C_r, C_theta, D, z, h_r, h_i = args
    for name, t in zip(_INPUT_NAMES, args):
        if t.dtype != torch.float32:
            # the reference fails in data_ptr<float>() (ssm_adaptive_unitary_forward.cu:231-245)
            raise RuntimeError(f"expected scalar type Float for {name} but found {t.dtype}")
        if not t.is_cuda:
            raise RuntimeError(f"{name} must be a GPU tensor")
    if u.dim() != 3:
        raise RuntimeError(f"expected u of shape (b, d, l), got {tuple(u.shape)}")
    b, d, l = u.shape
    if x.dim() != 3 or x.shape[0] != d or x.shape[2] != d:
        raise RuntimeError(f"expected x of shape (d, n, d) with d = {d}, got {tuple(x.shape)}")
    n = x.shape[1]
    want = {"dt": (b, d, l), "z": (b, d, l), "x_bias": (d, n), "B_r": (n,), "B_theta": (n,), "C_r": (n,),
            "C_theta": (n,), "D": (d,), "prev_hid_real": (b, d, n), "prev_hidden_state_imag": (b, d, n)}
    for name, t in zip(_INPUT_NAMES, args):
        if name in want and tuple(t.shape) != want[name]:
            raise RuntimeError(f"expected {name} of shape {want[name]}, got {tuple(t.shape)}")
    return b, d, n, l


def _composite_scan(u, dt, x, x_bias, Bt, Ct, D, z, h_r, h_i):
    """Differentiable torch ops around ONE core-scan launch.  Bt, Ct: complex (n,) constants or (b, n, l)
    time-varying; z None: no gate."""
    b, d, l = u.shape
    n = x.shape[1]
    # phase projection: theta[b, j, i, l]  (state index before channel so that (b, j) is a batch)
    xm = x.permute(1, 0, 2).reshape(n * d, d)                          # (j i) x r
    # one strided-batched GEMM straight into (b, (j i), l); the 2-D x 3-D form of matmul goes through
    # transposed copies of the whole phase tensor
    theta = torch.baddbmm(x_bias.t().reshape(1, n * d, 1), xm.unsqueeze(0).expand(b, n * d, d), u).view(b, n, d, l)
    us = F.silu(u)
    row = lambda c: (c[None, :, None].expand(b, n, l) if c.dim() == 1 else c).reshape(b * n, 1, l)
    h0 = torch.complex(h_r, h_i).permute(0, 2, 1).reshape(b * n, d, 1)
    # us, dt stay (b, d, l): each of their batch elements serves the n consecutive (batch, state) pairs
    y, hL = scan.unitary_scan(us, dt.contiguous(), theta.reshape(b * n, d, l), row(Bt), row(Ct), None, None, h0,
                              return_last_state=True)
    y = y.view(b, n, d, l).sum(dim=1)
    y = y + us * D[None, :, None]
    if z is not None:
        y = y * F.silu(z)
    hL = hL.view(b, n, d).permute(0, 2, 1)
    return y, hL.real.contiguous(), hL.imag.contiguous()


def _composite(u, dt, x, x_bias, B_r, B_theta, C_r, C_theta, D, z, h_r, h_i):
    """The operator as differentiable torch ops around ONE core-scan launch."""
    _check_op_inputs((u, dt, x, x_bias, B_r, B_theta, C_r, C_theta, D, z, h_r, h_i))
    return _composite_scan(u, dt, x, x_bias, torch.polar(B_r, B_theta), torch.polar(C_r, C_theta), D, z, h_r, h_i)


# ---- dispatcher ops -------------------------------------------------------------------------

_lib = torch.library.Library(_NS, "FRAGMENT")
_lib.define(_FWD_SCHEMA)
_lib.define(_BWD_SCHEMA)


def fused_supported(b: int, d: int, n: int, l: int) -> bool:
    """Whether the fused kernels take this shape (n <= 64, d <= 512); beyond it the dispatcher ops run
    the composite route (same HIP core scan, phase tensor materialised)."""
    return L.load().aussm_ssm_adaptive_unitary_workspace_floats(b, d, n, l, 0) > 0


def _workspace(b, d, n, l, backward, device):
    floats = L.load().aussm_ssm_adaptive_unitary_workspace_floats(b, d, n, l, int(backward))
    return torch.empty(floats, device=device, dtype=torch.float32)


def _fwd_impl(u, dt, x, x_bias, B_r, B_theta, C_r, C_theta, D, z, h_r, h_i):
    args = [t.contiguous() for t in (u, dt, x, x_bias, B_r, B_theta, C_r, C_theta, D, z, h_r, h_i)]
    b, d, n, l = _check_op_inputs(args)
    if not fused_supported(b, d, n, l):
        with torch.no_grad():
            return _composite(*args)
    with torch.cuda.device(u.device):
        y, nh_r, nh_i = torch.empty_like(args[0]), torch.empty_like(args[10]), torch.empty_like(args[11])
        ws = _workspace(b, d, n, l, False, u.device)
        L.check(L.load().aussm_ssm_adaptive_unitary_fwd(
            *[L.ptr(t) for t in args], L.ptr(y), L.ptr(nh_r), L.ptr(nh_i), L.ptr(ws), b, d, n, l,
            scan._stream()), "aussm_ssm_adaptive_unitary_fwd")
    return y, nh_r, nh_i


def _bwd_impl(grad_y, grad_hr, grad_hi, u, dt, x, x_bias, B_r, B_theta, C_r, C_theta, D, z, h_r, h_i,
              nh_r=None, nh_i=None):
    args = [t.contiguous() for t in (u, dt, x, x_bias, B_r, B_theta, C_r, C_theta, D, z, h_r, h_i)]
    b, d, n, l = _check_op_inputs(args)
    grads_in = [grad_y.contiguous(), grad_hr.contiguous(), grad_hi.contiguous()]
    if not fused_supported(b, d, n, l):
        with torch.enable_grad():
            leaves = [t.detach().requires_grad_(True) for t in args]
            grads = torch.autograd.grad(_composite(*leaves), leaves, grads_in, allow_unused=True)
        return tuple(torch.zeros_like(t) if g is None else g.contiguous() for g, t in zip(grads, leaves))
    for name, t, like in zip(("grad_y", "grad_next_hid_real", "grad_next_hid_imag"), grads_in,
                             (args[0], args[10], args[11])):
        if t.dtype != torch.float32 or tuple(t.shape) != tuple(like.shape):
            raise RuntimeError(f"expected {name} float32 of shape {tuple(like.shape)}, got {t.dtype} {tuple(t.shape)}")
    with torch.cuda.device(u.device):
        outs = [torch.empty_like(t) for t in args]
        ws = _workspace(b, d, n, l, True, u.device)
        L.check(L.load().aussm_ssm_adaptive_unitary_bwd(
            *[L.ptr(t) for t in grads_in], *[L.ptr(t) for t in args],
            L.ptr(None if nh_r is None else nh_r.contiguous()), L.ptr(None if nh_i is None else nh_i.contiguous()),
            *[L.ptr(t) for t in outs], L.ptr(ws),
            b, d, n, l, scan._stream()), "aussm_ssm_adaptive_unitary_bwd")
    return tuple(outs)


_lib.impl("ssm_adaptive_unitary", _fwd_impl, "CUDA")
_lib.impl("ssm_adaptive_backward_unitary", _bwd_impl, "CUDA")

# The backward operator above gets what the reference's gets: gradients and the twelve inputs, so it
# first re-runs the forward recurrence to find the state at the end of the sequence, where the
# reverse sweep starts.  The autograd formula has that state already (it is an output of the forward
# operator), so it calls this variant, which takes it as two more inputs and skips the re-run.
_own = torch.library.Library("aussm_amd", "FRAGMENT")
_own.define(_BWD_SCHEMA.replace("ssm_adaptive_backward_unitary(", "ssm_adaptive_backward_unitary_from_state(")
            .replace("Tensor prev_hidden_state_imag) ->", "Tensor prev_hidden_state_imag, Tensor next_hid_real, "
                     "Tensor next_hid_imag) ->"))
_own.impl("ssm_adaptive_backward_unitary_from_state", _bwd_impl, "CUDA")


@torch.library.register_fake(f"{_NS}::ssm_adaptive_unitary")
def _fwd_fake(u, dt, x, x_bias, B_r, B_theta, C_r, C_theta, D, z, h_r, h_i):
    return torch.empty_like(u), torch.empty_like(h_r), torch.empty_like(h_i)


@torch.library.register_fake(f"{_NS}::ssm_adaptive_backward_unitary")
def _bwd_fake(grad_y, grad_hr, grad_hi, u, dt, x, x_bias, B_r, B_theta, C_r, C_theta, D, z, h_r, h_i):
    return tuple(torch.empty_like(t) for t in (u, dt, x, x_bias, B_r, B_theta, C_r, C_theta, D, z, h_r, h_i))


@torch.library.register_fake("aussm_amd::ssm_adaptive_backward_unitary_from_state")
def _bwd_state_fake(grad_y, grad_hr, grad_hi, u, dt, x, x_bias, B_r, B_theta, C_r, C_theta, D, z, h_r, h_i, nh_r, nh_i):
    return tuple(torch.empty_like(t) for t in (u, dt, x, x_bias, B_r, B_theta, C_r, C_theta, D, z, h_r, h_i))


def ssm_adaptive_unitary(u: Tensor, dt: Tensor, x: Tensor, x_bias: Tensor, B_r: Tensor, B_theta: Tensor,
                         C_r: Tensor, C_theta: Tensor, D: Tensor, z: Tensor, prev_hidden_state_real: Tensor,
                         prev_hidden_state_imag: Tensor) -> Tuple[Tensor, Tensor, Tensor]:
    """The operator call (ops.py:97-105): (y, next_hid_real, next_hid_imag)."""
    return torch.ops.extension_cpp.ssm_adaptive_unitary.default(
        u, dt, x, x_bias, B_r, B_theta, C_r, C_theta, D, z, prev_hidden_state_real, prev_hidden_state_imag)


def backward_unitary(ctx, grad_y, grad_next_hidden_state_real, grad_next_hidden_state_imag):
    """Autograd formula (ops.py:109-146): gradients for the 12 inputs, in input order."""
    saved = ctx.saved_tensors
    try:
        return torch.ops.aussm_amd.ssm_adaptive_backward_unitary_from_state.default(
            grad_y, grad_next_hidden_state_real, grad_next_hidden_state_imag, *saved)
    except RuntimeError:
        shapes = {k: tuple(t.shape) for k, t in zip(_INPUT_NAMES, saved[:12])}
        shapes["grad_y"] = tuple(grad_y.shape)
        print(f"Runtime Error for {shapes}")
        raise


def setup_context_unitary(ctx, inputs, output):
    # like the reference (ops.py:148-151) the 12 inputs are kept for the backward pass - no intermediate of
    # the size of the sequence - plus the two (b, d, n) end states, where the reverse sweep starts
    ctx.save_for_backward(*inputs, output[1], output[2])


torch.library.register_autograd(f"{_NS}::ssm_adaptive_unitary", backward_unitary,
                                setup_context=setup_context_unitary)


# ---- front-end ------------------------------------------------------------------------------

def pad_to_multiple_of(tensor: Tensor, multiple_of: int) -> Tensor:
    """Zero-pad the last dimension up to a multiple (ops.py:21-25)."""
    length = tensor.shape[-1]
    padded = -(-length // multiple_of) * multiple_of
    return F.pad(tensor, (0, padded - length), value=0)


def ssm_adaptive_interface(u: Tensor, dt: Tensor, x: Tensor, x_bias: Tensor, B: Tensor, C: Tensor, D: Tensor,
                           z: Tensor, unitary: bool = True, preal: bool = False,
                           max_parallel_length: int = 2048, save_intermediates: bool = False, **kwargs) -> Tensor:
    """Front-end of the adaptive-unitary operator (ops.py:28-93).

    u, dt, z: (b, d, l) float32; x: (d, n, d); x_bias: (d, n); B, C: (n,) complex64; D: (d,).
    B and C are given in the reference's parameterisation: radius = softplus(real part),
    phase = imaginary part.  The sequence is processed in launches of at most
    `max_parallel_length` steps with the complex state carried from launch to launch, starting
    from zero, exactly as the reference does; unknown keyword arguments are ignored as there.
    (The reference zero-pads the sequence to a multiple of 16 for its kernel; this kernel takes
    any length, and the padded steps never influence the returned y.)

    save_intermediates (not in the reference): False, the default, goes through the dispatcher
    operator, i.e. the fused kernels: the phase tensor (b, d, n, l) is never stored and the backward
    pass keeps only the twelve inputs and the end state and recomputes, as the reference's does
    (ops.py:148-151).  True takes the composite route instead (BLAS phase projection + core scan),
    which holds the phase tensor and the scan's checkpoints for the backward pass - n times the
    memory, and slower at the benchmark's training shape; it is kept as an independent cross-check.
    """
    assert not (unitary and preal), "Both unitary and preal cannot be used at the same time"
    if not unitary:
        raise NotImplementedError("other kernels not implemented")
    if max_parallel_length < 1:
        raise ValueError("max_parallel_length must be positive")
    b, d, l = u.shape
    n = x.shape[1]
    B_r = F.softplus(B.real).contiguous()
    B_theta = B.imag.contiguous()
    C_r = F.softplus(C.real).contiguous()
    C_theta = C.imag.contiguous()
    h_r = torch.zeros((b, d, n), device=u.device, dtype=torch.float32)
    h_i = torch.zeros_like(h_r)
    outs = []
    for s in range(0, l, max_parallel_length):
        e = min(s + max_parallel_length, l)
        op = _composite if save_intermediates else ssm_adaptive_unitary
        y, h_r, h_i = op(u[:, :, s:e].contiguous(), dt[:, :, s:e].contiguous(), x.contiguous(),
                         x_bias.contiguous(), B_r, B_theta, C_r, C_theta, D.contiguous(),
                         z[:, :, s:e].contiguous(), h_r, h_i)
        outs.append(y)
    return outs[0] if len(outs) == 1 else torch.cat(outs, dim=-1)


def reference_ssm_adaptive_unitary_optimized_polar(u: Tensor, dt: Tensor, x: Tensor, x_bias: Tensor, B: Tensor,
                                                   C: Tensor, D: Tensor, z: Optional[Tensor] = None,
                                                   diagnostic: bool = False, z_prod: bool = True, binary: bool = False,
                                                   no_graded_rotation: bool = False, unitary: bool = True) -> Tensor:
    """The callable `SSMauBlock(cuda=False)` selects in the reference (aussm.py:842-843; ops.py:614-769):
    there a pure-PyTorch cumulative-sum form of the same operator.  Here the name and signature are kept
    and every case runs on the HIP kernels; there is no eager or CPU path behind it.
      * constant complex B, C of shape (n,) with the gate (the default, what the blocks call): the fused
        kernels of ssm_adaptive_interface, one launch sequence, any length;
      * B and / or C given as real phases of shape (b, n, l) (unit modulus, ops.py:721-723, :745-746), or
        z_prod=False (no gate, ops.py:759-761): the composite route - phase projection by BLAS, one core-scan
        launch with every (batch, state) pair as a batch element.
    The remaining research switches of the reference (diagnostic outputs, binary or ungraded rotations) replace
    the rotation by sign functions and return (b, l, d, n) intermediates; they are not implemented and raise."""
    if diagnostic or binary or no_graded_rotation or not unitary:
        raise NotImplementedError("diagnostic outputs and binary / ungraded rotations are not implemented")
    if z_prod and z is None:
        raise ValueError("z is required (z_prod=True)")
    if not u.is_cuda:
        raise RuntimeError("scan inputs must be on the GPU (no CPU implementation is shipped)")
    if B.dim() == 1 and C.dim() == 1 and z_prod:
        return ssm_adaptive_interface(u, dt, x, x_bias, B, C, D, z, unitary=True, max_parallel_length=max(1, u.shape[-1]))
    b, d, l = u.shape
    n = x.shape[1]

    def coefficient(c, name):
        if c.dim() == 1:                                   # radius = softplus(real part), phase = imaginary part
            return torch.polar(F.softplus(c.real), c.imag)
        if c.is_complex() or tuple(c.shape) != (b, n, l):
            raise RuntimeError(f"expected {name} complex of shape ({n},) or real phases of shape {(b, n, l)}")
        return torch.polar(torch.ones_like(c), c)
    zero = torch.zeros((b, d, n), device=u.device, dtype=torch.float32)
    y, _, _ = _composite_scan(u.contiguous(), dt, x, x_bias, coefficient(B, "B"), coefficient(C, "C"), D,
                              z if z_prod else None, zero, zero)
    return y


# ---- the positive-real adaptive scan of the reference's pure-PyTorch file -------------------------------------
# Upstream it has no reachable kernel (ssm_adaptive_interface raises for unitary=False, ops.py:86-87, as this
# package's does) and no caller in the models; the two callables keep their names and signatures and run the
# recurrence on the HIP scan kernels.  The decay exp(x.u) differs per (channel, state) pair, so every pair is one
# channel with a single state of the complex scan (log-modulus = the contracted decay, phase 0): the launch
# covers d n channels, the products with B_t in front of it and with C_t behind it are elementwise torch, and
# autograd runs through the scan's own backward kernels.

def _preal_scan(log_a: Tensor, w: Tensor, B: Tensor, C: Tensor) -> Tensor:
    """sum_j C_l[b,j] h_l[b,i,j] with h_l = exp(log_a_l) h_{l-1} + w_l[b,i] B_l[b,j], h_0 = 0.
    log_a: (b, d, n, l); w: (b, d, l); B, C: (b, n, l) real."""
    b, d, n, l = log_a.shape
    inp = (w[:, :, None, :] * B[:, None, :, :]).reshape(b, d * n, l)
    one = torch.ones((b, d * n, l), device=w.device, dtype=torch.float32)
    unit = torch.ones((b, 1, l), device=w.device, dtype=torch.complex64)
    h = scan.complex_scan(inp, one, log_a.reshape(b, d * n, l).contiguous(), torch.zeros_like(one), unit, unit)
    return (h.view(b, d, n, l) * C[:, None, :, :]).sum(2)


def _preal_check(u, dt, x, B, C, D, z):
    for name, t in (("u", u), ("dt", dt), ("x", x), ("B", B), ("C", C), ("D", D), ("z", z)):
        if t.dtype != torch.float32:
            raise RuntimeError(f"expected {name} to be float32, got {t.dtype}")
        if not t.is_cuda:
            raise RuntimeError("scan inputs must be on the GPU (no CPU implementation is shipped)")
    if x.dim() != 3:
        raise RuntimeError("x must be (d, n, d)")


def reference_ssm_adaptive_preal(u: Tensor, dt: Tensor, x: Tensor, B: Tensor, C: Tensor, D: Tensor, z: Tensor) -> Tensor:
    """Name, signature and arithmetic of extension-cpp/extension_cpp/ops.py:300-357:
    h_l = exp(x.u_l) h_{l-1} + dt_l B_l silu(u_l),  y_l = (sum_j C_l h_l + D silu(u_l)) silu(z_l), from a zero state.
    u, dt, z: (b, d, l); x: (d, n, d); B, C: (b, n, l) real; D: (d,)."""
    _preal_check(u, dt, x, B, C, D, z)
    log_a = torch.einsum("ijr,brl->bijl", x, u)
    us = F.silu(u)
    y = _preal_scan(log_a, dt * us, B, C)
    return (y + us * D[None, :, None]) * F.silu(z)


def reference_ssm_adaptive_preal_optimized(u: Tensor, dt: Tensor, x: Tensor, x_bias: Tensor, B: Tensor, C: Tensor,
                                           D: Tensor, z: Tensor) -> Tensor:
    """Name, signature and arithmetic of extension-cpp/extension_cpp/ops.py:465-510: the decay is
    exp((x.u_l + x_bias) dt_l) and the raw input enters (no silu).  Upstream evaluates it with cumulative sums
    of exp(-G), which overflow on long sequences; here it is the recurrence itself."""
    _preal_check(u, dt, x, B, C, D, z)
    log_a = (torch.einsum("ijr,brl->bijl", x, u) + x_bias[None, :, :, None]) * dt[:, :, None, :]
    y = _preal_scan(log_a, dt * u, B, C)
    return (y + u * D[None, :, None]) * F.silu(z)
