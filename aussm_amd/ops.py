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

How it maps onto the core scan kernel: dividing the state by the constant Bt_j is not needed --
instead every (batch, state) pair becomes one batch element of a core scan with ONE state per
channel: its phase is theta[b, j] (channels x time), its B_t and C_t are the constants Bt_j and
Ct_j, and the sum over j is taken afterwards.  The phase projection is a plain GEMM
(x as a (d n) x d matrix times u), done by the BLAS behind torch.matmul.  The backward operator
re-runs this composition under autograd, so its scan gradients come from the HIP reverse scan.
"""
from __future__ import annotations

from typing import Tuple

import torch
import torch.nn.functional as F
from torch import Tensor

from . import scan

__all__ = ["ssm_adaptive_unitary", "ssm_adaptive_interface", "pad_to_multiple_of"]

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


def _composite(u, dt, x, x_bias, B_r, B_theta, C_r, C_theta, D, z, h_r, h_i):
    """The operator as differentiable torch ops around ONE core-scan launch."""
    b, d, n, l = _check_op_inputs((u, dt, x, x_bias, B_r, B_theta, C_r, C_theta, D, z, h_r, h_i))
    # phase projection: theta[b, j, i, l]  (state index before channel so that (b, j) is a batch)
    xm = x.permute(1, 0, 2).reshape(n * d, d)                          # (j i) x r
    # one strided-batched GEMM straight into (b, (j i), l); the 2-D x 3-D form of matmul goes through
    # transposed copies of the whole phase tensor
    theta = torch.baddbmm(x_bias.t().reshape(1, n * d, 1), xm.unsqueeze(0).expand(b, n * d, d), u).view(b, n, d, l)
    us = F.silu(u)
    Bt = torch.polar(B_r, B_theta)                                     # (n,)
    Ct = torch.polar(C_r, C_theta)
    row = lambda c: c[None, :, None].expand(b, n, l).reshape(b * n, 1, l)
    h0 = torch.complex(h_r, h_i).permute(0, 2, 1).reshape(b * n, d, 1)
    # us, dt stay (b, d, l): each of their batch elements serves the n consecutive (batch, state) pairs
    y, hL = scan.unitary_scan(us, dt.contiguous(), theta.reshape(b * n, d, l), row(Bt), row(Ct), None, None, h0,
                              return_last_state=True)
    y = y.view(b, n, d, l).sum(dim=1)
    y = (y + us * D[None, :, None]) * F.silu(z)
    hL = hL.view(b, n, d).permute(0, 2, 1)
    return y, hL.real.contiguous(), hL.imag.contiguous()


# ---- dispatcher ops -------------------------------------------------------------------------

_lib = torch.library.Library(_NS, "FRAGMENT")
_lib.define(_FWD_SCHEMA)
_lib.define(_BWD_SCHEMA)


def _fwd_impl(u, dt, x, x_bias, B_r, B_theta, C_r, C_theta, D, z, h_r, h_i):
    with torch.no_grad():
        return _composite(u, dt, x, x_bias, B_r, B_theta, C_r, C_theta, D, z, h_r, h_i)


def _bwd_impl(grad_y, grad_hr, grad_hi, u, dt, x, x_bias, B_r, B_theta, C_r, C_theta, D, z, h_r, h_i):
    with torch.enable_grad():
        leaves = [t.detach().requires_grad_(True) for t in (u, dt, x, x_bias, B_r, B_theta, C_r, C_theta, D, z,
                                                              h_r, h_i)]
        outs = _composite(*leaves)
        grads = torch.autograd.grad(outs, leaves, [grad_y.contiguous(), grad_hr.contiguous(), grad_hi.contiguous()],
                                    allow_unused=True)
    return tuple(torch.zeros_like(t) if g is None else g.contiguous() for g, t in zip(grads, leaves))


_lib.impl("ssm_adaptive_unitary", _fwd_impl, "CUDA")
_lib.impl("ssm_adaptive_backward_unitary", _bwd_impl, "CUDA")


@torch.library.register_fake(f"{_NS}::ssm_adaptive_unitary")
def _fwd_fake(u, dt, x, x_bias, B_r, B_theta, C_r, C_theta, D, z, h_r, h_i):
    return torch.empty_like(u), torch.empty_like(h_r), torch.empty_like(h_i)


@torch.library.register_fake(f"{_NS}::ssm_adaptive_backward_unitary")
def _bwd_fake(grad_y, grad_hr, grad_hi, u, dt, x, x_bias, B_r, B_theta, C_r, C_theta, D, z, h_r, h_i):
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
        return torch.ops.extension_cpp.ssm_adaptive_backward_unitary.default(
            grad_y, grad_next_hidden_state_real, grad_next_hidden_state_imag, *saved)
    except RuntimeError:
        shapes = {k: tuple(t.shape) for k, t in zip(_INPUT_NAMES, saved)}
        shapes["grad_y"] = tuple(grad_y.shape)
        print(f"Runtime Error for {shapes}")
        raise


def setup_context_unitary(ctx, inputs, output):
    # like the reference (ops.py:148-151): only the 12 inputs are kept for the backward pass
    ctx.save_for_backward(*inputs)


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
                           max_parallel_length: int = 2048, save_intermediates: bool = True, **kwargs) -> Tensor:
    """Front-end of the adaptive-unitary operator (ops.py:28-93).

    u, dt, z: (b, d, l) float32; x: (d, n, d); x_bias: (d, n); B, C: (n,) complex64; D: (d,).
    B and C are given in the reference's parameterisation: radius = softplus(real part),
    phase = imaginary part.  The sequence is processed in launches of at most
    `max_parallel_length` steps with the complex state carried from launch to launch, starting
    from zero, exactly as the reference does; unknown keyword arguments are ignored as there.
    (The reference zero-pads the sequence to a multiple of 16 for its kernel; this kernel takes
    any length, and the padded steps never influence the returned y.)

    save_intermediates (not in the reference): True keeps the phase tensor (b, n, d, l) and the
    scan's checkpoints for the backward pass; False goes through the dispatcher operator, whose
    backward pass keeps only the twelve inputs and recomputes, as the reference's does
    (ops.py:148-151) - less memory, one more phase projection and forward scan per step.
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
