"""Core selective scans on MI355X: Python host over the C ABI of libaussm_hip.so.

Three operators, each differentiable through torch.autograd:

    unitary_scan(u, delta, theta, Bc, Cc, D, z, h0)        a_l = exp(i theta_l)
    complex_scan(u, delta, rho, theta, Bc, Cc, D, z, h0)   a_l = exp(rho_l + i theta_l)
    selective_scan_fn(u, delta, A, B, C, D, z, delta_bias, delta_softplus, return_last_state)
                                                            a_l = exp(delta_l A)   (Mamba S6)

    h_l[b,d,n] = a_l h_{l-1}[b,d,n] + delta_l[b,d] B_l[b,n] u_l[b,d]
    y_l[b,d]   = Re sum_n C_l[b,n] h_l[b,d,n] + D[d] u_l[b,d]          (* silu(z_l[b,d]))

selective_scan_fn keeps the argument names and meaning of the call at
ai-modules/wavesAI/model/aussm.py:791-802 of the reference; the unitary/complex
recurrences are those of extension-cpp/extension_cpp/ops.py:215-223 and :270-291.

Tensors must live on the GPU.  u, delta, B, C may be float32 or bfloat16 (both
the same); everything else is float32 and the state is accumulated in float32.
Complex B_t/C_t are torch.complex64 tensors (b, n, l) or, for bfloat16, real
tensors (b, n, l, 2) holding (re, im).
"""
from __future__ import annotations

from typing import Optional

import torch

from . import _lib
from ._lib import check, ptr

Tensor = torch.Tensor

# Checkpoint interval (timesteps) of the forward pass.  The unitary backward pass regenerates the
# states by running the recurrence in reverse and only uses checkpoints to stop rounding drift,
# so a long interval is enough; the complex and real backward passes recompute every tile from
# its checkpoint and need one per tile.
UNITARY_CK = 256
# ... and where the launch is not split along L nothing ties the interval to a segment length: measured
# against the float64 oracle the gradients do not change between an interval of 256 and one checkpoint at
# the end of 2048 or 8192 steps (the reverse recurrence is norm-preserving), so such a call keeps a
# checkpoint every UNITARY_CK_LONG steps only
UNITARY_CK_LONG = 4096


def unitary_ck(b: int, d: int, n: int, l: int) -> int:
    """Checkpoint interval of the unitary scan for a shape: UNITARY_CK, or half of it where that
    lets a launch with few (batch, channel) pairs be split into more segments along L (a segment
    is a whole number of checkpoint blocks); calls that are not split at all checkpoint every
    UNITARY_CK_LONG steps (one checkpoint, at the end, for shorter sequences)."""
    lib = _lib.load()
    half = UNITARY_CK // 2
    s_half, s_full = (lib.aussm_unitary_split_segments(b, d, n, l, ck) for ck in (half, UNITARY_CK))
    if s_half > s_full:
        return half
    if s_full <= 1:
        return min(UNITARY_CK_LONG, -(-l // _lib.TILE) * _lib.TILE)
    return UNITARY_CK
TILE_CK = _lib.TILE


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _in_dtype(t: Tensor) -> int:
    if t.dtype == torch.float32:
        return _lib.F32
    if t.dtype == torch.bfloat16:
        return _lib.BF16
    raise RuntimeError(f"expected float32 or bfloat16 scan input, got {t.dtype}")


def _f32(t: Optional[Tensor], name: str, shape=None) -> Optional[Tensor]:
    if t is None:
        return None
    if t.dtype != torch.float32:
        raise RuntimeError(f"expected {name} to be float32, got {t.dtype}")
    if shape is not None and tuple(t.shape) != tuple(shape):
        raise RuntimeError(f"expected {name} of shape {tuple(shape)}, got {tuple(t.shape)}")
    return t.contiguous()


def _check_bdl(u: Tensor, delta: Tensor):
    if u.dim() != 3:
        raise RuntimeError(f"expected u of shape (b, d, l), got {tuple(u.shape)}")
    if not u.is_cuda:
        raise RuntimeError("scan inputs must be on the GPU (no CPU implementation is shipped)")
    if delta.shape != u.shape or delta.dtype != u.dtype:
        raise RuntimeError("delta must match u in shape and dtype")
    return u.shape


def _complex_as_real(t: Tensor, name: str, b: int, l: int, dtype: torch.dtype) -> Tensor:
    """(b, n, l) complex64 or (b, n, l, 2) real -> contiguous real (b, n, l, 2) of `dtype`."""
    if t.is_complex():
        if t.dtype != torch.complex64:
            raise RuntimeError(f"expected {name} to be complex64, got {t.dtype}")
        t = torch.view_as_real(t)
    if t.dim() != 4 or t.shape[0] != b or t.shape[2] != l or t.shape[3] != 2:
        raise RuntimeError(f"expected {name} of shape (b, n, l) complex or (b, n, l, 2), got {tuple(t.shape)}")
    if t.dtype != dtype:
        raise RuntimeError(f"{name} must have the dtype of u ({dtype}), got {t.dtype}")
    return t.contiguous()


def num_checkpoints(L: int, ck: int) -> int:
    return (L + ck - 1) // ck


# --------------------------------------------------------------------------------------------
# raw launches (no autograd)
# --------------------------------------------------------------------------------------------

def unitary_aux(u, n: int, ck: int) -> Tensor:
    """The optional auxiliary buffer of the unitary scan for inputs shaped like u (b, d, l) with n
    states and checkpoint interval ck: the forward call may leave intermediate results in it that
    spare the backward call a recomputation, and a call that splits a long sequence over more
    workgroups keeps its segment states there."""
    lib = _lib.load()
    b, d, l = u.shape
    return torch.empty((lib.aussm_unitary_aux_floats(b, d, n, l, ck or _lib.TILE),), device=u.device,
                       dtype=torch.float32)


def unitary_aux_useful(b: int, d: int, n: int, l: int, ck: int, in_dtype: int, urep: int = 1) -> bool:
    """False when neither direction of the scan would touch an auxiliary buffer for this shape (the
    vector-ALU kernels use it only for the segment states of a call that is split along the sequence), so
    that the autograd wrapper does not allocate and keep a buffer for nothing."""
    lib = _lib.load()
    return bool(lib.aussm_unitary_kernel_mode(0, b, d, n, l, ck, in_dtype, urep, 1)
                or lib.aussm_unitary_kernel_mode(1, b, d, n, l, ck, in_dtype, urep, 1)
                or lib.aussm_unitary_split_segments(b, d, n, l, ck) > 1)


def unitary_fwd_raw(u, delta, theta, Bri, Cri, D=None, z=None, h0=None, want_state=False, ck=0, aux=None, ck_arg=0):
    """Launch aussm_unitary_fwd(_aux).  Bri/Cri are real views (b, n, l, 2).  Returns (y, hL, hck);
    hL is (b, d, n, 2) or None, hck is the checkpoint tensor when ck > 0.  u and delta may have a
    batch size that divides theta's: each of their batch elements then serves that many
    consecutive ones of theta."""
    lib = _lib.load()
    b, d, l = theta.shape
    urep = b // u.shape[0]
    n = Bri.shape[1]
    y = torch.empty((b, d, l), device=u.device, dtype=torch.float32)
    hL = torch.empty((b, d, n, 2), device=u.device, dtype=torch.float32) if want_state else None
    hck = None
    if ck:
        hck = torch.empty((b, num_checkpoints(l, ck), n, 2, d), device=u.device, dtype=torch.float32)
    check(lib.aussm_unitary_fwd_aux(ptr(u), ptr(delta), ptr(theta), ptr(Bri), ptr(Cri), ptr(D), ptr(z), ptr(h0),
                                    ptr(y), ptr(hL), ptr(hck), ptr(aux), b, d, n, l, ck or ck_arg or _lib.TILE, _in_dtype(u),
                                    urep, _stream()),
          "aussm_unitary_fwd_aux")
    return y, hL, hck


def unitary_bwd_raw(dy, dhL, u, delta, theta, Bri, Cri, D, hck, ck, want_dD=True, want_dh0=False, aux=None):
    """Gradients; du and ddelta come back per batch element of theta (b, d, l) also when u and delta
    are shared by several of them (the caller adds them up)."""
    lib = _lib.load()
    b, d, l = theta.shape
    urep = b // u.shape[0]
    n = Bri.shape[1]
    f32 = dict(device=u.device, dtype=torch.float32)
    du, ddelta, dtheta = (torch.empty((b, d, l), **f32) for _ in range(3))
    # accumulated into with atomics by the kernel: start from zero (one allocation, one fill launch; the pad keeps
    # every view 16-byte aligned)
    nbc = b * n * l * 2
    pad = (nbc + 3) // 4 * 4
    acc = torch.zeros((2 * pad + d,), **f32)
    dB, dC = acc[:nbc].view(b, n, l, 2), acc[pad:pad + nbc].view(b, n, l, 2)
    dD = acc[2 * pad:2 * pad + d] if (want_dD and D is not None) else None
    dh0 = torch.empty((b, d, n, 2), **f32) if want_dh0 else None
    check(lib.aussm_unitary_bwd_aux(ptr(dy), ptr(dhL), ptr(u), ptr(delta), ptr(theta), ptr(Bri), ptr(Cri), ptr(D),
                                    ptr(hck), ptr(aux), ptr(du), ptr(ddelta), ptr(dtheta), ptr(dB), ptr(dC), ptr(dD),
                                    ptr(dh0), b, d, n, l, ck, _in_dtype(u), urep, _stream()),
          "aussm_unitary_bwd_aux")
    return du, ddelta, dtheta, dB, dC, dD, dh0


# --------------------------------------------------------------------------------------------
# autograd
# --------------------------------------------------------------------------------------------

class _UnitaryScanFn(torch.autograd.Function):
    """y, hL = scan(u, delta, theta, B, C, D, h0) with all tensors real (complex ones as (..., 2))."""

    @staticmethod
    def forward(ctx, u, delta, theta, Bri, Cri, D, h0):
        ck = unitary_ck(theta.shape[0], theta.shape[1], Bri.shape[1], theta.shape[2])
        b, d, l = theta.shape
        n = Bri.shape[1]
        aux = unitary_aux(theta, n, ck) if unitary_aux_useful(b, d, n, l, ck, _in_dtype(u), b // u.shape[0]) else None
        y, hL, hck = unitary_fwd_raw(u, delta, theta, Bri, Cri, D, None, h0, want_state=True, ck=ck, aux=aux)
        ctx.save_for_backward(u, delta, theta, Bri, Cri, D, hck, aux)
        ctx.ck = ck
        ctx.has_h0 = h0 is not None
        return y, hL

    @staticmethod
    def backward(ctx, dy, dhL):
        u, delta, theta, Bri, Cri, D, hck, aux = ctx.saved_tensors
        dy = dy.contiguous()
        dhL = None if dhL is None else dhL.contiguous()
        du, ddelta, dtheta, dB, dC, dD, dh0 = unitary_bwd_raw(
            dy, dhL, u, delta, theta, Bri, Cri, D, hck, ctx.ck,
            want_dD=D is not None and ctx.needs_input_grad[5], want_dh0=ctx.has_h0 and ctx.needs_input_grad[6],
            aux=aux)
        if u.shape[0] != theta.shape[0]:             # u, delta shared by consecutive batch elements
            du = du.view(u.shape[0], -1, *u.shape[1:]).sum(dim=1)
            ddelta = ddelta.view(u.shape[0], -1, *u.shape[1:]).sum(dim=1)
        return (du.to(u.dtype), ddelta.to(delta.dtype), dtheta, dB.to(Bri.dtype), dC.to(Cri.dtype), dD, dh0)


class _GateFn(torch.autograd.Function):
    """y = y_pre silu(z) behind the unitary scan, whose backward kernels take the gradient of the ungated output:
    one pass forward, one backward (dy_pre = dy silu(z), dz = dy y_pre silu'(z)); reference
    extension-cpp/extension_cpp/ops.py:226."""

    @staticmethod
    def forward(ctx, y_pre, z):
        lib = _lib.load()
        y_pre = y_pre.contiguous()
        y = torch.empty_like(y_pre)
        check(lib.aussm_gate_fwd(ptr(y_pre), ptr(z), ptr(y), y_pre.numel(), _stream()), "aussm_gate_fwd")
        ctx.save_for_backward(y_pre, z)
        return y

    @staticmethod
    def backward(ctx, dy):
        lib = _lib.load()
        y_pre, z = ctx.saved_tensors
        dy = dy.contiguous()
        dy_pre, dz = torch.empty_like(y_pre), torch.empty_like(z)
        check(lib.aussm_gate_bwd(ptr(dy), ptr(y_pre), ptr(z), ptr(dy_pre), ptr(dz), dy.numel(), _stream()), "aussm_gate_bwd")
        return dy_pre, dz


def unitary_scan(u: Tensor, delta: Tensor, theta: Tensor, Bc: Tensor, Cc: Tensor, D: Optional[Tensor] = None,
                 z: Optional[Tensor] = None, h0: Optional[Tensor] = None, return_last_state: bool = False):
    """Adaptive-unitary scan.  u, delta, theta, z: (b, d, l); Bc, Cc: (b, n, l) complex64 (or
    (b, n, l, 2) real); D: (d,); h0: (b, d, n) complex64.  Returns y (b, d, l) float32, and the final
    state (b, d, n) complex64 if return_last_state.  u and delta may be (b / r, d, l): batch element i
    of theirs then serves the r consecutive batch elements i r .. i r + r - 1 of everything else
    (one input, r phase sequences)."""
    bu, d, l = _check_bdl(u, delta)
    u = u.contiguous()
    delta = delta.contiguous()
    b = theta.shape[0] if theta.dim() == 3 else bu
    if b % bu != 0:
        raise RuntimeError(f"batch size of theta ({b}) must be a multiple of that of u ({bu})")
    theta = _f32(theta, "theta", (b, d, l))
    Bri = _complex_as_real(Bc, "B", b, l, u.dtype)
    Cri = _complex_as_real(Cc, "C", b, l, u.dtype)
    n = Bri.shape[1]
    if Cri.shape[1] != n:
        raise RuntimeError("B and C must have the same state size")
    D = _f32(D, "D", (d,))
    z = _f32(z, "z", (b, d, l))
    h0r = None
    if h0 is not None:
        if h0.dtype != torch.complex64 or tuple(h0.shape) != (b, d, n):
            raise RuntimeError(f"expected h0 complex64 of shape {(b, d, n)}")
        h0r = torch.view_as_real(h0).contiguous()
    needs_grad = torch.is_grad_enabled() and any(
        t is not None and t.requires_grad for t in (u, delta, theta, Bri, Cri, D, z, h0r))
    if needs_grad:
        y, hL = _UnitaryScanFn.apply(u, delta, theta, Bri, Cri, D, h0r)
        if z is not None:
            y = _GateFn.apply(y, z)
    else:
        # no backward pass: the auxiliary buffer serves as workspace only (prepared operands of the
        # matrix-core kernels, segment states of a launch that is split along L); no checkpoints are kept
        lib = _lib.load()
        ck = unitary_ck(b, d, n, l)
        # (the buffer of a shape that the matrix-core kernels serve starts with b d l floats that only a backward
        # call would read; anything beyond them - segment states, operand images - is workspace of this call)
        work = lib.aussm_unitary_aux_floats(b, d, n, l, ck) - _lib.AUX_PAD not in (0, b * d * l)
        aux = unitary_aux(theta, n, ck) if (work and u.shape[0] == b) else None
        y, hL, _ = unitary_fwd_raw(u, delta, theta, Bri, Cri, D, z, h0r, want_state=return_last_state,
                                   ck=0, aux=aux, ck_arg=ck if aux is not None else 0)
    if return_last_state:
        return y, torch.view_as_complex(hL)
    return y


# --------------------------------------------------------------------------------------------
# complex scan
# --------------------------------------------------------------------------------------------

REC_CK = 16          # checkpoint interval the recomputing backward kernels (complex, real) need
REC_MAX_STATE = _lib.MAX_STATE   # largest state size those kernels take (16 states per launch, one launch per block)


def _scan_workspace(variant: int, u: Tensor, n: int, ck: int) -> Optional[Tensor]:
    """Workspace of a complex / real call for inputs shaped like u (aussm_scan_workspace_floats): segment
    states that let a call with few (batch, channel group) pairs split along the sequence, and the float
    copies of bfloat16 B_t / C_t.  None when the call needs neither."""
    b, d, l = u.shape
    floats = _lib.load().aussm_scan_workspace_floats(variant, b, d, n, l, ck, _in_dtype(u))
    return torch.empty((floats,), device=u.device, dtype=torch.float32) if floats else None


def complex_fwd_raw(u, delta, rho, theta, Bri, Cri, D=None, z=None, h0=None, want_state=False, ck=0):
    lib = _lib.load()
    b, d, l = u.shape
    n = Bri.shape[1]
    y = torch.empty((b, d, l), device=u.device, dtype=torch.float32)
    hL = torch.empty((b, d, n, 2), device=u.device, dtype=torch.float32) if want_state else None
    hck = torch.empty((b, num_checkpoints(l, ck), n, 2, d), device=u.device, dtype=torch.float32) if ck else None
    ws = _scan_workspace(_lib.VAR_COMPLEX, u, n, ck or _lib.TILE)
    check(lib.aussm_complex_fwd(ptr(u), ptr(delta), ptr(rho), ptr(theta), ptr(Bri), ptr(Cri), ptr(D), ptr(z),
                                ptr(h0), ptr(y), ptr(hL), ptr(hck), ptr(ws), b, d, n, l, ck or _lib.TILE,
                                _in_dtype(u), _stream()), "aussm_complex_fwd")
    return y, hL, hck


def complex_bwd_raw(dy, dhL, u, delta, rho, theta, Bri, Cri, D, h0, hck, want_dD=True, want_dh0=False, z=None):
    lib = _lib.load()
    b, d, l = u.shape
    n = Bri.shape[1]
    f32 = dict(device=u.device, dtype=torch.float32)
    du, ddelta, drho, dtheta = (torch.empty((b, d, l), **f32) for _ in range(4))
    dB = torch.zeros((b, n, l, 2), **f32)
    dC = torch.zeros((b, n, l, 2), **f32)
    dD = torch.zeros((d,), **f32) if (want_dD and D is not None) else None
    dh0 = torch.empty((b, d, n, 2), **f32) if want_dh0 else None
    dz = torch.empty((b, d, l), **f32) if z is not None else None
    ws = _scan_workspace(_lib.VAR_COMPLEX, u, n, REC_CK)
    check(lib.aussm_complex_bwd(ptr(dy), ptr(dhL), ptr(u), ptr(delta), ptr(rho), ptr(theta), ptr(Bri), ptr(Cri),
                                ptr(D), ptr(h0), ptr(hck), ptr(du), ptr(ddelta), ptr(drho), ptr(dtheta), ptr(dB),
                                ptr(dC), ptr(dD), ptr(dh0), ptr(z), ptr(dz), ptr(ws), b, d, n, l, REC_CK,
                                _in_dtype(u), _stream()), "aussm_complex_bwd")
    return du, ddelta, drho, dtheta, dB, dC, dD, dh0, dz


class _ComplexScanFn(torch.autograd.Function):
    """The gate z (optional) is applied by the forward kernel and differentiated by the backward kernel."""

    @staticmethod
    def forward(ctx, u, delta, rho, theta, Bri, Cri, D, h0, z):
        y, hL, hck = complex_fwd_raw(u, delta, rho, theta, Bri, Cri, D, z, h0, want_state=True, ck=REC_CK)
        ctx.save_for_backward(u, delta, rho, theta, Bri, Cri, D, h0, hck, z)
        return y, hL

    @staticmethod
    def backward(ctx, dy, dhL):
        u, delta, rho, theta, Bri, Cri, D, h0, hck, z = ctx.saved_tensors
        dhL = None if dhL is None else dhL.contiguous()
        du, ddelta, drho, dtheta, dB, dC, dD, dh0, dz = complex_bwd_raw(
            dy.contiguous(), dhL, u, delta, rho, theta, Bri, Cri, D, h0, hck,
            want_dD=D is not None and ctx.needs_input_grad[6], want_dh0=h0 is not None and ctx.needs_input_grad[7], z=z)
        return (du.to(u.dtype), ddelta.to(delta.dtype), drho, dtheta, dB.to(Bri.dtype), dC.to(Cri.dtype), dD, dh0, dz)


def complex_scan(u: Tensor, delta: Tensor, rho: Tensor, theta: Tensor, Bc: Tensor, Cc: Tensor,
                 D: Optional[Tensor] = None, z: Optional[Tensor] = None, h0: Optional[Tensor] = None,
                 return_last_state: bool = False):
    """Complex scan, a_l = exp(rho_l + i theta_l).  Shapes as unitary_scan plus rho (b, d, l)."""
    b, d, l = _check_bdl(u, delta)
    u = u.contiguous()
    delta = delta.contiguous()
    rho = _f32(rho, "rho", (b, d, l))
    theta = _f32(theta, "theta", (b, d, l))
    Bri = _complex_as_real(Bc, "B", b, l, u.dtype)
    Cri = _complex_as_real(Cc, "C", b, l, u.dtype)
    n = Bri.shape[1]
    if Cri.shape[1] != n:
        raise RuntimeError("B and C must have the same state size")
    D = _f32(D, "D", (d,))
    z = _f32(z, "z", (b, d, l))
    h0r = None
    if h0 is not None:
        if h0.dtype != torch.complex64 or tuple(h0.shape) != (b, d, n):
            raise RuntimeError(f"expected h0 complex64 of shape {(b, d, n)}")
        h0r = torch.view_as_real(h0).contiguous()
    needs_grad = torch.is_grad_enabled() and any(
        t is not None and t.requires_grad for t in (u, delta, rho, theta, Bri, Cri, D, z, h0r))
    if needs_grad:
        if n > REC_MAX_STATE:
            raise RuntimeError(f"the complex backward pass supports at most {REC_MAX_STATE} states per channel")
        y, hL = _ComplexScanFn.apply(u, delta, rho, theta, Bri, Cri, D, h0r, z)
    else:
        y, hL, _ = complex_fwd_raw(u, delta, rho, theta, Bri, Cri, D, z, h0r, want_state=return_last_state)
    if return_last_state:
        return y, torch.view_as_complex(hL)
    return y


# --------------------------------------------------------------------------------------------
# real (Mamba S6) selective scan
# --------------------------------------------------------------------------------------------

def real_fwd_raw(u, delta, A, Bm, Cm, D=None, z=None, delta_bias=None, delta_softplus=False, h0=None,
                 want_state=False, ck=0):
    lib = _lib.load()
    b, d, l = u.shape
    n = A.shape[1]
    y = torch.empty((b, d, l), device=u.device, dtype=torch.float32)
    hL = torch.empty((b, d, n), device=u.device, dtype=torch.float32) if want_state else None
    hck = torch.empty((b, num_checkpoints(l, ck), n, 1, d), device=u.device, dtype=torch.float32) if ck else None
    ws = _scan_workspace(_lib.VAR_REAL, u, n, ck or _lib.TILE)
    check(lib.aussm_real_fwd(ptr(u), ptr(delta), ptr(A), ptr(Bm), ptr(Cm), ptr(D), ptr(z), ptr(delta_bias),
                             int(bool(delta_softplus)), ptr(h0), ptr(y), ptr(hL), ptr(hck), ptr(ws), b, d, n, l,
                             ck or _lib.TILE, _in_dtype(u), _stream()), "aussm_real_fwd")
    return y, hL, hck


def real_bwd_raw(dy, dhL, u, delta, A, Bm, Cm, D, delta_bias, delta_softplus, h0, hck, want_dD=True,
                 want_dh0=False, z=None):
    lib = _lib.load()
    b, d, l = u.shape
    n = A.shape[1]
    f32 = dict(device=u.device, dtype=torch.float32)
    du, ddelta = torch.empty((b, d, l), **f32), torch.empty((b, d, l), **f32)
    dA = torch.zeros((d, n), **f32)
    dB = torch.zeros((b, n, l), **f32)
    dC = torch.zeros((b, n, l), **f32)
    dD = torch.zeros((d,), **f32) if (want_dD and D is not None) else None
    dh0 = torch.empty((b, d, n), **f32) if want_dh0 else None
    dz = torch.empty((b, d, l), **f32) if z is not None else None
    ws = _scan_workspace(_lib.VAR_REAL, u, n, REC_CK)
    check(lib.aussm_real_bwd(ptr(dy), ptr(dhL), ptr(u), ptr(delta), ptr(A), ptr(Bm), ptr(Cm), ptr(D),
                             ptr(delta_bias), int(bool(delta_softplus)), ptr(h0), ptr(hck), ptr(du), ptr(ddelta),
                             ptr(dA), ptr(dB), ptr(dC), ptr(dD), ptr(dh0), ptr(z), ptr(dz), ptr(ws), b, d, n, l, REC_CK,
                             _in_dtype(u), _stream()), "aussm_real_bwd")
    return du, ddelta, dA, dB, dC, dD, dh0, dz


class _RealScanFn(torch.autograd.Function):
    """The gate z (optional) is applied by the forward kernel and differentiated by the backward kernel."""

    @staticmethod
    def forward(ctx, u, delta, A, Bm, Cm, D, delta_bias, h0, delta_softplus, z):
        y, hL, hck = real_fwd_raw(u, delta, A, Bm, Cm, D, z, delta_bias, delta_softplus, h0,
                                  want_state=True, ck=REC_CK)
        ctx.save_for_backward(u, delta, A, Bm, Cm, D, delta_bias, h0, hck, z)
        ctx.delta_softplus = delta_softplus
        return y, hL

    @staticmethod
    def backward(ctx, dy, dhL):
        u, delta, A, Bm, Cm, D, delta_bias, h0, hck, z = ctx.saved_tensors
        dhL = None if dhL is None else dhL.contiguous()
        du, ddelta, dA, dB, dC, dD, dh0, dz = real_bwd_raw(
            dy.contiguous(), dhL, u, delta, A, Bm, Cm, D, delta_bias, ctx.delta_softplus, h0, hck,
            want_dD=D is not None and ctx.needs_input_grad[5], want_dh0=h0 is not None and ctx.needs_input_grad[7], z=z)
        dbias = ddelta.sum(dim=(0, 2)) if (delta_bias is not None and ctx.needs_input_grad[6]) else None
        return (du.to(u.dtype), ddelta.to(delta.dtype), dA, dB.to(Bm.dtype), dC.to(Cm.dtype), dD, dbias, dh0, None, dz)


def selective_scan_fn(u: Tensor, delta: Tensor, A: Tensor, B: Tensor, C: Tensor, D: Optional[Tensor] = None,
                      z: Optional[Tensor] = None, delta_bias: Optional[Tensor] = None,
                      delta_softplus: bool = False, return_last_state: bool = False,
                      h0: Optional[Tensor] = None):
    """Mamba S6 selective scan with the argument names and meaning of the reference's call
    (ai-modules/wavesAI/model/aussm.py:791-802):

        u, delta, z: (b, d, l); A: (d, n) float32; B, C: (b, n, l); D, delta_bias: (d,) float32.
        delta <- softplus(delta + delta_bias) if delta_softplus (bias alone if not);
        h_l = exp(delta_l A) h_{l-1} + delta_l B_l u_l;  y_l = C_l . h_l + D u_l;  y *= silu(z).

    Returns y (b, d, l) float32, plus the last state (b, d, n) if return_last_state.
    `h0` (b, d, n), a start state, is an extension over the reference's signature."""
    b, d, l = _check_bdl(u, delta)
    u = u.contiguous()
    delta = delta.contiguous()
    A = _f32(A, "A")
    if A.dim() != 2 or A.shape[0] != d:
        raise RuntimeError(f"expected A of shape (d, n) with d = {d}, got {tuple(A.shape)}")
    n = A.shape[1]
    for name, t in (("B", B), ("C", C)):
        if tuple(t.shape) != (b, n, l):
            raise RuntimeError(f"expected {name} of shape {(b, n, l)}, got {tuple(t.shape)}")
        if t.dtype != u.dtype:
            raise RuntimeError(f"{name} must have the dtype of u ({u.dtype}), got {t.dtype}")
    Bm, Cm = B.contiguous(), C.contiguous()
    D = _f32(D, "D", (d,))
    z = _f32(z, "z", (b, d, l))
    delta_bias = _f32(delta_bias, "delta_bias", (d,))
    h0 = _f32(h0, "h0", (b, d, n))
    needs_grad = torch.is_grad_enabled() and any(
        t is not None and t.requires_grad for t in (u, delta, A, Bm, Cm, D, z, delta_bias, h0))
    if needs_grad:
        if n > REC_MAX_STATE:
            raise RuntimeError(f"the S6 backward pass supports at most {REC_MAX_STATE} states per channel")
        y, hL = _RealScanFn.apply(u, delta, A, Bm, Cm, D, delta_bias, h0, bool(delta_softplus), z)
    else:
        y, hL, _ = real_fwd_raw(u, delta, A, Bm, Cm, D, z, delta_bias, delta_softplus, h0,
                                want_state=return_last_state)
    if return_last_state:
        return y, hL
    return y
