"""Depthwise causal convolution along the sequence on channels-last tensors, the step the blocks
apply to the scan's input (`self.conv1d(x)[:, :, :l]`, ai-modules/wavesAI/model/aussm.py:762 and
:863), as HIP kernels behind the C ABI (aussm_causal_conv1d_fwd / _bwd).

    y[b, l, d] = bias[d] + sum_k weight[d, 0, k] * x[b, l - (K - 1) + k, d]

The blocks hold x as (b, l, d); the reference transposes to (b, d, l) for nn.Conv1d and back.
Here the kernels read the (b, l, d) data in place (a column slice of a wider tensor included).
"""
from __future__ import annotations

from typing import Optional

import torch
from torch import Tensor

from . import _lib
from ._lib import check, ptr

__all__ = ["causal_conv1d", "swap_last2"]


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _rows(x: Tensor):
    """x usable in place: float32, channel stride 1, rows that do not overlap."""
    b, l, d = x.shape
    if x.dtype != torch.float32 or x.stride(2) != 1 or x.stride(1) < d or x.stride(0) < (l - 1) * x.stride(1) + d:
        x = x.float().contiguous()
    return x


class _CausalConv1dFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, weight, bias):
        lib = _lib.load()
        b, l, d = x.shape
        k = weight.shape[-1]
        xr = _rows(x)
        w = weight.reshape(d, k).float().contiguous()
        bs = None if bias is None else bias.float().contiguous()
        y = torch.empty((b, l, d), device=x.device, dtype=torch.float32)
        check(lib.aussm_causal_conv1d_fwd(ptr(xr), ptr(w), ptr(bs), ptr(y), b, l, d, k, xr.stride(0), xr.stride(1),
                                          _stream()), "aussm_causal_conv1d_fwd")
        ctx.save_for_backward(xr, w)
        ctx.has_bias = bias is not None
        ctx.wshape = weight.shape
        return y

    @staticmethod
    def backward(ctx, dy):
        lib = _lib.load()
        xr, w = ctx.saved_tensors
        b, l, d = xr.shape
        k = w.shape[1]
        dy = dy.float().contiguous()
        dx = torch.empty((b, l, d), device=dy.device, dtype=torch.float32)
        dw = torch.zeros((d, k), device=dy.device, dtype=torch.float32)     # accumulated into by the kernel
        db = torch.zeros((d,), device=dy.device, dtype=torch.float32) if ctx.has_bias else None
        check(lib.aussm_causal_conv1d_bwd(ptr(dy), ptr(xr), ptr(w), ptr(dx), ptr(dw), ptr(db), b, l, d, k,
                                          xr.stride(0), xr.stride(1), _stream()), "aussm_causal_conv1d_bwd")
        return dx, dw.reshape(ctx.wshape), db


def causal_conv1d(x: Tensor, weight: Tensor, bias: Optional[Tensor] = None) -> Tensor:
    """x (b, l, d) on the GPU; weight (d, 1, k) or (d, k) as nn.Conv1d(d, d, k, groups=d) holds it;
    bias (d,) or None.  Returns (b, l, d) float32."""
    if x.dim() != 3 or not x.is_cuda:
        raise ValueError("causal_conv1d expects a (b, l, d) tensor on the GPU")
    if weight.shape[0] != x.shape[2] or weight.numel() != x.shape[2] * weight.shape[-1]:
        raise ValueError(f"weight {tuple(weight.shape)} does not fit {x.shape[2]} channels")
    return _CausalConv1dFn.apply(x, weight, bias)


class _SwapLast2Fn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x):
        return _swap_last2(x)

    @staticmethod
    def backward(ctx, dy):
        return _swap_last2(dy)


def _swap_last2(x: Tensor) -> Tensor:
    lib = _lib.load()
    b, r, c = x.shape
    xr = _rows(x)
    y = torch.empty((b, c, r), device=x.device, dtype=torch.float32)
    check(lib.aussm_swap_last2(ptr(xr), ptr(y), b, r, c, xr.stride(0), xr.stride(1), _stream()), "aussm_swap_last2")
    return y


_ACTS = {"silu": 1, "softplus": 2}


class _SwapActFn(torch.autograd.Function):
    """swap_last2 with the elementwise step done in the same pass, both directions."""

    @staticmethod
    def forward(ctx, x, bias, act):
        lib = _lib.load()
        b, r, c = x.shape
        xr = _rows(x)
        bs = None if bias is None else bias.float().contiguous()
        y = torch.empty((b, c, r), device=x.device, dtype=torch.float32)
        check(lib.aussm_swap_last2_act(ptr(xr), ptr(bs), None, ptr(y), b, r, c, xr.stride(0), xr.stride(1), 0, 0,
                                       act, 0, _stream()), "aussm_swap_last2_act")
        ctx.save_for_backward(xr, bs)
        ctx.act = act
        return y

    @staticmethod
    def backward(ctx, dy):
        lib = _lib.load()
        xr, bs = ctx.saved_tensors
        b, r, c = xr.shape
        dy = dy.float().contiguous()                    # (b, c, r)
        dx = torch.empty((b, r, c), device=dy.device, dtype=torch.float32)
        check(lib.aussm_swap_last2_act(ptr(dy), ptr(bs), ptr(xr), ptr(dx), b, c, r, dy.stride(0), dy.stride(1),
                                       xr.stride(0), xr.stride(1), ctx.act, 1, _stream()), "aussm_swap_last2_act")
        dbias = dx.sum((0, 1)) if (bs is not None and ctx.needs_input_grad[1]) else None
        return dx, dbias, None


def swap_last2(x: Tensor, act: Optional[str] = None, bias: Optional[Tensor] = None) -> Tensor:
    """Contiguous (b, c, r) copy of x (b, r, c) on the GPU: `x.transpose(1, 2).contiguous()` between
    the blocks' (b, l, d) activations and the scans' (b, d, l) tensors, through LDS tiles.
    act ("silu" or "softplus") with an optional per-channel bias (c,): the copy holds
    act(x + bias) instead, computed (and differentiated) in the same pass."""
    if x.dim() != 3 or not x.is_cuda:
        raise ValueError("swap_last2 expects a (b, r, c) tensor on the GPU")
    if act is None:
        if bias is not None:
            raise ValueError("a bias needs an activation")
        if x.shape[0] > 65535:
            return x.transpose(1, 2).contiguous()
        return _SwapLast2Fn.apply(x)
    if act not in _ACTS:
        raise ValueError(f"unknown activation {act!r}")
    if x.shape[0] > 65535 or x.dtype != torch.float32:
        v = x if bias is None else x + bias
        return (torch.nn.functional.silu(v) if act == "silu" else torch.nn.functional.softplus(v)).transpose(1, 2).contiguous()
    return _SwapActFn.apply(x, bias, _ACTS[act])
