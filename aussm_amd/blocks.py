"""The callers of the scan operators: counterparts of the reference's blocks in
ai-modules/wavesAI/model/aussm.py, with the scans running on the HIP kernels.

    ModelArgsSSMau (:35-62)   ModelArgsMamba (:64-91)   ModelBlockArgs (:94-97)
    SSMauBlock (:808-902)     MambaBlock (:717-805)     ResidualBlock (:681-714)
    RMSNorm (:905-916)        SSMTS (:100-227)

The modules keep the reference's parameter names, shapes, creation order and initialisers, so a
given torch.manual_seed produces the same initial weights and a reference state_dict loads
unchanged.  Behaviour kept on purpose: the dt_proj bias is added twice in SSMauBlock (:878-880)
and is passed again as delta_bias in MambaBlock (:789-802); the xA_proj weight is reshaped
"(n d1) d -> d1 n d" and scaled by 1/sqrt(d_model) (:882-891); conv1d output is trimmed to the
input length (:863).

Every block takes an optional `scan_impl` callable.  The default is the HIP operator; tests
pass a CPU implementation with the same signature to check the plumbing around the scan.
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Callable, List, Optional, Union

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import conv, ops, scan


def _causal_conv(conv1d: nn.Conv1d, x: torch.Tensor, l: int) -> torch.Tensor:
    """`conv1d(x^T)[:, :, :l]^T` of ai-modules/wavesAI/model/aussm.py:762 / :863 for x (b, l, d).
    On the GPU the HIP kernel reads x where it lies; tensors on the CPU (the blocks are also used
    there, with an injected scan) go through nn.Conv1d itself."""
    k = conv1d.kernel_size[0]
    if x.is_cuda and conv1d.groups == conv1d.in_channels == conv1d.out_channels and conv1d.padding[0] == k - 1:
        return conv.causal_conv1d(x, conv1d.weight, conv1d.bias)
    return conv1d(x.transpose(1, 2))[:, :, :l].transpose(1, 2)


class _LinearFn(torch.autograd.Function):
    """`F.linear` whose weight gradient is formed in slices of the (batch x length) rows.  The blocks' weight
    gradients are products with a short result (at most 1024 x 512) and a very long sum (b l = 23040 rows for the
    (32, 720) batches of the time-series model): as ONE product the library GEMM runs them on a few dozen workgroups
    (measured on an MI355X: 310 us for 1024 x 256, 12 GFLOP); as a batch of `_WGRAD_SLICES` products over slices of the
    rows, summed afterwards, the same result takes 100 us and carries a third of the rounding error."""

    @staticmethod
    def forward(ctx, x, weight, bias):
        ctx.save_for_backward(x, weight)
        ctx.has_bias = bias is not None
        return F.linear(x, weight, bias)

    @staticmethod
    def backward(ctx, dy):
        x, weight = ctx.saved_tensors
        n, m = weight.shape
        dx = dw = db = None
        if ctx.needs_input_grad[0]:
            dx = dy @ weight
        d2 = dy.reshape(-1, n)
        if ctx.needs_input_grad[1]:
            x2 = x.reshape(-1, m)
            s = _WGRAD_SLICES
            dw = torch.bmm(d2.reshape(s, -1, n).transpose(1, 2), x2.reshape(s, -1, m)).sum(0)
        if ctx.has_bias and ctx.needs_input_grad[2]:
            db = d2.sum(0)
        return dx, dw, db


_WGRAD_SLICES = 8
_WGRAD_MIN_ROWS = 4096


def _linear(layer: nn.Linear, x: torch.Tensor) -> torch.Tensor:
    """`layer(x)`; on the GPU, for inputs of many rows, with the weight gradient of `_LinearFn`."""
    rows = x.numel() // max(x.shape[-1], 1)
    if (x.is_cuda and x.dtype == torch.float32 and layer.weight.dtype == torch.float32 and rows >= _WGRAD_MIN_ROWS
            and rows % _WGRAD_SLICES == 0 and torch.is_grad_enabled() and layer.weight.requires_grad):
        return _LinearFn.apply(x, layer.weight, layer.bias)
    return layer(x)


def _swap_act(x: torch.Tensor, act: str, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """`_swap(act(x + bias))` in one pass on the GPU (the elementwise step rides on the layout change)."""
    if x.is_cuda and x.dtype == torch.float32:
        return conv.swap_last2(x, act=act, bias=bias)
    v = x if bias is None else x + bias
    return _swap(F.silu(v) if act == "silu" else F.softplus(v))


def _swap(x: torch.Tensor) -> torch.Tensor:
    """Contiguous copy with the last two dimensions swapped: (b, l, d) <-> (b, d, l), the
    `rearrange` calls around the scans (ai-modules/wavesAI/model/aussm.py:760-803, :861-900)."""
    if x.is_cuda and x.dtype == torch.float32:
        return conv.swap_last2(x)
    return x.transpose(1, 2).contiguous()


@dataclass
class ModelArgsSSMau:
    d_model: int
    d_state: int
    dt_rank: Union[int, str] = "auto"
    d_conv: int = 4
    conv_bias: bool = True
    bias: bool = False
    verbose: bool = False
    conv_1d: bool = True
    cuda: bool = True

    def __post_init__(self):
        self.block = SSMauBlock
        if self.dt_rank == "auto":
            self.dt_rank = self.d_state


@dataclass
class ModelArgsMamba:
    d_model: int
    d_state: int = 16
    expand: int = 2
    dt_rank: Union[int, str] = "auto"
    d_conv: int = 4
    conv_bias: bool = True
    bias: bool = False
    verbose: bool = False

    def __post_init__(self):
        self.block = MambaBlock
        self.d_inner = int(self.expand * self.d_model)
        if self.dt_rank == "auto":
            self.dt_rank = math.ceil(self.d_model / 16)


@dataclass
class ModelBlockArgs:
    layers: List[Union[ModelArgsSSMau, ModelArgsMamba]]
    d_model: int


class RMSNorm(nn.Module):
    def __init__(self, d_model: int, eps: float = 1e-5):
        super().__init__()
        self.eps = eps
        self.weight = nn.Parameter(torch.ones(d_model))

    def forward(self, x):
        # x * rsqrt(mean(x^2) + eps) * weight (ai-modules/wavesAI/model/aussm.py:905-916) as torch's fused op
        return F.rms_norm(x, (x.shape[-1],), self.weight, self.eps)


class MambaBlock(nn.Module):
    """A Mamba (S6) block; the scan is selective_scan_fn on the HIP real-scan kernels."""

    def __init__(self, args: ModelArgsMamba, scan_impl: Optional[Callable] = None):
        super().__init__()
        self.args = args
        self.in_proj = nn.Linear(args.d_model, args.d_inner * 2, bias=args.bias)
        self.conv1d = nn.Conv1d(in_channels=args.d_inner, out_channels=args.d_inner, bias=args.conv_bias,
                                kernel_size=args.d_conv, groups=args.d_inner, padding=args.d_conv - 1)
        self.out_proj = nn.Linear(args.d_inner, args.d_model, bias=args.bias)
        self.x_proj = nn.Linear(args.d_inner, args.dt_rank + args.d_state * 2, bias=False)
        self.dt_proj = nn.Linear(args.dt_rank, args.d_inner, bias=True)
        self.D = nn.Parameter(torch.ones(args.d_inner))
        A = torch.arange(1, args.d_state + 1, dtype=torch.float32).repeat(args.d_inner, 1)
        self.A_log = nn.Parameter(torch.log(A))
        self.A_log._no_weight_decay = True
        self.scan_impl = scan_impl or scan.selective_scan_fn

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        (b, l, d) = x.shape
        x_and_z = _linear(self.in_proj, x)
        (x, z) = x_and_z.split(split_size=[self.args.d_inner, self.args.d_inner], dim=-1)
        x = _causal_conv(self.conv1d, x, l)
        y = self.ssm_mamba(x, z)
        return _linear(self.out_proj, y)

    def ssm_mamba(self, x, z):
        (b, l, d_in) = x.shape
        x_proj = _linear(self.x_proj, x)
        dt, B, C = x_proj.split([self.args.dt_rank, self.args.d_state, self.args.d_state], dim=-1)
        dt = _linear(self.dt_proj, dt)
        A = -torch.exp(self.A_log.float())
        y = self.scan_impl(
            _swap_act(x, "silu"),                       # x = F.silu(x), aussm.py:787
            _swap(dt),
            A.contiguous(),
            _swap(B),
            _swap(C),
            self.D.float().contiguous(),
            z=_swap(z),
            delta_bias=self.dt_proj.bias.float(),
            delta_softplus=True,
            return_last_state=False,
        )
        return _swap(y)


class SSMauBlock(nn.Module):
    """A single AUSSM block; the scan is ssm_adaptive_interface on the HIP unitary-scan kernels."""

    def __init__(self, args: ModelArgsSSMau, scan_impl: Optional[Callable] = None):
        super().__init__()
        self.args = args
        self.in_proj = nn.Linear(args.d_model, args.d_model * 2, bias=args.bias)
        self.conv1d = nn.Conv1d(in_channels=args.d_model, out_channels=args.d_model, bias=args.conv_bias,
                                kernel_size=args.d_conv, groups=args.d_model, padding=args.d_conv - 1)
        self.out_proj = nn.Linear(args.d_model, args.d_model, bias=args.bias)
        self.x_proj = nn.Linear(args.d_model, args.dt_rank, bias=False)
        self.dt_proj = nn.Linear(args.dt_rank, args.d_model, bias=True)
        self.D = nn.Parameter(torch.ones(args.d_model))
        self.C = nn.Parameter(torch.randn(args.d_state, dtype=torch.complex64), requires_grad=True)
        self.B = nn.Parameter(torch.randn(args.d_state, dtype=torch.complex64), requires_grad=True)
        self.xA_proj = nn.Linear(args.d_model, args.d_model * args.d_state, bias=True)
        self.xA_proj.bias.data.uniform_(-torch.pi, torch.pi)
        if scan_impl is not None:
            self.optimized_SSMa_function = scan_impl
        elif args.cuda:
            self.optimized_SSMa_function = lambda **kw: ops.ssm_adaptive_interface(**kw, unitary=True)
        else:
            # the reference's pure-PyTorch form (aussm.py:842-843): same name, same signature, HIP kernels
            self.optimized_SSMa_function = ops.reference_ssm_adaptive_unitary_optimized_polar

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        (b, l, d) = x.shape
        x_and_z = _linear(self.in_proj, x)
        (x, z) = x_and_z.split(split_size=[self.args.d_model, self.args.d_model], dim=-1)
        if self.args.conv_1d:
            x = _causal_conv(self.conv1d, x, l)
        y = self.ssm_au(x, z)
        return _linear(self.out_proj, y)

    def ssm_au(self, x, z):
        b, l, d_in = x.shape
        n = self.args.d_state
        dt = _linear(self.dt_proj, _linear(self.x_proj, x))
        # dt = softplus(dt + self.dt_proj.bias) of aussm.py:879-880 happens inside the layout change below
        # "(n dstate1) dstate -> dstate1 n dstate"
        x_param = self.xA_proj.weight.view(n, d_in, d_in).permute(1, 0, 2)
        x_bias = self.xA_proj.bias.view(n, d_in).t()
        self.ssm_args = {
            "u": _swap(x),
            "dt": _swap_act(dt, "softplus", self.dt_proj.bias.float()),
            "x": x_param.contiguous() * (1 / math.sqrt(self.args.d_model)),
            "x_bias": x_bias.contiguous(),
            "B": self.B.contiguous(),
            "C": self.C.contiguous(),
            "D": self.D.float().contiguous(),
            "z": _swap(z),
        }
        y = self.optimized_SSMa_function(**self.ssm_args)
        return _swap(y)


class ResidualBlock(nn.Module):
    """Norm -> mixer -> add."""

    def __init__(self, args: Union[ModelArgsSSMau, ModelArgsMamba], scan_impl: Optional[Callable] = None):
        super().__init__()
        self.args = args
        self.mixer = args.block(args, scan_impl=scan_impl)
        self.norm = RMSNorm(args.d_model)

    def forward(self, x):
        return self.mixer(self.norm(x)) + x


class SSMTS(nn.Module):
    """Time-series model: Linear embedding -> residual AUSSM ('a') / Mamba ('m') blocks given by a
    layer string such as "a|m|a|m" -> RMSNorm -> Linear read-out."""

    def __init__(self, d_model: int, input_dim: int, output_dim: int, layers: Optional[str] = None,
                 d_state: int = 16, mamba_expand: int = 2, dt_rank: Union[int, str] = "auto", d_conv: int = 4,
                 conv_bias: bool = True, bias: bool = False, ssmau_cuda: bool = True, ssmau_conv_1d: bool = True,
                 embedding_decay: bool = True, verbose: bool = False,
                 ssmau_scan_impl: Optional[Callable] = None, mamba_scan_impl: Optional[Callable] = None):
        super().__init__()
        if layers is None:
            layers = "m|a"
        self.n_layers = len(layers.split("|"))
        self.output_dim = output_dim
        self.d_model = d_model
        self.d_state = d_state
        self.dt_rank = dt_rank
        self.d_conv = d_conv
        self.input_dim = input_dim
        self.mamba_expand = mamba_expand
        self.conv_bias = conv_bias
        self.verbose = verbose
        self.bias = bias
        self.ssmau_conv_1d = ssmau_conv_1d
        self.embedding_decay = embedding_decay
        self.ssmau_cuda = ssmau_cuda

        self.args = ModelBlockArgs(self.parse_layer_string(layers), self.d_model)
        self.embedding = nn.Linear(self.input_dim, self.d_model)
        self.layers = nn.ModuleList([
            ResidualBlock(a, scan_impl=ssmau_scan_impl if isinstance(a, ModelArgsSSMau) else mamba_scan_impl)
            for a in self.args.layers])
        self.norm_f = RMSNorm(self.d_model)
        self.output = nn.Linear(self.d_model, self.output_dim, bias=False)

    def parse_layer_string(self, layer_string: str):
        layer_args = []
        for layer in layer_string.replace(" ", "").split("|"):
            if layer == "a":
                layer_args.append(ModelArgsSSMau(self.d_model, self.d_state, self.dt_rank, self.d_conv,
                                                 self.conv_bias, self.bias, self.verbose,
                                                 conv_1d=self.ssmau_conv_1d, cuda=self.ssmau_cuda))
            elif layer == "m":
                layer_args.append(ModelArgsMamba(self.d_model, self.d_state, self.mamba_expand, self.dt_rank,
                                                 self.d_conv, self.conv_bias, self.bias, self.verbose))
            else:
                raise NotImplementedError(f"Layer type \"{layer}\" not recognized")
        return layer_args

    def get_parameter_groups_for_optimizer(self):
        emb = {"params": self.embedding.parameters()}
        if self.embedding_decay:
            emb["weight_decay"] = 0.0
        return [emb, {"params": self.layers.parameters()}, {"params": self.norm_f.parameters()},
                {"params": self.output.parameters()}]

    def forward(self, input_ids, **kwargs):
        x = _linear(self.embedding, input_ids)
        for layer in self.layers:
            x = layer(x)
        return _linear(self.output, self.norm_f(x))
