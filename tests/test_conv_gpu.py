"""The depthwise causal convolution of the blocks (HIP, channels-last, through the C ABI) against
the CPU restatement of the reference's nn.Conv1d call: outputs and all three gradients, on a
contiguous tensor and on a column slice of a wider one (what the blocks pass), float32 tolerance
atol = rtol = 1e-5 (a handful of fused multiply-adds per output)."""
import pytest
import torch

from oracle import scan_oracle as O

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("b,l,d,k,sliced", [(2, 37, 70, 4, False), (3, 16, 64, 4, True), (1, 5, 3, 2, True),
                                            (2, 9, 130, 8, False), (4, 720, 256, 4, True)])
def test_causal_conv_matches_reference_conv(b, l, d, k, sliced):
    from aussm_amd import conv
    g = torch.Generator().manual_seed(b + l + d)
    wide = torch.randn(b, l, 2 * d, generator=g)
    w = torch.randn(d, 1, k, generator=g)
    bias = torch.randn(d, generator=g)
    dy = torch.randn(b, l, d, generator=g)

    def run(dev):
        src = wide.clone().to(dev).requires_grad_(True)
        x = src[:, :, :d] if sliced else src[:, :, d:].contiguous()
        wd, bd = w.clone().to(dev).requires_grad_(True), bias.clone().to(dev).requires_grad_(True)
        y = O.causal_conv1d_bld(x, wd, bd) if dev == "cpu" else conv.causal_conv1d(x, wd, bd)
        (y * dy.to(dev)).sum().backward()
        return y.detach(), src.grad, wd.grad, bd.grad

    want = run("cpu")
    print(f"case conv b={b} l={l} d={d} k={k} sliced={sliced}", flush=True)
    got = run("cuda")
    torch.cuda.synchronize()
    for name, a, e in zip(("y", "dx", "dw", "dbias"), got, want):
        scale = max(1.0, float(e.abs().max()))
        torch.testing.assert_close(a.cpu() / scale, e / scale, atol=1e-5, rtol=1e-5, msg=lambda m: f"{name}: {m}")


def test_causal_conv_without_bias_and_rejections():
    from aussm_amd import conv
    x = torch.randn(2, 8, 6, device="cuda", requires_grad=True)
    w = torch.randn(6, 1, 4, device="cuda", requires_grad=True)
    y = conv.causal_conv1d(x, w, None)
    y.sum().backward()
    want = O.causal_conv1d_bld(x.detach().cpu(), w.detach().cpu(), None)
    torch.testing.assert_close(y.detach().cpu(), want, atol=1e-5, rtol=1e-5)
    with pytest.raises(ValueError):
        conv.causal_conv1d(x.cpu(), w, None)
    with pytest.raises(ValueError):
        conv.causal_conv1d(x, w[:5], None)
    with pytest.raises(Exception):
        conv.causal_conv1d(x, torch.randn(6, 1, 9, device="cuda"), None)     # K > 8 is rejected by the library


@pytest.mark.parametrize("b,r,c,sliced", [(2, 37, 70, False), (3, 720, 256, True), (1, 1, 5, False), (2, 33, 31, True)])
def test_swap_last2_matches_transpose(b, r, c, sliced):
    from aussm_amd import conv
    g = torch.Generator().manual_seed(r + c)
    wide = torch.randn(b, r, 2 * c, generator=g).cuda().requires_grad_(True)
    x = wide[:, :, c:] if sliced else wide[:, :, :c].contiguous()
    print(f"case swap b={b} r={r} c={c} sliced={sliced}", flush=True)
    y = conv.swap_last2(x)
    assert y.is_contiguous() and y.shape == (b, c, r)
    assert torch.equal(y, x.transpose(1, 2))
    dy = torch.randn(b, c, r, generator=g).cuda()
    (gx,) = torch.autograd.grad(y, wide, dy)
    want = torch.zeros_like(wide)
    (want[:, :, c:] if sliced else want[:, :, :c]).copy_(dy.transpose(1, 2))
    assert torch.equal(gx, want)


@pytest.mark.parametrize("b,r,c,sliced", [(2, 37, 70, False), (3, 720, 256, True), (1, 1, 5, False), (2, 33, 31, True)])
@pytest.mark.parametrize("act,with_bias", [("silu", False), ("softplus", True), ("softplus", False)])
def test_swap_last2_with_activation(b, r, c, sliced, act, with_bias):
    """The layout change with silu / softplus(x + bias) done in the same pass, against torch's own
    elementwise functions in float64 (values and the gradients of x and bias); large arguments
    exercise softplus' linear branch (threshold 20)."""
    import torch.nn.functional as F
    from aussm_amd import conv
    g = torch.Generator().manual_seed(7 * r + c)
    wide = (torch.randn(b, r, 2 * c, generator=g) * 12).cuda().requires_grad_(True)
    bias = torch.randn(c, generator=g).cuda().requires_grad_(True) if with_bias else None
    x = wide[:, :, c:] if sliced else wide[:, :, :c]
    print(f"case swap+{act} b={b} r={r} c={c} sliced={sliced} bias={with_bias}", flush=True)
    y = conv.swap_last2(x, act=act, bias=bias)
    assert y.is_contiguous() and y.shape == (b, c, r)
    dy = torch.randn(b, c, r, generator=g).cuda()
    grads = torch.autograd.grad(y, [wide] + ([bias] if with_bias else []), dy)
    wide64 = wide.detach().double().requires_grad_(True)
    bias64 = bias.detach().double().requires_grad_(True) if with_bias else None
    x64 = wide64[:, :, c:] if sliced else wide64[:, :, :c]
    v = x64 if bias64 is None else x64 + bias64
    y64 = (F.silu(v) if act == "silu" else F.softplus(v)).transpose(1, 2)
    want = torch.autograd.grad(y64, [wide64] + ([bias64] if with_bias else []), dy.double())
    torch.testing.assert_close(y.double(), y64, atol=1e-5, rtol=1e-5)
    for a, w in zip(grads, want):
        scale = max(1.0, float(w.abs().max()))
        torch.testing.assert_close(a.double() / scale, w / scale, atol=1e-5, rtol=1e-5)
    with pytest.raises(ValueError):
        conv.swap_last2(x, act="tanh")
