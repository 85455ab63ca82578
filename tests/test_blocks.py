"""Blocks around the scan operators (counterparts of ai-modules/wavesAI/model/aussm.py).

CPU tests exercise the plumbing with the oracle's scans injected (benchmark configuration 0:
SSMauBlock(d_model=8, d_state=4) on x ~ N(0,1) of shape (8, 256, 8), loss = mean(y^2)).
GPU tests build the same seeded module twice, once on the oracle scans (CPU) and once on the
HIP operators, and compare outputs and every parameter gradient."""
import pytest
import torch

from aussm_amd import blocks
from oracle import scan_oracle as O


def oracle_ssmau(**kw):
    return O.adaptive_unitary_loop(kw["u"], kw["dt"], kw["x"], kw["x_bias"], kw["B"], kw["C"], kw["D"], kw["z"])


def oracle_mamba(u, delta, A, B, C, D, z=None, delta_bias=None, delta_softplus=False, return_last_state=False):
    return O.real_core_loop(u, delta, A, B, C, D, z, delta_bias, delta_softplus)[0]


SSMAU_KEYS = ["in_proj.weight", "conv1d.weight", "conv1d.bias", "out_proj.weight", "x_proj.weight",
              "dt_proj.weight", "dt_proj.bias", "D", "C", "B", "xA_proj.weight", "xA_proj.bias"]
MAMBA_KEYS = ["in_proj.weight", "conv1d.weight", "conv1d.bias", "out_proj.weight", "x_proj.weight",
              "dt_proj.weight", "dt_proj.bias", "D", "A_log"]


def _step(module, x):
    y = module(x)
    (y ** 2).mean().backward()
    return y.detach().cpu(), {k: p.grad.detach().cpu() for k, p in module.named_parameters()}


def test_config0_plumbing_cpu():
    torch.manual_seed(0)
    blk = blocks.SSMauBlock(blocks.ModelArgsSSMau(d_model=8, d_state=4), scan_impl=oracle_ssmau)
    x = torch.randn(8, 256, 8)
    y, grads = _step(blk, x)
    assert y.shape == (8, 256, 8) and torch.isfinite(y).all()
    assert sorted(grads) == sorted(SSMAU_KEYS)
    for k, g in grads.items():
        assert torch.isfinite(torch.view_as_real(g) if g.is_complex() else g).all(), k
        assert g.abs().max() > 0, f"no gradient reached {k}"
    # shapes handed to the operator
    a = blk.ssm_args
    assert a["u"].shape == (8, 8, 256) and a["x"].shape == (8, 4, 8) and a["x_bias"].shape == (8, 4)
    assert a["B"].dtype == torch.complex64 and a["B"].shape == (4,)


def test_parameter_names_and_seeded_init():
    args = blocks.ModelArgsSSMau(d_model=8, d_state=4)
    assert args.dt_rank == 4                                    # 'auto' -> d_state (aussm.py:61-62)
    torch.manual_seed(3)
    a = blocks.SSMauBlock(args, scan_impl=oracle_ssmau)
    torch.manual_seed(3)
    b = blocks.SSMauBlock(args, scan_impl=oracle_ssmau)
    assert sorted(a.state_dict()) == sorted(SSMAU_KEYS)
    for k in SSMAU_KEYS:
        assert torch.equal(a.state_dict()[k], b.state_dict()[k])
    assert a.xA_proj.bias.abs().max() <= torch.pi
    m = blocks.ModelArgsMamba(d_model=32)
    assert m.d_inner == 64 and m.dt_rank == 2                   # ceil(32/16) (aussm.py:90-91)
    mb = blocks.MambaBlock(m, scan_impl=oracle_mamba)
    assert sorted(mb.state_dict()) == sorted(MAMBA_KEYS)
    torch.testing.assert_close(mb.A_log[5], torch.log(torch.arange(1, 17, dtype=torch.float32)))


def test_ssmts_layer_string_cpu():
    torch.manual_seed(1)
    net = blocks.SSMTS(d_model=16, input_dim=5, output_dim=3, layers="a | m|a", d_state=4,
                       ssmau_scan_impl=oracle_ssmau, mamba_scan_impl=oracle_mamba)
    kinds = [type(l.mixer).__name__ for l in net.layers]
    assert kinds == ["SSMauBlock", "MambaBlock", "SSMauBlock"]
    y, grads = _step(net, torch.randn(2, 24, 5))
    assert y.shape == (2, 24, 3)
    assert all(g.abs().max() > 0 for g in grads.values())
    with pytest.raises(NotImplementedError):
        blocks.SSMTS(d_model=16, input_dim=5, output_dim=3, layers="a|q")
    groups = net.get_parameter_groups_for_optimizer()
    assert groups[0]["weight_decay"] == 0.0 and len(groups) == 4


def _compare(make, x, atol=1e-4, rtol=1e-4, gtol=2e-4):
    torch.manual_seed(5)
    ref = make(True)
    torch.manual_seed(5)
    dev = make(False).cuda()
    for (k, a), (_, b) in zip(ref.state_dict().items(), dev.state_dict().items()):
        assert torch.equal(a, b.cpu()), k
    y_ref, g_ref = _step(ref, x)
    y_dev, g_dev = _step(dev, x.cuda())
    torch.testing.assert_close(y_dev, y_ref, atol=atol, rtol=rtol)
    for k in g_ref:
        w, g = g_ref[k], g_dev[k]
        if w.is_complex():
            w, g = torch.view_as_real(w), torch.view_as_real(g)
        scale = max(1e-6, float(w.abs().max()))
        torch.testing.assert_close(g / scale, w / scale, atol=gtol, rtol=gtol, msg=lambda m, k=k: f"grad {k}: {m}")


@pytest.mark.gpu
def test_config0_hip_matches_oracle_backend():
    x = torch.randn(8, 256, 8, generator=torch.Generator().manual_seed(0))
    print("case config0 SSMauBlock d_model=8 d_state=4 x=(8,256,8)", flush=True)
    _compare(lambda cpu: blocks.SSMauBlock(blocks.ModelArgsSSMau(d_model=8, d_state=4),
                                           scan_impl=oracle_ssmau if cpu else None), x)


@pytest.mark.gpu
def test_mamba_block_hip_matches_oracle_backend():
    x = torch.randn(3, 70, 32, generator=torch.Generator().manual_seed(1))
    print("case MambaBlock d_model=32 x=(3,70,32)", flush=True)
    _compare(lambda cpu: blocks.MambaBlock(blocks.ModelArgsMamba(d_model=32),
                                           scan_impl=oracle_mamba if cpu else None), x)


@pytest.mark.gpu
def test_ssmts_hybrid_hip_matches_oracle_backend():
    """Benchmark configuration 4 at reduced width and length: layers a|m|a|m, 21 -> 21 channels."""
    x = torch.randn(2, 48, 21, generator=torch.Generator().manual_seed(2))
    print("case SSMTS d_model=32 layers=a|m|a|m x=(2,48,21)", flush=True)
    _compare(lambda cpu: blocks.SSMTS(d_model=32, input_dim=21, output_dim=21, layers="a|m|a|m", d_state=16,
                                      ssmau_scan_impl=oracle_ssmau if cpu else None,
                                      mamba_scan_impl=oracle_mamba if cpu else None), x,
             atol=3e-4, rtol=3e-4)


@pytest.mark.gpu
def test_ssmts_full_width_and_length_matches_oracle_backend(monkeypatch):
    """Benchmark configuration 4 at its full width and sequence length (d_model=256, l=720, layers a|m|a|m) on
    two sequences of the batch: outputs and every parameter gradient against the same seeded network running
    on the oracle's scans on the CPU.  (The batch size only multiplies the work; the full batch is
    test_ssmts_full_size_step_runs.)  fp32 GEMMs of width 256-512 on both sides in different orders: 5e-4.
    The linear layers take the weight gradient they use at the full batch (slices of the rows, summed), which
    1440 rows would not select by themselves."""
    monkeypatch.setattr(blocks, "_WGRAD_MIN_ROWS", 1)
    x = torch.randn(2, 720, 21, generator=torch.Generator().manual_seed(4))
    print("case SSMTS d_model=256 layers=a|m|a|m x=(2,720,21) vs oracle backend", flush=True)
    _compare(lambda cpu: blocks.SSMTS(d_model=256, input_dim=21, output_dim=21, layers="a|m|a|m",
                                      ssmau_scan_impl=oracle_ssmau if cpu else None,
                                      mamba_scan_impl=oracle_mamba if cpu else None), x,
             atol=5e-4, rtol=5e-4, gtol=5e-4)


@pytest.mark.gpu
def test_ssmts_full_size_step_runs():
    """Benchmark configuration 4 at full size: one training step, MSE against a random target."""
    torch.manual_seed(0)
    net = blocks.SSMTS(d_model=256, input_dim=21, output_dim=21, layers="a|m|a|m").cuda()
    x = torch.randn(32, 720, 21, device="cuda")
    tgt = torch.randn(32, 720, 21, device="cuda")
    print("case SSMTS full size d_model=256 x=(32,720,21)", flush=True)
    loss = F_mse(net(x), tgt)
    loss.backward()
    assert torch.isfinite(loss)
    for k, p in net.named_parameters():
        g = torch.view_as_real(p.grad) if p.grad.is_complex() else p.grad
        assert torch.isfinite(g).all(), k


def F_mse(a, b):
    return ((a - b) ** 2).mean()


def test_linear_with_sliced_weight_gradient_is_linear_cpu():
    """`_LinearFn` against torch's own `F.linear` in float64: output and the three gradients, for a 3-d input, an
    input that is a slice of a wider tensor (the dt columns of x_proj's output) and a layer without bias."""
    g = torch.Generator().manual_seed(11)
    for (shape, n, bias, sl) in [((4, 6, 5), 7, True, None), ((2, 8, 9), 3, False, 4), ((16, 5), 2, True, None)]:
        x = torch.randn(*shape, generator=g, dtype=torch.float64)
        w = torch.randn(n, sl or shape[-1], generator=g, dtype=torch.float64)
        b = torch.randn(n, generator=g, dtype=torch.float64) if bias else None
        dy = torch.randn(*shape[:-1], n, generator=g, dtype=torch.float64)
        res = []
        for fn in (lambda a, ww, bb: blocks._LinearFn.apply(a, ww, bb), torch.nn.functional.linear):
            leaves = [t.clone().requires_grad_(True) if t is not None else None for t in (x, w, b)]
            inp = leaves[0][..., :sl] if sl else leaves[0]
            y = fn(inp, leaves[1], leaves[2])
            y.backward(dy)
            res.append([y.detach()] + [t.grad for t in leaves if t is not None])
        for a, want in zip(*res):
            torch.testing.assert_close(a, want, atol=1e-12, rtol=1e-12)


def test_rmsnorm_is_the_reference_formula_cpu():
    """x * rsqrt(mean(x^2, -1) + eps) * weight (ai-modules/wavesAI/model/aussm.py:905-916)."""
    torch.manual_seed(3)
    norm = blocks.RMSNorm(24)
    with torch.no_grad():
        norm.weight.copy_(torch.randn(24))
    x = torch.randn(2, 5, 24)
    want = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + norm.eps) * norm.weight
    torch.testing.assert_close(norm(x), want, atol=1e-6, rtol=1e-6)
