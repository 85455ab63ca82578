"""The fused operator kernels (aussm_ssm_adaptive_unitary_fwd / _bwd behind
torch.ops.extension_cpp.ssm_adaptive_unitary and ssm_adaptive_backward_unitary) against the CPU oracle's
sequential-loop restatement of the operator in float64 (oracle.scan_oracle.adaptive_unitary_op_loop) and
its autograd gradients: all three outputs, all twelve gradients, explicit start state and state
gradients, ragged shapes (l not a multiple of the 16-step tile, d not a multiple of 32 or of the
channels per workgroup, n < 16).  Tolerance: the benchmark contract's 1e-4 after normalising each
tensor by its largest oracle entry (the reference's own forward tolerance is atol 7e-5, rtol 5e-5,
extension-cpp/test/test_extension.py:95).  A last case at the benchmark's training shape checks the
fused kernels against the package's composite route (BLAS phase projection + core scan)."""
import pytest
import torch

from oracle import scan_oracle as O

pytestmark = pytest.mark.gpu

IN_NAMES = ["u", "dt", "x", "x_bias", "B_r", "B_theta", "C_r", "C_theta", "D", "z", "h_re", "h_im"]


def _inputs(b, d, n, l, seed, dtype=torch.float64, xscale=None):
    u, dt, x, xb, Bp, Cp, D, z = O.make_adaptive_inputs(b=b, d=d, n=n, l=l, binary_u=False, seed=seed, dtype=dtype)
    if xscale is not None:
        x = x * xscale
    Br, Bt, Cr, Ct = O.polar_params(Bp, Cp)
    g = torch.Generator().manual_seed(seed + 100)
    hr = torch.randn(b, d, n, generator=g, dtype=torch.float64).to(dtype)
    hi = torch.randn(b, d, n, generator=g, dtype=torch.float64).to(dtype)
    return [u, dt, x, xb, Br, Bt, Cr, Ct, D, z, hr, hi]


def _close(got, want, name, tol=1e-4):
    scale = max(1e-3, float(want.abs().max()))
    torch.testing.assert_close(got.double().cpu() / scale, want.double() / scale, atol=tol, rtol=tol,
                               msg=lambda m: f"{name}: {m}")


SHAPES = [(2, 8, 4, 256), (3, 20, 5, 48), (2, 37, 16, 45), (1, 70, 11, 130), (2, 16, 16, 14),
          (2, 12, 64, 70), (2, 9, 24, 33), (1, 21, 40, 50),          # more than 16 states: 4, 2 and 4 (3 padded) blocks per channel
          (1, 300, 16, 35), (1, 512, 32, 20), (2, 160, 8, 1), (1, 100, 3, 17)]   # wide: one wavefront per SIMD above d = 256


@pytest.mark.parametrize("shape", SHAPES)
def test_fused_forward_matches_oracle(shape):
    from aussm_amd import ops  # noqa: F401
    b, d, n, l = shape
    print(f"case fused fwd b={b} d={d} n={n} l={l}", flush=True)
    args = _inputs(b, d, n, l, seed=3, xscale=d ** -0.5)
    want = O.adaptive_unitary_op_loop(*args)
    got = torch.ops.extension_cpp.ssm_adaptive_unitary(*[a.float().cuda() for a in args])
    for w, g_, name in zip(want, got, ("y", "next_hid_real", "next_hid_imag")):
        _close(g_, w, name)


@pytest.mark.parametrize("shape", SHAPES)
def test_fused_backward_matches_oracle_autograd(shape):
    from aussm_amd import ops  # noqa: F401
    b, d, n, l = shape
    print(f"case fused bwd b={b} d={d} n={n} l={l}", flush=True)
    args = _inputs(b, d, n, l, seed=5, xscale=d ** -0.5)
    g = torch.Generator().manual_seed(9)
    gy = torch.randn(b, d, l, generator=g, dtype=torch.float64)
    ghr = torch.randn(b, d, n, generator=g, dtype=torch.float64)
    ghi = torch.randn(b, d, n, generator=g, dtype=torch.float64)
    leaves = [a.clone().requires_grad_(True) for a in args]
    outs = O.adaptive_unitary_op_loop(*leaves)
    want = torch.autograd.grad(outs, leaves, [gy, ghr, ghi])
    got = torch.ops.extension_cpp.ssm_adaptive_backward_unitary(
        *[t.float().cuda() for t in (gy, ghr, ghi)], *[a.float().cuda() for a in args])
    assert len(got) == 12
    for w, g_, name in zip(want, got, IN_NAMES):
        assert g_.shape == w.shape, name
        _close(g_, w, "gradient wrt " + name)


@pytest.mark.parametrize("kfloats", [16, 256])
def test_small_blocks_walk_the_problem_in_many_launches(kfloats):
    """A tiny block budget forces what long sequences and large batches get: the forward call in several chunks
    along the sequence, the backward call in (batch group) x (chunk) blocks with the state and its adjoint handed
    from launch to launch.  Same results as the oracle."""
    from aussm_amd import ops, _lib  # noqa: F401
    b, d, n, l = 5, 24, 16, 300
    print(f"case fused small blocks kfloats={kfloats}", flush=True)
    args = _inputs(b, d, n, l, seed=11, xscale=d ** -0.5)
    g = torch.Generator().manual_seed(12)
    grads = [torch.randn(b, d, l, generator=g, dtype=torch.float64), torch.randn(b, d, n, generator=g, dtype=torch.float64),
             torch.randn(b, d, n, generator=g, dtype=torch.float64)]
    leaves = [a.clone().requires_grad_(True) for a in args]
    outs = O.adaptive_unitary_op_loop(*leaves)
    want = torch.autograd.grad(outs, leaves, grads)
    dev = [a.float().cuda() for a in args]
    with _lib.options(block_kfloats=kfloats):
        got_f = torch.ops.extension_cpp.ssm_adaptive_unitary(*dev)
        got_b = torch.ops.extension_cpp.ssm_adaptive_backward_unitary(*[t.float().cuda() for t in grads], *dev)
        got_s = torch.ops.aussm_amd.ssm_adaptive_backward_unitary_from_state(*[t.float().cuda() for t in grads], *dev,
                                                                              got_f[1], got_f[2])
    for w, g_, name in zip(outs, got_f, ("y", "next_hid_real", "next_hid_imag")):
        _close(g_, w.detach(), name)
    for w, g1, g2, name in zip(want, got_b, got_s, IN_NAMES):
        _close(g1, w, "gradient wrt " + name)
        _close(g2, w, "gradient (from state) wrt " + name)


def test_backward_from_saved_state_equals_backward_from_inputs():
    """The autograd formula hands the forward call's end state to the backward kernels; the reference-shaped
    backward operator recomputes it.  Same gradients either way."""
    from aussm_amd import ops  # noqa: F401
    args = [a.float().cuda() for a in _inputs(3, 24, 16, 100, seed=8, xscale=24 ** -0.5)]
    g = torch.Generator().manual_seed(4)
    grads = [torch.randn(3, 24, 100, generator=g).cuda(), torch.randn(3, 24, 16, generator=g).cuda(),
             torch.randn(3, 24, 16, generator=g).cuda()]
    _, nh_r, nh_i = torch.ops.extension_cpp.ssm_adaptive_unitary(*args)
    a = torch.ops.extension_cpp.ssm_adaptive_backward_unitary(*grads, *args)
    b = torch.ops.aussm_amd.ssm_adaptive_backward_unitary_from_state(*grads, *args, nh_r, nh_i)
    for x, y, name in zip(a, b, IN_NAMES):
        _close(y, x.cpu(), "gradient wrt " + name, tol=1e-5)


def test_fused_autograd_through_the_operator():
    """loss.backward() through torch.ops.extension_cpp.ssm_adaptive_unitary reaches the fused backward."""
    from aussm_amd import ops
    args = _inputs(2, 12, 6, 40, seed=7, xscale=12 ** -0.5)
    leaves = [a.clone().requires_grad_(True) for a in args]
    y, hr, hi = O.adaptive_unitary_op_loop(*leaves)
    (y.square().mean() + (hr * hi).mean()).backward()
    dev = [a.float().cuda().requires_grad_(True) for a in args]
    y2, hr2, hi2 = ops.ssm_adaptive_unitary(*dev)
    (y2.square().mean() + (hr2 * hi2).mean()).backward()
    for w, g_, name in zip(leaves, dev, IN_NAMES):
        _close(g_.grad, w.grad, "gradient wrt " + name)


def test_fused_matches_composite_at_training_shape():
    """b=32, d=256, n=16, l=720 (the benchmark's training configuration of one block): the fused kernels
    against the composite route, forward and the gradients of the large tensors."""
    from aussm_amd import ops
    b, d, n, l = 32, 256, 16, 720
    print("case fused vs composite b=32 d=256 n=16 l=720", flush=True)
    args = [a.float().cuda() for a in _inputs(b, d, n, l, seed=1, dtype=torch.float32, xscale=d ** -0.5)]
    g = torch.Generator().manual_seed(2)
    gy = torch.randn(b, d, l, generator=g).cuda()
    zeros = torch.zeros(b, d, n, device="cuda")
    inputs_bytes = sum(a.numel() * 4 for a in args)
    # The fused route never holds the phase tensor (b d n l floats = 377 MB here).  What a call allocates on top of
    # its inputs - outputs and workspace - stays within the operator's input footprint for the forward call; for the
    # backward call within that (twelve gradients the size of the inputs) plus a workspace whose size does not grow
    # with the sequence: one block of phase adjoints (100 MiB at most) and the prepared operands of its products.
    torch.cuda.synchronize()
    torch.cuda.reset_peak_memory_stats()
    base = torch.cuda.memory_allocated()
    y, hr, hi = torch.ops.extension_cpp.ssm_adaptive_unitary(*args)
    torch.cuda.synchronize()
    peak_fwd = torch.cuda.max_memory_allocated() - base
    torch.cuda.reset_peak_memory_stats()
    base = torch.cuda.memory_allocated()
    grads = torch.ops.extension_cpp.ssm_adaptive_backward_unitary(gy, zeros, zeros, *args)
    torch.cuda.synchronize()
    peak_bwd = torch.cuda.max_memory_allocated() - base
    print(f"inputs {inputs_bytes / 1e6:.0f} MB, forward call +{peak_fwd / 1e6:.0f} MB, backward call +{peak_bwd / 1e6:.0f} MB", flush=True)
    assert peak_fwd <= inputs_bytes, (peak_fwd, inputs_bytes)
    assert peak_bwd <= inputs_bytes + 140 * 2 ** 20 and peak_bwd < b * d * n * l * 4, (peak_bwd, inputs_bytes)
    leaves = [a.clone().requires_grad_(True) for a in args]
    yc, hrc, hic = ops._composite(*leaves)
    want = torch.autograd.grad([yc], leaves, [gy], allow_unused=True)
    _close(y, yc.detach().cpu(), "y")
    _close(hr, hrc.detach().cpu(), "next_hid_real")
    _close(hi, hic.detach().cpu(), "next_hid_imag")
    for w, g_, name in zip(want, grads, IN_NAMES):
        _close(g_, w.cpu(), "gradient wrt " + name, tol=2e-4)


def test_shapes_beyond_the_fused_kernels_take_the_composite_route():
    """n > 64: the dispatcher operators still answer (through the core scan), forward and backward."""
    from aussm_amd import ops
    b, d, n, l = 2, 8, 72, 40
    assert not ops.fused_supported(b, d, n, l) and ops.fused_supported(b, d, 64, l)
    args = _inputs(b, d, n, l, seed=6, xscale=d ** -0.5)
    leaves = [a.clone().requires_grad_(True) for a in args]
    y, hr, hi = O.adaptive_unitary_op_loop(*leaves)
    (y.square().mean() + (hr * hi).mean()).backward()
    dev = [a.float().cuda().requires_grad_(True) for a in args]
    y2, hr2, hi2 = ops.ssm_adaptive_unitary(*dev)
    _close(y2.detach(), y.detach(), "y")
    (y2.square().mean() + (hr2 * hi2).mean()).backward()
    for w, g_, name in zip(leaves, dev, IN_NAMES):
        _close(g_.grad, w.grad, "gradient wrt " + name)
