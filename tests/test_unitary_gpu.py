"""GPU parity of the adaptive-unitary core scan (HIP, through the C ABI) against the CPU oracle.

Tolerances: the benchmark contract's atol = rtol = 1e-4 for float32 inputs.  Gradients are
compared after normalising by the largest magnitude of the oracle's gradient tensor, so that
the absolute part of the tolerance is meaningful for every tensor."""
import pytest
import torch

from oracle import scan_oracle as O

pytestmark = pytest.mark.gpu

ATOL = RTOL = 1e-4


def _dev(p):
    return {k: v.cuda() for k, v in p.items()}


def _close(got, want, what):
    scale = max(1.0, float(want.abs().max()))
    torch.testing.assert_close(got.cpu() / scale, want / scale, atol=ATOL, rtol=RTOL, msg=lambda m: f"{what}: {m}")


SHAPES = [
    (2, 5, 3, 7),        # everything ragged: partial channel group, partial state group, partial tile
    (1, 64, 16, 32),     # exactly one tile, one channel group
    (2, 70, 16, 100),    # two channel groups, second one partial
    (3, 130, 4, 257),    # N = 4 -> one state per wavefront; checkpoint boundary crossed (L > 256)
    (2, 64, 8, 96),
    (1, 96, 32, 64),
    (1, 32, 64, 40),     # largest supported state size
    (2, 128, 1, 33),
]


@pytest.mark.parametrize("B,D,N,L", SHAPES)
def test_forward_matches_oracle(B, D, N, L):
    from aussm_amd import scan
    p = O.make_core_inputs(B, D, N, L, seed=B + D + N + L, gate=True)
    g = torch.Generator().manual_seed(1)
    h0 = torch.complex(torch.randn(B, D, N, generator=g), torch.randn(B, D, N, generator=g))
    print(f"case unitary fwd B={B} D={D} N={N} L={L}", flush=True)
    want_y, want_h = O.unitary_core_loop(p["u"], p["delta"], p["theta"], p["Bc"], p["Cc"], p["Dskip"], p["z"], h0)
    q = _dev(p)
    y, hL = scan.unitary_scan(q["u"], q["delta"], q["theta"], q["Bc"], q["Cc"], q["Dskip"], q["z"], h0.cuda(),
                              return_last_state=True)
    _close(y, want_y, "y")
    _close(torch.view_as_real(hL), torch.view_as_real(want_h), "hL")
    # optional arguments absent
    want_y, _ = O.unitary_core_loop(p["u"], p["delta"], p["theta"], p["Bc"], p["Cc"])
    y = scan.unitary_scan(q["u"], q["delta"], q["theta"], q["Bc"], q["Cc"])
    _close(y, want_y, "y (no skip, gate, h0)")


@pytest.mark.parametrize("B,D,N,L", SHAPES)
@pytest.mark.parametrize("gate", [False, True])
def test_gradients_match_oracle(B, D, N, L, gate):
    from aussm_amd import scan
    p = O.make_core_inputs(B, D, N, L, seed=7 * B + D + N + L, gate=gate)
    g = torch.Generator().manual_seed(2)
    h0 = torch.complex(torch.randn(B, D, N, generator=g), torch.randn(B, D, N, generator=g))
    dhL = torch.complex(torch.randn(B, D, N, generator=g), torch.randn(B, D, N, generator=g))
    names = ["u", "delta", "theta", "Bc", "Cc", "Dskip"] + (["z"] if gate else [])
    print(f"case unitary bwd B={B} D={D} N={N} L={L} gate={gate}", flush=True)

    def run(fn, dev):
        leaves = {k: p[k].clone().to(dev).requires_grad_(True) for k in names}
        h = h0.clone().to(dev).requires_grad_(True)
        y, hL = fn(leaves["u"], leaves["delta"], leaves["theta"], leaves["Bc"], leaves["Cc"], leaves["Dskip"],
                   leaves.get("z"), h)
        loss = (y * p["dy"].to(dev)).sum() + (hL * dhL.to(dev).conj()).real.sum()
        loss.backward()
        out = {k: v.grad for k, v in leaves.items()}
        out["h0"] = h.grad
        return out

    want = run(O.unitary_core_loop, "cpu")
    got = run(lambda *a: scan.unitary_scan(*a, return_last_state=True), "cuda")
    for k in want:
        w, gk = want[k], got[k]
        if w.is_complex():
            w, gk = torch.view_as_real(w), torch.view_as_real(gk)
        _close(gk, w, f"d{k}")


def test_rejects_bad_arguments():
    from aussm_amd import scan
    p = _dev(O.make_core_inputs(1, 4, 2, 8))
    with pytest.raises(RuntimeError):
        scan.unitary_scan(p["u"].double(), p["delta"].double(), p["theta"], p["Bc"], p["Cc"])
    with pytest.raises(RuntimeError):
        scan.unitary_scan(p["u"], p["delta"], p["theta"][:, :, :4], p["Bc"], p["Cc"])
    with pytest.raises(RuntimeError):
        scan.unitary_scan(p["u"].cpu(), p["delta"].cpu(), p["theta"].cpu(), p["Bc"].cpu(), p["Cc"].cpu())
    big = _dev(O.make_core_inputs(1, 4, 65, 8))
    with pytest.raises(RuntimeError):
        scan.unitary_scan(big["u"], big["delta"], big["theta"], big["Bc"], big["Cc"])


@pytest.mark.gpu
@pytest.mark.parametrize("b,r,d,n,l", [(2, 3, 70, 1, 52), (1, 4, 33, 2, 37), (3, 2, 64, 1, 128)])
def test_inputs_shared_by_consecutive_batch_elements(b, r, d, n, l):
    """u and delta of batch size b serve b * r phase sequences (how the drop-in operator runs its
    states): outputs and gradients equal those of the call with u and delta replicated, and the
    gradients of u and delta are the sums over the r users."""
    from aussm_amd import scan
    p = O.make_core_inputs(b * r, d, n, l, seed=b + r + l)
    u, delta = p["u"][::r].contiguous(), p["delta"][::r].contiguous()
    dev = "cuda"

    def run(fn, uu, dd, device):
        lv = [t.clone().to(device).requires_grad_(True) for t in (uu, dd, p["theta"], p["Bc"], p["Cc"], p["Dskip"])]
        y = fn(*lv)
        (y * p["dy"].to(device)).sum().backward()
        return [y.detach()] + [t.grad for t in lv]

    rep = lambda t: t[:, None].expand(b, r, d, l).reshape(b * r, d, l)
    want = run(lambda uu, dd, *a: O.unitary_core_loop(rep(uu), rep(dd), *a)[0], u, delta, "cpu")
    print(f"case shared inputs b={b} r={r} d={d} n={n} l={l}", flush=True)
    got = run(scan.unitary_scan, u, delta, dev)
    torch.cuda.synchronize()
    for name, w, g in zip(("y", "du", "ddelta", "dtheta", "dB", "dC", "dD"), want, got):
        if w.is_complex():
            w, g = torch.view_as_real(w), torch.view_as_real(g)
        scale = max(1.0, float(w.abs().max()))
        torch.testing.assert_close(g.cpu() / scale, w / scale, atol=1e-4, rtol=1e-4, msg=lambda m: f"{name}: {m}")


@pytest.mark.gpu
@pytest.mark.parametrize("n,offset", [(4096, 0), (1027, 0), (1000, 1), (5, 3)])
def test_gate_kernels(n, offset):
    """aussm_gate_fwd / _bwd (y = y_pre silu(z) and its two gradients) against the formula in float64, aligned
    and unaligned views, lengths that are not a multiple of four."""
    from aussm_amd import scan, _lib
    lib = _lib.load()
    g = torch.Generator().manual_seed(n + offset)
    base = [torch.randn(n + 8, generator=g).cuda() for _ in range(3)]
    ypre, z, dy = (t[offset:offset + n] for t in base)
    y, dyp, dz = (torch.empty(n + 8, device="cuda")[offset:offset + n] for _ in range(3))
    print(f"case gate kernels n={n} offset={offset}", flush=True)
    scan.check(lib.aussm_gate_fwd(scan.ptr(ypre), scan.ptr(z), scan.ptr(y), n, scan._stream()), "gate_fwd")
    scan.check(lib.aussm_gate_bwd(scan.ptr(dy), scan.ptr(ypre), scan.ptr(z), scan.ptr(dyp), scan.ptr(dz), n, scan._stream()), "gate_bwd")
    torch.cuda.synchronize()
    a, v, d = ypre.double().cpu(), z.double().cpu(), dy.double().cpu()
    sg = torch.sigmoid(v)
    torch.testing.assert_close(y.double().cpu(), a * v * sg, atol=1e-6, rtol=1e-6)
    torch.testing.assert_close(dyp.double().cpu(), d * v * sg, atol=1e-6, rtol=1e-6)
    torch.testing.assert_close(dz.double().cpu(), d * a * sg * (1 + v * (1 - sg)), atol=1e-6, rtol=1e-6)
