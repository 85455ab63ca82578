"""GPU parity of the complex and real (Mamba S6) core scans against the CPU oracle, forward and
gradients, atol = rtol = 1e-4 (gradients normalised by the oracle gradient's largest magnitude).

The S6 oracle restates the published selective-scan formula; the reference holds no test or
fixture for the third-party selective_scan_fn it calls, so parity with THAT package is unpinned
(the oracle itself is pinned by brute force, closed forms and gradcheck in test_oracle.py)."""
import pytest
import torch

from oracle import scan_oracle as O

pytestmark = pytest.mark.gpu

ATOL = RTOL = 1e-4


def _close(got, want, what):
    scale = max(1.0, float(want.abs().max()))
    torch.testing.assert_close(got.cpu() / scale, want / scale, atol=ATOL, rtol=RTOL, msg=lambda m: f"{what}: {m}")


SHAPES = [
    (2, 5, 3, 7),
    (1, 64, 16, 32),
    (2, 70, 16, 100),
    (3, 130, 4, 257),
    (2, 64, 8, 96),
    (2, 128, 1, 33),
    (1, 40, 16, 16),
    (1, 33, 2, 17),
    (2, 40, 64, 50),          # more than 16 states: the backward pass takes one launch per block of 16
    (1, 70, 24, 33),
    (2, 20, 37, 40),
    # 9 to 15 states: the backward workgroups of eight wavefronts (two states each) are partly filled - whole
    # wavefronts without states, and with an odd count one wavefront with a single state
    (2, 70, 12, 100),
    (1, 33, 9, 50),
    (1, 20, 29, 300),
    # few (batch, channel group) pairs and at least 256 steps: the launch is split along the sequence
    # (segments of 128 steps here; the last one ragged, a single step in (3, 130, 4, 257) above)
    (2, 70, 16, 600),
    (1, 40, 64, 300),
    (1, 33, 2, 513),
]


def _h0(B, D, N, cplx, seed):
    g = torch.Generator().manual_seed(seed)
    r = lambda: torch.randn(B, D, N, generator=g)
    return torch.complex(r(), r()) if cplx else r()


@pytest.mark.parametrize("B,D,N,L", SHAPES)
def test_complex_forward(B, D, N, L):
    from aussm_amd import scan
    p = O.make_core_inputs(B, D, N, L, seed=B + D + N + L, variant="complex", gate=True)
    h0 = _h0(B, D, N, True, 1)
    print(f"case complex fwd B={B} D={D} N={N} L={L}", flush=True)
    want_y, want_h = O.complex_core_loop(p["u"], p["delta"], p["rho"], p["theta"], p["Bc"], p["Cc"], p["Dskip"],
                                         p["z"], h0)
    q = {k: v.cuda() for k, v in p.items()}
    y, hL = scan.complex_scan(q["u"], q["delta"], q["rho"], q["theta"], q["Bc"], q["Cc"], q["Dskip"], q["z"],
                              h0.cuda(), return_last_state=True)
    _close(y, want_y, "y")
    _close(torch.view_as_real(hL), torch.view_as_real(want_h), "hL")


@pytest.mark.parametrize("B,D,N,L", SHAPES)
@pytest.mark.parametrize("gate", [False, True])
def test_complex_gradients(B, D, N, L, gate):
    from aussm_amd import scan
    p = O.make_core_inputs(B, D, N, L, seed=3 * B + D + N + L, variant="complex", gate=gate)
    h0, dhL = _h0(B, D, N, True, 2), _h0(B, D, N, True, 3)
    names = ["u", "delta", "rho", "theta", "Bc", "Cc", "Dskip"] + (["z"] if gate else [])
    print(f"case complex bwd B={B} D={D} N={N} L={L} gate={gate}", flush=True)

    def run(fn, dev):
        lv = {k: p[k].clone().to(dev).requires_grad_(True) for k in names}
        h = h0.clone().to(dev).requires_grad_(True)
        y, hL = fn(lv["u"], lv["delta"], lv["rho"], lv["theta"], lv["Bc"], lv["Cc"], lv["Dskip"], lv.get("z"), h)
        ((y * p["dy"].to(dev)).sum() + (hL * dhL.to(dev).conj()).real.sum()).backward()
        out = {k: v.grad for k, v in lv.items()}
        out["h0"] = h.grad
        return out

    want = run(O.complex_core_loop, "cpu")
    got = run(lambda *a: scan.complex_scan(*a, return_last_state=True), "cuda")
    for k in want:
        w, gk = want[k], got[k]
        if w.is_complex():
            w, gk = torch.view_as_real(w), torch.view_as_real(gk)
        _close(gk, w, f"d{k}")


@pytest.mark.parametrize("B,D,N,L", SHAPES)
@pytest.mark.parametrize("softplus", [False, True])
def test_real_forward(B, D, N, L, softplus):
    from aussm_amd import scan
    p = O.make_core_inputs(B, D, N, L, seed=B + D + N + L, variant="real", gate=True)
    g = torch.Generator().manual_seed(5)
    bias = torch.randn(D, generator=g) * 0.5
    delta = torch.randn(B, D, L, generator=g) if softplus else p["delta"]
    h0 = _h0(B, D, N, False, 4)
    print(f"case real fwd B={B} D={D} N={N} L={L} softplus={softplus}", flush=True)
    want_y, want_h = O.real_core_loop(p["u"], delta, p["A"], p["Bm"], p["Cm"], p["Dskip"], p["z"],
                                      delta_bias=bias if softplus else None, delta_softplus=softplus, h0=h0)
    q = {k: v.cuda() for k, v in p.items()}
    y, hL = scan.selective_scan_fn(q["u"], delta.cuda(), q["A"], q["Bm"], q["Cm"], q["Dskip"], z=q["z"],
                                   delta_bias=bias.cuda() if softplus else None, delta_softplus=softplus,
                                   return_last_state=True, h0=h0.cuda())
    _close(y, want_y, "y")
    _close(hL, want_h, "hL")
    # the reference's call pattern: no start state, no last state
    want_y, _ = O.real_core_loop(p["u"], delta, p["A"], p["Bm"], p["Cm"], p["Dskip"], p["z"],
                                 delta_bias=bias, delta_softplus=True)
    y = scan.selective_scan_fn(q["u"], delta.cuda(), q["A"], q["Bm"], q["Cm"], q["Dskip"], z=q["z"],
                               delta_bias=bias.cuda(), delta_softplus=True, return_last_state=False)
    _close(y, want_y, "y (reference call pattern)")


@pytest.mark.parametrize("B,D,N,L", SHAPES)
@pytest.mark.parametrize("softplus,gate", [(False, False), (True, True)])
def test_real_gradients(B, D, N, L, softplus, gate):
    from aussm_amd import scan
    p = O.make_core_inputs(B, D, N, L, seed=5 * B + D + N + L, variant="real", gate=gate)
    g = torch.Generator().manual_seed(6)
    p["bias"] = torch.randn(D, generator=g) * 0.5
    if softplus:
        p["delta"] = torch.randn(B, D, L, generator=g)
    h0, dhL = _h0(B, D, N, False, 7), _h0(B, D, N, False, 8)
    names = ["u", "delta", "A", "Bm", "Cm", "Dskip"] + (["z"] if gate else []) + (["bias"] if softplus else [])
    print(f"case real bwd B={B} D={D} N={N} L={L} softplus={softplus} gate={gate}", flush=True)

    def run(fn, dev):
        lv = {k: p[k].clone().to(dev).requires_grad_(True) for k in names}
        h = h0.clone().to(dev).requires_grad_(True)
        y, hL = fn(lv["u"], lv["delta"], lv["A"], lv["Bm"], lv["Cm"], lv["Dskip"], lv.get("z"), lv.get("bias"),
                   softplus, h)
        ((y * p["dy"].to(dev)).sum() + (hL * dhL.to(dev)).sum()).backward()
        out = {k: v.grad for k, v in lv.items()}
        out["h0"] = h.grad
        return out

    want = run(lambda u, dl, A, Bm, Cm, D, z, bias, sp, h: O.real_core_loop(u, dl, A, Bm, Cm, D, z, bias, sp, h), "cpu")
    got = run(lambda u, dl, A, Bm, Cm, D, z, bias, sp, h: scan.selective_scan_fn(
        u, dl, A, Bm, Cm, D, z=z, delta_bias=bias, delta_softplus=sp, return_last_state=True, h0=h), "cuda")
    for k in want:
        _close(got[k], want[k], f"d{k}")


def test_state_limit():
    """64 states per channel is the limit of both directions (AUSSM_MAX_STATE)."""
    from aussm_amd import scan
    p = {k: v.cuda() for k, v in O.make_core_inputs(1, 8, 65, 16, variant="real").items()}
    with pytest.raises(RuntimeError):
        scan.selective_scan_fn(p["u"], p["delta"], p["A"], p["Bm"], p["Cm"])


@pytest.mark.parametrize("seed", range(20))
def test_random_shapes_and_input_types(seed):
    """Seeded sweep over both variants, ragged and tile-aligned lengths (the backward kernels take
    a branch-free path for tiles that lie inside the sequence), state counts that leave wavefronts
    partly or wholly idle, and float32 / bfloat16 inputs (odd lengths make bf16 rows start at odd
    element offsets).  bf16: the oracle runs on the already rounded values; gradients that come
    back in bf16 are compared at the contract's 2e-2."""
    import random
    from aussm_amd import scan
    r = random.Random(500 + seed)
    variant = r.choice(["real", "complex"])
    B, D, N = r.randint(1, 3), r.randint(1, 140), r.randint(1, 16)
    L = r.choice([r.randint(1, 70), 16 * r.randint(1, 12), r.randint(1, 200)])
    lowp = r.random() < 0.5
    p = O.make_core_inputs(B, D, N, L, seed=seed, variant=variant)
    names = ["u", "delta", "A", "Bm", "Cm", "Dskip"] if variant == "real" else ["u", "delta", "rho", "theta", "Bc", "Cc", "Dskip"]
    low = ("u", "delta", "Bm", "Cm", "Bc", "Cc")
    if lowp:
        for k in names:
            if k in low:
                t = p[k]
                p[k] = (torch.view_as_complex(torch.view_as_real(t).bfloat16().float().contiguous()) if t.is_complex()
                        else t.bfloat16().float())
    leaves = [p[k].clone().requires_grad_(True) for k in names]
    y_want = (O.real_core_loop if variant == "real" else O.complex_core_loop)(*leaves)[0]
    (y_want * p["dy"]).sum().backward()

    def dev(k):
        t = p[k].clone().cuda()
        if lowp and k in low:
            t = (torch.view_as_real(t).contiguous() if t.is_complex() else t).to(torch.bfloat16)
        return t.requires_grad_(True)

    dv = [dev(k) for k in names]
    print(f"case variants sweep seed={seed} {variant} B={B} D={D} N={N} L={L} bf16={lowp}", flush=True)
    y = (scan.selective_scan_fn if variant == "real" else scan.complex_scan)(*dv)
    (y * p["dy"].cuda()).sum().backward()
    torch.cuda.synchronize()
    _close(y.detach(), y_want.detach(), "y")
    for k, w, t in zip(names, leaves, dv):
        g, want = t.grad, w.grad
        if not g.is_complex():
            g = g.float()
            if want.is_complex():
                g = torch.view_as_complex(g.contiguous())
        if want.is_complex():
            g, want = torch.view_as_real(g), torch.view_as_real(want)
        tol = 2e-2 if (lowp and k in low) else ATOL
        scale = max(1.0, float(want.abs().max()))
        torch.testing.assert_close(g.cpu() / scale, want / scale, atol=tol, rtol=tol, msg=lambda m, k=k: f"d{k}: {m}")


@pytest.mark.parametrize("variant", ["complex", "real"])
@pytest.mark.parametrize("lowp", [False, True])
def test_split_along_sequence_matches_unsplit(variant, lowp):
    """12 (batch, channel group) pairs of 4136 steps run as 22 segments side by side; the same call with the
    split switched off is the comparison (itself checked against the oracle above at small sizes).  Outputs,
    final state and every gradient, gate and initial state included, float32 and bfloat16 inputs."""
    from aussm_amd import _lib, scan
    B, D, N, L = 4, 192, 16, 4136
    lib = _lib.load()
    assert lib.aussm_scan_workspace_floats(_lib.VAR_COMPLEX if variant == "complex" else _lib.VAR_REAL, B, D, N, L, 16, 0) > 0
    p = O.make_core_inputs(B, D, N, L, seed=11, variant=variant, gate=True)
    names = (["u", "delta", "A", "Bm", "Cm", "Dskip", "z"] if variant == "real"
             else ["u", "delta", "rho", "theta", "Bc", "Cc", "Dskip", "z"])
    low = ("u", "delta", "Bm", "Cm", "Bc", "Cc")
    h0, dhL = _h0(B, D, N, variant == "complex", 5), _h0(B, D, N, variant == "complex", 6)

    def run():
        lv = {}
        for k in names:
            t = p[k].clone().cuda()
            if lowp and k in low:
                t = (torch.view_as_real(t).contiguous() if t.is_complex() else t).to(torch.bfloat16)
            lv[k] = t.requires_grad_(True)
        h = h0.clone().cuda().requires_grad_(True)
        if variant == "real":
            y, hL = scan.selective_scan_fn(lv["u"], lv["delta"], lv["A"], lv["Bm"], lv["Cm"], lv["Dskip"], z=lv["z"],
                                           return_last_state=True, h0=h)
        else:
            y, hL = scan.complex_scan(lv["u"], lv["delta"], lv["rho"], lv["theta"], lv["Bc"], lv["Cc"], lv["Dskip"],
                                      lv["z"], h, return_last_state=True)
        ((y * p["dy"].cuda()).sum() + (hL * dhL.cuda().conj()).real.sum()).backward()
        torch.cuda.synchronize()
        out = {k: (v.grad if v.grad.is_complex() else v.grad.float()) for k, v in lv.items()}
        out["h0"] = h.grad
        out["y"], out["hL"] = y.detach(), hL.detach()
        return out

    print(f"case split vs unsplit {variant} bf16={lowp} B={B} D={D} N={N} L={L}", flush=True)
    got = run()
    with _lib.options(split_cap=0):
        want = run()
    for k in want:
        w, g = want[k], got[k]
        if w.is_complex():
            w, g = torch.view_as_real(w), torch.view_as_real(g)
        tol = 2e-2 if (lowp and k in low) else ATOL
        scale = max(1.0, float(w.abs().max()))
        torch.testing.assert_close(g / scale, w / scale, atol=tol, rtol=tol, msg=lambda m, k=k: f"{k}: {m}")


@pytest.mark.parametrize("seed", range(12))
def test_split_random_shapes_match_unsplit(seed):
    """Seeded sweep of calls that split along the sequence (few batch x channel-group pairs, ragged lengths,
    1 to 64 states, gate / initial state / softplus and bias present or not) against the same call with the
    split switched off: outputs, final state and every gradient."""
    import random
    from aussm_amd import _lib, scan
    r = random.Random(900 + seed)
    variant = r.choice(["real", "complex"])
    B, D = r.randint(1, 3), r.choice([r.randint(1, 64), r.randint(65, 200)])
    N = r.choice([1, 3, 8, 16, 17, 33, 64])
    L = r.choice([r.randint(257, 700), 128 * r.randint(2, 6), 4 * r.randint(65, 300)])
    gate, with_h0, softplus = r.random() < 0.5, r.random() < 0.5, r.random() < 0.5
    p = O.make_core_inputs(B, D, N, L, seed=seed, variant=variant, gate=gate)
    names = (["u", "delta", "A", "Bm", "Cm", "Dskip"] if variant == "real"
             else ["u", "delta", "rho", "theta", "Bc", "Cc", "Dskip"]) + (["z"] if gate else [])
    h0 = _h0(B, D, N, variant == "complex", 7) if with_h0 else None
    dhL = _h0(B, D, N, variant == "complex", 8)
    bias = torch.randn(D, generator=torch.Generator().manual_seed(seed)) if variant == "real" and softplus else None

    def run():
        lv = {k: p[k].clone().cuda().requires_grad_(True) for k in names}
        h = h0.clone().cuda().requires_grad_(True) if with_h0 else None
        if variant == "real":
            y, hL = scan.selective_scan_fn(lv["u"], lv["delta"], lv["A"], lv["Bm"], lv["Cm"], lv["Dskip"], z=lv.get("z"),
                                           delta_bias=None if bias is None else bias.cuda(), delta_softplus=softplus,
                                           return_last_state=True, h0=h)
        else:
            y, hL = scan.complex_scan(lv["u"], lv["delta"], lv["rho"], lv["theta"], lv["Bc"], lv["Cc"], lv["Dskip"],
                                      lv.get("z"), h, return_last_state=True)
        ((y * p["dy"].cuda()).sum() + (hL * dhL.cuda().conj()).real.sum()).backward()
        torch.cuda.synchronize()
        out = {k: v.grad for k, v in lv.items()}
        if with_h0:
            out["h0"] = h.grad
        out["y"], out["hL"] = y.detach(), hL.detach()
        return out

    print(f"case split sweep seed={seed} {variant} B={B} D={D} N={N} L={L} gate={gate} h0={with_h0} softplus={softplus}",
          flush=True)
    vcode = _lib.VAR_COMPLEX if variant == "complex" else _lib.VAR_REAL
    assert _lib.load().aussm_scan_workspace_floats(vcode, B, D, N, L, 16, 0) > 0
    got = run()
    with _lib.options(split_cap=0):
        want = run()
    for k in want:
        w, g = want[k], got[k]
        if w.is_complex():
            w, g = torch.view_as_real(w), torch.view_as_real(g)
        scale = max(1.0, float(w.abs().max()))
        torch.testing.assert_close(g / scale, w / scale, atol=ATOL, rtol=RTOL, msg=lambda m, k=k: f"{k}: {m}")
