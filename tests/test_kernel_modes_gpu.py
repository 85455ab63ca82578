"""Every unitary kernel of the library against the CPU oracle on the same inputs.

The launcher picks a matrix-core kernel for the common case (float32 inputs, N <= 16, L a multiple
of 4, aligned tensors) and the generic kernel otherwise; the library options
unitary_fwd / unitary_bwd (aussm_set_option) force one of them.  Each mode must meet the float32 tolerance of the benchmark
contract, atol = rtol = 1e-4 after normalising by the largest magnitude of the expected tensor, on
shapes that exercise a partial channel group, a partial last chunk, N < 16, a carried-in state, the
output gate and phases large enough to take the range-reduction path."""
import pytest
import torch

from oracle import scan_oracle as O

pytestmark = pytest.mark.gpu

FWD_MODES = ["0", "2", "3", "6"]          # generic, bf16 x2 pieces, bf16 x3 pieces, prepared operands (two wavefronts per SIMD)
BWD_MODES = ["0", "2", "3", "5", "6"]     # generic, two pieces, 3 along the sequence and 2 over the channel, three pieces, prepared operands
SHAPES = [(2, 80, 16, 200), (1, 64, 5, 36), (2, 128, 16, 512), (1, 5, 6, 8)]
NAMES = ("u", "delta", "theta", "Bc", "Cc", "Dskip")


def _close(got, want, what, tol=1e-4):
    if want.is_complex():
        got, want = torch.view_as_real(got), torch.view_as_real(want)
    scale = max(1.0, float(want.abs().max()))
    torch.testing.assert_close(got.cpu().float() / scale, want.float() / scale, atol=tol, rtol=tol,
                               msg=lambda m: f"{what}: {m}")


def _opts(**kw):
    """Library options for the duration of a block (aussm_set_option through the C ABI)."""
    from aussm_amd import _lib
    return _lib.options(**kw)


def _inputs(B, D, N, L, seed, big_theta):
    p = O.make_core_inputs(B, D, N, L, seed=seed, gate=True)
    if big_theta:
        p["theta"] = p["theta"] * 20.0          # |theta| up to ~40 rad: range reduction inside the kernels
    g = torch.Generator().manual_seed(seed + 1)
    p["h0"] = torch.complex(torch.randn(B, D, N, generator=g), torch.randn(B, D, N, generator=g))
    return p


@pytest.mark.parametrize("mode", FWD_MODES)
@pytest.mark.parametrize("B,D,N,L", SHAPES)
@pytest.mark.parametrize("big_theta", [False, True])
def test_forward_modes(mode, B, D, N, L, big_theta):
    from aussm_amd import scan
    p = _inputs(B, D, N, L, 11 + B + D + L, big_theta)
    want_y, want_h = O.unitary_core_loop(p["u"], p["delta"], p["theta"], p["Bc"], p["Cc"], p["Dskip"], p["z"], p["h0"])
    q = {k: v.cuda() for k, v in p.items()}
    print(f"case fwd mode={mode} B={B} D={D} N={N} L={L} big={big_theta}", flush=True)
    with _opts(unitary_fwd=mode):
        y, hL = scan.unitary_scan(q["u"], q["delta"], q["theta"], q["Bc"], q["Cc"], q["Dskip"], q["z"], q["h0"],
                                  return_last_state=True)
        torch.cuda.synchronize()
    _close(y, want_y, "y")
    _close(hL, want_h, "hL")


@pytest.mark.parametrize("mode", BWD_MODES)
@pytest.mark.parametrize("B,D,N,L", SHAPES)
@pytest.mark.parametrize("big_theta", [False, True])
def test_backward_modes(mode, B, D, N, L, big_theta):
    from aussm_amd import scan
    p = _inputs(B, D, N, L, 23 + B + D + L, big_theta)
    g = torch.Generator().manual_seed(5)
    dh = torch.complex(torch.randn(B, D, N, generator=g), torch.randn(B, D, N, generator=g))

    def run(fn, dev):
        lv = [p[k].clone().to(dev).requires_grad_(True) for k in NAMES]
        h0 = p["h0"].clone().to(dev).requires_grad_(True)
        y, hL = fn(*lv, None, h0)
        loss = (y * p["dy"].to(dev)).sum() + (torch.view_as_real(hL) * torch.view_as_real(dh.to(dev))).sum()
        loss.backward()
        return [t.grad for t in lv] + [h0.grad]

    want = run(lambda *a: O.unitary_core_loop(*a), "cpu")
    print(f"case bwd mode={mode} B={B} D={D} N={N} L={L} big={big_theta}", flush=True)
    with _opts(unitary_bwd=mode):
        got = run(lambda *a: scan.unitary_scan(*a, return_last_state=True), "cuda")
        torch.cuda.synchronize()
    for k, w, gt in zip(NAMES + ("h0",), want, got):
        _close(gt, w, f"d{k}", tol=2e-4 if big_theta else 1e-4)


def test_auxiliary_buffer_is_never_consumed_stale():
    """The forward call may leave Im(P_t S_t) in the auxiliary buffer for the backward call.  A
    forward kernel that does not fill it must clear its tag: run a filling forward + backward, then
    (same shape, so the allocator hands back the same memory) a non-filling forward followed by the
    matrix-core backward on DIFFERENT inputs, through the raw C-ABI wrappers with one shared buffer."""
    from aussm_amd import scan
    B, D, N, L = 2, 64, 16, 256
    aux = None
    for seed, fwd_mode in ((1, "3"), (2, "0"), (3, "6"), (4, "0")):
        p = O.make_core_inputs(B, D, N, L, seed=seed)
        leaves = [p[k].clone().requires_grad_(True) for k in NAMES]
        y, _ = O.unitary_core_loop(*leaves)
        (y * p["dy"]).sum().backward()
        want = [t.grad for t in leaves]
        q = {k: v.cuda() for k, v in p.items()}
        Bri = torch.view_as_real(q["Bc"]).contiguous()
        Cri = torch.view_as_real(q["Cc"]).contiguous()
        if aux is None:
            aux = scan.unitary_aux(q["u"], N, scan.UNITARY_CK)
        print(f"case aux seed={seed} fwd_mode={fwd_mode}", flush=True)
        with _opts(unitary_fwd=fwd_mode):
            yk, _, hck = scan.unitary_fwd_raw(q["u"], q["delta"], q["theta"], Bri, Cri, q["Dskip"], None, None,
                                              want_state=False, ck=scan.UNITARY_CK, aux=aux)
        got = scan.unitary_bwd_raw(q["dy"], None, q["u"], q["delta"], q["theta"], Bri, Cri, q["Dskip"], hck,
                                   scan.UNITARY_CK, aux=aux)
        torch.cuda.synchronize()
        _close(yk, y.detach(), "y")
        du, ddelta, dtheta, dB, dC, dD, _ = got
        for k, w, gt in zip(NAMES, want, (du, ddelta, dtheta, torch.view_as_complex(dB), torch.view_as_complex(dC), dD)):
            _close(gt, w, f"d{k} (forward mode {fwd_mode})")


@pytest.mark.parametrize("B,D,N,L,cap", [(1, 64, 16, 1024, None), (1, 64, 16, 1024, "2"), (2, 80, 8, 512, None),
                                         (1, 40, 16, 2048, None)])
def test_sequence_split_over_workgroups(B, D, N, L, cap):
    """With few (batch, channel) pairs the launcher cuts the sequence into segments that run in
    parallel (segment end states from a zero start, a chain over the segments, then every segment
    from its true incoming state; the adjoint likewise in reverse).  Outputs, the final state and
    every gradient, with a carried-in state and an upstream gradient of the final state, against
    the CPU oracle and against the same call with the split switched off."""
    from aussm_amd import scan, _lib
    lib = _lib.load()
    # the shapes are chosen so that the split happens: its states need room behind the per-(b,d,l) part
    assert lib.aussm_unitary_aux_floats(B, D, N, L, scan.UNITARY_CK) > B * D * L + 64
    p = _inputs(B, D, N, L, 3 + L + D, big_theta=(D == 80))
    g = torch.Generator().manual_seed(9)
    dh = torch.complex(torch.randn(B, D, N, generator=g), torch.randn(B, D, N, generator=g))

    def run(fn, dev):
        lv = [p[k].clone().to(dev).requires_grad_(True) for k in NAMES]
        h0 = p["h0"].clone().to(dev).requires_grad_(True)
        y, hL = fn(*lv, None, h0)
        loss = (y * p["dy"].to(dev)).sum() + (torch.view_as_real(hL) * torch.view_as_real(dh.to(dev))).sum()
        loss.backward()
        return [y.detach(), hL.detach()] + [t.grad for t in lv] + [h0.grad]

    names = ("y", "hL") + tuple("d" + k for k in NAMES) + ("dh0",)
    want = run(lambda *a: O.unitary_core_loop(*a), "cpu")
    print(f"case split B={B} D={D} N={N} L={L} cap={cap}", flush=True)
    with _opts(**({"split_cap": cap} if cap else {})):
        got = run(lambda *a: scan.unitary_scan(*a, return_last_state=True), "cuda")
        torch.cuda.synchronize()
    with _opts(split_cap=0):
        whole = run(lambda *a: scan.unitary_scan(*a, return_last_state=True), "cuda")
        torch.cuda.synchronize()
    for k, w, gt, wh in zip(names, want, got, whole):
        _close(gt, w, k, tol=2e-4 if D == 80 else 1e-4)
        _close(gt, wh.cpu(), k + " (split vs whole)", tol=2e-5)


@pytest.mark.parametrize("B,D,N,L,force", [
    (1, 64, 32, 1024, False),      # more than 16 states
    (2, 70, 24, 1000, False),      # ... ragged channel group, a last segment shorter than the others
    (1, 40, 16, 1026, False),      # a length that is not a multiple of 4
    (2, 33, 64, 777, False),       # odd everything
    (1, 64, 16, 1024, True),       # a shape of the matrix-core kernels sent to the vector-ALU ones by option
    (1, 64, 4, 2048, False),       # few states: the vector-ALU kernels by default
])
def test_vector_alu_kernels_split_along_the_sequence(B, D, N, L, force):
    """The unitary scan on the vector-ALU kernels splits like the complex and real scans do: outputs, final state
    and every gradient, with a carried-in state and an upstream gradient of the final state, against the CPU
    oracle and against the same call with the split switched off."""
    from aussm_amd import scan, _lib
    lib = _lib.load()
    ck = scan.unitary_ck(B, D, N, L)
    assert lib.aussm_unitary_split_segments(B, D, N, L, ck) > 1, "the shape is meant to split"
    p = _inputs(B, D, N, L, 5 + L + D, False)
    g = torch.Generator().manual_seed(10)
    dh = torch.complex(torch.randn(B, D, N, generator=g), torch.randn(B, D, N, generator=g))

    def run(fn, dev):
        lv = [p[k].clone().to(dev).requires_grad_(True) for k in NAMES]
        h0 = p["h0"].clone().to(dev).requires_grad_(True)
        y, hL = fn(*lv, None, h0)
        loss = (y * p["dy"].to(dev)).sum() + (torch.view_as_real(hL) * torch.view_as_real(dh.to(dev))).sum()
        loss.backward()
        return [y.detach(), hL.detach()] + [t.grad for t in lv] + [h0.grad]

    names = ("y", "hL") + tuple("d" + k for k in NAMES) + ("dh0",)
    want = run(lambda *a: O.unitary_core_loop(*a), "cpu")
    print(f"case vector-ALU split B={B} D={D} N={N} L={L} force={force}", flush=True)
    forced = {"unitary_fwd": 0, "unitary_bwd": 0} if force else {}
    with _opts(**forced):
        assert lib.aussm_unitary_kernel_mode(0, B, D, N, L, ck, 0, 1, 1) == 0 and lib.aussm_unitary_kernel_mode(1, B, D, N, L, ck, 0, 1, 1) == 0
        got = run(lambda *a: scan.unitary_scan(*a, return_last_state=True), "cuda")
        torch.cuda.synchronize()
    with _opts(split_cap=0, **forced):
        whole = run(lambda *a: scan.unitary_scan(*a, return_last_state=True), "cuda")
        torch.cuda.synchronize()
    for k, w, gt, wh in zip(names, want, got, whole):
        _close(gt, w, k, tol=1e-4)
        _close(gt, wh.cpu(), k + " (split vs whole)", tol=2e-5)
    # ... and without gradients (no checkpoints; the buffer is workspace only)
    with torch.no_grad():
        y, hL = scan.unitary_scan(*[p[k].cuda() for k in NAMES], None, p["h0"].cuda(), return_last_state=True)
    _close(y, want[0], "y (no grad)", tol=1e-4)
    _close(hL, want[1], "hL (no grad)", tol=1e-4)


# (the third one is split along L on the matrix-core kernels, the fourth on the vector-ALU kernels)
@pytest.mark.parametrize("B,D,N,L", [(2, 80, 16, 200), (1, 64, 7, 64), (1, 64, 16, 1024), (1, 64, 32, 1024)])
def test_bf16_inputs_equal_the_float_run_on_the_same_values(B, D, N, L):
    """bfloat16 u / delta / B / C are widened exactly inside the matrix-core kernels: outputs and
    (float32) gradients must agree with the float32 call on the same, already rounded, values to
    float32 rounding — far inside the 2e-2 the contract allows for bf16 inputs."""
    from aussm_amd import scan
    p = {k: v.cuda() for k, v in O.make_core_inputs(B, D, N, L, seed=17).items()}
    ck = scan.UNITARY_CK
    lo = {k: p[k].to(torch.bfloat16) for k in ("u", "delta")}
    lo["Bri"] = torch.view_as_real(p["Bc"]).to(torch.bfloat16).contiguous()
    lo["Cri"] = torch.view_as_real(p["Cc"]).to(torch.bfloat16).contiguous()
    hi = {k: v.float() for k, v in lo.items()}
    outs = []
    for q in (lo, hi):
        aux = scan.unitary_aux(q["u"], N, ck)
        print(f"case bf16-vs-float dtype={q['u'].dtype} B={B} D={D} N={N} L={L}", flush=True)
        y, hL, hck = scan.unitary_fwd_raw(q["u"], q["delta"], p["theta"], q["Bri"], q["Cri"], p["Dskip"], None, None,
                                          want_state=True, ck=ck, aux=aux)
        g = scan.unitary_bwd_raw(p["dy"], None, q["u"], q["delta"], p["theta"], q["Bri"], q["Cri"], p["Dskip"], hck, ck,
                                 aux=aux)
        torch.cuda.synchronize()
        outs.append((y, hL) + tuple(g[:6]))
    for name, a, b in zip(("y", "hL", "du", "ddelta", "dtheta", "dB", "dC", "dD"), *outs):
        _close(a, b.cpu(), name, tol=1e-5)


@pytest.mark.parametrize("seed", range(24))
def test_random_shapes_inputs_and_checkpoint_intervals(seed):
    """A seeded sweep over what the launcher has to get right together: partial channel groups and
    chunks, every N the matrix-core kernels serve, checkpoint intervals 32 / 64 / 256 (which also
    set the segment length of the split along L), float32 and bfloat16 inputs, output gate, carried
    state and upstream gradient of the final state.  Forward and backward through the raw wrappers
    against the CPU oracle on the same (for bf16: already rounded) values."""
    import random
    from aussm_amd import scan
    r = random.Random(1000 + seed)
    B, D, N = r.randint(1, 3), r.randint(1, 150), r.randint(6, 16)
    ck = r.choice([32, 64, 256])
    L = ck * r.randint(1, 6) if r.random() < 0.6 else 4 * r.randint(1, 160)
    lowp, gate, carried = r.random() < 0.4, r.random() < 0.5, r.random() < 0.5
    p = O.make_core_inputs(B, D, N, L, seed=seed, gate=gate)
    g = torch.Generator().manual_seed(seed)
    h0 = torch.complex(torch.randn(B, D, N, generator=g), torch.randn(B, D, N, generator=g)) if carried else None
    dh = torch.complex(torch.randn(B, D, N, generator=g), torch.randn(B, D, N, generator=g)) if carried else None
    if lowp:
        for k in ("u", "delta", "Bc", "Cc"):
            t = p[k]
            p[k] = (torch.view_as_complex(torch.view_as_real(t).bfloat16().float().contiguous()) if t.is_complex()
                    else t.bfloat16().float())
    # oracle (gradients of the gated output are only needed for the ungated backward kernel: gate off there)
    leaves = [p[k].clone().requires_grad_(True) for k in NAMES]
    h0l = h0.clone().requires_grad_(True) if carried else None
    y_want, hL_want = O.unitary_core_loop(*leaves, p.get("z"), h0l)
    y_ng, hL_ng = O.unitary_core_loop(*leaves, None, h0l)
    loss = (y_ng * p["dy"]).sum()
    if carried:
        loss = loss + (torch.view_as_real(hL_ng) * torch.view_as_real(dh)).sum()
    loss.backward()
    want = [t.grad for t in leaves]

    dt = torch.bfloat16 if lowp else torch.float32
    q = {k: v.cuda() for k, v in p.items()}
    u, de = q["u"].to(dt), q["delta"].to(dt)
    Bri = torch.view_as_real(q["Bc"]).to(dt).contiguous()
    Cri = torch.view_as_real(q["Cc"]).to(dt).contiguous()
    h0d = torch.view_as_real(h0).contiguous().cuda() if carried else None
    dhd = torch.view_as_real(dh).contiguous().cuda() if carried else None
    aux = scan.unitary_aux(u, N, ck)
    print(f"case sweep seed={seed} B={B} D={D} N={N} L={L} ck={ck} bf16={lowp} gate={gate} carried={carried}", flush=True)
    y, hL, _ = scan.unitary_fwd_raw(u, de, q["theta"], Bri, Cri, q["Dskip"], q.get("z"), h0d, want_state=True, ck=ck, aux=aux)
    _close(y, y_want.detach(), "y")
    _close(torch.view_as_complex(hL), hL_want.detach(), "hL")
    _, _, hck = scan.unitary_fwd_raw(u, de, q["theta"], Bri, Cri, q["Dskip"], None, h0d, want_state=False, ck=ck, aux=aux)
    du, dde, dth, dB, dC, dD, dh0 = scan.unitary_bwd_raw(q["dy"], dhd, u, de, q["theta"], Bri, Cri, q["Dskip"], hck, ck,
                                                         want_dh0=carried, aux=aux)
    torch.cuda.synchronize()
    got = (du, dde, dth, torch.view_as_complex(dB), torch.view_as_complex(dC), dD)
    for k, w, gt in zip(NAMES, want, got):
        _close(gt, w, f"d{k}")
    if carried:
        _close(torch.view_as_complex(dh0), h0l.grad, "dh0")


def test_forward_only_call_takes_the_split_too():
    """Without a backward pass unitary_scan allocates the auxiliary buffer only when the launch is
    split along L (configuration 1 of the benchmark contract, B=16 D=128 L=1024 forward only, is such a call): same outputs as with the split off."""
    from aussm_amd import scan
    B, D, N, L = 2, 64, 16, 1024
    p = _inputs(B, D, N, L, 77, big_theta=False)
    q = {k: v.cuda() for k, v in p.items()}
    want_y, want_h = O.unitary_core_loop(p["u"], p["delta"], p["theta"], p["Bc"], p["Cc"], p["Dskip"], p["z"], p["h0"])
    print("case forward-only split", flush=True)
    with torch.no_grad():
        y, hL = scan.unitary_scan(q["u"], q["delta"], q["theta"], q["Bc"], q["Cc"], q["Dskip"], q["z"], q["h0"],
                                  return_last_state=True)
        with _opts(split_cap=0):
            y0, hL0 = scan.unitary_scan(q["u"], q["delta"], q["theta"], q["Bc"], q["Cc"], q["Dskip"], q["z"], q["h0"],
                                        return_last_state=True)
    torch.cuda.synchronize()
    _close(y, want_y, "y")
    _close(hL, want_h, "hL")
    _close(y, y0.cpu(), "y split vs whole", tol=2e-5)
    assert not torch.equal(y, y0), "the split should have changed the association order"
