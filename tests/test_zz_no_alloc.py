"""aussm_unitary_fwd_static, the entry point that allocates nothing: its workspace (the segment
states of a launch that is split along L) is a device array inside the library.  Called through the
C ABI and compared with aussm_unitary_fwd_aux on the same inputs (the benchmark contract's 1e-4 is
the bar; with the workspace entry point told to run the same kernel family - the static one has no
room for prepared operands - the results are equal bit for bit), twice in a row, the second call on
a smaller input, and once more on a shape that does not need the workspace at all."""
import pytest
import torch

from oracle import scan_oracle as O

pytestmark = pytest.mark.gpu


def _run_both(B, D, N, L, seed, gate, fwd_mode=None):
    from aussm_amd import scan, _lib
    lib = _lib.load()
    p = O.make_core_inputs(B, D, N, L, seed=seed, gate=gate)
    q = {k: v.cuda() for k, v in p.items()}
    g = torch.Generator().manual_seed(seed + 100)
    h0 = torch.view_as_real(torch.complex(torch.randn(B, D, N, generator=g), torch.randn(B, D, N, generator=g))).contiguous().cuda()
    Bri = torch.view_as_real(q["Bc"]).contiguous()
    Cri = torch.view_as_real(q["Cc"]).contiguous()
    ck = scan.unitary_ck(B, D, N, L)
    ptr, stream = scan.ptr, scan._stream()
    z = q.get("z")
    # the existing entry point, workspace from torch
    aux = scan.unitary_aux(q["u"], N, ck)
    y_ref = torch.empty((B, D, L), device="cuda")
    h_ref = torch.empty((B, D, N, 2), device="cuda")
    with _lib.options(unitary_fwd=fwd_mode):
        scan.check(lib.aussm_unitary_fwd_aux(ptr(q["u"]), ptr(q["delta"]), ptr(q["theta"]), ptr(Bri), ptr(Cri),
                                             ptr(q["Dskip"]), ptr(z), ptr(h0), ptr(y_ref), ptr(h_ref), None, ptr(aux),
                                             B, D, N, L, ck, 0, 1, stream), "aussm_unitary_fwd_aux")
    # the entry point under test: inputs and outputs only
    y = torch.full((B, D, L), float("nan"), device="cuda")
    hL = torch.full((B, D, N, 2), float("nan"), device="cuda")
    scan.check(lib.aussm_unitary_fwd_static(ptr(q["u"]), ptr(q["delta"]), ptr(q["theta"]), ptr(Bri), ptr(Cri),
                                            ptr(q["Dskip"]), ptr(z), ptr(h0), ptr(y), ptr(hL), B, D, N, L, ck, 0, stream),
               "aussm_unitary_fwd_static")
    torch.cuda.synchronize()
    return (y, hL), (y_ref, h_ref), lib.aussm_unitary_split_segments(B, D, N, L, ck)


def test_static_entry_point_matches_the_workspace_one_twice_in_a_row():
    from aussm_amd import scan, _lib
    lib = _lib.load()
    scan.check(lib.aussm_static_init(), "aussm_static_init")
    for B, D, N, L, seed, gate in ((4, 128, 16, 2048, 21, False), (2, 64, 16, 1024, 22, True), (3, 200, 12, 260, 23, False)):
        print(f"case static B={B} D={D} N={N} L={L}", flush=True)
        (y, hL), (y_ref, h_ref), ns = _run_both(B, D, N, L, seed, gate)
        if L >= 1024:
            assert ns > 1, "the shape was chosen so that the launch is split and the workspace is used"
        torch.testing.assert_close(y, y_ref, atol=1e-4, rtol=1e-4)
        torch.testing.assert_close(hL, h_ref, atol=1e-4, rtol=1e-4)
        # the kernels that build their operands themselves (what a call without room for prepared operands runs)
        (y, hL), (y_ref, h_ref), _ = _run_both(B, D, N, L, seed, gate, fwd_mode=3)
        assert torch.equal(y, y_ref) and torch.equal(hL, h_ref), "same kernels on the same inputs: bit for bit"


def test_static_entry_point_rejects_what_does_not_fit():
    import ctypes
    from aussm_amd import _lib
    lib = _lib.load()
    one = ctypes.c_void_p(256)          # never dereferenced: the call is rejected before any launch
    # B=4 D=256 N=16 L=16384: 64 fine segments -> 2.2 M floats of segment states, more than the static 4 MiB
    rc = lib.aussm_unitary_fwd_static(one, one, one, one, one, None, None, None, one, None, 4, 256, 16, 16384, 256, 0, None)
    assert rc == -6 and b"scratch" in lib.aussm_error_string(rc)
