"""The C-ABI library: it loads without a GPU and exports every symbol include/aussm_hip.h declares;
argument checks that need no device run here too (they return before any launch)."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "aussm_hip.h")


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(aussm_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_entry_points():
    names = declared_symbols()
    for must in ("aussm_unitary_fwd", "aussm_unitary_bwd", "aussm_complex_fwd", "aussm_complex_bwd",
                 "aussm_real_fwd", "aussm_real_bwd", "aussm_version", "aussm_error_string",
                 "aussm_unitary_fwd_aux", "aussm_unitary_bwd_aux", "aussm_unitary_aux_floats",
                 "aussm_causal_conv1d_fwd", "aussm_causal_conv1d_bwd", "aussm_swap_last2", "aussm_unitary_split_segments",
                 "aussm_set_option", "aussm_get_option"):
        assert must in names


def test_library_exports_every_declared_symbol():
    from aussm_amd import _lib
    if not os.path.exists(_lib.LIB_PATH):
        pytest.skip("library not built (python -m aussm_amd.build)")
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for name in declared_symbols():
        assert hasattr(lib, name), f"{name} is declared in the header but not exported"
    for name in _lib.EXPORTED:
        assert name in declared_symbols(), f"{name} is bound in Python but not declared in the header"


def test_argument_checks_without_a_device():
    from aussm_amd import _lib
    if not os.path.exists(_lib.LIB_PATH):
        pytest.skip("library not built")
    lib = _lib.load()
    assert lib.aussm_version() >= 100
    assert lib.aussm_num_checkpoints(2048, 256) == 8 and lib.aussm_num_checkpoints(33, 32) == 2
    assert lib.aussm_bwd_checkpoint_interval(0) == 0 and lib.aussm_bwd_checkpoint_interval(2) == 16
    one = ctypes.c_void_p(256)      # never dereferenced: every call below is rejected before launch
    null = None
    # NULL required pointer
    rc = lib.aussm_unitary_fwd(null, one, one, one, one, null, null, null, one, null, null, 1, 1, 1, 32, 32, 0, null)
    assert rc == -1 and b"NULL" in lib.aussm_error_string(rc)
    # state size out of range
    rc = lib.aussm_unitary_fwd(one, one, one, one, one, null, null, null, one, null, null, 1, 1, 65, 32, 32, 0, null)
    assert rc == -2
    # checkpoint interval not a multiple of the tile
    rc = lib.aussm_unitary_fwd(one, one, one, one, one, null, null, null, one, null, null, 1, 1, 1, 32, 48, 0, null)
    assert rc == -3
    # unknown dtype
    rc = lib.aussm_unitary_fwd(one, one, one, one, one, null, null, null, one, null, null, 1, 1, 1, 32, 32, 7, null)
    assert rc == -4
    # misaligned complex tensor
    rc = lib.aussm_unitary_fwd(one, one, one, ctypes.c_void_p(260), one, null, null, null, one, null, null,
                               1, 1, 1, 32, 32, 0, null)
    assert rc == -5
    # the auxiliary buffer: size query, alignment check, NULL accepted like the plain entry points
    # per-(b,d,l) part + tag, then per (batch element, 32-step chunk) one 30 KiB image of prepared operands for the
    # backward pass and one of 24 KiB for the forward pass
    img = lambda b, l: b * ((l + 31) // 32) * (1920 + 1536) * 4
    assert lib.aussm_unitary_aux_floats(32, 512, 16, 2048, 256) == 32 * 512 * 2048 + 64 + img(32, 2048)
    assert lib.aussm_unitary_aux_floats(0, 1, 1, 1, 32) == 0
    # few (batch, channel) pairs and a long sequence: room for the states of 64 segments of 256 steps
    assert lib.aussm_unitary_aux_floats(4, 256, 16, 16384, 256) == (4 * 256 * 16384 + 64 + 4 * 64 * 256 * (2 * 16 + 2)
                                                                    + img(4, 16384))
    # ... which needs whole checkpoint blocks per segment, and states the matrix-core kernels serve.  Where it does
    # not apply, the segment area is what the vector-ALU kernels' split takes: ns segments of whole checkpoint blocks
    # (the last one ragged), (2 n + 2) floats per (batch, segment, channel), rounded up to 64 floats
    def gen(b, d, n, l, ck):
        want = min(64, -(-256 // (b * -(-d // 64))))
        ls = -(-(-(-l // want)) // ck) * ck
        return -(-(b * -(-l // ls) * d * (2 * n + 2)) // 64) * 64
    assert gen(4, 256, 16, 16388, 256) == 4 * 13 * 256 * 34
    assert lib.aussm_unitary_aux_floats(4, 256, 16, 16384 + 4, 256) == (4 * 256 * (16384 + 4) + 64 + gen(4, 256, 16, 16388, 256)
                                                                        + img(4, 16388))
    # (sizes do not depend on the option table: below the state size the matrix-core kernels take by default the images
    # are still provided for, because an option can ask for those kernels)
    assert lib.aussm_unitary_aux_floats(4, 256, 4, 16384, 256) == (4 * 256 * 16384 + 64 + gen(4, 256, 4, 16384, 256)
                                                                   + img(4, 16384))
    # a shape only the vector-ALU kernels serve: no per-(b,d,l) part, no images
    assert lib.aussm_unitary_aux_floats(4, 256, 32, 16384, 256) == 64 + gen(4, 256, 32, 16384, 256)
    assert lib.aussm_unitary_aux_floats(32, 512, 32, 2048, 256) == 64
    lib.aussm_ssm_adaptive_unitary_workspace_floats.restype = ctypes.c_size_t
    w0 = lib.aussm_ssm_adaptive_unitary_workspace_floats(32, 256, 16, 720, 1)
    assert lib.aussm_set_option(5, 64) == 0 and lib.aussm_ssm_adaptive_unitary_workspace_floats(32, 256, 16, 720, 1) == w0
    assert lib.aussm_set_option(5, 1 << 20) == 0 and lib.aussm_ssm_adaptive_unitary_workspace_floats(32, 256, 16, 720, 1) == w0
    assert lib.aussm_set_option(5, -1) == 0
    # options: unset by default, settable, restorable
    assert lib.aussm_get_option(0) == -1 and lib.aussm_set_option(0, 3) == 0 and lib.aussm_get_option(0) == 3
    assert lib.aussm_set_option(0, -1) == 0 and lib.aussm_get_option(0) == -1 and lib.aussm_set_option(99, 1) == -2
    assert lib.aussm_unitary_split_segments(4, 256, 16, 16384, 256) == 16
    assert lib.aussm_unitary_split_segments(16, 128, 16, 1024, 256) == 4
    assert lib.aussm_unitary_split_segments(16, 128, 16, 1024, 128) == 8
    assert lib.aussm_unitary_split_segments(32, 512, 16, 2048, 256) == 1
    assert lib.aussm_unitary_split_segments(4, 256, 32, 16384, 256) == 16      # vector-ALU kernels: their own split
    assert lib.aussm_unitary_split_segments(4, 256, 16, 16386, 256) == 13
    rc = lib.aussm_unitary_fwd_aux(one, one, one, one, one, null, null, null, one, null, null, ctypes.c_void_p(260),
                                   1, 1, 1, 32, 32, 0, 1, null)
    assert rc == -5
    rc = lib.aussm_unitary_fwd_aux(null, one, one, one, one, null, null, null, one, null, null, null,
                                   1, 1, 1, 32, 32, 0, 1, null)
    assert rc == -1
    # u / delta shared by urep consecutive batch elements: urep must divide B
    rc = lib.aussm_unitary_fwd_aux(one, one, one, one, one, null, null, null, one, null, null, null,
                                   3, 1, 1, 32, 32, 0, 2, null)
    assert rc == -2
    rc = lib.aussm_unitary_bwd_aux(*([one] * 17), 3, 1, 1, 32, 32, 0, 0, null)
    assert rc == -2
    # the recomputing backward kernels insist on their checkpoint interval and on the state limit of the library
    args = [one] * 9 + [0] + [one] * 11 + [null]          # ..., z, dz, workspace
    assert lib.aussm_real_bwd(*args, 1, 1, 1, 32, 32, 0, null) == -3
    assert lib.aussm_real_bwd(*args, 1, 1, 65, 32, 16, 0, null) == -2
    # workspace for the split of the complex / real scans along the sequence: none for full launches
    lib.aussm_scan_workspace_floats.restype = ctypes.c_size_t
    assert lib.aussm_scan_workspace_floats(2, 32, 512, 16, 2048, 16, 0) == 0
    assert lib.aussm_scan_workspace_floats(0, 4, 256, 16, 16384, 16, 0) == 0       # the unitary scan has its own
    assert lib.aussm_scan_workspace_floats(2, 4, 256, 16, 16384, 16, 0) >= 4 * 16 * 256 * 18
    assert lib.aussm_scan_workspace_floats(1, 4, 256, 16, 16384, 16, 0) >= 4 * 16 * 256 * 34
    # bf16 inputs: float copies of B_t and C_t, and no call without the workspace that holds them
    assert lib.aussm_scan_workspace_floats(1, 32, 512, 16, 2048, 16, 1) == 2 * 32 * 16 * 2048 * 2
    assert lib.aussm_real_bwd(*args, 1, 1, 1, 32, 16, 1, null) == -1
    # the blocks' causal convolution: kernel length limit, overlapping rows, required pointers
    assert lib.aussm_causal_conv1d_fwd(one, one, null, one, 1, 8, 4, 9, 32, 4, null) == -2
    assert lib.aussm_causal_conv1d_fwd(one, one, null, one, 1, 8, 4, 4, 32, 3, null) == -2      # row stride < D
    assert lib.aussm_causal_conv1d_fwd(one, one, null, one, 2, 8, 4, 4, 16, 4, null) == -2      # batches overlap
    assert lib.aussm_causal_conv1d_fwd(null, one, null, one, 1, 8, 4, 4, 32, 4, null) == -1
    assert lib.aussm_causal_conv1d_bwd(one, one, one, one, null, null, 1, 8, 4, 4, 32, 4, null) == -1


def test_python_layer_fails_loudly_without_library(monkeypatch, tmp_path):
    from aussm_amd import _lib
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "missing.so"))
    with pytest.raises(_lib.AussmError):
        _lib.load()


@pytest.mark.gpu
def test_hbm_probe_computes_what_it_says():
    """The measurement aid of `bench.py --hbm-probe`: both access patterns write o1 = a + b c and o2 = 2 o1."""
    import torch
    from aussm_amd import _lib, scan
    lib = _lib.load()
    rows, L = 128, 192
    a, b, c = (torch.randn(rows, L, device="cuda") for _ in range(3))
    want = a.double() + b.double() * c.double()
    for pattern in (0, 1):
        o1, o2 = torch.zeros_like(a), torch.zeros_like(a)
        print(f"case hbm probe pattern {pattern}", flush=True)
        _lib.check(lib.aussm_hbm_probe(_lib.ptr(a), _lib.ptr(b), _lib.ptr(c), _lib.ptr(o1), _lib.ptr(o2), rows, L, pattern, 1,
                                       scan._stream()), "aussm_hbm_probe")
        torch.cuda.synchronize()
        torch.testing.assert_close(o1.double(), want, atol=1e-5, rtol=1e-5)
        torch.testing.assert_close(o2.double(), 2 * want, atol=2e-5, rtol=1e-5)
    one = ctypes.c_void_p(256)
    assert lib.aussm_hbm_probe(one, one, one, one, one, 100, 192, 0, 1, None) == -2      # rows not a multiple of 64
