"""Committed fixtures (tests/golden/scan_fixtures.npz, written by tests/golden/make_fixtures.py):
the float32 oracle must reproduce them on the CPU, and the HIP operators on the GPU."""
import os

import numpy as np
import pytest
import torch

from oracle import scan_oracle as O

FIX = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "scan_fixtures.npz"))


def t(name):
    return torch.from_numpy(FIX[name])


def c(name):
    return torch.view_as_complex(t(name).contiguous())


def core_inputs(variant):
    g = lambda k: t(f"{variant}_{k}")
    if variant == "real":
        return [g("u"), g("delta"), g("A"), g("Bm"), g("Cm"), g("Dskip"), g("z")]
    mid = [g("theta")] if variant == "unitary" else [g("rho"), g("theta")]
    return [g("u"), g("delta")] + mid + [c(f"{variant}_Bc"), c(f"{variant}_Cc"), g("Dskip"), g("z")]


ORACLE = {"unitary": O.unitary_core_loop, "complex": O.complex_core_loop, "real": O.real_core_loop}


@pytest.mark.parametrize("variant", ["unitary", "complex", "real"])
def test_oracle_reproduces_fixtures(variant):
    y, h = ORACLE[variant](*core_inputs(variant))
    torch.testing.assert_close(y, t(f"{variant}_y"), atol=2e-5, rtol=2e-5)
    want_h = c(f"{variant}_hL") if variant != "real" else t("real_hL")
    torch.testing.assert_close(h, want_h, atol=2e-5, rtol=2e-5)


def test_oracle_reproduces_adaptive_fixture():
    args = [t(f"adaptive_{k}") for k in ("u", "dt", "x", "x_bias")] + [c("adaptive_B"), c("adaptive_C")] + \
           [t("adaptive_D"), t("adaptive_z")]
    torch.testing.assert_close(O.adaptive_unitary_loop(*args), t("adaptive_y"), atol=7e-5, rtol=5e-5)
    torch.testing.assert_close(O.adaptive_unitary_polar(*args), t("adaptive_y"), atol=7e-5, rtol=5e-5)


@pytest.mark.gpu
@pytest.mark.parametrize("variant", ["unitary", "complex", "real"])
def test_hip_reproduces_fixtures(variant):
    from aussm_amd import scan
    fn = {"unitary": scan.unitary_scan, "complex": scan.complex_scan}.get(variant)
    ins = [a.cuda() for a in core_inputs(variant)]
    if variant == "real":
        y, h = scan.selective_scan_fn(*ins[:6], z=ins[6], return_last_state=True)
        want_h = t("real_hL")
    else:
        y, h = fn(*ins, return_last_state=True)
        h, want_h = torch.view_as_real(h), t(f"{variant}_hL")
    torch.testing.assert_close(y.cpu(), t(f"{variant}_y"), atol=1e-4, rtol=1e-4)
    torch.testing.assert_close(h.cpu(), want_h, atol=1e-4, rtol=1e-4)


@pytest.mark.gpu
def test_hip_reproduces_adaptive_fixture():
    from aussm_amd import ops
    args = [t(f"adaptive_{k}") for k in ("u", "dt", "x", "x_bias")] + [c("adaptive_B"), c("adaptive_C")] + \
           [t("adaptive_D"), t("adaptive_z")]
    y = ops.ssm_adaptive_interface(*[a.cuda() for a in args], unitary=True)
    torch.testing.assert_close(y.cpu(), t("adaptive_y"), atol=7e-5, rtol=5e-5)


def test_oracle_reproduces_conv_fixture():
    y = O.causal_conv1d_bld(t("conv_x"), t("conv_w"), t("conv_b"))
    torch.testing.assert_close(y, t("conv_y"), atol=1e-6, rtol=1e-6)


@pytest.mark.gpu
def test_hip_reproduces_conv_fixture():
    from aussm_amd import conv
    y = conv.causal_conv1d(t("conv_x").cuda(), t("conv_w").cuda(), t("conv_b").cuda())
    torch.testing.assert_close(y.cpu(), t("conv_y"), atol=1e-5, rtol=1e-5)
