"""The shape-only ("fake" / meta) implementations of the two dispatcher operators
(schemas: extension-cpp/extension_cpp/csrc/cuda/ssm_adaptive_unitary_forward.cu:284-285).  They are
what tracing and fake-tensor propagation see; no device is needed to exercise them."""
import torch


def _meta_args(b=3, d=8, n=4, l=32):
    m = lambda *s: torch.empty(*s, device="meta")
    return [m(b, d, l), m(b, d, l), m(d, n, d), m(d, n), m(n), m(n), m(n), m(n), m(d), m(b, d, l), m(b, d, n), m(b, d, n)]


def test_forward_operator_on_meta_tensors():
    from aussm_amd import ops  # noqa: F401  (registers the operators)
    args = _meta_args()
    y, hr, hi = torch.ops.extension_cpp.ssm_adaptive_unitary(*args)
    assert y.shape == args[0].shape and y.device.type == "meta" and y.dtype == torch.float32
    assert hr.shape == args[10].shape and hi.shape == args[11].shape


def test_backward_operator_on_meta_tensors():
    from aussm_amd import ops  # noqa: F401
    args = _meta_args()
    grads = torch.ops.extension_cpp.ssm_adaptive_backward_unitary(args[0], args[10], args[11], *args)
    assert len(grads) == 12
    for g, a in zip(grads, args):
        assert g.shape == a.shape and g.device.type == "meta"


def test_fake_tensor_mode_propagates_shapes():
    from torch._subclasses.fake_tensor import FakeTensorMode
    from aussm_amd import ops  # noqa: F401
    with FakeTensorMode():
        args = [torch.empty(a.shape) for a in _meta_args(b=2, d=16, n=4, l=48)]
        y, hr, hi = torch.ops.extension_cpp.ssm_adaptive_unitary(*args)
        assert tuple(y.shape) == (2, 16, 48) and tuple(hr.shape) == (2, 16, 4) and tuple(hi.shape) == (2, 16, 4)
