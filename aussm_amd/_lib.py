"""ctypes binding of libaussm_hip.so (declarations: include/aussm_hip.h).

The library is the only compute path of this package: if it is missing or a
call fails, an exception is raised — there is no fallback.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_int, c_void_p

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libaussm_hip.so")

F32, BF16 = 0, 1
TILE = 32
AUX_PAD = 64          # floats between the per-(b,d,l) part of the auxiliary buffer and the segment states
MAX_STATE = 64
VAR_UNITARY, VAR_COMPLEX, VAR_REAL = 0, 1, 2   # variant codes of the C ABI

_lib = None

_P = c_void_p
_I = c_int
_LL = ctypes.c_longlong

# name -> argtypes; every entry point returns int
_SIGNATURES = {
    "aussm_version": [],
    "aussm_set_option": [_I, _I],
    "aussm_get_option": [_I],
    "aussm_num_checkpoints": [_I, _I],
    "aussm_bwd_checkpoint_interval": [_I],
    "aussm_unitary_split_segments": [_I] * 5,
    "aussm_unitary_kernel_mode": [_I] * 9,
    "aussm_unitary_fwd": [_P] * 11 + [_I] * 6 + [_P],
    "aussm_unitary_bwd": [_P] * 16 + [_I] * 6 + [_P],
    "aussm_unitary_fwd_aux": [_P] * 12 + [_I] * 7 + [_P],
    "aussm_unitary_bwd_aux": [_P] * 17 + [_I] * 7 + [_P],
    "aussm_static_init": [],
    "aussm_unitary_fwd_static": [_P] * 10 + [_I] * 6 + [_P],
    "aussm_complex_fwd": [_P] * 13 + [_I] * 6 + [_P],
    "aussm_complex_bwd": [_P] * 22 + [_I] * 6 + [_P],
    "aussm_real_fwd": [_P] * 8 + [_I] + [_P] * 5 + [_I] * 6 + [_P],
    "aussm_real_bwd": [_P] * 9 + [_I] + [_P] * 12 + [_I] * 6 + [_P],
    "aussm_causal_conv1d_fwd": [_P] * 4 + [_I] * 4 + [_LL] * 2 + [_P],
    "aussm_causal_conv1d_bwd": [_P] * 6 + [_I] * 4 + [_LL] * 2 + [_P],
    "aussm_swap_last2": [_P] * 2 + [_I] * 3 + [_LL] * 2 + [_P],
    "aussm_swap_last2_act": [_P] * 4 + [_I] * 3 + [_LL] * 4 + [_I] * 2 + [_P],
    "aussm_gate_fwd": [_P] * 3 + [ctypes.c_size_t, _P],
    "aussm_gate_bwd": [_P] * 5 + [ctypes.c_size_t, _P],
    "aussm_hbm_probe": [_P] * 5 + [_I] * 4 + [_P],
    "aussm_ssm_adaptive_unitary_fwd": [_P] * 16 + [_I] * 4 + [_P],
    "aussm_ssm_adaptive_unitary_bwd": [_P] * 30 + [_I] * 4 + [_P],
}

EXPORTED = tuple(_SIGNATURES) + ("aussm_error_string", "aussm_unitary_aux_floats",
                                 "aussm_ssm_adaptive_unitary_workspace_floats", "aussm_scan_workspace_floats")


OPT_UNITARY_FWD, OPT_UNITARY_BWD, OPT_SPLIT_CAP, OPT_GENERIC_NW, OPT_GENERIC_NT, OPT_BLOCK_KFLOATS = range(6)


class AussmError(RuntimeError):
    pass


def load() -> ctypes.CDLL:
    """Load the HIP library (once).  Raises AussmError if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    # PyTorch ships its own HIP runtime.  It has to be in the process before this library is
    # opened so that both resolve to the same runtime (two runtimes in one process do not share
    # a device context).
    import torch  # noqa: F401
    if not os.path.exists(LIB_PATH):
        raise AussmError(
            f"{LIB_PATH} not found: build it with `python -m aussm_amd.build` "
            "(the HIP library is required; there is no CPU fallback)")
    lib = ctypes.CDLL(LIB_PATH)
    for name, argtypes in _SIGNATURES.items():
        fn = getattr(lib, name)
        fn.argtypes = argtypes
        fn.restype = c_int
    lib.aussm_unitary_aux_floats.argtypes = [_I, _I, _I, _I, _I]
    lib.aussm_unitary_aux_floats.restype = ctypes.c_size_t
    lib.aussm_ssm_adaptive_unitary_workspace_floats.argtypes = [_I, _I, _I, _I, _I]
    lib.aussm_ssm_adaptive_unitary_workspace_floats.restype = ctypes.c_size_t
    lib.aussm_scan_workspace_floats.argtypes = [_I] * 7
    lib.aussm_scan_workspace_floats.restype = ctypes.c_size_t
    lib.aussm_error_string.argtypes = [c_int]
    lib.aussm_error_string.restype = c_char_p
    _lib = lib
    return lib


def check(code: int, what: str) -> None:
    if code != 0:
        msg = load().aussm_error_string(code).decode()
        raise AussmError(f"{what} failed with code {code}: {msg}")


def ptr(t) -> c_void_p | None:
    """Device pointer of a tensor (None -> NULL)."""
    return None if t is None else c_void_p(t.data_ptr())


class options:
    """Context manager: library options (aussm_set_option) for the duration of a block, e.g.
    `with options(unitary_fwd=0, split_cap=0): ...`; the previous values come back on exit."""
    _KEYS = {"unitary_fwd": OPT_UNITARY_FWD, "unitary_bwd": OPT_UNITARY_BWD, "split_cap": OPT_SPLIT_CAP,
             "generic_nw": OPT_GENERIC_NW, "generic_nt": OPT_GENERIC_NT, "block_kfloats": OPT_BLOCK_KFLOATS}

    def __init__(self, **kw):
        self.kw = {self._KEYS[k]: (-1 if v is None else int(v)) for k, v in kw.items()}

    def __enter__(self):
        lib = load()
        self.old = {k: lib.aussm_get_option(k) for k in self.kw}
        for k, v in self.kw.items():
            check(lib.aussm_set_option(k, v), "aussm_set_option")
        return self

    def __exit__(self, *exc):
        lib = load()
        for k, v in self.old.items():
            lib.aussm_set_option(k, v)
        return False
