"""The C-ABI library loads without a GPU, exports every symbol the header declares, and refuses to
compute before endia_hip_init (no silent CPU path)."""
import ctypes
import os
import re

import pytest

from conftest import ROOT
from endia_amd import _lib as L

HEADER = os.path.join(ROOT, "include", "endia_hip.h")


def declared_symbols():
    text = open(HEADER).read()
    return sorted(set(re.findall(r"ENDIA_API\s+[\w\s\*]+?\b(endia_hip_\w+)\s*\(", text)))


def test_header_declares_something():
    syms = declared_symbols()
    assert len(syms) >= 30 and "endia_hip_sgemm" in syms and "endia_hip_adam_step" in syms


def test_every_declared_symbol_is_exported():
    handle = ctypes.CDLL(L.LIB_PATH)
    missing = [s for s in declared_symbols() if not hasattr(handle, s)]
    assert not missing, "declared in include/endia_hip.h but not exported: %s" % missing


def test_python_binding_covers_the_header():
    bound = set(L.SIGNATURES) | {"endia_hip_last_error"}
    assert set(declared_symbols()) == bound


def test_calls_fail_loudly_without_init():
    import torch  # noqa: F401  (device probe only)
    if torch.cuda.is_available():
        pytest.skip("a GPU is present; the not-initialised path is covered on CPU hosts")
    lib = L.lib()
    assert lib.endia_hip_sgd_step(4, None, None, ctypes.c_float(0.1)) == L.ERR_NOT_INIT
    assert b"endia_hip_init" in lib.endia_hip_last_error()
    rc = lib.endia_hip_init(0)
    assert rc == L.ERR_RUNTIME and b"no HIP device" in lib.endia_hip_last_error()
    with pytest.raises(L.EndiaHipError):
        import endia_amd as nd
        nd.zeros([4])


def test_conv_out_shape_needs_no_device():
    # shape rule conv2d_op.mojo:65-84; stride 2 / pad 1 case of test_conv2d_op.mojo
    d = L.Conv2dDesc(2, 3, 9, 10, 4, 3, 2, 2, 2, 1, 1, 1, 1, 1)
    P, Q = ctypes.c_int64(), ctypes.c_int64()
    assert L.lib().endia_hip_conv2d_out_shape(ctypes.byref(d), ctypes.byref(P), ctypes.byref(Q)) == 0
    assert (P.value, Q.value) == (5, 6)
    d.groups = 2
    assert L.lib().endia_hip_conv2d_out_shape(ctypes.byref(d), ctypes.byref(P), ctypes.byref(Q)) == L.ERR_UNSUPPORTED
