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


def test_mojo_binding_names_every_symbol():
    """bindings/endia_hip.mojo (source only: no Mojo toolchain here) declares one method per exported entry point."""
    text = open(os.path.join(ROOT, "bindings", "endia_hip.mojo")).read()
    missing = [s for s in declared_symbols() if '"%s"' % s not in text]
    assert not missing, "not bound in bindings/endia_hip.mojo: %s" % missing
    for signature in ("fn matmul_fwd(inout curr: Array, args: List[Array]) raises",
                      "fn matmul_vjp(primals: List[Array], grad: Array, out: Array) raises -> List[Array]"):
        assert signature in text  # the reference's op interface (endia/functional/_utils.mojo:208-239)


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


@pytest.mark.parametrize("lang", [("c", "-std=c99"), ("c", "-std=c11"), ("c++", "-std=c++11")])
def test_header_is_plain_c(lang, tmp_path):
    """The header compiles on its own as strict C and as C++ (no torch or HIP types in the boundary)."""
    import subprocess
    unit = tmp_path / ("only_header.c" if lang[0] == "c" else "only_header.cpp")
    unit.write_text('#include "endia_hip.h"\nint unit_is_not_empty;\n')
    cc = "gcc" if lang[0] == "c" else "g++"
    res = subprocess.run([cc, lang[1], "-Wall", "-Wextra", "-pedantic", "-Werror", "-fsyntax-only", "-I",
                          os.path.join(ROOT, "include"), str(unit)], capture_output=True, text=True)
    assert res.returncode == 0, res.stderr


def test_c_client_builds_and_fails_loudly_without_a_device():
    """tests/c_abi/train_step.c links against the library through the header alone; without a GPU its
    first call reports the missing device (exit 2) instead of computing anything on the host."""
    import subprocess
    import torch
    exe = os.path.join(ROOT, "tests", "c_abi", "train_step")
    if not os.path.exists(exe):
        import __graft_entry__ as G
        G.build_c_client()
    if torch.cuda.is_available():
        pytest.skip("a GPU is present; the client's numerical check runs in the gpu tests")
    res = subprocess.run([exe], capture_output=True, text=True, timeout=60)
    assert res.returncode == 2 and "no HIP device" in res.stderr, (res.returncode, res.stderr)


@pytest.mark.gpu
def test_c_client_trains_one_step_on_the_device():
    """The plain-C client runs forward, backward and the SGD update of a two-layer MLP through the C ABI
    and compares every tensor with its own double-precision loops (1e-4 relative, checked in the client)."""
    import subprocess
    exe = os.path.join(ROOT, "tests", "c_abi", "train_step")
    assert os.path.exists(exe), "tests/c_abi/train_step is built by __graft_entry__.build()"
    res = subprocess.run([exe], capture_output=True, text=True, timeout=100)
    print(res.stdout, res.stderr)
    assert res.returncode == 0, (res.returncode, res.stdout, res.stderr)
    assert "worst relative error" in res.stdout


def test_col_sum_plan_clamps_to_the_scratch():
    """The row splits of a column sum, a host-side computation (no device): with unlimited scratch a 4096 x 4096 input
    on 256 CUs is cut into 64 pieces; the 262144 floats of endia_hip_col_sum_static allow exactly those 64 (which is why
    that entry point agrees with endia_hip_reduce_add bit for bit there); less scratch, or a device with more CUs,
    forces fewer pieces, down to refusing columns that do not fit at all; a small input needs no first stage."""
    lib = L.lib()

    def plan(R, C, cus, scratch, aligned=1):
        S, rows = ctypes.c_int64(), ctypes.c_int64()
        assert lib.endia_hip_col_sum_plan(R, C, cus, scratch, aligned, ctypes.byref(S), ctypes.byref(rows)) == 0
        return S.value, rows.value

    assert plan(4096, 4096, 256, 0) == (64, 64)
    assert plan(4096, 4096, 256, 1 << 18) == (64, 64)
    assert plan(4096, 4096, 256, 1 << 16) == (16, 256)        # room for 16 partial rows only
    assert plan(4096, 4096, 1024, 0) == (64, 64) and plan(4096, 4096, 1024, 1 << 17) == (32, 128)
    assert plan(24, 1 << 18, 256, 1 << 18) == (1, 24)
    assert plan(24, (1 << 18) + 4, 256, 1 << 18)[0] == -1      # does not fit
    assert plan(40, 96, 256, 1 << 18) == (0, 40)               # one launch
    assert plan(1024, 2048, 256, 0) == (0, 1024)               # a mid-size aligned input: one launch as well
    assert plan(1024, 2048, 256, 0, aligned=0)[0] >= 1         # ... unless it cannot be read 16 bytes at a time
    assert plan(1024, 2050, 256, 0)[0] >= 1
    for R, C, cus, scratch in [(5000, 772, 256, 1 << 18), (100000, 64, 304, 4096), (2000, 5000, 8, 0)]:
        S, rows = plan(R, C, cus, scratch)
        assert S >= 1 and (S - 1) * rows < R <= S * rows and (scratch == 0 or S * C <= scratch)
    assert lib.endia_hip_col_sum_plan(0, 4, 256, 0, 1, None, None) == L.ERR_INVALID
