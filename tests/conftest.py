import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

GOLDEN = os.path.join(ROOT, "tests", "golden")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def rel_l2(x, ref):
    x = np.asarray(x, dtype=np.complex128 if np.iscomplexobj(x) or np.iscomplexobj(ref) else np.float64)
    ref = np.asarray(ref, dtype=x.dtype)
    den = np.linalg.norm(ref.ravel())
    return float(np.linalg.norm((x - ref).ravel()) / (den if den > 0 else 1.0))


def mean_rel(x, ref):
    """The reference's is_close metric (endia/utils/array_conversions.mojo:63-135)."""
    from oracle.endia_ref import is_close_metric
    return is_close_metric(x, ref)


# Tolerance of the build: per-tensor relative error <= 1e-4 (the reference's own test tolerance,
# array_conversions.mojo:63-64), both as ||x - ref|| / ||ref|| and as the reference's mean relative metric.
RTOL = 1e-4


def assert_close(x, ref, tol=RTOL, what="", mean_tol=None):
    """Both metrics: ||x - ref||_2 / ||ref||_2 <= tol, and the reference's own is_close figure (mean over the elements
    of |x - ref| / max(|ref|, 1e-6), array_conversions.mojo:108-135) <= max(tol, 1e-4), its tests' tolerance, unless
    the caller states another bound for it (`mean_tol`) and why."""
    x, ref = np.asarray(x), np.asarray(ref)
    assert x.size == ref.size, "%s: size %s vs %s" % (what, x.shape, ref.shape)
    x = x.reshape(ref.shape)
    e = rel_l2(x, ref)
    assert np.isfinite(e) and e <= tol, "%s: relative L2 error %.3e > %.1e" % (what, e, tol)
    m = mean_rel(x, ref)
    bound = max(tol, RTOL) if mean_tol is None else mean_tol
    assert np.isfinite(m) and m <= bound, "%s: mean relative error %.3e > %.1e" % (what, m, bound)


@pytest.fixture(scope="session")
def golden():
    def load(name):
        return np.load(os.path.join(GOLDEN, name + ".npz"))
    return load


class Dev:
    """Thin helper over the C ABI for tests: device buffers in, numpy out."""

    def __init__(self):
        import ctypes
        from endia_amd import _lib as L
        self.L, self.ct = L, ctypes
        L.ensure_init()
        self._live = []

    def alloc(self, nbytes):
        p = self.ct.c_void_p()
        self.L.call("endia_hip_malloc", int(nbytes), self.ct.byref(p))
        self._live.append(p.value)
        return p.value

    def put(self, a):
        a = np.ascontiguousarray(a, dtype=np.complex64 if np.iscomplexobj(a) else np.float32)
        p = self.alloc(max(a.nbytes, 4))
        if a.nbytes:
            self.L.call("endia_hip_memcpy_h2d", p, a.ctypes.data, a.nbytes)
        return p

    def get(self, p, shape, dtype=np.float32):
        out = np.empty(shape, dtype=dtype)
        if out.nbytes:
            self.L.call("endia_hip_memcpy_d2h", out.ctypes.data, p, out.nbytes)
        return out

    def call(self, name, *args):
        self.L.call(name, *args)

    def release(self):
        for p in self._live:
            self.L.call("endia_hip_free", p)
        self._live = []


@pytest.fixture()
def dev():
    d = Dev()
    yield d
    d.release()
