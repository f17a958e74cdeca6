"""Comparison helpers: the host-side mirror of endia/utils/array_conversions.mojo."""
import numpy as np


def to_numpy(x):
    return x.to_numpy()


def relative_difference(x, ref):
    """The metric behind the reference's is_close (array_conversions.mojo:63-135): the MEAN over elements
    of |x - ref| / max(|ref|, floor), floor = 1e-6 for real data and 1e-9 on |ref| for complex data."""
    x = x.to_numpy() if hasattr(x, "to_numpy") else np.asarray(x)
    ref = np.asarray(ref).reshape(x.shape) if np.asarray(ref).size == x.size else np.asarray(ref)
    if np.iscomplexobj(x) or np.iscomplexobj(ref):
        mag = np.maximum(np.abs(ref), 1e-9)
        d = (np.abs(x.real - ref.real) + np.abs(x.imag - ref.imag)) / mag
    else:
        d = np.abs(x.astype(np.float64) - ref.astype(np.float64)) / np.maximum(np.abs(ref.astype(np.float64)), 1e-6)
    return float(d.mean()) if d.size else 0.0


def is_close(x, ref, rtol=10e-5):
    return relative_difference(x, ref) <= rtol
