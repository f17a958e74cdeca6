"""numpy front end of the CPU oracle (oracle/endia_ref.c). TEST INFRASTRUCTURE ONLY.

Only tests/, __graft_entry__.smoke() and the cpu_baseline leg of bench.py may import this module;
the product (endia_amd/) never does. Arrays are float32; complex arrays are numpy complex64 on this
side and interleaved (re, im) float32 inside the C library.
"""
import ctypes
import os
import subprocess
from ctypes import POINTER, c_float, c_int32, c_int64, c_uint32, c_void_p

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
# ENDIA_REF_LIB selects another build of the same source (the sanitizer build, oracle/Makefile)
LIB_PATH = os.environ.get("ENDIA_REF_LIB") or os.path.join(_HERE, "libendia_ref.so")

OP = dict(relu=0, tanh=1, sin=2, cos=3, neg=4, square=5, sqrt=6, abs=7, identity=8, greater0=9, exp=10, log=11,
          sigmoid=12, sinh=13, cosh=14, tan=15, asin=16, acos=17, atan=18, reciprocal=19, sign=20)
BIN = dict(add=0, sub=1, mul=2, div=3, greater=4, pow=5, greater_equal=6, less=7, less_equal=8, equal=9, not_equal=10)


def build():
    subprocess.run(["make", "-C", _HERE, "-B", "libendia_ref.so"], check=True, capture_output=True)
    return LIB_PATH


class ConvDesc(ctypes.Structure):
    _fields_ = [(n, c_int64) for n in (
        "N", "C", "H", "W", "K", "R", "S", "stride_h", "stride_w", "pad_h", "pad_w", "dil_h", "dil_w", "groups")]


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        _lib = ctypes.CDLL(LIB_PATH)
        _lib.ref_mlp_step.restype = c_float
    return _lib


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _ptr(a):
    return c_void_p(a.ctypes.data)


def _i64(v):
    v = list(v)
    return (c_int64 * max(len(v), 1))(*v)


def _elem_strides(a, itemsize):
    return [s // itemsize for s in a.strides]


def as_strided(x, shape, stride, offset=0):
    """as_strided followed by contiguous(): the gather of functional/_utils.mojo:79-205 over x's storage."""
    x = np.ascontiguousarray(x)
    cplx = np.iscomplexobj(x)
    x = x.astype(np.complex64 if cplx else np.float32)
    out = np.zeros(tuple(shape), dtype=x.dtype)
    lib().ref_strided_copy(c_int32(len(shape)), _i64(shape), _i64(stride), c_int64(offset), _ptr(x), _ptr(out),
                           c_int32(1 if cplx else 0))
    return out


def strided_scatter(src, target_shape, stride, offset=0, accumulate=False):
    """Pad.__call__ (accumulate False) / AsStridedInv.__call__ (True): src written or added through the view
    (src.shape, stride, offset) of a zero array of target_shape."""
    cplx = np.iscomplexobj(src)
    src = np.ascontiguousarray(src, dtype=np.complex64 if cplx else np.float32)
    out = np.zeros(tuple(target_shape), dtype=src.dtype)
    lib().ref_strided_scatter(c_int32(src.ndim), _i64(src.shape), _i64(stride), c_int64(offset), _ptr(src), _ptr(out),
                              c_int32(1 if accumulate else 0), c_int32(1 if cplx else 0))
    return out


def matmul(a, b):
    """matmul_fwd on 2-D or batched operands; a and b may be strided views (e.g. x.T)."""
    cplx = np.iscomplexobj(a) or np.iscomplexobj(b)
    dt = np.complex64 if cplx else np.float32
    a = np.asarray(a, dtype=dt)
    b = np.asarray(b, dtype=dt)
    batch_shape = np.broadcast_shapes(a.shape[:-2], b.shape[:-2])
    a = np.broadcast_to(a, batch_shape + a.shape[-2:])
    b = np.broadcast_to(b, batch_shape + b.shape[-2:])
    M, K = a.shape[-2:]
    K2, N = b.shape[-2:]
    assert K == K2
    out = np.zeros(batch_shape + (M, N), dtype=dt)
    fn = lib().ref_cmatmul if cplx else lib().ref_matmul
    # flatten batch dims one matrix at a time so arbitrary batch strides are honoured
    for idx in np.ndindex(*batch_shape):
        am, bm = a[idx], b[idx]
        isz = am.itemsize
        ars, acs = _elem_strides(am, isz)
        brs, bcs = _elem_strides(bm, isz)
        o = out[idx]
        fn(c_int64(1), c_int64(M), c_int64(N), c_int64(K), c_void_p(am.ctypes.data), c_int64(0), c_int64(ars),
           c_int64(acs), c_void_p(bm.ctypes.data), c_int64(0), c_int64(brs), c_int64(bcs), c_void_p(o.ctypes.data))
    return out


def unary(op, x):
    x = _f32(x)
    y = np.empty_like(x)
    lib().ref_unary(c_int32(OP[op]), c_int64(x.size), _ptr(x), _ptr(y))
    return y


def unary_vjp(op, x, g):
    x, g = _f32(x), _f32(g)
    dx = np.empty_like(x)
    lib().ref_unary_vjp(c_int32(OP[op]), c_int64(x.size), _ptr(x), _ptr(g), _ptr(dx))
    return dx


def unary_complex(op, z):
    """complex -> complex forward body of a unary op."""
    z = np.ascontiguousarray(z, dtype=np.complex64)
    y = np.empty_like(z)
    lib().ref_unary_complex(c_int32(OP[op]), c_int64(z.size), _ptr(z), _ptr(y))
    return y


def cabs(z):
    z = np.ascontiguousarray(z, dtype=np.complex64)
    y = np.empty(z.shape, dtype=np.float32)
    lib().ref_cabs(c_int64(z.size), _ptr(z), _ptr(y))
    return y


def cabs_vjp(z, g):
    z = np.ascontiguousarray(z, dtype=np.complex64)
    g = _f32(g)
    dz = np.empty_like(z)
    lib().ref_cabs_vjp(c_int64(z.size), _ptr(z), _ptr(g), _ptr(dz))
    return dz


def binary(op, a, b):
    """Broadcasting elementwise op (add, sub, mul, div, pow and the comparisons)."""
    cplx = np.iscomplexobj(a) or np.iscomplexobj(b)
    dt = np.complex64 if cplx else np.float32
    a = np.ascontiguousarray(a, dtype=dt)
    b = np.ascontiguousarray(b, dtype=dt)
    shape = np.broadcast_shapes(a.shape, b.shape)
    av, bv = np.broadcast_to(a, shape), np.broadcast_to(b, shape)
    out = np.empty(shape, dtype=dt)
    isz = a.itemsize
    lib().ref_binary(c_int32(BIN[op]), c_int32(len(shape)), _i64(shape), _i64(_elem_strides(av, isz)),
                     _i64(_elem_strides(bv, isz)), _ptr(a), _ptr(b), _ptr(out), c_int32(1 if cplx else 0))
    return out


def reduce_add(x, axes):
    """Sum over `axes`, keeping them as size 1 (ReduceAdd)."""
    cplx = np.iscomplexobj(x)
    x = np.ascontiguousarray(x, dtype=np.complex64 if cplx else np.float32)
    axes = [ax % x.ndim for ax in axes]
    mask = 0
    for ax in axes:
        mask |= 1 << ax
    oshape = tuple(1 if i in axes else s for i, s in enumerate(x.shape))
    out = np.zeros(oshape, dtype=x.dtype)
    lib().ref_reduce_add(c_int32(x.ndim), _i64(x.shape), c_uint32(mask), _ptr(x), _ptr(out), c_int32(1 if cplx else 0))
    return out


_REDUCE_OPS = {"max": 0, "min": 1, "mul": 2, "argmax": 3, "argmin": 4}


def reduce_op(kind, x, axes):
    """ReduceMax / ReduceMin / ReduceMul / ReduceArgMax / ReduceArgMin over `axes`, kept as size 1; the arg variants
    take one axis and return positions as floats."""
    x = _f32(x)
    axes = [ax % x.ndim for ax in ([axes] if isinstance(axes, int) else axes)]
    if kind.startswith("arg") and len(set(axes)) != 1:
        raise ValueError("argmax / argmin reduce one axis")
    mask = 0
    for ax in axes:
        mask |= 1 << ax
    out = np.zeros(tuple(1 if i in axes else s for i, s in enumerate(x.shape)), dtype=np.float32)
    lib().ref_reduce_op(c_int32(_REDUCE_OPS[kind]), c_int32(x.ndim), _i64(x.shape), c_uint32(mask), _ptr(x), _ptr(out))
    return out


def variance(x, axes=(0,), unbiased=True, keepdims=False):
    """variance_op.mojo:35-79 with the ops above: reduce_add, the count as a float, sub, mul, reduce_add, div."""
    x = _f32(x)
    axes = list(axes)
    res = reduce_add(x, axes)
    count = np.float32(x.size // max(res.size, 1))
    divisor = count - np.float32(1) if unbiased else count
    mean_res = binary("div", res, np.full((1,), count, np.float32))
    diff = binary("sub", x, mean_res)
    var = binary("div", reduce_add(binary("mul", diff, diff), axes), np.full((1,), divisor, np.float32))
    return var if keepdims else _squeeze(var)


def std(x, axes=(0,), unbiased=True, keepdims=False):
    """std_op.mojo:35-65."""
    return unary("sqrt", variance(x, axes, unbiased, keepdims))


def _squeeze(a):
    """Squeeze: every size-1 axis goes, one stays if all are (squeeze_op.mojo:31-60)."""
    shape = [s for s in a.shape if s != 1] or [1]
    return a.reshape(shape)


def mse(pred, target):
    """Returns (loss, dpred) as the reference's op chain produces them."""
    pred, target = _f32(pred), _f32(target)
    loss = np.zeros(1, dtype=np.float32)
    dpred = np.empty_like(pred)
    lib().ref_mse(c_int64(pred.size), _ptr(pred), _ptr(target), _ptr(loss), _ptr(dpred))
    return loss[0], dpred


def _desc(xshape, wshape, stride, padding, dilation):
    N, C, H, W = xshape
    K, C2, R, S = wshape
    assert C == C2
    return ConvDesc(N, C, H, W, K, R, S, stride[0], stride[1], padding[0], padding[1], dilation[0], dilation[1], 1)


def conv2d_out_shape(xshape, wshape, stride, padding, dilation):
    N, C, H, W = xshape
    K, _, R, S = wshape
    P = (H + 2 * padding[0] - dilation[0] * (R - 1) - 1) // stride[0] + 1
    Q = (W + 2 * padding[1] - dilation[1] * (S - 1) - 1) // stride[1] + 1
    return (N, K, P, Q)


def conv2d(x, w, bias=None, stride=(1, 1), padding=(0, 0), dilation=(1, 1)):
    x, w = _f32(x), _f32(w)
    d = _desc(x.shape, w.shape, stride, padding, dilation)
    y = np.empty(conv2d_out_shape(x.shape, w.shape, stride, padding, dilation), dtype=np.float32)
    b = _f32(bias) if bias is not None else None
    lib().ref_conv2d_fwd(ctypes.byref(d), _ptr(x), _ptr(w), _ptr(b) if b is not None else None, _ptr(y))
    return y


def conv2d_bwd(x, w, dy, stride=(1, 1), padding=(0, 0), dilation=(1, 1)):
    """Returns (dx, dw, db): the adjoints of the conv2d forward loop."""
    x, w, dy = _f32(x), _f32(w), _f32(dy)
    d = _desc(x.shape, w.shape, stride, padding, dilation)
    dx, dw, db = np.empty_like(x), np.empty_like(w), np.empty(w.shape[0], dtype=np.float32)
    lib().ref_conv2d_bwd(ctypes.byref(d), _ptr(x), _ptr(w), _ptr(dy), _ptr(dx), _ptr(dw), _ptr(db))
    return dx, dw, db


class PoolDesc(ctypes.Structure):
    _fields_ = [(n, c_int64) for n in ("N", "C", "D", "H", "W")] + [
        (n, c_int64 * 3) for n in ("kernel", "stride", "padding", "dilation")]


def _triple(v, n, fill):
    v = [v] if isinstance(v, int) else list(v)
    assert len(v) == n
    return [fill] * (3 - n) + v


def _pool_desc(xshape, kernel, stride, padding, dilation):
    nsp = len(xshape) - 2
    d = PoolDesc()
    d.N, d.C = xshape[0], xshape[1]
    d.D, d.H, d.W = [1] * (3 - nsp) + list(xshape[2:])
    d.kernel[:] = _triple(kernel, nsp, 1)
    d.stride[:] = _triple(stride, nsp, 1)
    d.padding[:] = _triple(padding, nsp, 0)
    d.dilation[:] = _triple(dilation, nsp, 1)
    return d, nsp


def pool(mode, x, kernel, stride=1, padding=0, dilation=1):
    """max / avg pooling of [N, C, spatial...] with 1 to 3 spatial axes."""
    x = _f32(x)
    nsp = x.ndim - 2
    stride, padding, dilation = ([v] * nsp if isinstance(v, int) else v for v in (stride, padding, dilation))
    d, nsp = _pool_desc(x.shape, kernel, stride, padding, dilation)
    o = (c_int64 * 3)()
    lib().ref_pool_out_shape(ctypes.byref(d), o)
    y = np.empty(tuple(x.shape[:2]) + tuple(o[3 - nsp:]), np.float32)
    lib().ref_pool_fwd(ctypes.byref(d), c_int32(0 if mode == "max" else 1), _ptr(x), _ptr(y))
    return y


def pool_bwd(mode, x, dy, kernel, stride=1, padding=0, dilation=1):
    x, dy = _f32(x), _f32(dy)
    nsp = x.ndim - 2
    stride, padding, dilation = ([v] * nsp if isinstance(v, int) else v for v in (stride, padding, dilation))
    d, nsp = _pool_desc(x.shape, kernel, stride, padding, dilation)
    dx = np.empty_like(x)
    lib().ref_pool_bwd(ctypes.byref(d), c_int32(0 if mode == "max" else 1), _ptr(x), _ptr(dy), _ptr(dx))
    return dx


class Conv3dDesc(ctypes.Structure):
    _fields_ = [(n, c_int64) for n in ("N", "C", "D", "H", "W", "K", "T", "R", "S")] + [
        (n, c_int64 * 3) for n in ("stride", "padding", "dilation")]


def _conv3d_desc(xshape, wshape, stride, padding, dilation):
    nsp = len(xshape) - 2
    d = Conv3dDesc()
    d.N, d.C, d.K = xshape[0], xshape[1], wshape[0]
    d.D, d.H, d.W = [1] * (3 - nsp) + list(xshape[2:])
    d.T, d.R, d.S = [1] * (3 - nsp) + list(wshape[2:])
    stride, padding, dilation = ([v] * nsp if isinstance(v, int) else list(v) for v in (stride, padding, dilation))
    d.stride[:] = _triple(stride, nsp, 1)
    d.padding[:] = _triple(padding, nsp, 0)
    d.dilation[:] = _triple(dilation, nsp, 1)
    o = (c_int64 * 3)()
    lib().ref_conv3d_out_shape(ctypes.byref(d), o)
    return d, tuple(o[3 - nsp:])


def convnd(x, w, bias=None, stride=1, padding=0, dilation=1):
    """conv1d / conv2d / conv3d by the rank of x ([N, C, spatial...]), via the 3-D loop."""
    x, w = _f32(x), _f32(w)
    d, osp = _conv3d_desc(x.shape, w.shape, stride, padding, dilation)
    y = np.empty((x.shape[0], w.shape[0]) + osp, np.float32)
    b = _f32(bias) if bias is not None else None
    lib().ref_conv3d(ctypes.byref(d), _ptr(x), _ptr(w), _ptr(b) if b is not None else None, _ptr(y), None, None, None, None)
    return y


def convnd_bwd(x, w, dy, stride=1, padding=0, dilation=1):
    x, w, dy = _f32(x), _f32(w), _f32(dy)
    d, _ = _conv3d_desc(x.shape, w.shape, stride, padding, dilation)
    dx, dw, db = np.empty_like(x), np.empty_like(w), np.empty(w.shape[0], np.float32)
    lib().ref_conv3d(ctypes.byref(d), _ptr(x), _ptr(w), None, None, _ptr(dy), _ptr(dx), _ptr(dw), _ptr(db))
    return dx, dw, db


def sgd(p, g, lr):
    p = _f32(p).copy()
    g = _f32(g)
    lib().ref_sgd(c_int64(p.size), _ptr(p), _ptr(g), c_float(lr))
    return p


def adam(p, g, m, v, lr=1e-3, b1=0.9, b2=0.999, eps=1e-8, t=1.0):
    p, m, v = _f32(p).copy(), _f32(m).copy(), _f32(v).copy()
    g = _f32(g)
    lib().ref_adam(c_int64(p.size), _ptr(p), _ptr(g), _ptr(m), _ptr(v), c_float(lr), c_float(b1), c_float(b2),
                   c_float(eps), c_float(t))
    return p, m, v


def sgd_momentum(p, g, vel, lr, momentum=0.0, weight_decay=0.0):
    p, vel = _f32(p).copy(), _f32(vel).copy()
    g = _f32(g)
    lib().ref_sgd_momentum(c_int64(p.size), _ptr(p), _ptr(g), _ptr(vel), c_float(lr), c_float(momentum), c_float(weight_decay))
    return p, vel


def adagrad(p, g, cache, lr=0.01, eps=1e-8):
    p, cache = _f32(p).copy(), _f32(cache).copy()
    g = _f32(g)
    lib().ref_adagrad(c_int64(p.size), _ptr(p), _ptr(g), _ptr(cache), c_float(lr), c_float(eps))
    return p, cache


def rmsprop(p, g, cache, lr=0.01, alpha=0.99, eps=1e-8):
    p, cache = _f32(p).copy(), _f32(cache).copy()
    g = _f32(g)
    lib().ref_rmsprop(c_int64(p.size), _ptr(p), _ptr(g), _ptr(cache), c_float(lr), c_float(alpha), c_float(eps))
    return p, cache


def mlp_step(widths, act, x, target, Ws, bs, opt="none", lr=1e-3, b1=0.9, b2=0.999, eps=1e-8, t=1.0, state=None):
    """One fwd + bwd (+ optimizer) step. Ws/bs are updated IN PLACE when opt != "none".

    Returns (loss, dWs, dbs). state = dict(mW=[...], vW=[...], mb=[...], vb=[...]) for Adam.
    """
    L = len(widths) - 1
    x, target = _f32(x), _f32(target)
    for l in range(L):
        assert Ws[l].dtype == np.float32 and Ws[l].flags.c_contiguous and Ws[l].shape == (widths[l], widths[l + 1])
        assert bs[l].dtype == np.float32 and bs[l].flags.c_contiguous
    dWs = [np.zeros_like(W) for W in Ws]
    dbs = [np.zeros((1, widths[l + 1]), dtype=np.float32) for l in range(L)]  # kept leading axis, as the reference
    PP = c_void_p * L

    def arr(lst):
        return PP(*[a.ctypes.data for a in lst])

    optc = dict(none=0, sgd=1, adam=2)[opt]
    if optc == 2:
        st = state
        mW, vW, mb, vb = arr(st["mW"]), arr(st["vW"]), arr(st["mb"]), arr(st["vb"])
    else:
        mW = vW = mb = vb = None
    loss = lib().ref_mlp_step(c_int32(L), _i64(widths), c_int64(x.shape[0]), c_int32(OP[act]), _ptr(x), _ptr(target),
                              arr(Ws), arr(bs), arr(dWs), arr(dbs), c_int32(optc), c_float(lr), c_float(b1),
                              c_float(b2), c_float(eps), c_float(t), mW, vW, mb, vb)
    return float(loss), dWs, dbs


def is_close_metric(x, ref):
    """The reference's comparison metric (endia/utils/array_conversions.mojo:63-135): mean over elements
    of |x - ref| / max(|ref|, floor); floor 1e-6 (real) or 1e-9 (complex, on |ref|)."""
    x, ref = np.asarray(x), np.asarray(ref)
    if np.iscomplexobj(ref) or np.iscomplexobj(x):
        mag = np.maximum(np.abs(ref), 1e-9)
        d = (np.abs(x.real - ref.real) + np.abs(x.imag - ref.imag)) / mag
    else:
        d = np.abs(x.astype(np.float64) - ref.astype(np.float64)) / np.maximum(np.abs(ref), 1e-6)
    return float(d.mean()) if d.size else 0.0
