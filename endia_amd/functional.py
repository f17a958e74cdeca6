"""Functional ops: forward kernels and VJP rules, the host-side mirror of endia/functional/.

Each op is registered the way the reference's `op_array` does it
(endia/functional/_utils.mojo:208-316): the forward body runs eagerly, and when any argument
requires a gradient the output keeps its arguments and its `vjp(primals, grad, out)` rule. VJP rules
are written in terms of these same ops, so a gradient built with `create_graph=True` is itself a
differentiable graph, which is the reference's whole higher-order mechanism
(endia/autograd/functional.mojo:63-65). A primal that does not require a gradient gets `None`, the
counterpart of the reference's `Array(0)` placeholder.

Every forward body is one or two calls into libendia_hip.so.
"""
import numpy as np

from . import _lib as L
from ._array import Array, Buffer, _contiguous_copy, _prod, contiguous_strides


# --------------------------------------------------------------------------------------------------
# registration
# --------------------------------------------------------------------------------------------------
_in_rule = [False]  # set by the reverse walk while a VJP rule runs


def _register(out, args, name, vjp, meta=None):
    out._name = name
    if _in_rule[0]:
        out._internal = True  # made by a VJP rule: no user code holds this node
    if any(a._requires_grad for a in args):
        out._requires_grad = True
        out._args = list(args)
        out._vjp = vjp
        out._meta = meta
    return out


def _view(base, shape, strides, offset, args, name, vjp, meta=None, is_complex=None):
    out = Array(shape, is_complex=base.is_complex_ if is_complex is None else is_complex, _buffer=base._buf,
                _strides=strides, _offset=offset)
    return _register(out, args, name, vjp, meta)


def contiguous(x):
    """contiguous(): functional/_utils.mojo:201-205 (a strided gather copy when x is a view)."""
    return x if x.is_contiguous() else _contiguous_copy(x)


_fusion = None  # set by endia_amd.fusion: while it traces a function, ops on its symbols build an expression
_fused_rules = {}


def _fused_rule(name, fn):
    """A VJP rule written in elementwise ops, as ONE differentiable fused launch (endia_amd.fusion). Used by passes that
    record their own graph (create_graph=True): the reference records two to four elementwise nodes per rule there
    (e.g. cos and mul for sin_op.mojo:92), and a second-order pass then pays one launch per node and per node's rule."""
    f = _fused_rules.get(name)
    if f is None:
        f = _fused_rules[name] = _fusion.fuse(fn, name)
    return f


def detach(x):
    if _fusion is not None and _fusion.tracing(x):
        return x
    return Array(x._shape, is_complex=x.is_complex_, _buffer=x._buf, _strides=x._strides, _offset=x._offset)


# --------------------------------------------------------------------------------------------------
# creation (init_ops.mojo). Random data is generated on the host with a seeded numpy Generator: the
# reference's generators are time-seeded (init_ops.mojo:230,260) and cannot be reproduced.
# --------------------------------------------------------------------------------------------------
_rng = np.random.default_rng(0)


def seed(s):
    global _rng
    _rng = np.random.default_rng(s)


def array(data, requires_grad=False):
    return Array.from_numpy(np.asarray(data), requires_grad=requires_grad)


def zeros(shape, requires_grad=False, is_complex=False):
    return Array(shape, requires_grad=requires_grad, is_complex=is_complex)


def full(shape, value, requires_grad=False):
    out = Array.empty(shape)
    L.call("endia_hip_fill", out.data_ptr(), out.size(), float(value))
    out._requires_grad = requires_grad
    return out


def ones(shape, requires_grad=False):
    return full(shape, 1.0, requires_grad)


def eye(n, requires_grad=False):
    return array(np.eye(n, dtype=np.float32), requires_grad)


def arange(start, end, step=1.0, requires_grad=False):
    return array(np.arange(start, end, step, dtype=np.float32), requires_grad)


def randn(shape, mean=0.0, std=1.0, requires_grad=False):
    return array((_rng.standard_normal(tuple(shape)) * std + mean).astype(np.float32), requires_grad)


def randu(shape, min=0.0, max=1.0, requires_grad=False):
    return array(_rng.uniform(min, max, tuple(shape)).astype(np.float32), requires_grad)


def randn_complex(shape, requires_grad=False):
    z = _rng.standard_normal(tuple(shape)) + 1j * _rng.standard_normal(tuple(shape))
    return array(z.astype(np.complex64), requires_grad)


def rand_he_normal(shape, fan_in, requires_grad=False):
    """He-normal init, std = sqrt(2 / fan_in): init_ops.mojo:285-287."""
    return randn(shape, 0.0, float(np.sqrt(2.0 / fan_in)), requires_grad)


def linspace(start=0.0, end=1.0, num=50, requires_grad=False):
    """init_ops.mojo:94-107: start, then `num - 1` additions of the fp32 step (so the last value carries their rounding)."""
    step = (np.float32(end) - np.float32(start)) / np.float32(num - 1)
    out, value = np.empty(num, np.float32), np.float32(start)
    for i in range(num):
        out[i] = value
        value = np.float32(value + step)
    return array(out, requires_grad)


def _overwrite(arg, values):
    """In-place initialisers write through to the buffer of a contiguous array (zeros_ / randu_ / ... : init_ops.mojo:126-265)."""
    arg.copy_from_numpy(np.asarray(values).reshape(arg.shape()))
    return arg


def fill_(arg, value):
    """init_ops.mojo:185-193."""
    arg._buf.version += 1
    if not arg.is_contiguous() or arg.is_complex_:
        return _overwrite(arg, np.full(arg.shape(), value, np.complex64 if arg.is_complex_ else np.float32))
    if arg.size():
        L.call("endia_hip_fill", arg.data_ptr(), arg.size(), float(value))
    return arg


def zeros_(arg):
    return fill_(arg, 0.0)


def ones_(arg):
    return fill_(arg, 1.0)


def randu_(arg, min=0.0, max=1.0):
    """init_ops.mojo:227-236."""
    return _overwrite(arg, _rng.uniform(min, max, tuple(arg.shape())).astype(np.float32))


def randn_(arg, mean=0.0, std=1.0):
    """init_ops.mojo:255-264."""
    return _overwrite(arg, (_rng.standard_normal(tuple(arg.shape())) * std + mean).astype(np.float32))


def zeros_like(arg):
    return zeros(arg.shape(), arg._requires_grad)


def ones_like(arg):
    return ones(arg.shape(), arg._requires_grad)


def fill_like(arg, value):
    return full(arg.shape(), value, arg._requires_grad)


def eye_like(arg):
    """init_ops.mojo:162-182: ones where the last two indices agree."""
    shape = arg.shape()
    block = np.eye(shape[-2], shape[-1], dtype=np.float32)
    return array(np.broadcast_to(block, shape).copy(), arg._requires_grad)


def randu_like(arg, min=0.0, max=1.0):
    return randu(arg.shape(), min, max, arg._requires_grad)


def randn_like(arg, mean=0.0, std=1.0):
    return randn(arg.shape(), mean, std, arg._requires_grad)


# the initialisation schemes of init_ops.mojo:285-416: a normal or uniform draw whose scale follows the fan sizes
def rand_he_normal_(arg, fan_in=1.0):
    return randn_(arg, 0.0, float(np.sqrt(2.0 / fan_in)))


def rand_he_normal_like(arg, fan_in=1.0):
    return rand_he_normal(arg.shape(), fan_in, arg._requires_grad)


def rand_he_uniform(shape, fan_in=1.0, requires_grad=False):
    limit = float(np.sqrt(6.0 / fan_in))
    return randu(shape, -limit, limit, requires_grad)


def rand_he_uniform_(arg, fan_in=1.0):
    limit = float(np.sqrt(6.0 / fan_in))
    return randu_(arg, -limit, limit)


def rand_he_uniform_like(arg, fan_in=1.0):
    return rand_he_uniform(arg.shape(), fan_in, arg._requires_grad)


def rand_xavier_normal(shape, fan_in=1.0, fan_out=1.0, requires_grad=False):
    return randn(shape, 0.0, float(np.sqrt(2.0 / (fan_in + fan_out))), requires_grad)


def rand_xavier_normal_(arg, fan_in=1.0, fan_out=1.0):
    return randn_(arg, 0.0, float(np.sqrt(2.0 / (fan_in + fan_out))))


def rand_xavier_normal_like(arg, fan_in=1.0, fan_out=1.0):
    return rand_xavier_normal(arg.shape(), fan_in, fan_out, arg._requires_grad)


def rand_xavier_uniform(shape, fan_in=1.0, fan_out=1.0, requires_grad=False):
    limit = float(np.sqrt(6.0 / (fan_in + fan_out)))
    return randu(shape, -limit, limit, requires_grad)


def rand_xavier_uniform_(arg, fan_in=1.0, fan_out=1.0):
    limit = float(np.sqrt(6.0 / (fan_in + fan_out)))
    return randu_(arg, -limit, limit)


def rand_xavier_uniform_like(arg, fan_in=1.0, fan_out=1.0):
    return rand_xavier_uniform(arg.shape(), fan_in, fan_out, arg._requires_grad)


def rand_lecun_normal(shape, fan_in=1.0, requires_grad=False):
    return randn(shape, 0.0, float(np.sqrt(1.0 / fan_in)), requires_grad)


def rand_lecun_normal_(arg, fan_in=1.0):
    return randn_(arg, 0.0, float(np.sqrt(1.0 / fan_in)))


def rand_lecun_normal_like(arg, fan_in=1.0):
    return rand_lecun_normal(arg.shape(), fan_in, arg._requires_grad)


def rand_lecun_uniform(shape, fan_in=1.0, requires_grad=False):
    limit = float(np.sqrt(3.0 / fan_in))
    return randu(shape, -limit, limit, requires_grad)


def rand_lecun_uniform_(arg, fan_in=1.0):
    limit = float(np.sqrt(3.0 / fan_in))
    return randu_(arg, -limit, limit)


def rand_lecun_uniform_like(arg, fan_in=1.0):
    return rand_lecun_uniform(arg.shape(), fan_in, arg._requires_grad)


def complex(real, imag=None):
    """complex(real, imag): init_ops.mojo:419-433."""
    r = contiguous(real)
    i = contiguous(imag) if imag is not None else None
    out = Array.empty(r._shape, is_complex=True)
    L.call("endia_hip_complex_pack", r.size(), r.data_ptr(), i.data_ptr() if i is not None else None, out.data_ptr())

    def vjp(primals, grad, out_):
        return [real_part(grad) if primals[0]._requires_grad else None] + (
            [imag_part(grad) if primals[1]._requires_grad else None] if len(primals) > 1 else [])

    return _register(out, [real] + ([imag] if imag is not None else []), "complex", vjp)


# --------------------------------------------------------------------------------------------------
# view ops (endia/functional/view_ops)
# --------------------------------------------------------------------------------------------------
def _norm_axes(axes, ndim):
    return [a + ndim if a < 0 else a for a in axes]


def expand(x, shape, ignore_axes=()):
    """Broadcast view with stride 0 on expanded axes (expand_op.mojo:36-199). Its VJP is the sum over
    those axes, KEPT as size 1 (expand_op.mojo:121-126): this is the bias gradient."""
    shape = list(shape)
    ign = _norm_axes(list(ignore_axes), x.ndim())
    if x.ndim() == len(shape) and all(i in ign or x._shape[i] == shape[i] for i in range(x.ndim())):
        return x
    diff = len(shape) - x.ndim()
    if diff < 0:
        raise ValueError("expand: source has more dimensions than the target")
    new_shape = list(shape[:diff])
    new_strides = [0] * diff
    for i in range(x.ndim()):
        if i in ign:
            new_shape.append(x._shape[i])
            new_strides.append(x._strides[i])
        elif x._shape[i] == shape[i + diff]:
            new_shape.append(x._shape[i])
            new_strides.append(x._strides[i])
        elif x._shape[i] == 1:
            new_shape.append(shape[i + diff])
            new_strides.append(0)
        else:
            raise ValueError("expand: cannot broadcast %s to %s" % (x.shape(), shape))

    def vjp(primals, grad, out):
        lead = grad.ndim() - out.ndim()
        axes = [i + lead for i in range(out.ndim()) if out._strides[i] == 0 and out._shape[i] != 1]
        return [reduce_add(grad, axes) if axes else grad]

    return _view(x, new_shape, new_strides, x._offset, [x], "brdcst", vjp)


def permute(x, axes):
    """permute_op.mojo:35-143. Given fewer axes than dimensions, they permute the trailing ones."""
    nd = x.ndim()
    axes = list(axes)
    if len(axes) < nd:
        k = len(axes)
        axes = list(range(nd - k)) + [nd + a if a < 0 else nd - k + a for a in axes]
    else:
        axes = _norm_axes(axes, nd)
    if sorted(axes) != list(range(nd)):
        raise ValueError("permute: bad axes %s" % axes)
    shape = [x._shape[a] for a in axes]
    strides = [x._strides[a] for a in axes]

    def vjp(primals, grad, out):
        lead = grad.ndim() - nd
        inv = [0] * nd
        for i, a in enumerate(axes):
            inv[a] = i
        return [permute(grad, list(range(lead)) + [lead + i for i in inv])]

    return _view(x, shape, strides, x._offset, [x], "permute", vjp)


def squeeze(x):
    """Drop every size-1 axis, keeping one if all are (squeeze_op.mojo:31-60)."""
    ax = [i for i, s in enumerate(x._shape) if s == 1]
    if len(ax) == x.ndim() and ax:
        ax.pop()
    if not ax:
        return x
    shape = [s for i, s in enumerate(x._shape) if i not in ax]
    strides = [s for i, s in enumerate(x._strides) if i not in ax]
    in_shape = list(x._shape)

    def vjp(primals, grad, out):
        lead = grad.ndim() - out.ndim()
        return [reshape(grad, list(grad._shape[:lead]) + in_shape)]

    return _view(x, shape, strides, x._offset, [x], "squeeze", vjp)


def unsqueeze(x, axes):
    axes = sorted(_norm_axes(list(axes), x.ndim() + len(axes)))
    shape, strides = list(x._shape), list(x._strides)
    for a in axes:
        shape.insert(a, 1)
        strides.insert(a, 0)
    in_shape = list(x._shape)

    def vjp(primals, grad, out):
        lead = grad.ndim() - out.ndim()
        return [reshape(grad, list(grad._shape[:lead]) + in_shape)]

    return _view(x, shape, strides, x._offset, [x], "unsqueeze", vjp)


def reshape(x, shape):
    """view_op.mojo:33-141: a view when x is contiguous, otherwise a copy first."""
    shape = list(shape)
    if -1 in shape:
        known = _prod([s for s in shape if s != -1])
        shape[shape.index(-1)] = x.size() // max(known, 1)
    if _prod(shape) != x.size():
        raise ValueError("reshape: %s -> %s changes the element count" % (x.shape(), shape))
    src = x if x.is_contiguous() else _contiguous_copy(x)
    in_shape = list(x._shape)

    def vjp(primals, grad, out):
        lead = grad.ndim() - out.ndim()
        return [reshape(grad, list(grad._shape[:lead]) + in_shape)]

    return _view(src, shape, contiguous_strides(shape), src._offset, [x], "reshape", vjp)


def _dot(a, b):  # the module's own `sum` is the array op
    t = 0
    for u, v in zip(a, b):
        t += u * v
    return t


def _norm_slices(slices, shape):
    """Python-style (start, stop, step) per axis, step > 0, clamped to the axis; missing axes are whole."""
    out = []
    for i, n in enumerate(shape):
        sl = slices[i] if i < len(slices) else slice(None)
        if isinstance(sl, int):
            sl = slice(sl, sl + 1 if sl != -1 else None)
        start, stop, step = sl.indices(n)
        if step <= 0:
            raise ValueError("array_slice: steps must be positive")
        out.append((start, max(stop, start), step))
    return out


def array_slice(x, slices):
    """A view of a block of x: start / stop / step per leading axis (array_slice_op.mojo:41-83: stride times
    step, offset plus start times stride). Its VJP pads the gradient back with zeros (:104-120)."""
    if len(slices) > x.ndim():
        raise ValueError("array_slice: %d slices for %d dimensions" % (len(slices), x.ndim()))
    norm = _norm_slices(list(slices), x._shape)
    shape = [(stop - start + step - 1) // step for start, stop, step in norm]
    strides = [st * step for st, (_, _, step) in zip(x._strides, norm)]
    offset = x._offset + _dot(x._strides, [start for start, _, _ in norm])
    in_shape = list(x._shape)

    def vjp(primals, grad, out):
        lead = grad.ndim() - out.ndim()
        whole = [slice(None)] * lead
        return [pad(grad, list(grad._shape[:lead]) + in_shape, whole + [slice(a, b, c) for a, b, c in norm])]

    return _view(x, shape, strides, offset, [x], "slice", vjp)


def pad(x, target_shape, slices_in_target):
    """x copied into the block `slices_in_target` of a zero array of `target_shape` (pad_op.mojo:35-142); the
    VJP is the same block of the gradient (:83-101)."""
    target_shape = list(target_shape)
    if len(target_shape) != x.ndim():
        raise ValueError("pad: target has %d dimensions, the array %d" % (len(target_shape), x.ndim()))
    norm = _norm_slices(list(slices_in_target), target_shape)
    block = [(stop - start + step - 1) // step for start, stop, step in norm]
    if block != list(x._shape):
        raise ValueError("Error in pad: target_shape and sliced_curr shape do not match")  # pad_op.mojo:137-140
    out = Array(target_shape, is_complex=x.is_complex_)
    src = contiguous(x)
    if src.size():
        L.call("endia_hip_strided_scatter", x.ndim(), L.i64_array(x._shape),
               L.i64_array([st * step for st, (_, _, step) in zip(out._strides, norm)]),
               _dot(out._strides, [start for start, _, _ in norm]), src.data_ptr(), out._buf.ptr, 0,
               1 if x.is_complex_ else 0)

    def vjp(primals, grad, o):
        lead = grad.ndim() - o.ndim()
        return [array_slice(grad, [slice(None)] * lead + [slice(a, b, c) for a, b, c in norm])]

    return _register(out, [x], "pad", vjp)


def _check_window(name, numel, shape, stride, storage_offset):
    if len(shape) != len(stride) or any(s < 0 for s in shape) or any(s < 0 for s in stride) or storage_offset < 0:
        raise ValueError("%s: shape and stride must have equal length and no negative entries" % name)
    last = storage_offset + _dot([n - 1 for n in shape], stride) if _prod(shape) else 0
    if last >= numel and _prod(shape):
        raise ValueError("%s: the view reaches element %d of a buffer of %d" % (name, last, numel))


def as_strided(x, shape, stride, storage_offset=0):
    """A view of x's storage with the given shape, strides and offset, as torch.as_strided (as_strided_op.mojo:
    33-160; the view is taken over the base buffer, :47-60). Windows may overlap. VJP: as_strided_inv (:67-89)."""
    shape, stride = [int(s) for s in shape], [int(s) for s in stride]
    base = contiguous(x)
    _check_window("as_strided", base.size(), shape, stride, storage_offset)
    in_shape = list(x._shape)

    def vjp(primals, grad, out):
        if grad.ndim() != len(shape):
            raise ValueError("as_strided: batched cotangents are not supported")
        return [as_strided_inv(grad, in_shape, shape, stride, storage_offset)]

    return _view(base, shape, stride, base._offset + storage_offset, [x], "as_strided", vjp)


def as_strided_inv(g, target_shape, shape, stride, storage_offset=0):
    """Adjoint of as_strided: g added through an as_strided view into a zero array of target_shape
    (as_strided_op.mojo:169-190). Where windows overlap the contributions add up. VJP: as_strided (:197-215)."""
    shape, stride = [int(s) for s in shape], [int(s) for s in stride]
    if list(g._shape) != shape:
        raise ValueError("as_strided_inv: the array has shape %s, the view %s" % (g.shape(), shape))
    out = Array(list(target_shape), is_complex=g.is_complex_)
    _check_window("as_strided_inv", out.size(), shape, stride, storage_offset)
    src = contiguous(g)
    if src.size():
        L.call("endia_hip_strided_scatter", len(shape), L.i64_array(shape), L.i64_array(stride), storage_offset,
               src.data_ptr(), out._buf.ptr, 1, 1 if g.is_complex_ else 0)

    def vjp(primals, grad, o):
        return [as_strided(grad, shape, stride, storage_offset)]

    return _register(out, [g], "as_strided_inv", vjp)


def concat(arrays, axis=0):
    """The arrays joined along `axis` (index_ops/concat_op.mojo:27-110; its forward allocates the result but
    copies nothing and its VJP returns no gradients, :64-95, so the arithmetic here is numpy.concatenate's:
    each argument is written into its block, and each gradient is that block of the cotangent)."""
    arrays = list(arrays)
    if not arrays:
        raise ValueError("concat: no arrays")
    nd = arrays[0].ndim()
    axis = axis + nd if axis < 0 else axis
    if not 0 <= axis < nd:
        raise ValueError("Error: Axis out of bounds")
    for a in arrays[1:]:
        if a.ndim() != nd or any(a._shape[j] != arrays[0]._shape[j] for j in range(nd) if j != axis) \
                or a.is_complex_ != arrays[0].is_complex_:
            raise ValueError("Error: Incompatible shapes for concatenation")
    shape = list(arrays[0]._shape)
    shape[axis] = _dot([a._shape[axis] for a in arrays], [1] * len(arrays))
    out = Array(shape, is_complex=arrays[0].is_complex_, _zero=False)
    blocks, at = [], 0
    for a in arrays:
        blocks.append((at, at + a._shape[axis]))
        src = contiguous(a)
        if src.size():
            L.call("endia_hip_strided_scatter", nd, L.i64_array(a._shape), L.i64_array(out._strides),
                   at * out._strides[axis], src.data_ptr(), out._buf.ptr, 0, 1 if a.is_complex_ else 0)
        at += a._shape[axis]

    def vjp(primals, grad, o):
        lead = grad.ndim() - o.ndim()
        return [array_slice(grad, [slice(None)] * (lead + axis) + [slice(b0, b1)]) for b0, b1 in blocks]

    return _register(out, arrays, "concat", vjp)


def real_part(x):
    """real(): stride-2 fp32 view of a complex array (real_op.mojo:43-52); VJP complex(g, 0) (:74-77)."""
    if not x.is_complex_:
        return x

    def vjp(primals, grad, out):
        return [complex(grad)]

    return _view(x, x._shape, [2 * s for s in x._strides], 2 * x._offset, [x], "real", vjp, is_complex=False)


def imag_part(x):
    if not x.is_complex_:
        return zeros(x._shape)
    return _view(x, x._shape, [2 * s for s in x._strides], 2 * x._offset + 1, [x], "imag", None, is_complex=False)


real = real_part
imag = imag_part


# --------------------------------------------------------------------------------------------------
# binary elementwise ops (endia/functional/binary_ops)
# --------------------------------------------------------------------------------------------------
def _broadcast_shape(a, b):
    sa, sb = list(a._shape), list(b._shape)
    n = max(len(sa), len(sb))
    sa = [1] * (n - len(sa)) + sa
    sb = [1] * (n - len(sb)) + sb
    out = []
    for x, y in zip(sa, sb):
        if x == y or y == 1:
            out.append(x)
        elif x == 1:
            out.append(y)
        else:
            raise ValueError("cannot broadcast %s with %s" % (a.shape(), b.shape()))
    return out


def _binary(op, name, a, b, vjp):
    if _fusion is not None and _fusion.tracing(a, b):
        return _fusion.sym_binary(op, name, a, b, vjp)
    if a.is_complex_ != b.is_complex_:
        a = a if a.is_complex_ else complex(a)
        b = b if b.is_complex_ else complex(b)
    shape = _broadcast_shape(a, b)
    # binary_op_array expands both operands to the broadcast shape (binary_ops/_utils.mojo:83-86); the
    # expanded views take part in autograd, so broadcast axes are summed on the way back
    ea, eb = expand(a, shape), expand(b, shape)
    out = Array.empty(shape, is_complex=a.is_complex_)
    if len(shape) > 8:
        raise ValueError("more than 8 dimensions")
    if out.size():
        L.call("endia_hip_binary", op, len(shape), L.i64_array(shape), L.i64_array(ea._strides), L.i64_array(eb._strides),
               ea.data_ptr(), eb.data_ptr(), out.data_ptr(), 1 if out.is_complex_ else 0)
    return _register(out, [ea, eb], name, vjp)


def add(a, b):
    def vjp(primals, grad, out):  # add_op.mojo:107-110
        return [grad if primals[0]._requires_grad else None, grad if primals[1]._requires_grad else None]
    return _binary(L.BIN_ADD, "add", a, b, vjp)


def sub(a, b):
    def vjp(primals, grad, out):  # sub_op.mojo:109-112
        return [grad if primals[0]._requires_grad else None, neg(grad) if primals[1]._requires_grad else None]
    return _binary(L.BIN_SUB, "sub", a, b, vjp)


def mul(a, b):
    def vjp(primals, grad, out):  # mul_op.mojo:125-128 (no conjugation for complex operands)
        if primals[0] is primals[1] and primals[0]._requires_grad and not primals[0].is_complex_ and grad._shape == primals[0]._shape \
                and (_fusion is None or not _fusion.tracing(grad, primals[0])):
            # x * x: both contributions, x g + x g, as one launch and one node instead of two products and their sum
            return [_fused_rule("twice_mul", lambda x_, g_: mul(add(x_, x_), g_))(primals[0], grad), None]
        return [mul(primals[1], grad) if primals[0]._requires_grad else None,
                mul(primals[0], grad) if primals[1]._requires_grad else None]
    return _binary(L.BIN_MUL, "mul", a, b, vjp)


def div(a, b):
    def vjp(primals, grad, out):  # div_op.mojo:108-114
        lhs = div(grad, primals[1]) if primals[0]._requires_grad else None
        rhs = div(mul(neg(grad), primals[0]), mul(primals[1], primals[1])) if primals[1]._requires_grad else None
        return [lhs, rhs]
    return _binary(L.BIN_DIV, "div", a, b, vjp)


def pow(a, b):
    """Elementwise a ** b as exp(log|a| * b) * cos(arg(a) * b) (pow_op.mojo:139-146); broadcasting."""
    def vjp(primals, grad, out):  # pow_op.mojo:109-115
        lhs = mul(mul(grad, primals[1]), div(out, primals[0])) if primals[0]._requires_grad else None
        rhs = mul(mul(grad, out), log(primals[0])) if primals[1]._requires_grad else None
        return [lhs, rhs]
    return _binary(L.BIN_POW, "pow", a, b, vjp)


pow_to = pow


def _comparison(op, name, a, b):
    if _fusion is not None and _fusion.tracing(a, b):  # inside a fused expression; a plain number is an immediate
        return _fusion.sym_binary(op, name, a, b, None)
    if a.is_complex_ or b.is_complex_:
        raise ValueError("%s is implemented for real arrays only" % name)
    return _binary(op, name, detach(a), detach(b), None)


def greater(a, b):
    """1.0 where a > b, else 0.0; not differentiable (greater_op.mojo:46-60)."""
    return _comparison(L.BIN_GREATER, "greater", a, b)


def greater_equal(a, b):
    """1.0 where a >= b (comparison_ops/greater_equal_op.mojo)."""
    return _comparison(L.BIN_GREATER_EQUAL, "greater_equal", a, b)


def less(a, b):
    """1.0 where a < b (comparison_ops/less_op.mojo)."""
    return _comparison(L.BIN_LESS, "less", a, b)


def less_equal(a, b):
    """1.0 where a <= b (comparison_ops/less_equal_op.mojo)."""
    return _comparison(L.BIN_LESS_EQUAL, "less_equal", a, b)


def equal(a, b):
    """1.0 where a == b (comparison_ops/equal_op.mojo)."""
    return _comparison(L.BIN_EQUAL, "equal", a, b)


def not_equal(a, b):
    """1.0 where a != b (comparison_ops/not_equal_op.mojo)."""
    return _comparison(L.BIN_NOT_EQUAL, "not_equal", a, b)


def pow_int(x, p):
    """x ** p for a small non-negative integer p, as repeated products (x ** 2 is `square`)."""
    if int(p) != p or p < 0:
        raise ValueError("only non-negative integer powers are implemented")
    p = int(p)
    if p == 0:
        return ones(x._shape)
    if p == 2:
        return square(x)
    out = x
    for _ in range(p - 1):
        out = mul(out, x)
    return out


# --------------------------------------------------------------------------------------------------
# unary elementwise ops (endia/functional/unary_ops)
# --------------------------------------------------------------------------------------------------
def _unary(op, name, x, vjp):
    if _fusion is not None and _fusion.tracing(x):
        return _fusion.sym_unary(op, name, x, vjp)
    src = contiguous(x)
    out = Array.empty(x._shape, is_complex=x.is_complex_)
    if out.size():
        L.call("endia_hip_unary_fwd", op, src.size(), src.data_ptr(), out.data_ptr(), 1 if x.is_complex_ else 0)

    def first_order_vjp(primals, grad, out_):
        # The rule handed in is the reference's, written in differentiable ops (two to four launches); it is what a
        # create_graph pass records. An ordinary pass computes the same g * op'(x) with the one kernel made for it.
        from .autograd.functional import building_graph
        p = primals[0]
        if building_graph() and not (p.is_complex_ or grad.is_complex_ or op in _NO_VJP_KERNEL or grad._shape != p._shape or not p.size()):
            try:  # the same rule, recorded as one fused node
                return [_fused_rule("vjp_" + name, lambda x, g, o: vjp([x], g, o)[0])(p, grad, out_)]
            except _fusion.FusionError:
                return vjp(primals, grad, out_)
        if building_graph() or p.is_complex_ or grad.is_complex_ or op in _NO_VJP_KERNEL or grad._shape != p._shape or not p.size():
            return vjp(primals, grad, out_)
        g, xs_ = contiguous(grad), contiguous(p)
        dx = Array.empty(p._shape)
        L.call("endia_hip_unary_vjp", op, p.size(), xs_.data_ptr(), g.data_ptr(), dx.data_ptr(), 0)
        return [dx]

    return _register(out, [x], name, first_order_vjp if vjp is not None else None)


_NO_VJP_KERNEL = (L.OP_SIGN, L.OP_IDENTITY, L.OP_ABS)


def relu(x):
    if x.is_complex_:
        raise ValueError("relu is not defined for complex arrays")  # relu_op.mojo:51-52

    def vjp(primals, grad, out):  # greater(x, zeros) * g : relu_op.mojo:95
        return [mul(greater(primals[0], zeros([primals[0]._shape[-1]])), grad)]
    return _unary(L.OP_RELU, "relu", x, vjp)


def tanh(x):
    def vjp(primals, grad, out):  # (1 - square(tanh(x))) * g, recomputed from the input: tanh_op.mojo:92
        return [mul(1 - square(tanh(primals[0])), grad)]
    return _unary(L.OP_TANH, "tanh", x, vjp)


def sin(x):
    def vjp(primals, grad, out):  # sin_op.mojo:92
        return [mul(cos(primals[0]), grad)]
    return _unary(L.OP_SIN, "sin", x, vjp)


def cos(x):
    def vjp(primals, grad, out):  # cos_op.mojo:93
        return [mul(neg(sin(primals[0])), grad)]
    return _unary(L.OP_COS, "cos", x, vjp)


def neg(x):
    def vjp(primals, grad, out):  # neg_op.mojo:91
        return [neg(grad)]
    return _unary(L.OP_NEG, "neg", x, vjp)


def square(x):
    def vjp(primals, grad, out):  # 2 * x * g : square_op.mojo:96
        return [mul(2 * primals[0], grad)]
    return _unary(L.OP_SQUARE, "square", x, vjp)


def sqrt(x):
    def vjp(primals, grad, out):  # g / (2 * sqrt(x)) : sqrt_op.mojo:91
        return [div(grad, 2 * sqrt(primals[0]))]
    return _unary(L.OP_SQRT, "sqrt", x, vjp)


def sign(x):
    """z / |z| (sign_op.mojo:78-81); used by the VJP of abs. Its own VJP hands the gradient on (sign_op.mojo:58)."""
    def vjp(primals, grad, out):
        return [grad]
    return _unary(L.OP_SIGN, "sign", x, vjp)


def exp(x):
    def vjp(primals, grad, out):  # exp_op.mojo:92
        return [mul(exp(primals[0]), grad)]
    return _unary(L.OP_EXP, "exp", x, vjp)


def log(x):
    """log of the modulus for real x (log_op.mojo:111-113)."""
    def vjp(primals, grad, out):  # log_op.mojo:91
        return [div(grad, primals[0])]
    return _unary(L.OP_LOG, "log", x, vjp)


def _real_only(x, name):
    if x.is_complex_:
        raise ValueError("%s is implemented for real arrays only" % name)


def sigmoid(x):
    _real_only(x, "sigmoid")

    def vjp(primals, grad, out):  # out * (1 - out) * grad : sigmoid_op.mojo:98
        return [mul(mul(out, 1 - out), grad)]
    return _unary(L.OP_SIGMOID, "sigmoid", x, vjp)


def sinh(x):
    def vjp(primals, grad, out):  # sinh_op.mojo:88
        return [mul(cosh(primals[0]), grad)]
    return _unary(L.OP_SINH, "sinh", x, vjp)


def cosh(x):
    def vjp(primals, grad, out):  # cosh_op.mojo:89
        return [mul(sinh(primals[0]), grad)]
    return _unary(L.OP_COSH, "cosh", x, vjp)


def tan(x):
    _real_only(x, "tan")

    def vjp(primals, grad, out):  # grad * (1 + square(out)) : tan_op.mojo:81
        return [mul(grad, 1 + square(out))]
    return _unary(L.OP_TAN, "tan", x, vjp)


def asin(x):
    _real_only(x, "asin")

    def vjp(primals, grad, out):  # grad / sqrt(1 - x ** 2) : asin_op.mojo:83
        return [div(grad, sqrt(1 - primals[0] ** 2))]
    return _unary(L.OP_ASIN, "asin", x, vjp)


def acos(x):
    _real_only(x, "acos")

    def vjp(primals, grad, out):  # -1 / sqrt(1 - x ** 2) * grad : acos_op.mojo:91
        return [mul(-1 / sqrt(1 - primals[0] ** 2), grad)]
    return _unary(L.OP_ACOS, "acos", x, vjp)


def atan(x):
    _real_only(x, "atan")

    def vjp(primals, grad, out):  # grad / (1 + square(x)) : atan_op.mojo:85
        return [div(grad, 1 + square(primals[0]))]
    return _unary(L.OP_ATAN, "atan", x, vjp)


def reciprocal(x):
    def vjp(primals, grad, out):  # -grad / square(x) : reciprocal_op.mojo:95
        return [div(neg(grad), square(primals[0]))]
    return _unary(L.OP_RECIPROCAL, "reciprocal", x, vjp)


def _abs_raw(x):
    src = contiguous(x)
    out = Array.empty(x._shape)
    if out.size():
        L.call("endia_hip_unary_fwd", L.OP_ABS, src.size(), src.data_ptr(), out.data_ptr(), 1 if x.is_complex_ else 0)
    return out


def abs(x):
    """to_abs: |x| as a real array (abs_op.mojo:114-115,157); VJP sign(x) * g (abs_op.mojo:93), where for a
    complex x the real cotangent first becomes complex(g, 0) (real_op.mojo:74-77)."""
    def vjp(primals, grad, out_):
        z = primals[0]
        if z.is_complex_:
            return [mul(sign(z), complex(grad))]
        return [mul(sign(z), grad)]

    if _fusion is not None and _fusion.tracing(x):
        return _fusion.sym_unary(L.OP_ABS, "abs", x, vjp)
    return _register(_abs_raw(x), [x], "abs", vjp)


# --------------------------------------------------------------------------------------------------
# reductions (endia/functional/reduce_ops)
# --------------------------------------------------------------------------------------------------
def _col_sum_parks(src):
    """Whether the column sum of the contiguous real [R, C] array `src` is of the size whose launches are worth sharing (the
    two-stage reduction for a few hundred to a few thousand rows), and products are being put off at all."""
    R_, C_ = src._shape
    return (L.defer_products[0] and not L.capturing and 64 <= R_ <= 2048 and (1 << 20) < R_ * C_ <= (1 << 22) and C_ % 4 == 0
            and src.data_ptr() % 16 == 0)


def _park_col_sum(src, out, scale):
    L.park_col_sum(src._shape[0], src._shape[1], src.data_ptr(), out._buf.address + 4 * out._offset, scale, src._buf, out._buf)


def reduce_add(x, axes, _scale=1.0):
    """Sum over `axes`, keeping them as size 1 (reduce_add_op.mojo:57-61,65-210); VJP = expand (:234)."""
    axes = sorted(set(_norm_axes(list(axes), x.ndim())))
    src = contiguous(x)
    oshape = [1 if i in axes else s for i, s in enumerate(x._shape)]
    out = Array.empty(oshape, is_complex=x.is_complex_)
    mask = 0
    for a in axes:
        mask |= 1 << a
    if x.ndim() > 8:
        raise ValueError("more than 8 dimensions")
    if out.size():
        if axes == [0] and x.ndim() == 2 and not x.is_complex_ and _col_sum_parks(src):
            # a bias gradient of a second-order pass: put off, so that the sums of the pass share one launch
            _park_col_sum(src, out, float(_scale))
        else:
            L.call("endia_hip_reduce_add", x.ndim(), L.i64_array(x._shape), mask, src.data_ptr(), out.data_ptr(),
                   float(_scale), 1 if x.is_complex_ else 0)
    in_shape = list(x._shape)
    scale = float(_scale)

    def vjp(primals, grad, out_):
        lead = grad.ndim() - out_.ndim()
        if scale != 1.0:
            # the seed of a scalar loss times a constant is a constant: kept per value, so that a step spends no launch on it
            grad = _scaled_seed(scale) if _holds_seed(grad) else grad * scale
        return [expand(grad, list(grad._shape[:lead]) + in_shape)]

    return _register(out, [x], "reduce_add", vjp)


_SCALED_SEEDS = {}


def _holds_seed(grad):
    """True for the seed of a scalar output and for its views (the squeeze / reshape on top of a reduction hands
    the seed down as a view of the same buffer)."""
    if grad._is_seed:
        return True
    from .autograd.functional import _SEED
    return bool(_SEED) and grad.size() == 1 and grad._buf is _SEED[0]._buf and grad._offset == _SEED[0]._offset


def _scaled_seed(value):
    """full([1], value), made once per value and never written: what ones(1) * value is for every backward pass."""
    arr = _SCALED_SEEDS.get(value)
    if arr is None:
        if len(_SCALED_SEEDS) > 64:
            _SCALED_SEEDS.clear()
        arr = _SCALED_SEEDS[value] = full([1], value)
    return arr


def sum(x):
    """Sum over all axes, shape [1] (sum_op.mojo:35-62)."""
    return squeeze(reduce_add(x, list(range(x.ndim()))))


def mean(x, axes=None, keepdims=False):
    """mean_op.mojo:35-65: reduce_add divided by the number of reduced elements."""
    axes = list(range(x.ndim())) if axes is None else axes
    kept = 1
    for i, n in enumerate(x._shape):
        if i not in _norm_axes(list(axes), x.ndim()):
            kept *= n
    divisor = float(x.size() // max(kept, 1))
    if x.is_complex_ or divisor == 0.0:
        out = reduce_add(x, axes) / divisor
    else:
        # the division rides in the reduction's last stage as a multiplication by 1 / count (one rounding away from
        # the reference's sum / count), and in the VJP as a constant factor
        out = reduce_add(x, axes, _scale=1.0 / divisor)
    return out if keepdims else squeeze(out)


def _reduce_other(x, axis, keepdims, op, name, cite):
    """Shared body of reduce_max / reduce_min / reduce_mul / reduce_argmax / reduce_argmin: the reduced axes stay as
    size 1 unless keepdims is False, in which case every size-1 axis is squeezed away, as the reference does."""
    if x.is_complex_:
        raise ValueError("Warning in %s:  The %s operation does not support complex numbers." % (name, name))
    axes = sorted(set(_norm_axes([axis] if isinstance(axis, int) else list(axis), x.ndim())))
    if x.ndim() > 8:
        raise ValueError("more than 8 dimensions")
    if op in (L.REDUCE_ARGMAX, L.REDUCE_ARGMIN) and len(axes) != 1:
        raise ValueError("%s: exactly one axis (the reference's result for several axes is not a position)" % name)
    src = contiguous(x)
    out = Array.empty([1 if i in axes else s for i, s in enumerate(x._shape)])
    mask = 0
    for a in axes:
        mask |= 1 << a
    if out.size():
        L.call("endia_hip_reduce", op, x.ndim(), L.i64_array(x._shape), mask, src.data_ptr(), out.data_ptr())

    def vjp(primals, grad, out_):
        raise NotImplementedError("%s has no backward rule in the reference (%s); none is provided here" % (name, cite))

    out = _register(out, [x], name, vjp)
    return out if keepdims else squeeze(out)


def reduce_max(x, axis, keepdims=False):
    """Maximum over `axis` (an int or a list), reduce_max_op.mojo:66-190, 228-257."""
    return _reduce_other(x, axis, keepdims, L.REDUCE_MAX, "reduce_max", "reduce_max_op.mojo:196-198 is the default rule")


def reduce_min(x, axis, keepdims=False):
    """Minimum over `axis`, reduce_min_op.mojo:66-190, 228-257."""
    return _reduce_other(x, axis, keepdims, L.REDUCE_MIN, "reduce_min", "reduce_min_op.mojo:196-198 is the default rule")


def reduce_argmax(x, axis, keepdims=False):
    """Position of the first maximum along one axis, as a float array (reduce_argmax_op.mojo:66-163, 218-247)."""
    return _reduce_other(x, axis, keepdims, L.REDUCE_ARGMAX, "reduce_argmax", "reduce_argmax_op.mojo:169-171 is the default rule")


def reduce_argmin(x, axis, keepdims=False):
    """Position of the first minimum along one axis, as a float array (reduce_argmin_op.mojo:66-163, 218-247)."""
    return _reduce_other(x, axis, keepdims, L.REDUCE_ARGMIN, "reduce_argmin", "reduce_argmin_op.mojo:169-171 is the default rule")


def reduce_mul(x, axis, keepdims=False):
    """Product over `axis` (reduce_mul_op.mojo:65-210, 288-321). The reference's backward rule for it is a placeholder
    that hands the cotangent through unchanged (reduce_mul_op.mojo:238-255, its test file says the rule is still to be written)."""
    return _reduce_other(x, axis, keepdims, L.REDUCE_MUL, "reduce_mul", "reduce_mul_op.mojo:238-255 is a placeholder")


def prod(x):
    """Product of all elements, shape [1] (prod_op.mojo:35-62)."""
    return squeeze(reduce_mul(x, list(range(x.ndim())), keepdims=True))


def variance(x, axes=(0,), unbiased=True, keepdims=False):
    """variance_op.mojo:35-79, op for op: the mean from reduce_add, the squared differences, their sum divided by
    count - 1 (or count). Differentiable through those ops."""
    axes = list(axes)
    res = reduce_add(x, axes)
    count = float(x.size() // max(res.size(), 1))
    divisor = count - 1.0 if unbiased else count
    diff = x - res / count
    out = reduce_add(diff * diff, axes) / divisor
    return out if keepdims else squeeze(out)


def std(x, axes=(0,), unbiased=True, keepdims=False):
    """std_op.mojo:35-65: sqrt(variance)."""
    return sqrt(variance(x, axes, unbiased, keepdims))


# --------------------------------------------------------------------------------------------------
# gradients that absorb an earlier contribution
# --------------------------------------------------------------------------------------------------
# Where a tensor has several consumers the reverse walk adds their contributions with one `add` launch each
# (autograd/functional.mojo:51-57). A rule whose last step is a matrix product can do that addition in the product's
# epilogue instead. The walk offers, per VJP call, the gradient a primal already holds (`_absorb`: id(primal) ->
# (gradient, exclusive)); a rule that uses the offer marks its result `_absorbed`, and the walk stores it as the new
# total without adding. Two forms: the earlier gradient is a row broadcast over the rows (the cotangent of a bias
# gradient on its way to the layer's pre-activation): it becomes the bias operand of the product's epilogue, the
# result is a fresh array; or it is a plain array that nobody else holds (`exclusive`): the product accumulates into
# its buffer. Never offered while a pass records its own graph, where every contribution stays a node.
_absorb = None
_absorbed_launches = [0]  # how many `add` launches the protocol has replaced (read by the tests)


def _absorb_offer(primal):
    return _absorb.get(id(primal)) if _absorb else None


def _as_bias_row(g, rows, cols):
    """g viewed as [rows, cols] is one row of memory repeated: that row as an array of its own, else None."""
    if g.is_complex_ or list(g._shape) != [rows, cols] or g._strides[0] != 0 or (cols > 1 and g._strides[1] != 1):
        return None
    return Array([cols], _buffer=g._buf, _offset=g._offset)


_CUS = []


def _would_park(M, N, K):
    """The size test of _sgemm: fewer 256 x 128 tiles than CUs, yet large enough for a one-tile-per-CU launch."""
    if not _CUS:
        _CUS.append(L.device_info()[1])
    return (L.defer_products[0] and not L.capturing and -(-M // 256) * -(-N // 128) < _CUS[0] and M >= 256 and N >= 128 and K >= 256)


def _sgemm(ta, tb, M, N, K, A_, lda, B_, ldb, out, epi=L.EPI_NONE, bias=None):
    """One real, unbatched product C = op(A) op(B) (+ bias row, or on top of what C holds) into `out`, a contiguous
    array. A product that cannot fill the chip alone (fewer 256 x 128 tiles than CUs) but is large enough to be worth a
    one-tile-per-CU launch is parked (_lib.park_product) so that it can share a launch with the independent products
    that a backward pass issues next to it; anything else is launched here."""
    parkable = _would_park(M, N, K) and lda % 4 == 0 and ldb % 4 == 0 and (epi & 0xff) in (L.EPI_NONE, L.EPI_BIAS)
    a_ptr, b_ptr = A_.data_ptr(), B_.data_ptr()
    bias_ptr = bias.data_ptr() if isinstance(bias, Array) else bias
    if not parkable or (a_ptr | b_ptr) & 15:
        L.call("endia_hip_sgemm", ta, tb, M, N, K, a_ptr, lda, b_ptr, ldb, out.data_ptr(), N, 1, 0, 0, 0, epi, L.OP_IDENTITY,
               bias_ptr, None, None)
        return
    obuf = out._buf
    if epi & L.GEMM_ACCUMULATE:  # what is parked and writes, or reads, the buffer this product adds to goes first
        if obuf.pending:
            L.flush(obuf)
        if L.parked_uses(obuf):
            L.flush()
    buffers = [A_._buf, B_._buf] + ([bias._buf] if isinstance(bias, Array) else [])
    c_ptr = obuf.address + 4 * out._offset
    L.park_product((ta, tb, M, N, K, a_ptr, lda, b_ptr, ldb, c_ptr, N, epi, bias_ptr), buffers, obuf)


# --------------------------------------------------------------------------------------------------
# matmul (endia/functional/binary_ops/matmul_op.mojo)
# --------------------------------------------------------------------------------------------------
def _gemm_operand(x):
    """Describe the last two axes of x for the GEMM: (array, trans, ld, batch_stride).

    A row-major matrix (unit column stride) is passed as is; its transpose view (unit row stride) is
    passed with the transpose flag, so `.T()` never costs a copy (the reference copies:
    matmul_op.mojo:111-136). Leading axes must collapse to one batch stride; otherwise x is copied.
    """
    def describe(a):
        rows, cols = a._shape[-2], a._shape[-1]
        rs, cs = a._strides[-2], a._strides[-1]
        if (cs == 1 or cols == 1) and (rs >= cols or rows == 1):
            trans, ld = 0, (rs if rows > 1 else max(cols, 1))
        elif (rs == 1 or rows == 1) and (cs >= rows or cols == 1):
            trans, ld = 1, (cs if cols > 1 else max(rows, 1))
        else:
            return None
        # collapse the batch axes
        bshape = [s for s in a._shape[:-2]]
        bstr = [s for s in a._strides[:-2]]
        dims = [(s, st) for s, st in zip(bshape, bstr) if s != 1]
        if not dims:
            return a, trans, ld, 0
        if all(st == 0 for _, st in dims):
            return a, trans, ld, 0
        ok = all(dims[i][1] == dims[i + 1][1] * dims[i + 1][0] for i in range(len(dims) - 1))
        if ok:
            return a, trans, ld, dims[-1][1]
        return None

    d = describe(x)
    if d is None:
        d = describe(_contiguous_copy(x))
    return d


def _is_transposed_matrix(x):
    """x is a real 2-D transposed view of a row-major matrix (unit ROW stride), larger than a vector."""
    return (x.ndim() == 2 and not x.is_complex_ and x._shape[0] > 1 and x._shape[1] > 1
            and x._strides[0] == 1 and x._strides[1] >= x._shape[0])


def matmul(a, b, vjp_rule=None, _ca=0, _cb=0, _into=None):
    """Batched matrix product with broadcast batch axes (matmul_op.mojo:36-90,309-346).

    VJP (matmul_op.mojo:278-283): dA = g @ B.T(), dB = A.T() @ g. For complex operands the reference codes exactly
    that, WITHOUT conjugation: vjp_rule="reference", the default. vjp_rule="wirtinger" selects g @ B^H, A^H @ g, the
    conjugate-Wirtinger gradient of a real loss that PyTorch returns; its conjugations are flags of the complex GEMM
    (`_ca`, `_cb`: the product is taken with conj(a), conj(b)), never materialised copies. vjp_rule=None takes the
    process-wide choice of set_complex_vjp_rule(). Real operands are unaffected.
    """
    if vjp_rule is None:
        vjp_rule = _complex_vjp_rule[0]
    if vjp_rule not in ("reference", "wirtinger"):
        raise ValueError("matmul: vjp_rule must be 'reference' or 'wirtinger'")
    _conj_vjp = vjp_rule == "wirtinger"
    if a.ndim() < 2 or b.ndim() < 2:
        raise ValueError("Invalid shapes for matmul, i.e. ndim < 2")
    if a._shape[-1] != b._shape[-2]:
        raise ValueError("Invalid shapes for matmul, i.e. shapes are not compatible for matmul")
    if a.is_complex_ != b.is_complex_:
        a = a if a.is_complex_ else complex(a)
        b = b if b.is_complex_ else complex(b)
    ba, bb = list(a._shape[:-2]), list(b._shape[:-2])
    n = max(len(ba), len(bb))
    ba_p = [1] * (n - len(ba)) + ba
    bb_p = [1] * (n - len(bb)) + bb
    bshape = []
    for x, y in zip(ba_p, bb_p):
        if x == y or y == 1:
            bshape.append(x)
        elif x == 1:
            bshape.append(y)
        else:
            raise ValueError("Error: matmul Incompatible shapes for broadcasting")
    M, K, N = a._shape[-2], a._shape[-1], b._shape[-1]
    out_shape = bshape + [M, N]
    ea = expand(a, bshape + [M, K], [-2, -1])
    eb = expand(b, bshape + [K, N], [-2, -1])
    A_, ta, lda, sa = _gemm_operand(ea)
    B_, tb, ldb, sb = _gemm_operand(eb)
    batch = _prod(bshape)
    # `_into` (an offer of the reverse walk, see _absorb above): (earlier gradient of this product's shape, exclusive)
    epi, bias_row, out = L.EPI_NONE, None, None
    if _into is not None and not a.is_complex_ and len(out_shape) == 2 and M * N * K > 0:
        g0, exclusive = _into
        bias_row = _as_bias_row(g0, M, N)
        if bias_row is not None:
            epi = L.EPI_BIAS
        elif exclusive and list(g0._shape) == out_shape and g0.is_contiguous() and not g0.is_complex_:
            epi, out = L.EPI_NONE | L.GEMM_ACCUMULATE, Array(out_shape, _buffer=g0._buf, _offset=g0._offset)
    if out is None:
        out = Array.empty(out_shape, is_complex=a.is_complex_)
    if epi != L.EPI_NONE:
        out._absorbed = True
        _absorbed_launches[0] += 1
    if out.size():
        if a.is_complex_:
            L.call("endia_hip_cgemm", ta, _ca, tb, _cb, M, N, K, A_.data_ptr(), lda, B_.data_ptr(), ldb, out.data_ptr(), N,
                   batch, sa, sb, M * N, _cgemm_algo[0], 0)
        elif batch == 1 and K > 0:
            _sgemm(ta, tb, M, N, K, A_, lda, B_, ldb, out, epi, bias_row)
        else:
            L.call("endia_hip_sgemm", ta, tb, M, N, K, A_.data_ptr(), lda, B_.data_ptr(), ldb, out.data_ptr(), N, batch,
                   sa, sb, M * N, epi, L.OP_IDENTITY, None, None, None)

    def vjp(primals, grad, out_):
        p0, p1 = primals
        if _conj_vjp and p0.is_complex_:
            # with A' = conj^ca(A), B' = conj^cb(B): dA = conj^ca(g B'^H), dB = conj^cb(A'^H g)
            lhs = matmul(grad, p1.T(), "wirtinger", _ca, _ca ^ (1 - _cb)) if p0._requires_grad else None
            rhs = matmul(p0.T(), grad, "wirtinger", _cb ^ (1 - _ca), _cb) if p1._requires_grad else None
        else:
            # A gradient is laid out like its primal: for a transposed view (x.T() of a row-major x) the same product is
            # taken as its transpose, B g^T for (g B^T)^T, and handed on as that array's .T(). The view's own VJP then
            # returns a ROW-MAJOR gradient for x, and what meets it there (the sum with another contribution, a fused
            # elementwise rule) takes the flat kernels instead of the transposed ones.
            lhs = rhs = None
            o0 = _absorb_offer(p0) if p0 is not p1 else None
            o1 = _absorb_offer(p1) if p0 is not p1 else None
            if p0._requires_grad:
                if _is_transposed_matrix(p0):
                    lhs = _keep_absorbed(matmul(p1, grad.T(), "reference", _into=_transposed_offer(o0)))
                else:
                    lhs = matmul(grad, p1.T(), "reference", _into=o0)
            if p1._requires_grad:
                if _is_transposed_matrix(p1):
                    rhs = _keep_absorbed(matmul(grad.T(), p0, "reference", _into=_transposed_offer(o1)))
                else:
                    rhs = matmul(p0.T(), grad, "reference", _into=o1)
        return [lhs, rhs]

    return _register(out, [ea, eb], "matmul", vjp)


def _transposed_offer(offer):
    """The walk's offer for a primal that is a transposed view, as seen by the product that computes the gradient's
    transpose: only the in-place form applies (the transpose of a row broadcast is not one)."""
    if offer is None or not offer[1] or offer[0].ndim() != 2:
        return None
    return (offer[0].T(), True)


def _keep_absorbed(prod):
    t = prod.T()
    if prod._absorbed:
        t._absorbed = True
    return t


_cgemm_algo = [L.CGEMM_4M]
_complex_vjp_rule = ["reference"]


def set_complex_vjp_rule(name):
    """The rule matmul's VJP uses for complex operands when a call does not name one: 'reference' (the reference's
    code, no conjugation: matmul_op.mojo:278-283; the default) or 'wirtinger' (g B^H, A^H g)."""
    if name not in ("reference", "wirtinger"):
        raise ValueError("set_complex_vjp_rule: 'reference' or 'wirtinger'")
    _complex_vjp_rule[0] = name


def set_complex_matmul_algorithm(name):
    """'4m' (the reference's four real products, default) or '3m' (three products, larger rounding error)."""
    _cgemm_algo[0] = {"4m": L.CGEMM_4M, "3m": L.CGEMM_3M}[name.lower()]


def conj(x):
    """conj_op.mojo:44,54: (re, -im); VJP conj(g)."""
    if not x.is_complex_:
        return x
    out = complex(real_part(x), neg(contiguous(imag_part(x))))
    out._args, out._vjp = [], None

    def vjp(primals, grad, out_):
        return [conj(grad)]

    return _register(out, [x], "conj", vjp)


# --------------------------------------------------------------------------------------------------
# loss (endia/functional/loss_ops/mse_op.mojo)
# --------------------------------------------------------------------------------------------------
def mse(pred, target):
    """mse = sum((pred - target) * (pred - target)) / pred.size()  (mse_op.mojo:17-20), as ONE kernel
    that also writes the gradient 2 (pred - target) / n which the reference's VJP chain
    (div -> sum -> mul(d, d) -> sub) arrives at. Under create_graph=True the VJP is rebuilt from
    differentiable ops instead, so higher-order derivatives see the same graph as the reference."""
    if pred.is_complex_ or target.is_complex_ or pred._shape != target._shape:
        diff = sub(pred, target)
        return sum(mul(diff, diff)) / float(pred.size())
    lazy = pred._lazy_mlp
    if lazy is not None and not target._requires_grad and _starts_on_16(target) and L.withdraw_launch(lazy[0]):
        # pred is the output of a whole-model forward that has not been launched yet: one launch for the forward pass, the
        # loss, its gradient and the cotangents of all layers (mlp_mse_loss), writing the same activation arrays
        pred._lazy_mlp = None
        return _mlp_mse_fused(lazy, pred, target)
    p, t = contiguous(pred), contiguous(target)
    loss = Array.empty([1])
    need_grad = pred._requires_grad
    dpred = Array.empty(pred._shape) if need_grad else None
    L.call("endia_hip_mse_fwd_bwd", p.size(), p.data_ptr(), t.data_ptr(), loss.data_ptr(),
           dpred.data_ptr() if need_grad else None)
    n = float(pred.size())

    def vjp(primals, grad, out_):
        from .autograd.functional import building_graph
        pr, tg = primals
        if building_graph() or tg._requires_grad or not grad._is_seed:
            d = sub(pr, tg)
            g = (d * 2.0) * (grad / n)
            return [g if pr._requires_grad else None, neg(g) if tg._requires_grad else None]
        return [dpred, None]

    return _register(loss, [pred, target], "mse", vjp)


# --------------------------------------------------------------------------------------------------
# conv2d (endia/functional/spacial_ops/conv2d_op.mojo)
# --------------------------------------------------------------------------------------------------
def _pair(v):
    return (int(v), int(v)) if np.isscalar(v) else (int(v[0]), int(v[1]))


def conv2d(x, kernel, bias=None, stride=1, padding=0, dilation=1, groups=1, act=None):
    """NCHW cross-correlation (conv2d_op.mojo:88-196; tuple order is (height, width)). The reference has
    no backward rule for it (conv2d_op.mojo:198-200); the VJP here is the adjoint of its forward loop.
    act="relu" (no counterpart in the reference) applies the activation in the kernel's epilogue and its
    derivative on the way into the gradients, instead of as separate passes over the output."""
    if act not in (None, "relu"):
        raise ValueError("conv2d: act must be None or 'relu'")
    if x.ndim() != 4:
        raise ValueError("Input must be 4-dimensional (batch_size, in_channels, height, width) for 2D convolution!")
    if x._shape[1] != kernel._shape[1]:
        raise ValueError("Input channels must match kernel channels for 2D convolution!")
    if x.is_complex_ or kernel.is_complex_:
        raise ValueError("conv2d is not defined for complex arrays")  # conv2d_op.mojo:216-217
    (sh, sw), (ph, pw), (dh, dw) = _pair(stride), _pair(padding), _pair(dilation)
    N, C, H, W = x._shape
    K, _, R, S = kernel._shape
    desc = L.Conv2dDesc(N, C, H, W, K, R, S, sh, sw, ph, pw, dh, dw, groups)
    import ctypes
    P, Q = ctypes.c_int64(), ctypes.c_int64()
    L.call("endia_hip_conv2d_out_shape", ctypes.byref(desc), ctypes.byref(P), ctypes.byref(Q))
    xs, ks = contiguous(x), contiguous(kernel)
    bsrc = contiguous(bias) if bias is not None else None
    out = Array.empty([N, K, P.value, Q.value])
    L.call("endia_hip_conv2d_fwd", ctypes.byref(desc), xs.data_ptr(), ks.data_ptr(),
           bsrc.data_ptr() if bsrc is not None else None, out.data_ptr(), L.OP_RELU if act == "relu" else L.OP_IDENTITY)

    def vjp(primals, grad, out_):
        from .autograd.functional import building_graph
        if building_graph():
            raise NotImplementedError("conv2d has no second-order rule")
        if grad.ndim() != out_.ndim():
            raise NotImplementedError("conv2d has no rule for a cotangent with leading Jacobian axes (non-scalar output)")
        if act == "relu":
            # one call for all three; the ReLU's derivative is applied to the cotangent as the kernels load it. A
            # cotangent that is one value spread over the whole array (the gradient of a mean or a sum: a stride-0
            # view) is handed over as that one value.
            scalar = bool(grad.size()) and all(st == 0 or n == 1 for st, n in zip(grad._strides, grad._shape))
            g = Array([1], _buffer=grad._buf, _strides=[1], _offset=grad._offset) if scalar else contiguous(grad)
            wanted = [p_._requires_grad for p_ in primals]
            outs = [Array.empty(p_._shape) if w_ else None for p_, w_ in zip(primals, wanted)]
            L.call("endia_hip_conv2d_bwd_relu", ctypes.byref(desc), xs.data_ptr(), ks.data_ptr(), out_.data_ptr(), g.data_ptr(),
                   1 if scalar else 0, *[o.data_ptr() if o is not None else None for o in (outs + [None])[:3]])
            return outs
        g = contiguous(grad)
        res = []
        if primals[0]._requires_grad:
            dx = Array.empty(primals[0]._shape)
            L.call("endia_hip_conv2d_bwd_data", ctypes.byref(desc), g.data_ptr(), ks.data_ptr(), dx.data_ptr())
            res.append(dx)
        else:
            res.append(None)
        if primals[1]._requires_grad:
            dw = Array.empty(primals[1]._shape)
            L.call("endia_hip_conv2d_bwd_weight", ctypes.byref(desc), xs.data_ptr(), g.data_ptr(), dw.data_ptr())
            res.append(dw)
        else:
            res.append(None)
        if len(primals) > 2:
            if primals[2]._requires_grad:
                db = Array.empty(primals[2]._shape)
                L.call("endia_hip_conv2d_bwd_bias", ctypes.byref(desc), g.data_ptr(), db.data_ptr())
                res.append(db)
            else:
                res.append(None)
        return res

    args = [x, kernel] + ([bias] if bias is not None else [])
    return _register(out, args, "conv2d", vjp)


def conv1d(x, kernel, bias=None, stride=1, padding=0, dilation=1, groups=1):
    """[N, C, L] cross-correlation with kernel [K, C, S] (conv1d_op.mojo): the 2-D kernels on a height-1 image."""
    if x.ndim() != 3:
        raise ValueError("Input must be 3-dimensional (batch_size, in_channels, length) for 1D convolution!")
    if x._shape[1] != kernel._shape[1]:
        raise ValueError("Input channels must match kernel channels for 1D convolution!")
    N, C, Ln = x._shape
    K, _, S = kernel._shape
    y = conv2d(reshape(x, [N, C, 1, Ln]), reshape(kernel, [K, C, 1, S]), bias, (1, int(stride)), (0, int(padding)),
               (1, int(dilation)), groups)
    return reshape(y, [N, K, y._shape[-1]])


def conv3d(x, kernel, bias=None, stride=(1, 1, 1), padding=(0, 0, 0), dilation=(1, 1, 1), groups=1):
    """[N, C, D, H, W] cross-correlation with kernel [K, C, T, R, S] (conv3d_op.mojo:104-259; tuple order is
    (depth, height, width)). The reference has no backward rule for it (conv3d_op.mojo:261-263); the VJP here
    is the adjoint of its forward loop."""
    import ctypes
    if x.ndim() != 5:
        raise ValueError("Input must be 5-dimensional (batch_size, in_channels, depth, height, width) for 3D convolution!")
    if x._shape[1] != kernel._shape[1]:
        raise ValueError("Input channels must match kernel channels for 3D convolution!")
    if x.is_complex_ or kernel.is_complex_:
        raise ValueError("Complex numbers are not supported for conv3d!")
    desc = L.Conv3dDesc()
    desc.N, desc.C, desc.D, desc.H, desc.W = x._shape
    desc.K, _, desc.T, desc.R, desc.S = kernel._shape
    desc.stride[:], desc.padding[:], desc.dilation[:] = _tuple_n(stride, 3), _tuple_n(padding, 3), _tuple_n(dilation, 3)
    desc.groups = groups
    o = (ctypes.c_int64 * 3)()
    L.call("endia_hip_conv3d_out_shape", ctypes.byref(desc), o)
    xs, ks = contiguous(x), contiguous(kernel)
    bsrc = contiguous(bias) if bias is not None else None
    out = Array.empty([desc.N, desc.K, o[0], o[1], o[2]])
    L.call("endia_hip_conv3d_fwd", ctypes.byref(desc), xs.data_ptr(), ks.data_ptr(),
           bsrc.data_ptr() if bsrc is not None else None, out.data_ptr(), L.OP_IDENTITY)

    def vjp(primals, grad, out_):
        from .autograd.functional import building_graph
        if building_graph():
            raise NotImplementedError("conv3d has no second-order rule")
        if grad.ndim() != out_.ndim():
            raise NotImplementedError("conv3d has no rule for a cotangent with leading Jacobian axes (non-scalar output)")
        g = contiguous(grad)
        res = [None] * len(primals)
        if primals[0]._requires_grad:
            res[0] = Array.empty(primals[0]._shape)
            L.call("endia_hip_conv3d_bwd_data", ctypes.byref(desc), g.data_ptr(), ks.data_ptr(), res[0].data_ptr())
        if primals[1]._requires_grad:
            res[1] = Array.empty(primals[1]._shape)
            L.call("endia_hip_conv3d_bwd_weight", ctypes.byref(desc), xs.data_ptr(), g.data_ptr(), res[1].data_ptr())
        if len(primals) > 2 and primals[2]._requires_grad:
            res[2] = Array.empty(primals[2]._shape)
            L.call("endia_hip_conv3d_bwd_bias", ctypes.byref(desc), g.data_ptr(), res[2].data_ptr())
        return res

    return _register(out, [x, kernel] + ([bias] if bias is not None else []), "conv3d", vjp)


# --------------------------------------------------------------------------------------------------
# pooling (endia/functional/spacial_ops/{max,avg}_pool{1,2,3}d_op.mojo)
# --------------------------------------------------------------------------------------------------
def _tuple_n(v, n):
    return (int(v),) * n if np.isscalar(v) else tuple(int(e) for e in v)


_POOL_RANK_ERR = {
    1: "Input must be 3-dimensional (batch_size, channels, length) for 1D pooling!",
    2: "Input must be 4-dimensional (batch_size, channels, height, width) for 2D pooling!",
    3: "Input must be 5-dimensional (batch_size, channels, depth, height, width) for 3D pooling!",
}


def _pool(x, mode, nsp, kernel_size, stride, padding, dilation):
    """Shared body of the six pooling ops. The reference has no backward rule for them (vjp = default_vjp,
    max_pool2d_op.mojo:152-154); the VJP here is the adjoint of its forward loop."""
    import ctypes
    name = ("max" if mode == L.POOL_MAX else "avg") + "_pool%dd" % nsp
    if x.ndim() != nsp + 2:
        raise ValueError(_POOL_RANK_ERR[nsp])
    if x.is_complex_:
        raise ValueError("Complex numbers are not supported for %s!" % name)
    desc = L.PoolDesc()
    desc.N, desc.C = x._shape[0], x._shape[1]
    desc.D, desc.H, desc.W = [1] * (3 - nsp) + list(x._shape[2:])
    for field, v, fill in (("kernel", kernel_size, 1), ("stride", stride, 1), ("padding", padding, 0), ("dilation", dilation, 1)):
        getattr(desc, field)[:] = [fill] * (3 - nsp) + list(_tuple_n(v, nsp))
    o = (ctypes.c_int64 * 3)()
    L.call("endia_hip_pool_out_shape", ctypes.byref(desc), o)
    out_shape = list(x._shape[:2]) + list(o[3 - nsp:])
    xs = contiguous(x)
    out = Array.empty(out_shape)
    arg = Buffer(4 * max(out.size(), 1)) if (mode == L.POOL_MAX and x._requires_grad) else None
    L.call("endia_hip_pool_fwd", ctypes.byref(desc), mode, xs.data_ptr(), out.data_ptr(), arg.ptr if arg else None)

    def vjp(primals, grad, out_):
        from .autograd.functional import building_graph
        if building_graph():
            raise NotImplementedError("%s has no second-order rule" % name)
        if grad.ndim() != out_.ndim():
            raise NotImplementedError("%s has no rule for a cotangent with leading Jacobian axes (non-scalar output)" % name)
        g = contiguous(grad)
        dx = Array.empty(primals[0]._shape)
        L.call("endia_hip_pool_bwd", ctypes.byref(desc), mode, g.data_ptr(), arg.ptr if arg else None, dx.data_ptr())
        return [dx]

    return _register(out, [x], name, vjp)


def max_pool1d(x, kernel_size, stride=1, padding=0, dilation=1):
    return _pool(x, L.POOL_MAX, 1, kernel_size, stride, padding, dilation)


def max_pool2d(x, kernel_size, stride=(1, 1), padding=(0, 0), dilation=(1, 1)):
    return _pool(x, L.POOL_MAX, 2, kernel_size, stride, padding, dilation)


def max_pool3d(x, kernel_size, stride=(1, 1, 1), padding=(0, 0, 0), dilation=(1, 1, 1)):
    return _pool(x, L.POOL_MAX, 3, kernel_size, stride, padding, dilation)


def avg_pool1d(x, kernel_size, stride=1, padding=0, dilation=1):
    return _pool(x, L.POOL_AVG, 1, kernel_size, stride, padding, dilation)


def avg_pool2d(x, kernel_size, stride=(1, 1), padding=(0, 0), dilation=(1, 1)):
    return _pool(x, L.POOL_AVG, 2, kernel_size, stride, padding, dilation)


def avg_pool3d(x, kernel_size, stride=(1, 1, 1), padding=(0, 0, 0), dilation=(1, 1, 1)):
    return _pool(x, L.POOL_AVG, 3, kernel_size, stride, padding, dilation)


# --------------------------------------------------------------------------------------------------
# fused dense layer: act(x @ W + b) as one GEMM with an epilogue (nn/modules/_mlp.mojo:50-52)
# --------------------------------------------------------------------------------------------------
_ACT = {None: L.OP_IDENTITY, "identity": L.OP_IDENTITY, "relu": L.OP_RELU, "tanh": L.OP_TANH, "sin": L.OP_SIN}
_ACT_FN = {"relu": relu, "tanh": tanh, "sin": sin}


def linear(x, W, b, act=None):
    """out = act(x @ W + b) with W [in, out] (no transpose: _mlp.mojo:50).

    Forward: one MFMA GEMM whose epilogue adds the bias row and applies the activation. Backward of a
    first-order pass: dW = x^T g' (TN GEMM), db = column sum of g', dx = g' W^T (NT GEMM) where
    g' = g * act'(.). When x is itself the output of a fused layer with a single consumer, that
    layer's activation derivative is applied in the epilogue of THIS layer's dx GEMM and the gradient
    is handed over marked as already carrying it. With create_graph=True the rules are written in
    differentiable ops instead: relu and tanh through the layer's own output, sin through the stored
    pre-activation, which for that purpose is a node of its own (the kernel writes both z and sin(z)).
    """
    if x.ndim() != 2 or x.is_complex_ or W.is_complex_ or act not in _ACT:
        z = add(matmul(x, W), b)
        return _ACT_FN[act](z) if act in _ACT_FN else z
    xs, Ws, bs_ = contiguous(x), contiguous(W), contiguous(b)
    B, K = xs._shape
    N = Ws._shape[1]
    out = Array.empty([B, N])
    keep_z = act == "sin" and (x._requires_grad or W._requires_grad or b._requires_grad)
    z = Array.empty([B, N]) if keep_z else None
    epi = L.EPI_BIAS if _ACT[act] == L.OP_IDENTITY else L.EPI_BIAS_ACT
    L.call("endia_hip_sgemm", 0, 0, B, N, K, xs.data_ptr(), K, Ws.data_ptr(), N, out.data_ptr(), N, 1, 0, 0, 0, epi,
           _ACT[act], bs_.data_ptr(), None, z.data_ptr() if keep_z else None)
    if keep_z:
        zz = _linear_node(z, x, W, b, xs, Ws, None)
        return _sin_of_linear_node(out, zz)
    return _linear_node(out, x, W, b, xs, Ws, act)


def _starts_on_16(*arrays):
    """Views that begin on a 16-byte boundary of their (256-byte aligned) buffers, or would after the contiguous copy a
    non-contiguous one gets: what the whole-model entry points ask of everything but the weights."""
    return all((a._offset * 4) % 16 == 0 or not a.is_contiguous() for a in arrays)


def mlp_forward(x, weights, biases, act=None):
    """The whole dense stack of nn.MLP.forward (nn/modules/_mlp.mojo:47-53) as ONE op: act after every layer but the
    last. For small models (every width at most 128, like the reference's benchmark model) the forward pass is one
    launch and the backward pass two (endia_hip_mlp_fwd / endia_hip_mlp_bwd); anything else, and complex operands, fall
    back to one fused layer at a time. First order only: a pass with create_graph=True, or a non-scalar output's
    Jacobian seed, needs the per-layer graph (`nn.MLP(fused=True)`) and is refused here."""
    import ctypes
    Lyr = len(weights)
    widths = [x._shape[-1]] + [w._shape[1] for w in weights]
    small = (x.ndim() == 2 and 1 <= Lyr <= L.MLP_MAX_LAYERS and act in (None, "identity", "relu", "tanh") and x.size() > 0
             and not x.is_complex_ and all(1 <= n <= L.MLP_MAX_WIDTH for n in widths)
             and all(w.ndim() == 2 and not w.is_complex_ and w._shape[0] == widths[i] for i, w in enumerate(weights))
             and all(b.size() == widths[i + 1] and not b.is_complex_ for i, b in enumerate(biases))
             and _starts_on_16(x, *biases))
    if not small:
        h = x
        for i in range(Lyr):
            h = linear(h, weights[i], biases[i], None if i == Lyr - 1 else act)
        return h
    B = x._shape[0]
    xs = contiguous(x)
    Ws, bs_ = [contiguous(w) for w in weights], [contiguous(b) for b in biases]
    hs = [Array.empty([B, widths[i + 1]]) for i in range(Lyr)]
    desc = L.MlpDesc()
    desc.layers, desc.act, desc.batch = Lyr, _ACT[act], B
    desc.widths[:Lyr + 1] = widths
    ptrs = lambda arrs: (ctypes.c_void_p * Lyr)(*[a.data_ptr() if a is not None else None for a in arrs])
    # The forward launch is parked, not issued: mse() of this output (the reference script's next call, mlp_imp.mojo:56-60)
    # withdraws it and runs the launch that evaluates the loss and the cotangents of all layers as well; anything else that
    # reads the output, or any call that is not a pure function of fresh buffers, launches it as it is.
    x_ptr, W_ptrs, b_ptrs = xs.data_ptr(), ptrs(Ws), ptrs(bs_)
    h_ptrs = (ctypes.c_void_p * Lyr)(*[h._buf.address for h in hs])

    def launch_forward():
        L._raw_call("endia_hip_mlp_fwd", ctypes.byref(desc), x_ptr, W_ptrs, b_ptrs, h_ptrs)

    if L.defer_products[0]:
        ticket = L.park_launch(launch_forward, [h._buf for h in hs])
        hs[-1]._lazy_mlp = (ticket, xs, Ws, bs_, hs, desc, widths, act, x, list(weights), list(biases))
    else:
        launch_forward()

    def vjp(primals, grad, out_):
        from .autograd.functional import building_graph
        if building_graph() or grad.ndim() != out_.ndim():
            raise NotImplementedError("mlp_forward is a first-order op; build the model with fused=True for higher-order or Jacobian passes")
        deltas = [Array.empty([B, widths[i + 1]]) for i in range(Lyr - 1)] + [contiguous(grad)]
        pW, pb = primals[1:1 + Lyr], primals[1 + Lyr:]
        dW = [Array.empty([widths[i], widths[i + 1]]) if pW[i]._requires_grad else None for i in range(Lyr)]
        db = [Array.empty([1, widths[i + 1]]) if pb[i]._requires_grad else None for i in range(Lyr)]  # kept axis, like Expand.vjp
        dx = Array.empty([B, widths[0]]) if primals[0]._requires_grad else None
        L.call("endia_hip_mlp_bwd", ctypes.byref(desc), xs.data_ptr(), ptrs(Ws), ptrs(hs), ptrs(deltas), ptrs(dW), ptrs(db),
               dx.data_ptr() if dx is not None else None)
        return [dx] + dW + db

    return _register(hs[-1], [x] + list(weights) + list(biases), "mlp", vjp)


def mlp_mse_loss(x, target, weights, biases, act=None):
    """mse(mlp_forward(x, weights, biases, act), target) for a small model (see mlp_forward) with the loss evaluated by the
    forward launch itself (endia_hip_mlp_fwd_mse_delta: the outputs of a work-group's rows are still on chip when the
    last layer is done, so the squared differences, the loss gradient 2 (out - target) / n and, since every row is
    independent through the whole chain, the cotangents of all layers cost no launch of their own). backward() then is
    the one launch of endia_hip_mlp_wgrad: with the optimizer, 3 launches for a training step of the reference's script
    (mlp_imp.mojo:56-68). A cotangent other than the seed runs the chain again from the scaled loss gradient. Anything the fused launch does not cover (a model
    that is not small, a target that needs a gradient, complex operands) is mse(mlp_forward(...)); a second-order pass
    fails as it does for mlp_forward. Returns the loss, shape [1]."""
    import ctypes
    Lyr = len(weights)
    widths = [x._shape[-1]] + [w._shape[1] for w in weights]
    small = (x.ndim() == 2 and 1 <= Lyr <= L.MLP_MAX_LAYERS and act in (None, "identity", "relu", "tanh") and x.size() > 0
             and not x.is_complex_ and not target._requires_grad and not target.is_complex_
             and list(target._shape) == [x._shape[0], widths[-1]]
             and all(1 <= n <= L.MLP_MAX_WIDTH for n in widths)
             and all(w.ndim() == 2 and not w.is_complex_ and w._shape[0] == widths[i] for i, w in enumerate(weights))
             and all(b.size() == widths[i + 1] and not b.is_complex_ for i, b in enumerate(biases))
             and _starts_on_16(x, target, *biases))
    if not small:
        return mse(mlp_forward(x, weights, biases, act), target)
    B = x._shape[0]
    xs = contiguous(x)
    Ws, bs_ = [contiguous(w) for w in weights], [contiguous(b) for b in biases]
    hs = [Array.empty([B, widths[i + 1]]) for i in range(Lyr)]
    desc = L.MlpDesc()
    desc.layers, desc.act, desc.batch = Lyr, _ACT[act], B
    desc.widths[:Lyr + 1] = widths
    return _mlp_mse_launch(x, target, list(weights), list(biases), xs, Ws, bs_, hs, desc, widths, None)


def _mlp_mse_fused(lazy, pred, target):
    """mse(pred, target) where pred is the output of a whole-model forward whose launch was still parked (and has just
    been withdrawn): the launch of mlp_mse_loss on the very arrays that forward pass was going to write."""
    _, xs, Ws, bs_, hs, desc, widths, act, x, weights, biases = lazy
    return _mlp_mse_launch(x, target, weights, biases, xs, Ws, bs_, hs, desc, widths, pred)


def _mlp_mse_launch(x, target, weights, biases, xs, Ws, bs_, hs, desc, widths, pred):
    import ctypes
    Lyr, B = len(weights), x._shape[0]
    ts = contiguous(target)
    loss = Array.empty([1])
    ptrs = lambda arrs: (ctypes.c_void_p * Lyr)(*[a.data_ptr() if a is not None else None for a in arrs])
    # With something to differentiate, the forward launch goes on to the cotangents of all layers for the loss gradient
    # (rows are independent through the whole chain), and backward() is left with the weight gradients.
    wants = [a._requires_grad for a in [x] + list(weights) + list(biases)]
    deltas = [Array.empty([B, widths[i + 1]]) for i in range(Lyr)]
    dx0 = Array.empty([B, widths[0]]) if wants[0] else None
    if any(wants):
        L.call("endia_hip_mlp_fwd_mse_delta", ctypes.byref(desc), xs.data_ptr(), ptrs(Ws), ptrs(bs_), ts.data_ptr(), ptrs(hs), ptrs(deltas),
               loss.data_ptr(), dx0.data_ptr() if dx0 is not None else None)
    else:
        L.call("endia_hip_mlp_fwd_mse", ctypes.byref(desc), xs.data_ptr(), ptrs(Ws), ptrs(bs_), ts.data_ptr(), ptrs(hs), deltas[-1].data_ptr(),
               loss.data_ptr())

    def vjp(primals, grad, out_):
        from .autograd.functional import building_graph
        if building_graph():
            raise NotImplementedError("mlp_mse_loss is a first-order op; use mse(model.forward(x), target) with fused=True for higher-order passes")
        pW, pb = primals[2:2 + Lyr], primals[2 + Lyr:]
        dW = [Array.empty([widths[i], widths[i + 1]]) if pW[i]._requires_grad else None for i in range(Lyr)]
        db = [Array.empty([1, widths[i + 1]]) if pb[i]._requires_grad else None for i in range(Lyr)]  # kept axis, like Expand.vjp
        want_dx = primals[0]._requires_grad
        if _holds_seed(grad) and any(wants) and (dx0 is not None or not want_dx):
            L.call("endia_hip_mlp_wgrad", ctypes.byref(desc), xs.data_ptr(), ptrs(hs), ptrs(deltas), ptrs(dW), ptrs(db))
            if pred is not None and not pred.has_grad():
                pred.grad_(deltas[-1])  # what mse's own rule would have stored on the model's output
            return [dx0 if want_dx else None, None] + dW + db
        # a cotangent other than the seed scales the stored loss gradient; the chain is run again from there
        last = deltas[-1] if _holds_seed(grad) else mul(deltas[-1], grad)
        again = [Array.empty([B, widths[i + 1]]) for i in range(Lyr - 1)] + [contiguous(last)]
        dx = Array.empty([B, widths[0]]) if want_dx else None
        L.call("endia_hip_mlp_bwd", ctypes.byref(desc), xs.data_ptr(), ptrs(Ws), ptrs(hs), ptrs(again), ptrs(dW), ptrs(db),
               dx.data_ptr() if dx is not None else None)
        return [dx, None] + dW + db

    return _register(loss, [x, target] + list(weights) + list(biases), "mlp_mse", vjp)


def _fused_act_of(px):
    """The activation a gradient may absorb on its way to px: px is the output of a fused layer (or the
    fused sin node on top of one), nothing else consumes it and it holds no earlier gradient."""
    m = px._meta
    if not m or m.get("act") not in _ACT_FN or px._consumers != 1 or px.has_grad():
        return None
    return m


def _sin_of_linear_node(out, zz):
    n = out.size()

    def vjp(primals, grad, out_):
        from .autograd.functional import building_graph
        z = primals[0]
        if building_graph() and grad._shape == z._shape:
            return [_fused_rule("cos_mul", lambda zz_, g: mul(cos(zz_), g))(z, grad)]  # sin_op.mojo:92 as one node
        if building_graph() or grad.ndim() != out_.ndim():  # (a Jacobian seed's leading axes broadcast through mul)
            return [mul(cos(z), grad)]  # sin_op.mojo:92
        if grad._act_applied:
            # the layer above already multiplied by cos(z): for the pre-activation node that IS its gradient, so it is
            # handed on as a plain array (z.grad() then shows dL/dz, not the hidden activation's dL/dh)
            return [Array(grad._shape, _buffer=grad._buf, _strides=grad._strides, _offset=grad._offset)]
        offer = _absorb_offer(z)
        if offer is not None and offer[0]._shape == z._shape and grad._shape == z._shape and not offer[0].is_complex_:
            # z already holds a gradient (a second-order pass reaches the pre-activation twice): one launch for both
            gz = _fused_rule("cos_mul_add", lambda zz_, g_, e_: add(mul(cos(zz_), g_), e_))(detach(z), detach(grad), detach(offer[0]))
            gz._absorbed = True
            _absorbed_launches[0] += 1
            return [gz]
        g = contiguous(grad)
        gz = Array.empty(out_._shape)
        L.call("endia_hip_unary_vjp", L.OP_SIN, n, z.data_ptr(), g.data_ptr(), gz.data_ptr(), 0)
        return [gz]

    return _register(out, [zz], "sin", vjp, {"act": "sin", "aux": zz, "from_output": False})


def _linear_node(out, x, W, b, xs, Ws, act):
    B, K = xs._shape
    N = Ws._shape[1]

    def vjp(primals, grad, out_):
        from .autograd.functional import building_graph
        px, pW, pb = primals
        lead = grad.ndim() - out_.ndim()  # leading axes of a Jacobian seed (autograd/functional.mojo:35-37)
        if building_graph() or lead:
            if act == "tanh" and not lead:
                g = _fused_rule("tanh_out_mul", lambda o, gg: mul(1 - square(o), gg))(out_, grad)
            elif act == "relu" and not lead:
                g = _fused_rule("relu_out_mul", lambda o, gg: mul(greater(o, 0.0), gg))(out_, grad)
            elif act == "tanh":
                g = mul(1 - square(out_), grad)                      # tanh_op.mojo:92 with tanh(z) = out
            elif act == "relu":
                g = mul(greater(out_, zeros([N])), grad)             # relu_op.mojo:95; out > 0 iff z > 0
            else:
                g = grad
            # matmul treats the leading axes as a batch; the bias gradient sums the layer's batch axis, which follows them
            return [matmul(g, pW.T()) if px._requires_grad else None,
                    matmul(px.T(), g) if pW._requires_grad else None,
                    reduce_add(g, [lead]) if pb._requires_grad else None]
        g = contiguous(grad)
        if act in _ACT_FN and not grad._act_applied:  # relu and tanh derivatives from the stored output
            gp = Array.empty([B, N])
            L.call("endia_hip_unary_vjp_from_output", _ACT[act], B * N, out_.data_ptr(), g.data_ptr(), gp.data_ptr())
            g = gp
        # endia_hip_linear_bwd: dW = x^T g, db = column sums of g, dx = (g W^T) * act'(.) of the layer below -- one
        # launch for a small layer, the separate GEMMs (and the reduction) for a large one
        db = Array.empty([1, N]) if pb._requires_grad else None  # kept leading axis, like Expand.vjp (expand_op.mojo:121-126)
        dW = Array.empty([K, N]) if pW._requires_grad else None
        dx, flags, aux = None, L.OP_IDENTITY, None
        if px._requires_grad:
            dx = Array.empty([B, K])
            pm = _fused_act_of(px)
            if pm:  # px is a fused layer's output with this one consumer: its activation derivative rides along
                flags = _ACT[pm["act"]] | (L.ACT_FROM_OUTPUT if pm["from_output"] else 0)
                aux = contiguous(pm["aux"])
                dx._act_applied = True
                # what px.grad() shows is dL/dpx itself; nobody reads it in a training step, so it is made on demand
                # (it multiplies by the weights as they are when it runs: asked for after an optimizer step or any
                # other in-place write to W it would silently use the new ones, so it refuses then. It keeps this
                # layer's cotangent alive until it has run once or zero_grad / remove_grad drops it.)
                w_version = Ws._buf.version

                def true_grad():
                    if Ws._buf.version != w_version:
                        raise RuntimeError("the gradient of a hidden activation of a fused layer is computed on first use and was asked for "
                                           "after the layer's weights were updated in place: read it before optimizer.step(), or build "
                                           "the model with fused=False")
                    return matmul(detach(g), detach(Ws).T())
                dx._true_grad = true_grad
        # A weight or an input that already holds a gradient nobody else refers to (second-order passes reach both
        # twice) takes this layer's product on top of it in the GEMM's epilogue instead of through an `add` launch.
        def in_place(offer, shape):
            if offer is None or not offer[1] or B * K * N == 0:
                return None
            g0 = offer[0]
            if list(g0._shape) != shape or not g0.is_contiguous() or g0.is_complex_:
                return None
            _absorbed_launches[0] += 1
            tot = Array(shape, _buffer=g0._buf, _offset=g0._offset)
            tot._absorbed = True
            return tot
        accW = in_place(_absorb_offer(pW), [K, N]) if dW is not None and pW is not px else None
        accX = in_place(_absorb_offer(px), [B, K]) if dx is not None and aux is None and pW is not px else None
        # The data gradient first, the weight gradient last (an optimizer that updates inside backward() then finds it in
        # the last-level cache). Products that accumulate, or that are of the size that shares launches (_would_park), go
        # through _sgemm piece by piece; a large layer's bias gradient is a reduction of its own either way, a small one's
        # rides in the weight-gradient launch. Everything else is one endia_hip_linear_bwd call.
        split = B * N > (1 << 20)
        own_W = accW is not None or (dW is not None and split and _would_park(K, N, B))
        if accX is not None:
            _sgemm(0, 1, B, K, N, g, N, Ws, N, accX, L.EPI_NONE | L.GEMM_ACCUMULATE)
        lib_dx = dx if accX is None else None
        if own_W:
            if lib_dx is not None:
                L.call("endia_hip_linear_bwd", B, K, N, xs.data_ptr(), Ws.data_ptr(), g.data_ptr(), flags,
                       aux.data_ptr() if aux is not None else None, lib_dx.data_ptr(), None, None)
            tgt = accW if accW is not None else dW
            epi_w = L.EPI_NONE | (L.GEMM_ACCUMULATE if accW is not None else 0)
            if db is not None and split:
                if _col_sum_parks(g):
                    _park_col_sum(g, db, 1.0)
                else:
                    L.call("endia_hip_reduce_add", 2, L.i64_array([B, N]), 1, g.data_ptr(), db.data_ptr(), 1.0, 0)
                _sgemm(1, 0, K, N, B, xs, K, g, N, tgt, epi_w)
            else:
                L.call("endia_hip_sgemm", 1, 0, K, N, B, xs.data_ptr(), K, g.data_ptr(), N, tgt.data_ptr(), N, 1, 0, 0, 0,
                       epi_w | (L.GEMM_COLSUM_B if db is not None else 0), L.OP_IDENTITY, None, None,
                       db.data_ptr() if db is not None else None)
        elif lib_dx is not None or dW is not None or db is not None:
            L.call("endia_hip_linear_bwd", B, K, N, xs.data_ptr(), Ws.data_ptr(), g.data_ptr(), flags,
                   aux.data_ptr() if aux is not None else None, lib_dx.data_ptr() if lib_dx is not None else None,
                   dW.data_ptr() if dW is not None else None, db.data_ptr() if db is not None else None)
        return [accX if accX is not None else dx, accW if accW is not None else dW, db]

    meta = {"act": act, "aux": out, "from_output": True} if act in _ACT_FN else {"act": None}
    return _register(out, [x, W, b], "linear", vjp, meta)
