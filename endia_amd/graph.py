"""Captured steps: record one training step's kernels into a HIP graph and replay it with one launch.

The reference has a trace-cache JIT for repeated graphs (endia/compile/fx.mojo); on the GPU the
equivalent for launch-latency-bound steps is a HIP graph of the very kernels the eager step issues.
Nothing is compiled or fused differently: the captured step computes bit for bit what the eager
step computes.

    def step():
        loss = nd.mse(mlp.forward(x), y)
        loss.backward()
        opt.step()          # SGD / Adagrad / RMSprop, or Adam(capturable=True); see below
        loss.zero_grad()
        return loss

    step()                          # once eagerly: fills the buffer pool and the reduction workspace
    captured = nd.capture(step)     # records, does not execute
    for batch in data:
        x.copy_from_numpy(batch)    # inputs are updated in place: the graph reads fixed addresses
        captured.replay()
    print(captured.outputs.item())

Scalar kernel arguments are frozen at capture time. Adam's bias correction 1 - beta^t changes every step:
`Adam(..., capturable=True)` keeps t in device memory, where the update kernel reads it and a last tiny
kernel adds one, so nothing in the recorded launches depends on the step number; an Adam whose counter
lives on the host refuses to run inside a capture.
"""
import ctypes

from . import _lib as L
from ._array import Array, _contiguous_copy


class CapturedStep:
    def __init__(self, fn):
        self.handle = None
        L.call("endia_hip_graph_begin")
        L.capturing = True
        try:
            self.outputs = fn()
        except BaseException:
            L.capturing = False
            h = ctypes.c_int64()
            if L.lib().endia_hip_graph_end(ctypes.byref(h)) == 0:
                L.lib().endia_hip_graph_destroy(h.value)
            raise
        L.capturing = False
        h = ctypes.c_int64()
        L.call("endia_hip_graph_end", ctypes.byref(h))
        self.handle = h.value

    def replay(self):
        if self.handle is None:
            raise RuntimeError("this captured step has been closed")
        L.call("endia_hip_graph_launch", self.handle)
        return self.outputs

    __call__ = replay

    def close(self):
        if self.handle is not None:
            try:
                L.lib().endia_hip_graph_destroy(self.handle)
            except Exception:
                pass
            self.handle = None

    def __del__(self):
        self.close()


def capture(fn):
    """Record everything `fn()` enqueues and return a CapturedStep; `fn` must not read device data."""
    return CapturedStep(fn)


def _leaves(tree, out):
    """The arrays of a nest of lists/tuples, left to right."""
    if isinstance(tree, Array):
        out.append(tree)
    elif isinstance(tree, (list, tuple)):
        for t in tree:
            _leaves(t, out)
    elif tree is not None:
        raise TypeError("jit: arguments and results must be arrays or lists of arrays, not %s" % type(tree).__name__)
    return out


def _rebuild(tree, it):
    if isinstance(tree, Array):
        return next(it)
    if isinstance(tree, (list, tuple)):
        return type(tree)(_rebuild(t, it) for t in tree)
    return None


class JitCallable:
    """jit(fn): the call-compatible counterpart of the reference's caching Callable (endia/compile/callable.mojo:60-98,
    endia/compile/functional.mojo:43-88).

    The reference keeps one set of argument arrays per jitted function, copies each call's inputs into them, runs
    the cached graph and hands back copies of the results. The same here, with a HIP graph as the cache: the first
    call with a given list of input shapes runs `fn` once eagerly on private copies of the inputs (which sizes the
    buffer pool), records a second run into a graph, and from then on a call is: copy the inputs in (device to
    device), one graph launch, copy the results out. `fn` must be a pure function of its array arguments that
    enqueues the same kernels on every call and reads no device data on the host (no item(), to_numpy() or host
    uploads inside); one that does fails at the first call with the library's "not allowed while a step is being
    captured" error. Inputs of another shape get a graph of their own.
    """

    def __init__(self, fn):
        self.fn = fn
        self._cache = {}

    def __call__(self, *args):
        if L.capturing:  # a jitted function used inside a captured step is simply part of that step
            return self.fn(*args)
        given = _leaves(args, [])
        key = tuple((tuple(a._shape), a.is_complex_, a._requires_grad) for a in given)
        entry = self._cache.get(key)
        if entry is None:
            held = [_contiguous_copy(a).requires_grad_(a._requires_grad) for a in given]
            private = _rebuild(args, iter(held))
            self.fn(*private)
            step = CapturedStep(lambda: self.fn(*private))
            entry = self._cache[key] = (held, step, _leaves(step.outputs, []))
        else:
            for mine, a in zip(entry[0], given):
                mine._assign_from(a)
        held, step, results = entry
        step.replay()
        return _rebuild(step.outputs, iter([_contiguous_copy(r) for r in results]))

    def close(self):
        for _, step, _ in self._cache.values():
            step.close()
        self._cache.clear()


def jit(fn, compile_with_MAX=False):
    """nd.jit(fn): see JitCallable. `compile_with_MAX` is accepted for call compatibility and must stay False: there
    is no MAX engine here (endia/compile/functional.mojo:43-55)."""
    if compile_with_MAX:
        raise NotImplementedError("jit: compile_with_MAX=True asks for the MAX engine, which this library does not have")
    return JitCallable(fn)
