"""SGD, Adam, Adagrad and RMSprop: the host-side mirror of endia/optim/{sgd,adam,adagrad,rmsprop}.mojo.

The reference builds every update from separate Array ops; here `step()` is one fused kernel per
parameter tensor, writing the parameter (and the moments) in place, which is what the reference's
`-=` does through a raw copy (endia/_array/_array.mojo:998-1006). A gradient may carry a kept leading
axis ([1, N] for an [N] bias: view_ops/expand_op.mojo:121-126); only the element count must match.
"""
import numpy as np

from . import _lib as L
from . import functional as F
from ._array import Array


def _flat_grad(p):
    if not p.has_grad():
        raise ValueError("optimizer.step(): a parameter has no gradient")
    g = F.contiguous(p.grad())
    if g.size() != p.size():
        raise ValueError("gradient of shape %s does not match parameter %s" % (g.shape(), p.shape()))
    return g


class SGD:
    """sgd.mojo:14-63: plain `p -= lr * p.grad()`, or with momentum (velocity = momentum * velocity - lr * (grad +
    weight_decay * p); p += velocity) and / or weight decay."""

    def __init__(self, params, lr=0.01, momentum=0.0, weight_decay=0.0):
        self.params = list(params)
        self.lr, self.momentum, self.weight_decay = (float(np.float32(v)) for v in (lr, momentum, weight_decay))
        self.velocity = [Array(p.shape()) for p in self.params] if self.momentum > 0 else []

    def step(self):
        if self.momentum == 0 and self.weight_decay == 0 and len(self.params) > 1:
            # plain SGD: every parameter tensor in one launch
            import ctypes
            grads = [_flat_grad(p) for p in self.params]
            k = len(self.params)
            assert all(p.is_contiguous() for p in self.params)
            L.call("endia_hip_sgd_step_multi", k, L.i64_array([p.size() for p in self.params]),
                   (ctypes.c_void_p * k)(*[p.data_ptr() for p in self.params]),
                   (ctypes.c_void_p * k)(*[g.data_ptr() for g in grads]), self.lr)
            for p in self.params:
                p.clear_args()
                p._buf.version += 1
            return
        for i, p in enumerate(self.params):
            g = _flat_grad(p)
            assert p.is_contiguous()
            if self.momentum > 0 or self.weight_decay > 0:
                vel = self.velocity[i].data_ptr() if self.momentum > 0 else None
                L.call("endia_hip_sgd_momentum_step", p.size(), p.data_ptr(), g.data_ptr(), vel, self.lr, self.momentum,
                       self.weight_decay)
            else:
                L.call("endia_hip_sgd_step", p.size(), p.data_ptr(), g.data_ptr(), self.lr)
            p.clear_args()
            p._buf.version += 1


class Adagrad:
    """adagrad.mojo:14-45."""

    def __init__(self, params, lr=0.01, eps=1e-8):
        self.params = list(params)
        self.lr, self.eps = float(np.float32(lr)), float(np.float32(eps))
        self.cache = [Array(p.shape()) for p in self.params]

    def step(self):
        for p, c in zip(self.params, self.cache):
            g = _flat_grad(p)
            assert p.is_contiguous()
            L.call("endia_hip_adagrad_step", p.size(), p.data_ptr(), g.data_ptr(), c.data_ptr(), self.lr, self.eps)
            p.clear_args()
            p._buf.version += 1


class RMSprop:
    """rmsprop.mojo:14-53."""

    def __init__(self, params, lr=0.01, alpha=0.99, eps=1e-8):
        self.params = list(params)
        self.lr, self.alpha, self.eps = (float(np.float32(v)) for v in (lr, alpha, eps))
        self.cache = [Array(p.shape()) for p in self.params]

    def step(self):
        for p, c in zip(self.params, self.cache):
            g = _flat_grad(p)
            assert p.is_contiguous()
            L.call("endia_hip_rmsprop_step", p.size(), p.data_ptr(), g.data_ptr(), c.data_ptr(), self.lr, self.alpha, self.eps)
            p.clear_args()
            p._buf.version += 1


class Adam:
    """adam.mojo:14-65. `t` is an fp32 counter that starts at 1 and grows by one per step().

    capturable=True (or the first step() taken while a step is being captured) keeps the counter in device memory
    and updates every parameter tensor in one launch that reads it there, so the step can be replayed as a HIP
    graph; the bias corrections then come from the device's powf (last-bit differences from the host's).

    fused_backward=True (no counterpart in the reference): backward() itself applies this optimizer's update to a
    parameter the moment that parameter's gradient is complete (every consumer in the graph has contributed), while
    the gradient is still in the last-level cache and before the walk moves on to the layers below; step() then only
    updates what backward() did not reach and advances t. Same arithmetic, same results as step() after backward();
    `p.grad()` stays readable. For loops that run exactly one backward() per step(): a second backward() before
    step() would update again. Passes with create_graph=True never update. Not together with capturable."""

    def __init__(self, params, lr=0.001, beta1=0.9, beta2=0.999, eps=1e-8, capturable=False, fused_backward=False):
        self.params = list(params)
        self.lr, self.beta1, self.beta2, self.eps = (float(np.float32(v)) for v in (lr, beta1, beta2, eps))
        self.t = 1.0
        self.m = [Array(p.shape()) for p in self.params]
        self.v = [Array(p.shape()) for p in self.params]
        self._t_dev = None
        if capturable and fused_backward:
            raise ValueError("Adam: fused_backward and capturable cannot be combined")
        if capturable:
            self._device_counter()
        self._updated = [False] * len(self.params)
        if fused_backward:
            for i, p in enumerate(self.params):
                p._on_final_grad = (lambda leaf, i=i: self._update(i))

    def _update(self, i):
        if self._updated[i] or L.capturing:
            return
        p = self.params[i]
        g = _flat_grad(p)
        assert p.is_contiguous()
        L.call("endia_hip_adam_step", p.size(), p.data_ptr(), g.data_ptr(), self.m[i].data_ptr(), self.v[i].data_ptr(), self.lr,
               self.beta1, self.beta2, self.eps, self.t)
        p.clear_args()
        p._buf.version += 1
        self._updated[i] = True

    def _device_counter(self):
        if self._t_dev is None:
            if L.capturing:
                raise RuntimeError("Adam: take one eager step() (or pass capturable=True) before capturing, so that the "
                                   "device step counter exists when the capture starts")
            from . import functional as F
            self._t_dev = F.full([1], self.t)
        return self._t_dev

    def step_count(self):
        """The counter t that the next step() will use."""
        return float(self._t_dev.item()) if self._t_dev is not None else self.t

    def step(self):
        if self._t_dev is not None or L.capturing:
            import ctypes
            t_dev = self._device_counter()
            grads = [_flat_grad(p) for p in self.params]
            k = len(self.params)
            assert all(p.is_contiguous() for p in self.params)
            vp = ctypes.c_void_p * k
            L.call("endia_hip_adam_step_multi", k, L.i64_array([p.size() for p in self.params]),
                   vp(*[p.data_ptr() for p in self.params]), vp(*[g.data_ptr() for g in grads]),
                   vp(*[m.data_ptr() for m in self.m]), vp(*[v.data_ptr() for v in self.v]),
                   self.lr, self.beta1, self.beta2, self.eps, t_dev.data_ptr())
            for p in self.params:
                p.clear_args()
                p._buf.version += 1
            return
        for i in range(len(self.params)):
            self._update(i)
        self._updated = [False] * len(self.params)
        self.t += 1.0
