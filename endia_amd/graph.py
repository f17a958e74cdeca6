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
