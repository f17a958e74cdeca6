"""endia_amd: Endia's reverse-mode training-step path on one AMD MI355X (gfx950).

The public names mirror the reference's `endia` package (endia/__init__.mojo,
endia/functional/__init__.mojo): `Array` / `Tensor` / `ndarray`, the functional ops, `backward` /
`grad` / `jacobian` / `hessian` / `value_and_grad`, `nn.MLP`, `optim.SGD` / `optim.Adam`. All
arithmetic runs in libendia_hip.so (hand-written HIP kernels behind the C ABI of
include/endia_hip.h); importing this package without that library raises.
"""
from . import _lib

_lib.lib()  # fail loudly when the HIP library has not been built

from ._array import Array, Tensor, ndarray  # noqa: E402
from .functional import (  # noqa: E402,F401
    abs, acos, add, arange, array, array_slice, as_strided, as_strided_inv, asin, atan, avg_pool1d, avg_pool2d, avg_pool3d, complex, concat, conj, contiguous, conv1d,
    conv2d, conv3d, cos, cosh, detach, div, equal, exp,
    expand, eye, full, greater, greater_equal, imag, less, less_equal, linear, log, matmul, mlp_forward, mlp_mse_loss, max_pool1d, max_pool2d, max_pool3d, mean, mse, mul, neg,
    not_equal, ones, pad, permute, pow, pow_to, prod, rand_he_normal, randn, randn_complex, randu, real, reciprocal, reduce_add,
    reduce_argmax, reduce_argmin, reduce_max, reduce_min, reduce_mul,
    relu, reshape, seed, set_complex_matmul_algorithm, set_complex_vjp_rule, sigmoid, sign, sin, sinh, sqrt, square, squeeze, std, sub, sum, tan,
    tanh, unsqueeze, variance, zeros,
)
from .functional import (  # noqa: E402,F401  the rest of the initialisers (endia/functional/init_ops/init_ops.mojo)
    eye_like, fill_, fill_like, linspace, ones_, ones_like, rand_he_normal_, rand_he_normal_like, rand_he_uniform,
    rand_he_uniform_, rand_he_uniform_like, rand_lecun_normal, rand_lecun_normal_, rand_lecun_normal_like,
    rand_lecun_uniform, rand_lecun_uniform_, rand_lecun_uniform_like, rand_xavier_normal, rand_xavier_normal_,
    rand_xavier_normal_like, rand_xavier_uniform, rand_xavier_uniform_, rand_xavier_uniform_like, randn_, randn_like,
    randu_, randu_like, zeros_, zeros_like,
)
from .autograd.functional import backward, grad, hessian, jacobian, value_and_grad  # noqa: E402,F401
from . import autograd, fusion, graph, nn, optim, utils  # noqa: E402,F401
from .fusion import fuse  # noqa: E402,F401
from .graph import capture, jit  # noqa: E402,F401


def synchronize():
    """Block until every kernel enqueued so far has finished."""
    _lib.call("endia_hip_sync")
