"""Checks at the benchmark's full sizes (4096 x 4096 operands, batch 4096) that need no CPU GEMM: streaming and
reduction kernels directly against numpy float64, Adam against its closed form after the first step, and the
whole wide-MLP backward pass against a directional finite difference of its own forward pass."""
import numpy as np
import pytest

from conftest import assert_close
from endia_amd import _lib as L

pytestmark = pytest.mark.gpu

N = 4096


def test_streaming_kernels_full_size(dev):
    rng = np.random.default_rng(100)
    x = rng.standard_normal((N, N)).astype(np.float32)
    g = rng.standard_normal((N, N)).astype(np.float32)
    dx_, dg = dev.put(x), dev.put(g)
    dy = dev.alloc(x.nbytes)
    x64, g64 = x.astype(np.float64), g.astype(np.float64)
    dev.call("endia_hip_unary_fwd", L.OP_TANH, N * N, dx_, dy, 0)
    assert_close(dev.get(dy, (N, N)), np.tanh(x64), tol=1e-6, what="tanh")
    dev.call("endia_hip_unary_vjp", L.OP_TANH, N * N, dx_, dg, dy, 0)
    assert_close(dev.get(dy, (N, N)), (1 - np.tanh(x64) ** 2) * g64, tol=1e-6, what="tanh vjp")
    # bias gradient: column sums of a 4096 x 4096 cotangent
    db = dev.alloc(4 * N)
    dev.call("endia_hip_reduce_add", 2, L.i64_array([N, N]), 1, dg, db, 1.0, 0)
    col = dev.get(db, (N,))
    scale = np.abs(g64).sum(axis=0)
    assert np.all(np.abs(col - g64.sum(axis=0)) <= 1e-6 * scale)
    # loss over 16.7 M elements: the reference's sequential fp32 sum would itself be off by ~1e-4 here;
    # the two-stage tree stays at fp32 round-off
    dl = dev.alloc(4)
    dev.call("endia_hip_mse_fwd_bwd", N * N, dx_, dg, dl, dy)
    assert_close(dev.get(dl, (1,)), [((x64 - g64) ** 2).mean()], tol=1e-6, what="mse")
    assert_close(dev.get(dy, (N, N)), 2 * (x64 - g64) / (N * N), tol=1e-6, what="mse grad")


def test_adam_and_sgd_full_size_closed_form(dev):
    rng = np.random.default_rng(101)
    p = rng.standard_normal((N, N)).astype(np.float32)
    g = (rng.standard_normal((N, N)) * 1e-2).astype(np.float32)
    dp, dg = dev.put(p), dev.put(g)
    dm, dv = dev.put(np.zeros_like(p)), dev.put(np.zeros_like(p))
    dev.call("endia_hip_adam_step", N * N, dp, dg, dm, dv, 1e-3, 0.9, 0.999, 1e-8, 1.0)
    # first step from zero moments: m_hat = g, v_hat = g^2, so the update is -lr * g / (|g| + eps)
    g64 = g.astype(np.float64)
    upd = dev.get(dp, (N, N)).astype(np.float64) - p
    ref = -1e-3 * g64 / (np.abs(g64) + 1e-8)
    assert np.abs(upd - ref).max() <= 2e-7  # half an ulp of parameters of size ~4, plus the update's own rounding
    # the reference's scalars are fp32 (adam.mojo:19-23): 1 - beta1 = 0.100000024, 1 - beta2 = 0.0009999871
    omb1 = float(np.float32(1) - np.float32(0.9))
    omb2 = float(np.float32(1) - np.float32(0.999))
    assert_close(dev.get(dm, (N, N)), omb1 * g64, tol=1e-6, what="m")
    assert_close(dev.get(dv, (N, N)), omb2 * g64 * g64, tol=1e-6, what="v")
    dev.call("endia_hip_memcpy_h2d", dp, p.ctypes.data, p.nbytes)
    dev.call("endia_hip_sgd_step", N * N, dp, dg, 0.5)
    np.testing.assert_array_equal(dev.get(dp, (N, N)), p - np.float32(0.5) * g)


def test_wide_mlp_backward_matches_directional_derivative():
    """The wide benchmark configuration (batch 4096, 4096-wide layers, tanh, MSE; 4 of the 8 layers to keep the
    test short). <grad, v> from one backward pass must equal the central difference of the loss along v."""
    import endia_amd as nd
    rng = np.random.default_rng(102)
    layers = 4
    Ws = [(rng.standard_normal((N, N)) / 64).astype(np.float32) for _ in range(layers)]
    bs = [(rng.standard_normal(N) / 64).astype(np.float32) for _ in range(layers)]
    vW = [rng.standard_normal((N, N)).astype(np.float32) for _ in range(layers)]
    vb = [rng.standard_normal(N).astype(np.float32) for _ in range(layers)]
    x = nd.array(rng.standard_normal((N, N)).astype(np.float32))
    y = nd.array(rng.standard_normal((N, N)).astype(np.float32))

    def loss_at(eps, want_grad=False):
        mlp = nd.nn.MLP([N] * (layers + 1), compute_backward=want_grad, activation="tanh", fused=True)
        for i in range(layers):
            mlp.weights[i] = nd.array(Ws[i] + np.float32(eps) * vW[i], requires_grad=want_grad)
            mlp.biases[i] = nd.array(bs[i] + np.float32(eps) * vb[i], requires_grad=want_grad)
        loss = nd.mse(mlp.forward(x), y)
        if not want_grad:
            return float(loss.item())
        loss.backward()
        dot = 0.0
        for i in range(layers):
            dot += float(np.vdot(mlp.weights[i].grad().to_numpy().astype(np.float64), vW[i]))
            dot += float(np.vdot(mlp.biases[i].grad().to_numpy().astype(np.float64).reshape(-1), vb[i]))
        return float(loss.item()), dot

    l0, analytic = loss_at(0.0, True)
    eps = 2e-4
    numeric = (loss_at(eps) - loss_at(-eps)) / (2 * eps)
    # fp32 forward passes limit the difference quotient to about 1e-7 * loss / eps relative to the derivative
    assert abs(numeric - analytic) <= 2e-2 * abs(analytic) + 1e-3, (l0, analytic, numeric)


def test_size_limits_are_reported_not_launched(dev):
    lib = L.lib()
    p = dev.alloc(64)
    big = 1 << 31
    assert lib.endia_hip_sgemm(0, 0, big, 4, 4, p, 4, p, 4, p, 4, 1, 0, 0, 0, 0, L.OP_IDENTITY, None, None, None) == L.ERR_INVALID
    assert b"too large" in lib.endia_hip_last_error()
    assert lib.endia_hip_sgemm(0, 0, 4, 4, 4, p, 4, p, 4, p, 4, 70000, 16, 16, 16, 0, L.OP_IDENTITY, None, None, None) == L.ERR_INVALID
    import ctypes
    d = L.Conv2dDesc(1 << 20, 64, 56, 56, 128, 3, 3, 1, 1, 1, 1, 1, 1, 1)
    P, Q = ctypes.c_int64(), ctypes.c_int64()
    assert lib.endia_hip_conv2d_out_shape(ctypes.byref(d), ctypes.byref(P), ctypes.byref(Q)) == L.ERR_UNSUPPORTED
    d = L.Conv2dDesc(1, 1, 2, 2, 1, 5, 5, 1, 1, 0, 0, 1, 1, 1)
    assert lib.endia_hip_conv2d_out_shape(ctypes.byref(d), ctypes.byref(P), ctypes.byref(Q)) == L.ERR_INVALID
    assert lib.endia_hip_reduce_add(9, L.i64_array([1] * 9), 0, p, p, ctypes.c_float(1.0), 0) == L.ERR_INVALID
    assert lib.endia_hip_binary(99, 1, L.i64_array([4]), L.i64_array([1]), L.i64_array([1]), p, p, p, 0) == L.ERR_INVALID


def test_empty_inputs_are_noops(dev):
    """Zero-sized tensors: every entry point returns success without touching memory."""
    z = L.i64_array([0, 8])
    dev.call("endia_hip_unary_fwd", L.OP_TANH, 0, None, None, 0)
    dev.call("endia_hip_unary_vjp", L.OP_TANH, 0, None, None, None, 0)
    dev.call("endia_hip_binary", L.BIN_ADD, 2, z, L.i64_array([8, 1]), L.i64_array([8, 1]), None, None, None, 0)
    dev.call("endia_hip_axpby", 0, 1.0, None, 0.0, None, None)
    dev.call("endia_hip_fill", None, 0, 1.0)
    dev.call("endia_hip_strided_copy", 2, z, L.i64_array([8, 1]), 0, None, None, 0)
    dev.call("endia_hip_sgd_step", 0, None, None, 0.1)
    dev.call("endia_hip_adam_step", 0, None, None, None, None, 1e-3, 0.9, 0.999, 1e-8, 1.0)
    dev.call("endia_hip_sgemm", 0, 0, 0, 8, 8, None, 8, None, 8, None, 8, 1, 0, 0, 0, 0, L.OP_IDENTITY, None, None, None)
    dev.call("endia_hip_cgemm", 0, 0, 0, 0, 8, 0, 8, None, 8, None, 8, None, 8, 1, 0, 0, 0, L.CGEMM_4M, 0)
    import endia_amd as nd
    e = nd.zeros([0, 8], requires_grad=True)
    assert nd.tanh(e).shape() == [0, 8]
    assert nd.reduce_add(e, [0]).to_numpy().tolist() == [[0.0] * 8]
    assert (e @ nd.zeros([8, 3])).shape() == [0, 3]
