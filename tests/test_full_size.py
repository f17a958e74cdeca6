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


def test_streaming_kernels_past_2_31_elements(dev):
    """2^31 + 4096 elements (8.6 GB per array): element indices no longer fit 32 bits. Constant inputs, so the expected
    values are known without a host copy of the arrays; the head and the tail of every result are read back."""
    n = (1 << 31) + 4096
    x, y = dev.alloc(4 * n), dev.alloc(4 * n)

    def ends(p):
        return np.concatenate([dev.get(p, (512,)), dev.get(p + 4 * (n - 512), (512,))])

    dev.call("endia_hip_fill", x, n, 0.5)
    dev.call("endia_hip_unary_fwd", L.OP_SQUARE, n, x, y, 0)
    np.testing.assert_array_equal(ends(y), np.full(1024, 0.25, np.float32))
    dev.call("endia_hip_axpby", n, 2.0, y, 1.0, x, y)            # y = 2 * 0.25 + 0.5
    np.testing.assert_array_equal(ends(y), np.ones(1024, np.float32))
    dev.call("endia_hip_sgd_step", n, x, y, 0.5)                 # x = 0.5 - 0.5 * 1
    np.testing.assert_array_equal(ends(x), np.zeros(1024, np.float32))
    one = L.i64_array([1])
    dev.call("endia_hip_binary", L.BIN_ADD, 1, L.i64_array([n]), one, one, x, y, x, 0)   # x = 0 + 1
    np.testing.assert_array_equal(ends(x), np.ones(1024, np.float32))
    total = dev.alloc(4)
    dev.call("endia_hip_reduce_add", 1, L.i64_array([n]), 1, x, total, 1.0, 0)
    assert abs(float(dev.get(total, (1,))[0]) - n) <= 1e-6 * n


@pytest.mark.parametrize("K", [8, 2])
def test_gemm_output_past_2_31_elements(dev, K):
    """C = A B with 65536 x 40000 outputs (2.6e9 elements, 10.5 GB): output offsets need 64 bits. K = 8 takes the MFMA
    kernel, K = 2 the one-thread-per-output kernel; rows from the top, the middle and the end of C against float64."""
    M, N = 65536, 40000
    rng = np.random.default_rng(K)
    A = rng.standard_normal((M, K)).astype(np.float32)
    B = rng.standard_normal((K, N)).astype(np.float32)
    dA, dB, dC = dev.put(A), dev.put(B), dev.alloc(4 * M * N)
    dev.call("endia_hip_sgemm", 0, 0, M, N, K, dA, K, dB, N, dC, N, 1, 0, 0, 0, L.EPI_NONE, L.OP_IDENTITY, None, None, None)
    for r in (0, 1, 32767, 53688, M - 2, M - 1):   # row 53688 starts past element 2^31
        got = dev.get(dC + 4 * r * N, (N,))
        assert_close(got, A[r].astype(np.float64) @ B.astype(np.float64), tol=1e-6, what="row %d" % r)


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


def test_fused_program_full_size(dev):
    """tanh(a * b + bias) and both of its gradients over 4096 x 4096 elements against numpy float64."""
    import ctypes
    rng = np.random.default_rng(102)
    a = rng.standard_normal((N, N)).astype(np.float32)
    b = rng.standard_normal((N, N)).astype(np.float32)
    g = rng.standard_normal((N, N)).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    da, db_, dg, dbias = dev.put(a), dev.put(b), dev.put(g), dev.put(bias)
    dy, d1, d2 = dev.alloc(a.nbytes), dev.alloc(a.nbytes), dev.alloc(a.nbytes)
    I, S, M = L.EW_SRC_INPUT, L.EW_SRC_SLOT, L.EW_SRC_IMM

    def run(ins, modes, outs, steps):
        pin = (ctypes.c_void_p * len(ins))(*ins)
        pm = (ctypes.c_int32 * len(ins))(*modes)
        po = (ctypes.c_void_p * len(outs))(*outs)
        arr = (L.EwStep * len(steps))(*[L.EwStep(*s) for s in steps])
        dev.call("endia_hip_ew_program", N, N, len(ins), pin, pm, len(outs), po, len(steps), arr)

    run([da, db_, dbias], [L.EW_FULL, L.EW_FULL, L.EW_ROW_VECTOR], [dy],
        [(L.EW_LOAD, 0, I, 0, 0.0), (L.EW_BINARY, L.BIN_MUL, I, 1, 0.0), (L.EW_BINARY, L.BIN_ADD, I, 2, 0.0),
         (L.EW_UNARY, L.OP_TANH, 0, 0, 0.0), (L.EW_STORE, 0, 0, 0, 0.0)])
    z = a.astype(np.float64) * b + bias
    y64 = np.tanh(z)
    assert_close(dev.get(dy, (N, N)), y64, tol=1e-6, what="tanh(a*b+bias)")
    # gradients from the stored output: t = (1 - y^2) * g; da = t * b; db = t * a
    run([da, db_, dy, dg], [L.EW_FULL] * 4, [d1, d2],
        [(L.EW_LOAD, 0, I, 2, 0.0), (L.EW_UNARY, L.OP_SQUARE, 0, 0, 0.0), (L.EW_RBINARY, L.BIN_SUB, M, 0, 1.0),
         (L.EW_BINARY, L.BIN_MUL, I, 3, 0.0), (L.EW_SAVE, 0, 0, 0, 0.0), (L.EW_BINARY, L.BIN_MUL, I, 1, 0.0),
         (L.EW_STORE, 0, 0, 0, 0.0), (L.EW_LOAD, 0, S, 0, 0.0), (L.EW_BINARY, L.BIN_MUL, I, 0, 0.0),
         (L.EW_STORE, 0, 0, 1, 0.0)])
    t = (1 - y64 * y64) * g
    assert_close(dev.get(d1, (N, N)), t * b, tol=1e-5, what="d/da")
    assert_close(dev.get(d2, (N, N)), t * a, tol=1e-5, what="d/db")


def test_pooling_full_size_properties(dev):
    """2x2 stride-2 pooling of a [64,128,56,56] array: forward against numpy, and size-independent properties of
    the backward: average pooling is linear with <pool(x), g> = <x, pool_bwd(g)>; max pooling hands every output
    gradient to exactly one input, so the sums agree and dx is zero wherever x is not its window's maximum."""
    import ctypes
    rng = np.random.default_rng(103)
    shape = (64, 128, 56, 56)
    x = rng.standard_normal(shape).astype(np.float32)
    g = rng.standard_normal((64, 128, 28, 28)).astype(np.float32)
    d = L.PoolDesc()
    d.N, d.C, d.D, d.H, d.W = 64, 128, 1, 56, 56
    d.kernel[:], d.stride[:], d.padding[:], d.dilation[:] = [1, 2, 2], [1, 2, 2], [0, 0, 0], [1, 1, 1]
    dx_, dg = dev.put(x), dev.put(g)
    dy, darg, ddx = dev.alloc(g.nbytes), dev.alloc(g.nbytes), dev.alloc(x.nbytes)
    win = x.reshape(64, 128, 28, 2, 28, 2)
    g64_ = g.astype(np.float64)
    for mode, want in ((L.POOL_MAX, win.max(axis=(3, 5))), (L.POOL_AVG, win.astype(np.float64).mean(axis=(3, 5)))):
        dev.call("endia_hip_pool_fwd", ctypes.byref(d), mode, dx_, dy, darg if mode == L.POOL_MAX else None)
        y = dev.get(dy, g.shape)
        assert_close(y, want, tol=1e-6, what="pool forward")
        dev.call("endia_hip_pool_bwd", ctypes.byref(d), mode, dg, darg if mode == L.POOL_MAX else None, ddx)
        dxv = dev.get(ddx, shape).astype(np.float64)
        if mode == L.POOL_AVG:
            lhs, rhs = np.vdot(y.astype(np.float64), g), np.vdot(x.astype(np.float64), dxv)
            assert abs(lhs - rhs) <= 1e-6 * np.abs(y.astype(np.float64) * g).sum()
            assert_close(dxv, np.repeat(np.repeat(g.astype(np.float64) / 4, 2, axis=2), 2, axis=3), tol=1e-6, what="avg grad")
        else:
            assert abs(dxv.sum() - g.astype(np.float64).sum()) <= 1e-6 * np.abs(g).sum()
            is_max = x == np.repeat(np.repeat(want, 2, axis=2), 2, axis=3)
            assert np.all(dxv[~is_max] == 0)
            np.testing.assert_array_equal(dxv.reshape(64, 128, 28, 2, 28, 2).sum(axis=(3, 5)), g64_)


def test_conv3d_full_size_properties(dev):
    """conv3d at the benchmark shape (x [8,32,16,56,56], w [64,32,3,3,3], pad 1): adjoint identities
    <conv(x,w), g> = <x, dX> = <w, dW>, db = sum of g, and a float64 probe of scattered output elements."""
    import ctypes
    rng = np.random.default_rng(104)
    xs, ws = (8, 32, 16, 56, 56), (64, 32, 3, 3, 3)
    x = rng.standard_normal(xs).astype(np.float32)
    w = (rng.standard_normal(ws) * 0.05).astype(np.float32)
    g = rng.standard_normal((8, 64, 16, 56, 56)).astype(np.float32)
    d = L.Conv3dDesc()
    d.N, d.C, d.D, d.H, d.W, d.K, d.T, d.R, d.S = 8, 32, 16, 56, 56, 64, 3, 3, 3
    d.stride[:], d.padding[:], d.dilation[:], d.groups = [1, 1, 1], [1, 1, 1], [1, 1, 1], 1
    dx_, dw_, dg = dev.put(x), dev.put(w), dev.put(g)
    dy, ddx, ddw, ddb = dev.alloc(g.nbytes), dev.alloc(x.nbytes), dev.alloc(w.nbytes), dev.alloc(4 * 64)
    dev.call("endia_hip_conv3d_fwd", ctypes.byref(d), dx_, dw_, None, dy, L.OP_IDENTITY)
    dev.call("endia_hip_conv3d_bwd_data", ctypes.byref(d), dg, dw_, ddx)
    dev.call("endia_hip_conv3d_bwd_weight", ctypes.byref(d), dx_, dg, ddw)
    dev.call("endia_hip_conv3d_bwd_bias", ctypes.byref(d), dg, ddb)
    y = dev.get(dy, g.shape)
    g64 = g.astype(np.float64)
    lhs = np.vdot(y.astype(np.float64), g64)
    tol = 1e-5 * np.abs(y.astype(np.float64) * g64).sum()
    assert abs(lhs - np.vdot(x.astype(np.float64), dev.get(ddx, xs))) <= tol
    assert abs(lhs - np.vdot(w.astype(np.float64), dev.get(ddw, ws))) <= tol
    assert_close(dev.get(ddb, (64,)), g64.sum(axis=(0, 2, 3, 4)), tol=1e-5, what="db")
    xp = np.pad(x.astype(np.float64), ((0, 0), (0, 0), (1, 1), (1, 1), (1, 1)))
    for n, k, z, r, c in [(0, 0, 0, 0, 0), (7, 63, 15, 55, 55), (3, 17, 8, 30, 1), (5, 40, 1, 0, 55), (2, 9, 15, 27, 28)]:
        want = (xp[n, :, z:z + 3, r:r + 3, c:c + 3] * w[k].astype(np.float64)).sum()
        assert abs(y[n, k, z, r, c] - want) <= 1e-4 * max(1.0, abs(want))


def test_hvp_full_size_symmetry_and_linearity():
    """The second-order benchmark configuration (batch 1024, 4 layers 2048 wide, sin, loss sum(out^2)): the
    Hessian is symmetric, so <u, H v> = <v, H u>, and H (2 v) = 2 H v. Both hold for any size, so they check
    the double-backward path at its real shapes without a CPU reference of that size."""
    import endia_amd as nd
    rng = np.random.default_rng(103)
    B, Wd, Ly = 1024, 2048, 4
    mlp = nd.nn.MLP([Wd] * (Ly + 1), compute_backward=True, activation="sin", fused=True)
    for i in range(Ly):
        mlp.weights[i] = nd.array((rng.standard_normal((Wd, Wd)) / np.sqrt(Wd)).astype(np.float32), requires_grad=True)
        mlp.biases[i] = nd.array((rng.standard_normal(Wd) / np.sqrt(Wd)).astype(np.float32), requires_grad=True)
    x = nd.array(rng.standard_normal((B, Wd)).astype(np.float32))
    shapes = [p.shape() for p in mlp.params()]
    u = [rng.standard_normal(s).astype(np.float32) for s in shapes]
    v = [rng.standard_normal(s).astype(np.float32) for s in shapes]

    def hvp(vec):
        out = mlp.forward(x)
        loss = nd.sum(out * out)
        loss.backward(create_graph=True)
        s = None
        for p, w in zip(mlp.params(), vec):
            term = nd.sum(p.grad() * nd.array(w))
            s = term if s is None else s + term
        hv = nd.grad(outs=s, inputs=mlp.params())
        loss.zero_grad()
        return [h.to_numpy().astype(np.float64).reshape(-1) for h in hv]

    def dot(a, b):
        return float(sum(np.dot(p, q.astype(np.float64).reshape(-1)) for p, q in zip(a, b)))

    Hv, Hu = hvp(v), hvp(u)
    uHv, vHu = dot(Hv, u), dot(Hu, v)
    assert abs(uHv - vHu) <= 1e-3 * max(abs(uHv), abs(vHu)), (uHv, vHu)
    H2v = hvp([2 * w for w in v])
    for a, b in zip(H2v, Hv):
        assert_close(a, 2 * b, tol=1e-5, what="H (2 v) = 2 H v")
    assert all(np.isfinite(h).all() for h in Hv) and dot(Hv, v) != 0.0


@pytest.mark.parametrize("algo", ["4m", "3m"])
def test_complex_mlp_full_size_directional_derivative(algo):
    """The complex benchmark configuration (batch 2048, 4 complex layers 2048 wide, loss sum |out|^2). With the
    Wirtinger rule the gradient g satisfies dL(W + eps V)/d eps = Re <g, V>, whatever the size; checked with a
    central difference for both GEMM algorithms. (The reference's rule without conjugation is not the
    gradient of a real loss; it is compared with the oracle's composition of the same products at small sizes.)"""
    import endia_amd as nd
    rng = np.random.default_rng(104)
    n, Ly = 2048, 4
    nd.set_complex_matmul_algorithm(algo)
    try:
        Wn = [((rng.standard_normal((n, n)) + 1j * rng.standard_normal((n, n))) / np.sqrt(2 * n)).astype(np.complex64)
              for _ in range(Ly)]
        Vn = [(rng.standard_normal((n, n)) + 1j * rng.standard_normal((n, n))).astype(np.complex64) for _ in range(Ly)]
        z = nd.array((rng.standard_normal((n, n)) + 1j * rng.standard_normal((n, n))).astype(np.complex64))

        def loss_at(eps, want_grad):
            Ws = [nd.array(W + np.complex64(eps) * V, requires_grad=want_grad) for W, V in zip(Wn, Vn)]
            h = z
            for W in Ws:
                h = nd.matmul(h, W, vjp_rule="wirtinger")
            loss = nd.sum(nd.square(nd.abs(h)))
            if not want_grad:
                return float(loss.item())
            loss.backward()
            return float(loss.item()), sum(float(np.vdot(W.grad().to_numpy().astype(np.complex128), V).real)
                                           for W, V in zip(Ws, Vn))

        l0, analytic = loss_at(0.0, True)
        eps = 1e-4
        numeric = (loss_at(eps, False) - loss_at(-eps, False)) / (2 * eps)
        assert abs(numeric - analytic) <= 2e-2 * abs(analytic), (algo, l0, analytic, numeric)
    finally:
        nd.set_complex_matmul_algorithm("4m")
