"""Pins the CPU oracle (oracle/endia_ref.c) without a GPU.

Every function of the oracle is checked against something it did not produce: the PyTorch-float64
golden fixtures (the reference's own test oracle), the three known answers in the reference's docs,
numpy float64 closed forms, and algebraic invariants. Tolerance: 1e-4 relative, the reference's test
tolerance (endia/utils/array_conversions.mojo:63-64); most results agree to ~1e-6.
"""
import numpy as np
import pytest

from conftest import assert_close, mean_rel
from oracle import endia_ref as R


def test_matmul_golden(golden):
    g = golden("matmul")
    assert_close(R.matmul(g["a"], g["b"]), g["out"], what="matmul fwd")
    # gradients of sum(a @ b): grad = ones; dA = g @ B.T, dB = A.T @ g summed over the broadcast batch axis
    ones = np.ones((2, 30, 50), np.float32)
    da = R.matmul(ones, g["b"].T)
    db = R.reduce_add(R.matmul(np.swapaxes(g["a"], -1, -2), ones), [0])
    assert_close(da, g["da"], what="matmul dA")
    assert_close(db, g["db"], what="matmul dB")
    assert mean_rel(R.matmul(g["a"], g["b"]), g["out"]) <= 1e-4
    # square operands through transposed VIEWS: the documented semantics dX = g W^T, dW = X^T g
    assert_close(R.matmul(g["sg"], g["sb"].T), g["dsa"], what="square dA")
    assert_close(R.matmul(g["sa"].T, g["sg"]), g["dsb"], what="square dB")


def test_matmul_complex_golden(golden):
    g = golden("matmul")
    assert_close(R.matmul(g["ca"], g["cb"]), g["cout"], what="complex matmul fwd")


def test_matmul_brute_force_tiny():
    rng = np.random.default_rng(0)
    for M, N, K in [(1, 1, 1), (3, 2, 17), (5, 7, 33), (2, 3, 16)]:
        a = rng.standard_normal((M, K)).astype(np.float32)
        b = rng.standard_normal((K, N)).astype(np.float32)
        ref = np.zeros((M, N))
        for m in range(M):
            for n in range(N):
                for k in range(K):
                    ref[m, n] += float(a[m, k]) * float(b[k, n])
        assert_close(R.matmul(a, b), ref, tol=1e-6, what="brute force %s" % ((M, N, K),))


def test_matmul_adjoint_identity():
    # <A B, G> = <A, G B^T> = <B, A^T G>
    rng = np.random.default_rng(1)
    A, B, G = (rng.standard_normal(s).astype(np.float32) for s in [(9, 20), (20, 11), (9, 11)])
    lhs = np.vdot(R.matmul(A, B).astype(np.float64), G)
    assert abs(lhs - np.vdot(A.astype(np.float64), R.matmul(G, B.T))) < 1e-3 * abs(lhs)
    assert abs(lhs - np.vdot(B.astype(np.float64), R.matmul(A.T, G))) < 1e-3 * abs(lhs)


@pytest.mark.parametrize("op", ["relu", "tanh", "sin", "cos", "neg", "square", "sqrt", "abs"])
def test_unary_golden(golden, op):
    g = golden("unary")
    x = g["xp"] if op == "sqrt" else g["x"]
    assert_close(R.unary(op, x), g[op], what=op)
    assert_close(R.unary_vjp(op, x, np.ones_like(x)), g["d" + op], what="d" + op)


MORE_UNARY = ["exp", "log", "sigmoid", "sinh", "cosh", "tan", "asin", "acos", "atan", "reciprocal"]


def _more_src(g, op):
    return g["xp"] if op in ("log", "reciprocal", "sign") else (g["xu"] if op in ("tan", "asin", "acos") else g["x"])


@pytest.mark.parametrize("op", MORE_UNARY)
def test_unary_more_golden(golden, op):
    g = golden("unary_more")
    x = _more_src(g, op)
    assert_close(R.unary(op, x), g[op], what=op)
    assert_close(R.unary_vjp(op, x, np.ones_like(x)), g["d" + op], what="d" + op)


def test_unary_more_special_values(golden):
    g = golden("unary_more")
    assert_close(R.unary("sign", g["xp"]), g["sign"], what="sign")
    assert_close(R.unary("sign", -g["xp"]), -g["sign"], what="sign of negatives")
    assert np.isnan(R.unary("sign", np.zeros(1, np.float32))[0])        # x / |x| at 0 (sign_op.mojo:78-79)
    # log is the log of the modulus (log_op.mojo:111-113), so a negative input gives log|x|, not NaN
    np.testing.assert_allclose(R.unary("log", np.array([-np.e], np.float32)), [1.0], rtol=1e-6)
    # sign hands the gradient on unchanged (sign_op.mojo:58)
    gr = np.arange(4, dtype=np.float32)
    np.testing.assert_array_equal(R.unary_vjp("sign", np.ones(4, np.float32), gr), gr)


@pytest.mark.parametrize("op", ["sin", "cos", "tanh", "exp", "log", "sinh", "cosh", "sqrt", "reciprocal", "sign"])
def test_unary_complex_golden(golden, op):
    g = golden("unary_more")
    assert_close(R.unary_complex(op, g["z"]), g["c" + op], what="complex " + op)


def test_pow_and_comparisons_golden(golden):
    g = golden("binary_more")
    y = R.binary("pow", g["a"], g["b"])
    assert_close(y, g["pow"], what="pow")
    # VJP as the reference composes it: g*b*(out/a), g*out*log(a), broadcast axis summed (pow_op.mojo:109-115)
    gy = np.ones_like(y)
    da = R.binary("mul", R.binary("mul", gy, g["b"]), R.binary("div", y, g["a"]))
    db = R.reduce_add(R.binary("mul", R.binary("mul", gy, y), R.unary("log", g["a"])), [0])
    assert_close(da, g["dpow_a"], what="dpow/da")
    assert_close(db, g["dpow_b"], what="dpow/db")
    assert_close(R.binary("pow", g["an"], g["ei"]), g["pow_neg"], what="negative base, integer exponent")
    for name in ("greater", "greater_equal", "less", "less_equal", "equal", "not_equal"):
        np.testing.assert_array_equal(R.binary(name, g["ca"], g["cb"]), g[name], err_msg=name)


def test_unary_special_values():
    # strict > in the relu mask (greater_op.mojo:57-59); sqrt of a negative is 0, not NaN (sqrt_op.mojo:111-114)
    x = np.array([0.0, -0.0, 1e-30, -1.0], np.float32)
    np.testing.assert_array_equal(R.unary_vjp("relu", x, np.ones(4, np.float32)), [0, 0, 1, 0])
    np.testing.assert_array_equal(R.unary("sqrt", np.array([-4.0, 4.0], np.float32)), [0, 2])
    # the reference's tanh formula overflows to NaN for large |x| (sinh(2x)/(cosh(2x)+1))
    assert np.isnan(R.unary("tanh", np.array([60.0], np.float32))[0])


@pytest.mark.parametrize("op", ["add", "sub", "mul", "div"])
def test_binary_golden(golden, op):
    g = golden("binary")
    b = g["b2"] if op == "div" else g["b"]
    assert_close(R.binary(op, g["a"], b), g[op], what=op)
    # gradients of sum(sin(a op b)) through the reference's VJP rules
    y = R.binary(op, g["a"], b)
    gy = np.cos(y.astype(np.float64)).astype(np.float32)
    if op == "add":
        da, db = gy, gy
    elif op == "sub":
        da, db = gy, R.unary("neg", gy)
    elif op == "mul":
        da, db = R.binary("mul", b, gy), R.binary("mul", g["a"], gy)
    else:
        da = R.binary("div", gy, b)
        db = R.binary("div", R.binary("mul", R.unary("neg", gy), g["a"]), R.binary("mul", b, b))
    assert_close(da, g[op + "_da"], what=op + " dA")
    assert_close(R.reduce_add(db, [0]), g[op + "_db"], what=op + " dB")  # Expand.vjp: sum over the broadcast axis


def test_binary_complex_golden(golden):
    g = golden("binary")
    assert_close(R.binary("mul", g["ca"], g["cb"]), g["cmul"], what="complex mul")
    assert_close(R.binary("div", g["ca"], g["cb"]), g["cdiv"], what="complex div")
    assert_close(R.binary("add", g["ca"], g["cb"]), g["cadd"], what="complex add")


def test_reduce_golden(golden):
    g = golden("reduce")
    assert_close(R.reduce_add(g["x"], [0, 2]), g["sum02"], what="reduce_add (0,2)")
    assert_close(R.reduce_add(g["x"], [0, 1, 2]), g["total"], what="sum")
    assert_close(R.reduce_add(g["x"], [1]) / np.float32(30), g["mean1"], what="mean")
    # the broadcast-gradient rule pinned by test_expand_op.mojo:35-52
    assert_close(R.reduce_add(g["x"], [0, 1]), g["dexpand"], what="expand vjp")
    # rank-1 full reduction takes the SIMD path (reduce_add_op.mojo:160-190)
    v = g["x"].reshape(-1)[:1003]
    assert_close(R.reduce_add(v, [0]), [v.astype(np.float64).sum()], what="rank-1 sum")


def test_other_reductions_golden_and_brute_force(golden):
    """max / min / argmax / argmin / product / variance / std of the oracle against torch float64 (the reference's own
    check: test_reduce_max_op.mojo:18-34 and its siblings, test_std_op.mojo:18-58, test_variance_op.mojo:18-59), against
    plain loops on a small array, and on the cases the loops' starting values decide."""
    g = golden("reduce_more")
    x = g["x"]
    np.testing.assert_array_equal(R.reduce_op("max", x, [1]).reshape(2, 40), g["max1"])
    np.testing.assert_array_equal(R.reduce_op("min", x, [1]).reshape(2, 40), g["min1"])
    np.testing.assert_array_equal(R.reduce_op("argmax", x, [1]).reshape(2, 40), g["argmax1"])
    np.testing.assert_array_equal(R.reduce_op("argmin", x, [1]).reshape(2, 40), g["argmin1"])
    np.testing.assert_array_equal(R.reduce_op("argmax", x, [2]).reshape(2, 30), g["argmax2"])
    np.testing.assert_array_equal(R.reduce_op("max", x, [0, 2]).reshape(30), g["max02"])
    np.testing.assert_array_equal(R.reduce_op("min", x, [1, 2]).reshape(2), g["min12"])
    assert_close(R.reduce_op("mul", x, [1]).reshape(2, 40), g["prod1"], what="product over axis 1")
    assert_close(R.reduce_op("mul", x[0, :8, :5], [0, 1]).reshape(1), g["prod_all"], what="product of everything")
    assert_close(R.variance(x, [1]), g["var1"], what="variance")
    assert_close(R.std(x, [1]), g["std1"], what="std")
    assert_close(R.std(x, [1], keepdims=True), g["std1_keep"], what="std, kept axis")
    assert_close(R.variance(x, [0, 2], unbiased=False), g["var02_biased"], what="biased variance over two axes")
    # plain loops
    small = x[1, :4, :6]
    for j in range(6):
        col = [float(v) for v in small[:, j]]
        assert R.reduce_op("max", small, [0])[0, j] == max(col)
        assert R.reduce_op("argmin", small, [0])[0, j] == col.index(min(col))
        p = np.float32(1)
        for v in small[:, j]:
            p = np.float32(p * v)
        assert R.reduce_op("mul", small, [0])[0, j] == p
    # ties go to the first position; an axis holding only the starting value leaves -1; a size-1 axis gives 0
    np.testing.assert_array_equal(R.reduce_op("argmax", np.array([[1, 3, 3], [2, 2, 1]], np.float32), [1]).reshape(-1), [1, 0])
    np.testing.assert_array_equal(R.reduce_op("argmax", np.full((2, 3), -np.inf, np.float32), [1]).reshape(-1), [-1, -1])
    np.testing.assert_array_equal(R.reduce_op("argmin", np.ones((3, 1), np.float32), [1]).reshape(-1), [0, 0, 0])


def test_mse_golden(golden):
    g = golden("mse")
    loss, dpred = R.mse(g["pred"], g["target"])
    assert_close([loss], g["loss"], what="mse")
    assert_close(dpred, g["dpred"], what="mse grad")


@pytest.mark.parametrize("tag,st,pd,dl", [("s2p1", (2, 2), (1, 1), (1, 1)), ("s1p1", (1, 1), (1, 1), (1, 1)),
                                         ("s2p2d2", (2, 1), (2, 0), (2, 1))])
def test_conv2d_golden(golden, tag, st, pd, dl):
    g = golden("conv2d")
    y = R.conv2d(g["x"], g["w"], g["b"], st, pd, dl)
    assert_close(y, g[tag + "_y"], what="conv2d fwd " + tag)
    dx, dw, db = R.conv2d_bwd(g["x"], g["w"], g[tag + "_g"], st, pd, dl)
    assert_close(dx, g[tag + "_dx"], what="conv2d dx " + tag)
    assert_close(dw, g[tag + "_dw"], what="conv2d dw " + tag)
    assert_close(db, g[tag + "_db"], what="conv2d db " + tag)


def test_conv2d_adjoint_identity():
    # <conv(x, w), dy> = <x, dX> = <w, dW>; the reference has no conv2d VJP, this is what defines ours
    rng = np.random.default_rng(2)
    x = rng.standard_normal((2, 3, 7, 6)).astype(np.float32)
    w = rng.standard_normal((5, 3, 3, 3)).astype(np.float32)
    y = R.conv2d(x, w, None, (2, 1), (1, 2), (1, 2))
    dy = rng.standard_normal(y.shape).astype(np.float32)
    dx, dw, db = R.conv2d_bwd(x, w, dy, (2, 1), (1, 2), (1, 2))
    lhs = np.vdot(y.astype(np.float64), dy)
    assert abs(lhs - np.vdot(x.astype(np.float64), dx)) < 1e-4 * abs(lhs) + 1e-4
    assert abs(lhs - np.vdot(w.astype(np.float64), dw)) < 1e-4 * abs(lhs) + 1e-4
    assert_close(db, dy.astype(np.float64).sum(axis=(0, 2, 3)), what="db")


def test_optimizers_golden(golden):
    g = golden("optim")
    p = g["p0"]
    for i in range(3):
        p = R.sgd(p, g["g%d" % i], 1e-3)
        assert_close(p, g["sgd_p%d" % (i + 1)], tol=1e-6, what="sgd step %d" % i)
    p, m, v = g["p0"], np.zeros_like(g["p0"]), np.zeros_like(g["p0"])
    for i in range(3):
        before = p
        p, m, v = R.adam(p, g["g%d" % i], m, v, 1e-3, 0.9, 0.999, 1e-8, float(i + 1))
        assert_close(p, g["adam_p%d" % (i + 1)], tol=1e-6, what="adam step %d" % i)
        prev = g["p0"] if i == 0 else g["adam_p%d" % i]
        # also on the UPDATE, which is what the arithmetic actually produces
        assert_close(p.astype(np.float64) - before, g["adam_p%d" % (i + 1)].astype(np.float64) - prev, tol=2e-3,
                     what="adam update %d" % i)


def test_more_optimizers_golden(golden):
    """SGD momentum / weight decay, Adagrad, RMSprop (optim/sgd.mojo:42-60, adagrad.mojo:36-45, rmsprop.mojo:39-53)
    against torch.optim, three steps each. The reference stores velocity = -lr * (torch's momentum buffer)."""
    g = golden("optim")
    cases = {
        "sgdm": lambda p, gr, st: R.sgd_momentum(p, gr, st, 1e-2, 0.9, 0.0),
        "sgdmw": lambda p, gr, st: R.sgd_momentum(p, gr, st, 1e-2, 0.9, 0.05),
        "sgdw": lambda p, gr, st: R.sgd_momentum(p, gr, st, 1e-2, 0.0, 0.05),
        "adagrad": lambda p, gr, st: R.adagrad(p, gr, st, 1e-2, 1e-8),
        "rmsprop": lambda p, gr, st: R.rmsprop(p, gr, st, 1e-2, 0.99, 1e-8),
    }
    for name, fn in cases.items():
        p, st = g["p0"], np.zeros_like(g["p0"])
        for i in range(3):
            p, st = fn(p, g["g%d" % i], st)
            assert_close(p, g["%s_p%d" % (name, i + 1)], tol=2e-6, what="%s step %d" % (name, i))


def _mlp_case(g, n_layers):
    Ws = [np.ascontiguousarray(g["W%d" % i]) for i in range(n_layers)]
    bs = [np.ascontiguousarray(g["b%d" % i]) for i in range(n_layers)]
    widths = [Ws[0].shape[0]] + [W.shape[1] for W in Ws]
    return widths, Ws, bs


def test_mlp_sine_sgd_golden(golden):
    g = golden("mlp_sine")
    widths, Ws, bs = _mlp_case(g, 8)
    for step in range(3):
        loss, dWs, dbs = R.mlp_step(widths, "relu", g["x"], g["y"], Ws, bs, opt="sgd", lr=1e-3)
        assert_close([loss], g["loss%d" % step], what="loss step %d" % step)
        if step == 0:
            for i in range(8):
                assert_close(dWs[i], g["dW%d" % i], what="dW%d" % i)
                assert dbs[i].shape == (1, widths[i + 1])  # kept leading axis (expand_op.mojo:121-126)
                assert_close(dbs[i], g["db%d" % i], what="db%d" % i)
    for i in range(8):
        assert_close(Ws[i], g["W%d_after" % i], what="W%d after 3 steps" % i)
        assert_close(bs[i], g["b%d_after" % i], what="b%d after 3 steps" % i)


def test_mlp_tanh_adam_golden(golden):
    g = golden("mlp_tanh_adam")
    widths, Ws, bs = _mlp_case(g, 3)
    state = {k: [np.zeros_like(a) for a in (Ws if k.endswith("W") else bs)] for k in ("mW", "vW", "mb", "vb")}
    for step in range(2):
        loss, dWs, dbs = R.mlp_step(widths, "tanh", g["x"], g["y"], Ws, bs, opt="adam", lr=1e-3, t=float(step + 1),
                                    state=state)
        assert_close([loss], g["loss%d" % step], what="loss")
        if step == 0:
            for i in range(3):
                assert_close(dWs[i], g["dW%d" % i], what="dW%d" % i)
                assert_close(dbs[i], g["db%d" % i], what="db%d" % i)
    for i in range(3):
        assert_close(Ws[i], g["W%d_after" % i], what="W%d after Adam" % i)
        assert_close(bs[i], g["b%d_after" % i], what="b%d after Adam" % i)


def test_doc_known_answers():
    # README.md:74-76: y = sum(x^2) at [1,2,3] -> 14, dy/dx = [2,4,6]
    x = np.array([1, 2, 3], np.float32)
    assert R.reduce_add(R.unary("square", x), [0])[0] == 14.0
    np.testing.assert_array_equal(R.unary_vjp("square", x, np.ones(3, np.float32)), [2, 4, 6])
    # examples/custom_ops_examples/custom_mul.mojo:64-71: sum(a*b) = 32, grads [4,5,6] and [1,2,3]
    a, b = np.array([1, 2, 3], np.float32), np.array([4, 5, 6], np.float32)
    assert R.reduce_add(R.binary("mul", a, b), [0])[0] == 32.0
    one = np.ones(3, np.float32)
    np.testing.assert_array_equal(R.binary("mul", b, one), [4, 5, 6])
    np.testing.assert_array_equal(R.binary("mul", a, one), [1, 2, 3])


def test_complex_abs_and_vjp():
    rng = np.random.default_rng(3)
    z = (rng.standard_normal(50) + 1j * rng.standard_normal(50)).astype(np.complex64)
    assert_close(R.cabs(z), np.abs(z.astype(np.complex128)), what="|z|")
    g = rng.standard_normal(50).astype(np.float32)
    assert_close(R.cabs_vjp(z, g), g * z.astype(np.complex128) / np.abs(z.astype(np.complex128)), what="abs vjp")


def test_complex_mlp_conjugate_convention(golden):
    # Sum |out|^2 through identity layers. With the reference's coded rules (no conjugation,
    # matmul_op.mojo:278-283) the gradient is conj(torch's); with conjugated operands it equals torch's.
    g = golden("complex_mlp")
    Ws = [g["W%d" % i] for i in range(3)]
    acts = [g["z"]]
    for W in Ws:
        acts.append(R.matmul(acts[-1], W))
    assert_close(acts[-1], g["out"], what="complex forward")
    delta = 2 * acts[-1]  # abs -> square -> sum chain gives 2 z in both conventions
    for i in (2, 1, 0):
        dW_wirtinger = R.matmul(np.conj(acts[i]).T, delta)
        assert_close(dW_wirtinger, g["dW%d" % i], what="Wirtinger dW%d" % i)
        delta = R.matmul(delta, np.conj(Ws[i]).T)


POOL_CASES = ["1d", "2d", "3d", "2d_dil"]


def _pool_cfg(g, name):
    k, st, pad, dil = (tuple(int(v) for v in row) for row in g["cfg_" + name])
    return k, st, pad, dil


@pytest.mark.parametrize("name", POOL_CASES)
def test_pool_golden(golden, name):  # test_max_pool2d_op.mojo, test_avg_pool2d_op.mojo and siblings: forward vs torch
    g = golden("pool")
    k, st, pad, dil = _pool_cfg(g, name)
    x, gy = g["x_" + name], g["g_" + name]
    assert_close(R.pool("max", x, k, st, pad, dil), g["max_" + name], tol=1e-7, what="max_pool" + name)
    assert_close(R.pool_bwd("max", x, gy, k, st, pad, dil), g["dmax_" + name], tol=1e-6, what="max_pool grad " + name)
    if "avg_" + name in g.files:
        assert_close(R.pool("avg", x, k, st, pad, dil), g["avg_" + name], tol=1e-6, what="avg_pool" + name)
        assert_close(R.pool_bwd("avg", x, gy, k, st, pad, dil), g["davg_" + name], tol=1e-6, what="avg_pool grad " + name)


def test_avg_pool_dilated_brute_force():
    """torch's average pooling has no dilation; check that case against a direct numpy restatement and the
    adjoint identity <pool(x), g> = <x, pool_bwd(g)> (average pooling is linear)."""
    rng = np.random.default_rng(3)
    x = rng.standard_normal((2, 2, 9, 8)).astype(np.float32)
    k, st, pad, dil = (2, 3), (2, 1), (1, 2), (3, 2)
    y = R.pool("avg", x, k, st, pad, dil)
    want = np.zeros(y.shape)
    for oy in range(y.shape[2]):
        for ox in range(y.shape[3]):
            taps = [(oy * st[0] - pad[0] + a * dil[0], ox * st[1] - pad[1] + b * dil[1]) for a in range(k[0]) for b in range(k[1])]
            taps = [(r, c) for r, c in taps if 0 <= r < 9 and 0 <= c < 8]
            want[:, :, oy, ox] = sum(x[:, :, r, c].astype(np.float64) for r, c in taps) / len(taps) if taps else 0.0
    assert_close(y, want, tol=1e-6, what="dilated avg_pool")
    gy = rng.standard_normal(y.shape).astype(np.float32)
    lhs = np.vdot(y.astype(np.float64), gy)
    rhs = np.vdot(x.astype(np.float64), R.pool_bwd("avg", x, gy, k, st, pad, dil))
    assert abs(lhs - rhs) <= 1e-5 * abs(lhs)
    # an empty window (all taps outside) gives -inf for max and 0 for average (avg_pool2d_op.mojo:137-140)
    z = np.ones((1, 1, 2), np.float32)
    assert R.pool("max", z, 1, 1, 2)[0, 0, 0] == -np.inf and R.pool("avg", z, 1, 1, 2)[0, 0, 0] == 0.0


@pytest.mark.parametrize("name", ["1d", "3d", "3d_unit"])
def test_conv1d_conv3d_golden(golden, name):  # test_conv1d_op.mojo, test_conv3d_op.mojo: forward vs torch
    g = golden("convnd")
    st, pad, dil = (tuple(int(v) for v in row) for row in g["cfg_" + name])
    x, w, b, gy = (g[k + "_" + name] for k in ("x", "w", "b", "g"))
    assert_close(R.convnd(x, w, b, st, pad, dil), g["y_" + name], tol=1e-6, what="conv" + name)
    dx, dw, db = R.convnd_bwd(x, w, gy, st, pad, dil)
    assert_close(dx, g["dx_" + name], tol=1e-6, what="dx " + name)
    assert_close(dw, g["dw_" + name], tol=1e-6, what="dw " + name)
    assert_close(db, g["db_" + name], tol=1e-6, what="db " + name)


def test_convnd_reduces_to_conv2d(golden):
    """The 3-D loop with depth 1 is the 2-D loop: both restatements must agree exactly."""
    g = golden("conv2d")
    x, w, b = g["x"], g["w"], g["b"]
    y2 = R.conv2d(x, w, b, (2, 2), (1, 1), (1, 1))
    np.testing.assert_array_equal(R.convnd(x, w, b, (2, 2), (1, 1), (1, 1)), y2)


def test_views_golden(golden):
    """The oracle's strided gather and scatter against torch: as_strided with overlapping windows and its
    gradient (the two cases of test_as_strided_op.mojo), a stepped slice, pad."""
    g = golden("views")
    assert_close(R.as_strided(g["as_x"], (1, 2, 40, 2, 2), (16, 8, 2, 2, 1)), g["as_y"], tol=0, what="as_strided")
    x2 = g["as_x2"]
    cot = np.cos(R.as_strided(x2, (30, 30, 2), (9, 30, 2)).astype(np.float64)).astype(np.float32)
    assert_close(R.strided_scatter(cot, x2.shape, (9, 30, 2), 0, accumulate=True), g["as_dx2"], what="as_strided grad")
    # slice [1:6:2, 2:, ::3] of a (7, 9, 10) array: element strides (90, 10, 1) -> (180, 10, 3), offset 90 + 20
    assert_close(R.as_strided(g["sl_x"], (3, 7, 4), (180, 10, 3), 110), g["sl_y"], tol=0, what="slice")
    assert_close(R.strided_scatter(g["sl_g"], (7, 9, 10), (180, 10, 3), 110), g["sl_dx"], tol=0, what="slice grad")
    # pad: a (3, 4) block at [1:4, 2:9:2] of a (5, 9) target: strides (9, 2), offset 11
    assert_close(R.strided_scatter(g["pad_x"], (5, 9), (9, 2), 11), g["pad_y"], tol=0, what="pad")
    assert_close(R.as_strided(g["pad_g"], (3, 4), (9, 2), 11), g["pad_dx"], tol=0, what="pad grad")


def test_strided_scatter_brute_force():
    """Overlapping windows accumulate: a sliding window of 3 with stride 1 over 6 elements, by hand."""
    src = np.arange(12, dtype=np.float32).reshape(4, 3)
    want = np.zeros(6, np.float32)
    for i in range(4):
        for j in range(3):
            want[i + j] += src[i, j]
    np.testing.assert_array_equal(R.strided_scatter(src, (6,), (1, 1), 0, accumulate=True), want)
    z = (np.arange(6) + 1j * np.arange(6)).astype(np.complex64).reshape(2, 3)
    out = R.strided_scatter(z, (4, 4), (4, 1), 5)
    want = np.zeros((4, 4), np.complex64)
    want[1:3, 1:4] = z
    np.testing.assert_array_equal(out, want)
