"""The host-side mirror of the reference API (Array / backward() / grad(), nn.MLP, optim) running on
the HIP library, checked against the PyTorch-float64 golden fixtures and the CPU oracle. The tests
follow the shape of the reference's own (tests/test_endia/test_functional/...): forward, gradient of
sum(op(x)), complex forward. Tolerance 1e-4 relative per tensor."""
import numpy as np
import pytest

from conftest import assert_close, mean_rel

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def nd():
    import endia_amd
    return endia_amd


def test_matmul_and_grad(nd, golden):  # test_matmul_op.mojo:18-59
    g = golden("matmul")
    a, b = nd.array(g["a"], requires_grad=True), nd.array(g["b"], requires_grad=True)
    res = nd.matmul(a, b)
    assert_close(res.to_numpy(), g["out"], what="matmul")
    assert nd.utils.is_close(res, g["out"])
    nd.sum(res).backward()
    assert_close(a.grad().to_numpy(), g["da"], what="grad0")
    assert_close(b.grad().to_numpy(), g["db"], what="grad1")  # shape [1,40,50]: kept broadcast axis
    assert mean_rel(b.grad().to_numpy().reshape(40, 50), g["db"]) <= 1e-4


def test_matmul_square_transposed_views(nd, golden):
    # dX = g W^T with a SQUARE W: the documented semantics, not the reference's contiguity-shortcut defect
    g = golden("matmul")
    a, b = nd.array(g["sa"], requires_grad=True), nd.array(g["sb"], requires_grad=True)
    nd.sum(nd.matmul(a, b) * nd.array(g["sg"])).backward()
    assert_close(a.grad().to_numpy(), g["dsa"], what="dA")
    assert_close(b.grad().to_numpy(), g["dsb"], what="dB")


def test_matmul_complex(nd, golden):  # test_matmul_op.mojo:62-75
    g = golden("matmul")
    res = nd.matmul(nd.array(g["ca"]), nd.array(g["cb"]))
    assert res.is_complex()
    assert_close(res.to_numpy(), g["cout"], what="complex matmul")


@pytest.mark.parametrize("op", ["relu", "tanh", "sin", "cos", "neg", "square", "sqrt", "abs"])
def test_unary_grad(nd, golden, op):  # test_relu_op.mojo:32-49 and siblings
    g = golden("unary")
    x = nd.array(g["xp"] if op == "sqrt" else g["x"], requires_grad=True)
    y = getattr(nd, op)(x)
    assert_close(y.to_numpy(), g[op], what=op)
    nd.sum(y).backward()
    assert_close(x.grad().to_numpy(), g["d" + op], what="grad " + op)


MORE_UNARY = ["exp", "log", "sigmoid", "sinh", "cosh", "tan", "asin", "acos", "atan", "reciprocal"]


def _more_src(g, op):
    return g["xp"] if op in ("log", "reciprocal") else (g["xu"] if op in ("tan", "asin", "acos") else g["x"])


@pytest.mark.parametrize("op", MORE_UNARY)
def test_unary_more_grad(nd, golden, op):  # test_exp_op.mojo, test_log_op.mojo, ... : forward and grad of sum(op(x))
    g = golden("unary_more")
    x = nd.array(_more_src(g, op), requires_grad=True)
    y = getattr(nd, op)(x)
    assert_close(y.to_numpy(), g[op], what=op)
    nd.sum(y).backward()
    assert_close(x.grad().to_numpy(), g["d" + op], what="grad " + op)


def test_pow_grad_and_comparisons(nd, golden):  # test_pow_op.mojo
    g = golden("binary_more")
    a, b = nd.array(g["a"], requires_grad=True), nd.array(g["b"], requires_grad=True)
    y = nd.pow(a, b)
    assert_close(y.to_numpy(), g["pow"], what="pow")
    nd.sum(y).backward()
    assert_close(a.grad().to_numpy(), g["dpow_a"], what="dpow/da")
    assert_close(b.grad().to_numpy(), g["dpow_b"], what="dpow/db")
    ca, cb = nd.array(g["ca"]), nd.array(g["cb"])
    for name in ("greater", "greater_equal", "less", "less_equal", "equal", "not_equal"):
        np.testing.assert_array_equal(getattr(nd, name)(ca, cb).to_numpy(), g[name], err_msg=name)
    x = nd.array(np.array([1.5, -2.0, 3.0], np.float32), requires_grad=True)
    np.testing.assert_allclose((x ** 3).to_numpy(), [3.375, -8.0, 27.0], rtol=1e-5)
    np.testing.assert_allclose((2.0 ** x).to_numpy(), [2 ** 1.5, 0.25, 8.0], rtol=1e-5)


def test_fused_expression_forward_and_gradients(nd, golden):
    """A fused expression must equal the same ops run one by one, in value and in every gradient, with
    full, row-vector and one-element inputs; and both must equal float64."""
    g = golden("binary")
    a_np, b_np = g["a"], g["b2"][0]          # [2,30,40], [40]
    s_np = np.array([0.7], np.float32)

    def expr(a, b, s):
        return nd.sigmoid(a * b + 1.0) * nd.tanh(a - s) / (nd.square(b) + 2.0)

    fused = nd.fuse(expr)
    outs = []
    for f in (fused, expr):
        a, b, s = (nd.array(v, requires_grad=True) for v in (a_np, b_np, s_np))
        y = f(a, b, s)
        nd.sum(nd.sin(y)).backward()
        outs.append([y.to_numpy(), a.grad().to_numpy(), b.grad().to_numpy(), s.grad().to_numpy()])
    for got, want, what in zip(outs[0], outs[1], ["value", "da", "db", "ds"]):
        assert got.shape == want.shape, what
        assert_close(got, want, tol=1e-5, what="fused vs op by op: " + what)
    import torch
    ta, tb, ts = (torch.tensor(v, dtype=torch.float64, requires_grad=True) for v in (a_np, b_np, s_np))
    ty = torch.sigmoid(ta * tb + 1.0) * torch.tanh(ta - ts) / (tb * tb + 2.0)
    torch.sin(ty).sum().backward()
    for got, want, what in zip(outs[0], [ty.detach(), ta.grad, tb.grad, ts.grad], ["value", "da", "db", "ds"]):
        assert_close(got, want.numpy(), what="fused vs float64: " + what)


def test_fused_expression_one_launch_each_way(nd):
    """The fused forward is one program and the fused backward one program (plus the reductions of
    broadcast inputs): count library calls."""
    from endia_amd import _lib as L
    calls = []
    orig = L.call

    def spy(name, *args):
        calls.append(name)
        return orig(name, *args)

    f = nd.fuse(lambda a, b: nd.relu(a * b) + nd.exp(-nd.abs(a)))
    a = nd.array(np.linspace(-2, 2, 64, dtype=np.float32).reshape(4, 16), requires_grad=True)
    b = nd.array(np.linspace(1, 3, 64, dtype=np.float32).reshape(4, 16), requires_grad=True)
    f(a, b)  # traced and compiled
    L.call = spy
    try:
        y = f(a, b)
        fwd = [c for c in calls if c not in ("endia_hip_malloc", "endia_hip_free")]
        assert fwd == ["endia_hip_ew_program"], fwd
        del calls[:]
        seed = nd.ones([4, 16])
        y._vjp(y._args, seed, y)
        bwd = [c for c in calls if c not in ("endia_hip_malloc", "endia_hip_free", "endia_hip_fill")]
        assert bwd == ["endia_hip_ew_program"], bwd
    finally:
        L.call = orig
    x64 = np.linspace(-2, 2, 64).reshape(4, 16)
    w64 = np.linspace(1, 3, 64).reshape(4, 16)
    assert_close(y.to_numpy(), np.maximum(x64 * w64, 0) + np.exp(-np.abs(x64)), what="fused value")


def test_fused_expression_second_order(nd):
    """Under create_graph the fused gradient is rebuilt from differentiable ops, so a Hessian-vector
    product through a fused expression equals the one through the plain ops and float64."""
    rng = np.random.default_rng(11)
    x_np, v_np = rng.standard_normal((6, 8)).astype(np.float32), rng.standard_normal((6, 8)).astype(np.float32)

    def expr(x):
        return nd.sin(x) * nd.exp(x * 0.5)

    res = []
    for f in (nd.fuse(expr), expr):
        x = nd.array(x_np, requires_grad=True)
        nd.sum(f(x)).backward(create_graph=True)
        gx = x.grad()
        hv = nd.grad(outs=nd.sum(gx * nd.array(v_np)), inputs=x)[0]
        res.append((gx.to_numpy(), hv.to_numpy()))
    assert_close(res[0][0], res[1][0], tol=1e-5, what="gradient")
    assert_close(res[0][1], res[1][1], tol=1e-5, what="hessian-vector product")
    x64 = x_np.astype(np.float64)
    e = np.exp(0.5 * x64)
    assert_close(res[0][0], e * (np.cos(x64) + 0.5 * np.sin(x64)), what="gradient vs float64")
    assert_close(res[0][1], v_np * e * (np.cos(x64) - 0.75 * np.sin(x64)), what="hvp vs float64")


@pytest.mark.parametrize("op", ["add", "sub", "mul", "div"])
def test_binary_grad(nd, golden, op):  # test_add_op.mojo:34-60, test_mul_op.mojo:34-59
    g = golden("binary")
    a = nd.array(g["a"], requires_grad=True)
    b = nd.array(g["b2"] if op == "div" else g["b"], requires_grad=True)
    y = getattr(nd, op)(a, b)
    assert_close(y.to_numpy(), g[op], what=op)
    nd.sum(nd.sin(y)).backward(create_graph=True)  # the reference's add/mul tests build the graph too
    assert_close(a.grad().to_numpy(), g[op + "_da"], what="dA")
    assert_close(b.grad().to_numpy(), g[op + "_db"], what="dB")


def test_reduce_mean_expand_grad(nd, golden):  # test_reduce_add_op / test_mean_op / test_expand_op
    g = golden("reduce")
    x = nd.array(g["x"], requires_grad=True)
    r = nd.reduce_add(x, [0, 2])
    assert r.shape() == [1, 30, 1]
    assert_close(r.to_numpy(), g["sum02"], what="reduce_add")
    nd.sum(nd.sin(r)).backward()
    assert_close(x.grad().to_numpy(), g["dsum02"], what="d reduce_add")
    x2 = nd.array(g["x"], requires_grad=True)
    m = nd.mean(x2, [1])
    assert m.shape() == [2, 40]
    assert_close(m.to_numpy(), g["mean1"], what="mean")
    nd.sum(nd.sin(m)).backward()
    assert_close(x2.grad().to_numpy(), g["dmean1"], what="d mean")
    b = nd.array(g["bsrc"], requires_grad=True)
    e = nd.expand(b, [2, 30, 40])
    nd.sum(e * nd.array(g["x"])).backward()
    assert b.grad().shape() == [1, 1, 40]  # kept axes, as Expand.vjp leaves them
    assert_close(b.grad().to_numpy(), g["dexpand"], what="d expand")


def test_other_reductions_and_their_gradients(nd, golden):
    """reduce_max / reduce_min / reduce_argmax / reduce_argmin / reduce_mul / prod / variance / std as the reference's
    tests call them (test_reduce_max_op.mojo:18-34 and siblings, test_std_op.mojo:18-58, test_variance_op.mojo:18-59)."""
    g = golden("reduce_more")
    x = nd.array(g["x"])
    for name, fn, axis, key in (("max", nd.reduce_max, [1], "max1"), ("min", nd.reduce_min, [1], "min1"),
                                ("argmax", nd.reduce_argmax, [1], "argmax1"), ("argmin", nd.reduce_argmin, [1], "argmin1"),
                                ("argmax last axis", nd.reduce_argmax, 2, "argmax2"), ("max over two axes", nd.reduce_max, [0, 2], "max02")):
        out = fn(x, axis)
        assert out.shape() == list(g[key].shape), name
        np.testing.assert_array_equal(out.to_numpy(), g[key], err_msg=name)
    assert nd.reduce_max(x, [1], keepdims=True).shape() == [2, 1, 40]
    assert_close(nd.reduce_mul(x, [1]).to_numpy(), g["prod1"], what="reduce_mul")
    assert_close(nd.prod(nd.array(g["x"][0, :8, :5].copy())).to_numpy(), g["prod_all"], what="prod")
    assert_close(nd.variance(x, [1]).to_numpy(), g["var1"], what="variance")
    assert_close(nd.variance(x, [0, 2], unbiased=False).to_numpy(), g["var02_biased"], what="biased variance")
    assert_close(nd.std(x, [1]).to_numpy(), g["std1"], what="std")
    assert_close(nd.std(x, [1], keepdims=True).to_numpy(), g["std1_keep"], what="std, kept axis")
    for fn, key in ((nd.std, "dstd1"), (nd.variance, "dvar1")):
        xg = nd.array(g["x"], requires_grad=True)
        nd.sum(fn(xg, [1])).backward()
        assert_close(xg.grad().to_numpy(), g[key], what=key)
    # no backward rule exists for the extrema or the product (the reference's are the default / a placeholder): refused loudly
    xg = nd.array(g["x"], requires_grad=True)
    with pytest.raises(NotImplementedError):
        nd.sum(nd.reduce_max(xg, [1])).backward()
    with pytest.raises(ValueError):
        nd.reduce_argmax(x, [0, 1])
    with pytest.raises(ValueError):
        nd.reduce_max(nd.complex(x, x), [1])


def test_permute_reshape_views(nd):
    rng = np.random.default_rng(0)
    a = rng.standard_normal((2, 3, 4)).astype(np.float32)
    x = nd.array(a, requires_grad=True)
    p = nd.permute(x, [2, 0, 1])
    np.testing.assert_array_equal(p.to_numpy(), a.transpose(2, 0, 1))
    np.testing.assert_array_equal(x.T().to_numpy(), np.swapaxes(a, -1, -2))
    w = rng.standard_normal((4, 2, 3)).astype(np.float32)
    nd.sum(p * nd.array(w)).backward()
    assert_close(x.grad().to_numpy(), w.transpose(1, 2, 0), what="permute vjp")
    np.testing.assert_array_equal(nd.reshape(x.T(), [6, 4]).to_numpy(), np.swapaxes(a, -1, -2).reshape(6, 4))


def test_doc_example_second_order(nd):  # README.md:56-76
    x = nd.arange(1.0, 4.0, requires_grad=True)
    y = nd.sum(x ** 2)
    y.backward(create_graph=True)
    dy_dx = x.grad()
    d2y = nd.grad(outs=nd.sum(dy_dx), inputs=x)[0]
    assert y.item() == 14.0
    np.testing.assert_array_equal(dy_dx.to_numpy(), [2, 4, 6])
    np.testing.assert_array_equal(d2y.to_numpy(), [2, 2, 2])


def test_doc_example_functional(nd):  # README.md:92-108
    def foo(x):
        return nd.sum(x ** 2)
    foo_jac = nd.grad(foo)
    foo_hes = nd.jacobian(foo_jac)
    x = nd.arange(1.0, 4.0)
    np.testing.assert_array_equal(foo_jac(x).to_numpy(), [2, 4, 6])
    np.testing.assert_array_equal(foo_hes(x).to_numpy(), 2 * np.eye(3, dtype=np.float32))
    (v,), (gr,) = nd.value_and_grad(foo)(x)  # one list per order, as the reference returns it (callable.mojo:186-195)
    assert v.item() == 14.0
    np.testing.assert_array_equal(gr.to_numpy(), [2, 4, 6])


def test_custom_op_example(nd):  # examples/custom_ops_examples/custom_mul.mojo:64-71
    a = nd.array([1.0, 2.0, 3.0], requires_grad=True)
    b = nd.array([4.0, 5.0, 6.0], requires_grad=True)
    c = nd.sum(nd.mul(a, b))
    c.backward()
    assert c.item() == 32.0
    np.testing.assert_array_equal(a.grad().to_numpy(), [4, 5, 6])
    np.testing.assert_array_equal(b.grad().to_numpy(), [1, 2, 3])


def test_gradient_accumulation_multi_use(nd):
    # x used twice: the two cotangents are added by an `add` op (autograd/functional.mojo:55-57)
    x = nd.array([0.5, -1.0, 2.0], requires_grad=True)
    y = nd.sum(nd.sin(x) * x)
    y.backward()
    v = np.array([0.5, -1.0, 2.0])
    assert_close(x.grad().to_numpy(), np.cos(v) * v + np.sin(v), what="product rule")
    y.zero_grad()
    assert not x.has_grad()


def test_mse_fused_matches_composed(nd, golden):
    g = golden("mse")
    p = nd.array(g["pred"], requires_grad=True)
    loss = nd.mse(p, nd.array(g["target"]))
    loss.backward()
    assert_close([loss.item()], g["loss"], what="mse")
    assert_close(p.grad().to_numpy(), g["dpred"], what="mse grad")
    p2 = nd.array(g["pred"], requires_grad=True)
    d = nd.sub(p2, nd.array(g["target"]))
    loss2 = nd.sum(d * d) / float(p2.size())  # mse_op.mojo:17-20 verbatim
    loss2.backward()
    assert_close([loss2.item()], g["loss"], what="composed mse")
    assert_close(p2.grad().to_numpy(), g["dpred"], what="composed mse grad")


def _load_mlp(nd, g, n_layers, act, fused):
    widths = [g["W0"].shape[0]] + [g["W%d" % i].shape[1] for i in range(n_layers)]
    mlp = nd.nn.MLP(widths, compute_backward=True, activation=act, fused=fused)
    for i in range(n_layers):
        mlp.weights[i] = nd.array(g["W%d" % i], requires_grad=True)
        mlp.biases[i] = nd.array(g["b%d" % i], requires_grad=True)
    return mlp, widths


@pytest.mark.parametrize("fused", [True, False, "model"])
def test_mlp_sine_sgd(nd, golden, fused):
    """The reference's benchmark model (mlp_imp.mojo:25-75) for three SGD steps, against torch float64
    and against the CPU oracle's restatement of the same tape."""
    from oracle import endia_ref as R
    g = golden("mlp_sine")
    mlp, widths = _load_mlp(nd, g, 8, "relu", fused)
    opt = nd.optim.SGD(mlp.params(), lr=1e-3)
    x, y = nd.array(g["x"]), nd.array(g["y"])
    Wr = [np.ascontiguousarray(g["W%d" % i]) for i in range(8)]
    br = [np.ascontiguousarray(g["b%d" % i]) for i in range(8)]
    for step in range(3):
        pred = mlp.forward(x)
        loss = nd.mse(pred, y)
        loss.backward()
        loss_ref, dWr, dbr = R.mlp_step(widths, "relu", g["x"], g["y"], Wr, br, opt="sgd", lr=1e-3)
        assert_close([loss.item()], g["loss%d" % step], what="loss %d" % step)
        assert_close([loss.item()], [loss_ref], what="loss %d vs oracle" % step)
        for i in range(8):
            assert_close(mlp.weights[i].grad().to_numpy(), dWr[i], what="dW%d step %d vs oracle" % (i, step))
            assert_close(mlp.biases[i].grad().to_numpy(), dbr[i], what="db%d step %d vs oracle" % (i, step))
            if step == 0:
                assert_close(mlp.weights[i].grad().to_numpy(), g["dW%d" % i], what="dW%d" % i)
                assert_close(mlp.biases[i].grad().to_numpy(), g["db%d" % i], what="db%d" % i)
        opt.step()
        loss.zero_grad()
    for i in range(8):
        assert_close(mlp.weights[i].to_numpy(), g["W%d_after" % i], what="W%d after" % i)
        assert_close(mlp.biases[i].to_numpy(), g["b%d_after" % i], what="b%d after" % i)


@pytest.mark.parametrize("fused", [True, False, "model"])
def test_mlp_tanh_adam(nd, golden, fused):
    g = golden("mlp_tanh_adam")
    mlp, widths = _load_mlp(nd, g, 3, "tanh", fused)
    opt = nd.optim.Adam(mlp.params(), lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8)
    x, y = nd.array(g["x"]), nd.array(g["y"])
    for step in range(2):
        loss = nd.mse(mlp.forward(x), y)
        loss.backward()
        assert_close([loss.item()], g["loss%d" % step], what="loss")
        if step == 0:
            for i in range(3):
                assert_close(mlp.weights[i].grad().to_numpy(), g["dW%d" % i], what="dW%d" % i)
                assert_close(mlp.biases[i].grad().to_numpy(), g["db%d" % i], what="db%d" % i)
        opt.step()
        loss.zero_grad()
    for i in range(3):
        assert_close(mlp.weights[i].to_numpy(), g["W%d_after" % i], what="W%d after Adam" % i)
        assert_close(mlp.biases[i].to_numpy(), g["b%d_after" % i], what="b%d after Adam" % i)


@pytest.mark.parametrize("seeded", [False, True])
@pytest.mark.parametrize("fused", [True, False])
def test_hvp_double_backward(nd, golden, fused, seeded):
    """Hessian-vector product by create_graph=True double backward (README.md:69-71 pattern) on a sin MLP
    with loss = sum(out^2); also <u, Hv> = <v, Hu>. seeded: the second pass starts from the first-order
    gradients with v as their cotangents (grad_outs) instead of from the scalar sum <gradients, v>."""
    g = golden("hvp_sin")
    mlp, _ = _load_mlp(nd, g, 3, "sin", fused)
    x = nd.array(g["x"])

    def hvp(vs):
        out = mlp.forward(x)
        loss = nd.sum(out * out)
        loss.backward(create_graph=True)
        grads = [p.grad().to_numpy() for p in mlp.params()]
        if seeded:
            firsts = [p.grad() for p in mlp.params()]
            hv = nd.grad(outs=firsts, inputs=mlp.params(),
                         grad_outs=[nd.reshape(nd.array(v), f.shape()) for v, f in zip(vs, firsts)])
        else:
            s = None
            for p, v in zip(mlp.params(), vs):
                term = nd.sum(p.grad() * nd.reshape(nd.array(v), p.grad().shape()))
                s = term if s is None else s + term
            hv = nd.grad(outs=s, inputs=mlp.params())
        res = [h.to_numpy() for h in hv]
        loss.zero_grad()
        return float(loss.item()), grads, res

    vs = []
    for i in range(3):
        vs += [g["vW%d" % i], g["vb%d" % i]]
    loss, grads, hv = hvp(vs)
    assert_close([loss], g["loss"], what="loss")
    for i in range(3):
        assert_close(grads[2 * i], g["gW%d" % i], what="gW%d" % i)
        assert_close(grads[2 * i + 1], g["gb%d" % i], what="gb%d" % i)
        assert_close(hv[2 * i], g["hW%d" % i], what="HvW%d" % i)
        assert_close(hv[2 * i + 1], g["hb%d" % i], what="Hvb%d" % i)
    rng = np.random.default_rng(5)
    us = [rng.standard_normal(v.shape).astype(np.float32) for v in vs]
    _, _, hu = hvp(us)
    uHv = sum(float(np.vdot(u.astype(np.float64), h.reshape(u.shape))) for u, h in zip(us, hv))
    vHu = sum(float(np.vdot(v.astype(np.float64), h.reshape(v.shape))) for v, h in zip(vs, hu))
    assert abs(uHv - vHu) <= 1e-4 * max(abs(uHv), abs(vHu))


def test_gradient_accumulation_inside_the_product_launch(nd, golden):
    """Where a tensor has several consumers the walk sums their contributions with `add` (autograd/functional.mojo:51-57).
    A matmul / linear / sin rule takes the earlier gradient into its own launch instead (a bias row or an in-place
    accumulate in the GEMM epilogue, one fused elementwise launch): the Hessian-vector product with that switched on
    and off gives the same numbers, launches are saved, and an array that user code holds is never written."""
    from endia_amd.autograd import functional as AF
    from endia_amd import functional as F
    g = golden("hvp_sin")
    x = nd.array(g["x"])
    vs = []
    for i in range(3):
        vs += [g["vW%d" % i], g["vb%d" % i]]

    def hvp(fused):
        mlp, _ = _load_mlp(nd, g, 3, "sin", fused)
        out = mlp.forward(x)
        loss = nd.sum(out * out)
        loss.backward(create_graph=True)
        firsts = [p.grad() for p in mlp.params()]
        hv = nd.grad(outs=firsts, inputs=mlp.params(), grad_outs=[nd.reshape(nd.array(v), f.shape()) for v, f in zip(vs, firsts)])
        res = [h.to_numpy() for h in hv]
        loss.zero_grad()
        return res

    for fused in (True, False):
        before = F._absorbed_launches[0]
        with_absorb = hvp(fused)
        saved = F._absorbed_launches[0] - before
        AF.absorb_enabled[0] = False
        try:
            plain = hvp(fused)
            assert F._absorbed_launches[0] - before == saved
        finally:
            AF.absorb_enabled[0] = True
        assert saved >= (8 if fused else 4), "only %d additions were taken into product launches" % saved
        for i in range(3):
            assert_close(with_absorb[2 * i], g["hW%d" % i], what="HvW%d" % i)
            assert_close(with_absorb[2 * i + 1], g["hb%d" % i], what="Hvb%d" % i)
        for a, b in zip(with_absorb, plain):
            assert_close(a, b, tol=2e-6, mean_tol=1e-4, what="with and without in-launch accumulation")

    # a cotangent that the caller holds is an output's gradient and then meets a product's contribution: it must be
    # read, not accumulated into
    rng = np.random.default_rng(11)
    a = nd.array(rng.standard_normal((6, 5)).astype(np.float32), requires_grad=True)
    Mn = rng.standard_normal((5, 5)).astype(np.float32)
    cn, dn = rng.standard_normal((6, 5)).astype(np.float32), rng.standard_normal((6, 5)).astype(np.float32)
    y = a * 1.0
    w = nd.matmul(y, nd.array(Mn))
    c, d = nd.array(cn), nd.array(dn)
    (ga,) = nd.grad(outs=[y, w], inputs=[a], grad_outs=[c, d])
    np.testing.assert_array_equal(c.to_numpy(), cn)
    np.testing.assert_array_equal(d.to_numpy(), dn)
    assert_close(ga.to_numpy(), cn.astype(np.float64) + dn.astype(np.float64) @ Mn.T.astype(np.float64), what="two contributions")
    # three products into one tensor: the second and third accumulate in place into the first one's result
    a = nd.array(rng.standard_normal((6, 5)).astype(np.float32), requires_grad=True)
    Ms = [rng.standard_normal((5, 4)).astype(np.float32) for _ in range(3)]
    before = F._absorbed_launches[0]
    total = None
    for M in Ms:
        t = nd.sum(nd.matmul(a, nd.array(M)))
        total = t if total is None else total + t
    total.backward()
    assert F._absorbed_launches[0] - before == 2
    assert_close(a.grad().to_numpy(), np.ones((6, 4)) @ np.sum([M.astype(np.float64) for M in Ms], 0).T, what="three products")
    # matmul(a, a): both gradients go to the same tensor and nothing is offered
    a = nd.array(rng.standard_normal((4, 4)).astype(np.float32), requires_grad=True)
    b = nd.array(rng.standard_normal((4, 4)).astype(np.float32), requires_grad=True)
    an, bn = a.to_numpy().astype(np.float64), b.to_numpy().astype(np.float64)
    nd.sum(nd.matmul(a, a) + nd.matmul(a, b)).backward()
    one = np.ones((4, 4))
    assert_close(a.grad().to_numpy(), one @ an.T + an.T @ one + one @ bn.T, what="matmul(a, a) + matmul(a, b)")


def test_parked_products_share_launches(nd):
    """Mid-size products of a backward pass are parked and launched together (functional._sgemm, _lib.park_product).
    A two-layer sin model of 1024-wide layers, batch 512: gradient and Hessian-vector product with parking on and off
    agree, reading any result launches what it depends on, in-place accumulation into a parked product's output keeps
    its order, and an optimizer step sees finished gradients."""
    from endia_amd import _lib as L
    rng = np.random.default_rng(21)
    Bn, Wd = 512, 1024
    Wn = [(rng.standard_normal((Wd, Wd)) / np.sqrt(Wd)).astype(np.float32) for _ in range(2)]
    bn = [(0.1 * rng.standard_normal(Wd)).astype(np.float32) for _ in range(2)]
    vn = [rng.standard_normal(a.shape).astype(np.float32) for a in (Wn[0], bn[0], Wn[1], bn[1])]
    xn = rng.standard_normal((Bn, Wd)).astype(np.float32)

    def run():
        mlp = nd.nn.MLP([Wd] * 3, compute_backward=True, activation="sin", fused=True)
        for i in range(2):
            mlp.weights[i], mlp.biases[i] = nd.array(Wn[i], requires_grad=True), nd.array(bn[i], requires_grad=True)
        out = mlp.forward(nd.array(xn))
        loss = nd.sum(out * out)
        loss.backward(create_graph=True)
        firsts = [p.grad() for p in mlp.params()]
        hv = nd.grad(outs=firsts, inputs=mlp.params(), grad_outs=[nd.reshape(nd.array(v), f.shape()) for v, f in zip(vn, firsts)])
        res = [f.to_numpy() for f in firsts] + [h.to_numpy() for h in hv]
        loss.zero_grad()
        return res

    parked = run()
    assert not L._parked
    L.defer_products[0] = False
    try:
        plain = run()
    finally:
        L.defer_products[0] = True
    for k, (a, b) in enumerate(zip(parked, plain)):
        assert_close(a, b, tol=2e-6, mean_tol=1e-4, what="tensor %d with and without parking" % k)
    # float64 on the host
    import torch
    tW = [torch.tensor(w, dtype=torch.float64, requires_grad=True) for w in Wn]
    tb = [torch.tensor(b, dtype=torch.float64, requires_grad=True) for b in bn]
    h = torch.sin(torch.tensor(xn, dtype=torch.float64) @ tW[0] + tb[0])
    o = h @ tW[1] + tb[1]
    ps = [tW[0], tb[0], tW[1], tb[1]]
    gs = torch.autograd.grad((o * o).sum(), ps, create_graph=True)
    hv = torch.autograd.grad(gs, ps, grad_outputs=[torch.tensor(v, dtype=torch.float64) for v in vn])
    for k, t in enumerate(list(gs) + list(hv)):
        assert_close(parked[k], t.detach().numpy(), what="tensor %d vs float64" % k, mean_tol=1e-3)
    # a first-order step: the optimizer (an in-place writer) must see launched gradients
    a = nd.array(xn[:, :512].copy())
    W = nd.array(Wn[0][:512, :512].copy(), requires_grad=True)
    opt = nd.optim.SGD([W], lr=0.5)
    y = nd.matmul(a, W)                       # parked (512 x 512 x 512 is below the size that parks: run it anyway)
    z = nd.matmul(nd.array(xn), nd.array(Wn[1]))  # 512 x 1024 x 1024: parked
    assert L._parked
    nd.sum(y).backward()
    opt.step()
    assert not L._parked
    assert_close(W.to_numpy(), Wn[0][:512, :512] - 0.5 * (xn[:, :512].astype(np.float64).T @ np.ones((Bn, 512))), what="SGD after parked products")
    assert_close(z.to_numpy(), xn.astype(np.float64) @ Wn[1], what="a parked product read later")


def test_parked_column_sums_share_a_launch(nd):
    """The bias gradients of a reverse pass over layers of a few thousand rows (functional.reduce_add and the fused layer's
    rule put them off, _lib.park_col_sum) go out as one endia_hip_col_sum_multi call at the end of the pass. Batch 2048 into
    two 1024-wide sin layers: first-order bias gradients are bit for bit those of a pass with the parking off, the
    Hessian-vector product agrees, a sum that is put off outside a pass is launched by whoever reads it, and by an in-place
    writer of its input before that writes."""
    from endia_amd import _lib as L
    from endia_amd import functional as F
    rng = np.random.default_rng(23)
    Bn, Wd = 2048, 1024
    Wn = [(rng.standard_normal((Wd, Wd)) / np.sqrt(Wd)).astype(np.float32) for _ in range(2)]
    bn = [(0.1 * rng.standard_normal(Wd)).astype(np.float32) for _ in range(2)]
    vn = [rng.standard_normal(a.shape).astype(np.float32) for a in (Wn[0], bn[0], Wn[1], bn[1])]
    xn = rng.standard_normal((Bn, Wd)).astype(np.float32)
    seen = []
    raw = L._raw_call

    def spy(name, *args):
        if name == "endia_hip_col_sum_multi":
            seen.append(args[0])
        return raw(name, *args)

    def run():
        mlp = nd.nn.MLP([Wd] * 3, compute_backward=True, activation="sin", fused=True)
        for i in range(2):
            mlp.weights[i], mlp.biases[i] = nd.array(Wn[i], requires_grad=True), nd.array(bn[i], requires_grad=True)
        out = mlp.forward(nd.array(xn))
        loss = nd.sum(out * out)
        loss.backward(create_graph=True)
        assert not L._parked_sums  # the end of the pass launched them
        firsts = [p.grad() for p in mlp.params()]
        hv = nd.grad(outs=firsts, inputs=mlp.params(), grad_outs=[nd.reshape(nd.array(v), f.shape()) for v, f in zip(vn, firsts)])
        assert not L._parked_sums
        res = [f.to_numpy() for f in firsts] + [h.to_numpy() for h in hv]
        loss.zero_grad()
        return res

    L._raw_call = spy
    try:
        parked = run()
        assert seen == [2, 2], "merged calls of the two passes: %r" % (seen,)
        L.defer_products[0] = False
        try:
            plain = run()
        finally:
            L.defer_products[0] = True
        assert seen == [2, 2]
        np.testing.assert_array_equal(parked[1], plain[1])  # first-order bias gradients: the same kernel body either way
        np.testing.assert_array_equal(parked[3], plain[3])
        for k, (a, b) in enumerate(zip(parked, plain)):
            assert_close(a, b, tol=2e-6, mean_tol=1e-4, what="tensor %d with and without parking" % k)
        # outside a pass: the read launches it
        x = nd.array(xn)
        s = F.reduce_add(x, [0])
        assert len(L._parked_sums) == 1
        got = s.to_numpy()
        assert not L._parked_sums and seen[-1] == 1
        ref64 = xn.astype(np.float64).sum(axis=0, keepdims=True)
        assert np.all(np.abs(got - ref64) <= 1e-5 * np.abs(xn).astype(np.float64).sum(axis=0, keepdims=True))
        # an optimizer step writes the summed tensor in place: the sum of the old values goes first
        W = nd.array(xn, requires_grad=True)
        s = F.reduce_add(W, [0])
        assert len(L._parked_sums) == 1
        W.grad_(nd.array(np.ones_like(xn)))
        nd.optim.SGD([W], lr=1.0).step()
        assert not L._parked_sums
        np.testing.assert_array_equal(s.to_numpy(), got)
        np.testing.assert_array_equal(W.to_numpy(), xn - 1.0)
    finally:
        L._raw_call = raw


def test_optimizer_classes(nd, golden):
    g = golden("optim")
    makers = {
        "sgdm": lambda ps: nd.optim.SGD(ps, lr=1e-2, momentum=0.9),
        "sgdmw": lambda ps: nd.optim.SGD(ps, lr=1e-2, momentum=0.9, weight_decay=0.05),
        "sgdw": lambda ps: nd.optim.SGD(ps, lr=1e-2, weight_decay=0.05),
        "adagrad": lambda ps: nd.optim.Adagrad(ps, lr=1e-2, eps=1e-8),
        "rmsprop": lambda ps: nd.optim.RMSprop(ps, lr=1e-2, alpha=0.99, eps=1e-8),
        "adam": lambda ps: nd.optim.Adam(ps, lr=1e-3),
        "sgd": lambda ps: nd.optim.SGD(ps, lr=1e-3),
    }
    for name, mk in makers.items():
        p = nd.array(g["p0"], requires_grad=True)
        opt = mk([p])
        for i in range(3):
            p.grad_(nd.array(g["g%d" % i]))
            opt.step()
            assert_close(p.to_numpy(), g["%s_p%d" % (name, i + 1)], tol=2e-6, what="%s step %d" % (name, i))


@pytest.mark.parametrize("fused", [True, False, "model"])
def test_adam_applied_inside_backward(nd, fused):
    """optim.Adam(fused_backward=True): backward() updates each parameter as soon as its gradient is complete. Three
    steps give bit for bit the parameters, moments and gradients of step() after backward(), for a tanh MLP in every
    fusion mode, with a weight shared by two layers (its update has to wait for both contributions), and a pass with
    create_graph=True does not update anything."""
    rng = np.random.default_rng(17)
    widths = [12, 32, 32, 5]
    Wn = [(rng.standard_normal((widths[i], widths[i + 1])) / np.sqrt(widths[i])).astype(np.float32) for i in range(3)]
    bn = [(0.1 * rng.standard_normal(widths[i + 1])).astype(np.float32) for i in range(3)]
    xn, yn = rng.standard_normal((20, 12)).astype(np.float32), rng.standard_normal((20, 5)).astype(np.float32)

    def run(inside):
        mlp = nd.nn.MLP(widths, compute_backward=True, activation="tanh", fused=fused)
        for i in range(3):
            mlp.weights[i], mlp.biases[i] = nd.array(Wn[i], requires_grad=True), nd.array(bn[i], requires_grad=True)
        opt = nd.optim.Adam(mlp.params(), lr=1e-2, fused_backward=inside)
        x, y = nd.array(xn), nd.array(yn)
        grads = []
        for _ in range(3):
            loss = nd.mse(mlp.forward(x), y)
            loss.backward()
            grads.append([p.grad().to_numpy() for p in mlp.params()])
            opt.step()
            loss.zero_grad()
        return [p.to_numpy() for p in mlp.params()], [m.to_numpy() for m in opt.m + opt.v], grads, opt.t

    p1, s1, g1, t1 = run(True)
    p0, s0, g0, t0 = run(False)
    assert t1 == t0 == 4.0
    for a, b in zip(p1 + s1 + sum(g1, []), p0 + s0 + sum(g0, [])):
        np.testing.assert_array_equal(a, b)
    if fused == "model":
        return
    # one weight used by two layers: updated once, after the second contribution
    W = nd.array(Wn[1], requires_grad=True)
    x = nd.array(rng.standard_normal((20, 32)).astype(np.float32))
    opt = nd.optim.Adam([W], lr=1e-2, fused_backward=True)
    ref_W = nd.array(Wn[1], requires_grad=True)
    ref = nd.optim.Adam([ref_W], lr=1e-2)
    for w, o in ((W, opt), (ref_W, ref)):
        h = nd.tanh(nd.matmul(x, w))
        nd.sum(nd.matmul(h, w)).backward()
        o.step()
    np.testing.assert_array_equal(W.to_numpy(), ref_W.to_numpy())
    # a pass that records its graph leaves the parameters alone
    before = W.to_numpy()
    nd.sum(nd.matmul(x, W)).backward(create_graph=True)
    np.testing.assert_array_equal(W.to_numpy(), before)
    with pytest.raises(ValueError):
        nd.optim.Adam([W], capturable=True, fused_backward=True)


def test_complex_mlp_both_conventions(nd, golden):
    """Identity complex layers, loss = sum |out|^2. `vjp_rule="wirtinger"` gives the Wirtinger-conjugate
    gradients (equal to torch); the default follows the reference's coded rule without conjugation
    (matmul_op.mojo:278-283), checked against the oracle's composition of the same products."""
    from oracle import endia_ref as R
    g = golden("complex_mlp")
    for conj in (True, False):
        Ws = [nd.array(g["W%d" % i], requires_grad=True) for i in range(3)]
        h = nd.array(g["z"])
        for W in Ws:
            h = nd.matmul(h, W, vjp_rule="wirtinger" if conj else "reference")
        loss = nd.sum(nd.square(nd.abs(h)))
        assert_close(h.to_numpy(), g["out"], what="forward")
        assert_close([loss.item()], g["loss"], what="loss")
        loss.backward()
        if conj:
            for i in range(3):
                assert_close(Ws[i].grad().to_numpy(), g["dW%d" % i], what="Wirtinger dW%d" % i)
        else:
            acts = [g["z"]]
            for i in range(3):
                acts.append(R.matmul(acts[-1], g["W%d" % i]))
            delta = 2 * acts[-1]
            for i in (2, 1, 0):
                assert_close(Ws[i].grad().to_numpy(), R.matmul(acts[i].T, delta), what="reference-rule dW%d" % i)
                delta = R.matmul(delta, g["W%d" % i].T)


def test_conv2d_autograd(nd, golden):
    g = golden("conv2d")
    x, w, b = (nd.array(g[k], requires_grad=True) for k in ("x", "w", "b"))
    y = nd.conv2d(x, w, b, stride=2, padding=1)  # the reference's forward test: test_conv2d_op.mojo:54-62
    assert_close(y.to_numpy(), g["s2p1_y"], what="conv2d")
    nd.sum(y * nd.array(g["s2p1_g"])).backward()
    assert_close(x.grad().to_numpy(), g["s2p1_dx"], what="dx")
    assert_close(w.grad().to_numpy(), g["s2p1_dw"], what="dw")
    assert_close(b.grad().to_numpy(), g["s2p1_db"], what="db")
    # relu + mean loss, the benchmark configuration's head
    x2, w2, b2 = (nd.array(g[k], requires_grad=True) for k in ("x", "w", "b"))
    loss = nd.mean(nd.relu(nd.conv2d(x2, w2, b2, stride=1, padding=1)))
    loss.backward()
    import torch
    tx, tw, tb = (torch.tensor(g[k], dtype=torch.float64, requires_grad=True) for k in ("x", "w", "b"))
    tl = torch.relu(torch.nn.functional.conv2d(tx, tw, tb, stride=1, padding=1)).mean()
    tl.backward()
    assert_close([loss.item()], [tl.item()], what="loss")
    assert_close(w2.grad().to_numpy(), tw.grad.numpy(), what="dw")
    assert_close(b2.grad().to_numpy(), tb.grad.numpy(), what="db")
    assert_close(x2.grad().to_numpy(), tx.grad.numpy(), what="dx")


@pytest.mark.parametrize("fused", [True, "model"])
def test_captured_step_matches_eager(nd, golden, fused):
    """The sine-fit MLP step recorded into a HIP graph: every replay must leave exactly the parameters the
    eager step leaves. Replays are interleaved with eager work and synchronisations."""
    g = golden("mlp_sine")

    def build():
        mlp, _ = _load_mlp(nd, g, 8, "relu", fused)
        opt = nd.optim.SGD(mlp.params(), lr=1e-3, momentum=0.9)
        x, y = nd.array(g["x"]), nd.array(g["y"])

        def step():
            loss = nd.mse(mlp.forward(x), y)
            loss.backward()
            opt.step()
            loss.zero_grad()
            return loss
        return mlp, step, x

    mlp_e, step_e, _ = build()
    mlp_c, step_c, x_c = build()
    step_e()
    step_c()                                  # warm-up: pool and workspace sized
    captured = nd.capture(step_c)             # recorded, not executed
    scratch = nd.randn([300, 70])
    for it in range(4):
        loss_e = step_e()
        loss_c = captured.replay()
        nd.synchronize()
        scratch = nd.tanh(scratch @ nd.randn([70, 70]))   # eager work between replays reuses pool buffers
        assert loss_c.item() == loss_e.item(), "replay %d" % it
        for pe, pc in zip(mlp_e.params(), mlp_c.params()):
            np.testing.assert_array_equal(pc.to_numpy(), pe.to_numpy())
    # new input through the fixed buffer
    xb = np.linspace(0, 1, 128, dtype=np.float32).reshape(128, 1)
    x_c.copy_from_numpy(xb)
    before = mlp_c.weights[3].to_numpy()
    captured.replay()
    assert not np.array_equal(mlp_c.weights[3].to_numpy(), before)
    captured.close()
    with pytest.raises(RuntimeError):
        captured.replay()
    # host reads are refused inside a capture, and so is an Adam whose step counter still lives on the host; the
    # failed captures leave the library usable
    with pytest.raises(nd._lib.EndiaHipError, match="captured"):
        nd.capture(lambda: scratch.to_numpy())
    mlp_a, _ = _load_mlp(nd, g, 8, "relu", True)
    adam = nd.optim.Adam(mlp_a.params())
    for p in mlp_a.params():
        p.grad_(nd.zeros(p.shape()))
    with pytest.raises(RuntimeError, match="capturable"):
        nd.capture(adam.step)
    assert nd.sum(nd.ones([5])).item() == 5.0


def test_captured_step_with_split_reductions(nd):
    """A captured step whose products are split along K inside their launches (few tiles per CU, K >= 256): the groups
    of a tile meet through arrival counters that the last arriver puts back to zero, so every replay must give what
    the eager step gives, bit for bit."""
    rng = np.random.default_rng(21)
    x = nd.array(rng.standard_normal((256, 512)).astype(np.float32))
    y = nd.array(rng.standard_normal((256, 512)).astype(np.float32))

    def build():
        r = np.random.default_rng(3)
        mlp = nd.nn.MLP([512, 512, 512], compute_backward=True)
        for prm in mlp.params():
            prm.copy_from_numpy((r.standard_normal(prm.shape()) * 0.04).astype(np.float32))
        return mlp, nd.optim.SGD(mlp.params(), lr=1e-2)

    def make(mlp, opt):
        def step():
            loss = nd.mse(mlp.forward(x), y)
            loss.backward()
            opt.step()
            loss.zero_grad()
            return loss
        return step

    (mlp_e, opt_e), (mlp_c, opt_c) = build(), build()
    step_e, step_c = make(mlp_e, opt_e), make(mlp_c, opt_c)
    step_e()
    step_c()
    captured = nd.capture(step_c)
    for it in range(4):
        loss_e = step_e()
        loss_c = captured.replay()
        assert loss_c.item() == loss_e.item(), "loss at replay %d" % it
        for pe, pc in zip(mlp_e.params(), mlp_c.params()):
            np.testing.assert_array_equal(pc.to_numpy(), pe.to_numpy(), err_msg="parameters at replay %d" % it)
    captured.close()


def test_captured_adam_step(nd, golden):
    """Adam with its step counter in device memory (capturable=True): the captured step, replayed, follows the
    eager host-counter Adam and the oracle's Adam step for step (1e-6: the bias corrections come from the device's
    powf), and the counter advances by one per replay."""
    from oracle import endia_ref as R
    g = golden("mlp_sine")
    mlp_e, _ = _load_mlp(nd, g, 8, "relu", True)
    mlp_c, _ = _load_mlp(nd, g, 8, "relu", True)
    opt_e = nd.optim.Adam(mlp_e.params(), lr=1e-2)
    opt_c = nd.optim.Adam(mlp_c.params(), lr=1e-2, capturable=True)
    x, y = nd.array(g["x"]), nd.array(g["y"])

    def make(mlp, opt):
        def step():
            loss = nd.mse(mlp.forward(x), y)
            loss.backward()
            opt.step()
            loss.zero_grad()
            return loss
        return step

    step_e, step_c = make(mlp_e, opt_e), make(mlp_c, opt_c)
    step_e()
    step_c()                                   # eager, through the device-counter path
    assert opt_c.step_count() == 2.0
    captured = nd.capture(step_c)
    for it in range(5):
        loss_e = step_e()
        loss_c = captured.replay()
        assert_close([loss_c.item()], [loss_e.item()], tol=1e-5, what="loss at replay %d" % it)
        for pe, pc in zip(mlp_e.params(), mlp_c.params()):
            assert_close(pc.to_numpy(), pe.to_numpy(), tol=2e-6, what="parameters at replay %d" % it)
    assert opt_c.step_count() == 7.0 and opt_e.t == 7.0
    captured.close()
    # one tensor, three steps, against the oracle's Adam
    rng = np.random.default_rng(12)
    p0 = rng.standard_normal((37, 5)).astype(np.float32)
    grads = [rng.standard_normal((37, 5)).astype(np.float32) for _ in range(3)]
    p = nd.array(p0, requires_grad=True)
    opt = nd.optim.Adam([p], lr=1e-2, capturable=True)
    pr, m, v = p0.copy(), np.zeros_like(p0), np.zeros_like(p0)
    for i, gr in enumerate(grads):
        p.grad_(nd.array(gr))
        opt.step()
        pr, m, v = R.adam(pr, gr, m, v, lr=1e-2, t=float(i + 1))
        assert_close(p.to_numpy(), pr, tol=1e-6, what="oracle step %d" % i)


def test_shape_errors(nd):
    with pytest.raises(ValueError, match="ndim < 2"):
        nd.matmul(nd.zeros([3]), nd.zeros([3, 3]))
    with pytest.raises(ValueError, match="not compatible"):
        nd.matmul(nd.zeros([2, 3]), nd.zeros([4, 3]))
    with pytest.raises(ValueError, match="complex"):
        nd.relu(nd.zeros([2], is_complex=True))
    with pytest.raises(ValueError, match="4-dimensional"):
        nd.conv2d(nd.zeros([3, 3]), nd.zeros([1, 1, 1, 1]))


@pytest.mark.parametrize("name", ["1d", "2d", "3d", "2d_dil"])
def test_pooling_ops(nd, golden, name):  # test_max_pool2d_op.mojo / test_avg_pool2d_op.mojo and siblings, plus gradients
    g = golden("pool")
    k, st, pad, dil = (tuple(int(v) for v in row) for row in g["cfg_" + name])
    nsp = len(k)
    if nsp == 1:
        k, st, pad, dil = k[0], st[0], pad[0], dil[0]
    for kind in ("max", "avg"):
        if kind + "_" + name not in g.files:
            continue
        x = nd.array(g["x_" + name], requires_grad=True)
        y = getattr(nd, "%s_pool%dd" % (kind, nsp))(x, k, st, pad, dil)
        assert_close(y.to_numpy(), g[kind + "_" + name], what=kind)
        nd.sum(y * nd.array(g["g_" + name])).backward()
        assert_close(x.grad().to_numpy(), g["d" + kind + "_" + name], what=kind + " grad")
    with pytest.raises(ValueError):
        nd.max_pool2d(nd.zeros([2, 3, 4]), (2, 2))


def test_conv1d(nd, golden):  # test_conv1d_op.mojo, plus gradients
    g = golden("convnd")
    st, pad, dil = (int(row[0]) for row in g["cfg_1d"])
    x, w, b = (nd.array(g[k + "_1d"], requires_grad=True) for k in ("x", "w", "b"))
    y = nd.conv1d(x, w, b, st, pad, dil)
    assert_close(y.to_numpy(), g["y_1d"], what="conv1d")
    nd.sum(y * nd.array(g["g_1d"])).backward()
    assert_close(x.grad().to_numpy(), g["dx_1d"], what="dx")
    assert_close(w.grad().to_numpy(), g["dw_1d"], what="dw")
    assert_close(b.grad().to_numpy(), g["db_1d"], what="db")


@pytest.mark.parametrize("name", ["3d", "3d_unit"])
def test_conv3d(nd, golden, name):  # test_conv3d_op.mojo, plus gradients
    g = golden("convnd")
    st, pad, dil = (tuple(int(v) for v in row) for row in g["cfg_" + name])
    x, w, b = (nd.array(g[k + "_" + name], requires_grad=True) for k in ("x", "w", "b"))
    y = nd.conv3d(x, w, b, st, pad, dil)
    assert_close(y.to_numpy(), g["y_" + name], what="conv3d")
    nd.sum(y * nd.array(g["g_" + name])).backward()
    assert_close(x.grad().to_numpy(), g["dx_" + name], what="dx")
    assert_close(w.grad().to_numpy(), g["dw_" + name], what="dw")
    assert_close(b.grad().to_numpy(), g["db_" + name], what="db")
    with pytest.raises(ValueError):
        nd.conv3d(nd.zeros([1, 2, 3, 4]), w)


def test_as_strided(nd, golden):  # test_as_strided_op.mojo: the same two cases
    g = golden("views")
    y = nd.as_strided(nd.array(g["as_x"]), shape=[1, 2, 40, 2, 2], stride=[16, 8, 2, 2, 1], storage_offset=0)
    np.testing.assert_array_equal(y.to_numpy(), g["as_y"])
    arr = nd.array(g["as_x2"], requires_grad=True)
    res = nd.sum(nd.sin(nd.as_strided(arr, shape=[30, 30, 2], stride=[9, 30, 2], storage_offset=0)))
    res.backward()
    assert_close(arr.grad().to_numpy(), g["as_dx2"], what="as_strided grad (overlapping windows)")
    with pytest.raises(ValueError, match="reaches element"):
        nd.as_strided(arr, [30, 30, 2], [90, 30, 2], 0)
    # second order: the gradient of as_strided_inv is as_strided again (as_strided_op.mojo:197-215)
    a = nd.array(g["as_x2"][:4, :3, 0].copy(), requires_grad=True)
    win = nd.as_strided(a, [3, 2, 2], [3, 1, 1], 1)
    (da,) = nd.grad([nd.sum(win * win * win)], [a], create_graph=True)
    (dda,) = nd.grad([nd.sum(da)], [a])
    x = g["as_x2"][:4, :3, 0].astype(np.float64).reshape(-1)
    cnt = np.zeros(12)
    for i in range(3):
        for j in range(2):
            for k in range(2):
                cnt[1 + 3 * i + j + k] += 1
    assert_close(da.to_numpy().reshape(-1), 3 * x * x * cnt, what="first derivative")
    assert_close(dda.to_numpy().reshape(-1), 6 * x * cnt, what="second derivative")


def test_slice_pad_concat(nd, golden):
    g = golden("views")
    x = nd.array(g["sl_x"], requires_grad=True)
    y = x[1:6:2, 2:, ::3]
    assert y.shape() == [3, 7, 4] and not y.is_contiguous()
    np.testing.assert_array_equal(y.to_numpy(), g["sl_y"])
    nd.sum(y * nd.array(g["sl_g"])).backward()
    np.testing.assert_array_equal(x.grad().to_numpy(), g["sl_dx"])
    np.testing.assert_array_equal(nd.array_slice(x, [slice(2, 3)]).to_numpy(), g["sl_x"][2:3])
    np.testing.assert_array_equal(x[-1].to_numpy(), g["sl_x"][-1:])   # an integer keeps its axis

    p = nd.array(g["pad_x"], requires_grad=True)
    big = nd.pad(p, [5, 9], [slice(1, 4), slice(2, 9, 2)])
    np.testing.assert_array_equal(big.to_numpy(), g["pad_y"])
    nd.sum(big * nd.array(g["pad_g"])).backward()
    np.testing.assert_array_equal(p.grad().to_numpy(), g["pad_dx"])
    with pytest.raises(ValueError, match="do not match"):
        nd.pad(p, [5, 9], [slice(0, 4), slice(0, 4)])

    cs = [nd.array(g["cat_%d" % i], requires_grad=True) for i in (1, 2, 3)]
    cat = nd.concat(cs, axis=1)
    np.testing.assert_array_equal(cat.to_numpy(), g["cat_y"])
    nd.sum(cat * nd.array(g["cat_g"])).backward()
    for i, c in enumerate(cs):
        np.testing.assert_array_equal(c.grad().to_numpy(), g["cat_d%d" % (i + 1)])
    np.testing.assert_array_equal(nd.concat(cs, axis=-2).to_numpy(), g["cat_y"])
    with pytest.raises(ValueError, match="Incompatible"):
        nd.concat([cs[0], nd.zeros([2, 3, 5])], axis=1)

    # slices compose with the other ops: a strided block feeds a matmul, gradient flows back through the view
    a = nd.array(g["sl_x"][0], requires_grad=True)             # (9, 10)
    w = nd.array(g["pad_x"].T.copy())                          # (4, 3)
    out = nd.sum(a[1:8:2, 2:6] @ w)
    out.backward()
    want = np.zeros((9, 10), np.float32)
    want[1:8:2, 2:6] = np.ones((4, 3), np.float32) @ g["pad_x"]
    assert_close(a.grad().to_numpy(), want, what="grad through slice and matmul")

    # __setitem__ writes through the view (array or scalar)
    z = nd.zeros([4, 6])
    z[1:3, ::2] = nd.array(np.arange(6, dtype=np.float32).reshape(2, 3))
    z[3, 1:3] = 7.0
    want = np.zeros((4, 6), np.float32)
    want[1:3, ::2] = np.arange(6).reshape(2, 3)
    want[3, 1:3] = 7
    np.testing.assert_array_equal(z.to_numpy(), want)

    # complex arrays move as pairs
    zc = nd.array((g["pad_x"] + 1j * g["pad_x"][::-1]).astype(np.complex64))
    np.testing.assert_array_equal(zc[1:, ::2].to_numpy(), (g["pad_x"] + 1j * g["pad_x"][::-1])[1:, ::2])


@pytest.mark.parametrize("ca,cb", [(0, 0), (0, 1), (1, 0), (1, 1)])
def test_complex_matmul_wirtinger_flags(nd, ca, cb):
    """The Wirtinger rule runs its conjugations as flags of the complex GEMM. For every flag pair the product
    conj^ca(A) conj^cb(B) and both gradients of sum(Re(P) * G) must equal torch's (complex128 autograd)."""
    import torch
    rng = np.random.default_rng(40 + 2 * ca + cb)
    A = (rng.standard_normal((9, 12)) + 1j * rng.standard_normal((9, 12))).astype(np.complex64)
    B = (rng.standard_normal((12, 7)) + 1j * rng.standard_normal((12, 7))).astype(np.complex64)
    G = rng.standard_normal((9, 7)).astype(np.float32)
    ta, tb = (torch.tensor(v, dtype=torch.complex128, requires_grad=True) for v in (A, B))
    tp = (ta.conj() if ca else ta) @ (tb.conj() if cb else tb)
    (tp.real * torch.tensor(G, dtype=torch.float64)).sum().backward()
    a, b = nd.array(A, requires_grad=True), nd.array(B, requires_grad=True)
    p = nd.matmul(a, b, "wirtinger", ca, cb)
    assert_close(p.to_numpy(), tp.detach().resolve_conj().numpy(), what="product")
    nd.sum(nd.real(p) * nd.array(G)).backward()
    assert_close(a.grad().to_numpy(), ta.grad.resolve_conj().numpy(), what="dA")
    assert_close(b.grad().to_numpy(), tb.grad.resolve_conj().numpy(), what="dB")


def test_conv2d_fused_relu_step(nd, golden):
    """conv2d(..., act="relu") under a mean loss (the convolution benchmark's step): the activation runs in the
    kernel's epilogue, and its derivative meets the broadcast mean gradient in one pass. Same numbers as the
    op-by-op composition and as torch; also with an ordinary full-size cotangent."""
    import torch
    g = golden("conv2d")
    tx, tw, tb = (torch.tensor(g[k], dtype=torch.float64, requires_grad=True) for k in ("x", "w", "b"))
    ty = torch.relu(torch.nn.functional.conv2d(tx, tw, tb, stride=1, padding=1))
    ty.mean().backward()
    x, w, b = (nd.array(g[k], requires_grad=True) for k in ("x", "w", "b"))
    y = nd.conv2d(x, w, b, stride=1, padding=1, act="relu")
    assert_close(y.to_numpy(), ty.detach().numpy(), what="relu(conv2d)")
    loss = nd.mean(y)
    loss.backward()
    assert_close([loss.item()], [ty.mean().item()], what="loss")
    assert_close(x.grad().to_numpy(), tx.grad.numpy(), what="dx")
    assert_close(w.grad().to_numpy(), tw.grad.numpy(), what="dw")
    assert_close(b.grad().to_numpy(), tb.grad.numpy(), what="db")
    # a dense cotangent takes the other branch (one relu-gradient kernel on the stored output)
    cot = np.random.default_rng(9).standard_normal(ty.shape).astype(np.float32)
    for t in (tx, tw, tb):
        t.grad = None
    ty2 = torch.relu(torch.nn.functional.conv2d(tx, tw, tb, stride=1, padding=1))
    (ty2 * torch.tensor(cot, dtype=torch.float64)).sum().backward()
    x, w, b = (nd.array(g[k], requires_grad=True) for k in ("x", "w", "b"))
    nd.sum(nd.conv2d(x, w, b, stride=1, padding=1, act="relu") * nd.array(cot)).backward()
    assert_close(x.grad().to_numpy(), tx.grad.numpy(), what="dx (dense cotangent)")
    assert_close(w.grad().to_numpy(), tw.grad.numpy(), what="dw (dense cotangent)")
    with pytest.raises(ValueError, match="act"):
        nd.conv2d(x, w, b, act="tanh")


def test_random_mlps_vs_oracle(nd):
    """Seeded sweep over small MLPs (widths and batches on both sides of the one-launch layer backward's limits,
    1-wide and unaligned layers, every activation, fused and op-by-op): loss and every gradient against the CPU
    oracle's step."""
    from oracle import endia_ref as R
    rng = np.random.default_rng(81)
    widths_pool = [1, 4, 8, 30, 32, 33, 64, 100, 128, 132, 160]
    for case in range(36):
        depth = int(rng.integers(1, 5))
        widths = [int(rng.choice(widths_pool)) for _ in range(depth + 1)]
        batch = int(rng.choice([8, 20, 100, 128, 130, 256]))
        act = ["relu", "tanh", "sin"][case % 3]
        # per-layer fused, op by op, and the whole model as one op (one launch forward, two backward, when every width
        # is at most 128 and the activation is relu or tanh; the per-layer kernels otherwise)
        fused = [True, True, "model", False, "model", True][case % 6]
        Ws = [(rng.standard_normal((widths[i], widths[i + 1])) * np.sqrt(1.0 / widths[i])).astype(np.float32) for i in range(depth)]
        bs = [(rng.standard_normal(widths[i + 1]) * 0.1).astype(np.float32) for i in range(depth)]
        xb = rng.standard_normal((batch, widths[0])).astype(np.float32)
        yb = rng.standard_normal((batch, widths[-1])).astype(np.float32)
        loss_ref, dWr, dbr = R.mlp_step(widths, act, xb, yb, [w.copy() for w in Ws], [b.copy() for b in bs])
        mlp = nd.nn.MLP(widths, compute_backward=True, activation=act, fused=fused)
        for i in range(depth):
            mlp.weights[i] = nd.array(Ws[i], requires_grad=True)
            mlp.biases[i] = nd.array(bs[i], requires_grad=True)
        x, y = nd.array(xb), nd.array(yb)
        loss = nd.mse(mlp.forward(x), y)
        loss.backward()
        what = "case %d: widths %s batch %d %s fused=%s" % (case, widths, batch, act, fused)
        assert_close([loss.item()], [loss_ref], what=what + " loss")
        for i in range(depth):
            assert_close(mlp.weights[i].grad().to_numpy(), dWr[i], what=what + " dW%d" % i)
            assert_close(mlp.biases[i].grad().to_numpy(), dbr[i], tol=2e-4, what=what + " db%d" % i)
        loss.zero_grad()


def test_random_expression_graphs_vs_torch(nd):
    """Seeded random graphs over three leaves: elementwise ops with broadcasting, views (permute, reshape, slices),
    reductions and matmuls, tensors used more than once (gradient accumulation), first and second order. Value and
    every gradient against PyTorch float64 running the same sequence of ops."""
    import torch
    rng = np.random.default_rng(2024)
    unary = [("sin", nd.sin, torch.sin), ("cos", nd.cos, torch.cos), ("tanh", nd.tanh, torch.tanh),
             ("sigmoid", nd.sigmoid, torch.sigmoid), ("square", nd.square, torch.square),
             ("relu", nd.relu, torch.relu), ("neg", nd.neg, torch.neg)]
    for case in range(30):
        m, k, n = (int(rng.choice([3, 8, 17, 32])) for _ in range(3))
        leaves_np = [rng.standard_normal((m, k)), rng.standard_normal((k, n)), rng.standard_normal((n,))]
        leaves_np = [(0.7 * a).astype(np.float32) for a in leaves_np]
        ours = [nd.array(a, requires_grad=True) for a in leaves_np]
        theirs = [torch.tensor(a, dtype=torch.float64, requires_grad=True) for a in leaves_np]
        # pool of (ours, theirs) values of shape [m, n]
        pool = [(nd.matmul(ours[0], ours[1]) + ours[2], torch.matmul(theirs[0], theirs[1]) + theirs[2])]
        trace = ["A@B+c"]
        for _ in range(int(rng.integers(3, 9))):
            kind = int(rng.integers(0, 7))
            a, ta = pool[int(rng.integers(len(pool)))]
            b, tb = pool[int(rng.integers(len(pool)))]
            if kind == 0:
                name, f, tf = unary[int(rng.integers(len(unary)))]
                pool.append((f(a), tf(ta)))
                trace.append(name)
            elif kind == 1:
                op = int(rng.integers(3))
                pool.append(((a + b, a - b, a * b)[op], (ta + tb, ta - tb, ta * tb)[op]))
                trace.append("+-*"[op])
            elif kind == 2:  # division by something bounded away from zero
                pool.append((a / (nd.square(b) + 1.5), ta / (torch.square(tb) + 1.5)))
                trace.append("/")
            elif kind == 3:  # row and column sums broadcast back
                ax = int(rng.integers(2))
                pool.append((a * nd.reduce_add(b, [ax]), ta * tb.sum(dim=ax, keepdim=True)))
                trace.append("bcast-sum%d" % ax)
            elif kind == 4:  # through a transposed view and back
                pool.append((nd.permute(nd.sin(nd.permute(a, [1, 0])), [1, 0]), torch.sin(ta.T).T))
                trace.append("T-sin-T")
            elif kind == 5:  # a slice padded back to the full shape by its gradient only: multiply a sub-block
                r0, c0 = int(rng.integers(0, m - 1)), int(rng.integers(0, n - 1))
                sub, tsub = a[r0:, c0:], ta[r0:, c0:]
                pool.append((a * nd.mean(nd.tanh(sub)), ta * torch.tanh(tsub).mean()))
                trace.append("slice-mean")
            else:  # another product through the leaves: (a^T a) scaled into [m, n] via A B
                g_, tg = nd.matmul(nd.permute(a, [1, 0]), b), torch.matmul(ta.T, tb)       # [n, n]
                pool.append((nd.matmul(a, nd.tanh(g_) * (1.0 / n)), torch.matmul(ta, torch.tanh(tg) / n)))
                trace.append("a@tanh(a^T b)")
        out, tout = pool[-1]
        for extra, textra in pool[:-1][::2]:  # tie earlier nodes in, so no branch of the graph is dead
            out, tout = out + 0.1 * extra, tout + 0.1 * textra
        loss, tloss = nd.sum(nd.square(out)) / float(m * n), torch.square(tout).sum() / (m * n)
        what = "case %d (%s)" % (case, " ".join(trace))
        second = case % 3 == 0
        if second:  # gradient of the squared gradient norm w.r.t. the first leaf, i.e. a double backward
            loss.backward(create_graph=True)
            tg0, = torch.autograd.grad(tloss, theirs[0], create_graph=True)
            g0 = ours[0].grad()
            loss.zero_grad()  # drop the first pass's stored gradients everywhere, as grad() does (functional.mojo:77-82)
            loss2, tloss2 = nd.sum(nd.square(g0)), torch.square(tg0).sum()
            loss2.backward()
            tloss2.backward()
            assert_close([loss2.item()], [tloss2.item()], tol=2e-4, what=what + " squared gradient norm")
        else:
            loss.backward()
            tloss.backward()
            assert_close([loss.item()], [tloss.item()], what=what + " value")
        for i, (lf, tl) in enumerate(zip(ours, theirs)):
            want = tl.grad.numpy() if tl.grad is not None else np.zeros(lf.shape())
            assert_close(lf.grad().to_numpy().reshape(want.shape), want, tol=5e-4 if second else 1e-4, what=what + " grad of leaf %d" % i)


def test_initialisers(nd):
    """The rest of init_ops.mojo: shapes, the values that are fixed (zeros/ones/eye/fill/linspace), and for the random
    schemes the scale the fan sizes fix (he: sqrt(2/fan_in), sqrt(6/fan_in); xavier: sqrt(2/(in+out)), sqrt(6/(in+out));
    lecun: sqrt(1/fan_in), sqrt(3/fan_in); init_ops.mojo:285-416). The draws themselves are time-seeded in the reference
    and cannot be compared."""
    base = nd.array(np.arange(24, dtype=np.float32).reshape(2, 3, 4), requires_grad=True)
    for made, want in ((nd.zeros_like(base), 0.0), (nd.ones_like(base), 1.0), (nd.fill_like(base, 2.5), 2.5)):
        assert made.shape() == [2, 3, 4] and made.requires_grad()
        np.testing.assert_array_equal(made.to_numpy(), np.full((2, 3, 4), want, np.float32))
    np.testing.assert_array_equal(nd.eye_like(base).to_numpy(), np.broadcast_to(np.eye(3, 4, dtype=np.float32), (2, 3, 4)))
    np.testing.assert_array_equal(nd.linspace(0.0, 1.0, 5).to_numpy(), np.float32([0, 0.25, 0.5, 0.75, 1.0]))
    # (the grid crosses zero at its 223rd point, which is 1e-16 in float64 and 1e-7 in float32: that one element alone
    # puts the mean relative figure at 1e-3, so it is given its own bound; the L2 bound stays 1e-4)
    assert_close(nd.linspace(-2.0, 7.0, 1000).to_numpy(), np.linspace(-2.0, 7.0, 1000), what="linspace", mean_tol=2e-3)

    work = nd.array(np.arange(12, dtype=np.float32).reshape(3, 4))
    before = work.data_ptr()
    for fn, want in ((nd.ones_, 1.0), (nd.zeros_, 0.0), (lambda a: nd.fill_(a, -3.0), -3.0)):
        assert fn(work) is work and work.data_ptr() == before
        np.testing.assert_array_equal(work.to_numpy(), np.full((3, 4), want, np.float32))
    cz = nd.fill_(nd.complex(nd.ones([2, 2]), nd.ones([2, 2])), 4.0)
    np.testing.assert_array_equal(cz.to_numpy(), np.full((2, 2), 4.0, np.complex64))
    with pytest.raises(ValueError):
        nd.fill_(nd.permute(work, [1, 0]), 1.0)

    nd.seed(5)
    big = nd.zeros([400, 500])
    draw = nd.randu_(big, -2.0, 6.0).to_numpy()
    assert draw.min() >= -2.0 and draw.max() <= 6.0 and abs(draw.mean() - 2.0) < 0.05
    draw = nd.randn_(big, 1.0, 3.0).to_numpy()
    assert abs(draw.mean() - 1.0) < 0.05 and abs(draw.std() - 3.0) < 0.05
    assert nd.randu_like(big).shape() == [400, 500] and nd.randn_like(big).shape() == [400, 500]

    fan_in, fan_out = 50.0, 30.0
    normal = {"rand_he_normal": (np.sqrt(2 / fan_in), (fan_in,)), "rand_lecun_normal": (np.sqrt(1 / fan_in), (fan_in,)),
              "rand_xavier_normal": (np.sqrt(2 / (fan_in + fan_out)), (fan_in, fan_out))}
    uniform = {"rand_he_uniform": (np.sqrt(6 / fan_in), (fan_in,)), "rand_lecun_uniform": (np.sqrt(3 / fan_in), (fan_in,)),
               "rand_xavier_uniform": (np.sqrt(6 / (fan_in + fan_out)), (fan_in, fan_out))}
    for name, (scale, fans) in list(normal.items()) + list(uniform.items()):
        for draw in (getattr(nd, name)([400, 500], *fans).to_numpy(), getattr(nd, name + "_like")(big, *fans).to_numpy(),
                     getattr(nd, name + "_")(big, *fans).to_numpy()):
            assert draw.shape == (400, 500) and abs(draw.mean()) < 0.02 * scale * 3
            if name in normal:
                assert abs(draw.std() / scale - 1.0) < 0.02, name
            else:  # uniform on (-limit, limit): bounded, and std = limit / sqrt(3)
                assert np.abs(draw).max() <= scale and abs(draw.std() * np.sqrt(3) / scale - 1.0) < 0.02, name


def test_jit_follows_the_eager_callable(nd):
    """nd.jit over a function and over value_and_grad(function) (the reference's examples/benchmarks use both:
    endia/compile/functional.mojo:43-88): every call must return what the eager callable returns for the same inputs,
    bit for bit, on fresh arrays, also after the inputs change and for a second input shape; results of earlier
    calls stay what they were."""
    rng = np.random.default_rng(77)

    def foo(args):
        h = nd.tanh(nd.matmul(args[0], args[1]) + args[2])
        return nd.sum(h * h)

    eager = nd.value_and_grad(foo)
    fast = nd.jit(nd.value_and_grad(foo), compile_with_MAX=False)
    plain = nd.jit(foo)
    kept = []
    for shape in ((16, 24, 8), (16, 24, 8), (5, 7, 3), (16, 24, 8)):
        m, k, n = shape
        args = [nd.array(rng.standard_normal(s).astype(np.float32)) for s in ((m, k), (k, n), (n,))]
        want, got = eager(args), fast(args)
        assert [len(group) for group in got] == [1, 3]  # [[value], [three gradients]]
        want, got = want[0] + want[1], got[0] + got[1]
        for w, g in zip(want, got):
            np.testing.assert_array_equal(g.to_numpy(), w.to_numpy())
        np.testing.assert_array_equal(plain(args).to_numpy(), want[0].to_numpy())
        kept.append((got, [w.to_numpy() for w in want]))
    for got, want in kept:  # a later call does not write into an earlier call's results
        for g, w in zip(got, want):
            np.testing.assert_array_equal(g.to_numpy(), w)
    assert len(fast._cache) == 2

    def reads_the_device(args):
        return nd.sum(args[0]) * float(args[0].item())

    with pytest.raises(RuntimeError, match="captured"):
        nd.jit(reads_the_device)([nd.ones([4])])
    nd.sum(nd.ones([4])).item()  # the library is usable after the failed capture
    with pytest.raises(NotImplementedError):
        nd.jit(foo, compile_with_MAX=True)
    fast.close()
    plain.close()


@pytest.mark.parametrize("act", ["tanh", "relu", "sin"])
def test_jacobian_and_hessian_through_fused_layers(nd, act):
    """A non-scalar output seeds backward with an identity Jacobian (autograd/functional.mojo:35-37), so every VJP
    rule sees a cotangent with leading axes; the last pass of a hessian sees two sets of them. The fused dense layer
    must give what the reference's matmul -> add -> activation chain gives (and what torch float64 gives)."""
    import torch
    rng = np.random.default_rng(5)
    B, dims = 3, [4, 6, 5, 2]
    Ws = [(rng.standard_normal((dims[i], dims[i + 1])) / np.sqrt(dims[i])).astype(np.float32) for i in range(3)]
    bs = [(0.1 * rng.standard_normal(dims[i + 1])).astype(np.float32) for i in range(3)]
    x0 = rng.standard_normal((B, dims[0])).astype(np.float32)

    def model(fused):
        m = nd.nn.MLP(dims, compute_backward=True, activation=act, fused=fused)
        for i in range(3):
            m.weights[i], m.biases[i] = nd.array(Ws[i], requires_grad=True), nd.array(bs[i], requires_grad=True)
        return m

    tact = {"tanh": torch.tanh, "relu": torch.relu, "sin": torch.sin}[act]

    def tf(x):
        h = x
        for i in range(3):
            h = h @ torch.tensor(Ws[i], dtype=torch.float64) + torch.tensor(bs[i], dtype=torch.float64)
            if i < 2:
                h = tact(h)
        return h

    xt = torch.tensor(x0, dtype=torch.float64)
    jac_ref = torch.autograd.functional.jacobian(tf, xt).numpy()                       # [B, 2, B, 4]
    hes_ref = torch.autograd.functional.hessian(lambda x: (tf(x) ** 2).sum(), xt).numpy()  # [B, 4, B, 4]
    for fused in (True, False):
        m = model(fused)
        jac = nd.jacobian(lambda x: m.forward(x))(nd.array(x0))
        assert jac.shape() == [B, 2, B, 4]
        assert_close(jac.to_numpy(), jac_ref, what="jacobian fused=%s %s" % (fused, act))
        hes = nd.hessian(lambda x: nd.sum(m.forward(x) ** 2))(nd.array(x0))
        assert hes.shape() == [B, 4, B, 4]
        assert_close(hes.to_numpy(), hes_ref, what="hessian fused=%s %s" % (fused, act))
    # parameter Jacobians: leading axes on dW (matmul's batch) and on db (the layer's batch axis is summed, not axis 0)
    m = model(True)
    x = nd.array(x0)
    out = m.forward(x)
    out.backward()
    Wt = [torch.tensor(w, dtype=torch.float64, requires_grad=True) for w in Ws]
    bt = [torch.tensor(b, dtype=torch.float64, requires_grad=True) for b in bs]

    def tparams(*p):
        h = xt
        for i in range(3):
            h = h @ p[2 * i] + p[2 * i + 1]
            if i < 2:
                h = tact(h)
        return h

    flat = [t for pair in zip(Wt, bt) for t in pair]
    refs = torch.autograd.functional.jacobian(tparams, tuple(flat))
    for i, (p, r) in enumerate(zip(m.params(), refs)):
        got = p.grad().to_numpy()
        assert got.size == r.numel(), (i, got.shape, tuple(r.shape))
        assert_close(got.reshape(tuple(r.shape)), r.numpy(), what="parameter %d Jacobian" % i)
    with pytest.raises(NotImplementedError):  # ops without such a rule refuse instead of reading the wrong elements
        xc = nd.array(rng.standard_normal((1, 2, 5, 5)).astype(np.float32), requires_grad=True)
        nd.conv2d(xc, nd.array(rng.standard_normal((3, 2, 3, 3)).astype(np.float32))).backward()


@pytest.mark.parametrize("act", ["tanh", "relu", "sin"])
def test_hidden_activation_gradients_of_fused_layers(nd, act):
    """The fused backward hands dL/dh * act'(h) from one layer's dx GEMM to the layer below; what h.grad() and
    grad(outs, inputs=[h]) return must still be dL/dh, as in the op-by-op chain, and the parameter gradients must
    not change when a hidden gradient is read."""
    rng = np.random.default_rng(9)
    B, dims = 16, [8, 32, 24, 4]
    Ws = [(rng.standard_normal((dims[i], dims[i + 1])) / np.sqrt(dims[i])).astype(np.float32) for i in range(3)]
    bs = [(0.1 * rng.standard_normal(dims[i + 1])).astype(np.float32) for i in range(3)]
    x0 = rng.standard_normal((B, dims[0])).astype(np.float32)
    y0 = rng.standard_normal((B, dims[-1])).astype(np.float32)
    afn = {"tanh": nd.tanh, "relu": nd.relu, "sin": nd.sin}[act]

    def run(fused):
        W = [nd.array(w, requires_grad=True) for w in Ws]
        b = [nd.array(v, requires_grad=True) for v in bs]
        h, hidden = nd.array(x0), []
        for i in range(3):
            if fused:
                h = nd.linear(h, W[i], b[i], act if i < 2 else None)
            else:
                h = h @ W[i] + b[i]
                h = afn(h) if i < 2 else h
            if i < 2:
                hidden.append(h)
        loss = nd.mse(h, nd.array(y0))
        return loss, hidden, W, b

    loss_f, hid_f, W_f, b_f = run(True)
    loss_u, hid_u, W_u, b_u = run(False)
    loss_f.backward()
    loss_u.backward()
    for hf, hu in zip(hid_f, hid_u):
        assert hf.has_grad()
        assert_close(hf.grad().to_numpy(), hu.grad().to_numpy(), what="dL/dh of a fused hidden layer (%s)" % act)
    for pf, pu in zip(W_f + b_f, W_u + b_u):
        assert_close(pf.grad().to_numpy().reshape(-1), pu.grad().to_numpy().reshape(-1), what="parameter gradient")
    # the functional form on a fresh graph
    loss_f, hid_f, _, _ = run(True)
    got = nd.grad(outs=[loss_f], inputs=hid_f)
    for g, hu in zip(got, hid_u):
        assert_close(g.to_numpy(), hu.grad().to_numpy(), what="grad(outs, inputs=[h]) (%s)" % act)
    if act == "sin":
        # the fused sin layer keeps its pre-activation as a node of its own: its gradient is dL/dz = dL/dh * cos(z)
        loss_f, hid_f, _, _ = run(True)
        loss_f.backward()
        for hf, hu in zip(hid_f, hid_u):
            z = hf.args()[0]
            zu = hu.args()[0]
            assert_close(z.grad().to_numpy(), zu.grad().to_numpy(), what="dL/dz of a fused sin layer")
    # a hidden gradient is computed on first use with the layer's weights: after an in-place update it refuses
    loss_f, hid_f, W_f, b_f = run(True)
    loss_f.backward()
    early = hid_f[1].grad().to_numpy()          # read before the step: fine, and kept
    nd.optim.SGD(W_f + b_f, lr=0.1).step()
    np.testing.assert_array_equal(hid_f[1].grad().to_numpy(), early)
    with pytest.raises(RuntimeError, match="updated in place"):
        hid_f[0].grad()
    loss_f.zero_grad()
    assert not hid_f[0].has_grad()


def test_callable_mixed_argnums(nd):
    """grad(grad(f, argnums=[0]), argnums=[1]) is the cross derivative: every order differentiates with respect to
    its own arguments (callable.mojo:105-110,146-151). Checked against torch float64."""
    import torch
    rng = np.random.default_rng(21)
    a0, b0 = rng.standard_normal(5).astype(np.float32), rng.standard_normal(5).astype(np.float32)

    def f(args):
        return nd.sum(nd.sin(args[0] * args[1]) + args[0] * args[0] * args[1])

    def tf(a, b):
        return (torch.sin(a * b) + a * a * b).sum()

    at, bt = torch.tensor(a0, dtype=torch.float64), torch.tensor(b0, dtype=torch.float64)
    H = torch.autograd.functional.hessian(tf, (at, bt))
    args = [nd.array(a0), nd.array(b0)]
    d_ab = nd.grad(nd.grad(f, argnums=[0]), argnums=[1])(args)   # d/db of df/da: [5, 5]
    assert_close(d_ab.to_numpy(), H[0][1].numpy(), what="d2f / da db")
    d_aa = nd.hessian(f, argnums=[0])(args)
    assert_close(d_aa.to_numpy(), H[0][0].numpy(), what="d2f / da da")
    d_ba = nd.grad(nd.grad(f, argnums=[1]), argnums=[0])(args)
    assert_close(d_ba.to_numpy(), H[1][0].numpy(), what="d2f / db da")
    both = nd.grad(f)(args)  # -1: every argument
    ga, gb = torch.autograd.grad(tf(at.requires_grad_(), bt.requires_grad_()), (at, bt))
    assert_close(both[0].to_numpy(), ga.numpy(), what="df/da")
    assert_close(both[1].to_numpy(), gb.numpy(), what="df/db")
    # value_and_grad of a second-order callable keeps every order: [[value], [df/da], [d2f/da db]]
    nested = nd.value_and_grad(nd.grad(f, argnums=[0]), argnums=[1])(args)
    assert [len(g) for g in nested] == [1, 1, 1]
    assert_close(nested[0][0].to_numpy(), [float(tf(at, bt))], what="value")
    assert_close(nested[1][0].to_numpy(), ga.numpy(), what="first order kept")
    assert_close(nested[2][0].to_numpy(), H[0][1].numpy(), what="second order")


def test_whole_model_mse_loss_op(nd):
    """functional.mlp_mse_loss (endia_hip_mlp_fwd_mse: the forward launch also evaluates the MSE loss and its gradient; the
    work-groups' partial sums meet at a ticket) against mse(per-layer forward) + backward: loss and every gradient for
    ragged shapes, a frozen parameter, many row groups, the input's gradient, a cotangent other than the seed, three calls
    in a row bit-identical (the ticket is back at zero), and what it refuses."""
    rng = np.random.default_rng(321)
    for widths, batch, act in [([1, 32, 64, 128, 128, 128, 64, 32, 1], 128, "relu"), ([7, 50, 3, 128, 20], 37, "tanh"),
                               ([128, 128], 16, None), ([5, 17], 1, "relu"), ([3, 8, 2], 1000, "relu"), ([40, 100, 9], 5000, "tanh")]:
        Lyr = len(widths) - 1
        Wn = [(rng.standard_normal((widths[i], widths[i + 1])) / np.sqrt(widths[i])).astype(np.float32) for i in range(Lyr)]
        bn = [(0.2 * rng.standard_normal(widths[i + 1])).astype(np.float32) for i in range(Lyr)]
        xn = rng.standard_normal((batch, widths[0])).astype(np.float32)
        tn = rng.standard_normal((batch, widths[-1])).astype(np.float32)

        def run(whole, scale=None):
            x, t = nd.array(xn, requires_grad=True), nd.array(tn)
            W = [nd.array(w, requires_grad=(i != 1)) for i, w in enumerate(Wn)]  # the second weight matrix is frozen
            b = [nd.array(v, requires_grad=True) for v in bn]
            if whole:
                loss = nd.mlp_mse_loss(x, t, W, b, act)
            else:
                out = x
                for i in range(Lyr):
                    out = nd.linear(out, W[i], b[i], act if i < Lyr - 1 else None)
                loss = nd.mse(out, t)
            (loss if scale is None else loss * scale).backward()
            grads = [x.grad().to_numpy()] + [w.grad().to_numpy() for w in W if w.has_grad()] + [v.grad().to_numpy().reshape(-1) for v in b]
            assert not W[1].has_grad() if Lyr > 1 else True
            return loss.to_numpy(), grads

        what = "widths %s batch %d %s: " % (widths, batch, act)
        for scale in (None, 3.0):
            l_w, g_w = run(True, scale)
            l_l, g_l = run(False, scale)
            assert_close(l_w, l_l, tol=1e-5, what=what + "loss")
            assert len(g_w) == len(g_l)
            for k, (a, b_) in enumerate(zip(g_w, g_l)):
                assert_close(a, b_, tol=2e-5, mean_tol=1e-3, what=what + "gradient %d" % k)  # (mean metric: a few values sum to ~0)
        l_w, g_w = run(True)
        for _ in range(2):
            l_2, g_2 = run(True)
            np.testing.assert_array_equal(l_2, l_w)
            for a, b_ in zip(g_2, g_w):
                np.testing.assert_array_equal(a, b_)
    # through the model class, and the cases the op does not cover
    mlp = nd.nn.MLP([4, 16, 2], compute_backward=True, fused="model")
    x, t = nd.array(xn[:8, :4].copy()), nd.array(tn[:8, :2].copy())
    a = mlp.mse_loss(x, t)
    b_ = nd.mse(mlp.forward(x), t)
    assert_close(a.to_numpy(), b_.to_numpy(), tol=1e-6, what="MLP.mse_loss")
    with pytest.raises(NotImplementedError):
        a.backward(create_graph=True)
    wide = nd.nn.MLP([4, 200, 2], compute_backward=True, fused="model")  # too wide for the fused launch: the per-layer route
    assert_close(wide.mse_loss(x, t).to_numpy(), nd.mse(wide.forward(x), t).to_numpy(), tol=1e-6, what="wide model")


def test_mse_of_a_whole_model_forward_is_one_launch(nd):
    """mse(mlp.forward(x), y), the reference script's two calls (mlp_imp.mojo:56-60), on a whole-model MLP: the forward
    launch is parked and mse() turns it into the launch that also evaluates the loss and all cotangents. Same loss,
    gradients, output values and output gradient as the per-layer model; reading the output first, a target that needs a
    gradient, or a second consumer of the output all still work; a captured step replays it."""
    from endia_amd import _lib as L
    rng = np.random.default_rng(5)
    widths = [3, 32, 64, 2]
    Wn = [(rng.standard_normal((widths[i], widths[i + 1])) / np.sqrt(widths[i])).astype(np.float32) for i in range(3)]
    bn = [(0.2 * rng.standard_normal(widths[i + 1])).astype(np.float32) for i in range(3)]
    xn, yn = rng.standard_normal((40, 3)).astype(np.float32), rng.standard_normal((40, 2)).astype(np.float32)

    def model(fused):
        mlp = nd.nn.MLP(widths, compute_backward=True, activation="relu", fused=fused)
        for i in range(3):
            mlp.weights[i], mlp.biases[i] = nd.array(Wn[i], requires_grad=True), nd.array(bn[i], requires_grad=True)
        return mlp

    ref = model(True)
    out_r = ref.forward(nd.array(xn))
    loss_r = nd.mse(out_r, nd.array(yn))
    loss_r.backward()
    for variant in ("plain", "read_first", "target_grad", "two_consumers"):
        mlp = model("model")
        x, y = nd.array(xn), nd.array(yn, requires_grad=(variant == "target_grad"))
        calls = []
        orig = L._raw_call
        L._raw_call = lambda name, *a: (calls.append(name), orig(name, *a))[1]
        try:
            out = mlp.forward(x)
            assert L._parked and not [c for c in calls if c.startswith("endia_hip_mlp")]
            if variant == "read_first":
                first = out.to_numpy()
            loss = nd.mse(out, y)
            if variant == "two_consumers":
                loss = loss + nd.sum(out) * 0.0
            loss.backward()
        finally:
            L._raw_call = orig
        launches = [c for c in calls if c.startswith("endia_hip_mlp")]
        if variant == "plain":
            assert launches == ["endia_hip_mlp_fwd_mse_delta", "endia_hip_mlp_wgrad"], launches
        elif variant in ("read_first", "target_grad"):
            assert launches[0] == "endia_hip_mlp_fwd", launches
        assert_close(loss.to_numpy(), loss_r.to_numpy(), tol=1e-6, what=variant + ": loss")
        assert_close(out.to_numpy(), out_r.to_numpy(), tol=1e-6, what=variant + ": output")
        for p, q in zip(mlp.params(), ref.params()):
            assert_close(p.grad().to_numpy().reshape(-1), q.grad().to_numpy().reshape(-1), tol=2e-5, mean_tol=1e-3, what=variant + ": gradient")
        if variant == "plain":
            assert_close(out.grad().to_numpy(), out_r.grad().to_numpy(), tol=1e-6, what="gradient of the model's output")
    # captured and replayed
    mlp = model("model")
    opt = nd.optim.SGD(mlp.params(), lr=0.05)
    x, y = nd.array(xn), nd.array(yn)

    def step():
        loss = nd.mse(mlp.forward(x), y)
        loss.backward()
        opt.step()
        loss.zero_grad()
        return loss

    eager = [float(step().item()) for _ in range(2)]
    cap = nd.capture(step)
    assert not L._parked
    replayed = [float(cap.replay().item()) for _ in range(3)]
    assert eager[1] < eager[0] and replayed[0] < eager[1] and replayed[2] < replayed[1]
    cap.close()


def test_whole_model_forward_with_cotangents_entry_points(nd):
    """endia_hip_mlp_fwd_mse_delta + endia_hip_mlp_wgrad through the C ABI against endia_hip_mlp_fwd_mse +
    endia_hip_mlp_bwd: the same loss, activations, cotangents of every layer, dx, dW and db, bit for bit (the chain is
    the same arithmetic whether it runs in the forward launch or in its own), on both sides of the 2048-row switch, with
    and without dx, with gradients that are not asked for, and twice in a row."""
    import ctypes
    from endia_amd import _lib as L
    from endia_amd._array import Array
    rng = np.random.default_rng(77)
    act_code = {None: L.OP_IDENTITY, "relu": L.OP_RELU, "tanh": L.OP_TANH}
    for widths, batch, act, want_dx in [([1, 32, 64, 128, 128, 128, 64, 32, 1], 128, "relu", False), ([7, 50, 3, 128, 20], 37, "tanh", True),
                                        ([128, 128], 16, None, True), ([5, 17], 1, "relu", False), ([33, 128, 65, 12], 1024, "tanh", True),
                                        ([33, 128, 65, 12], 2048, "relu", True), ([33, 128, 65, 12], 2500, "relu", True), ([6, 9, 4], 3, "relu", True)]:
        Lyr = len(widths) - 1
        W = [nd.array((rng.standard_normal((widths[i], widths[i + 1])) / np.sqrt(widths[i])).astype(np.float32)) for i in range(Lyr)]
        b = [nd.array((0.2 * rng.standard_normal(widths[i + 1])).astype(np.float32)) for i in range(Lyr)]
        x = nd.array(rng.standard_normal((batch, widths[0])).astype(np.float32))
        t = nd.array(rng.standard_normal((batch, widths[-1])).astype(np.float32))
        desc = L.MlpDesc()
        desc.layers, desc.act, desc.batch = Lyr, act_code[act], batch
        desc.widths[:Lyr + 1] = widths
        ptrs = lambda arrs: (ctypes.c_void_p * Lyr)(*[a.data_ptr() if a is not None else None for a in arrs])
        new = lambda shape: Array.empty(list(shape))

        def two_calls():
            h = [new([batch, widths[i + 1]]) for i in range(Lyr)]
            delta = [new([batch, widths[i + 1]]) for i in range(Lyr)]
            dW = [new([widths[i], widths[i + 1]]) if i != 1 else None for i in range(Lyr)]  # the second dW is not asked for
            db = [new([widths[i + 1]]) for i in range(Lyr)]
            dx, loss = (new([batch, widths[0]]) if want_dx else None), new([1])
            L.call("endia_hip_mlp_fwd_mse", ctypes.byref(desc), x.data_ptr(), ptrs(W), ptrs(b), t.data_ptr(), ptrs(h), delta[-1].data_ptr(), loss.data_ptr())
            L.call("endia_hip_mlp_bwd", ctypes.byref(desc), x.data_ptr(), ptrs(W), ptrs(h), ptrs(delta), ptrs(dW), ptrs(db), dx.data_ptr() if dx else None)
            return [loss] + h + delta + [a for a in dW if a is not None] + db + ([dx] if dx else [])

        def fused():
            h = [new([batch, widths[i + 1]]) for i in range(Lyr)]
            delta = [new([batch, widths[i + 1]]) for i in range(Lyr)]
            dW = [new([widths[i], widths[i + 1]]) if i != 1 else None for i in range(Lyr)]
            db = [new([widths[i + 1]]) for i in range(Lyr)]
            dx, loss = (new([batch, widths[0]]) if want_dx else None), new([1])
            L.call("endia_hip_mlp_fwd_mse_delta", ctypes.byref(desc), x.data_ptr(), ptrs(W), ptrs(b), t.data_ptr(), ptrs(h), ptrs(delta), loss.data_ptr(),
                   dx.data_ptr() if dx else None)
            L.call("endia_hip_mlp_wgrad", ctypes.byref(desc), x.data_ptr(), ptrs(h), ptrs(delta), ptrs(dW), ptrs(db))
            return [loss] + h + delta + [a for a in dW if a is not None] + db + ([dx] if dx else [])

        ref = [a.to_numpy() for a in two_calls()]
        for _ in range(2):  # the loss sum meets at a ticket: the same bits on every call
            again = [a.to_numpy() for a in two_calls()]
            for k, (g, r) in enumerate(zip(again, ref)):
                np.testing.assert_array_equal(g, r, err_msg="widths %s batch %d %s: tensor %d differs between runs" % (widths, batch, act, k))
        for _ in range(3):
            got = [a.to_numpy() for a in fused()]
            assert len(got) == len(ref)
            for k, (g, r) in enumerate(zip(got, ref)):
                np.testing.assert_array_equal(g, r, err_msg="widths %s batch %d %s: tensor %d" % (widths, batch, act, k))
    # arguments the entry points refuse
    with pytest.raises(Exception):
        L.call("endia_hip_mlp_fwd_mse_delta", ctypes.byref(desc), x.data_ptr(), ptrs(W), ptrs(b), t.data_ptr(), ptrs(W), None, x.data_ptr(), None)


def test_whole_model_entry_points_want_aligned_arrays(nd):
    """Everything but the weights is read and written 16 bytes at a time: an activation, bias or cotangent array that
    starts 4 bytes off a 16-byte boundary is refused by the entry points, and the ops send such views down the
    per-layer route instead."""
    import ctypes
    from endia_amd import _lib as L
    from endia_amd._array import Array
    rng = np.random.default_rng(80)
    widths, batch = [8, 16, 4], 6
    W = [nd.array(rng.standard_normal((widths[i], widths[i + 1])).astype(np.float32)) for i in range(2)]
    b = [nd.array(rng.standard_normal(widths[i + 1]).astype(np.float32)) for i in range(2)]
    x = nd.array(rng.standard_normal((batch, 8)).astype(np.float32))
    desc = L.MlpDesc()
    desc.layers, desc.act, desc.batch = 2, L.OP_RELU, batch
    desc.widths[:3] = widths
    ptrs = lambda ps: (ctypes.c_void_p * 2)(*ps)
    big = Array.empty([batch * 16 + 4])
    h_ok = [Array.empty([batch, 16]), Array.empty([batch, 4])]
    L.call("endia_hip_mlp_fwd", ctypes.byref(desc), x.data_ptr(), ptrs([w.data_ptr() for w in W]), ptrs([v.data_ptr() for v in b]),
           ptrs([h.data_ptr() for h in h_ok]))
    with pytest.raises(L.EndiaHipError, match="16-byte"):
        L.call("endia_hip_mlp_fwd", ctypes.byref(desc), x.data_ptr(), ptrs([w.data_ptr() for w in W]), ptrs([v.data_ptr() for v in b]),
               ptrs([big.data_ptr() + 4, h_ok[1].data_ptr()]))
    # the op: a bias that is a view one float into its buffer
    raw = nd.array(np.concatenate([[0.0], b[0].to_numpy()]).astype(np.float32))
    odd = raw[1:]
    assert odd._offset == 1
    got = nd.mlp_forward(x, W, [odd, b[1]], "relu").to_numpy()
    want = nd.mlp_forward(x, W, b, "relu").to_numpy()
    assert_close(got, want, tol=1e-6, what="bias view with an odd offset")


def test_whole_model_large_batch_repeats_bit_for_bit(nd):
    """65 536 rows of four 128-wide layers: the weight gradients are summed over 64 row slices by a second launch and
    the loss over 4096 work-groups that meet at a ticket. Three runs of forward + loss + chain + gradients give the
    same bits (fixed order of every sum), and the gradients match float64."""
    import ctypes
    from endia_amd import _lib as L
    from endia_amd._array import Array
    rng = np.random.default_rng(79)
    widths, batch = [128] * 5, 65536
    Lyr = 4
    Wn = [(rng.standard_normal((128, 128)) / np.sqrt(128)).astype(np.float32) for _ in range(Lyr)]
    bn = [(0.2 * rng.standard_normal(128)).astype(np.float32) for _ in range(Lyr)]
    xn = rng.standard_normal((batch, 128)).astype(np.float32)
    tn = rng.standard_normal((batch, 128)).astype(np.float32)
    W, b, x, t = [nd.array(w) for w in Wn], [nd.array(v) for v in bn], nd.array(xn), nd.array(tn)
    desc = L.MlpDesc()
    desc.layers, desc.act, desc.batch = Lyr, L.OP_TANH, batch
    desc.widths[:Lyr + 1] = widths
    ptrs = lambda arrs: (ctypes.c_void_p * Lyr)(*[a.data_ptr() for a in arrs])

    def run():
        h = [Array.empty([batch, 128]) for _ in range(Lyr)]
        delta = [Array.empty([batch, 128]) for _ in range(Lyr)]
        dW, db = [Array.empty([128, 128]) for _ in range(Lyr)], [Array.empty([128]) for _ in range(Lyr)]
        loss = Array.empty([1])
        L.call("endia_hip_mlp_fwd_mse_delta", ctypes.byref(desc), x.data_ptr(), ptrs(W), ptrs(b), t.data_ptr(), ptrs(h), ptrs(delta),
               loss.data_ptr(), None)
        L.call("endia_hip_mlp_wgrad", ctypes.byref(desc), x.data_ptr(), ptrs(h), ptrs(delta), ptrs(dW), ptrs(db))
        return [loss.to_numpy()] + [a.to_numpy() for a in dW + db]

    first = run()
    for _ in range(2):
        for k, (g, r) in enumerate(zip(run(), first)):
            np.testing.assert_array_equal(g, r, err_msg="tensor %d differs between runs" % k)
    # float64 chain rule on the host
    hs = [xn.astype(np.float64)]
    for i in range(Lyr):
        z = hs[-1] @ Wn[i].astype(np.float64) + bn[i]
        hs.append(np.tanh(z) if i < Lyr - 1 else z)
    d = 2.0 * (hs[-1] - tn) / tn.size
    assert_close(first[0], [np.mean((hs[-1] - tn) ** 2)], tol=1e-5, what="loss")
    for i in reversed(range(Lyr)):
        assert_close(first[1 + i], hs[i].T @ d, what="dW%d" % i)
        assert_close(first[1 + Lyr + i], d.sum(0), what="db%d" % i)
        if i:
            d = (d @ Wn[i].astype(np.float64).T) * (1.0 - hs[i] ** 2)


def test_whole_model_entry_points_unaligned_and_deep(nd):
    """The whole-model entry points against float64 numpy (the chain rule written out) where the per-layer comparison
    does not reach: weight matrices that start 4 bytes off a 16-byte boundary (the cotangent chain then reads W element
    by element), and the deepest model the entry points take (16 layers: every LDS row block of the forward launch)."""
    import ctypes
    from endia_amd import _lib as L
    from endia_amd._array import Array
    rng = np.random.default_rng(78)
    for widths, batch, act, off in [([12, 40, 128, 24, 8], 50, "tanh", 1), ([12, 40, 128, 24, 8], 2100, "relu", 1),
                                    ([8] * 17, 10, "tanh", 0), ([128] * 17, 9, "relu", 0)]:
        Lyr = len(widths) - 1
        Wn = [(rng.standard_normal((widths[i], widths[i + 1])) / np.sqrt(widths[i])).astype(np.float32) for i in range(Lyr)]
        bn = [(0.2 * rng.standard_normal(widths[i + 1])).astype(np.float32) for i in range(Lyr)]
        xn = rng.standard_normal((batch, widths[0])).astype(np.float32)
        tn = rng.standard_normal((batch, widths[-1])).astype(np.float32)
        # weights inside larger buffers, `off` floats past their start
        Wbuf = [nd.array(np.concatenate([np.zeros(off, np.float32), w.reshape(-1)])) for w in Wn]
        Wp = [wb.data_ptr() + 4 * off for wb in Wbuf]
        b = [nd.array(v) for v in bn]
        x, t = nd.array(xn), nd.array(tn)
        desc = L.MlpDesc()
        desc.layers, desc.act, desc.batch = Lyr, {"relu": L.OP_RELU, "tanh": L.OP_TANH}[act], batch
        desc.widths[:Lyr + 1] = widths
        vp = lambda ps: (ctypes.c_void_p * Lyr)(*ps)
        ptrs = lambda arrs: vp([a.data_ptr() for a in arrs])
        h = [Array.empty([batch, widths[i + 1]]) for i in range(Lyr)]
        delta = [Array.empty([batch, widths[i + 1]]) for i in range(Lyr)]
        dW = [Array.empty([widths[i], widths[i + 1]]) for i in range(Lyr)]
        db = [Array.empty([widths[i + 1]]) for i in range(Lyr)]
        dx, loss = Array.empty([batch, widths[0]]), Array.empty([1])
        L.call("endia_hip_mlp_fwd_mse_delta", ctypes.byref(desc), x.data_ptr(), vp(Wp), ptrs(b), t.data_ptr(), ptrs(h), ptrs(delta), loss.data_ptr(),
               dx.data_ptr())
        L.call("endia_hip_mlp_wgrad", ctypes.byref(desc), x.data_ptr(), ptrs(h), ptrs(delta), ptrs(dW), ptrs(db))
        # float64: h_l = act(h_{l-1} W_l + b_l) (none after the last layer), loss = mean((h_L - t)^2)
        f = (lambda z: np.maximum(z, 0)) if act == "relu" else np.tanh
        slope = (lambda o: (o > 0).astype(np.float64)) if act == "relu" else (lambda o: 1 - o * o)
        hs = [xn.astype(np.float64)]
        for i in range(Lyr):
            z = hs[-1] @ Wn[i].astype(np.float64) + bn[i]
            hs.append(z if i == Lyr - 1 else f(z))
        d = 2 * (hs[-1] - tn) / tn.size
        what = "widths %s batch %d %s offset %d: " % (widths[:5], batch, act, off)
        assert_close(loss.to_numpy(), [np.mean((hs[-1] - tn) ** 2)], tol=1e-5, what=what + "loss")
        for i in reversed(range(Lyr)):
            assert_close(delta[i].to_numpy(), d, tol=2e-5, mean_tol=1e-3, what=what + "delta %d" % i)
            assert_close(dW[i].to_numpy(), hs[i].T @ d, tol=2e-5, mean_tol=1e-3, what=what + "dW %d" % i)
            assert_close(db[i].to_numpy(), d.sum(0), tol=2e-5, mean_tol=1e-3, what=what + "db %d" % i)
            d = d @ Wn[i].astype(np.float64).T
            if i > 0:
                d = d * slope(hs[i])
        assert_close(dx.to_numpy(), d, tol=2e-5, mean_tol=1e-3, what=what + "dx")
        for i in range(Lyr):
            assert_close(h[i].to_numpy(), hs[i + 1], tol=1e-5, what=what + "h %d" % i)


def test_whole_model_mlp_op(nd):
    """functional.mlp_forward through the C ABI's endia_hip_mlp_fwd / endia_hip_mlp_bwd: the same numbers as the
    per-layer path for ragged widths and batches (rows and columns that do not fill an MFMA block), batches on both
    sides of the switch from four to sixteen rows per work-group (2048 rows), the input gradient, a parameter that
    needs no gradient, two calls in a row (bit-identical), and the cases it refuses."""
    rng = np.random.default_rng(123)
    for widths, batch, act in [([1, 32, 64, 128, 128, 128, 64, 32, 1], 128, "relu"), ([7, 50, 3, 128, 20], 37, "tanh"),
                               ([128, 128], 16, None), ([5, 17], 1, "relu"), ([40, 100, 100, 9], 300, "relu"),
                               ([33, 128, 65, 12], 2048, "tanh"), ([33, 128, 65, 12], 2500, "relu")]:
        Lyr = len(widths) - 1
        Wn = [(rng.standard_normal((widths[i], widths[i + 1])) / np.sqrt(widths[i])).astype(np.float32) for i in range(Lyr)]
        bn = [(0.2 * rng.standard_normal(widths[i + 1])).astype(np.float32) for i in range(Lyr)]
        xn = rng.standard_normal((batch, widths[0])).astype(np.float32)
        gn = rng.standard_normal((batch, widths[-1])).astype(np.float32)

        def run(whole):
            x = nd.array(xn, requires_grad=True)
            W = [nd.array(w, requires_grad=(i != 1)) for i, w in enumerate(Wn)]  # the second weight matrix is frozen
            b = [nd.array(v, requires_grad=True) for v in bn]
            if whole:
                out = nd.mlp_forward(x, W, b, act)
            else:
                out = x
                for i in range(Lyr):
                    out = nd.linear(out, W[i], b[i], act if i < Lyr - 1 else None)
            nd.sum(out * nd.array(gn)).backward()
            grads = [x.grad().to_numpy()] + [w.grad().to_numpy() for w in W if w.has_grad()] + [v.grad().to_numpy().reshape(-1) for v in b]
            assert not W[1].has_grad() if Lyr > 1 else True
            return out.to_numpy(), grads

        out_w, g_w = run(True)
        out_l, g_l = run(False)
        what = "widths %s batch %d %s: " % (widths, batch, act)
        assert_close(out_w, out_l, tol=1e-5, what=what + "output")
        assert len(g_w) == len(g_l)
        for k, (a, b_) in enumerate(zip(g_w, g_l)):
            assert_close(a, b_, tol=2e-5, mean_tol=1e-3, what=what + "gradient %d" % k)  # (mean metric: a few values sum to ~0)
        out_2, g_2 = run(True)
        np.testing.assert_array_equal(out_2, out_w)
        for a, b_ in zip(g_2, g_w):
            np.testing.assert_array_equal(a, b_)
    # wider layers, sin, or complex operands take the per-layer kernels; second-order passes are refused
    wide = nd.mlp_forward(nd.ones([4, 200]), [nd.ones([200, 8])], [nd.zeros([8])], "relu")
    np.testing.assert_array_equal(wide.to_numpy(), np.full((4, 8), 200.0, np.float32))
    x = nd.array(xn[:8, :4].copy(), requires_grad=True)
    y = nd.sum(nd.mlp_forward(x, [nd.array(np.ones((4, 3), np.float32), requires_grad=True)], [nd.zeros([3])], "relu"))
    with pytest.raises(NotImplementedError):
        y.backward(create_graph=True)
