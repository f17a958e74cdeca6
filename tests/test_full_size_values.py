"""Every gradient tensor of the benchmark configurations, at the benchmark shapes, against float64 on the host.

The device runs the configuration through the public API (the path bench.py times); the host repeats it in
float64 (complex128) with torch's CPU GEMMs, which at these sizes takes seconds. Each tensor must agree to 1e-4 in
both metrics of assert_close (relative L2 and the reference's mean relative error); observed differences are the
fp32 round-off of the device's arithmetic, 1e-7 ... 1e-5.
"""
import numpy as np
import pytest

from conftest import assert_close

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def nd():
    import endia_amd
    from endia_amd import _lib
    # The device context is created BEFORE torch does any work: torch's wheel carries a HIP runtime of its own, its
    # autograd engine asks that copy for a device count, and of two runtimes in one process only the first to open
    # the GPU driver gets the device (the other then reports that no device exists).
    _lib.ensure_init()
    return endia_amd


@pytest.fixture(scope="module")
def torch(nd):
    import torch as t
    return t


def test_wide_mlp_every_gradient_at_full_size(nd, torch):
    """Batch 4096, 8 layers 4096 -> 4096 with bias, tanh between, MSE, one Adam step: the headline configuration.
    The forward GEMMs run the bias + tanh epilogue and the data-gradient GEMMs the tanh' epilogue of the 256 x 256
    tile, so this is also the value check of those epilogues at 4096^3."""
    n, layers = 4096, 8
    rng = np.random.default_rng(200)
    Ws = [(rng.standard_normal((n, n)) / np.sqrt(n)).astype(np.float32) for _ in range(layers)]
    bs = [(rng.standard_normal(n) / np.sqrt(n)).astype(np.float32) for _ in range(layers)]
    x = rng.standard_normal((n, n)).astype(np.float32)
    t = rng.standard_normal((n, n)).astype(np.float32)

    mlp = nd.nn.MLP([n] * (layers + 1), compute_backward=True, activation="tanh", fused=True)
    for i in range(layers):
        mlp.weights[i] = nd.array(Ws[i], requires_grad=True)
        mlp.biases[i] = nd.array(bs[i], requires_grad=True)
    opt = nd.optim.Adam(mlp.params(), lr=1e-3)
    loss = nd.mse(mlp.forward(nd.array(x)), nd.array(t))
    loss.backward()
    got_loss = float(loss.item())
    got_dW = [w.grad().to_numpy() for w in mlp.weights]
    got_db = [b.grad().to_numpy().reshape(-1) for b in mlp.biases]
    opt.step()
    got_W = [w.to_numpy() for w in mlp.weights]
    got_b = [b.to_numpy() for b in mlp.biases]
    del mlp, opt, loss

    f64 = torch.float64
    W64 = [torch.tensor(w, dtype=f64) for w in Ws]
    b64 = [torch.tensor(b, dtype=f64) for b in bs]
    acts = [torch.tensor(x, dtype=f64)]
    for i in range(layers):
        z = acts[-1] @ W64[i] + b64[i]
        acts.append(torch.tanh(z) if i < layers - 1 else z)
    diff = acts[-1] - torch.tensor(t, dtype=f64)
    assert_close([got_loss], [float((diff * diff).mean())], tol=1e-5, what="loss")
    delta = 2.0 * diff / diff.numel()

    def adam_first_step(p, g):  # zero moments, t = 1: m_hat = g, v_hat = g^2 (adam.mojo:47-65)
        return p - 1e-3 * g / (g.abs() + 1e-8)

    for i in reversed(range(layers)):
        dW = acts[i].t() @ delta
        db = delta.sum(dim=0)
        assert_close(got_dW[i], dW.numpy(), what="dW of layer %d" % i)
        assert_close(got_db[i], db.numpy(), what="db of layer %d" % i)
        # The update is lr * g / (|g| + eps): where |g| is far above eps (all but a few weights) it is +-lr, so the
        # parameters after the step are checked against the float64 rule applied to the DEVICE's gradient
        assert_close(got_W[i], adam_first_step(W64[i], torch.tensor(got_dW[i], dtype=f64)).numpy(), tol=1e-6,
                     what="W of layer %d after Adam" % i)
        assert_close(got_b[i], adam_first_step(b64[i], torch.tensor(got_db[i], dtype=f64)).numpy(), tol=1e-6,
                     what="b of layer %d after Adam" % i)
        if i:
            delta = (delta @ W64[i].t()) * (1.0 - acts[i] * acts[i])


def test_hvp_every_tensor_at_full_size(nd, torch):
    """Batch 1024, 4 layers 2048 wide, sin, loss sum(out^2): gradient and Hessian-vector product of all 8 parameter
    tensors against torch's double backward in float64."""
    B, n, layers = 1024, 2048, 4
    rng = np.random.default_rng(201)
    Ws = [(rng.standard_normal((n, n)) / np.sqrt(n)).astype(np.float32) for _ in range(layers)]
    bs = [(rng.standard_normal(n) / np.sqrt(n)).astype(np.float32) for _ in range(layers)]
    vW = [rng.standard_normal((n, n)).astype(np.float32) for _ in range(layers)]
    vb = [rng.standard_normal(n).astype(np.float32) for _ in range(layers)]
    x = rng.standard_normal((B, n)).astype(np.float32)

    f64 = torch.float64
    tW = [torch.tensor(w, dtype=f64, requires_grad=True) for w in Ws]
    tb = [torch.tensor(b, dtype=f64, requires_grad=True) for b in bs]
    h = torch.tensor(x, dtype=f64)
    for i in range(layers):
        h = h @ tW[i] + tb[i]
        if i < layers - 1:
            h = torch.sin(h)
    tloss = (h * h).sum()
    params = [p for pair in zip(tW, tb) for p in pair]
    vecs = [torch.tensor(v, dtype=f64) for pair in zip(vW, vb) for v in pair]
    grads = torch.autograd.grad(tloss, params, create_graph=True)
    s = sum((g * v).sum() for g, v in zip(grads, vecs))
    hv_ref = torch.autograd.grad(s, params)

    # H v sums thousands of products of either sign, so some of its 4 M entries per tensor are thousands of times
    # smaller than the typical one, and the reference's metric (mean of |error| / |value|) is carried by those: ANY
    # float32 evaluation exceeds 1e-4 in it here. Its bound is therefore taken from torch's own float32 CPU run of the
    # same computation (twice its figure, at least 1e-4); the relative L2 bound stays 1e-4.
    from conftest import mean_rel
    f32 = torch.float32
    sW = [torch.tensor(w, dtype=f32, requires_grad=True) for w in Ws]
    sb = [torch.tensor(b, dtype=f32, requires_grad=True) for b in bs]
    hs = torch.tensor(x, dtype=f32)
    for i in range(layers):
        hs = hs @ sW[i] + sb[i]
        if i < layers - 1:
            hs = torch.sin(hs)
    sparams = [p for pair in zip(sW, sb) for p in pair]
    sgrads = torch.autograd.grad((hs * hs).sum(), sparams, create_graph=True)
    hv_f32 = torch.autograd.grad(sum((g * v.to(f32)).sum() for g, v in zip(sgrads, vecs)), sparams)
    bound1 = [max(1e-4, 2 * mean_rel(a.detach().numpy().reshape(-1), r.detach().numpy().reshape(-1))) for a, r in zip(sgrads, grads)]
    bound2 = [max(1e-4, 2 * mean_rel(a.numpy().reshape(-1), r.numpy().reshape(-1))) for a, r in zip(hv_f32, hv_ref)]
    print("mean-relative bounds from the float32 CPU run: gradient %s, H v %s" % (["%.1e" % b for b in bound1], ["%.1e" % b for b in bound2]))

    # fused / per-op layers; the second pass from the scalar <gradients, v> or seeded with v (grad_outs)
    for fused, seeded in ((True, True), (True, False), (False, False)):
        mlp = nd.nn.MLP([n] * (layers + 1), compute_backward=True, activation="sin", fused=fused)
        for i in range(layers):
            mlp.weights[i] = nd.array(Ws[i], requires_grad=True)
            mlp.biases[i] = nd.array(bs[i], requires_grad=True)
        out = mlp.forward(nd.array(x))
        loss = nd.sum(out * out)
        loss.backward(create_graph=True)
        first = [p.grad().to_numpy() for p in mlp.params()]
        firsts = [p.grad() for p in mlp.params()]
        vs_dev = [nd.reshape(nd.array(v), f.shape()) for f, v in zip(firsts, [v for pair in zip(vW, vb) for v in pair])]
        if seeded:
            hv = [a.to_numpy() for a in nd.grad(outs=firsts, inputs=mlp.params(), grad_outs=vs_dev)]
        else:
            total = None
            for f, v in zip(firsts, vs_dev):
                term = nd.sum(f * v)
                total = term if total is None else total + term
            hv = [a.to_numpy() for a in nd.grad(outs=total, inputs=mlp.params())]
        assert_close([float(loss.item())], [float(tloss)], tol=1e-5, what="loss")
        loss.zero_grad()
        for i, (g1, g2, r1, r2) in enumerate(zip(first, hv, grads, hv_ref)):
            name = "%s of layer %d (fused=%s, seeded=%s)" % ("W" if i % 2 == 0 else "b", i // 2, fused, seeded)
            assert_close(g1.reshape(-1), r1.detach().numpy().reshape(-1), what="gradient, " + name, mean_tol=bound1[i])
            assert_close(g2.reshape(-1), r2.numpy().reshape(-1), what="H v, " + name, mean_tol=bound2[i])
            print("%s: H v mean-relative %.2e (bound %.1e)" % (name, mean_rel(g2.reshape(-1), r2.numpy().reshape(-1)), bound2[i]))


@pytest.mark.parametrize("algo", ["4m", "3m"])
def test_complex_mlp_every_gradient_at_full_size(nd, torch, algo):
    """Batch 2048, 4 complex layers 2048 -> 2048, identity, loss sum |out|^2, under both VJP rules: the Wirtinger
    rule against torch's complex128 autograd, and the reference's coded rule without conjugation
    (matmul_op.mojo:278-283: dA = g B^T, dB = A^T g, seeded with 2 z by its abs / square rules) against the same
    products in complex128."""
    n, layers = 2048, 4
    rng = np.random.default_rng(202)

    def crandn(scale):
        return ((rng.standard_normal((n, n)) + 1j * rng.standard_normal((n, n))) * scale).astype(np.complex64)

    Ws = [crandn(1.0 / np.sqrt(n)) for _ in range(layers)]
    z = crandn(1.0)
    c128 = torch.complex128
    tW = [torch.tensor(w, dtype=c128, requires_grad=True) for w in Ws]
    acts = [torch.tensor(z, dtype=c128)]
    for w in tW:
        acts.append(acts[-1] @ w)
    tloss = (acts[-1].abs() ** 2).sum()
    wirtinger = torch.autograd.grad(tloss, tW)
    with torch.no_grad():
        literal, delta = [None] * layers, 2.0 * acts[-1]
        for i in reversed(range(layers)):
            literal[i] = acts[i].transpose(0, 1) @ delta
            delta = delta @ tW[i].transpose(0, 1)

    nd.set_complex_matmul_algorithm(algo)
    try:
        for rule, refs in (("wirtinger", wirtinger), ("reference", literal)):
            Wd = [nd.array(w, requires_grad=True) for w in Ws]
            h = nd.array(z)
            for w in Wd:
                h = nd.matmul(h, w, vjp_rule=rule)
            loss = nd.sum(nd.square(nd.abs(h)))
            loss.backward()
            assert_close([float(loss.item())], [float(tloss)], tol=1e-5, what="loss")
            assert_close(h.to_numpy(), acts[-1].detach().numpy(), what="forward (%s)" % algo)
            for i in range(layers):
                assert_close(Wd[i].grad().to_numpy(), refs[i].detach().numpy(), what="%s-rule dW%d (%s)" % (rule, i, algo))
            loss.zero_grad()
    finally:
        nd.set_complex_matmul_algorithm("4m")


def test_conv2d_every_gradient_at_full_size(nd, torch):
    """x [64,64,56,56], w [128,64,3,3], bias, stride 1, pad 1, ReLU, mean loss: the output and dX, dW, db in full
    against torch's float64 convolution and autograd; with and without the ReLU fused into the convolution."""
    rng = np.random.default_rng(203)
    x = rng.standard_normal((64, 64, 56, 56)).astype(np.float32)
    w = (rng.standard_normal((128, 64, 3, 3)) * np.sqrt(2.0 / (64 * 9))).astype(np.float32)
    b = (rng.standard_normal(128) * 0.1).astype(np.float32)
    f64 = torch.float64
    tx, tw, tb = (torch.tensor(a, dtype=f64, requires_grad=True) for a in (x, w, b))
    tz = torch.nn.functional.conv2d(tx, tw, tb, stride=1, padding=1)
    z64 = tz.detach().numpy()
    for fused in (True, False):
        dx_, dw_, db_ = nd.array(x, requires_grad=True), nd.array(w, requires_grad=True), nd.array(b, requires_grad=True)
        if fused:
            y = nd.conv2d(dx_, dw_, db_, stride=1, padding=1, act="relu")
        else:
            y = nd.relu(nd.conv2d(dx_, dw_, db_, stride=1, padding=1))
        loss = nd.mean(y)
        loss.backward()
        tag = " (fused relu)" if fused else " (separate relu)"
        yv = y.to_numpy()
        assert_close(yv, np.maximum(z64, 0.0), what="relu(conv2d)" + tag)
        assert_close([float(loss.item())], [float(np.maximum(z64, 0.0).mean())], tol=1e-5, what="mean loss" + tag)
        # ReLU's derivative is a step: where the pre-activation is within float32 round-off of zero, a float32 and a
        # float64 evaluation may land on different sides, and each such element moves the gradients by a whole term.
        # Those elements are counted and must all be round-off cases; the float64 gradients are then taken through
        # the DEVICE's mask, so that what is compared is the arithmetic, not the tie-breaking.
        mask = yv > 0
        flipped = mask != (z64 > 0)
        assert flipped.sum() <= 100 and np.all(np.abs(z64[flipped]) <= 1e-5), (int(flipped.sum()), tag)
        for t in (tx, tw, tb):
            t.grad = None
        tz.backward(torch.tensor(mask / float(mask.size), dtype=f64), retain_graph=True)
        assert_close(dx_.grad().to_numpy(), tx.grad.numpy(), what="dX" + tag)
        assert_close(dw_.grad().to_numpy(), tw.grad.numpy(), what="dW" + tag)
        assert_close(db_.grad().to_numpy().reshape(-1), tb.grad.numpy(), what="db" + tag)
        loss.zero_grad()
