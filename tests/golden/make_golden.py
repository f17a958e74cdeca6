"""Writes the golden fixtures of this directory with PyTorch float64 on the CPU.

PyTorch float64 is the oracle of the reference's own tests (every test converts to float64 torch
tensors and compares: endia/utils/array_conversions.mojo:41-135, e.g.
tests/test_endia/test_functional/test_binary_ops/test_matmul_op.mojo:18-59); the reference itself is
Mojo and cannot run here, and it ships no fixture files. Inputs are seeded, shapes follow the
reference's tests ((2,30,40) @ (40,50), ...). Run:  python tests/golden/make_golden.py [fixture names]
(every fixture is always computed, so the random stream is the same; only the named ones are written).
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
torch.manual_seed(0)
rng = np.random.default_rng(1234)


def f32(*shape, scale=1.0):
    return (rng.standard_normal(shape) * scale).astype(np.float32)


def c64(*shape):
    return (rng.standard_normal(shape) + 1j * rng.standard_normal(shape)).astype(np.complex64)


def t64(a, grad=False):
    dt = torch.complex128 if np.iscomplexobj(a) else torch.float64
    return torch.tensor(a, dtype=dt, requires_grad=grad)


def save(name, **arrays):
    if len(sys.argv) > 1 and name not in sys.argv[1:]:
        return
    # expected values are stored rounded to fp32 / complex64: 6e-8 relative, far below the 1e-4 gate
    arrays = {k: (v.astype(np.complex64) if np.iscomplexobj(v) else v.astype(np.float32)) if v.size > 1 else v
              for k, v in arrays.items()}
    np.savez_compressed(os.path.join(HERE, name + ".npz"), **arrays)
    print("wrote", name, {k: v.shape for k, v in arrays.items()})


# ---- matmul: forward, gradients of sum(matmul) (test_matmul_op.mojo:18-75) ------------------------
a, b = f32(2, 30, 40), f32(40, 50)
ta, tb = t64(a, True), t64(b, True)
out = torch.matmul(ta, tb)
out.sum().backward()
ca, cb = c64(2, 30, 40), c64(40, 50)
cout = torch.matmul(t64(ca), t64(cb))
# square case (the shape class of dX = dY W^T in the MLP configs)
sa, sb, sg = f32(64, 64), f32(64, 64), f32(64, 64)
tsa, tsb = t64(sa, True), t64(sb, True)
(torch.matmul(tsa, tsb) * t64(sg)).sum().backward()
save("matmul", a=a, b=b, out=out.detach().numpy(), da=ta.grad.numpy(), db=tb.grad.numpy(), ca=ca, cb=cb,
     cout=cout.numpy(), sa=sa, sb=sb, sg=sg, dsa=tsa.grad.numpy(), dsb=tsb.grad.numpy())

# ---- complex matmul gradients under the Wirtinger-conjugate convention (what torch computes) -------
za, zb = c64(6, 10), c64(10, 8)
tza, tzb = t64(za, True), t64(zb, True)
(torch.matmul(tza, tzb).abs() ** 2).sum().backward()
save("cmatmul_grad", za=za, zb=zb, dza=tza.grad.numpy(), dzb=tzb.grad.numpy())

# ---- elementwise: forward and gradient of sum(op(x)) (test_relu_op.mojo, test_tanh_op.mojo, ...) ----
x = f32(2, 30, 40)
xp = np.abs(x) + 0.1
d = {"x": x, "xp": xp}
for name, fn, src in [("relu", torch.relu, x), ("tanh", torch.tanh, x), ("sin", torch.sin, x), ("cos", torch.cos, x),
                      ("neg", torch.neg, x), ("square", torch.square, x), ("sqrt", torch.sqrt, xp),
                      ("abs", torch.abs, x)]:
    t = t64(src, True)
    y = fn(t)
    y.sum().backward()
    d[name] = y.detach().numpy()
    d["d" + name] = t.grad.numpy()
save("unary", **d)

# ---- binary with broadcasting and their gradients (test_add_op.mojo:34-60, test_mul_op.mojo:34-59) ---
a, b = f32(2, 30, 40), f32(30, 40)
b2 = np.abs(b) + 0.5
d = {"a": a, "b": b, "b2": b2}
for name, fn, rhs in [("add", torch.add, b), ("sub", torch.sub, b), ("mul", torch.mul, b), ("div", torch.div, b2)]:
    ta, tb = t64(a, True), t64(rhs, True)
    y = fn(ta, tb)
    torch.sin(y).sum().backward()
    d[name] = y.detach().numpy()
    d[name + "_da"] = ta.grad.numpy()
    d[name + "_db"] = tb.grad.numpy()
ca, cb = c64(3, 5), c64(5)
d.update(ca=ca, cb=cb, cmul=(t64(ca) * t64(cb)).numpy(), cdiv=(t64(ca) / t64(cb)).numpy(),
         cadd=(t64(ca) + t64(cb)).numpy())
save("binary", **d)

# ---- reductions (test_reduce_add_op.mojo:18-55, test_mean_op.mojo:18-55, test_expand_op.mojo:18-52) ---
x = f32(2, 30, 40)
t = t64(x, True)
r = torch.sum(t, dim=(0, 2), keepdim=True)
torch.sin(r).sum().backward()
t2 = t64(x, True)
m = torch.mean(t2, dim=(1,))
torch.sin(m).sum().backward()
bsrc = f32(40)
t3 = t64(bsrc, True)
e = t3.expand(2, 30, 40)
(e * t64(x)).sum().backward()
save("reduce", x=x, sum02=r.detach().numpy(), dsum02=t.grad.numpy(), mean1=m.detach().numpy(), dmean1=t2.grad.numpy(),
     total=np.array([x.astype(np.float64).sum()]), bsrc=bsrc, dexpand=t3.grad.numpy())

# ---- mse + gradient (loss_ops/mse_op.mojo:17-20; no reference test) ----------------------------------
p, tg = f32(16, 8), f32(16, 8)
tp = t64(p, True)
loss = torch.nn.functional.mse_loss(tp, t64(tg))
loss.backward()
save("mse", pred=p, target=tg, loss=np.array([loss.item()]), dpred=tp.grad.numpy())

# ---- conv2d forward (test_conv2d_op.mojo:18-67: stride 2, pad 1) and gradients ------------------------
x, w, bb = f32(2, 3, 9, 10), f32(4, 3, 3, 2), f32(4)
d = {"x": x, "w": w, "b": bb}
for tag, st, pd, dl in [("s2p1", (2, 2), (1, 1), (1, 1)), ("s1p1", (1, 1), (1, 1), (1, 1)), ("s2p2d2", (2, 1), (2, 0), (2, 1))]:
    tx, tw, tb = t64(x, True), t64(w, True), t64(bb, True)
    y = torch.nn.functional.conv2d(tx, tw, tb, stride=st, padding=pd, dilation=dl)
    g = f32(*y.shape)
    (y * t64(g)).sum().backward()
    d.update({tag + "_y": y.detach().numpy(), tag + "_g": g, tag + "_dx": tx.grad.numpy(), tag + "_dw": tw.grad.numpy(),
              tag + "_db": tb.grad.numpy()})
save("conv2d", **d)

# ---- optimizers against torch.optim (optim/sgd.mojo:61-62, optim/adam.mojo:47-65; no reference test) ----
p0 = f32(50, 7)
gs = [f32(50, 7, scale=0.1) for _ in range(3)]
d = {"p0": p0, "g0": gs[0], "g1": gs[1], "g2": gs[2]}
for name, mk in [("sgd", lambda q: torch.optim.SGD([q], lr=1e-3)),
                 ("adam", lambda q: torch.optim.Adam([q], lr=1e-3, betas=(0.9, 0.999), eps=1e-8))]:
    q = t64(p0, True)
    opt = mk(q)
    for i, g in enumerate(gs):
        q.grad = t64(g)
        opt.step()
        d["%s_p%d" % (name, i + 1)] = q.detach().numpy().copy()
for name, mk in [("sgdm", lambda q: torch.optim.SGD([q], lr=1e-2, momentum=0.9)),
                 ("sgdmw", lambda q: torch.optim.SGD([q], lr=1e-2, momentum=0.9, weight_decay=0.05)),
                 ("sgdw", lambda q: torch.optim.SGD([q], lr=1e-2, weight_decay=0.05)),
                 ("adagrad", lambda q: torch.optim.Adagrad([q], lr=1e-2, eps=1e-8)),
                 ("rmsprop", lambda q: torch.optim.RMSprop([q], lr=1e-2, alpha=0.99, eps=1e-8))]:
    q = t64(p0, True)
    opt = mk(q)
    for i, g in enumerate(gs):
        q.grad = t64(g)
        opt.step()
        d["%s_p%d" % (name, i + 1)] = q.detach().numpy().copy()
save("optim", **d)

# ---- the reference's sine-fit MLP, three SGD steps (benchmarks/mlp_benchmarks/mlp_imp.mojo:25-75) -----
widths = [1, 32, 64, 128, 128, 128, 64, 32, 1]
xb = rng.uniform(0, 1, (128, 1)).astype(np.float32)
yb = np.sin(2 * np.pi * xb).astype(np.float32)
Ws = [f32(widths[i], widths[i + 1], scale=np.sqrt(2.0 / widths[i])) for i in range(8)]
bs = [f32(widths[i + 1], scale=np.sqrt(2.0 / widths[i])) for i in range(8)]
d = {"x": xb, "y": yb}
for i in range(8):
    d["W%d" % i], d["b%d" % i] = Ws[i], bs[i]
tW = [t64(W, True) for W in Ws]
tb_ = [t64(b, True) for b in bs]
opt = torch.optim.SGD(tW + tb_, lr=1e-3)
for step in range(3):
    h = t64(xb)
    for i in range(8):
        h = h @ tW[i] + tb_[i]
        if i < 7:
            h = torch.relu(h)
    loss = torch.nn.functional.mse_loss(h, t64(yb))
    opt.zero_grad()
    loss.backward()
    if step == 0:
        for i in range(8):
            d["dW%d" % i], d["db%d" % i] = tW[i].grad.numpy().copy(), tb_[i].grad.numpy().copy()
    d["loss%d" % step] = np.array([loss.item()])
    opt.step()
for i in range(8):
    d["W%d_after" % i], d["b%d_after" % i] = tW[i].detach().numpy(), tb_[i].detach().numpy()
save("mlp_sine", **d)

# ---- tanh MLP + Adam, small cousin of the wide config (batch 32, 3 layers of 48) ----------------------
B, H, Lyr = 32, 48, 3
xb, yb = f32(B, H), f32(B, H)
Ws = [f32(H, H, scale=1 / np.sqrt(H)) for _ in range(Lyr)]
bs = [f32(H, scale=1 / np.sqrt(H)) for _ in range(Lyr)]
d = {"x": xb, "y": yb}
for i in range(Lyr):
    d["W%d" % i], d["b%d" % i] = Ws[i], bs[i]
tW = [t64(W, True) for W in Ws]
tb_ = [t64(b, True) for b in bs]
opt = torch.optim.Adam(tW + tb_, lr=1e-3, betas=(0.9, 0.999), eps=1e-8)
for step in range(2):
    h = t64(xb)
    for i in range(Lyr):
        h = h @ tW[i] + tb_[i]
        if i < Lyr - 1:
            h = torch.tanh(h)
    loss = torch.nn.functional.mse_loss(h, t64(yb))
    opt.zero_grad()
    loss.backward()
    if step == 0:
        for i in range(Lyr):
            d["dW%d" % i], d["db%d" % i] = tW[i].grad.numpy().copy(), tb_[i].grad.numpy().copy()
    d["loss%d" % step] = np.array([loss.item()])
    opt.step()
for i in range(Lyr):
    d["W%d_after" % i], d["b%d_after" % i] = tW[i].detach().numpy(), tb_[i].detach().numpy()
save("mlp_tanh_adam", **d)

# ---- Hessian-vector product by double backward: sin MLP, loss = sum(out^2) (README.md:69-71 pattern) ----
B, H, Lyr = 16, 24, 3
xb = f32(B, H)
Ws = [f32(H, H, scale=1 / np.sqrt(H)) for _ in range(Lyr)]
bs = [f32(H, scale=1 / np.sqrt(H)) for _ in range(Lyr)]
vW = [f32(H, H) for _ in range(Lyr)]
vb = [f32(H) for _ in range(Lyr)]
tW = [t64(W, True) for W in Ws]
tb_ = [t64(b, True) for b in bs]
h = t64(xb)
for i in range(Lyr):
    h = h @ tW[i] + tb_[i]
    if i < Lyr - 1:
        h = torch.sin(h)
loss = (h * h).sum()
params = tW + tb_
grads = torch.autograd.grad(loss, params, create_graph=True)
s = sum((g * t64(v)).sum() for g, v in zip(grads, vW + vb))
hv = torch.autograd.grad(s, params)
d = {"x": xb, "loss": np.array([loss.item()])}
for i in range(Lyr):
    d["W%d" % i], d["b%d" % i], d["vW%d" % i], d["vb%d" % i] = Ws[i], bs[i], vW[i], vb[i]
    d["gW%d" % i], d["gb%d" % i] = grads[i].detach().numpy(), grads[Lyr + i].detach().numpy()
    d["hW%d" % i], d["hb%d" % i] = hv[i].numpy(), hv[Lyr + i].numpy()
save("hvp_sin", **d)

# ---- complex MLP, identity layers, loss = sum |out|^2: Wirtinger-conjugate gradients (torch) -----------
B, H, Lyr = 8, 12, 3
zb = c64(B, H)
Ws = [(c64(H, H) / np.sqrt(2 * H)).astype(np.complex64) for _ in range(Lyr)]
tW = [t64(W, True) for W in Ws]
h = t64(zb)
for i in range(Lyr):
    h = h @ tW[i]
loss = (h.abs() ** 2).sum()
loss.backward()
d = {"z": zb, "loss": np.array([loss.item()]), "out": h.detach().numpy()}
for i in range(Lyr):
    d["W%d" % i], d["dW%d" % i] = Ws[i], tW[i].grad.numpy()
save("complex_mlp", **d)

# ---- the rest of the unary ops: forward and gradient of sum(op(x)) (test_exp_op.mojo, test_log_op.mojo, ...) ----
x = f32(2, 30, 40)
xp = np.abs(x) + 0.1                       # positive: log, reciprocal, sign
xu = (np.tanh(x) * 0.95).astype(np.float32)  # inside (-1, 1): asin, acos
d = {"x": x, "xp": xp, "xu": xu}
for name, fn, src in [("exp", torch.exp, x), ("log", torch.log, xp), ("sigmoid", torch.sigmoid, x),
                      ("sinh", torch.sinh, x), ("cosh", torch.cosh, x), ("tan", torch.tan, xu),
                      ("asin", torch.asin, xu), ("acos", torch.acos, xu), ("atan", torch.atan, x),
                      ("reciprocal", torch.reciprocal, xp)]:
    t = t64(src, True)
    y = fn(t)
    y.sum().backward()
    d[name] = y.detach().numpy()
    d["d" + name] = t.grad.numpy()
d["sign"] = np.sign(xp.astype(np.float64)) * 1.0
# complex forward bodies (the reference's tests run most unary ops on complex inputs too)
z = c64(2, 30, 40)
d["z"] = z
tz = t64(z)
for name, fn in [("sin", torch.sin), ("cos", torch.cos), ("tanh", torch.tanh), ("exp", torch.exp), ("log", torch.log),
                 ("sinh", torch.sinh), ("cosh", torch.cosh), ("sqrt", torch.sqrt), ("reciprocal", torch.reciprocal),
                 ("sign", torch.sgn)]:
    d["c" + name] = fn(tz).numpy()
save("unary_more", **d)

# ---- pow with broadcasting and its gradients (test_pow_op.mojo), comparisons (comparison_ops) -------------
a, b = (np.abs(f32(2, 30, 40)) + 0.2).astype(np.float32), f32(30, 40)
ta, tb = t64(a, True), t64(b, True)
y = torch.pow(ta, tb)
y.sum().backward()
an = f32(2, 30, 40)                         # negative bases with integer exponents
ei = rng.integers(0, 4, size=(30, 40)).astype(np.float32)
yn = torch.pow(t64(an), t64(ei))
ca, cb = f32(2, 30, 40).round(), f32(30, 40).round()   # many ties, so == and != see both outcomes
d = {"a": a, "b": b, "pow": y.detach().numpy(), "dpow_a": ta.grad.numpy(), "dpow_b": tb.grad.numpy(),
     "an": an, "ei": ei, "pow_neg": yn.numpy(), "ca": ca, "cb": cb}
tca, tcb = t64(ca), t64(cb)
for name, fn in [("greater", torch.gt), ("greater_equal", torch.ge), ("less", torch.lt), ("less_equal", torch.le),
                 ("equal", torch.eq), ("not_equal", torch.ne)]:
    d[name] = fn(tca, tcb).numpy().astype(np.float32)
save("binary_more", **d)

# ---- pooling: forward and gradient of sum(pool(x) * g) (test_max_pool2d_op.mojo, test_avg_pool2d_op.mojo and
# their 1-D / 3-D siblings compare the forward with torch; the gradients have no reference test). Average
# pooling divides by the taps inside the array, torch's count_include_pad=False. ------------------------
import torch.nn.functional as TF

d = {}
POOL_CASES = [  # name, x shape, kernel, stride, padding, dilation
    ("1d", (2, 3, 17), (3,), (2,), (1,), (1,)),
    ("2d", (2, 3, 13, 10), (3, 2), (2, 1), (1, 1), (1, 1)),
    ("3d", (2, 2, 7, 8, 6), (2, 3, 2), (1, 2, 2), (1, 1, 0), (1, 1, 1)),
    ("2d_dil", (1, 2, 12, 12), (2, 3), (1, 2), (1, 1), (2, 2)),
]
for name, xs, k, st, pad, dil in POOL_CASES:
    x = f32(*xs)
    nsp = len(xs) - 2
    mp = [TF.max_pool1d, TF.max_pool2d, TF.max_pool3d][nsp - 1]
    ap = [TF.avg_pool1d, TF.avg_pool2d, TF.avg_pool3d][nsp - 1]
    t = t64(x, True)
    y = mp(t, k, st, pad, dil)
    g = f32(*y.shape)
    (y * t64(g)).sum().backward()
    d.update({"x_" + name: x, "g_" + name: g, "max_" + name: y.detach().numpy(), "dmax_" + name: t.grad.numpy(),
              "cfg_" + name: np.array([k, st, pad, dil], dtype=np.int64)})
    if all(v == 1 for v in dil):
        t = t64(x, True)
        y = ap(t, k, st, pad, count_include_pad=False)
        (y * t64(g)).sum().backward()
        d.update({"avg_" + name: y.detach().numpy(), "davg_" + name: t.grad.numpy()})
save("pool", **d)

# ---- conv1d and conv3d with bias, stride / padding / dilation, and their gradients (test_conv1d_op.mojo,
# test_conv3d_op.mojo compare the forward with torch; the gradients are new) ----------------------------
d = {}
for name, xs, ws, st, pad, dil in [("1d", (3, 4, 29), (6, 4, 5), (2,), (3,), (2,)),
                                    ("3d", (2, 3, 6, 9, 8), (5, 3, 2, 3, 3), (1, 2, 1), (1, 1, 2), (2, 1, 1)),
                                    ("3d_unit", (2, 4, 5, 6, 8), (3, 4, 3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1))]:
    x, w, b = f32(*xs), f32(*ws, scale=0.3), f32(ws[0])
    tx, tw, tb = t64(x, True), t64(w, True), t64(b, True)
    conv = TF.conv1d if len(xs) == 3 else TF.conv3d
    y = conv(tx, tw, tb, st, pad, dil)
    g = f32(*y.shape)
    (y * t64(g)).sum().backward()
    d.update({"x_" + name: x, "w_" + name: w, "b_" + name: b, "g_" + name: g, "y_" + name: y.detach().numpy(),
              "dx_" + name: tx.grad.numpy(), "dw_" + name: tw.grad.numpy(), "db_" + name: tb.grad.numpy(),
              "cfg_" + name: np.array([st, pad, dil], dtype=np.int64)})
save("convnd", **d)

# ---- views: as_strided with overlapping windows and its gradient (test_as_strided_op.mojo: the same two
# cases, shapes (2,30,40) -> (1,2,40,2,2) and (30,30,2) with strides (9,30,2)), a strided slice and its
# gradient (array_slice_op.mojo:104-120 pads the cotangent), pad and concat ---------------------------------
d = {}
x = f32(2, 30, 40)
d["as_x"] = x
d["as_y"] = torch.as_strided(t64(x), (1, 2, 40, 2, 2), (16, 8, 2, 2, 1), 0).numpy()
x2 = np.arange(30 * 30 * 2, dtype=np.float32).reshape(30, 30, 2) * 0.01
t = t64(x2, True)
torch.sum(torch.sin(torch.as_strided(t, (30, 30, 2), (9, 30, 2), 0))).backward()
d["as_x2"], d["as_dx2"] = x2, t.grad.numpy()
x3 = f32(7, 9, 10)
t = t64(x3, True)
y = t[1:6:2, 2:, ::3]
g = f32(*y.shape)
(y * t64(g)).sum().backward()
d.update({"sl_x": x3, "sl_y": y.detach().numpy(), "sl_g": g, "sl_dx": t.grad.numpy()})
p = f32(3, 4)
t = t64(p, True)
big = torch.zeros(5, 9, dtype=torch.float64)
big[1:4, 2:9:2] = t
gb = f32(5, 9)
(big * t64(gb)).sum().backward()
d.update({"pad_x": p, "pad_y": big.detach().numpy(), "pad_g": gb, "pad_dx": t.grad.numpy()})
c1, c2, c3 = f32(2, 3, 4), f32(2, 5, 4), f32(2, 1, 4)
t1, t2, t3 = t64(c1, True), t64(c2, True), t64(c3, True)
y = torch.cat([t1, t2, t3], dim=1)
gc = f32(*y.shape)
(y * t64(gc)).sum().backward()
d.update({"cat_1": c1, "cat_2": c2, "cat_3": c3, "cat_y": y.detach().numpy(), "cat_g": gc, "cat_d1": t1.grad.numpy(),
          "cat_d2": t2.grad.numpy(), "cat_d3": t3.grad.numpy()})
save("views", **d)

# ---- the other reductions (test_reduce_max_op.mojo:18-34, test_reduce_min_op.mojo:18-34, test_reduce_argmax_op.mojo:18-33,
# test_reduce_argmin_op.mojo:18-33, test_reduce_mul_op.mojo:18-33, test_std_op.mojo:18-58, test_variance_op.mojo:18-59) ------
x = f32(2, 30, 40)
t = t64(x)
d = {"x": x, "max1": torch.max(t, dim=1)[0].numpy(), "min1": torch.min(t, dim=1)[0].numpy(),
     "argmax1": torch.argmax(t, dim=1).numpy().astype(np.float64), "argmin1": torch.argmin(t, dim=1).numpy().astype(np.float64),
     "max02": torch.amax(t, dim=(0, 2)).numpy(), "min12": torch.amin(t, dim=(1, 2)).numpy(),
     "argmax2": torch.argmax(t, dim=2).numpy().astype(np.float64), "prod1": torch.prod(t, 1).numpy(),
     "prod_all": torch.prod(t64(x[0, :8, :5])).numpy().reshape(1),
     "std1": torch.std(t, [1]).numpy(), "var1": torch.var(t, [1]).numpy(), "var02_biased": torch.var(t, [0, 2], unbiased=False).numpy(),
     "std1_keep": torch.std(t, [1], keepdim=True).numpy()}
tg = t64(x, True)
torch.sum(torch.std(tg, [1])).backward()
d["dstd1"] = tg.grad.numpy()
tg = t64(x, True)
torch.sum(torch.var(tg, [1])).backward()
d["dvar1"] = tg.grad.numpy()
save("reduce_more", **d)
