"""Fused elementwise expressions: `fuse(fn)` turns a Python function built from the elementwise ops of
`endia_amd.functional` into ONE kernel launch for the forward pass and ONE for all input gradients.

The reference fuses runs of unary ops on one array into a single SIMD loop (simd_op_list +
execute_fwds, endia/_array/_array.mojo:90-101,756-782) and leaves larger elementwise subgraphs to its
JIT (FxSubgraph, endia/compile/fx.mojo:105-159). Here the function is traced once with symbolic values;
because every op's VJP rule is itself written in these ops, tracing the rules gives the gradient
expressions for free (the same walk as endia/autograd/functional.mojo:26-67, on symbols). Both
expression graphs are compiled into programs for `endia_hip_ew_program`'s accumulator machine.

Inputs may be full arrays of the broadcast shape, row vectors over the last axis, or one-element
arrays; anything else is expanded and copied first. Real arrays only.
"""
import ctypes
import itertools

from . import _lib as L
from . import functional as F
from ._array import Array, _prod


class FusionError(ValueError):
    pass


class Sym:
    """A value inside a traced elementwise expression. Mimics the few Array attributes that VJP rules read."""

    _ids = itertools.count()

    def __init__(self, kind, shape, op=None, args=(), index=None, value=None, vjp=None, name="", requires_grad=True):
        self.kind = kind  # "input" | "imm" | "unary" | "binary"
        self._shape = tuple(shape)
        self.op, self.args, self.index, self.value = op, tuple(args), index, value
        self._vjp, self._name = vjp, name
        self._requires_grad = requires_grad
        self.is_complex_ = False
        self.id = next(Sym._ids)

    def shape(self):
        return list(self._shape)

    # operators mirror Array's (scalars become immediates instead of `full` arrays)
    def _bin(self, other, fn, reverse=False):
        return fn(other, self) if reverse else fn(self, other)

    def __add__(self, o): return self._bin(o, F.add)
    __radd__ = __add__
    def __sub__(self, o): return self._bin(o, F.sub)
    def __rsub__(self, o): return self._bin(o, F.sub, True)
    def __mul__(self, o): return self._bin(o, F.mul)
    __rmul__ = __mul__
    def __truediv__(self, o): return self._bin(o, F.div)
    def __rtruediv__(self, o): return self._bin(o, F.div, True)
    def __pow__(self, o): return self._bin(o, F.pow)
    def __rpow__(self, o): return self._bin(o, F.pow, True)
    def __neg__(self): return F.neg(self)


class _Trace:
    """State of one tracing pass: the shape being traced and the constant arrays captured on the way."""

    def __init__(self, shape, n_inputs):
        self.shape = tuple(shape)
        self.consts = []  # (Array, Sym) for arrays that VJP rules or the user's function close over
        self.n_inputs = n_inputs

    def lift(self, v):
        if isinstance(v, Sym):
            return v
        if isinstance(v, (int, float)):
            return Sym("imm", self.shape, value=float(v), requires_grad=False)
        if isinstance(v, Array):
            for arr, sym in self.consts:
                if arr is v:
                    return sym
            if v.is_complex_:
                raise FusionError("fused expressions are real only")
            sym = Sym("input", self.shape, index=self.n_inputs + len(self.consts), requires_grad=False)
            self.consts.append((v, sym))
            return sym
        raise FusionError("cannot use %r inside a fused expression" % (v,))


_active = [None]  # the _Trace in progress, if any


def tracing(*values):
    return _active[0] is not None and any(isinstance(v, Sym) for v in values)


def sym_unary(op, name, x, vjp):
    return Sym("unary", x._shape, op=op, args=(x,), vjp=vjp, name=name, requires_grad=x._requires_grad)


def sym_binary(op, name, a, b, vjp):
    t = _active[0]
    a, b = t.lift(a), t.lift(b)
    return Sym("binary", t.shape, op=op, args=(a, b), vjp=vjp, name=name,
               requires_grad=vjp is not None and (a._requires_grad or b._requires_grad))


def _sym_backward(root, g, wanted):
    """Reverse walk over the expression graph with symbolic cotangents; returns {input index: Sym}."""
    order, seen = [], set()

    def visit(n):
        if n.id in seen:
            return
        seen.add(n.id)
        for a in n.args:
            visit(a)
        order.append(n)

    visit(root)
    grads = {root.id: g}
    out = {}
    for n in reversed(order):
        gn = grads.get(n.id)
        if gn is None:
            continue
        if n.kind == "input":
            if n.index in wanted:
                out[n.index] = gn
            continue
        if n._vjp is None or not n._requires_grad:
            continue
        for a, ga in zip(n.args, n._vjp(list(n.args), gn, n)):
            if ga is None or not a._requires_grad:
                continue
            ga = _active[0].lift(ga)
            grads[a.id] = ga if a.id not in grads else F.add(grads[a.id], ga)
    return out


# ---- expression graph -> accumulator program ---------------------------------------------------------
def _compile(roots, alias=None):
    """Lower the expression graphs `roots` (one per output) to a step list. `alias` maps node ids whose
    value is already in memory to an input index."""
    alias = alias or {}
    uses = {}

    def count(n):
        uses[n.id] = uses.get(n.id, 0) + 1
        if uses[n.id] == 1 and n.id not in alias:
            for a in n.args:
                count(a)

    for r in roots:
        count(r)
    remaining = dict(uses)
    slot_of, free, steps = {}, list(range(L.EW_MAX_SLOTS)), []

    def leaf(n):
        return n.kind in ("input", "imm") or n.id in alias

    def operand(n):
        if n.id in alias:
            return (L.EW_SRC_INPUT, alias[n.id], 0.0)
        if n.kind == "input":
            return (L.EW_SRC_INPUT, n.index, 0.0)
        if n.kind == "imm":
            return (L.EW_SRC_IMM, 0, n.value)
        if n.id in slot_of:
            return (L.EW_SRC_SLOT, slot_of[n.id], 0.0)
        return None

    def alloc():
        if not free:
            raise FusionError("expression keeps more than %d intermediate values alive" % L.EW_MAX_SLOTS)
        return free.pop(0)

    def consume(n):
        if leaf(n):
            return
        remaining[n.id] -= 1
        if remaining[n.id] == 0 and n.id in slot_of:
            free.append(slot_of.pop(n.id))

    def emit(kind, op=0, src=(0, 0, 0.0)):
        steps.append((kind, op, src[0], src[1], src[2]))

    def evaluate(n):
        """Leave the value of n in the accumulator."""
        src = operand(n)
        if src is not None:
            emit(L.EW_LOAD, 0, src)
            return
        if n.kind == "unary":
            evaluate(n.args[0])
            emit(L.EW_UNARY, n.op)
            consume(n.args[0])
        else:
            a, b = n.args
            if operand(b) is not None:
                evaluate(a)
                emit(L.EW_BINARY, n.op, operand(b))
            elif operand(a) is not None:
                evaluate(b)
                emit(L.EW_RBINARY, n.op, operand(a))
            else:
                evaluate(a)
                if operand(b) is not None:      # b became addressable while a was computed
                    emit(L.EW_BINARY, n.op, operand(b))
                elif operand(a) is not None:    # a is kept in a slot for its other consumers
                    evaluate(b)
                    emit(L.EW_RBINARY, n.op, operand(a))
                else:
                    t = alloc()
                    emit(L.EW_SAVE, 0, (0, t, 0.0))
                    evaluate(b)
                    emit(L.EW_RBINARY, n.op, (L.EW_SRC_SLOT, t, 0.0))
                    free.append(t)
            consume(a)
            consume(b)
        if uses[n.id] > 1 and remaining[n.id] > 1:
            t = alloc()
            emit(L.EW_SAVE, 0, (0, t, 0.0))
            slot_of[n.id] = t

    for i, r in enumerate(roots):
        evaluate(r)
        emit(L.EW_STORE, 0, (0, i, 0.0))
        consume(r)
    if len(steps) > L.EW_MAX_STEPS:
        raise FusionError("expression needs %d steps, at most %d fit one program" % (len(steps), L.EW_MAX_STEPS))
    arr = (L.EwStep * len(steps))()
    for i, (kind, op, sk, si, imm) in enumerate(steps):
        arr[i] = L.EwStep(kind, op, sk, si, imm)
    return arr


def _launch(rows, cols, inputs, modes, outputs, steps):
    n_in, n_out = len(inputs), len(outputs)
    if n_in > L.EW_MAX_INPUTS:
        raise FusionError("%d inputs, at most %d fit one program" % (n_in, L.EW_MAX_INPUTS))
    pin = (ctypes.c_void_p * max(n_in, 1))(*[a.data_ptr() for a in inputs])
    pmode = (ctypes.c_int32 * max(n_in, 1))(*modes)
    pout = (ctypes.c_void_p * n_out)(*[a.data_ptr() for a in outputs])
    L.call("endia_hip_ew_program", rows, cols, n_in, pin, pmode, n_out, pout, len(steps), steps)


_UNARY_FN = {}
_BINARY_FN = {}


def _replay(node, env, cache):
    """Evaluate an expression graph with ordinary (differentiable) ops on arrays."""
    if node.id in cache:
        return cache[node.id]
    if node.kind == "input":
        v = env[node.index]
    elif node.kind == "imm":
        v = node.value
    elif node.kind == "unary":
        v = _UNARY_FN[node.op](_replay(node.args[0], env, cache))
    else:
        a, b = (_replay(x, env, cache) for x in node.args)
        if not isinstance(a, Sym) and not isinstance(b, Sym):  # (inside a trace, numbers become immediates)
            if not isinstance(a, Array) and not isinstance(b, Array):
                a = F.full([1], a)
            if not isinstance(a, Array):
                a = F.full([b._shape[-1]], a)
            if not isinstance(b, Array):
                b = F.full([a._shape[-1]], b)
        v = _BINARY_FN[node.op](a, b)
    cache[node.id] = v
    return v


class _Plan:
    """Everything traced for one (shape, input modes, requires_grad) signature."""


class FusedElementwise:
    def __init__(self, fn, name=None):
        self.fn = fn
        self.name = name or getattr(fn, "__name__", "fused")
        self._plans = {}

    # -- tracing -------------------------------------------------------------------------------
    def _plan(self, shape, modes, req):
        key = (tuple(shape), tuple(modes), tuple(req))
        plan = self._plans.get(key)
        if plan is not None:
            return plan
        if _active[0] is not None:
            raise FusionError("fused functions cannot be nested")
        n = len(modes)
        trace = _Trace(shape, n + 2)  # two inputs are reserved for the backward pass: cotangent, forward output
        _active[0] = trace
        try:
            ins = [Sym("input", shape, index=i, requires_grad=bool(req[i])) for i in range(n)]
            root = self.fn(*ins)
            if not isinstance(root, Sym) or root.kind in ("input", "imm"):
                raise FusionError("the fused function must return an elementwise expression of its arguments")
            plan = _Plan()
            plan.root, plan.n = root, n
            plan.fwd_consts = list(trace.consts)
            plan.fwd = _compile([root])
            plan.wanted = [i for i in range(n) if req[i]]
            plan.grads, plan.bwd = None, None
            if plan.wanted:
                g = Sym("input", shape, index=n, requires_grad=False)
                grads = _sym_backward(root, g, set(plan.wanted))
                plan.wanted = [i for i in plan.wanted if i in grads]
                plan.grads = [grads[i] for i in plan.wanted]
                plan.g_sym = g
                try:
                    plan.bwd = _compile(plan.grads, alias={root.id: n + 1}) if plan.grads else None
                except FusionError:
                    plan.bwd = None  # too many live values for one program: the gradients are replayed op by op
            plan.consts = list(trace.consts)
        finally:
            _active[0] = None
        self._plans[key] = plan
        return plan

    # -- call ----------------------------------------------------------------------------------
    def __call__(self, *args):
        arrays = []
        for a in args:
            if not isinstance(a, Array):
                raise TypeError("fused functions take arrays")
            if a.is_complex_:
                raise FusionError("fused expressions are real only")
            arrays.append(a)
        shape = list(arrays[0]._shape)
        for a in arrays[1:]:
            shape = _bshape(shape, list(a._shape))
        rows, cols = _prod(shape[:-1]), shape[-1]
        ins, modes = [], []
        for a in arrays:
            if list(a._shape) == shape:
                # a broadcast view of the full shape (the cotangent a reduction hands down) is read as what it is,
                # one element or one row, instead of being copied out
                spread = [st == 0 for n_, st in zip(a._shape, a._strides) if n_ != 1]
                if a.size() > 1 and all(spread):
                    ins.append(Array([1], _buffer=a._buf, _offset=a._offset)); modes.append(L.EW_SCALAR)
                elif rows > 1 and cols > 1 and a._strides[-1] == 1 and all(spread[:-1]):
                    ins.append(Array([cols], _buffer=a._buf, _offset=a._offset)); modes.append(L.EW_ROW_VECTOR)
                else:
                    ins.append(F.contiguous(a)); modes.append(L.EW_FULL)
            elif a.size() == 1:
                ins.append(a); modes.append(L.EW_SCALAR)
            elif a.size() == cols and a._shape[-1] == cols:
                ins.append(F.contiguous(a)); modes.append(L.EW_ROW_VECTOR)
            else:  # any other broadcast pattern is materialised; expand's VJP sums it back
                ins.append(F.contiguous(F.expand(a, shape))); modes.append(L.EW_FULL)
        req = [a._requires_grad for a in arrays]
        plan = self._plan(shape, modes, req)
        out = Array.empty(shape)
        if out.size():
            # the two reserved slots are unused by the forward program; any valid pointer will do
            fins = ins + [out, out] + [c for c, _ in plan.fwd_consts]
            fmodes = modes + [L.EW_FULL, L.EW_FULL] + [_const_mode(c, shape) for c, _ in plan.fwd_consts]
            if not plan.fwd_consts:
                fins, fmodes = ins, modes
            _launch(rows, cols, fins, fmodes, [out], plan.fwd)

        def vjp(primals, grad, out_):
            from .autograd.functional import building_graph
            res = [None] * len(primals)
            if not plan.wanted:
                return res
            if list(grad._shape) != shape and grad.size() == _prod(shape):
                grad = F.reshape(grad, shape)  # kept axes of length 1 in front (the cotangent of a reduction's operand)
            lead_n = max(0, len(grad._shape) - len(shape))
            lead = lead_n > 0  # a Jacobian seed's axes in front: the op-by-op rules broadcast over them
            if building_graph() and not lead:
                # A pass that records its own graph: every gradient expression becomes a fused function of
                # (inputs, cotangent, forward output, captured constants), so the recorded node is ONE launch and is
                # itself differentiable to any order by the same tracing. Expressions that do not fit a program
                # are replayed op by op.
                operands = list(primals) + [grad if list(grad._shape) == shape else F.expand(grad, shape), out_] + [c for c, _ in plan.consts]
                full = []
                for k, gs in enumerate(plan.grads):
                    try:
                        full.append(_gradient_function(plan, k)(*operands))
                    except FusionError:
                        env = dict(enumerate(operands))
                        f = _replay(gs, env, {})
                        full.append(f if isinstance(f, Array) else F.full(shape, f))
            elif plan.bwd is None or lead or building_graph():
                env = {i: p for i, p in enumerate(primals)}
                env[plan.n] = grad
                env[plan.n + 1] = out_
                for c, s in plan.consts:
                    env[s.index] = c
                cache = {}
                full = [_replay(gs, env, cache) for gs in plan.grads]
                full = [f if isinstance(f, Array) else F.full(shape, f) for f in full]
            else:
                gc = F.contiguous(grad if list(grad._shape) == shape else F.expand(grad, shape))
                full = [Array.empty(shape) for _ in plan.wanted]
                if out.size():
                    bins = ins + [gc, out_] + [c for c, _ in plan.consts]
                    bmodes = modes + [L.EW_FULL, L.EW_FULL] + [_const_mode(c, shape) for c, _ in plan.consts]
                    _launch(rows, cols, bins, bmodes, full, plan.bwd)
            for i, f in zip(plan.wanted, full):
                p = primals[i]
                own = list(f._shape)[lead_n:]  # the expression's own axes, behind those of a Jacobian seed
                if own != list(p._shape):
                    # a broadcast input: sum over the axes it was spread along, keeping them as size 1 like
                    # the VJP of the reference's expand (expand_op.mojo:121-126)
                    extra = len(own) - len(p._shape)
                    axes = [lead_n + k for k in range(len(own)) if k < extra or p._shape[k - extra] != own[k]]
                    f = F.reduce_add(f, axes)
                res[i] = f
            return res

        return F._register(out, arrays, "fused:" + self.name, vjp)


def _gradient_function(plan, k):
    """The k-th gradient expression of a traced plan as a fused function of its operands, in the order
    (inputs..., cotangent, forward output, constants...): operand i is what the expression calls input i."""
    cache = plan.__dict__.setdefault("grad_fns", {})
    fn = cache.get(k)
    if fn is None:
        expr = plan.grads[k]

        def rebuilt(*syms):  # the forward output is an operand: no need to evaluate its expression again
            return _replay(expr, dict(enumerate(syms)), {plan.root.id: syms[plan.n + 1]})

        fn = cache[k] = FusedElementwise(rebuilt, "grad%d" % k)
    return fn


def _bshape(sa, sb):
    n = max(len(sa), len(sb))
    sa, sb = [1] * (n - len(sa)) + sa, [1] * (n - len(sb)) + sb
    out = []
    for x, y in zip(sa, sb):
        if x != y and x != 1 and y != 1:
            raise ValueError("cannot broadcast %s with %s" % (sa, sb))
        out.append(x if y == 1 else y)
    return out


def _const_mode(c, shape):
    if list(c._shape) == list(shape) and c.is_contiguous():
        return L.EW_FULL
    if c.size() == 1:
        return L.EW_SCALAR
    if c.size() == shape[-1] and c._shape[-1] == shape[-1] and c.is_contiguous():
        return L.EW_ROW_VECTOR
    raise FusionError("a constant of shape %s cannot be broadcast to %s inside a fused expression" % (c.shape(), list(shape)))


def fuse(fn=None, name=None):
    """Decorator / wrapper: `f = fuse(lambda a, b: sigmoid(a * b + 1.0))`."""
    if fn is None:
        return lambda f: FusedElementwise(f, name)
    return FusedElementwise(fn, name)


def _fill_tables():
    for name, code in [("relu", L.OP_RELU), ("tanh", L.OP_TANH), ("sin", L.OP_SIN), ("cos", L.OP_COS), ("neg", L.OP_NEG),
                       ("square", L.OP_SQUARE), ("sqrt", L.OP_SQRT), ("abs", L.OP_ABS), ("exp", L.OP_EXP), ("log", L.OP_LOG),
                       ("sigmoid", L.OP_SIGMOID), ("sinh", L.OP_SINH), ("cosh", L.OP_COSH), ("tan", L.OP_TAN),
                       ("asin", L.OP_ASIN), ("acos", L.OP_ACOS), ("atan", L.OP_ATAN), ("reciprocal", L.OP_RECIPROCAL),
                       ("sign", L.OP_SIGN)]:
        _UNARY_FN[code] = getattr(F, name)
    for name, code in [("add", L.BIN_ADD), ("sub", L.BIN_SUB), ("mul", L.BIN_MUL), ("div", L.BIN_DIV), ("pow", L.BIN_POW),
                       ("greater", L.BIN_GREATER), ("greater_equal", L.BIN_GREATER_EQUAL), ("less", L.BIN_LESS),
                       ("less_equal", L.BIN_LESS_EQUAL), ("equal", L.BIN_EQUAL), ("not_equal", L.BIN_NOT_EQUAL)]:
        _BINARY_FN[code] = getattr(F, name)


_fill_tables()
F._fusion = __import__("sys").modules[__name__]
