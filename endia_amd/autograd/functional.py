"""Reverse-mode driver: the host-side mirror of endia/autograd/functional.mojo.

`jacrev` follows the reference's walk (functional.mojo:26-67): depth-first post-order over the
argument lists (endia/utils/general.mojo:18-32), a seed of ones(1) for a scalar output or an identity
Jacobian seed otherwise (:34-38), then the trace in reverse, calling each node's VJP rule and
accumulating with an `add` op where a tensor has several consumers (:51-57). Unless
`create_graph=True`, every stored gradient is cut from the graph that produced it (:63-65).

The functional wrappers (grad / jacobian / hessian / value_and_grad over a Python callable) follow the
non-JIT branch of Callable.__call__ (endia/compile/callable.mojo:100-197): repeated
backward(create_graph=True) passes, then detached copies of the results.
"""
import sys

from .. import _lib as L
from .. import functional as F
from .._array import Array, _contiguous_copy

_building_graph = [False]


def building_graph():
    """True while a backward pass runs with create_graph=True. Fused ops consult it to pick between
    their single-kernel first-order rule and a rule rebuilt from differentiable ops."""
    return _building_graph[0]


_SEED = []


def _seed_one():
    """ones(1), the seed of a scalar output (functional.mojo:34-38). It is read, never written, so one array
    serves every backward pass and a step spends no launch on filling it."""
    if not _SEED:
        seed = F.ones([1])
        seed._is_seed = True
        _SEED.append(seed)
    return _SEED[0]


def top_order(out):
    """Post-order DFS over args (general.mojo:26-32), iterative so deep graphs do not hit the
    interpreter's recursion limit."""
    trace, seen = [], set()
    stack = [(out, 0)]
    seen.add(id(out))
    while stack:
        node, i = stack[-1]
        if i < len(node._args):
            stack[-1] = (node, i + 1)
            child = node._args[i]
            if id(child) not in seen:
                seen.add(id(child))
                stack.append((child, 0))
        else:
            stack.pop()
            trace.append(node)
    return trace


def backward(arg, create_graph=False):
    jacrev(arg, create_graph)


def jacrev(arg, create_graph=False):
    out = arg
    trace = top_order(out)
    dims = out._shape[-1] if out._shape else 1
    if out.ndim() != 1 or dims != 1:
        n = out.size()
        seed = F.reshape(F.eye(n), out.shape() + out.shape())
    else:
        seed = _seed_one()
    out.grad_(seed)
    _reverse_walk(trace, create_graph)


class _Root:
    """Stands above several outputs so that one post-order walk covers all of their graphs."""

    def __init__(self, outs):
        self._args, self._vjp, self._consumers = list(outs), None, 0


def vjp_from(outs, cotangents, create_graph=False):
    """One reverse pass from several outputs at once, each seeded with its own cotangent (same shape as the
    output) instead of ones. No counterpart in the reference, whose grad(outs, inputs) seeds every output with
    ones, one backward pass per output (functional.mojo:70-97); this is the cotangent argument of a VJP, and
    it computes the gradient of sum_i <out_i, cotangent_i> without forming that sum."""
    outs, cotangents = list(outs), list(cotangents)
    if len(outs) != len(cotangents):
        raise ValueError("vjp_from: %d outputs but %d cotangents" % (len(outs), len(cotangents)))
    for o, c in zip(outs, cotangents):
        if list(o.shape()) != list(c.shape()):
            raise ValueError("vjp_from: cotangent of shape %s for an output of shape %s" % (c.shape(), o.shape()))
    trace = top_order(_Root(outs))
    for o, c in zip(outs, cotangents):
        o.grad_(F.add(o._grad, c) if o.has_grad() else c)
    _reverse_walk(trace, create_graph)


_VIEW_OPS = ("permute", "reshape", "squeeze", "unsqueeze")
absorb_enabled = [True]  # tests switch the in-launch accumulation off to compare with the walk's own `add`


def _offers(primals):
    """What the primals of one VJP call already hold, for rules that can add it in their own last launch
    (functional._absorb): id(primal) -> (gradient, exclusive). `exclusive`: no other name refers to the gradient array
    or shares its buffer (reference counts: the gradient slot, the local below and the call's argument; the array's
    buffer field and the call's argument), so a rule may accumulate into it in place."""
    offers = None
    if not absorb_enabled[0]:
        return None
    for p in primals:
        g = p._grad
        if g is None or not p._requires_grad or p._grad_fused is not None or g._is_seed:
            continue
        exclusive = sys.getrefcount(g) <= 3 and sys.getrefcount(g._buf) <= (3 if g._buf.pending else 2)  # (a parked product holds its output buffer)
        if offers is None:
            offers = {}
        offers[id(p)] = (g, exclusive)
    return offers


def _reverse_walk(trace, create_graph):
    """The trace in reverse: every node's VJP rule, contributions to one tensor summed with `add`
    (functional.mojo:46-65), or inside the launch that computes the later contribution where its rule can
    (functional._absorb). The outputs' gradients are already in place."""
    for node in trace:
        node._consumers = 0
    for node in trace:
        for a in node._args:
            a._consumers += 1
    for node in trace:
        node._contributions_left = node._consumers

    prev = _building_graph[0]
    _building_graph[0] = bool(create_graph)
    finished = []
    try:
        for curr in reversed(trace):
            primals = curr._args
            if not primals or curr._vjp is None:
                continue
            # a gradient that already carries this node's activation derivative travels in its own slot
            grad = curr._grad_fused if curr._grad_fused is not None else curr.grad()
            F._absorb = None if create_graph else _offers(primals)
            F._in_rule[0] = True
            try:
                primals_grads = curr._vjp(primals, grad, curr)
            finally:
                F._absorb = None
                F._in_rule[0] = False
            if not create_graph and curr._internal and curr._name in _VIEW_OPS:
                # a view that an earlier pass's rule made (x.T() inside a recorded matmul rule): nobody can ask for its
                # gradient, and letting go of it leaves the gradient it handed on as the only holder of that buffer
                grad = None
                curr._grad = None
            for primal, pg in zip(primals, primals_grads):
                primal._contributions_left -= 1
                if primal._on_final_grad is not None and primal._contributions_left == 0 and not create_graph:
                    finished.append(primal)  # every consumer has contributed once this one is stored
                if not primal._requires_grad or pg is None:
                    continue
                if primal.has_grad():
                    if pg._act_applied or primal._grad_fused is not None:
                        raise RuntimeError("internal: a fused activation gradient met an accumulated gradient")
                    if not pg._absorbed:  # (an absorbed contribution already holds the sum)
                        pg = F.add(pg, primal._grad)
                if pg._act_applied:
                    primal._grad_fused = pg
                    continue
                primal.grad_(pg)
                if not create_graph:
                    pg.clear_args()
            # An optimizer built with fused_backward=True updates a parameter as soon as its gradient is complete, while
            # the gradient still sits in the last-level cache; the walk goes on with the other layers meanwhile.
            while finished:
                leaf = finished.pop()
                if leaf._grad is not None:
                    leaf._on_final_grad(leaf)
        L.flush_col_sums()  # the pass is over: the bias gradients it put off go out as one launch
    finally:
        _building_graph[0] = prev


def _visit_all(out, fn):
    for node in top_order(out):
        fn(node)


def zero_grad_rec(out):
    """Array.zero_grad: drop the gradient of every node reachable from `out` (general.mojo:35-47)."""
    _visit_all(out, lambda n: n.remove_grad())


remove_grad_rec = zero_grad_rec


def grad(outs=None, inputs=None, retain_grads=True, create_graph=False, argnums=None, grad_outs=None):
    """Two forms, as in the reference:

    grad(outs=[...], inputs=[...]) -> list of gradients (functional.mojo:70-97);
    grad(f, argnums=...)           -> Callable computing the gradient of f (functional.mojo:100-128).

    grad_outs (not in the reference): one cotangent per output, of the output's shape; the outputs are then
    walked in ONE reverse pass seeded with them (vjp_from), which yields the gradient of
    sum_i <outs[i], grad_outs[i]>: a Hessian-vector product when the outputs are first-order gradients
    taken with create_graph=True.
    """
    if isinstance(outs, Callable):
        f = outs
        return Callable(f.func, f.argnums + [argnums if argnums is not None else [-1]], f.order + 1, False)
    if callable(outs) and not isinstance(outs, Array):
        return Callable(outs, [argnums if argnums is not None else [-1]], 1, False)
    single = isinstance(inputs, Array)
    outs = [outs] if isinstance(outs, Array) else list(outs)
    inputs = [inputs] if single else list(inputs)
    for o in outs:
        remove_grad_rec(o)
    for i in inputs:
        remove_grad_rec(i)
    if grad_outs is not None:
        vjp_from(outs, [grad_outs] if isinstance(grad_outs, Array) else grad_outs, create_graph)
    else:
        for o in outs:
            o.backward(create_graph=create_graph)
    res = []
    for i in inputs:
        g = i.grad()
        if not create_graph:
            g.clear_args()
            g.remove_grad()
        if not retain_grads:
            i.remove_grad()
        res.append(g)
    return res


class Callable:
    """grad(f) / jacobian(f) / hessian(f): endia/compile/callable.mojo:60-197, non-JIT branch."""

    def __init__(self, func, argnums, order, keep_outs):
        self.func = func
        self.argnums = [list(a) if isinstance(a, (list, tuple)) else [a] for a in argnums]
        self.order = order
        self.keep_outs = keep_outs

    def _wanted(self, order, n):
        chosen = self.argnums[order]
        return list(range(n)) if chosen[0] == -1 else [i for i in range(n) if i in chosen]

    def __call__(self, *args):
        single = len(args) == 1 and isinstance(args[0], Array)
        arrs = list(args[0]) if (len(args) == 1 and not single) else list(args)
        # fresh leaves, so that repeated calls never see stale graphs; an argument takes part in the graph when ANY
        # order differentiates with respect to it (callable.mojo:100-112)
        leaves = [F.detach(a) for a in arrs]
        for o in range(self.order):
            for i in self._wanted(o, len(leaves)):
                leaves[i].requires_grad_(True)
        res = self.func(leaves[0]) if single else self.func(leaves)
        outs = [res]
        per_order = [[res]]
        for o in range(self.order):
            idx = self._wanted(o, len(leaves))  # the arguments of THIS order (callable.mojo:146-151)
            nxt = []
            last = o == self.order - 1
            for arr in outs:
                remove_grad_rec(arr)
                arr.backward(create_graph=not last)
                for i in idx:
                    nxt.append(leaves[i].grad())
                for leaf in leaves:
                    leaf.remove_grad()
            outs = nxt
            per_order.append(nxt)
        # detach by copy (callable.mojo:165-176), device to device
        if not self.keep_outs:
            final = [_contiguous_copy(g) for g in outs]
            return final[0] if len(final) == 1 else final
        # value_and_grad: one list per order of differentiation, [[value], [first derivatives], ...] (callable.mojo:186-195)
        return [[_contiguous_copy(g) for g in group] for group in per_order]


def jacobian(f, argnums=None):
    return grad(f, argnums=argnums)


def hessian(f, argnums=None):
    return grad(grad(f, argnums=argnums), argnums=argnums)


def value_and_grad(f, argnums=None):
    if isinstance(f, Callable):
        return Callable(f.func, f.argnums + [argnums if argnums is not None else [-1]], f.order + 1, True)
    return Callable(f, [argnums if argnums is not None else [-1]], 1, True)
