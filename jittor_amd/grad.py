"""Reverse-mode gradients of the meta-operator path.

The gradient of every op on this path is again built from ops of the path, as
in the reference: ReindexOp -> reindex_reduce(add)
(python/jittor/src/ops/reindex_op.cc:76-80), ReindexReduceOp -> reindex
(+ an equality mask for maximum / minimum, ops/reindex_reduce_op.cc:45-63),
ReduceOp -> broadcast (ops/reduce_op.cc:339-362), BroadcastToOp -> reduce(add)
(ops/broadcast_to_op.cc:112-117), and the element-wise rules of
ops/binary_op.cc:491-561, ops/unary_op.cc:891-1019, ops/ternary_op.cc:49-56.
The driver follows python/jittor/src/grad.cc:85-284: only float vars carry
gradients, contributions of several consumers are added, a target the loss
does not depend on gets zeros.
"""
from . import core
from . import dtypes as dt
from .core import (Var, UnaryOp, BinaryOp, TernaryOp, BroadcastOp, ReduceOp, ReindexOp, ReindexReduceOp,
                   unary, binary, ternary, make_number, reindex, reindex_reduce, array)
from . import _lib


def _unary_grad(op, x, y, dout):
    """ops/unary_op.cc:891-1019 (y is the op's output)."""
    ns = op.op
    if not x.is_float():
        return None
    if ns in _lib.DTYPES or ns == "cast":
        return unary(dout, x.dtype)
    one = lambda: make_number(1, x)
    if ns == "negative":
        return unary(dout, "negative")
    if ns == "abs":
        return ternary(binary(x, make_number(0, x), "greater_equal"), dout, unary(dout, "negative"))
    if ns == "log":
        return binary(dout, x, "divide")
    if ns == "exp":
        return binary(dout, y, "multiply")
    if ns == "sqrt":
        return binary(dout, binary(make_number(2, x), y, "multiply"), "divide")
    if ns == "sin":
        return binary(dout, unary(x, "cos"), "multiply")
    if ns == "cos":
        return binary(dout, unary(unary(x, "sin"), "negative"), "multiply")
    if ns == "tan":
        c = unary(x, "cos")
        return binary(dout, binary(c, c, "multiply"), "divide")
    if ns == "asin":
        return binary(dout, unary(binary(one(), binary(x, x, "multiply"), "subtract"), "sqrt"), "divide")
    if ns == "acos":
        return unary(binary(dout, unary(binary(one(), binary(x, x, "multiply"), "subtract"), "sqrt"), "divide"), "negative")
    if ns == "atan":
        return binary(dout, binary(one(), binary(x, x, "multiply"), "add"), "divide")
    if ns == "sinh":
        return binary(dout, unary(x, "cosh"), "multiply")
    if ns == "cosh":
        return binary(dout, unary(x, "sinh"), "multiply")
    if ns == "tanh":
        c = unary(x, "cosh")
        return binary(dout, binary(c, c, "multiply"), "divide")
    if ns == "asinh":
        return binary(dout, unary(binary(binary(x, x, "multiply"), one(), "add"), "sqrt"), "divide")
    if ns == "acosh":
        return binary(dout, unary(binary(binary(x, x, "multiply"), one(), "subtract"), "sqrt"), "divide")
    if ns == "atanh":
        return binary(dout, binary(one(), binary(x, x, "multiply"), "subtract"), "divide")
    if ns == "sigmoid":
        return binary(dout, binary(y, binary(y, y, "multiply"), "subtract"), "multiply")
    if ns == "erf":
        r = unary(unary(binary(x, x, "multiply"), "negative"), "exp")
        return binary(dout, binary(r, make_number(2 / 1.7724538509055159, x), "multiply"), "multiply")
    if ns == "erfinv":
        r = unary(binary(y, y, "multiply"), "exp")
        return binary(dout, binary(r, make_number(1.7724538509055159 / 2, x), "multiply"), "multiply")
    return None      # round / floor / ceil / logical ops: no gradient


def _binary_grad(op, x, y, z, dout, index):
    """ops/binary_op.cc:491-561 (z is the op's output)."""
    ns = op.op
    if ns == "add":
        return dout
    if ns == "subtract":
        return dout if index == 0 else unary(dout, "negative")
    if ns == "multiply":
        return binary(y if index == 0 else x, dout, "multiply")
    if ns == "divide":
        if index == 0:
            return binary(dout, y, "divide")
        return binary(binary(unary(dout, "negative"), x, "multiply"), binary(y, y, "multiply"), "divide")
    if ns == "mod":
        if index == 0:
            return dout
        return unary(unary(binary(x, y, "divide"), "floor"), "negative")
    if ns in ("maximum", "minimum"):
        zeros = make_number(0, dout)
        cond = binary(y, z, "equal")
        return ternary(cond, dout, zeros) if index == 1 else ternary(cond, zeros, dout)
    if ns == "pow":
        if index == 0:
            d = binary(dout, y, "multiply")
            y_1 = binary(y, array(1), "subtract")
            return binary(d, binary(x, y_1, "pow"), "multiply")
        return binary(dout, binary(z, unary(x, "log"), "multiply"), "multiply")
    return None      # comparisons, logical and bitwise ops, floor_divide


def _op_grad(op, inputs, out, dout, index):
    x = inputs[index]
    if isinstance(op, UnaryOp):
        return _unary_grad(op, inputs[0], out, dout)
    if isinstance(op, BinaryOp):
        return _binary_grad(op, inputs[0], inputs[1], out, dout, index)
    if isinstance(op, TernaryOp):                       # ops/ternary_op.cc:49-56
        if index == 0:
            return None
        zeros = make_number(0, dout)
        return ternary(inputs[0], dout, zeros) if index == 1 else ternary(inputs[0], zeros, dout)
    if isinstance(op, BroadcastOp):                     # ops/broadcast_to_op.cc:112-117
        if op.bcast_mask == 0:
            return dout
        return core._reduce_mask(dout, "add", op.bcast_mask, op.keepdims_mask)
    if isinstance(op, ReduceOp):                        # ops/reduce_op.cc:339-362
        bc = lambda v: core._broadcast_mask(v, x.shape, op.reduce_mask, op.keepdims_mask)
        if op.op == "add":
            return bc(dout)
        if op.op == "multiply":
            return binary(bc(binary(dout, out, "multiply")), x, "divide")
        if op.op == "mean":
            a = bc(dout)
            return binary(a, make_number(1.0 * out.num / x.num, a), "multiply")
        if op.op in ("maximum", "minimum"):
            cond = binary(x, bc(out), "equal")
            return ternary(cond, bc(dout), make_number(0, x))
        return None
    if isinstance(op, ReindexOp):                       # ops/reindex_op.cc:76-80: no gradient for the extras
        if index:
            return None
        if getattr(op, "same_memory", False):           # a reshape: its gradient is the reshape back (ops/reshape_op.cc),
            from . import misc                          # which shares dout's buffer, instead of a scatter with atomics
            return misc.reshape(dout, list(x.shape))
        return reindex_reduce(dout, "add", x.shape, op.indexes, op.overflow_conditions, inputs[1:])
    if isinstance(op, ReindexReduceOp):                 # ops/reindex_reduce_op.cc:45-63
        if index:
            return None
        back = lambda v: reindex(v, x.shape, op.indexes, 0, op.overflow_conditions, inputs[1:])
        if op.op in ("add", "void"):                    # void (plain assignment, setitem_op.cc: the gradient of the value is the
            return back(dout)                           # gradient read back where it was written)
        if op.op == "multiply":
            return binary(back(binary(dout, out, "multiply")), x, "divide")
        if op.op in ("maximum", "minimum"):
            cond = binary(x, back(out), "equal")
            return ternary(cond, back(dout), make_number(0, x))
        return None
    return None


def grad(loss, targets, retain_graph=True):
    """jt.grad(loss, targets): list of d loss / d target (grad.cc:85-284).  The seed is ones of the
    loss's shape, so a non-scalar loss is summed implicitly, as in the reference."""
    single = isinstance(targets, Var)
    targets = [targets] if single else list(targets)
    if not loss.is_float():
        raise ValueError("Loss should be float")
    for t in targets:
        if not t.is_float():
            raise ValueError("Targets of grad should be float")

    # vars the loss depends on, through retained history
    nodes = {}
    stack = [loss]
    while stack:
        v = stack.pop()
        if v.id in nodes:
            continue
        nodes[v.id] = v
        if v._history is not None:
            stack.extend(v._history[1])
    # of those, the ones that depend on a target (ids grow from inputs to outputs)
    target_ids = {t.id for t in targets}
    order = sorted(nodes.values(), key=lambda v: v.id)
    dep = set()
    for v in order:
        if v.id in target_ids:
            dep.add(v.id)
        elif v._history is not None and any(u.id in dep for u in v._history[1]):
            dep.add(v.id)

    grads = {}
    if loss.id in dep:
        grads[loss.id] = make_number(1.0, loss)
    for v in reversed(order):
        g = grads.get(v.id)
        if g is None or v._history is None or v.id in target_ids and v._history is None:
            continue
        op, inputs = v._history
        for i, u in enumerate(inputs):
            if u.id not in dep or not u.is_float():
                continue
            saved = dt.amp_reg                                  # an op's gradient is built under the register
            dt.amp_reg |= getattr(op, "amp", 0)                 # the op was created with (grad.cc:48-55)
            try:
                du = _op_grad(op, inputs, v, g, i)
            finally:
                dt.amp_reg = saved
            if du is None:
                continue
            if du.shape != u.shape:
                raise RuntimeError("gradient of %r has shape %r, expected %r" % (op, du.shape, u.shape))
            grads[u.id] = du if u.id not in grads else binary(grads[u.id], du, "add")
    out = []
    for t in targets:
        g = grads.get(t.id)
        out.append(g if g is not None else make_number(0.0, t))
    return out[0] if single else out
