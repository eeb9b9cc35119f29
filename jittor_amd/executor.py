"""Executes pending Var graphs through libmjt.so.

Mirror of the part of Executor::run_sync that matters for this path
(python/jittor/src/executor.cc:200-716): collect the pending ops behind the
requested Vars, partition them into fused groups (element / broadcast ops
share a kernel, executor.cc:555; reduce, reindex and reindex_reduce start a
new one), recognise the convolution pattern the way ConvTuner does
(opt/tuner/conv_tuner.cc:218-411), allocate outputs and launch each group
once.  Everything runs on the device; there is no host path.
"""
import ctypes
import math

from . import _lib
from . import core
from .core import (Var, Buffer, UnaryOp, BinaryOp, TernaryOp, BroadcastOp,
                   ReduceOp, ReindexOp, ReindexReduceOp)
from ._lib import MjtError
from . import profiler as _profiler
from .flags import flags

stats = {"launches": 0, "fused_groups": 0, "fused_reduces": 0, "conv_matches": 0, "syncs": 0, "sunk_ops": 0, "matmul_matches": 0,
         "wgrad_kernel": 0, "wgrad_chunked": 0, "gather_reduces": 0, "fused_scatters": 0, "plans": 0, "replays": 0}


class ConvUnit:
    """reindex + broadcast + multiply + reduce.add matched as one convolution."""
    kind = "conv"
    fusable = False

    def __init__(self, reduce_op, x, w, params, absorbed, groups=1):
        self.out = reduce_op.out
        self.inputs = [x, w]
        self.params = params
        self.absorbed = absorbed
        self.groups = groups
        self.id = reduce_op.id


class GatherReduceUnit:
    """reindex -> reduce over the last axes of its result, run as one kernel that never writes the reindex result
    (the reference fuses a reindex with its consumer, executor.cc:555; pooling, pool.py:200-208)."""
    kind = "gather_reduce"
    fusable = False

    def __init__(self, reduce_op, reindex_op, nred, absorbed):
        self.out = reduce_op.out
        self.inputs = list(reindex_op.inputs)
        self.reindex = reindex_op
        self.op = reduce_op.op
        self.nred = nred
        self.absorbed = absorbed
        self.id = reduce_op.id


class MatmulUnit:
    """broadcast * broadcast -> reduce.add over 2-d operands matched as one matrix product
    (opt/tuner/matmul_tuner.cc:16-104)."""
    kind = "matmul"
    fusable = False

    def __init__(self, reduce_op, a, b, trans_a, trans_b):
        self.out = reduce_op.out
        self.inputs = [a, b]
        self.trans = (trans_a, trans_b)
        self.id = reduce_op.id


class ConvBwdDataUnit:
    """reindex_reduce.add <- multiply <- {broadcast(w), broadcast(dy)}: the gradient of the convolution with
    respect to its input (the pattern ConvTuner relays to conv_backward_x, conv_tuner.cc:375-397).  For
    stride 1 it is the forward kernel on dy with the weights flipped and transposed."""
    kind = "conv_bwd_x"
    fusable = False

    def __init__(self, root, dy, w, params, groups=1):
        self.out = root.out
        self.inputs = [dy, w]
        self.params = params
        self.groups = groups
        self.id = root.id


class ConvBwdWeightUnit:
    """reduce.add over (n, oh, ow) <- multiply <- {reindex(x), broadcast(dy)}: the gradient with respect to
    the weights (conv_backward_w).  It is the forward kernel with batch and channel axes of x and dy swapped,
    stride and dilation exchanged."""
    kind = "conv_bwd_w"
    fusable = False

    def __init__(self, root, x, dy, params, groups=1):
        self.out = root.out
        self.inputs = [x, dy]
        self.params = params
        self.groups = groups
        self.id = root.id


def _conv_affine(indexes, xshape, yshape):
    """Solves ['i0','i2','i3*s-p+i5*d','i4*s-p+i6*d'] for (sh, sw, ph, pw, dh, dw); None if it is not that."""
    aff = [_affine(s_, xshape, yshape) for s_ in indexes]
    if len(aff) != 4 or any(a_ is None for a_ in aff):
        return None

    def only(co, allowed):
        return all(co[k] == 0 for k in range(10) if k not in allowed)
    (c0n, con), (c0c, coc), (c0h, coh), (c0w, cow) = aff
    if c0n or c0c or con[0] != 1 or coc[2] != 1 or not only(con, (0,)) or not only(coc, (2,)):
        return None
    if not only(coh, (3, 5)) or not only(cow, (4, 6)):
        return None
    sh, dh, sw, dw = coh[3], coh[5], cow[4], cow[6]
    ph, pw = -c0h, -c0w
    if min(sh, dh, sw, dw) < 1 or ph < 0 or pw < 0:
        return None
    return sh, sw, ph, pw, dh, dw


def _lazy_op(v, cls):
    return v._op if (not v.materialised and isinstance(v._op, cls)) else None


_FLOAT_RANK = {"float16": 1, "bfloat16": 1, "float32": 2, "float64": 3}


def _lazy_broadcast(v):
    """The BroadcastOp behind v and the var it spreads, looking through float casts that change nothing:
    cast(broadcast(cast(s))) with only wider float types in between and v.dtype == s.dtype, which is what
    the gradient of a 16-bit convolution puts between dy and the product (the sum runs in float32,
    ops/reduce_op.cc:259-266).  Returns (op, source) or (None, None)."""
    chain = [v.dtype]
    u = v
    while not u.materialised and isinstance(u._op, UnaryOp) and u._op.op == "cast":
        u = u._op.inputs[0]
        chain.append(u.dtype)
    bo = _lazy_op(u, BroadcastOp)
    if bo is None:
        return None, None
    # behind the broadcast: go down through casts as far as they change nothing, i.e. to the deepest var of v's dtype
    # with only wider float types on the way (a var of v's dtype that is itself a narrowing cast stays what it is)
    def widening_only(types, r0):
        return all(_FLOAT_RANK.get(d, 0) > r0 or d == v.dtype for d in types)
    r0 = _FLOAT_RANK.get(v.dtype)
    src, best, below = bo.inputs[0], None, []
    while True:
        below.append(src.dtype)
        if src.dtype == v.dtype and r0 is not None and widening_only(chain + below, r0):
            best = src
        if src.materialised or not isinstance(src._op, UnaryOp) or src._op.op != "cast":
            break
        src = src._op.inputs[0]
    if best is None:
        if len(chain) == 1 and bo.inputs[0].dtype == v.dtype:
            return bo, bo.inputs[0]                      # no casts at all (any dtype)
        return None, None
    src = best
    return bo, src


def _match_conv_bwd(op):
    """The two gradient patterns of the meta-op convolution as jt.grad builds them."""
    if isinstance(op, ReindexReduceOp) and op.op == "add" and len(op.inputs) == 1 and not op.overflow_conditions:
        y7 = op.inputs[0]
        mul = _lazy_op(y7, BinaryOp)
        if mul is None or mul.op != "multiply" or y7.ndim != 7 or op.out.ndim != 4:
            return None
        params = _conv_affine(op.indexes, op.out.shape, y7.shape)
        if params is None:
            return None
        N, K, C, OH, OW, R, S = y7.shape
        for a, b in (mul.inputs, mul.inputs[::-1]):
            (ba, w), (bb, dy) = _lazy_broadcast(a), _lazy_broadcast(b)
            if ba is None or bb is None or ba.bcast_mask != 0b0011001 or bb.bcast_mask != 0b1100100:
                continue
            if list(w.shape) != [K, C, R, S] or list(dy.shape) != [N, K, OH, OW] or w.dtype != dy.dtype:
                continue
            if w.dtype not in ("float32", "bfloat16", "float16") or op.out.dtype not in ("float32", w.dtype):
                continue
            sh, sw, ph, pw, dh, dw = params
            if dh * (R - 1) - ph < 0 or dw * (S - 1) - pw < 0:
                continue
            H, W = op.out.shape[2], op.out.shape[3]
            if list(op.out.shape[:2]) != [N, C] or OH != (H + 2 * ph - dh * (R - 1) - 1) // sh + 1 \
                    or OW != (W + 2 * pw - dw * (S - 1) - 1) // sw + 1:
                continue
            return ConvBwdDataUnit(op, dy, w, params)
        return None
    if isinstance(op, ReduceOp) and op.op == "add" and op.reduce_mask == 0b0011001 and op.out.ndim == 4:
        y7 = op.inputs[0]
        if not y7.materialised and isinstance(y7._op, UnaryOp) and y7._op.op == "cast" and y7.dtype == "float32":
            y7 = y7._op.inputs[0]                             # 16-bit product summed in float32
        mul = _lazy_op(y7, BinaryOp)
        if mul is None or mul.op != "multiply" or y7.ndim != 7:
            return None
        N, K, C, OH, OW, R, S = y7.shape
        if list(op.out.shape) != [K, C, R, S]:
            return None
        for a, b in (mul.inputs, mul.inputs[::-1]):
            ra, (bb, dy) = _lazy_op(a, ReindexOp), _lazy_broadcast(b)
            if ra is None or bb is None or bb.bcast_mask != 0b1100100 or len(ra.inputs) != 1:
                continue
            if ra.overflow_conditions or ra.overflow_value != 0.0:
                continue
            x = ra.inputs[0]
            if x.ndim != 4 or list(dy.shape) != [N, K, OH, OW] or x.dtype != dy.dtype or x.shape[0] != N or x.shape[1] != C:
                continue
            if x.dtype not in ("float32", "bfloat16", "float16") or op.out.dtype not in ("float32", x.dtype):
                continue
            params = _conv_affine(ra.indexes, x.shape, y7.shape)
            if params is None:
                continue
            sh, sw, ph, pw, dh, dw = params
            H, W = x.shape[2], x.shape[3]
            # dy must be the output gradient of that convolution of x
            if OH != (H + 2 * ph - dh * (R - 1) - 1) // sh + 1 or OW != (W + 2 * pw - dw * (S - 1) - 1) // sw + 1:
                continue
            return ConvBwdWeightUnit(op, x, dy, params)
    return None


def _pending_ops(targets):
    """Pending producers behind `targets`, in topological order."""
    order, seen = [], set()
    stack = [(v, False) for v in targets]
    while stack:
        v, done = stack.pop()
        if v.materialised:
            continue
        op = v._op
        if done:
            if op.id not in seen:
                seen.add(op.id)
                order.append(op)
            continue
        if op.id in seen:
            continue
        stack.append((v, True))
        for u in op.inputs:
            if not u.materialised and u._op.id not in seen:
                stack.append((u, False))
    return order


def _affine(expr, xshape, yshape):
    return _lib.expr_affine(expr, xshape, yshape)


def _match_conv(red, consumers, targets):
    """reduce.add <- multiply <- {reindex(x), broadcast(w)} with
    xx = x.reindex([N,K,C,OH,OW,R,S], ['i0','i2','i3*s-p+i5*d','i4*s-p+i6*d']),
    ww = w.broadcast(xx.shape, [0,3,4]), sum over [2,5,6]
    (python/jittor/nn.py:1251-1262; matcher conv_tuner.cc:312-356)."""
    if red.op != "add" or red.reduce_mask != 0b1100100:
        return None
    yy = red.inputs[0]
    extra = set()
    if not yy.materialised and isinstance(yy._op, UnaryOp) and yy._op.op == "cast" and yy.dtype == "float32":
        # 16-bit inputs: the sum was rewritten to cast -> reduce(float32) -> cast (ops/reduce_op.cc:259-266);
        # fused, the product is an exact float temporary (opt/kernel_ir.cc:958-968), so the cast is a no-op
        extra.add(yy._op.id)
        yy = yy._op.inputs[0]
    if yy.materialised or yy.ndim != 7 or not isinstance(yy._op, BinaryOp) or yy._op.op != "multiply":
        return None
    a, b = yy._op.inputs
    for xx, ww in ((a, b), (b, a)):
        if xx.materialised or ww.materialised:
            continue
        ro, bo = xx._op, ww._op
        if not isinstance(ro, ReindexOp) or not isinstance(bo, BroadcastOp):
            continue
        if len(ro.inputs) != 1 or ro.overflow_conditions or ro.overflow_value != 0.0:
            continue
        x, w = ro.inputs[0], bo.inputs[0]
        if x.ndim != 4 or w.ndim != 4 or bo.bcast_mask != 0b0011001:
            continue
        if x.dtype != w.dtype or x.dtype not in ("float32", "bfloat16", "float16"):
            continue
        N, K, C, OH, OW, R, S = xx.shape
        if list(w.shape) != [K, C, R, S] or x.shape[0] != N or x.shape[1] != C:
            continue
        aff = [_affine(s, x.shape, xx.shape) for s in ro.indexes]
        if any(a_ is None for a_ in aff):
            continue
        def only(co, allowed):
            return all(co[k] == 0 for k in range(10) if k not in allowed)
        (c0n, con), (c0c, coc), (c0h, coh), (c0w, cow) = aff
        if c0n or c0c or con[0] != 1 or coc[2] != 1 or not only(con, (0,)) or not only(coc, (2,)):
            continue
        if not only(coh, (3, 5)) or not only(cow, (4, 6)):
            continue
        sh, dh, sw, dw = coh[3], coh[5], cow[4], cow[6]
        ph, pw = -c0h, -c0w
        if min(sh, dh, sw, dw) < 1 or ph < 0 or pw < 0:
            continue
        H, W = x.shape[2], x.shape[3]
        # the matcher checks oh / ow against the solved parameters (conv_tuner.cc:349-355)
        if OH != (H + 2 * ph - dh * (R - 1) - 1) // sh + 1 or OW != (W + 2 * pw - dw * (S - 1) - 1) // sw + 1:
            continue
        if red.out.dtype != "float32" and red.out.dtype != x.dtype:
            continue
        return ConvUnit(red, x, w, (sh, sw, ph, pw, dh, dw), {red.id, yy._op.id, ro.id, bo.id} | extra)
    return None


def _match_conv_grouped(op):
    """The grouped convolution as python/jittor/nn.py:1272-1294 writes it and its two gradients as jt.grad builds
    them, all over the 8-d product [N, G, K/G, C/G, OH, OW, R, S]:
        reindex_reduce.add <- multiply <- {reindex(a), reindex(b)}
    Each of x, w and y (or dy) has its own index pattern into that product; the one that is scattered into names the
    result (y: forward, x: input gradient, w: weight gradient), the other two are the gathered factors
    (the reference's tuner recognises the same three, opt/tuner/conv_tuner.cc:375-397)."""
    if op.op != "add" or len(op.inputs) != 1 or op.overflow_conditions or op.out.ndim != 4:
        return None
    yy = op.inputs[0]
    mul = _lazy_op(yy, BinaryOp)
    if mul is None or mul.op != "multiply" or yy.ndim != 8:
        return None
    N, G, KG, CG, OH, OW, R, S = yy.shape

    def is_sum(aff, terms, c0=0):
        """aff == c0 + sum(coef * i_k for k, coef in terms)"""
        return aff is not None and aff[0] == c0 and all(aff[1][k] == dict(terms).get(k, 0) for k in range(10))

    def role_of(exprs, vshape):
        """('y', None), ('w', None), ('x', params) or None for the index list of a var of shape vshape."""
        aff = [_affine(e, vshape, yy.shape) for e in exprs]
        if len(aff) != 4 or any(a_ is None for a_ in aff):
            return None
        if list(vshape) == [N, G * KG, OH, OW] and is_sum(aff[0], [(0, 1)]) and is_sum(aff[1], [(1, KG), (2, 1)]) \
                and is_sum(aff[2], [(4, 1)]) and is_sum(aff[3], [(5, 1)]):
            return "y", None
        if list(vshape) == [G * KG, CG, R, S] and is_sum(aff[0], [(1, KG), (2, 1)]) and is_sum(aff[1], [(3, 1)]) \
                and is_sum(aff[2], [(6, 1)]) and is_sum(aff[3], [(7, 1)]):
            return "w", None
        if vshape[0] == N and vshape[1] == G * CG and is_sum(aff[0], [(0, 1)]) and is_sum(aff[1], [(1, CG), (3, 1)]):
            (c0h, coh), (c0w, cow) = aff[2], aff[3]
            if any(coh[k] for k in range(10) if k not in (4, 6)) or any(cow[k] for k in range(10) if k not in (5, 7)):
                return None
            sh, dh, sw, dw, ph, pw = coh[4], coh[6], cow[5], cow[7], -c0h, -c0w
            if min(sh, dh, sw, dw) < 1 or ph < 0 or pw < 0:
                return None
            H, W = vshape[2], vshape[3]
            if OH != (H + 2 * ph - dh * (R - 1) - 1) // sh + 1 or OW != (W + 2 * pw - dw * (S - 1) - 1) // sw + 1:
                return None
            return "x", (sh, sw, ph, pw, dh, dw)
        return None

    target = role_of(op.indexes, op.out.shape)
    if target is None:
        return None
    found = {target[0]: (op.out, target[1])}
    ids = {op.id, mul.id}
    for v in mul.inputs:
        ro = _lazy_op(v, ReindexOp)
        if ro is None or len(ro.inputs) != 1 or ro.overflow_conditions:
            return None
        role = role_of(ro.indexes, ro.inputs[0].shape)
        if role is None or role[0] in found or (role[0] == "x" and ro.overflow_value != 0.0):
            return None
        found[role[0]] = (ro.inputs[0], role[1])
        ids.add(ro.id)
    (x, params), (w, _), (y, _) = found["x"], found["w"], found["y"]
    a, b = (v for r_, (v, _) in found.items() if r_ != target[0])
    if a.dtype != b.dtype or a.dtype not in ("float32", "bfloat16", "float16") or op.out.dtype not in ("float32", a.dtype):
        return None
    if target[0] == "y":
        return ConvUnit(op, x, w, params, ids, groups=G)
    if target[0] == "x":
        sh, sw, ph, pw, dh, dw = params
        if dh * (R - 1) - ph < 0 or dw * (S - 1) - pw < 0:
            return None
        return ConvBwdDataUnit(op, y, w, params, groups=G)
    return ConvBwdWeightUnit(op, x, y, params, groups=G)


def _match_gather_reduce(red, consumers, target_ids):
    """reduce(op) over the trailing axes of a reindex result."""
    if red.op not in ("add", "mean", "maximum", "minimum", "multiply"):
        return None
    xx, absorbed = red.inputs[0], {red.id}
    if not xx.materialised and isinstance(xx._op, UnaryOp) and xx._op.op == "cast" and xx.dtype == "float32" \
            and xx._op.inputs[0].dtype in ("float16", "bfloat16"):
        # a 16-bit sum or mean was rewritten to cast -> reduce(float32) -> cast: the kernel accumulates in float32 anyway
        if xx.id in target_ids:
            return None
        absorbed.add(xx._op.id)
        xx = xx._op.inputs[0]
    ro = _lazy_op(xx, ReindexOp)
    # other readers of the reindex result do not matter: the unit reads the reindex's own input, and the reindex
    # itself still runs if somebody needs its result in memory
    if ro is None or xx.id in target_ids or getattr(xx, "_stop_fuse", False):
        return None
    if getattr(ro, "same_memory", False) and flags["reshape_shares_memory"]:
        return None            # a reshape costs nothing by itself: the plain reduce kernels read its input's bytes
    nd, nred = xx.ndim, bin(red.reduce_mask).count("1")
    if nred < 1 or red.reduce_mask != ((1 << nred) - 1) << (nd - nred) or red.out.dtype == "bool":
        return None
    tail = 1
    for n in xx.shape[nd - nred:]:
        tail *= n
    if tail > 128:
        return None            # one lane walks the folded elements: beyond a pooling window the two-kernel path is faster
    absorbed.add(ro.id)
    return GatherReduceUnit(red, ro, nred, absorbed)


_matmul_ok = []


def _match_matmul(red):
    """reduce.add <- multiply <- {broadcast(xx), broadcast(yy)}: the three layouts the reference relays to its
    matmul op (matmul_tuner.cc:33-83), either operand order.  xx and yy are 2-d and the product 3-d, or all
    carry the same leading batch extents (the batched product nn.matmul hands to cublas_batched_matmul,
    python/jittor/nn.py:127-131)."""
    yy = red.inputs[0]
    if red.op != "add":
        return None
    if not yy.materialised and isinstance(yy._op, UnaryOp) and yy._op.op == "cast" and yy.dtype == "float32":
        yy = yy._op.inputs[0]                                 # 16-bit inputs: cast -> reduce(float32) -> cast
    nd = yy.ndim
    if yy.materialised or nd < 3 or not isinstance(yy._op, BinaryOp) or yy._op.op != "multiply":
        return None
    nb = nd - 3                                               # leading batch axes
    rm = red.reduce_mask >> nb
    if red.reduce_mask & ((1 << nb) - 1) or rm not in (0b001, 0b010, 0b100):
        return None
    a, b = yy._op.inputs
    if a.materialised or b.materialised or not isinstance(a._op, BroadcastOp) or not isinstance(b._op, BroadcastOp):
        return None
    xa, xb = a._op.inputs[0], b._op.inputs[0]
    am, bm = a._op.bcast_mask, b._op.bcast_mask
    if xa.ndim != nb + 2 or xb.ndim != nb + 2 or xa.dtype != xb.dtype or not xa.is_float():
        return None
    if (am | bm) & ((1 << nb) - 1) or xa.shape[:nb] != yy.shape[:nb] or xb.shape[:nb] != yy.shape[:nb]:
        return None                                           # a batch axis that is broadcast: not a plain batched product
    if red.out.dtype != xa.dtype and not (red.out.dtype == "float32" and xa.dtype in ("float16", "bfloat16")):
        return None
    table = {(0b010, 0b100, 0b001): (False, False), (0b001, 0b100, 0b010): (True, False), (0b100, 0b010, 0b001): (False, True)}
    for (p, q, pm, qm) in ((xa, xb, am >> nb, bm >> nb), (xb, xa, bm >> nb, am >> nb)):
        t = table.get((rm, pm, qm))
        if t is None:
            continue
        if not _matmul_ok:
            _matmul_ok.append(bool(_lib.load().mjt_matmul_available()))
        return MatmulUnit(red, p, q, t[0], t[1]) if _matmul_ok[0] else None
    return None


# ---- replay of a graph that was executed before -----------------------------------------------------
# The reference keeps what it worked out for a fused group and finds it again by the group's key
# (executor.cc:55-110, load_fused_op and the jit cache behind it); a training step asks for the same graph every time.
# Here the first execution of a graph records what it handed to the library: every call with its argument objects,
# and for every pointer and by-value scalar inside them the var it came from.  A later graph with the same signature
# (ops, their attributes, shapes, types, wiring, which results are asked for, flags) skips matching, partitioning and
# descriptor building: its vars get their buffers the way the recorded run gave them out, the pointers and scalars
# are written into the recorded argument objects, and the recorded calls are issued again.
class _VarPtr(int):
    """A device address that remembers the var (and the offset inside it) it was taken from."""

    def __new__(cls, value, var, off=0):
        o = int.__new__(cls, value)
        o.var, o.off = var, off
        return o

    def __add__(self, n):
        return _VarPtr(int(self) + n, self.var, self.off + n)

    __radd__ = __add__


class _Capture:
    def __init__(self, lib):
        self.lib = lib
        self.calls = []          # (library function, argument tuple) of every call that succeeded
        self.ptrs = []           # (struct or array, index or None, var, offset): a pointer field and where it came from
        self.scalars = []        # (FusedVar array, index, var): a by-value scalar and the host var it came from

    def __getattr__(self, name):                             # stands in for the library while recording
        fn = getattr(self.lib, name)
        if name == "mjt_matmul_available":
            return fn

        def call(*args):
            rc = fn(*args)
            if rc == 0:
                self.calls.append((fn, args))
            return rc
        return call


class _Plan:
    __slots__ = ("slots", "needs_ptr", "produce", "ptrs", "scalars", "calls", "stats", "cleared")


_cap = None
_plans = {}
_PLAN_LIMIT = 512


def _libh():
    return _cap if _cap is not None else _lib.ensure_init()


def _op_sig(op):
    if isinstance(op, (UnaryOp, BinaryOp)):
        return (op.kind, op.op)
    if isinstance(op, TernaryOp):
        return (op.kind,)
    if isinstance(op, BroadcastOp):
        return (op.kind, op.bcast_mask, op.keepdims_mask)
    if isinstance(op, ReduceOp):
        return (op.kind, op.op, op.reduce_mask, op.keepdims_mask)
    if isinstance(op, ReindexOp):
        return (op.kind, tuple(op.indexes), op.overflow_value, tuple(op.overflow_conditions), getattr(op, "same_memory", False))
    if isinstance(op, ReindexReduceOp):
        return (op.kind, op.op, tuple(op.indexes), tuple(op.overflow_conditions))
    return None


def _signature(ops, target_ids):
    """Hashable description of everything the execution of `ops` depends on besides the data, or None."""
    pos, leaf, parts = {}, {}, []
    for i, op in enumerate(ops):
        sig = _op_sig(op)
        out = op.out
        if sig is None or out is None:
            return None
        ins = []
        for u in op.inputs:
            k = pos.get(u.id)
            if k is not None:
                ins.append(k)
                continue
            l = leaf.get(u.id)
            if l is None:
                l = leaf[u.id] = len(leaf)
                ins.append((l, tuple(u.shape), u.dtype, u._op is None, u._buf is None, u._host is not None,
                            getattr(u, "_stop_fuse", False)))
            else:
                ins.append(-1 - l)
        pos[out.id] = i
        parts.append((sig, tuple(out.shape), out.dtype, out.id in target_ids, out._buf is None, getattr(out, "_stop_fuse", False),
                      tuple(ins)))
    return (tuple(parts), tuple(sorted((k, str(v)) for k, v in flags.items())), dt_amp())


def dt_amp():
    from . import dtypes
    return dtypes.amp_reg


def _capture(ops, target_ids, sig):
    """Executes `ops` and records the execution as a plan under `sig` (or marks the signature as not replayable)."""
    global _cap
    # a var's place in the graph: result of op i, or input j of op i (the first place it is seen at)
    slot_of, slots, held = {}, [], []
    made = {op.out.id for op in ops}
    for i, op in enumerate(ops):
        for j, u in enumerate(op.inputs):
            if u.id not in made and id(u) not in slot_of:
                slot_of[id(u)] = len(slots)
                slots.append(("in", i, j))
                held.append(u)
        slot_of[id(op.out)] = len(slots)
        slots.append(("out", i))
        held.append(op.out)
    had_inputs = [bool(op.inputs) for op in ops]
    before = dict(stats)
    cap = _cap = _Capture(_lib.ensure_init())
    try:
        _execute(ops, target_ids)
    finally:
        _cap = None
    plan = _Plan()
    # vars made during the execution (rearranged weights, column matrices, partial sums): a buffer of their own per replay
    def slot(v):
        k = slot_of.get(id(v))
        if k is None:
            if v._buf is None:
                return None
            k = slot_of[id(v)] = len(slots)
            slots.append(("tmp", v._buf.size))
            held.append(v)
        return k
    plan.ptrs, plan.scalars, needs_ptr = [], [], set()
    for obj, idx, v, off in cap.ptrs:
        k = slot(v)
        if k is None:
            _plans[sig] = False
            return
        plan.ptrs.append((obj, idx, k, off))
        needs_ptr.add(k)
    for arr, idx, v in cap.scalars:
        k = slot_of.get(id(v))
        if k is None or slots[k][0] != "in":
            _plans[sig] = False
            return
        plan.scalars.append((arr, idx, k))
    # who owns which buffer: inputs first, then the vars made on the way, then the results in the order of the ops
    owner, produce = {}, []
    for k, d in enumerate(slots):
        if d[0] != "out" and held[k]._buf is not None:
            owner.setdefault(id(held[k]._buf), k)
    for k, d in enumerate(slots):
        if d[0] != "out":
            continue
        buf = held[k]._buf
        if buf is None:
            continue
        src = owner.get(id(buf))
        if src is None:
            owner[id(buf)] = k
            produce.append((k, -1))
        else:
            produce.append((k, src))
            needs_ptr.add(src)
    plan.slots, plan.needs_ptr, plan.produce, plan.calls = slots, needs_ptr, produce, cap.calls
    plan.stats = [(key, stats[key] - before[key]) for key in stats if stats[key] != before[key]]
    plan.cleared = [(i, had_inputs[i] and not op.inputs) for i, op in enumerate(ops) if op.out is not None and op.out._op is None]
    if len(_plans) >= _PLAN_LIMIT:
        _plans.clear()
    _plans[sig] = plan
    stats["plans"] += 1


def _replay(plan, ops):
    slots = plan.slots
    n = len(slots)
    var, buf, base = [None] * n, [None] * n, [0] * n
    needs_ptr = plan.needs_ptr
    for k, d in enumerate(slots):
        kind = d[0]
        if kind == "in":
            v = var[k] = ops[d[1]].inputs[d[2]]
            if k in needs_ptr:
                base[k] = v._device_ptr()
                buf[k] = v._buf
        elif kind == "out":
            var[k] = ops[d[1]].out
        else:
            b = buf[k] = Buffer(d[1])
            base[k] = b.ptr
    for k, src in plan.produce:
        v = var[k]
        if src >= 0:
            v._buf = buf[src]
        elif v._buf is None:
            v._buf = Buffer(max(v.nbytes, 1))
        buf[k] = v._buf
        base[k] = v._buf.ptr
    for obj, idx, k, off in plan.ptrs:
        if idx is None:
            obj.ptr = base[k] + off
        else:
            obj[idx].ptr = base[k] + off
    for arr, idx, k in plan.scalars:
        fv = arr[idx]
        fv.fvalue, fv.ivalue = _scalar_value(var[k])
    check = _lib.check
    for fn, args in plan.calls:
        rc = fn(*args)
        if rc:
            check(rc)
    for key, d in plan.stats:
        stats[key] += d
    for i, clear_inputs in plan.cleared:
        op = ops[i]
        op.out._op = None
        if clear_inputs:
            op.inputs = []
    stats["replays"] += 1


def run_sync(targets, device_sync=False):
    targets = [t for t in targets if isinstance(t, Var)]
    stats["syncs"] += 1
    _lib.ensure_init()
    ops = _pending_ops(targets)
    if ops:
        target_ids = {t.id for t in targets}
        sig = _signature(ops, target_ids) if flags["enable_replay"] and _cap is None and _profiler.active() is None else None
        plan = _plans.get(sig) if sig is not None else False
        if plan is None:
            _capture(ops, target_ids, sig)
        elif plan is False:
            _execute(ops, target_ids)
        else:
            _replay(plan, ops)
    for t in targets:
        t._device_ptr()
    if device_sync:
        _lib.sync()


def _execute(ops, target_ids):
    consumers = {}
    for op in ops:
        for u in op.inputs:
            consumers.setdefault(u.id, []).append(op)

    # ---- convolution patterns -------------------------------------------------
    # A matched root op is replaced by a unit that reads the convolution's operands directly.  What the
    # units no longer read (the 7-d reindex / broadcast / product vars) is dropped by the liveness pass
    # below unless something else still consumes it.
    units = {}
    if flags["enable_conv_match"]:
        for op in ops:
            cu = None
            if isinstance(op, ReduceOp):
                cu = _match_conv(op, consumers, target_ids)
            if cu is None and isinstance(op, (ReduceOp, ReindexReduceOp)):
                cu = _match_conv_bwd(op)
            if cu is None and isinstance(op, ReindexReduceOp):
                cu = _match_conv_grouped(op)
            if cu is not None:
                units[op.id] = cu
                stats["conv_matches"] += 1
            elif isinstance(op, ReduceOp) and flags["enable_matmul_match"]:
                cu = _match_matmul(op)
                if cu is not None:
                    units[op.id] = cu
                    stats["matmul_matches"] += 1
            if cu is None and isinstance(op, ReduceOp) and flags["enable_gather_reduce"]:
                cu = _match_gather_reduce(op, consumers, target_ids)
                if cu is not None:
                    units[op.id] = cu
                    stats["gather_reduces"] += 1
    nodes = [units.get(op.id, op) for op in ops]
    produced_by = {node.out.id: node for node in nodes}
    needed = set()
    stack = list(target_ids)
    while stack:
        node = produced_by.get(stack.pop())
        if node is None or node.id in needed:
            continue
        needed.add(node.id)
        stack.extend(u.id for u in node.inputs)
    sched = [node for node in nodes if node.id in needed]
    consumers = {}
    for node in sched:
        for u in node.inputs:
            consumers.setdefault(u.id, []).append(node)

    # ---- element ops whose result is only ever broadcast move behind the broadcast ------------
    # broadcast(f(a, b)) == f(broadcast(a), broadcast(b)): the small op then runs inside the kernel of the
    # broadcast's consumers (recomputed per element) instead of as a launch of its own, as the reference's
    # fuser does with cheap shared producers (executor.cc:466-474; test_new_fused_op.py:24-40: a
    # normalisation is three kernels).  pre[b.id] = the ops to evaluate at b's output shape, in order;
    # leaves[b.id] = the vars they read through b's broadcast mask.
    pre, leaves = {}, {}
    if flags["enable_broadcast_sink"]:
        producer0 = {node.out.id: node for node in sched}
        sinkable = {}
        for node in reversed(sched):
            users = consumers.get(node.out.id, ())
            const = isinstance(node, BroadcastOp) and node.inputs[0]._op is None and node.inputs[0]._host is not None \
                and node.inputs[0].num == 1                  # a number spread over a small shape stays a number
            ok = (const or isinstance(node, (UnaryOp, BinaryOp, TernaryOp))) and node.out.id not in target_ids and users \
                and node.out._buf is None and not getattr(node.out, "_stop_fuse", False)
            if ok:
                for c in users:
                    if not (isinstance(c, BroadcastOp) or (sinkable.get(c.id) and c.out.shape == node.out.shape)):
                        ok = False
                        break
            if ok:
                for u in node.inputs:
                    if not (u.shape == node.out.shape or (u._op is None and u._host is not None and u.num == 1)):
                        ok = False
                        break
            sinkable[node.id] = bool(ok)
        for node in sched:
            if not isinstance(node, BroadcastOp):
                continue
            p = producer0.get(node.inputs[0].id)
            if p is None or not sinkable.get(p.id):
                continue
            chain, seen, lv = [], set(), []

            def visit(op):
                if op.id in seen:
                    return
                seen.add(op.id)
                for u in op.inputs:
                    q = producer0.get(u.id)
                    if q is not None and sinkable.get(q.id):
                        visit(q)
                    elif not any(u is w for w in lv):
                        lv.append(u)
                chain.append(op)

            visit(p)
            if len(chain) <= 32:
                pre[node.id], leaves[node.id] = chain, lv
        # a sunk op runs on its own only if some broadcast could not take its chain
        taken = set()
        for bid, chain in pre.items():
            taken.update(op.id for op in chain)
        left = {node.id for node in sched if isinstance(node, BroadcastOp) and node.id not in pre}
        keep_ids = set()
        stack = [producer0[node.inputs[0].id] for node in sched
                 if node.id in left and node.inputs[0].id in producer0 and producer0[node.inputs[0].id].id in taken]
        while stack:
            op = stack.pop()
            if op.id in keep_ids:
                continue
            keep_ids.add(op.id)
            stack.extend(producer0[u.id] for u in op.inputs if u.id in producer0 and producer0[u.id].id in taken)
        dropped = taken - keep_ids
        if dropped:
            stats["sunk_ops"] += len(dropped)
            sched = [node for node in sched if node.id not in dropped]

    def ins(op):
        return leaves.get(op.id, op.inputs)

    consumers = {}
    for node in sched:
        for u in ins(node):
            consumers.setdefault(u.id, []).append(node)

    # ---- stages: an op can share a kernel with its producer only inside a stage ---------
    producer = {}
    for op in sched:
        producer[op.out.id] = op
    stage = {}
    for op in sched:
        s = 0
        for u in ins(op):
            p = producer.get(u.id)
            if p is None:
                continue
            step = 0
            if not p.fusable or not op.fusable:
                step = 1 if not p.fusable else 0
            if isinstance(op, BroadcastOp) or (op.fusable and p.fusable and p.out.shape != op.out.shape):
                step = 1
            if getattr(u, "_stop_fuse", False):
                step = 1
            s = max(s, stage[p.id] + step)
        stage[op.id] = s
    # An element or broadcast op whose consumers all run in later stages waits for them: it then shares their
    # kernel instead of writing its result to memory first (`(x - mean) / std`: the subtraction could run as
    # soon as the mean is known, but belongs in the kernel of the division, which has to wait for std).
    for op in reversed(sched):
        if not op.fusable or op.out.id in target_ids or op.out._buf is not None:
            continue
        latest = None
        for c in consumers.get(op.out.id, ()):
            lim = stage[c.id]
            if isinstance(c, BroadcastOp) or getattr(op.out, "_stop_fuse", False) or (c.fusable and c.out.shape != op.out.shape):
                lim -= 1                                      # the consumer reads this result from memory
            latest = lim if latest is None else min(latest, lim)
        if latest is not None and latest > stage[op.id]:
            stage[op.id] = latest

    # ---- union element ops into groups ---------------------------------------------
    parent = {}

    def find(a):
        while parent[a] != a:
            parent[a] = parent[parent[a]]
            a = parent[a]
        return a

    for op in sched:
        parent[op.id] = op.id
    for op in sched:
        if not op.fusable:
            continue
        for u in op.inputs:
            p = producer.get(u.id)
            if p is not None and p.fusable and stage[p.id] == stage[op.id] and p.out.shape == op.out.shape \
                    and not isinstance(op, BroadcastOp) and not getattr(u, "_stop_fuse", False):
                parent[find(op.id)] = find(p.id)
    groups = {}
    for op in sched:
        if op.fusable:
            groups.setdefault(find(op.id), []).append(op)

    # ---- run stage by stage: element groups first, then the other ops ---------------------
    nstage = max(stage.values()) + 1 if stage else 0
    by_stage_groups = [[] for _ in range(nstage)]
    by_stage_other = [[] for _ in range(nstage)]
    for root, members in groups.items():
        by_stage_groups[stage[members[0].id]].append(members)
    for op in sched:
        if not op.fusable:
            by_stage_other[stage[op.id]].append(op)
    # a group whose single result feeds one reduce of the same stage becomes that reduce's prologue: the
    # result is never written to memory (element, broadcast and reduce ops share a group, executor.cc:555)
    prologue_of = {}
    absorbed_groups = set()
    if flags["enable_reduce_fusion"]:
        for members in (m for st in by_stage_groups for m in st):
            ids = {op.id for op in members}
            outs = [op.out for op in members
                    if op.out.id in target_ids or any(c.id not in ids for c in consumers.get(op.out.id, ()))]
            if len(outs) != 1 or outs[0].id in target_ids:
                continue
            users = consumers.get(outs[0].id, ())
            if len(users) != 1 or not isinstance(users[0], ReduceOp) or users[0].id in prologue_of:
                continue
            if stage[users[0].id] != stage[members[0].id] or outs[0].shape != members[-1].out.shape:
                continue
            prologue_of[users[0].id] = members
            absorbed_groups.add(id(members))
    # a group whose single result is what one reindex_reduce of the same stage scatters becomes that scatter's
    # prologue; a reindex with the scatter's own index program whose result only the group reads (the forward
    # pass's window tensor in a pooling gradient) is read through that program instead of being computed
    scatter_of, absorbed_nodes = {}, set()
    if flags["enable_scatter_fusion"]:
        for members in (m for st in by_stage_groups for m in st):
            if id(members) in absorbed_groups:
                continue
            ids = {op.id for op in members}
            outs = [op.out for op in members
                    if op.out.id in target_ids or any(c.id not in ids for c in consumers.get(op.out.id, ()))]
            if len(outs) != 1 or outs[0].id in target_ids:
                continue
            users = consumers.get(outs[0].id, ())
            if len(users) != 1 or not isinstance(users[0], ReindexReduceOp) or users[0].id in scatter_of:
                continue
            rr = users[0]
            if stage[rr.id] != stage[members[0].id] or outs[0].shape != members[-1].out.shape or rr.inputs[0].id != outs[0].id \
                    or any(e.id == outs[0].id for e in rr.inputs[1:]):
                continue
            gathered = {}
            for op in members:
                for u in op.inputs:
                    p = producer.get(u.id)
                    if isinstance(p, ReindexOp) and p.id not in ids and u._buf is None and u.id not in target_ids \
                            and p.indexes == rr.indexes and p.overflow_conditions == rr.overflow_conditions \
                            and [e.id for e in p.inputs[1:]] == [e.id for e in rr.inputs[1:]] \
                            and list(p.inputs[0].shape) == list(rr.out.shape) and not isinstance(op, BroadcastOp) \
                            and all(c.id in ids for c in consumers.get(u.id, ())):
                        gathered[u.id] = p
            scatter_of[rr.id] = (members, gathered)
            absorbed_groups.add(id(members))
            absorbed_nodes.update(p.id for p in gathered.values())

    def group_io(members, extra_out=None):
        ids = {op.id for op in members}
        made = {op.out.id for op in members}
        read = {}
        for op in members:
            for u in ins(op):
                if u.id not in made and not (u._op is None and u._host is not None and u.num == 1):
                    read[u.id] = u.nbytes
        outs = sum(op.out.nbytes for op in members
                   if extra_out is None and (op.out.id in target_ids or any(c.id not in ids for c in consumers.get(op.out.id, ()))))
        return sum(read.values()), outs + (extra_out.nbytes if extra_out is not None else 0)

    def timed(call, kind, io):
        rec = _profiler.active()
        return call() if rec is None else rec.run(call, kind, *io())

    for s in range(nstage):
        for members in by_stage_groups[s]:
            if id(members) not in absorbed_groups:
                timed(lambda: _run_group(members, consumers, target_ids, pre=pre), "fused", lambda: group_io(members))
        for op in by_stage_other[s]:
            if op.id in absorbed_nodes:
                continue
            sc = scatter_of.get(op.id)
            if sc is not None:
                if timed(lambda: _run_group(sc[0], consumers, target_ids, scatter=op, gathered=sc[1], pre=pre), "fused+scatter",
                         lambda: group_io(sc[0], op.out)):
                    continue
                for p in sc[1].values():                       # not taken in that form: the plain sequence
                    timed(lambda: _run_single(p), p.kind, lambda: (sum(u.nbytes for u in p.inputs), p.out.nbytes))
                timed(lambda: _run_group(sc[0], consumers, target_ids, pre=pre), "fused", lambda: group_io(sc[0]))
            members = prologue_of.get(op.id)
            if members is not None:
                if timed(lambda: _run_group(members, consumers, target_ids, reduce=op, pre=pre), "fused+reduce",
                         lambda: group_io(members, op.out)):
                    continue
                timed(lambda: _run_group(members, consumers, target_ids, pre=pre), "fused", lambda: group_io(members))
            timed(lambda: _run_single(op), op.kind, lambda: (sum(u.nbytes for u in op.inputs), op.out.nbytes))
    # materialised vars become leaves: the graph behind them can be dropped
    for op in sched:
        if op.out._buf is not None:
            op.out._op = None
            op.inputs = []


def _alloc_out(v):
    if v._buf is None:
        v._buf = Buffer(max(v.nbytes, 1))
    return v._buf.ptr if _cap is None else _VarPtr(v._buf.ptr, v)


def _ptr_of(v):
    p = v._device_ptr()
    return p if _cap is None else _VarPtr(p, v)


def _tensor(ptr, dtype, shape):
    t = _lib.tensor(ptr, dtype, shape)
    if _cap is not None and isinstance(ptr, _VarPtr):
        _cap.ptrs.append((t, None, ptr.var, ptr.off))
    return t


def _tensor_of(v):
    return _tensor(_ptr_of(v), v.dtype, v.shape)


def _tensor_array(vs):
    arr = (_lib.Tensor * max(1, len(vs)))(*[_lib.tensor(v._device_ptr(), v.dtype, v.shape) for v in vs])
    if _cap is not None:
        for i, v in enumerate(vs):
            _cap.ptrs.append((arr, i, v, 0))
    return arr


def _scalar_value(u):
    """(fvalue, ivalue) of a one-element host array that goes into a kernel by value (ops/array_op.cc:56-60)"""
    if u.dtype == "bfloat16":
        from .dtypes import bf16_bits_to_f32
        return float(bf16_bits_to_f32(u._host).reshape(-1)[0]), 0
    h = u._host.reshape(-1)[0]
    return (float(h), 0) if u.is_float() else (0.0, int(h))


def _run_single(op):
    lib = _libh()
    out = op.out
    stats["launches"] += 1
    if isinstance(op, ReduceOp):
        x = op.inputs[0]
        tx = _tensor_of(x)
        ty = _tensor(_alloc_out(out), out.dtype, out.shape)
        _lib.check(lib.mjt_reduce(ctypes.byref(tx), ctypes.byref(ty), _lib.OP_CODE[op.op], op.reduce_mask))
    elif isinstance(op, ReindexOp):
        x, extras = op.inputs[0], op.inputs[1:]
        if getattr(op, "same_memory", False) and flags["reshape_shares_memory"]:
            x._device_ptr()                                    # a row-major reinterpretation: the same bytes
            out._buf = x._buf
            stats["launches"] -= 1
            return
        tx = _tensor_of(x)
        ty = _tensor(_alloc_out(out), out.dtype, out.shape)
        ex = _tensor_array(extras)
        _lib.check(lib.mjt_reindex(ctypes.byref(tx), ctypes.byref(ty), len(op.indexes), _lib.c_strings(op.indexes),
                                   op.overflow_value, len(op.overflow_conditions),
                                   _lib.c_strings(op.overflow_conditions), len(extras), ex))
    elif isinstance(op, ReindexReduceOp):
        y, extras = op.inputs[0], op.inputs[1:]
        ty = _tensor_of(y)
        tx = _tensor(_alloc_out(out), out.dtype, out.shape)
        ex = _tensor_array(extras)
        _lib.check(lib.mjt_reindex_reduce(ctypes.byref(ty), ctypes.byref(tx), _lib.OP_CODE[op.op], len(op.indexes),
                                          _lib.c_strings(op.indexes), len(op.overflow_conditions),
                                          _lib.c_strings(op.overflow_conditions), len(extras), ex))
    elif isinstance(op, ConvUnit):
        x, w = op.inputs
        tx, tw = _tensor_of(x), _tensor_of(w)
        ty = _tensor(_alloc_out(out), out.dtype, out.shape)
        p = _lib.ConvParams(*op.params)
        if op.groups > 1:
            _lib.check(lib.mjt_conv2d_meta_grouped(ctypes.byref(tx), ctypes.byref(tw), ctypes.byref(ty), ctypes.byref(p),
                                                   op.groups))
        else:
            _lib.check(lib.mjt_conv2d_meta(ctypes.byref(tx), ctypes.byref(tw), ctypes.byref(ty), ctypes.byref(p)))
    elif isinstance(op, GatherReduceUnit):
        ro = op.reindex
        x, extras = ro.inputs[0], ro.inputs[1:]
        tx = _tensor_of(x)
        ts = _tensor(0, x.dtype, ro.out.shape)                       # the reindex result: its shape only
        tz = _tensor(_alloc_out(out), out.dtype, out.shape)
        ex = _tensor_array(extras)
        _lib.check(lib.mjt_reindex_then_reduce(ctypes.byref(tx), ctypes.byref(ts), ctypes.byref(tz), _lib.OP_CODE[op.op], op.nred,
                                               len(ro.indexes), _lib.c_strings(ro.indexes), ro.overflow_value,
                                               len(ro.overflow_conditions), _lib.c_strings(ro.overflow_conditions),
                                               len(extras), ex))
    elif isinstance(op, MatmulUnit):
        a, b = op.inputs
        n = a.shape[-1] if op.trans[0] else a.shape[-2]
        k = b.shape[-2] if op.trans[1] else b.shape[-1]
        ta, tb = _tensor_of(a), _tensor_of(b)
        # a kept reduced axis of extent 1 changes nothing in memory
        tc = _tensor(_alloc_out(out), out.dtype, list(a.shape[:-2]) + [n, k])
        _lib.check(lib.mjt_matmul(ctypes.byref(ta), ctypes.byref(tb), ctypes.byref(tc), int(op.trans[0]), int(op.trans[1])))
    elif isinstance(op, ConvBwdDataUnit):
        dy, w = op.inputs
        sh, sw, ph, pw, dh, dw = op.params
        K, C, R, S = w.shape
        G = op.groups
        if G == 1:
            # the library's own entry: transposed, flipped weights for stride 1, one convolution per stride phase otherwise
            td, tw = _tensor_of(dy), _tensor_of(w)
            tx = _tensor(_alloc_out(out), out.dtype, out.shape)
            p = _lib.ConvParams(sh, sw, ph, pw, dh, dw)
            _lib.check(lib.mjt_conv2d_meta_dgrad(ctypes.byref(td), ctypes.byref(tw), ctypes.byref(tx), ctypes.byref(p)))
            return
        with core.no_grad():
            if G > 1:
                # w [G*Kg, Cg, R, S] -> [G*Cg, Kg, R, S]: transposed within each group, taps flipped
                kg = K // G
                wt = core.reindex(w, [G * C, kg, R, S], ["i0/%d*%d+i1" % (C, kg), "i0%%%d" % C, "%d-i2" % (R - 1), "%d-i3" % (S - 1)])
            else:
                wt = core.reindex(w, [C, K, R, S], ["i1", "i0", "%d-i2" % (R - 1), "%d-i3" % (S - 1)])
        _run_single(wt._op)
        if sh != 1 or sw != 1:
            # a strided convolution's input gradient is the stride-1 one of dy with sh-1 (sw-1) zeros between its rows
            # (columns) and zeros up to the size that makes the result H x W: one reindex, out of range reads 0
            H, W = out.shape[2], out.shape[3]
            with core.no_grad():
                dy = core.reindex(dy, [dy.shape[0], K, H + 2 * ph - dh * (R - 1), W + 2 * pw - dw * (S - 1)],
                                  ["i0", "i1", "i2/%d" % sh, "i3/%d" % sw], 0.0, ["i2%%%d!=0" % sh, "i3%%%d!=0" % sw])
            _run_single(dy._op)
        tx, tw = _tensor_of(dy), _tensor_of(wt)
        ty = _tensor(_alloc_out(out), out.dtype, out.shape)
        p = _lib.ConvParams(1, 1, dh * (R - 1) - ph, dw * (S - 1) - pw, dh, dw)
        if G > 1:
            _lib.check(lib.mjt_conv2d_meta_grouped(ctypes.byref(tx), ctypes.byref(tw), ctypes.byref(ty), ctypes.byref(p), G))
        else:
            _lib.check(lib.mjt_conv2d_meta(ctypes.byref(tx), ctypes.byref(tw), ctypes.byref(ty), ctypes.byref(p)))
    elif isinstance(op, ConvBwdWeightUnit) and op.groups > 1:
        x, dy = op.inputs
        tx, td = _tensor_of(x), _tensor_of(dy)
        tw = _tensor(_alloc_out(out), out.dtype, out.shape)
        p = _lib.ConvParams(*op.params)
        _lib.check(lib.mjt_conv2d_meta_wgrad_grouped(ctypes.byref(tx), ctypes.byref(td), ctypes.byref(tw), ctypes.byref(p), op.groups))
    elif isinstance(op, ConvBwdWeightUnit):
        x, dy = op.inputs
        sh, sw, ph, pw, dh, dw = op.params
        N, C, H, W = x.shape
        _, K, OH, OW = dy.shape
        R, S = out.shape[2], out.shape[3]
        # (the kernel walks rows in chunks of 32 output columns: a width that fills less than 0.6 of its chunks and is no
        # multiple of 8 is better off as a product, 64 x 256 x 14 x 14 3x3: 68 us on the kernel, 59 as the product below)
        narrow = OW % 8 != 0 and OW < 0.6 * 32 * -(-OW // 32)
        if x.dtype in ("bfloat16", "float16") and flags["enable_conv_wgrad_kernel"] and not narrow:
            # the MFMA kernel; shapes it does not cover come back as unsupported and take the paths below
            tx, td = _tensor_of(x), _tensor_of(dy)
            tw = _tensor(_alloc_out(out), out.dtype, out.shape)
            p = _lib.ConvParams(sh, sw, ph, pw, dh, dw)
            rc = lib.mjt_conv2d_meta_wgrad(ctypes.byref(tx), ctypes.byref(td), ctypes.byref(tw), ctypes.byref(p))
            if rc == 0:
                stats["wgrad_kernel"] += 1
                return
            if rc != _lib.ERR_UNSUPPORTED:
                _lib.check(rc)
        if not _matmul_ok:
            _matmul_ok.append(bool(lib.mjt_matmul_available()))
        if _matmul_ok[0] and flags["enable_matmul_match"]:
            # dw[k, (c,r,s)] = sum over images of dy[n] [K, P] times cols[n]^T, cols[n] = the shifted input planes
            # [(c,r,s), P] (P = OH*OW, the innermost axis of both): one reindex per chunk of images, one
            # batched GEMM per chunk, one sum over the images.
            esz = _lib.DTYPE_SIZE[x.dtype]
            P, CRS = OH * OW, C * R * S
            pdt = "float32" if x.dtype in ("float16", "bfloat16") else x.dtype
            # 16-bit planes that are no 16-byte multiples (14 x 14, 7 x 7, 13 x 13 maps) would send every image's
            # product to the kernel without MFMAs.  The sum over images and pixels is one contraction: with the images of
            # a chunk side by side, dw = sum over chunks of dy' [K, nb*P] times cols' [(c,r,s), nb*P]^T, where nb images
            # make nb*P a multiple of 64 elements (the product kernel that copies its operands straight into LDS wants
            # that), or of 8.  Few chunks: long sums on large tiles and few partial results (us of kernels, bf16, 3x3,
            # 64 images: 256 x 14 x 14 -> 256: 441 -> 99; 512 x 7 x 7 -> 512: 632 -> 61).  Planes that are 16-byte
            # multiples stay with the product per image (128 x 28 x 28 -> 128: 159 us against 165 this way).
            nb0 = next((a // math.gcd(P, a) for a in (64, 8) if N % (a // math.gcd(P, a)) == 0), 0)
            if esz == 2 and (P * esz) % 16 != 0 and nb0 and CRS * N * P * esz <= (1 << 30):
                tiles = -(-K // 128) * -(-CRS // 128)
                chunks = N // nb0                                  # most chunks there can be
                while chunks % 2 == 0 and (chunks // 2) * tiles >= 256:
                    chunks //= 2
                nb = N // chunks
                L = nb * P
                stats["wgrad_chunked"] += 1
                with core.no_grad():
                    dyc = core.reindex(dy, [chunks, K, nb, OH, OW], ["i0*%d+i2" % nb, "i1", "i3", "i4"])
                    colsc = core.reindex(x, [chunks, C, R, S, nb, OH, OW],
                                         ["i0*%d+i4" % nb, "i1", "i5*%d-%d+i2*%d" % (sh, ph, dh), "i6*%d-%d+i3*%d" % (sw, pw, dw)], 0.0)
                _run_single(dyc._op)
                _run_single(colsc._op)
                ta = _tensor(_ptr_of(dyc), dy.dtype, [chunks, K, L])
                tb = _tensor(_ptr_of(colsc), x.dtype, [chunks, CRS, L])
                if chunks == 1:                                    # the product is the result, in the weights' dtype
                    tp = _tensor(_alloc_out(out), out.dtype, [1, K, CRS])
                    _lib.check(lib.mjt_matmul(ctypes.byref(ta), ctypes.byref(tb), ctypes.byref(tp), 0, 1))
                    stats["launches"] += 1
                    return
                part = Var([chunks, K, CRS], pdt)
                tp = _tensor(_alloc_out(part), pdt, [chunks, K, CRS])
                _lib.check(lib.mjt_matmul(ctypes.byref(ta), ctypes.byref(tb), ctypes.byref(tp), 0, 1))
                stats["launches"] += 1
                acc = out if out.dtype == pdt else Var([K, C, R, S], pdt)
                tpart = _tensor(_ptr_of(part), pdt, [chunks, K * CRS])
                tacc = _tensor(_alloc_out(acc), pdt, [K * CRS])
                _lib.check(lib.mjt_reduce(ctypes.byref(tpart), ctypes.byref(tacc), _lib.OP_CODE["add"], 0b01))
                if acc is not out:                                 # narrow the float32 sum to the weights' dtype
                    with core.no_grad():
                        narrowed = core.unary(acc, out.dtype)
                    _run_group([narrowed._op], {}, {narrowed.id})
                    out._buf = narrowed._buf
                return
            chunk = max(1, min(N, (1 << 30) // max(1, CRS * P * esz)))
            cols = Var([chunk, C, R, S, OH, OW], x.dtype)
            part = Var([N, K, CRS], pdt)
            cols_ptr, part_ptr = _alloc_out(cols), _alloc_out(part)
            idx = _lib.c_strings(["i0", "i1", "i4*%d-%d+i2*%d" % (sh, ph, dh), "i5*%d-%d+i3*%d" % (sw, pw, dw)])
            none, ex = _lib.c_strings([]), (_lib.Tensor * 1)()
            psz = _lib.DTYPE_SIZE[pdt]
            for n0 in range(0, N, chunk):
                nb = min(chunk, N - n0)
                tx = _tensor(_ptr_of(x) + n0 * C * H * W * esz, x.dtype, [nb, C, H, W])
                tc = _tensor(cols_ptr, x.dtype, [nb, C, R, S, OH, OW])
                _lib.check(lib.mjt_reindex(ctypes.byref(tx), ctypes.byref(tc), 4, idx, 0.0, 0, none, 0, ex))
                ta = _tensor(_ptr_of(dy) + n0 * K * P * esz, dy.dtype, [nb, K, P])
                tb = _tensor(cols_ptr, x.dtype, [nb, CRS, P])
                tp = _tensor(part_ptr + n0 * K * CRS * psz, pdt, [nb, K, CRS])
                _lib.check(lib.mjt_matmul(ctypes.byref(ta), ctypes.byref(tb), ctypes.byref(tp), 0, 1))
                stats["launches"] += 2
            acc = out if out.dtype == pdt else Var([K, C, R, S], pdt)
            tpart = _tensor(part_ptr, pdt, [N, K * CRS])
            tacc = _tensor(_alloc_out(acc), pdt, [K * CRS])
            _lib.check(lib.mjt_reduce(ctypes.byref(tpart), ctypes.byref(tacc), _lib.OP_CODE["add"], 0b01))
            if acc is not out:                                 # narrow the float32 sum to the weights' dtype
                with core.no_grad():
                    narrowed = core.unary(acc, out.dtype)
                _run_group([narrowed._op], {}, {narrowed.id})
                out._buf = narrowed._buf
            return
        with core.no_grad():
            xt = core.reindex(x, [C, N, H, W], ["i1", "i0", "i2", "i3"])
            dyt = core.reindex(dy, [K, N, OH, OW], ["i1", "i0", "i2", "i3"])
        _run_single(xt._op)
        _run_single(dyt._op)
        # as a convolution of x^T [C,N,H,W] with dy^T [K,N,OH,OW] (stride d, dilation s); rows and columns of x that
        # the stride never reaches make its output larger than R x S: the reindex below keeps the first R x S taps
        tmp = Var([C, K, (H + 2 * ph - sh * (OH - 1) - 1) // dh + 1, (W + 2 * pw - sw * (OW - 1) - 1) // dw + 1], out.dtype)
        tx, tw = _tensor_of(xt), _tensor_of(dyt)
        tt = _tensor(_alloc_out(tmp), tmp.dtype, tmp.shape)
        p = _lib.ConvParams(dh, dw, ph, pw, sh, sw)              # stride and dilation trade places
        _lib.check(lib.mjt_conv2d_meta(ctypes.byref(tx), ctypes.byref(tw), ctypes.byref(tt), ctypes.byref(p)))
        ty = _tensor(_alloc_out(out), out.dtype, out.shape)
        idx, none = _lib.c_strings(["i1", "i0", "i2", "i3"]), _lib.c_strings([])
        ex = (_lib.Tensor * 1)()
        _lib.check(lib.mjt_reindex(ctypes.byref(tt), ctypes.byref(ty), 4, idx, 0.0, 0, none, 0, ex))
    else:
        raise MjtError(-2, "no kernel for op %r" % (op,))


def _run_group(members, consumers, target_ids, reduce=None, pre=None, scatter=None, gathered=None):
    """One launch for a group of element / broadcast ops.  With `reduce` (the ReduceOp that consumes the
    group's only result) the group runs as that reduce's prologue; returns False when the library does
    not take the group in that form (a tensor broadcast inside it), True otherwise."""
    lib = _libh()
    member_ids = {op.id for op in members}
    shape = members[-1].out.shape
    fvars, fops, prov = [], [], []
    index = {}           # (var id, bcast mask) -> fused var index
    keep = []            # keeps arrays alive

    def add_var(role, dtype, ptr=None, fvalue=0.0, ivalue=0, mask=0, scalar=None):
        fv = _lib.FusedVar()
        fv.role, fv.dtype, fv.ptr = role, _lib.DTYPE_CODE[dtype], ptr
        fv.fvalue, fv.ivalue, fv.bcast_mask = float(fvalue), int(ivalue), mask
        fvars.append(fv)
        if _cap is not None:                                  # where the pointer / the value came from, for replays
            prov.append((len(fvars) - 1, ptr.var, ptr.off) if isinstance(ptr, _VarPtr) else (len(fvars) - 1, scalar, None) if scalar is not None else None)
        return len(fvars) - 1

    def external(u, mask):
        key = (u.id, mask)
        if key in index:
            return index[key]
        if gathered and u.id in gathered:
            i = add_var(_lib.VAR_GATHERED, u.dtype, ptr=_ptr_of(gathered[u.id].inputs[0]))
            index[key] = i
            return i
        if u._op is None and u._host is not None and u.num == 1:
            # one-element host array: by-value kernel argument (ops/array_op.cc:56-60)
            fval, ival = _scalar_value(u)
            i = add_var(_lib.VAR_SCALAR, u.dtype, fvalue=fval, ivalue=ival, scalar=u)
        else:
            i = add_var(_lib.VAR_INPUT, u.dtype, ptr=_ptr_of(u), mask=mask)
        index[key] = i
        return i

    def add_op(op, ins, oi):
        fo = _lib.FusedOp()
        if isinstance(op, UnaryOp):
            fo.kind, fo.op = _lib.FOP_UNARY, _lib.OP_CODE[op.op]
        elif isinstance(op, BinaryOp):
            fo.kind, fo.op = _lib.FOP_BINARY, _lib.OP_CODE[op.op]
        elif isinstance(op, TernaryOp):
            fo.kind, fo.op = _lib.FOP_TERNARY, 0
        else:
            fo.kind, fo.op = _lib.FOP_BROADCAST, 0
        for j, v in enumerate(ins):
            fo.inp[j] = v
        fo.out = oi
        fops.append(fo)
        return oi

    outputs = []
    for op in members:
        ins = []
        if isinstance(op, BroadcastOp) and pre and op.id in pre:
            # the element ops in front of this broadcast, evaluated per element of its output: what they read
            # is loaded through the broadcast's mask
            full = (1 << len(shape)) - 1
            mask = op.bcast_mask & full
            local = {}
            for q in pre[op.id]:
                qin = [local[u.id] if u.id in local else external(u, mask) for u in q.inputs]
                local[q.out.id] = add_op(q, qin, add_var(_lib.VAR_INTERMEDIATE, q.out.dtype))
            ins.append(local[op.inputs[0].id])
        elif isinstance(op, BroadcastOp):
            u = op.inputs[0]
            full = (1 << len(shape)) - 1
            ins.append(external(u, op.bcast_mask & full))
        else:
            for u in op.inputs:
                p = u._op
                if p is not None and p.id in member_ids and u._buf is None:
                    ins.append(index[(u.id, 0)])
                else:
                    ins.append(external(u, 0))
        out = op.out
        used_outside = out.id in target_ids or any(c.id not in member_ids for c in consumers.get(out.id, ()))
        if used_outside:
            oi = add_var(_lib.VAR_OUTPUT, out.dtype, ptr=None if reduce is not None or scatter is not None else _alloc_out(out))
            outputs.append(out)
        else:
            oi = add_var(_lib.VAR_INTERMEDIATE, out.dtype)
        index[(out.id, 0)] = oi
        add_op(op, ins, oi)
    if not outputs:
        return True
    desc = _lib.FusedDesc()
    desc.ndim = len(shape)
    for i, s in enumerate(shape):
        desc.shape[i] = s
    varr = (_lib.FusedVar * len(fvars))(*fvars)
    oarr = (_lib.FusedOp * len(fops))(*fops)
    desc.n_vars, desc.vars, desc.n_ops, desc.ops = len(fvars), varr, len(fops), oarr
    if _cap is not None:
        for pv in prov:
            if pv is not None and pv[2] is not None:
                _cap.ptrs.append((varr, pv[0], pv[1], pv[2]))
            elif pv is not None:
                _cap.scalars.append((varr, pv[0], pv[1]))
    if scatter is not None:
        rout, extras = scatter.out, scatter.inputs[1:]
        had_buf = rout._buf is not None
        tx = _tensor(_alloc_out(rout), rout.dtype, rout.shape)
        ex = _tensor_array(extras)
        rc = lib.mjt_fused_reindex_reduce(ctypes.byref(desc), ctypes.byref(tx), _lib.OP_CODE[scatter.op], len(scatter.indexes),
                                          _lib.c_strings(scatter.indexes), len(scatter.overflow_conditions),
                                          _lib.c_strings(scatter.overflow_conditions), len(extras), ex)
        if rc == _lib.ERR_UNSUPPORTED:
            if not had_buf:
                rout._buf = None
            return False
        _lib.check(rc)
        stats["launches"] += 1
        stats["fused_scatters"] += 1
        return True
    if reduce is not None:
        rout = reduce.out
        had_buf = rout._buf is not None
        ty = _tensor(_alloc_out(rout), rout.dtype, rout.shape)
        rc = lib.mjt_fused_reduce(ctypes.byref(desc), ctypes.byref(ty), _lib.OP_CODE[reduce.op], reduce.reduce_mask)
        if rc == -2:                                   # MJT_ERR_UNSUPPORTED: run the two kernels instead
            if not had_buf:
                rout._buf = None
            return False
        _lib.check(rc)
        stats["launches"] += 1
        stats["fused_reduces"] += 1
        return True
    stats["launches"] += 1
    stats["fused_groups"] += 1
    _lib.check(lib.mjt_fused_elementwise(ctypes.byref(desc)))
    return True
