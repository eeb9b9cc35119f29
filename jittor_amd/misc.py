"""Callers of the meta-operator path: the library functions the reference
writes with reindex / reindex_reduce / reduce, with the same signatures.

gather / scatter (python/jittor/misc.py:1563-1640), pad
(python/jittor/nn.py:1679-1700), pool (python/jittor/pool.py:200-208, the
meta-operator branch), transpose / permute, reshape, flip, basic slicing.
Everything here only builds Var graphs; execution is the path's kernels.
"""
import numbers

import numpy as np

from . import core
from .core import Var, reindex, reindex_reduce, ternary, binary, array, broadcast


def gather(x, dim, index):
    """out[i][j][k] = x[index[i][j][k]][j][k] (dim 0), ... (misc.py:1617-1640)."""
    nd = index.ndim
    if x.ndim != nd:
        raise ValueError("gather: index must have the rank of x")
    dim = dim + nd if dim < 0 else dim
    args = ",".join("i%d" % i for i in range(nd))
    idx = ["i%d" % i for i in range(nd)]
    idx[dim] = "@e0(%s)" % args
    return reindex(x, index.shape, idx, extras=[index])


def scatter(x, dim, index, src, reduce="void"):
    """x[index[i][j][k]][j][k] = src[i][j][k] (dim 0), ...; reduce 'void' (assign), 'add' or 'multiply'
    (misc.py:1563-1612).  Built from reindex_reduce: the scattered tensor starts from the op's identity,
    and for 'void' a count of updates per element selects between it and x."""
    if reduce not in ("void", "add", "multiply"):
        raise ValueError("scatter: reduce must be 'void', 'add' or 'multiply'")
    nd = index.ndim
    if x.ndim != nd:
        raise ValueError("scatter: index must have the rank of x")
    dim = dim + nd if dim < 0 else dim
    src = core._as_var(src)
    if src.num == 1 and list(src.shape) != list(index.shape):
        src = broadcast(src.cast(x.dtype) if src.dtype != x.dtype else src, index.shape)
    elif list(src.shape) != list(index.shape):
        src = src[tuple(slice(None, s) for s in index.shape)]
    if src.dtype != x.dtype:
        src = src.cast(x.dtype)
    args = ",".join("i%d" % i for i in range(nd))
    idx = ["i%d" % i for i in range(nd)]
    idx[dim] = "@e0(%s)" % args
    upd = reindex_reduce(src, reduce, x.shape, idx, extras=[index])
    if reduce == "add":
        return x + upd
    if reduce == "multiply":
        return x * upd
    one = broadcast(array(1, "int32"), index.shape)
    hit = reindex_reduce(one, "add", x.shape, idx, extras=[index])
    return ternary(hit > 0, upd, x)


def pad(x, padding, mode="constant", value=0):
    """padding = (left_last, right_last, left_prev, right_prev, ...) as nn.py:1679-1700."""
    if mode not in ("constant", "replicate", "reflect", "circular"):
        raise ValueError("only support constant,replicate,reflect,circular pad")
    padding = list(padding)
    if len(padding) % 2 or len(padding) // 2 > x.ndim:
        raise ValueError("pad: bad padding %r for rank %d" % (padding, x.ndim))
    left = [0] * (x.ndim - len(padding) // 2) + padding[::2][::-1]
    right = [0] * (x.ndim - len(padding) // 2) + padding[1::2][::-1]
    dims, shape = [], []
    for i, (n, l, r) in enumerate(zip(x.shape, left, right)):
        shape.append(n + l + r)
        if mode == "constant":
            dims.append("i%d-%d" % (i, l))
        elif mode == "replicate":
            dims.append("i%d<%d ? 0 : i%d > %d ? %d : i%d-%d" % (i, l, i, n + l - 1, n - 1, i, l))
        elif mode == "reflect":
            dims.append("i%d<%d ? %d-i%d : i%d > %d ? %d-i%d : i%d-%d" % (i, l, l, i, i, n + l - 1, 2 * (n - 1) + l, i, i, l))
        else:
            dims.append("i%d<%d ? %d+i%d : i%d > %d ? i%d-%d : i%d-%d" % (i, l, n - l, i, i, n + l - 1, i, n + l, i, l))
    return reindex(x, shape, dims, overflow_value=value)


def _pair(v):
    return (v, v) if isinstance(v, numbers.Integral) else tuple(v)


def pool(x, kernel_size, op, padding=0, stride=None):
    """2-d pooling of an NCHW Var as reindex + reduce (pool.py:200-208): window elements outside the
    image take the reindex overflow value 0, as in the reference's meta-operator branch."""
    kh, kw = _pair(kernel_size)
    sh, sw = _pair(stride if stride else kernel_size)
    ph, pw = _pair(padding)
    if op not in ("maximum", "minimum", "mean", "add"):
        raise ValueError("pool: op %r" % (op,))
    N, C, H, W = x.shape
    h = (H + ph * 2 - kh) // sh + 1
    w = (W + pw * 2 - kw) // sw + 1
    xx = reindex(x, [N, C, h, w, kh, kw], ["i0", "i1", "i2*%d-%d+i4" % (sh, ph), "i3*%d-%d+i5" % (sw, pw)])
    return core.reduce(xx, op, [4, 5])


def _lib_storage(dtype):
    from . import _lib
    return _lib.NP_STORAGE[dtype]


def where(cond, x=None, y=None):
    """jt.where(cond) -> one int32 index Var per axis of cond holding the positions where cond is non-zero, in
    row-major order (python/jittor/src/ops/where_op.cc:20-60; the result's length depends on the data, so cond is
    computed here); jt.where(cond, x, y) = ternary(cond, x, y) (:42-45)."""
    cond = core._as_var(cond)
    if x is not None or y is not None:
        if x is None or y is None:
            raise ValueError("where: give both x and y, or neither")
        return ternary(cond, x, y)
    import ctypes
    from . import _lib
    cond.sync()
    lib = _lib.ensure_init()
    tc = _lib.tensor(cond.raw_ptr(), cond.dtype, cond.shape)
    count = ctypes.c_int64()
    _lib.check(lib.mjt_where_count(ctypes.byref(tc), ctypes.byref(count)))
    n = count.value
    outs = [array(np.zeros(n, np.int32)) for _ in range(cond.ndim)]
    if n:
        to = (_lib.Tensor * cond.ndim)(*[_lib.tensor(o.raw_ptr(), "int32", [n]) for o in outs])
        _lib.check(lib.mjt_where(ctypes.byref(tc), n, to))
        for o in outs:
            o._host = None                              # the device buffer now holds the value
    for o in outs:
        o.is_scalar = False                             # an index list of one entry is no fused number
    return tuple(outs)


def concat(arr, dim=0):
    """jt.concat (python/jittor/contrib.py:22-58): every part is reindexed into the result's shape at its offset
    along `dim` (0 elsewhere) and the parts are added."""
    arr = [core._as_var(a) for a in arr]
    if not arr:
        raise ValueError("concat: empty list")
    nd = arr[0].ndim
    if dim < 0:
        dim += nd
    if not 0 <= dim < nd:
        raise ValueError("concat: dim %d out of range for rank %d" % (dim, nd))
    total = sum(a.shape[dim] for a in arr)
    indexes = ["i%d" % i for i in range(nd)]
    out, at = None, 0
    for a in arr:
        if a.ndim != nd or any(a.shape[i] != arr[0].shape[i] for i in range(nd) if i != dim):
            raise ValueError("concat: shapes %s and %s differ outside dim %d" % (list(arr[0].shape), list(a.shape), dim))
        shape = list(a.shape)
        shape[dim] = total
        indexes[dim] = "i%d-%d" % (dim, at)
        b = a.reindex(shape, list(indexes))
        if len(arr) >= 100:
            b.stop_fuse()
        out = b if out is None else out + b
        at += a.shape[dim]
    return out


def permute(x, *dims):
    if len(dims) == 1 and isinstance(dims[0], (list, tuple)):
        dims = tuple(dims[0])
    if not dims:
        dims = tuple(range(x.ndim))[::-1]
    dims = [d + x.ndim if d < 0 else d for d in dims]
    if sorted(dims) != list(range(x.ndim)):
        raise ValueError("permute: %r is not a permutation of the axes" % (dims,))
    idx = [None] * x.ndim
    for out_axis, in_axis in enumerate(dims):
        idx[in_axis] = "i%d" % out_axis
    return reindex(x, [x.shape[d] for d in dims], idx)


def transpose(x, *dims):
    return permute(x, *dims)


def flip(x, dim=0):
    dims = [dim] if isinstance(dim, numbers.Integral) else list(dim)
    dims = [d + x.ndim if d < 0 else d for d in dims]
    idx = ["%d-i%d" % (x.shape[i] - 1, i) if i in dims else "i%d" % i for i in range(x.ndim)]
    return reindex(x, x.shape, idx)


def reshape(x, *shape):
    """Row-major reinterpretation.  In the graph it is a reindex through the flat offset, so gradients and pattern
    matching see an ordinary op; when it runs, the result shares its input's buffer and nothing is launched (the
    reference aliases the buffer too, python/jittor/src/ops/reshape_op.cc)."""
    if len(shape) == 1 and isinstance(shape[0], (list, tuple)):
        shape = tuple(shape[0])
    shape = list(shape)
    total = x.num
    if shape.count(-1) > 1:
        raise ValueError("reshape: more than one -1")
    if -1 in shape:
        known = 1
        for s in shape:
            if s != -1:
                known *= s
        if known == 0 or total % known:
            raise ValueError("reshape: cannot infer -1 for %r from %d elements" % (shape, total))
        shape[shape.index(-1)] = total // known
    n = 1
    for s in shape:
        n *= s
    if n != total:
        raise ValueError("reshape: %r has %d elements, the Var has %d" % (shape, n, total))
    if shape == list(x.shape):
        return x
    # flat offset of the output coordinate, then the input coordinate it corresponds to
    flat, stride = [], 1
    for i in range(len(shape) - 1, -1, -1):
        flat.append("i%d*%d" % (i, stride))
        stride *= shape[i]
    flat = "(" + "+".join(flat[::-1]) + ")"
    idx, stride = [], 1
    for d in range(x.ndim - 1, -1, -1):
        idx.append("%s/%d%%%d" % (flat, stride, x.shape[d]))
        stride *= x.shape[d]
    y = reindex(x, shape, idx[::-1])
    y._op.same_memory = True             # values are functional (assign rebinds, nothing writes in place): sharing is safe
    return y


def _parse_key(x, key):
    """Splits an index into, per axis of x, what selects it: returns (out_shape, exprs, extras) where exprs[d] is
    the index expression of axis d of x in terms of the coordinates of the selection.  Integer Vars (also lists and
    numpy integer arrays, of any rank) index their axes together: they are broadcast against each other, right
    aligned, into one block of output dims that stands where the first of them stood
    (python/jittor/src/ops/getitem_op.cc:76-113)."""
    if not isinstance(key, tuple):
        key = (key,)
    key = tuple(array(np.asarray(k)) if isinstance(k, (list, np.ndarray)) else k for k in key)
    if sum(1 for k in key if k is Ellipsis) > 1:
        raise IndexError("an index can only have a single ellipsis")
    # a boolean mask stands for as many axes as it has dims
    width = lambda k: 0 if k is None or k is Ellipsis else k.ndim if isinstance(k, Var) and k.dtype == "bool" else 1
    n_real = sum(width(k) for k in key)
    if n_real > x.ndim:
        raise IndexError("too many indices for a Var of rank %d" % x.ndim)
    full, axis = [], 0
    for k in key:
        if k is Ellipsis:
            full.extend([slice(None)] * (x.ndim - n_real))
            axis += x.ndim - n_real
        elif isinstance(k, Var) and k.dtype == "bool":
            # a boolean mask selects the positions where it is true: the index Vars of where(mask), one per axis it covers
            # (the result's size depends on the data; python/jittor/src/ops/where_op.cc)
            if list(k.shape) != list(x.shape[axis:axis + k.ndim]):
                raise IndexError("boolean mask of shape %s does not match axes %d..%d of shape %s"
                                 % (list(k.shape), axis, axis + k.ndim - 1, list(x.shape)))
            full.extend(where(k))
            axis += k.ndim
        else:
            full.append(k)
            axis += width(k)
    full.extend([slice(None)] * (x.ndim - sum(1 for k in full if k is not None)))
    index_vars = [k for k in full if isinstance(k, Var)]
    for k in index_vars:
        if k.dtype == "bool" or k.is_float():
            raise IndexError("only integer Vars index an axis, got %s" % k.dtype)
    var_dim = max([k.ndim for k in index_vars], default=0)
    block = [1] * var_dim                                  # the index Vars' common shape
    for k in index_vars:
        for j in range(k.ndim):
            have, want = block[var_dim - 1 - j], k.shape[k.ndim - 1 - j]
            if have != want and have != 1 and want != 1:
                raise IndexError("index Vars of shapes %s do not broadcast" % [list(v.shape) for v in index_vars])
            block[var_dim - 1 - j] = want if have == 1 else have      # (an extent of 0 stays 0: an empty selection)
    out_shape, exprs, extras = [], [], []
    axis = 0
    first_var_dim = -1                                     # output dim where the block starts
    for k in full:
        if k is None:
            out_shape.append(1)
            continue
        n = x.shape[axis]
        if isinstance(k, numbers.Integral):
            k = int(k)
            if k < -n or k >= n:
                raise IndexError("index %d is out of bounds for axis %d with size %d" % (k, axis, n))
            exprs.append(str(k + n if k < 0 else k))
        elif isinstance(k, slice):
            start, stop, step = k.indices(n)
            count = len(range(start, stop, step))
            exprs.append("%d+i%d*(%d)" % (start, len(out_shape), step))
            out_shape.append(count)
        elif isinstance(k, Var):
            if first_var_dim < 0:
                first_var_dim = len(out_shape)
                out_shape.extend(block)
            # the Var's own dims, right aligned in the block; an extent of 1 reads element 0 along that dim
            coords = ["i%d" % (first_var_dim + var_dim - k.ndim + j) if k.shape[j] != 1 else "0" for j in range(k.ndim)]
            exprs.append("@e%d(%s)" % (len(extras), ",".join(coords)))
            extras.append(k)
        else:
            raise IndexError("unsupported index %r" % (k,))
        axis += 1
    return out_shape, exprs, extras


def getitem(x, key):
    """Indexing with integers, slices (positive or negative step), None, Ellipsis and integer Vars / lists / numpy
    arrays of any rank (broadcast against each other as in the reference); one reindex
    (python/jittor/src/ops/getitem_op.cc)."""
    out_shape, exprs, extras = _parse_key(x, key)
    if not out_shape:
        out_shape = [1]
    if 0 in out_shape:                                  # an empty selection (a mask that is false everywhere): nothing to launch
        return array(np.zeros(out_shape, _lib_storage(x.dtype)), x.dtype)
    return reindex(x, out_shape, exprs, extras=extras)


def setitem(x, key, value):
    """x[key] = value (python/jittor/src/ops/setitem_op.cc): the same keys as getitem.  The value, broadcast to
    the selection, is scattered into a tensor of x's shape (reindex_reduce 'void' with the selection's index
    expressions), a scatter of ones marks the cells that were written, and a ternary takes the new value there
    and x elsewhere (the construction of misc.scatter); x is rebound to the result.  With an index Var that holds
    duplicates, which of the values lands is undefined, as in the reference."""
    out_shape, exprs, extras = _parse_key(x, key)
    if not out_shape:
        out_shape = [1]
    if 0 in out_shape:                                  # nothing selected: x stays as it is
        return x
    value = core._as_var(value)
    if value.dtype != x.dtype:
        value = value.cast(x.dtype)
    vs = list(value.shape)
    if len(vs) > len(out_shape) and all(s == 1 for s in vs[:len(vs) - len(out_shape)]):
        value = reshape(value, vs[len(vs) - len(out_shape):])
    if list(value.shape) != out_shape:
        value = broadcast(value, out_shape)
    upd = reindex_reduce(value, "void", x.shape, exprs, extras=extras)
    one = broadcast(array(1, "int32"), out_shape)
    hit = reindex_reduce(one, "add", x.shape, exprs, extras=extras)
    old = x._split_off_value()                          # the ternary reads the old value, x is rebound to its result
    return x.assign(ternary(hit > 0, upd, old))


Var.gather = gather
Var.scatter = scatter
Var.permute = permute
Var.transpose = transpose
Var.reshape = reshape
Var.view = reshape
Var.flip = flip
Var.__getitem__ = getitem
Var.__setitem__ = lambda self, key, value: (setitem(self, key, value), None)[1]
Var.setitem = setitem
Var.where = where
