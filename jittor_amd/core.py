"""Lazy Var graph and op constructors of the meta-operator path.

Python mirror of the reference's graph layer for this path only:
Var (python/jittor/src/var.h:18-49), the op constructors with their rewrites
(ops/binary_op.cc:421-474, ops/unary_op.cc:860-889, ops/ternary_op.cc:21-47,
ops/broadcast_to_op.cc:23-168, ops/reduce_op.cc:257-337,
ops/reindex_op.cc:20-91, ops/reindex_reduce_op.cc:26-73, ops/array_op.cc:54-80).
Nothing executes until a Var is synchronised (lazy_execution,
var_holder.cc:25-33); execution is in executor.py.
"""
import math
import numbers
import weakref

import numpy as np

from . import _lib
from . import dtypes as dt
from ._lib import MjtError
from .flags import flags as _flags

_next_id = [0]
_grad_enabled = [True]


class no_grad:
    """Vars created inside keep no history (jt.no_grad, python/jittor/__init__.py)."""

    def __enter__(self):
        self._prev = _grad_enabled[0]
        _grad_enabled[0] = False
        return self

    def __exit__(self, *exc):
        _grad_enabled[0] = self._prev
        return False


def _new_id():
    _next_id[0] += 1
    return _next_id[0]


# --------------------------------------------------------------------------
# device buffers: freed blocks are kept per size and reused.  All work is
# queued on one stream, so reuse without a synchronisation is ordered.
# --------------------------------------------------------------------------
class _Pool:
    def __init__(self):
        self.free_blocks = {}
        self.cached_bytes = 0
        self.limit = 8 << 30

    @staticmethod
    def _round(n):
        n = max(int(n), 256)
        if n <= (1 << 20):
            return 1 << (n - 1).bit_length()
        return (n + (1 << 20) - 1) >> 20 << 20

    def alloc(self, nbytes):
        size = self._round(nbytes)
        lst = self.free_blocks.get(size)
        if lst:
            self.cached_bytes -= size
            return lst.pop(), size
        try:
            return _lib.alloc(size), size
        except MjtError:
            self.release_all()
            return _lib.alloc(size), size

    def free(self, ptr, size):
        if _lib.device() is None:
            return
        if self.cached_bytes + size > self.limit:
            _lib.free(ptr)
            return
        self.free_blocks.setdefault(size, []).append(ptr)
        self.cached_bytes += size

    def release_all(self):
        for lst in self.free_blocks.values():
            for p in lst:
                _lib.free(p)
        self.free_blocks.clear()
        self.cached_bytes = 0


pool = _Pool()


class Buffer:
    """Owns one device allocation."""

    def __init__(self, nbytes):
        self.ptr, self.size = pool.alloc(nbytes)

    def __del__(self):
        try:
            pool.free(self.ptr, self.size)
        except Exception:
            pass


# --------------------------------------------------------------------------
# ops
# --------------------------------------------------------------------------
class Op:
    kind = "op"
    fusable = False        # element / broadcast type (executor.cc:555)

    def __init__(self, inputs):
        self.inputs = list(inputs)
        me = weakref.ref(self)
        for v in self.inputs:              # who reads a Var (weakly): Var.assign moves them to the old value
            lst = v._consumers
            if lst is None:
                v._consumers = [me]
            else:
                lst.append(me)
                if len(lst) > 64 and len(lst) & (len(lst) - 1) == 0:     # a long-lived var (a weight): drop the dead readers now and then
                    lst[:] = [r for r in lst if r() is not None]
        self.id = _new_id()
        self._out_ref = None
        self.amp = dt.amp_reg & 63          # the register at creation; its gradient is built under it (op.cc:38, grad.cc:48-55)

    # The result is held weakly: a Var owns its producing op (and through it the inputs), never the other way round, so
    # a Var nobody refers to any more is released at once together with its buffer, without waiting for the cycle collector
    # (an op is only ever reached through its result or through a consumer of its result).
    @property
    def out(self):
        ref = self._out_ref
        return ref() if ref is not None else None

    @out.setter
    def out(self, v):
        self._out_ref = weakref.ref(v) if v is not None else None

    def __repr__(self):
        return "%s#%d" % (self.kind, self.id)


class UnaryOp(Op):
    kind = "unary"
    fusable = True

    def __init__(self, x, op):
        super().__init__([x])
        self.op = op


class BinaryOp(Op):
    kind = "binary"
    fusable = True

    def __init__(self, x, y, op):
        super().__init__([x, y])
        self.op = op


class TernaryOp(Op):
    kind = "ternary"
    fusable = True

    def __init__(self, c, x, y):
        super().__init__([c, x, y])


class BroadcastOp(Op):
    kind = "broadcast"
    fusable = True

    def __init__(self, x, bcast_mask, keepdims_mask):
        super().__init__([x])
        self.bcast_mask = bcast_mask
        self.keepdims_mask = keepdims_mask


class ReduceOp(Op):
    kind = "reduce"

    def __init__(self, x, op, reduce_mask, keepdims_mask):
        super().__init__([x])
        self.op = op
        self.reduce_mask = reduce_mask
        self.keepdims_mask = keepdims_mask


class ReindexOp(Op):
    kind = "reindex"

    def __init__(self, x, indexes, overflow_value, overflow_conditions, extras):
        super().__init__([x] + list(extras))
        self.indexes = list(indexes)
        self.overflow_value = float(overflow_value)
        self.overflow_conditions = list(overflow_conditions)


class ReindexReduceOp(Op):
    kind = "reindex_reduce"

    def __init__(self, y, op, indexes, overflow_conditions, extras):
        super().__init__([y] + list(extras))
        self.op = op
        self.indexes = list(indexes)
        self.overflow_conditions = list(overflow_conditions)


# --------------------------------------------------------------------------
# Var
# --------------------------------------------------------------------------
class Var:
    """Dense row-major tensor, computed on demand (var.h:18-49).  Rank 0
    becomes shape [1] (var.cc:105)."""

    __array_priority__ = 100

    def __init__(self, shape, dtype, op=None):
        shape = [int(s) for s in shape]
        if len(shape) == 0:
            shape = [1]
        if len(shape) > _lib.MAX_DIM:
            raise ValueError("at most %d dims are supported" % _lib.MAX_DIM)
        n = 1
        for e in shape:
            if e < 0:
                raise ValueError("Shape should greater than 0: %r" % (shape,))
            n *= e
        self.shape = shape
        self._num = n
        self.dtype = dtype
        self._op = op
        if op is not None:
            op.out = self
        # history for grad(): the producing op and its inputs outlive materialisation (the executor
        # clears _op / op.inputs of computed vars), like the reference's backward liveness
        # (python/jittor/src/node.h).  Cleared by stop_grad() and under no_grad().
        self._history = (op, tuple(op.inputs)) if op is not None and _grad_enabled[0] else None
        self._buf = None         # Buffer once materialised
        self._host = None        # host copy for array leaves (and fused scalars)
        self.is_scalar = False   # NodeFlags::_is_scalar
        self.id = _new_id()
        self._name = None
        self._consumers = None   # ops that take this Var as an input (weakly)
        # compile options: the flag's value at creation (var.cc:75)
        co = dict.__getitem__(_flags, "compile_options")
        self._compile_options = dict(co) if co else None

    # ---- properties ----
    @property
    def num(self):
        return self._num

    @property
    def ndim(self):
        return len(self.shape)

    @property
    def nbytes(self):
        return self.num * _lib.DTYPE_SIZE[self.dtype]

    def numel(self):
        return self.num

    @property
    def compile_options(self):
        """Options of the code generated for the op that makes this var: a dict name -> int
        (var_holder.h:265-273; the fused group they end up in reads them through
        FusedOp::get_loop_option, fused_op.cc:24-27,51-53).  nn.conv2d marks a grouped convolution with {"G": groups}
        (nn.py:1278).  They are kept and handed on as the reference does; the kernels of this library take every
        shape and layout decision from the operands themselves, so no option changes what runs."""
        return dict(self._compile_options or {})

    @compile_options.setter
    def compile_options(self, options):
        opts = {}
        for k, v in dict(options).items():
            if not isinstance(k, str) or isinstance(v, bool) or not isinstance(v, numbers.Integral):
                raise TypeError("compile_options maps names to integers, got %r: %r" % (k, v))
            opts[k] = int(v)
        self._compile_options = opts or None

    def name(self, n=None):
        if n is None:
            return self._name
        self._name = n
        return self

    def is_float(self):
        return dt.is_float(self.dtype)

    @property
    def materialised(self):
        return self._buf is not None or self._op is None

    def __repr__(self):
        return "jt.Var(shape=%s, dtype=%s%s)" % (self.shape, self.dtype, "" if self._op is None else ", lazy")

    def __len__(self):
        return self.shape[0]

    # ---- execution ----
    def sync(self, device_sync=False):
        from .executor import run_sync
        run_sync([self], device_sync)
        return self

    def _device_ptr(self):
        """Pointer of the materialised data (uploads an array leaf on first use)."""
        if self._buf is None:
            if self._op is not None:
                raise MjtError(-1, "internal: var %d is not computed" % self.id)
            self._buf = Buffer(max(self.nbytes, 1))
            if self.nbytes:
                _lib.ensure_init()
                _lib.h2d(self._buf.ptr, self._host)
        return self._buf.ptr

    def numpy(self):
        """Synchronises and returns a host copy (var_holder.h:278-290).
        bfloat16 data is returned as float32 (exactly representable)."""
        if self._op is None and self._host is not None:
            raw = self._host.copy()
        else:
            self.sync()
            raw = _lib.d2h(self._buf.ptr, self.shape, _lib.NP_STORAGE[self.dtype])
        if self.dtype == "bfloat16":
            return dt.bf16_bits_to_f32(raw)
        return raw

    @property
    def data(self):
        return self.numpy()

    def raw(self):
        """Host copy in storage format (bfloat16 stays uint16 bit patterns)."""
        if self._op is None and self._host is not None:
            return self._host.copy()
        self.sync()
        return _lib.d2h(self._buf.ptr, self.shape, _lib.NP_STORAGE[self.dtype])

    def item(self):
        if self.num != 1:
            raise ValueError("item() needs a one-element Var")
        return self.numpy().reshape(-1)[0].item()

    def fetch_sync(self):
        return self.numpy()

    def raw_ptr(self):
        self.sync()
        return self._device_ptr()

    # ---- op sugar ----
    def reindex(self, *args, **kw):
        return reindex(self, *args, **kw)

    def reindex_var(self, indexes, overflow_value=0, overflow_conditions=()):
        return reindex_var(self, indexes, overflow_value, overflow_conditions)

    def reindex_reduce(self, op, shape, indexes, overflow_conditions=(), extras=()):
        return reindex_reduce(self, op, shape, indexes, overflow_conditions, extras)

    def broadcast(self, shape, dims=()):
        return broadcast(self, shape, dims)

    def broadcast_var(self, y, dims=()):
        return broadcast_var(self, y, dims)

    def reduce(self, op, dims=(), keepdims=False):
        return reduce(self, op, dims, keepdims)

    def sum(self, dims=(), keepdims=False, dim=None):
        return reduce(self, "add", dims if dim is None else dim, keepdims)

    def max(self, dims=(), keepdims=False, dim=None):
        return reduce(self, "maximum", dims if dim is None else dim, keepdims)

    def min(self, dims=(), keepdims=False, dim=None):
        return reduce(self, "minimum", dims if dim is None else dim, keepdims)

    def mean(self, dims=(), keepdims=False, dim=None):
        return reduce(self, "mean", dims if dim is None else dim, keepdims)

    def prod(self, dims=(), keepdims=False, dim=None):
        return reduce(self, "multiply", dims if dim is None else dim, keepdims)

    product = prod

    def all(self, dims=(), keepdims=False):
        return reduce(self, "logical_and", dims, keepdims)

    def any(self, dims=(), keepdims=False):
        return reduce(self, "logical_or", dims, keepdims)

    def unary(self, op):
        return unary(self, op)

    def cast(self, dtype):
        return unary(self, dt.normalize_dtype(dtype))

    astype = cast

    def binary(self, y, op):
        return binary(self, y, op)

    def ternary(self, x, y):
        return ternary(self, x, y)

    def _split_off_value(self):
        """Moves this Var's present value to a new Var and hands every op that reads this Var over to it: the
        object is then free to be rebound without changing what was built from its old value (in the reference
        the Python object is a holder and ops refer to the node behind it, python/jittor/src/var_holder.h:37-60)."""
        old = Var.__new__(Var)
        old.__dict__.update(self.__dict__)           # the old value keeps its id: ids grow along the data flow (grad() orders by them)
        self.id = _new_id()
        old._consumers = self._consumers
        self._consumers = None
        self._op = self._history = self._buf = self._host = None     # nothing left here until assign() fills it
        if old._op is not None:
            old._op.out = old
        for ref in list(old._consumers or ()):
            op = ref()
            if op is None:
                continue
            op.inputs = [old if v is self else v for v in op.inputs]
            out = op.out
            if out is not None and out._history is not None:
                out._history = (out._history[0], tuple(old if v is self else v for v in out._history[1]))
        return old

    def assign(self, other):
        """This Var becomes `other` (shape, dtype and value), as VarHolder::assign rebinds a holder
        (python/jittor/src/var_holder.cc).  Ops built from the old value keep reading the old value."""
        # a Python number becomes an array of its own: the Vars _as_var keeps per number are shared by every
        # expression that names that number and must never be rebound
        other = other if isinstance(other, Var) else array(other)
        if other is self:
            return self
        if self._op is not None or self._buf is not None or self._host is not None:
            self._split_off_value()
        name = self._name
        src = other._split_off_value()                 # `other` stays valid: it now reads this Var (and has a new id)
        self.__dict__.update(src.__dict__)             # with the id of the value taken over
        self._name = name
        if self._op is not None:
            self._op.out = self
        alias = ReindexOp(self, ["i%d" % i for i in range(len(self.shape))], 0, [], [])
        other._op, other._buf, other._host = alias, None, None
        alias.out = other
        other._history = (alias, (self,)) if _grad_enabled[0] else None
        return self

    def stop_grad(self):
        """The var becomes a leaf for grad() (var_holder.h stop_grad)."""
        self._history = None
        return self

    def detach(self):
        return unary_clone(self).stop_grad()

    def stop_fuse(self):
        self._stop_fuse = True
        return self

    # arithmetic operators (the @pybind names of ops/binary_op.cc:29-419)
    def __add__(self, o): return binary(self, o, "add")
    def __radd__(self, o): return binary(o, self, "add")
    def __sub__(self, o): return binary(self, o, "subtract")
    def __rsub__(self, o): return binary(o, self, "subtract")
    def __mul__(self, o): return binary(self, o, "multiply")
    def __rmul__(self, o): return binary(o, self, "multiply")
    def __truediv__(self, o): return binary(self, o, "divide")
    def __rtruediv__(self, o): return binary(o, self, "divide")
    def __floordiv__(self, o): return binary(self, o, "floor_divide")
    def __rfloordiv__(self, o): return binary(o, self, "floor_divide")
    def __mod__(self, o): return binary(self, o, "mod")
    def __rmod__(self, o): return binary(o, self, "mod")
    def __pow__(self, o): return binary(self, o, "pow")
    def __rpow__(self, o): return binary(o, self, "pow")
    def __lt__(self, o): return binary(self, o, "less")
    def __le__(self, o): return binary(self, o, "less_equal")
    def __gt__(self, o): return binary(self, o, "greater")
    def __ge__(self, o): return binary(self, o, "greater_equal")
    def __eq__(self, o): return binary(self, o, "equal")
    def __ne__(self, o): return binary(self, o, "not_equal")
    def __lshift__(self, o): return binary(self, o, "left_shift")
    def __rshift__(self, o): return binary(self, o, "right_shift")
    def __and__(self, o): return binary(self, o, "bitwise_and")
    def __rand__(self, o): return binary(o, self, "bitwise_and")
    def __or__(self, o): return binary(self, o, "bitwise_or")
    def __ror__(self, o): return binary(o, self, "bitwise_or")
    def __xor__(self, o): return binary(self, o, "bitwise_xor")
    def __rxor__(self, o): return binary(o, self, "bitwise_xor")
    def __neg__(self): return unary(self, "negative")
    def __invert__(self): return unary(self, "bitwise_not")
    def __abs__(self): return unary(self, "abs")
    __hash__ = object.__hash__

    def maximum(self, o): return binary(self, o, "maximum")
    def minimum(self, o): return binary(self, o, "minimum")
    def logical_and(self, o): return binary(self, o, "logical_and")
    def logical_or(self, o): return binary(self, o, "logical_or")
    def logical_xor(self, o): return binary(self, o, "logical_xor")
    def logical_not(self): return unary(self, "logical_not")


def _install_unary_methods():
    for name in _lib.UNARY_OPS:
        if name in ("cast", "logical_not", "negative", "bitwise_not"):
            continue
        setattr(Var, name, (lambda n: lambda self: unary(self, n))(name))
    for name in _lib.DTYPES[1:]:
        setattr(Var, name, (lambda n: lambda self: unary(self, n))(name))


_install_unary_methods()


# --------------------------------------------------------------------------
# array: host data -> Var (ops/array_op.cc:54-80, pyjt/py_array_op.cc)
# --------------------------------------------------------------------------
def array(data, dtype=None):
    """Var from a number, list, numpy array or Var.  Python float -> float32,
    int -> int32, bool -> bool; float64 / int64 arrays are narrowed to 32 bit
    unless dtype is given (auto_convert_64_to_32).  One-element arrays are
    fused scalars (ops/array_op.cc:56-60)."""
    if isinstance(data, Var):
        if dtype is None:
            return unary_clone(data)
        return unary(data, dt.normalize_dtype(dtype))
    name = dt.normalize_dtype(dtype)
    if name == "bfloat16":
        host = dt.f32_to_bf16_bits(np.asarray(data, dtype=np.float32))
    elif name is not None:
        host = np.asarray(data, dtype=_lib.NP_STORAGE[name])
    else:
        host = np.asarray(data)
        if host.dtype == np.float64:
            host = host.astype(np.float32)
        elif host.dtype == np.int64:
            host = host.astype(np.int32)
        elif host.dtype == np.uint64:
            host = host.astype(np.uint32)
        if host.dtype.kind not in "biuf":
            raise ValueError("unsupported array data of dtype %s" % host.dtype)
        name = dt.np_to_dtype(host)
    host = np.ascontiguousarray(host)
    v = Var(host.shape, name)
    v._host = host.reshape(v.shape)
    if v.num == 1:
        v.is_scalar = True
    if dt.amp_reg & dt.AMP_ARRAY_PREFER and v.num != 1 and dt.is_float(name):
        # array-like ops follow the preference too (python/jittor/__init__.py:402-411)
        if dt.amp_reg & dt.AMP_PREFER32:
            return v if name == "float32" else unary(v, "float32")
        if dt.amp_reg & dt.AMP_PREFER16:
            return v if name == "float16" else unary(v, "float16")
    return v


def from_storage(raw, dtype):
    """Var from data already in storage format (bfloat16: uint16 bit patterns)."""
    name = dt.normalize_dtype(dtype)
    host = np.ascontiguousarray(raw, dtype=_lib.NP_STORAGE[name])
    v = Var(host.shape, name)
    v._host = host.reshape(v.shape)
    if v.num == 1:
        v.is_scalar = True
    return v


def unary_clone(x):
    # jt.array(var) clones; data-wise an identity broadcast-free copy
    return unary(x, "cast", force_dtype=x.dtype, allow_forward=False)


_scalar_vars = {}        # (type, value, sign) -> the host Var of a Python number: `x * 2.0` builds no new array each time


def _as_var(v):
    if isinstance(v, Var):
        return v
    tv = type(v)
    if tv is float or tv is int or tv is bool:
        key = (tv, v, math.copysign(1.0, v) if tv is float else 0)
        got = _scalar_vars.get(key)
        if got is None:
            if len(_scalar_vars) >= 4096:
                _scalar_vars.clear()
            got = _scalar_vars[key] = array(v)
        return got
    if isinstance(v, (numbers.Number, np.generic, list, tuple, np.ndarray, bool)):
        return array(v)
    raise TypeError("cannot convert %r to a Var" % type(v))


# --------------------------------------------------------------------------
# constructors
# --------------------------------------------------------------------------
def unary(x, op, force_dtype=None, allow_forward=True):
    """ops/unary_op.cc:860-889.  `op` is a unary op name or a dtype name."""
    x = _as_var(x)
    if op in _lib.DTYPES and op != "void":
        if op == x.dtype and allow_forward:
            return x                      # forward(x), unary_op.cc:867-870
        dtype, op = op, "cast"
    elif op == "cast" and force_dtype is not None:
        dtype = force_dtype
    else:
        if op not in _lib.UNARY_OPS:
            raise ValueError("unknown unary op %r" % (op,))
        dtype = dt.unary_dtype_infer(op, x.dtype)
    y = Var(x.shape, dtype, UnaryOp(x, op))
    y.is_scalar = x.is_scalar
    return y


def _need_broadcast(xshape, shape):
    """ops/broadcast_to_op.cc:98-103."""
    if len(xshape) < len(shape):
        return True
    for i in range(1, len(shape) + 1):
        if xshape[-i] != shape[-i] and shape[-i] != 1:
            return True
    return False


def _broadcast_shape(xshape, yshape, bmask, kmask):
    """infer_shape of ops/broadcast_to_op.cc:119-168.  Returns
    (zshape, bcast_mask, keepdims_mask) with the implicit broadcasts added."""
    xdim, ydim = len(xshape), len(yshape)
    cnt = bin(bmask & ~kmask).count("1")
    zdim = max(xdim, ydim - cnt) + cnt
    zz = [0] * zdim
    xi, yi = xdim - 1, ydim - 1
    for i in range(zdim - 1, -1, -1):
        bx, by = xi >= 0, yi >= 0
        xs = xshape[xi] if bx else 1
        ys = yshape[yi] if by else 1
        if bmask >> i & 1:
            yi -= 1
            if kmask >> i & 1:
                xi -= 1
            zz[i] = ys
            continue
        m = int(xs == 1 and (ys != 1 or not bx)) << i
        bmask |= m
        if bx:
            kmask |= m
        if (xs == 1 or ys == 1) and xs != ys:
            zs = xs * ys
        else:
            if xs != ys:
                raise ValueError("Shape not match %r %r" % (xshape, yshape))
            zs = xs
        zz[i] = zs
        xi -= 1
        yi -= 1
    return zz, bmask, kmask


def broadcast(x, shape, dims=()):
    """broadcast(x, shape, dims) / broadcast(x, y, dims): `dims` name the new
    axes of the output, the other axes align right to left
    (ops/broadcast_to_op.cc:23-96)."""
    x = _as_var(x)
    if isinstance(shape, Var):
        shape = shape.shape
    shape = [int(s) for s in shape]
    if isinstance(dims, numbers.Integral):
        dims = (dims,)
    dims = list(dims)
    if not dims and not _need_broadcast(x.shape, shape):
        return x                           # forward(x)
    if len(shape) == 0:
        raise ValueError("Number of shape should greater than 0.")
    for s in shape:
        if s < 0:
            raise ValueError("Shape should greater than 0.")
    ydim = max(x.ndim, len(shape) - len(dims)) + len(dims)
    bmask = 0
    for d in dims:
        if d < 0:
            d += ydim
        if not (0 <= d < ydim):
            raise ValueError("Wrong dims number: %r" % (dims,))
        bmask |= 1 << d
    zshape, bmask, kmask = _broadcast_shape(x.shape, shape, bmask, 0)
    z = Var(zshape, x.dtype, BroadcastOp(x, bmask, kmask))
    z.is_scalar = x.is_scalar
    return z


def broadcast_var(x, y, dims=()):
    return broadcast(x, _as_var(y).shape, dims)


def _broadcast_mask(x, shape, bmask, kmask):
    """make_broadcast_to(x, shape, dims_mask, keepdims_mask), used by grads."""
    if not bin(bmask).count("1"):
        return x
    zshape, bmask, kmask = _broadcast_shape(x.shape, list(shape), bmask, kmask)
    z = Var(zshape, x.dtype, BroadcastOp(x, bmask, kmask))
    z.is_scalar = x.is_scalar
    return z


def binary(x, y, op):
    """ops/binary_op.cc:421-474: broadcasts are inserted when ranks differ or
    an extent is 1 on one side only; other mismatches are errors."""
    x, y = _as_var(x), _as_var(y)
    if op not in _lib.BINARY_OPS:
        raise ValueError("unknown binary op %r" % (op,))
    need = x.ndim != y.ndim
    for i in range(1, min(x.ndim, y.ndim) + 1):
        xs, ys = x.shape[-i], y.shape[-i]
        if (xs == 1 or ys == 1) and xs != ys:
            need = True
            continue
        if xs != ys:
            raise ValueError("Shape not match, x:%r y:%r" % (x.shape, y.shape))
    if need:
        xp = broadcast(x, y.shape)
        yp = broadcast(y, x.shape)
        return binary(xp, yp, op)
    dtype = dt.binary_dtype_infer(op, x.dtype, y.dtype, x.is_scalar, y.is_scalar)
    return Var(x.shape, dtype, BinaryOp(x, y, op))


def ternary(cond, x, y):
    """ops/ternary_op.cc:21-47."""
    cond, x, y = _as_var(cond), _as_var(x), _as_var(y)
    bx = cond.ndim > x.ndim or cond.num > x.num
    by = cond.ndim > y.ndim or cond.num > y.num
    bx2 = cond.ndim < x.ndim or cond.num < x.num
    by2 = cond.ndim < y.ndim or cond.num < y.num
    if bx or by or bx2 or by2:
        if bx2:
            cond = broadcast(cond, x.shape)
        if by2:
            cond = broadcast(cond, y.shape)
        bx = cond.ndim > x.ndim or cond.num > x.num
        by = cond.ndim > y.ndim or cond.num > y.num
        if bx:
            x = broadcast(x, cond.shape)
        if by:
            y = broadcast(y, cond.shape)
        return ternary(cond, x, y)
    if not (x.ndim == y.ndim == cond.ndim):
        raise ValueError("Number of dims should be the same.")
    for a, b, c in zip(x.shape, y.shape, cond.shape):
        if not (a == b == c):
            raise ValueError("Shape not match %r %r %r" % (x.shape, y.shape, cond.shape))
    dtype = x.dtype if x.dtype == y.dtype else dt.dtype_infer(x.dtype, y.dtype, x.is_scalar, y.is_scalar)
    return Var(x.shape, dtype, TernaryOp(cond, x, y))


def reduce(x, op, dims=(), keepdims=False):
    """ops/reduce_op.cc:257-337."""
    x = _as_var(x)
    if op not in _lib.BINARY_OPS:
        raise ValueError("unknown reduce op %r" % (op,))
    if op not in dt.REDUCE_OPS:
        raise ValueError("reduce op %r is not associative; not supported on the device" % (op,))
    if isinstance(dims, numbers.Integral):
        dims = (dims,)
    dims = list(dims)
    xdim = x.ndim
    if not dims:
        rmask = (1 << xdim) - 1
    else:
        rmask = 0
        for d in dims:
            if d < 0:
                d += xdim
            if not (0 <= d < xdim):
                raise ValueError("Wrong dims number: %r" % (dims,))
            rmask |= 1 << d
    kmask = (1 << 30) - 1 if keepdims else 0
    return _reduce_mask(x, op, rmask, kmask)


def _reduce_mask(x, op, rmask, kmask):
    if not dt.amp_reg & dt.AMP_REDUCE16_DIRECT and x.dtype in ("float16", "bfloat16") and op in ("mean", "add"):
        # improve 16-bit float precision: cast -> reduce -> cast (reduce_op.cc:259-266, 295-302)
        return unary(_reduce_mask(unary(x, "float32"), op, rmask, kmask), x.dtype)
    ys = []
    for i in range(x.ndim):
        if rmask >> i & 1:
            if kmask >> i & 1:
                ys.append(1)
        else:
            ys.append(x.shape[i])
    if not ys:
        ys = [1]
        kmask |= 1
    dtype = dt.reduce_dtype_infer(op, x.dtype)
    y = Var(ys, dtype, ReduceOp(x, op, rmask, kmask))
    if len(ys) == 1 and y.num == 1:
        y.is_scalar = True
    return y


def reindex(x, shape, indexes=None, overflow_value=0, overflow_conditions=(), extras=()):
    """reindex(x, shape, indexes, overflow_value, overflow_conditions, extras)
    or reindex(x, [index Vars], overflow_value, overflow_conditions)
    (ops/reindex_op.cc:20-70)."""
    x = _as_var(x)
    if len(shape) and isinstance(shape[0], Var):
        # the Var-index form: second positional argument is overflow_value
        ov = indexes if indexes is not None else 0
        ofc = overflow_value if not isinstance(overflow_value, numbers.Number) else overflow_conditions
        return reindex_var(x, shape, ov, ofc)
    if indexes is None:
        raise ValueError("reindex needs index expressions")
    indexes = [str(s) for s in indexes]
    extras = [_as_var(e) for e in extras]
    if len(indexes) != x.ndim:
        raise ValueError("Number of x's shape and indexes should be the same.")
    shape = [int(s) for s in shape]
    if not shape:
        if not extras:
            raise ValueError("Number of shape should greater than 0.")
        shape = list(extras[0].shape)
    if len(shape) > _lib.MAX_DIM:
        raise ValueError("Too many dims")
    return Var(shape, x.dtype, ReindexOp(x, indexes, overflow_value, [str(s) for s in overflow_conditions], extras))


def reindex_var(x, indexes, overflow_value=0, overflow_conditions=()):
    """reindex(x, [idx Vars]) = reindex(x, idx[0].shape, ['@e0(i0,..)', ...], extras=idx)
    (ops/reindex_op.cc:35-70)."""
    x = _as_var(x)
    indexes = [_as_var(v) for v in indexes]
    if not indexes:
        raise ValueError("reindex_var needs index Vars")
    n = indexes[0].ndim
    if n > _lib.MAX_DIM:
        raise ValueError("Too many dims")
    coords = ",".join("i%d" % d for d in range(n))
    strs = ["@e%d(%s)" % (k, coords) for k in range(len(indexes))]
    return reindex(x, indexes[0].shape, strs, overflow_value, overflow_conditions, indexes)


def reindex_reduce(y, op, shape, indexes, overflow_conditions=(), extras=()):
    """ops/reindex_reduce_op.cc:26-73."""
    y = _as_var(y)
    if (op not in _lib.BINARY_OPS and op != "void") or op == "mean":
        raise ValueError("reindex_reduce: op %r is not a binary op" % (op,))
    indexes = [str(s) for s in indexes]
    shape = [int(s) for s in shape]
    if len(shape) != len(indexes):
        raise ValueError("Number of shape and indexes should be the same.")
    if not shape:
        raise ValueError("Number of shape should greater than 0.")
    for s in shape:
        if s < 0:
            raise ValueError("Shape should greater than 0.")
    extras = [_as_var(e) for e in extras]
    return Var(shape, y.dtype, ReindexReduceOp(y, op, indexes, [str(s) for s in overflow_conditions], extras))


def make_number(value, like):
    """ops/op_utils.cc:19-36: a [1] array of like's dtype broadcast to like."""
    v = array(value, like.dtype)
    return broadcast(v, like.shape)
