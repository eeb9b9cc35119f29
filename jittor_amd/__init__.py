"""jittor_amd: the meta-operator execution path of Jittor on MI355X (gfx950).

Keeps Jittor's Python signatures for this path -- jt.array, jt.reindex,
jt.reindex_reduce, Var.sum / max / min, jt.broadcast, unary / binary / ternary
ops -- on a small lazy Var graph that executes through libmjt.so
(include/mjt.h) into hand-written HIP kernels.  Signatures follow
python/jittor/__init__.pyi:203-206,280-285,368,823-891,1201-1263,2168,
4122-4190,4258 of the reference.
"""
import numbers as _numbers

import numpy as np

from . import _lib
from ._lib import MjtError, init, shutdown, sync as _device_sync, device_info
from .core import (Var, array, unary, binary, ternary, broadcast, broadcast_var,
                   reduce, reindex, reindex_var, reindex_reduce, make_number, from_storage)
from .executor import run_sync, stats as executor_stats
from .flags import flags, flag_scope
from . import dtypes
from . import nn
from .grad import grad
from . import misc
from . import profiler
from .profiler import profile_scope
from .misc import gather, scatter, pad, pool, permute, transpose, reshape, flip, concat, where
from .nn import matmul
from .core import no_grad

__all__ = ["Var", "array", "unary", "binary", "ternary", "broadcast", "broadcast_var",
           "reduce", "reindex", "reindex_var", "reindex_reduce", "nn", "sync", "sync_all",
           "fetch_sync", "grad", "no_grad", "gather", "scatter", "pad", "pool", "permute", "transpose", "reshape",
           "flip", "concat", "where", "matmul", "profile_scope", "MjtError"]


def sync(vars, device_sync=False):
    """jt.sync(vars): computes the given Vars (var_holder.cc:269-274)."""
    run_sync(list(vars), device_sync)


def sync_all(device_sync=True):
    if device_sync and _lib.device() is not None:
        _device_sync()


def fetch_sync(vars):
    vars = list(vars)
    run_sync(vars)
    return [v.numpy() for v in vars]


def clean():
    core.pool.release_all()


# ---- creation helpers --------------------------------------------------------
def zeros(shape, dtype="float32"):
    if isinstance(shape, _numbers.Integral):
        shape = [shape]
    return array(np.zeros(shape, dtype=np.float32), dtypes.normalize_dtype(dtype))


def ones(shape, dtype="float32"):
    if isinstance(shape, _numbers.Integral):
        shape = [shape]
    return array(np.ones(shape, dtype=np.float32), dtypes.normalize_dtype(dtype))


_rng = [np.random.default_rng(0)]


def set_seed(seed):
    _rng[0] = np.random.default_rng(seed)


def random(shape, dtype="float32", type="uniform"):
    """Host-generated random Var (the reference's generator,
    python/jittor/src/init.cc:78-84, is not reproduced: tests seed numpy)."""
    if isinstance(shape, _numbers.Integral):
        shape = [shape]
    if type == "normal":
        a = _rng[0].standard_normal(shape)
    else:
        a = _rng[0].random(shape)
    return array(a.astype(np.float32), dtypes.normalize_dtype(dtype))


def randn(*shape):
    if len(shape) == 1 and isinstance(shape[0], (list, tuple)):
        shape = shape[0]
    return random(list(shape), "float32", "normal")


def index(shape, dim, dtype="int32"):
    """jt.index(shape, dim): Var of `shape` holding the coordinate along `dim`."""
    shape = list(shape)
    a = array(np.arange(shape[dim]), dtype)
    return broadcast(a, shape, [d for d in range(len(shape)) if d != dim])


# ---- named ops ----------------------------------------------------------------
def _make_binary(name):
    def f(x, y):
        return binary(x, y, name)
    f.__name__ = name
    return f


def _make_unary(name):
    def f(x):
        return unary(x, name)
    f.__name__ = name
    return f


def _make_reduce(name):
    def f(x, dims=(), keepdims=False, dim=None):
        return reduce(x, name, dims if dim is None else dim, keepdims)
    f.__name__ = "reduce_" + name
    return f


for _n in _lib.BINARY_OPS:
    if _n != "mean":
        globals()[_n] = _make_binary(_n)
for _n in _lib.UNARY_OPS:
    if _n != "cast":
        globals()[_n] = _make_unary(_n)
for _n in _lib.DTYPES[1:]:
    globals()[_n] = (lambda n: lambda x: array(x, n) if not isinstance(x, Var) else unary(x, n))(_n)
for _n in dtypes.REDUCE_OPS:
    globals()["reduce_" + _n] = _make_reduce(_n)
float = float32  # noqa: F821
int = int32  # noqa: F821


def cast(x, dtype):
    return unary(x, dtypes.normalize_dtype(dtype))


def sum(x, dims=(), keepdims=False, dim=None):
    return reduce(x, "add", dims if dim is None else dim, keepdims)


def max(x, dims=(), keepdims=False, dim=None):
    return reduce(x, "maximum", dims if dim is None else dim, keepdims)


def min(x, dims=(), keepdims=False, dim=None):
    return reduce(x, "minimum", dims if dim is None else dim, keepdims)


def mean(x, dims=(), keepdims=False, dim=None):
    return reduce(x, "mean", dims if dim is None else dim, keepdims)


def prod(x, dims=(), keepdims=False, dim=None):
    return reduce(x, "multiply", dims if dim is None else dim, keepdims)


def ternary_out_hint(cond, x, y):
    return ternary(cond, x, y)


def histc(input, bins, min=0.0, max=0.0):
    """Histogram of an N-d Var with `bins` equal bins over [min, max] (python/jittor/misc.py:2212-2235): a
    scatter-add of ones by bin index floor((x - min) / ((max - min) / bins)).  Values outside [min, max] are
    not counted and values equal to max go to the last bin, as there; the reference selects the values in
    range with a boolean mask first, here they keep their place and get an index outside [0, bins), which
    reindex_reduce drops."""
    if bins <= 0:
        raise RuntimeError("bins must be > 0, but got %s" % bins)
    flat = input.reshape([input.num]) if input.ndim != 1 else input
    if min == 0 and max == 0:
        lo, hi = flat.min().item(), flat.max().item()
    else:
        lo, hi = min, max
    assert lo < hi
    bin_length = (hi - lo) / bins
    idx = unary((flat - lo) / bin_length, "floor_int")
    inside = binary(flat >= lo, flat < hi, "logical_and")
    idx = ternary(inside, idx, ternary(flat == hi, broadcast(array(bins - 1, "int32"), idx.shape),
                                       broadcast(array(-1, "int32"), idx.shape)))
    one = ones(flat.shape, "float32")
    return reindex_reduce(one, "add", [bins], ["@e0(i0)"], extras=[idx])
