"""CPU oracle for the meta-operator path.  TEST INFRASTRUCTURE ONLY.

This module restates, in numpy, the semantics of the reference's JIT kernel
templates.  Only tests, the smoke check and the cpu_baseline leg of the bench
may import it; the product path (jittor_amd) never does.

Every function cites the reference file:line it follows (paths relative to
python/jittor/src/ of the reference tree).

Pin status (which independent check fixes each function; the checks live in
tests/test_oracle_*.py):
  reindex          closed form sliding_window_view / np.pad / np.matmul,
                   brute-force coordinate loops, literal vectors of the
                   reference's tests (test_fused_op.py:248-251,
                   test_reindex_op.py:181-190)
  reindex_reduce   np.add.at / np.maximum.at / brute-force pooling loops
  reduce           np.<ufunc>.reduce on integer data (exact), float64 sums
  broadcast_to     np.broadcast_to, literal vectors (test_broadcast_to_op.py:125-135)
  binary/unary/ternary   numpy/scipy closed forms, literal vectors
  erfinv           scipy.special.erfinv
  conv_meta        float64 im2col GEMM, one-hot kernels (shift), linearity
  dtype inference  literal table of test_bf16.py / test_binary_op.py
"""
import re
import numpy as np

# --------------------------------------------------------------------------
# dtypes.  Names follow misc/nano_string.h:17-31.  bfloat16 has no numpy
# type: bf16 arrays are carried as uint16 bit patterns inside a BF16 wrapper.
# --------------------------------------------------------------------------
DTYPES = ["bool", "int8", "int16", "int32", "int64", "uint8", "uint16",
          "uint32", "uint64", "float16", "float32", "float64", "bfloat16"]

_NP = {"bool": np.bool_, "int8": np.int8, "int16": np.int16, "int32": np.int32,
       "int64": np.int64, "uint8": np.uint8, "uint16": np.uint16,
       "uint32": np.uint32, "uint64": np.uint64, "float16": np.float16,
       "float32": np.float32, "float64": np.float64}


class BF16:
    """bfloat16 array as raw uint16 bits."""

    def __init__(self, bits):
        self.bits = np.asarray(bits, dtype=np.uint16)

    @property
    def shape(self):
        return self.bits.shape

    def to_f32(self):
        # type/fp16_compute.h:243-247: bits<<16 reinterpreted as float
        return (self.bits.astype(np.uint32) << 16).view(np.float32)


def f32_to_bf16_bits(a):
    """type/fp16_compute.h:238-241: bf16(float) keeps the upper 16 bits
    (truncation, no rounding)."""
    a = np.ascontiguousarray(a, dtype=np.float32)
    return (a.view(np.uint32) >> 16).astype(np.uint16)


def dtype_name(a):
    if isinstance(a, BF16):
        return "bfloat16"
    return {np.dtype(v): k for k, v in _NP.items()}[np.asarray(a).dtype]


def _dsize_(name):          # log2(bytes), misc/nano_string.h:151-152
    return {"bool": 0, "int8": 0, "uint8": 0, "int16": 1, "uint16": 1,
            "float16": 1, "bfloat16": 1, "int32": 2, "uint32": 2,
            "float32": 2, "int64": 3, "uint64": 3, "float64": 3}[name]


def _is_float(name):
    return name in ("float16", "float32", "float64", "bfloat16")


BOOL_OPS = {"logical_not", "less", "less_equal", "greater", "greater_equal",
            "equal", "not_equal", "logical_and", "logical_or", "logical_xor"}
FLOAT_OPS = {"log", "exp", "sqrt", "mean", "divide", "sin", "asin", "sinh",
             "asinh", "tan", "atan", "tanh", "atanh", "cos", "acos", "cosh",
             "acosh", "sigmoid", "erf", "erfinv"}
INT_OPS = {"round_int", "floor_int", "ceil_int", "floor_divide"}
WHITE_OPS = {"exp", "pow"}
UNARY_OPS = ["abs", "negative", "logical_not", "bitwise_not", "log", "exp",
             "sqrt", "round", "floor", "ceil", "round_int", "floor_int",
             "ceil_int", "cast", "sin", "asin", "sinh", "asinh", "tan", "atan",
             "tanh", "atanh", "cos", "acos", "cosh", "acosh", "sigmoid", "erf",
             "erfinv"]
BINARY_OPS = ["pow", "maximum", "minimum", "add", "subtract", "multiply",
              "divide", "floor_divide", "mod", "less", "less_equal", "greater",
              "greater_equal", "equal", "not_equal", "left_shift",
              "right_shift", "logical_and", "logical_or", "logical_xor",
              "bitwise_and", "bitwise_or", "bitwise_xor", "mean"]


def float_dtype(dsize_, has_bf16=False):
    """misc/nano_string.h:205-215 with amp_reg == 0."""
    if dsize_ == 3:
        return "float64"
    if dsize_ == 2:
        return "float32"
    return "bfloat16" if has_bf16 else "float16"


def int_dtype(dsize_):
    """misc/nano_string.h:217-221."""
    return {3: "int64", 2: "int32", 1: "int16", 0: "int8"}[dsize_]


def dtype_infer(x, y, xscalar=False, yscalar=False):
    """misc/nano_string.h:223-235."""
    d = max(_dsize_(x), _dsize_(y))
    if xscalar:
        d = _dsize_(y)
    if yscalar:
        d = _dsize_(x)
    if _is_float(x) or _is_float(y):
        return float_dtype(d, "bfloat16" in (x, y))
    return int_dtype(d)


def binary_dtype_infer(op, x, y, xscalar=False, yscalar=False):
    """misc/nano_string.h:238-254 with amp_reg == 0."""
    if op in BOOL_OPS:
        return "bool"
    d = max(_dsize_(x), _dsize_(y))
    if xscalar:
        d = _dsize_(y)
    if yscalar:
        d = _dsize_(x)
    is_float = op not in INT_OPS and (_is_float(x) or _is_float(y) or op in FLOAT_OPS)
    if is_float:
        if op in WHITE_OPS:
            return "float64" if d == 3 else "float32"
        return float_dtype(d, "bfloat16" in (x, y))
    if x == "bool" and y == "bool":
        return "bool"
    return int_dtype(d)


def unary_dtype_infer(op, x):
    """misc/nano_string.h:256-266 with amp_reg == 0."""
    if op in BOOL_OPS:
        return "bool"
    d = _dsize_(x)
    if op in FLOAT_OPS:
        if op in WHITE_OPS:
            return "float64" if d == 3 else "float32"
        return float_dtype(d, x == "bfloat16")
    if op in INT_OPS:
        return int_dtype(d)
    return x


def reduce_dtype_infer(op, x):
    """misc/nano_string.h:268-277 with amp_reg == 0, plus the bool->int32
    rule of ops/reduce_op.cc:287-290."""
    if x == "bool":
        return "int32"
    if _is_float(x) or op in FLOAT_OPS:
        return "float64" if _dsize_(x) == 3 else "float32"
    return x


# --------------------------------------------------------------------------
# C arithmetic helpers
# --------------------------------------------------------------------------
def _as_compute(a):
    """Value as C would see it in an expression: bf16/fp16 convert to float
    (type/fp16_compute.h operator float), bool/int8/int16 promote to int."""
    if isinstance(a, BF16):
        return a.to_f32()
    a = np.asarray(a)
    if a.dtype == np.float16:
        return a.astype(np.float32)
    if a.dtype in (np.bool_, np.int8, np.int16, np.uint8, np.uint16):
        return a.astype(np.int32)
    return a


def c_cast(a, tz):
    """(Tz)(a) with C conversion rules: float->int truncates toward zero,
    ->bool is (a != 0), ->bfloat16 truncates the float bits."""
    a = _as_compute(a)
    if tz == "bfloat16":
        return BF16(f32_to_bf16_bits(a.astype(np.float32)))
    if tz == "bool":
        return a != 0
    with np.errstate(all="ignore"):
        if a.dtype.kind == "f" and np.dtype(_NP[tz]).kind in "iu":
            return np.trunc(a).astype(_NP[tz])
        return a.astype(_NP[tz])


def _c_div(a, b):
    """C '/': truncation toward zero for integers, IEEE for floats."""
    if a.dtype.kind == "f" or b.dtype.kind == "f":
        with np.errstate(all="ignore"):
            return a / b
    bb = np.where(b == 0, 1, b)
    q = a // bb
    fix = ((a % bb) != 0) & ((a < 0) != (bb < 0))
    return (q + fix).astype(np.result_type(a, b))


def _c_mod(a, b):
    bb = np.where(b == 0, 1, b)
    return (a - _c_div(a, bb) * bb).astype(np.result_type(a, b))


def _round_half_away(a):
    """std::round."""
    r = np.trunc(a)
    return np.copysign(r + np.where(np.abs(a - r) >= 0.5, np.sign(a), 0).astype(a.dtype), a)


# --------------------------------------------------------------------------
# element-wise ops: type/common_op_type.cc:82-163 (CPU map + shared map)
# --------------------------------------------------------------------------
def erfinv(y):
    """misc/cpu_math.cc:18-52: rational start + two Newton steps, in the
    working precision of y."""
    from scipy.special import erf
    y = np.asarray(y)
    T = y.dtype.type
    a = [T(v) for v in (0.886226899, -1.645349621, 0.914624893, -0.140543331)]
    b = [T(v) for v in (-2.118377725, 1.442710462, -0.329097515, 0.012229801)]
    c = [T(v) for v in (-1.970840454, -1.624906493, 3.429567803, 1.641345311)]
    d = [T(v) for v in (3.543889200, 1.637067800)]
    with np.errstate(all="ignore"):
        ya = np.abs(y)
        z = y * y
        num = ((a[3] * z + a[2]) * z + a[1]) * z + a[0]
        dem = (((b[3] * z + b[2]) * z + b[1]) * z + b[0]) * z + T(1)
        xc = y * num / dem
        z2 = np.sqrt(-np.log((T(1) - ya) / T(2)))
        num2 = ((c[3] * z2 + c[2]) * z2 + c[1]) * z2 + c[0]
        dem2 = (d[1] * z2 + d[0]) * z2 + T(1)
        xt = np.copysign(num2, y) / dem2
        x = np.where(ya <= T(0.7), xc, xt).astype(y.dtype)
        k = T(2) / T(np.sqrt(3.14159265358979323846))
        for _ in range(2):
            x = (x - (erf(x).astype(y.dtype) - y) / (k * np.exp(-x * x))).astype(y.dtype)
        x = np.where(ya == 1, np.copysign(T(np.inf), y), x)
        x = np.where(ya > 1, T(np.nan), x)
    return x.astype(y.dtype)


def unary(x, op, tz=None):
    """y[i] = OP(Ty, x[i], Tx): ops/unary_op.cc:1021-1027 with the CPU
    formulas of type/common_op_type.cc:82-118.  `op` may be a dtype name
    (= cast, ops/unary_op.cc:871-874)."""
    tx = dtype_name(x)
    if op in DTYPES:
        tz, op = op, "cast"
    if tz is None:
        tz = unary_dtype_infer(op, tx)
    xc = _as_compute(x)
    from scipy import special
    with np.errstate(all="ignore"):
        if op == "cast":
            return c_cast(x, tz)
        if op == "logical_not":
            r = ~(xc != 0)
        elif op == "bitwise_not":
            r = ~xc if xc.dtype != np.bool_ else ~xc.astype(np.int32)
        elif op == "negative":
            r = -xc
        elif op == "abs":
            r = np.abs(xc)
        elif op in ("log", "exp", "sqrt"):
            r = getattr(np, op)(_as_compute(c_cast(x, tz)))
        elif op in ("round", "round_int"):
            r = _round_half_away(xc if xc.dtype.kind == "f" else xc.astype(np.float64))
        elif op in ("floor", "ceil", "floor_int", "ceil_int"):
            f = np.floor if op.startswith("floor") else np.ceil
            r = f(xc if xc.dtype.kind == "f" else xc.astype(np.float64))
        elif op in ("sin", "cos", "tan", "sinh", "cosh", "tanh"):
            r = getattr(np, op)(xc if xc.dtype.kind == "f" else xc.astype(np.float64))
        elif op in ("asin", "acos", "atan", "asinh", "acosh", "atanh"):
            r = getattr(np, "arc" + op[1:])(xc if xc.dtype.kind == "f" else xc.astype(np.float64))
        elif op == "sigmoid":
            # Tz(1.0f/(1.0f+exp(min(Tz(-x), Tz(30 or 300)))))
            t = _as_compute(c_cast(-xc, tz))
            lim = t.dtype.type(30 if tz == "float32" else 300)
            r = np.float32(1.0) / (np.float32(1.0) + np.exp(np.minimum(t, lim)))
        elif op == "erf":
            r = special.erf(xc if xc.dtype.kind == "f" else xc.astype(np.float64))
        elif op == "erfinv":
            r = erfinv(xc if xc.dtype.kind == "f" else xc.astype(np.float64))
        else:
            raise ValueError("unknown unary op " + op)
    return c_cast(r, tz)


def binary(x, y, op, tz=None, xscalar=False, yscalar=False, rcount=None):
    """z[i] = OP(Tz, x[i], Tx, y[i], Ty): ops/binary_op.cc:563-570 with
    type/common_op_type.cc:120-152 (shared map) and :82-118 (CPU map)."""
    tx, ty = dtype_name(x), dtype_name(y)
    if tz is None:
        tz = binary_dtype_infer(op, tx, ty, xscalar, yscalar)
    a, b = _as_compute(x), _as_compute(y)
    with np.errstate(all="ignore"):
        if op == "add":
            r = a + b
        elif op == "subtract":
            r = a - b
        elif op == "multiply":
            r = a * b
        elif op in ("divide", "floor_divide"):
            r = _c_div(_as_compute(c_cast(x, tz)), _as_compute(c_cast(y, tz)))
        elif op == "mod":
            if tz == "float32" or tx == "float64":
                r = a - np.floor(a / b) * b
            else:
                r = _c_mod(a, b)
        elif op == "pow":
            # std::pow: float only when both operands are float, else double
            if a.dtype == np.float32 and b.dtype == np.float32:
                r = np.power(a, b)
            else:
                r = np.power(a.astype(np.float64), b.astype(np.float64))
        elif op in ("maximum", "minimum"):
            ca, cb = _as_compute(c_cast(x, tz)), _as_compute(c_cast(y, tz))
            # std::max(a,b) = (a<b)?b:a ; std::min(a,b) = (b<a)?b:a
            r = np.where(ca < cb, cb, ca) if op == "maximum" else np.where(cb < ca, cb, ca)
        elif op == "less":
            r = a < b
        elif op == "less_equal":
            r = a <= b
        elif op == "greater":
            r = a > b
        elif op == "greater_equal":
            r = a >= b
        elif op == "equal":
            r = a == b
        elif op == "not_equal":
            r = a != b
        elif op == "left_shift":
            r = a << b
        elif op == "right_shift":
            r = a >> b
        elif op == "logical_and":
            r = (a != 0) & (b != 0)
        elif op == "logical_or":
            r = (a != 0) | (b != 0)
        elif op == "logical_xor":
            r = (a != 0) != (b != 0)
        elif op == "bitwise_and":
            r = a & b
        elif op == "bitwise_or":
            r = a | b
        elif op == "bitwise_xor":
            r = a ^ b
        elif op == "mean":
            # (x + Tz(y)*Tz(rcount)), rcount = 1 for a plain binary op
            t = _as_compute(c_cast(y, tz))
            r = a + t * t.dtype.type(1 if rcount is None else rcount)
        else:
            raise ValueError("unknown binary op " + op)
    return c_cast(r, tz)


def ternary(cond, x, y, tz=None, xscalar=False, yscalar=False):
    """ops/ternary_op.cc:84-95: Tz xd=x[i]; Tz yd=y[i]; z[i]=cond[i]?xd:yd."""
    tx, ty = dtype_name(x), dtype_name(y)
    if tz is None:
        tz = tx if tx == ty else dtype_infer(tx, ty, xscalar, yscalar)
    c = _as_compute(cond) != 0
    xd, yd = c_cast(x, tz), c_cast(y, tz)
    if tz == "bfloat16":
        return BF16(np.where(c, xd.bits, yd.bits))
    return np.where(c, xd, yd).astype(_NP[tz])


# --------------------------------------------------------------------------
# broadcast: ops/broadcast_to_op.cc:119-168 (shape rule) and :177-194 (copy)
# --------------------------------------------------------------------------
def broadcast_shape(xshape, yshape, dims=()):
    """Returns (zshape, bcast_mask, keepdims_mask)."""
    xshape, yshape = list(xshape), list(yshape)
    count = len(dims)
    ydim0 = max(len(xshape), len(yshape) - count) + count
    bmask = 0
    for d in dims:
        if d < 0:
            d += ydim0
        if not (0 <= d < ydim0):
            raise ValueError("Wrong dims number: %r" % (dims,))
        bmask |= 1 << d
    kmask = 0
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


def broadcast_to(x, shape, dims=()):
    """z[i...] = x[sum (bcast_d ? 0 : i_d) * xstride_d]."""
    bf = isinstance(x, BF16)
    xa = x.bits if bf else np.asarray(x)
    zshape, bmask, _ = broadcast_shape(xa.shape, shape, dims)
    # x viewed with one axis per z axis: broadcast axes have extent 1
    xs = [1 if (bmask >> i & 1) else zshape[i] for i in range(len(zshape))]
    z = np.broadcast_to(xa.reshape(xs), zshape).copy()
    return BF16(z) if bf else z


# --------------------------------------------------------------------------
# reduce: ops/reduce_op.cc:257-337 (masks, shape) and :374-399 (loop nest)
# --------------------------------------------------------------------------
def _identity(op, tname):
    """init_OP of type/common_op_type.cc:116-117,142-151."""
    t = _NP[tname]
    if op in ("add", "mean", "void", "bitwise_or", "bitwise_xor"):
        return t(0)
    if op == "multiply":
        return t(1)
    if op == "maximum":
        return np.finfo(t).min if np.dtype(t).kind == "f" else (np.iinfo(t).min if tname != "bool" else False)
    if op == "minimum":
        return np.finfo(t).max if np.dtype(t).kind == "f" else (np.iinfo(t).max if tname != "bool" else True)
    if op == "logical_and":
        return t(1)
    if op in ("logical_or", "logical_xor"):
        return t(0)
    if op == "bitwise_and":
        return np.array(-1).astype(t)[()]
    raise ValueError("no identity for " + op)


def reduce_shape(xshape, dims, keepdims):
    xdim = len(xshape)
    if isinstance(dims, int):
        dims = (dims,)
    if len(dims) == 0:
        rmask = (1 << xdim) - 1
    else:
        rmask = 0
        for d in dims:
            if d < 0:
                d += xdim
            if not (0 <= d < xdim):
                raise ValueError("Wrong dims number: %r" % (dims,))
            rmask |= 1 << d
    ys = []
    for i in range(xdim):
        if rmask >> i & 1:
            if keepdims:
                ys.append(1)
        else:
            ys.append(xshape[i])
    if not ys:
        ys = [1]
    return ys, rmask


def reduce(x, op, dims=(), keepdims=False):
    """Kept axes outermost, reduced axes innermost, sequential accumulation
    in Ty starting from the identity (ops/reduce_op.cc:386-397)."""
    tx = dtype_name(x)
    xa = np.asarray(x)
    ty = reduce_dtype_infer(op, tx)
    yshape, rmask = reduce_shape(xa.shape, dims, keepdims)
    kept = [i for i in range(xa.ndim) if not (rmask >> i & 1)]
    red = [i for i in range(xa.ndim) if rmask >> i & 1]
    K = int(np.prod([xa.shape[i] for i in kept], dtype=np.int64)) if kept else 1
    R = int(np.prod([xa.shape[i] for i in red], dtype=np.int64)) if red else 1
    m = np.transpose(xa, kept + red).reshape(K, R)
    T = _NP[ty]
    init = np.full((K, 1), _identity(op, ty), dtype=T)
    with np.errstate(all="ignore"):
        if op in ("add", "mean"):
            v = m.astype(T)
            if op == "mean":
                v = v * T(np.float64(K) / np.float64(K * R))          # Ty(x) * Ty(rcount); rcount = y.num*1.0/x.num
            acc = np.cumsum(np.concatenate([init, v], 1), axis=1, dtype=T)[:, -1]
        elif op == "multiply":
            acc = np.cumprod(np.concatenate([init, m.astype(T)], 1), axis=1, dtype=T)[:, -1]
        elif op == "maximum":
            acc = np.maximum.reduce(np.concatenate([init, m.astype(T)], 1), axis=1)
        elif op == "minimum":
            acc = np.minimum.reduce(np.concatenate([init, m.astype(T)], 1), axis=1)
        elif op == "logical_and":
            acc = np.logical_and.reduce(m != 0, axis=1).astype(T)
        elif op == "logical_or":
            acc = np.logical_or.reduce(m != 0, axis=1).astype(T)
        elif op == "logical_xor":
            acc = np.logical_xor.reduce(m != 0, axis=1).astype(T)
        elif op == "bitwise_and":
            acc = np.bitwise_and.reduce(np.concatenate([init, m.astype(T)], 1), axis=1)
        elif op == "bitwise_or":
            acc = np.bitwise_or.reduce(np.concatenate([init, m.astype(T)], 1), axis=1)
        elif op == "bitwise_xor":
            acc = np.bitwise_xor.reduce(np.concatenate([init, m.astype(T)], 1), axis=1)
        else:
            raise ValueError("unknown reduce op " + op)
    return acc.astype(T).reshape(yshape)


# --------------------------------------------------------------------------
# index expressions: C integer expressions (ops/reindex_op.h:58-68,
# op_compiler.cc:665-699 for @eK(...), opt/expr.cc:16-52 for precedence)
# --------------------------------------------------------------------------
_TOK = re.compile(r"\s*(?:(@e\d+)|(0[xX][0-9a-fA-F]+|0[bB][01]+|\d+\.\d*(?:[eE][+-]?\d+)?f?|\d+)|([A-Za-z_]\w*)|(<<|>>|<=|>=|==|!=|&&|\|\||//|[-+*/%<>&^|!~?:(),]))")
_BINPREC = {"||": 1, "&&": 2, "|": 3, "^": 4, "&": 5, "==": 6, "!=": 6,
            "<": 7, "<=": 7, ">": 7, ">=": 7, "<<": 8, ">>": 8, "+": 9,
            "-": 9, "*": 10, "/": 10, "%": 10}
_CASTS = {"int": np.int32, "int32": np.int32, "int64": np.int64,
          "index_t": np.int64, "float": np.float32, "float32": np.float32,
          "double": np.float64, "float64": np.float64, "bool": np.bool_}


def _tokenize(s):
    out, pos = [], 0
    s = s.strip()
    while pos < len(s):
        m = _TOK.match(s, pos)
        if not m:
            raise ValueError("bad index expression %r at %d" % (s, pos))
        pos = m.end()
        if m.group(1):
            out.append(("ext", int(m.group(1)[2:])))
        elif m.group(2):
            out.append(("num", m.group(2)))
        elif m.group(3):
            out.append(("id", m.group(3)))
        else:
            if m.group(4) == "//":
                # opt/pass/loop_var_analyze_pass.cc:298-309 rejects '//'
                raise ValueError("'//' is not a C operator; use int(a/b)")
            out.append(("op", m.group(4)))
    return out


class _Parser:
    def __init__(self, s):
        self.t = _tokenize(s)
        self.p = 0

    def peek(self):
        return self.t[self.p] if self.p < len(self.t) else ("end", None)

    def take(self):
        tok = self.peek()
        self.p += 1
        return tok

    def expect(self, v):
        tok = self.take()
        if tok != ("op", v):
            raise ValueError("expected %r, got %r" % (v, tok))

    def parse(self):
        e = self.ternary()
        if self.peek()[0] != "end":
            raise ValueError("trailing tokens %r" % (self.t[self.p:],))
        return e

    def ternary(self):
        c = self.binary(1)
        if self.peek() == ("op", "?"):
            self.take()
            a = self.ternary()
            self.expect(":")
            b = self.ternary()
            return ("?", c, a, b)
        return c

    def binary(self, minprec):
        lhs = self.unary()
        while True:
            k, v = self.peek()
            if k != "op" or v not in _BINPREC or _BINPREC[v] < minprec:
                return lhs
            self.take()
            rhs = self.binary(_BINPREC[v] + 1)
            lhs = ("bin", v, lhs, rhs)

    def args(self):
        a = []
        self.expect("(")
        if self.peek() == ("op", ")"):
            self.take()
            return a
        while True:
            a.append(self.ternary())
            k, v = self.take()
            if (k, v) == ("op", ")"):
                return a
            if (k, v) != ("op", ","):
                raise ValueError("expected , or )")

    def unary(self):
        k, v = self.take()
        if k == "op" and v in "-+!~":
            return ("un", v, self.unary())
        if k == "op" and v == "(":
            e = self.ternary()
            self.expect(")")
            return e
        if k == "num":
            if v[:2].lower() == "0x":
                return ("const", np.int64(int(v, 16)))
            if v[:2].lower() == "0b":
                return ("const", np.int64(int(v[2:], 2)))
            if "." in v:
                return ("const", np.float32(v[:-1]) if v.endswith("f") else np.float64(v))
            return ("const", np.int64(int(v)))
        if k == "ext":
            return ("ext", v, self.args())
        if k == "id":
            if v in _CASTS and self.peek() == ("op", "("):
                a = self.args()
                if len(a) != 1:
                    raise ValueError("cast takes one argument")
                return ("cast", v, a[0])
            return ("var", v)
        raise ValueError("unexpected token %r" % ((k, v),))


def parse_expr(s):
    return _Parser(s).parse()


def eval_expr(e, env, extras):
    """Vectorised evaluation with C semantics.  Integers are carried as
    int64 (index_t is int32 in the reference unless a Var has >= 2^31
    elements, op.cc:158-192; no test here overflows int32)."""
    k = e[0]
    if k == "const":
        return e[1]
    if k == "var":
        if e[1] not in env:
            raise ValueError("unknown identifier %r" % e[1])
        return env[e[1]]
    if k == "cast":
        v = eval_expr(e[2], env, extras)
        v = np.asarray(v)
        t = _CASTS[e[1]]
        if v.dtype.kind == "f" and np.dtype(t).kind in "iu":
            v = np.trunc(v)
        return v.astype(t) if t is not np.bool_ else (v != 0)
    if k == "ext":
        idx, arr = e[1], None
        if idx >= len(extras):
            raise ValueError("@e%d out of range" % idx)
        arr = extras[idx]
        arr = arr.to_f32() if isinstance(arr, BF16) else np.asarray(arr)
        if len(e[2]) != arr.ndim:
            # op_compiler.cc:688 arity check
            raise ValueError("@e%d expects %d indexes" % (idx, arr.ndim))
        strides = [int(np.prod(arr.shape[j + 1:], dtype=np.int64)) for j in range(arr.ndim)]
        flat = 0
        for a, st in zip(e[2], strides):
            v = np.asarray(eval_expr(a, env, extras))
            if v.dtype.kind == "f":
                v = np.trunc(v)
            flat = flat + v.astype(np.int64) * st
        val = arr.reshape(-1)[flat]
        if val.dtype.kind in "iub":
            val = val.astype(np.int64)
        return val
    if k == "un":
        v = np.asarray(eval_expr(e[2], env, extras))
        if e[1] == "-":
            return -v
        if e[1] == "+":
            return v
        if e[1] == "!":
            return (v == 0).astype(np.int64)
        return ~v.astype(np.int64)
    if k == "?":
        c = np.asarray(eval_expr(e[1], env, extras))
        a = np.asarray(eval_expr(e[2], env, extras))
        b = np.asarray(eval_expr(e[3], env, extras))
        return np.where(c != 0, a, b)
    if k == "bin":
        op = e[1]
        a = np.asarray(eval_expr(e[2], env, extras))
        b = np.asarray(eval_expr(e[3], env, extras))
        if op == "+":
            return a + b
        if op == "-":
            return a - b
        if op == "*":
            return a * b
        if op == "/":
            return _c_div(a, b)
        if op == "%":
            return _c_mod(a, b)
        if op == "<<":
            return a << b
        if op == ">>":
            return a >> b
        if op == "<":
            return (a < b).astype(np.int64)
        if op == "<=":
            return (a <= b).astype(np.int64)
        if op == ">":
            return (a > b).astype(np.int64)
        if op == ">=":
            return (a >= b).astype(np.int64)
        if op == "==":
            return (a == b).astype(np.int64)
        if op == "!=":
            return (a != b).astype(np.int64)
        if op == "&":
            return a & b
        if op == "|":
            return a | b
        if op == "^":
            return a ^ b
        if op == "&&":
            return ((a != 0) & (b != 0)).astype(np.int64)
        if op == "||":
            return ((a != 0) | (b != 0)).astype(np.int64)
    raise ValueError("bad expression node %r" % (e,))


def _index_env(loop_shape, xshape, yshape):
    """i0..in over `loop_shape`, plus the names of ops/reindex_op.cc:121-130."""
    env = {}
    n = len(loop_shape)
    for d in range(n):
        sh = [1] * n
        sh[d] = loop_shape[d]
        env["i%d" % d] = np.arange(loop_shape[d], dtype=np.int64).reshape(sh)
    for name, shp in (("x", xshape), ("y", yshape)):
        st = 1
        for d in range(len(shp) - 1, -1, -1):
            env["%sshape%d" % (name, d)] = np.int64(shp[d])
            env["%sstride%d" % (name, d)] = np.int64(st)
            st *= shp[d]
    env["XDIM"] = np.int64(len(xshape))
    env["YDIM"] = np.int64(len(yshape))
    return env


def _targets(loop_shape, xshape, yshape, indexes, overflow_conditions, extras):
    """Flat x index and overflow flag for every loop coordinate
    (ops/reindex_op.cc:132-136, ops/reindex_reduce_op.cc:123-128)."""
    env = _index_env(loop_shape, xshape, yshape)
    ov = np.zeros(loop_shape, dtype=bool)
    flat = np.zeros(loop_shape, dtype=np.int64)
    st = 1
    strides = []
    for d in range(len(xshape) - 1, -1, -1):
        strides.insert(0, st)
        st *= xshape[d]
    for d, s in enumerate(indexes):
        v = np.asarray(eval_expr(parse_expr(s), env, extras))
        if v.dtype.kind == "f":
            v = np.trunc(v)          # index_t xid = <float expression>
        v = np.broadcast_to(v.astype(np.int64), loop_shape)
        ov |= (v < 0) | (v >= xshape[d])
        flat = flat + v * strides[d]
    for s in overflow_conditions:
        v = np.asarray(eval_expr(parse_expr(s), env, extras))
        ov |= np.broadcast_to(v != 0, loop_shape)
    return flat, ov


def reindex(x, shape, indexes, overflow_value=0, overflow_conditions=(), extras=()):
    """y[i...] = overflow ? Tx(ov) : x[idx(i...)]  (ops/reindex_op.cc:111-139)."""
    bf = isinstance(x, BF16)
    xa = x.bits if bf else np.asarray(x)
    if len(indexes) != xa.ndim:
        raise ValueError("Number of x's shape and indexes should be the same.")
    shape = list(shape) if len(shape) else list(np.asarray(extras[0]).shape)
    if not shape:
        raise ValueError("Number of shape should greater than 0.")
    flat, ov = _targets(shape, xa.shape, shape, indexes, overflow_conditions, extras)
    if bf:
        ovv = f32_to_bf16_bits(np.float32(overflow_value))[()]
    else:
        ovv = c_cast(np.float64(overflow_value), dtype_name(xa))[()]
    safe = np.where(ov, 0, flat)
    if xa.size == 0:
        y = np.full(shape, ovv, dtype=xa.dtype)
    else:
        y = np.where(ov, ovv, xa.reshape(-1)[safe]).astype(xa.dtype)
    return BF16(y) if bf else y


def reindex_reduce(y, op, shape, indexes, overflow_conditions=(), extras=()):
    """x initialised with init_OP, then for every y coordinate in row-major
    order: x[idx] = OP(x[idx], y[i]) unless overflow
    (ops/reindex_reduce_op.cc:93-131).  Sequential order is kept: numpy's
    ufunc.at applies updates one by one in index order."""
    ya = np.asarray(y)
    tx = dtype_name(ya)
    if op not in BINARY_OPS and op != "void" or op == "mean":
        raise ValueError("unsupported reindex_reduce op %r" % op)
    if len(shape) != len(indexes) or len(shape) == 0:
        raise ValueError("Number of shape and indexes should be the same.")
    if any(int(s) < 0 for s in shape):
        raise ValueError("Shape should greater than 0.")
    shape = [int(s) for s in shape]
    flat, ov = _targets(list(ya.shape), shape, list(ya.shape), indexes, overflow_conditions, extras)
    T = _NP[tx]
    n = int(np.prod(shape, dtype=np.int64))
    x = np.full(n, _identity(op, tx) if op != "void" else 0, dtype=T)
    keep = ~ov.reshape(-1)
    tgt = flat.reshape(-1)[keep]
    val = ya.reshape(-1)[keep]
    with np.errstate(all="ignore"):
        if op == "add":
            np.add.at(x, tgt, val)
        elif op == "subtract":
            np.subtract.at(x, tgt, val)
        elif op == "multiply":
            np.multiply.at(x, tgt, val)
        elif op == "maximum":
            # std::max(cur, v): NaN in v never replaces cur
            v2 = np.where(np.isnan(val), x.dtype.type(_identity(op, tx)), val) if T in (np.float32, np.float64) else val
            np.maximum.at(x, tgt, v2)
        elif op == "minimum":
            v2 = np.where(np.isnan(val), x.dtype.type(_identity(op, tx)), val) if T in (np.float32, np.float64) else val
            np.minimum.at(x, tgt, v2)
        elif op == "bitwise_and":
            np.bitwise_and.at(x, tgt, val)
        elif op == "bitwise_or":
            np.bitwise_or.at(x, tgt, val)
        elif op == "bitwise_xor":
            np.bitwise_xor.at(x, tgt, val)
        elif op == "void":
            x[tgt] = val          # last writer in loop order wins
        else:
            for t, v in zip(tgt, val):
                x[t] = binary(x[t:t + 1], np.asarray([v]), op, tx)[0]
    return x.reshape(shape)


# --------------------------------------------------------------------------
# meta-op convolution (python/jittor/nn.py:1245-1262 expressed with the ops
# above; dtype flow of opt/kernel_ir.cc:958-968 + ops/reduce_op.cc:259-266:
# float products, float32 accumulation in loop order (c, kh, kw))
# --------------------------------------------------------------------------
def conv_meta(x, w, stride=1, padding=0, dilation=1):
    """x [N,C,H,W], w [K,C,R,S] (float32 arrays or BF16); returns the
    float32 accumulator y [N,K,OH,OW]."""
    xf = x.to_f32() if isinstance(x, BF16) else np.asarray(x, dtype=np.float32)
    wf = w.to_f32() if isinstance(w, BF16) else np.asarray(w, dtype=np.float32)
    N, C, H, W = xf.shape
    K, _, R, S = wf.shape
    oh = (H + padding * 2 - R * dilation + dilation - 1) // stride + 1
    ow = (W + padding * 2 - S * dilation + dilation - 1) // stride + 1
    xx = reindex(xf, [N, K, C, oh, ow, R, S],
                 ["i0", "i2", "i3*%d-%d+i5*%d" % (stride, padding, dilation),
                  "i4*%d-%d+i6*%d" % (stride, padding, dilation)])
    ww = broadcast_to(wf, xx.shape, [0, 3, 4])
    yy = binary(xx, ww, "multiply")
    return reduce(yy, "add", [2, 5, 6])


def conv_meta_grouped(x, w, groups, stride=1, padding=0, dilation=1):
    """The grouped form, python/jittor/nn.py:1272-1294: x [N,G*Cg,H,W], w [K,Cg,R,S];
    reindex(x) * reindex(w) over [N,G,K/G,Cg,OH,OW,R,S], then reindex_reduce.add into
    [N,K,OH,OW] (a sequential float32 sum in the loop order of the 8-d product)."""
    xf = x.to_f32() if isinstance(x, BF16) else np.asarray(x, dtype=np.float32)
    wf = w.to_f32() if isinstance(w, BF16) else np.asarray(w, dtype=np.float32)
    N, C, H, W = xf.shape
    K, CpG, R, S = wf.shape
    G = groups
    assert C == CpG * G and K % G == 0
    oh = (H + padding * 2 - R * dilation + dilation - 1) // stride + 1
    ow = (W + padding * 2 - S * dilation + dilation - 1) // stride + 1
    shape = [N, G, K // G, CpG, oh, ow, R, S]
    xx = reindex(xf, shape, ["i0", "i1*%d+i3" % CpG, "i4*%d-%d+i6*%d" % (stride, padding, dilation),
                             "i5*%d-%d+i7*%d" % (stride, padding, dilation)])
    ww = reindex(wf, shape, ["i1*%d+i2" % (K // G), "i3", "i6", "i7"])
    yy = binary(xx, ww, "multiply")
    return reindex_reduce(yy, "add", [N, K, oh, ow], ["i0", "i1*%d+i2" % (K // G), "i4", "i5"])


def conv_meta_grouped_grads(x, w, dy, groups, stride=1, padding=0, dilation=1):
    """Gradients of conv_meta_grouped with respect to x and w for an output gradient dy, as jt.grad builds
    them over the same 8-d product: the scatter-add's gradient is a reindex of dy with the scatter's indexes
    (ops/reindex_reduce_op.cc:45-63), the product's is that times the other factor, and each reindex's
    gradient is a scatter-add with the reindex's own indexes, out-of-range ones dropped
    (ops/reindex_op.cc:76-80).  stride / padding / dilation: a number or a (vertical, horizontal) pair.
    Returns float32 (dx [N,G*Cg,H,W], dw [K,Cg,R,S])."""
    xf = x.to_f32() if isinstance(x, BF16) else np.asarray(x, dtype=np.float32)
    wf = w.to_f32() if isinstance(w, BF16) else np.asarray(w, dtype=np.float32)
    df = dy.to_f32() if isinstance(dy, BF16) else np.asarray(dy, dtype=np.float32)
    N, C, H, W = xf.shape
    K, CpG, R, S = wf.shape
    G = groups
    assert C == CpG * G and K % G == 0
    (sh, sw), (ph, pw), (dh, dw_) = [v if isinstance(v, (tuple, list)) else (v, v) for v in (stride, padding, dilation)]
    oh = (H + ph * 2 - R * dh + dh - 1) // sh + 1
    ow = (W + pw * 2 - S * dw_ + dw_ - 1) // sw + 1
    assert list(df.shape) == [N, K, oh, ow]
    shape = [N, G, K // G, CpG, oh, ow, R, S]
    xi = ["i0", "i1*%d+i3" % CpG, "i4*%d-%d+i6*%d" % (sh, ph, dh), "i5*%d-%d+i7*%d" % (sw, pw, dw_)]
    wi = ["i1*%d+i2" % (K // G), "i3", "i6", "i7"]
    yi = ["i0", "i1*%d+i2" % (K // G), "i4", "i5"]
    xx, ww, dd = reindex(xf, shape, xi), reindex(wf, shape, wi), reindex(df, shape, yi)
    dx = reindex_reduce(binary(dd, ww, "multiply"), "add", [N, C, H, W], xi)
    dw = reindex_reduce(binary(dd, xx, "multiply"), "add", [K, CpG, R, S], wi)
    return dx, dw


def conv_meta_wgrad(x, dy, R, S, stride=1, padding=0, dilation=1):
    """Gradient of conv_meta with respect to w for an output gradient dy, as jt.grad builds it from
    the op rules: the sum's gradient is a broadcast of dy over (c, kh, kw) (ops/reduce_op.cc:339-362),
    the product's is dy times the other factor, the broadcast's is a sum over its axes (n, oh, ow)
    (ops/broadcast_to_op.cc:112-117).  x [N,C,H,W], dy [N,K,OH,OW] (float32 arrays or BF16); returns the
    float32 accumulator dw [K,C,R,S]."""
    xf = x.to_f32() if isinstance(x, BF16) else np.asarray(x, dtype=np.float32)
    df = dy.to_f32() if isinstance(dy, BF16) else np.asarray(dy, dtype=np.float32)
    N, C, H, W = xf.shape
    _, K, oh, ow = df.shape
    xx = reindex(xf, [N, K, C, oh, ow, R, S],
                 ["i0", "i2", "i3*%d-%d+i5*%d" % (stride, padding, dilation),
                  "i4*%d-%d+i6*%d" % (stride, padding, dilation)])
    dd = broadcast_to(df, xx.shape, [2, 5, 6])
    return reduce(binary(xx, dd, "multiply"), "add", [0, 3, 4])

