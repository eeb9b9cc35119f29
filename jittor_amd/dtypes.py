"""dtype vocabulary and inference rules of the meta-operator path.

Restates python/jittor/src/misc/nano_string.h:199-277, including the
mixed-precision control register amp_reg (python/jittor/src/var.cc:28,65-71),
and the op classes of python/jittor/src/misc/nano_string.cc:45-160.
"""
import numpy as np

from ._lib import DTYPES, DTYPE_SIZE, NP_STORAGE, BINARY_OPS, UNARY_OPS

BOOL_OPS = {"logical_not", "less", "less_equal", "greater", "greater_equal",
            "equal", "not_equal", "logical_and", "logical_or", "logical_xor"}
FLOAT_OPS = {"log", "exp", "sqrt", "mean", "divide", "sin", "asin", "sinh",
             "asinh", "tan", "atan", "tanh", "atanh", "cos", "acos", "cosh",
             "acosh", "sigmoid", "erf", "erfinv"}
INT_OPS = {"round_int", "floor_int", "ceil_int", "floor_divide"}
WHITE_OPS = {"exp", "pow"}
# ops a parallel reduction may reorder
REDUCE_OPS = ["add", "multiply", "maximum", "minimum", "logical_and",
              "logical_or", "logical_xor", "bitwise_and", "bitwise_or",
              "bitwise_xor", "mean"]


# amp_reg bits (nano_string.h:199-203; bit 32: ops/reduce_op.cc:260)
AMP_PREFER32 = 1
AMP_PREFER16 = 2
AMP_KEEP_REDUCE = 4
AMP_KEEP_WHITE = 8
AMP_ARRAY_PREFER = 16
AMP_REDUCE16_DIRECT = 32      # a 16-bit add / mean is not rewritten to cast -> reduce(float32) -> cast
amp_reg = 0


def amp_reg_of_level(level):
    """auto_mixed_precision_level -> amp_reg (var.cc:65-71)."""
    if level <= 2:
        return 0
    return {3: AMP_KEEP_REDUCE | AMP_KEEP_WHITE, 4: AMP_PREFER16, 5: AMP_PREFER16 | AMP_ARRAY_PREFER,
            6: AMP_PREFER16 | AMP_ARRAY_PREFER | AMP_KEEP_REDUCE | AMP_KEEP_WHITE}.get(level, amp_reg)


def dsize_(name):
    return {1: 0, 2: 1, 4: 2, 8: 3}[DTYPE_SIZE[name]]


def is_float(name):
    return name in ("float16", "float32", "float64", "bfloat16")


def is_int(name):
    return name in ("int8", "int16", "int32", "int64", "uint8", "uint16", "uint32", "uint64")


def float_dtype(d, has_scalar=False, has_bf16=False):
    """nano_string.h:205-215."""
    if not has_scalar:
        if amp_reg & AMP_PREFER32:
            return "float32"
        if amp_reg & AMP_PREFER16:
            return "bfloat16" if has_bf16 else "float16"
    if d == 3:
        return "float64"
    if d == 2:
        return "float32"
    return "bfloat16" if has_bf16 else "float16"


def int_dtype(d):
    """nano_string.h:217-221."""
    return {3: "int64", 2: "int32", 1: "int16", 0: "int8"}[d]


def dtype_infer(x, y, xscalar=False, yscalar=False):
    """nano_string.h:223-235."""
    d = max(dsize_(x), dsize_(y))
    if xscalar:
        d = dsize_(y)
    if yscalar:
        d = dsize_(x)
    if is_float(x) or is_float(y):
        return float_dtype(d, xscalar or yscalar, "bfloat16" in (x, y))
    return int_dtype(d)


def binary_dtype_infer(op, x, y, xscalar=False, yscalar=False):
    """nano_string.h:238-254."""
    if op in BOOL_OPS:
        return "bool"
    d = max(dsize_(x), dsize_(y))
    if xscalar:
        d = dsize_(y)
    if yscalar:
        d = dsize_(x)
    fl = op not in INT_OPS and (is_float(x) or is_float(y) or op in FLOAT_OPS)
    if fl:
        if op in WHITE_OPS and not amp_reg & AMP_KEEP_WHITE:
            return "float64" if d == 3 else "float32"
        return float_dtype(d, xscalar or yscalar, "bfloat16" in (x, y))
    if x == "bool" and y == "bool":
        return "bool"
    return int_dtype(d)


def unary_dtype_infer(op, x):
    """nano_string.h:256-266."""
    if op in BOOL_OPS:
        return "bool"
    d = dsize_(x)
    if op in FLOAT_OPS:
        if op in WHITE_OPS and not amp_reg & AMP_KEEP_WHITE:
            return "float64" if d == 3 else "float32"
        return float_dtype(d, False, x == "bfloat16")
    if op in INT_OPS:
        return int_dtype(d)
    return x


def reduce_dtype_infer(op, x):
    """nano_string.h:268-277, and bool -> int32 of ops/reduce_op.cc:287-290."""
    if x == "bool":
        return "int32"
    if is_float(x) or op in FLOAT_OPS:
        if amp_reg & AMP_KEEP_REDUCE:
            return float_dtype(dsize_(x), False, x == "bfloat16")
        return "float64" if dsize_(x) == 3 else "float32"
    return x


def normalize_dtype(dtype):
    """Accepts a dtype name, a numpy dtype or a cast function (jt.float32)."""
    if dtype is None:
        return None
    if isinstance(dtype, str):
        name = {"float": "float32", "int": "int32", "double": "float64", "half": "float16"}.get(dtype, dtype)
    elif callable(dtype) and hasattr(dtype, "__name__") and dtype.__name__ in DTYPES:
        name = dtype.__name__
    else:
        name = np.dtype(dtype).name
        if name == "bool_":
            name = "bool"
    if name not in DTYPES or name == "void":
        raise ValueError("unknown dtype %r" % (dtype,))
    return name


def np_to_dtype(arr):
    name = arr.dtype.name
    return "bool" if name in ("bool", "bool_") else name


def f32_to_bf16_bits(a):
    """bfloat16 <- float keeps the upper 16 bits (type/fp16_compute.h:238-241)."""
    a = np.ascontiguousarray(a, dtype=np.float32)
    return (a.view(np.uint32) >> 16).astype(np.uint16)


def bf16_bits_to_f32(bits):
    return (np.asarray(bits, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)
