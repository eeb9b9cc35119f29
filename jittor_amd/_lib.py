"""ctypes binding of libmjt.so (declarations: include/mjt.h).

The library is the only execution path: when it cannot be loaded, or when a
call fails, an exception is raised -- there is no host fallback.
"""
import ctypes
import os

import numpy as np

MAX_DIM = 10
_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libmjt.so")

DTYPES = ["void", "bool", "int8", "int16", "int32", "int64", "uint8", "uint16",
          "uint32", "uint64", "float16", "float32", "float64", "bfloat16"]
DTYPE_CODE = {n: i for i, n in enumerate(DTYPES)}
DTYPE_SIZE = {"bool": 1, "int8": 1, "int16": 2, "int32": 4, "int64": 8,
              "uint8": 1, "uint16": 2, "uint32": 4, "uint64": 8, "float16": 2,
              "float32": 4, "float64": 8, "bfloat16": 2}
# numpy storage type per dtype (bfloat16 is carried as raw uint16 bits)
NP_STORAGE = {"bool": np.bool_, "int8": np.int8, "int16": np.int16,
              "int32": np.int32, "int64": np.int64, "uint8": np.uint8,
              "uint16": np.uint16, "uint32": np.uint32, "uint64": np.uint64,
              "float16": np.float16, "float32": np.float32,
              "float64": np.float64, "bfloat16": np.uint16}

OPS = ["pow", "maximum", "minimum", "add", "subtract", "multiply", "divide",
       "floor_divide", "mod", "less", "less_equal", "greater", "greater_equal",
       "equal", "not_equal", "left_shift", "right_shift", "logical_and",
       "logical_or", "logical_xor", "bitwise_and", "bitwise_or", "bitwise_xor",
       "mean", "abs", "negative", "logical_not", "bitwise_not", "log", "exp",
       "sqrt", "round", "floor", "ceil", "round_int", "floor_int", "ceil_int",
       "cast", "sin", "asin", "sinh", "asinh", "tan", "atan", "tanh", "atanh",
       "cos", "acos", "cosh", "acosh", "erf", "erfinv", "sigmoid", "void"]
OP_CODE = {n: i for i, n in enumerate(OPS)}
BINARY_OPS = OPS[:24]
UNARY_OPS = OPS[24:53]

VAR_INPUT, VAR_INTERMEDIATE, VAR_OUTPUT, VAR_SCALAR, VAR_GATHERED = 0, 1, 2, 3, 4
FOP_UNARY, FOP_BINARY, FOP_TERNARY, FOP_BROADCAST = 0, 1, 2, 3
ERR_INVALID, ERR_UNSUPPORTED, ERR_COMPILE, ERR_DEVICE, ERR_NOT_INIT = -1, -2, -3, -4, -5     # mjt_status


class MjtError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__("libmjt error %d: %s" % (code, msg))
        self.code = code


class Tensor(ctypes.Structure):
    _fields_ = [("ptr", ctypes.c_void_p), ("dtype", ctypes.c_int32),
                ("ndim", ctypes.c_int32), ("shape", ctypes.c_int64 * MAX_DIM)]


class DeviceInfo(ctypes.Structure):
    _fields_ = [("name", ctypes.c_char * 256), ("arch", ctypes.c_char * 64),
                ("compute_units", ctypes.c_int32), ("clock_khz", ctypes.c_int32),
                ("mem_clock_khz", ctypes.c_int32), ("mem_bus_bits", ctypes.c_int32),
                ("lds_bytes_per_block", ctypes.c_int32), ("wavefront", ctypes.c_int32),
                ("hbm_bytes", ctypes.c_uint64), ("l2_bytes", ctypes.c_uint64)]


class FusedVar(ctypes.Structure):
    _fields_ = [("role", ctypes.c_int32), ("dtype", ctypes.c_int32),
                ("ptr", ctypes.c_void_p), ("fvalue", ctypes.c_double),
                ("ivalue", ctypes.c_int64), ("bcast_mask", ctypes.c_uint32),
                ("reserved", ctypes.c_uint32)]


class FusedOp(ctypes.Structure):
    _fields_ = [("kind", ctypes.c_int32), ("op", ctypes.c_int32),
                ("inp", ctypes.c_int32 * 3), ("out", ctypes.c_int32)]


class FusedDesc(ctypes.Structure):
    _fields_ = [("ndim", ctypes.c_int32), ("shape", ctypes.c_int64 * MAX_DIM),
                ("n_vars", ctypes.c_int32), ("vars", ctypes.POINTER(FusedVar)),
                ("n_ops", ctypes.c_int32), ("ops", ctypes.POINTER(FusedOp))]


class ConvParams(ctypes.Structure):
    _fields_ = [("stride_h", ctypes.c_int32), ("stride_w", ctypes.c_int32),
                ("pad_h", ctypes.c_int32), ("pad_w", ctypes.c_int32),
                ("dil_h", ctypes.c_int32), ("dil_w", ctypes.c_int32)]


# every symbol include/mjt.h declares
EXPORTS = ["mjt_init", "mjt_shutdown", "mjt_last_error", "mjt_get_device_info",
           "mjt_dtype_name", "mjt_op_name", "mjt_dtype_from_name", "mjt_op_from_name",
           "mjt_alloc", "mjt_free", "mjt_h2d", "mjt_d2h", "mjt_d2d", "mjt_fill_u32",
           "mjt_sync", "mjt_event_create", "mjt_event_record", "mjt_event_elapsed_ms",
           "mjt_event_destroy", "mjt_reduce", "mjt_reduce_static", "mjt_reindex", "mjt_reindex_reduce",
           "mjt_fused_elementwise", "mjt_fused_reduce", "mjt_conv2d_meta", "mjt_conv2d_meta_pack", "mjt_conv2d_meta_packed", "mjt_conv2d_meta_grouped", "mjt_conv2d_meta_dgrad", "mjt_conv2d_meta_wgrad", "mjt_conv2d_meta_wgrad_grouped",
           "mjt_reindex_then_reduce", "mjt_fused_reindex_reduce", "mjt_matmul", "mjt_matmul_available",
           "mjt_expr_affine", "mjt_where_count", "mjt_where",
           "mjt_jit_stats", "mjt_last_kernel"]

_lib = None
_device = None


def load():
    """Loads libmjt.so (built by __graft_entry__.build() / csrc/Makefile)."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise MjtError(-5, "libmjt.so is not built (%s); run `make -C jittor_amd/csrc` "
                           "or __graft_entry__.build()" % LIB_PATH)
    lib = ctypes.CDLL(LIB_PATH)
    lib.mjt_last_error.restype = ctypes.c_char_p
    lib.mjt_last_kernel.restype = ctypes.c_char_p
    lib.mjt_dtype_name.restype = ctypes.c_char_p
    lib.mjt_op_name.restype = ctypes.c_char_p
    lib.mjt_shutdown.restype = None
    lib.mjt_alloc.argtypes = [ctypes.c_size_t, ctypes.POINTER(ctypes.c_void_p)]
    lib.mjt_free.argtypes = [ctypes.c_void_p]
    lib.mjt_h2d.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t]
    lib.mjt_d2h.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t]
    lib.mjt_d2d.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t]
    lib.mjt_fill_u32.argtypes = [ctypes.c_void_p, ctypes.c_uint32, ctypes.c_size_t]
    lib.mjt_event_create.argtypes = [ctypes.POINTER(ctypes.c_void_p)]
    lib.mjt_event_record.argtypes = [ctypes.c_void_p]
    lib.mjt_event_elapsed_ms.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.POINTER(ctypes.c_float)]
    lib.mjt_event_destroy.argtypes = [ctypes.c_void_p]
    lib.mjt_reduce.argtypes = [ctypes.POINTER(Tensor), ctypes.POINTER(Tensor), ctypes.c_int, ctypes.c_uint32]
    lib.mjt_reduce_static.argtypes = [ctypes.POINTER(Tensor), ctypes.POINTER(Tensor), ctypes.c_int, ctypes.c_uint32]
    strs = ctypes.POINTER(ctypes.c_char_p)
    lib.mjt_reindex.argtypes = [ctypes.POINTER(Tensor), ctypes.POINTER(Tensor), ctypes.c_int, strs,
                                ctypes.c_double, ctypes.c_int, strs, ctypes.c_int, ctypes.POINTER(Tensor)]
    lib.mjt_reindex_reduce.argtypes = [ctypes.POINTER(Tensor), ctypes.POINTER(Tensor), ctypes.c_int,
                                       ctypes.c_int, strs, ctypes.c_int, strs, ctypes.c_int,
                                       ctypes.POINTER(Tensor)]
    lib.mjt_reindex_then_reduce.argtypes = [ctypes.POINTER(Tensor), ctypes.POINTER(Tensor), ctypes.POINTER(Tensor), ctypes.c_int,
                                            ctypes.c_int, ctypes.c_int, strs, ctypes.c_double, ctypes.c_int, strs, ctypes.c_int,
                                            ctypes.POINTER(Tensor)]
    lib.mjt_fused_reindex_reduce.argtypes = [ctypes.POINTER(FusedDesc), ctypes.POINTER(Tensor), ctypes.c_int, ctypes.c_int, strs,
                                             ctypes.c_int, strs, ctypes.c_int, ctypes.POINTER(Tensor)]
    lib.mjt_fused_elementwise.argtypes = [ctypes.POINTER(FusedDesc)]
    lib.mjt_fused_reduce.argtypes = [ctypes.POINTER(FusedDesc), ctypes.POINTER(Tensor), ctypes.c_int, ctypes.c_uint32]
    lib.mjt_conv2d_meta.argtypes = [ctypes.POINTER(Tensor), ctypes.POINTER(Tensor), ctypes.POINTER(Tensor),
                                    ctypes.POINTER(ConvParams)]
    lib.mjt_conv2d_meta_pack.argtypes = [ctypes.POINTER(Tensor), ctypes.POINTER(Tensor), ctypes.POINTER(Tensor),
                                         ctypes.POINTER(ConvParams), ctypes.c_void_p, ctypes.c_size_t]
    lib.mjt_conv2d_meta_packed.argtypes = [ctypes.POINTER(Tensor), ctypes.POINTER(Tensor), ctypes.c_void_p, ctypes.POINTER(Tensor),
                                           ctypes.POINTER(ConvParams)]
    lib.mjt_conv2d_meta_grouped.argtypes = [ctypes.POINTER(Tensor), ctypes.POINTER(Tensor), ctypes.POINTER(Tensor),
                                            ctypes.POINTER(ConvParams), ctypes.c_int]
    lib.mjt_conv2d_meta_dgrad.argtypes = [ctypes.POINTER(Tensor), ctypes.POINTER(Tensor), ctypes.POINTER(Tensor),
                                          ctypes.POINTER(ConvParams)]
    lib.mjt_conv2d_meta_wgrad.argtypes = [ctypes.POINTER(Tensor), ctypes.POINTER(Tensor), ctypes.POINTER(Tensor),
                                          ctypes.POINTER(ConvParams)]
    lib.mjt_conv2d_meta_wgrad_grouped.argtypes = [ctypes.POINTER(Tensor), ctypes.POINTER(Tensor), ctypes.POINTER(Tensor),
                                                  ctypes.POINTER(ConvParams), ctypes.c_int]
    lib.mjt_matmul.argtypes = [ctypes.POINTER(Tensor), ctypes.POINTER(Tensor), ctypes.POINTER(Tensor), ctypes.c_int, ctypes.c_int]
    lib.mjt_matmul_available.argtypes = []
    lib.mjt_where_count.argtypes = [ctypes.POINTER(Tensor), ctypes.POINTER(ctypes.c_int64)]
    lib.mjt_where.argtypes = [ctypes.POINTER(Tensor), ctypes.c_int64, ctypes.POINTER(Tensor)]
    lib.mjt_expr_affine.argtypes = [ctypes.c_char_p, ctypes.POINTER(Tensor), ctypes.POINTER(Tensor),
                                    ctypes.POINTER(ctypes.c_int64), ctypes.POINTER(ctypes.c_int64)]
    lib.mjt_jit_stats.argtypes = [ctypes.POINTER(ctypes.c_int64), ctypes.POINTER(ctypes.c_int64)]
    _lib = lib
    return lib


def check(rc):
    if rc < 0:
        raise MjtError(rc, load().mjt_last_error().decode("utf-8", "replace"))
    return rc


def init(device=0):
    """Binds the library to a device (-1 = compile-only mode, no GPU needed)."""
    global _device
    lib = load()
    if _device is not None and _device != device:
        lib.mjt_shutdown()
        _device = None
    check(lib.mjt_init(int(device)))
    _device = device
    return lib


def device():
    return _device


def ensure_init():
    if _device is None:
        init(int(os.environ.get("MJT_DEVICE", "0")))
    return _lib


def shutdown():
    global _device
    if _lib is not None:
        _lib.mjt_shutdown()
    _device = None


def tensor(ptr, dtype, shape):
    t = Tensor()
    t.ptr = ptr
    t.dtype = DTYPE_CODE[dtype] if isinstance(dtype, str) else int(dtype)
    shape = list(shape)
    if len(shape) > MAX_DIM:
        raise MjtError(-1, "rank %d exceeds %d" % (len(shape), MAX_DIM))
    t.ndim = len(shape)
    for i, s in enumerate(shape):
        t.shape[i] = int(s)
    return t


def c_strings(items):
    arr = (ctypes.c_char_p * max(1, len(items)))()
    for i, s in enumerate(items):
        arr[i] = s.encode()
    return arr


def alloc(nbytes):
    p = ctypes.c_void_p()
    check(ensure_init().mjt_alloc(int(nbytes), ctypes.byref(p)))
    return p.value


def free(ptr):
    if _lib is not None and _device is not None and ptr:
        _lib.mjt_free(ctypes.c_void_p(ptr))


def h2d(ptr, array):
    array = np.ascontiguousarray(array)
    check(_lib.mjt_h2d(ctypes.c_void_p(ptr), array.ctypes.data_as(ctypes.c_void_p), array.nbytes))


def d2h(ptr, shape, np_dtype):
    out = np.empty(shape, dtype=np_dtype)
    if out.nbytes:
        check(_lib.mjt_d2h(out.ctypes.data_as(ctypes.c_void_p), ctypes.c_void_p(ptr), out.nbytes))
    return out


def sync():
    check(ensure_init().mjt_sync())


def device_info():
    di = DeviceInfo()
    check(ensure_init().mjt_get_device_info(ctypes.byref(di)))
    return di


def last_kernel():
    return load().mjt_last_kernel().decode()


def jit_stats():
    a, b = ctypes.c_int64(), ctypes.c_int64()
    load().mjt_jit_stats(ctypes.byref(a), ctypes.byref(b))
    return a.value, b.value


class Event:
    def __init__(self):
        self.h = ctypes.c_void_p()
        check(ensure_init().mjt_event_create(ctypes.byref(self.h)))

    def record(self):
        check(_lib.mjt_event_record(self.h))
        return self

    def elapsed_ms_since(self, start):
        ms = ctypes.c_float()
        check(_lib.mjt_event_elapsed_ms(start.h, self.h, ctypes.byref(ms)))
        return ms.value

    def __del__(self):
        try:
            if _device is not None and self.h:
                _lib.mjt_event_destroy(self.h)
        except Exception:
            pass


def expr_affine(expr, xshape, yshape):
    """(c0, coef[10]) when `expr` is affine in i0..i9, else None."""
    x, y = tensor(None, "float32", xshape), tensor(None, "float32", yshape)
    c0 = ctypes.c_int64()
    coef = (ctypes.c_int64 * MAX_DIM)()
    rc = check(load().mjt_expr_affine(expr.encode(), ctypes.byref(x), ctypes.byref(y), ctypes.byref(c0), coef))
    return (c0.value, list(coef)) if rc == 1 else None
