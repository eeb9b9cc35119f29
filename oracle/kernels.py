"""ctypes loader for oracle/_build/liboracle_kernels.so.  TEST INFRASTRUCTURE
ONLY (see oracle_kernels.cc): the C++ restatement of the reference's CPU
kernels for the benchmark configurations, used as checker and as the timed CPU
baseline."""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "_build", "liboracle_kernels.so")
_lib = None


def build(force=False):
    if force or not os.path.exists(_SO):
        subprocess.check_call(["make", "-B" if force else "-s", "-C", _HERE])
    return _SO


def load():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = ctypes.CDLL(_SO)
    return _lib


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def max_threads():
    return load().ork_max_threads()


def reduce_sum_axis1(x, threads=1):
    x = np.ascontiguousarray(x, np.float32)
    y = np.empty(x.shape[0], np.float32)
    load().ork_reduce_sum_axis1(_p(x), _p(y), x.shape[0], x.shape[1], threads)
    return y


def reindex_im2col3x3(x, threads=1, out=None):
    x = np.ascontiguousarray(x, np.float32)
    N, C, H, W = x.shape
    y = out if out is not None else np.empty((N, C, H, W, 3, 3), np.float32)
    load().ork_reindex_im2col3x3(_p(x), _p(y), N, C, H, W, threads)
    return y


def scatter_1d(v, idx, bins, op):
    v = np.ascontiguousarray(v, np.float32)
    idx = np.ascontiguousarray(idx, np.int32)
    x = np.empty(bins, np.float32)
    load().ork_scatter_1d(_p(v), _p(idx), _p(x), v.shape[0], bins, {"add": 0, "maximum": 1}[op])
    return x


def fused_chain(x, scale, bias, threads=1, out=None):
    x = np.ascontiguousarray(x, np.float32)
    s = np.ascontiguousarray(scale, np.float32).reshape(-1)
    b = np.ascontiguousarray(bias, np.float32).reshape(-1)
    z = out if out is not None else np.empty_like(x)
    load().ork_fused_chain(_p(x), _p(s), _p(b), _p(z), x.shape[0], x.shape[1], x.shape[2], threads)
    return z


def conv_meta_bf16(xbits, wbits, stride=1, pad=1, dil=1, threads=1):
    xbits = np.ascontiguousarray(xbits, np.uint16)
    wbits = np.ascontiguousarray(wbits, np.uint16)
    N, C, H, W = xbits.shape
    K, _, R, S = wbits.shape
    oh = (H + pad * 2 - R * dil + dil - 1) // stride + 1
    ow = (W + pad * 2 - S * dil + dil - 1) // stride + 1
    y = np.empty((N, K, oh, ow), np.float32)
    load().ork_conv_meta_bf16(_p(xbits), _p(wbits), _p(y), N, C, H, W, K, R, S, stride, pad, dil, threads)
    return y
