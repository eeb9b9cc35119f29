"""Callers that define the patterns of the path: relu and conv2d expressed
with meta-operators exactly as the reference writes them
(python/jittor/nn.py:166-183 and :1245-1269)."""
from . import core


def relu(x):
    """ternary(x > 0.0, x, 0.0) (python/jittor/nn.py:182-183)."""
    cond = core.binary(x, 0.0, "greater")
    return core.ternary(cond, x, 0.0)


def sigmoid(x):
    return core.unary(x, "sigmoid")


def _pair(v):
    return (v, v) if isinstance(v, int) else tuple(v)


def conv2d(x, weight, bias=None, stride=1, padding=0, dilation=1, groups=1):
    """The meta-op convolution: reindex + broadcast + multiply + sum over
    (C, Kh, Kw) (python/jittor/nn.py:1245-1269, groups == 1).  The executor
    recognises the group and runs it as one MFMA kernel."""
    if groups != 1:
        raise NotImplementedError("conv2d: groups > 1 is outside the meta-op convolution path")
    padding, stride, dilation = _pair(padding), _pair(stride), _pair(dilation)
    N, C, H, W = x.shape
    K = weight.shape[0]
    Kh, Kw = weight.shape[-2:]
    oh = (H + padding[0] * 2 - Kh * dilation[0] + dilation[0] - 1) // stride[0] + 1
    ow = (W + padding[1] * 2 - Kw * dilation[1] + dilation[1] - 1) // stride[1] + 1
    xx = x.reindex([N, K, C, oh, ow, Kh, Kw], [
        "i0",
        "i2",
        "i3*%d-%d+i5*%d" % (stride[0], padding[0], dilation[0]),
        "i4*%d-%d+i6*%d" % (stride[1], padding[1], dilation[1]),
    ])
    ww = weight.broadcast(xx.shape, [0, 3, 4])
    yy = xx * ww
    y = yy.sum([2, 5, 6])
    if bias is not None:
        b = bias.broadcast(y.shape, [0, 2, 3])
        y = y + b
    return y


def pad(x, padding, mode="constant", value=0):
    from .misc import pad as _pad
    return _pad(x, padding, mode, value)


def pool(x, kernel_size, op, padding=0, stride=None):
    from .misc import pool as _pool
    return _pool(x, kernel_size, op, padding, stride)


def max_pool2d(x, kernel_size, stride=None, padding=0):
    return pool(x, kernel_size, "maximum", padding, stride)


def avg_pool2d(x, kernel_size, stride=None, padding=0):
    return pool(x, kernel_size, "mean", padding, stride)
