"""Callers that define the patterns of the path: relu and conv2d expressed
with meta-operators exactly as the reference writes them
(python/jittor/nn.py:166-183 and :1245-1269)."""
import numpy as np

from . import core
from .flags import flags, flag_scope


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
    (C, Kh, Kw) (python/jittor/nn.py:1245-1269, groups == 1), or with groups > 1
    reindex(x) * reindex(w) -> reindex_reduce.add over an 8-d product
    (python/jittor/nn.py:1272-1294).  The executor recognises either group of ops
    and runs it as one kernel."""
    padding, stride, dilation = _pair(padding), _pair(stride), _pair(dilation)
    N, C, H, W = x.shape
    K = weight.shape[0]
    Kh, Kw = weight.shape[-2:]
    oh = (H + padding[0] * 2 - Kh * dilation[0] + dilation[0] - 1) // stride[0] + 1
    ow = (W + padding[1] * 2 - Kw * dilation[1] + dilation[1] - 1) // stride[1] + 1
    if groups != 1:
        G, CpG = groups, C // groups
        if groups < 1 or C % G or K % G or weight.shape[1] != CpG:
            raise ValueError("conv2d: %d input and %d output channels with weight %s do not form %d groups"
                             % (C, K, list(weight.shape), groups))
        oc = K
        xx = x.reindex([N, G, oc // G, CpG, oh, ow, Kh, Kw], [
            "i0",
            "i1*%d+i3" % CpG,
            "i4*%d-%d+i6*%d" % (stride[0], padding[0], dilation[0]),
            "i5*%d-%d+i7*%d" % (stride[1], padding[1], dilation[1]),
        ])
        xx.compile_options = {"G": G}                      # nn.py:1278
        ww = weight.reindex([N, G, oc // G, CpG, oh, ow, Kh, Kw], ["i1*%d+i2" % (oc // G), "i3", "i6", "i7"])
        yy = xx * ww
        y = yy.reindex_reduce("add", [N, oc, oh, ow], ["i0", "i1*%d+i2" % (oc // G), "i4", "i5"])
        if bias is not None:
            y = y + bias.broadcast(y.shape, [0, 2, 3])
        return y
    # 16-bit operands: the sum keeps their type and is not routed through float32 casts (amp_reg | 36, nn.py:1250)
    with flag_scope(amp_reg=flags.amp_reg | 36):
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


def conv_transpose(x, weight, bias=None, stride=1, padding=0, output_padding=0, groups=1, dilation=1):
    """The transposed convolution as python/jittor/nn.py:1535-1577 writes it (groups == 1): x [N, i, H, W] and
    weight [i, o, h, w] broadcast into [N, i, o, H, W, h, w], multiplied, and scattered with reindex_reduce.add
    into [N, o, h_out, w_out].  That graph is the input gradient of the convolution whose output x would be
    (conv_tuner.cc:375-397 relays it to the library's backward-data call); the executor recognises it the same
    way and runs it on the convolution kernels."""
    if groups != 1:
        raise NotImplementedError("conv_transpose: groups > 1")
    if x.ndim != 4:
        raise RuntimeError("Expected 4D input to conv_transpose, but got input of size: %s" % list(x.shape))
    stride, padding, dilation, output_padding = _pair(stride), _pair(padding), _pair(dilation), _pair(output_padding)
    N, C, H, W = x.shape
    i, o, h, w = weight.shape
    assert C == i, (C, i)
    if stride[0] <= 0 or stride[1] <= 0:
        raise RuntimeError("non-positive stride is not supported")
    assert output_padding[0] < max(stride[0], dilation[0]) and output_padding[1] < max(stride[1], dilation[1]), \
        "output padding must be smaller than max(stride, dilation)"
    h_out = (H - 1) * stride[0] + output_padding[0] - 2 * padding[0] + 1 + (h - 1) * dilation[0]
    w_out = (W - 1) * stride[1] + output_padding[1] - 2 * padding[1] + 1 + (w - 1) * dilation[1]
    shape = [N, i, o, H, W, h, w]
    with flag_scope(amp_reg=flags.amp_reg | 36):
        xx = x.broadcast(shape, [2, 5, 6])
        ww = weight.broadcast(shape, [0, 3, 4])
        y = (ww * xx).reindex_reduce("add", [N, o, h_out, w_out], [
            "i0",
            "i2",
            "i3*%d-%d+i5*%d" % (stride[0], padding[0], dilation[0]),
            "i4*%d-%d+i6*%d" % (stride[1], padding[1], dilation[1]),
        ])
    if bias is not None:
        y = y + bias.broadcast(y.shape, [0, 2, 3])
    return y


conv_transpose2d = conv_transpose


def unfold(x, kernel_size, dilation=1, padding=0, stride=1):
    """Sliding windows as columns, [n, c, h, w] -> [n, c * kh * kw, blocks] (python/jittor/nn.py:2450-2477): a
    padding reindex, then one reindex whose index expressions divide and take remainders."""
    assert x.ndim == 4
    kernel_size, dilation, padding, stride = _pair(kernel_size), _pair(dilation), _pair(padding), _pair(stride)
    assert kernel_size[0] > 0 and kernel_size[1] > 0, "kernel size must be positive"
    assert dilation[0] > 0 and dilation[1] > 0, "dilation must be positive"
    assert padding[0] >= 0 and padding[1] >= 0, "padding must be non-negative"
    assert stride[0] > 0 and stride[1] > 0, "stride must be positive"
    n, c, h, w = x.shape
    area = kernel_size[0] * kernel_size[1]
    blocks = [(x.shape[i] + 2 * padding[i - 2] - dilation[i - 2] * (kernel_size[i - 2] - 1) - 1) // stride[i - 2] + 1 for i in (2, 3)]
    if padding[0] != 0 or padding[1] != 0:
        x = x.reindex([n, c, h + padding[0] * 2, w + padding[1] * 2], ["i0", "i1", "i2-%d" % padding[0], "i3-%d" % padding[1]])
    return x.reindex([n, c * area, blocks[0] * blocks[1]], [
        "i0", "i1/%d" % area,
        "i2/%d*%d+(i1%%%d)/%d*%d" % (blocks[1], stride[0], area, kernel_size[1], dilation[0]),
        "i2%%%d*%d+(i1%%%d)%%%d*%d" % (blocks[1], stride[1], area, kernel_size[1], dilation[1])])


def fold(x, output_size, kernel_size, dilation=1, padding=0, stride=1):
    """Columns summed back into an image, [n, c * kh * kw, blocks] -> [n, c, H, W] (python/jittor/nn.py:2480-2501):
    one reindex_reduce.add with unfold's index expressions, then the crop of the padding."""
    assert x.ndim == 3
    assert output_size[0] > 0 and output_size[1] > 0, "output size must be positive."
    kernel_size, dilation, padding, stride = _pair(kernel_size), _pair(dilation), _pair(padding), _pair(stride)
    assert kernel_size[0] > 0 and kernel_size[1] > 0, "kernel size must be positive"
    assert dilation[0] > 0 and dilation[1] > 0, "dilation must be positive"
    assert padding[0] >= 0 and padding[1] >= 0, "padding must be non-negative"
    assert stride[0] > 0 and stride[1] > 0, "stride must be positive"
    n, cl, num = x.shape
    area = kernel_size[0] * kernel_size[1]
    blocks = [(output_size[i] + 2 * padding[i] - dilation[i] * (kernel_size[i] - 1) - 1) // stride[i] + 1 for i in (0, 1)]
    out = x.reindex_reduce("add", [n, cl // area, output_size[0] + 2 * padding[0], output_size[1] + 2 * padding[1]], [
        "i0", "i1/%d" % area,
        "i2/%d*%d+(i1%%%d)/%d*%d" % (blocks[1], stride[0], area, kernel_size[1], dilation[0]),
        "i2%%%d*%d+(i1%%%d)%%%d*%d" % (blocks[1], stride[1], area, kernel_size[1], dilation[1])])
    return out[:, :, padding[0]:padding[0] + output_size[0], padding[1]:padding[1] + output_size[1]]


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


def matmul_transpose(a, b):
    """a * b^T as broadcast, multiply, sum (python/jittor/nn.py:28-43); the executor recognises the group as
    a matrix product (opt/tuner/matmul_tuner.cc:16-104)."""
    a, b = core._as_var(a), core._as_var(b)
    assert a.shape[-1] == b.shape[-1], (a.shape, b.shape)
    if a.ndim != 2:
        from . import misc
        aa = misc.reshape(a, [-1, a.shape[-1]])
        cc = matmul_transpose(aa, b)
        return misc.reshape(cc, list(a.shape[:-1]) + [-1])
    assert a.ndim == 2 and b.ndim == 2
    shape = list(a.shape)[:-1] + list(b.shape)
    a = core.broadcast(a, shape, [len(shape) - 2])
    b = core.broadcast(b, shape)
    return core.reduce(core.binary(a, b, "multiply"), "add", [len(shape) - 1])


def matmul(a, b):
    """Matrix product with the reference's shape rules (python/jittor/nn.py:83-159): vectors, matrices and
    leading batch dimensions that broadcast, all through broadcast, multiply and sum."""
    from . import misc
    a, b = core._as_var(a), core._as_var(b)
    len_a, len_b = a.ndim, b.ndim
    if len_b == 1:
        return core.reduce(core.binary(a, b, "multiply"), "add", [-1])           # a: [n, m], b: [m] -> [n]
    if len_a == 1:
        return core.reduce(core.binary(core.broadcast_var(a, b, [-1]), b, "multiply"), "add", [0])   # [n] x [n, k] -> [k]
    len_c = max(len_a, len_b)
    (n, m), (m_, k) = a.shape[-2:], b.shape[-2:]
    assert m == m_, "dimension not match, a.shape:%s, b.shape:%s" % (a.shape, b.shape)
    if len_b == 2 and len_a > 2:
        cc = matmul(misc.reshape(a, [-1, m]), b)
        return misc.reshape(cc, list(a.shape[:-1]) + [k])
    # the leading axes broadcast against each other like any element-wise pair
    try:
        shape = list(np.broadcast_shapes(tuple(a.shape[:-2]), tuple(b.shape[:-2]))) + [n, m, k]
    except ValueError:
        raise AssertionError("dimension not match, a.shape:%s, b.shape:%s" % (a.shape, b.shape))
    a = core.broadcast(a, shape, [-1])
    b = core.broadcast(b, shape, [-3])
    return core.reduce(core.binary(a, b, "multiply"), "add", [-2])


def bmm(a, b):
    """[batch, n, m] x [batch, m, k] (python/jittor/nn.py:57-80)."""
    assert a.ndim >= 3 and a.ndim == b.ndim
    return matmul(a, b)


def linear(x, weight, bias=None):
    """x * weight^T + bias (python/jittor/nn.py: linear)."""
    y = matmul_transpose(x, weight)
    return y if bias is None else core.binary(y, bias, "add")


core.Var.matmul = core.Var.__matmul__ = matmul
