"""GPU tests of jt.grad on the meta-operator path: the gradients (themselves
built from reindex / reindex_reduce / reduce / broadcast / element-wise ops)
against closed-form numpy gradients in float64.  Cases follow the reference's
own gradient tests: pooling through reindex_reduce
(python/jittor/test/test_reindex_reduce_op.py:62-77), the meta-op convolution
(python/jittor/test/test_conv_tuner.py:105-133), reduce ops
(python/jittor/test/test_reduce_op.py)."""
import numpy as np
import pytest

import jittor_amd as jt
from oracle import oracle as O

pytestmark = pytest.mark.gpu


def close(a, b, rtol=1e-4, atol=1e-5):
    a = np.asarray(a, np.float64)
    b = np.asarray(b, np.float64)
    assert a.shape == b.shape, (a.shape, b.shape)
    err = np.abs(a - b).max() if a.size else 0.0
    assert np.allclose(a, b, rtol=rtol, atol=atol), "max abs err %g" % err


def sigmoid(x):
    return 1.0 / (1.0 + np.exp(-x))


def test_grad_fused_chain(gpu):
    rng = np.random.default_rng(0)
    x = rng.standard_normal((4, 8, 16)).astype(np.float32)
    s = rng.standard_normal((8, 1)).astype(np.float32)
    b = rng.standard_normal((1, 16)).astype(np.float32)
    w = rng.standard_normal((4, 8, 16)).astype(np.float32)
    vx, vs, vb = jt.array(x), jt.array(s), jt.array(b)
    f = jt.nn.relu(vx * vs + vb)
    out = (-f).exp() * vx.sigmoid()
    loss = (out * jt.array(w)).sum()
    gx, gs, gb = jt.grad(loss, [vx, vs, vb])
    X, S, B, W = (a.astype(np.float64) for a in (x, s, b, w))
    u = X * S + B
    e = np.exp(-np.maximum(u, 0))
    sg = sigmoid(X)
    du = W * e * sg * -1.0 * (u > 0)
    close(gx.numpy(), du * S + W * e * sg * (1 - sg))
    close(gs.numpy(), (du * X).sum(axis=(0, 2)).reshape(8, 1))
    close(gb.numpy(), du.sum(axis=(0, 1)).reshape(1, 16))


@pytest.mark.parametrize("op", ["exp", "log", "sqrt", "sin", "cos", "tan", "tanh", "sinh", "cosh", "asin", "acos", "atan",
                                "asinh", "acosh", "atanh", "sigmoid", "erf", "erfinv", "abs", "negative"])
def test_grad_unary(gpu, op):
    rng = np.random.default_rng(1)
    lo, hi = {"log": (0.5, 3), "sqrt": (0.5, 3), "acosh": (1.5, 3), "asin": (-0.8, 0.8), "acos": (-0.8, 0.8),
              "atanh": (-0.8, 0.8), "erfinv": (-0.8, 0.8), "tan": (-1, 1)}.get(op, (-2, 2))
    x = rng.uniform(lo, hi, 257).astype(np.float32)
    x[np.abs(x) < 0.05] = 0.5
    v = jt.array(x)
    g = jt.grad(v.unary(op).sum(), v).numpy()
    X = x.astype(np.float64)
    from scipy import special
    with np.errstate(all="ignore"):
        ref = _unary_refs(X, special)[op]
    close(g, ref, rtol=2e-4)


def _unary_refs(X, special):
    return {"exp": np.exp(X), "log": 1 / X, "sqrt": 0.5 / np.sqrt(X), "sin": np.cos(X), "cos": -np.sin(X), "tan": 1 / np.cos(X) ** 2,
           "tanh": 1 / np.cosh(X) ** 2, "sinh": np.cosh(X), "cosh": np.sinh(X), "asin": 1 / np.sqrt(1 - X * X),
           "acos": -1 / np.sqrt(1 - X * X), "atan": 1 / (1 + X * X), "asinh": 1 / np.sqrt(X * X + 1),
           "acosh": 1 / np.sqrt(np.maximum(X * X - 1, 1e-30)), "atanh": 1 / (1 - X * X), "sigmoid": sigmoid(X) * (1 - sigmoid(X)),
           "erf": 2 / np.sqrt(np.pi) * np.exp(-X * X), "erfinv": np.sqrt(np.pi) / 2 * np.exp(special.erfinv(X) ** 2),
           "abs": np.sign(X), "negative": -np.ones_like(X)}


def test_grad_binary(gpu):
    rng = np.random.default_rng(2)
    a = rng.uniform(0.5, 2, (5, 7)).astype(np.float32)
    b = rng.uniform(0.5, 2, (5, 7)).astype(np.float32)
    A, B = a.astype(np.float64), b.astype(np.float64)
    cases = {"add": (1 + 0 * A, 1 + 0 * B), "subtract": (1 + 0 * A, -1 + 0 * B), "multiply": (B, A), "divide": (1 / B, -A / B ** 2),
             "pow": (B * A ** (B - 1), A ** B * np.log(A)), "maximum": ((A > B) * 1.0, (B >= A) * 1.0),
             "minimum": ((A < B) * 1.0, (B <= A) * 1.0)}
    for op, (ga, gb) in cases.items():
        va, vb = jt.array(a), jt.array(b)
        da, db = jt.grad(jt.binary(va, vb, op).sum(), [va, vb])
        close(da.numpy(), ga, rtol=2e-4)
        close(db.numpy(), gb, rtol=2e-4)
    # a var used twice accumulates both contributions; an untouched target gets zeros
    va, vb = jt.array(a), jt.array(b)
    da, db = jt.grad((va * va + va).sum(), [va, vb])
    close(da.numpy(), 2 * A + 1)
    assert not db.numpy().any()


def test_grad_reduce_and_broadcast(gpu):
    rng = np.random.default_rng(3)
    x = rng.standard_normal((6, 5, 4)).astype(np.float32)
    X = x.astype(np.float64)
    w1 = rng.standard_normal((6, 4)).astype(np.float32)
    v = jt.array(x)
    close(jt.grad((v.sum(1) * jt.array(w1)).sum(), v).numpy(), np.repeat(w1[:, None, :], 5, 1))
    close(jt.grad((v.mean(1) * jt.array(w1)).sum(), v).numpy(), np.repeat(w1[:, None, :], 5, 1) / 5)
    g = jt.grad((v.max(1) * jt.array(w1)).sum(), v).numpy()
    ref = (X == X.max(1, keepdims=True)) * w1[:, None, :]
    close(g, ref)
    g = jt.grad((v.min([0, 2], keepdims=True)).sum(), v).numpy()
    close(g, (X == X.min(axis=(0, 2), keepdims=True)) * 1.0)
    g = jt.grad(v.prod(2).sum(), v).numpy()
    close(g, X.prod(2, keepdims=True) / X, rtol=1e-3)
    # broadcast: the gradient sums over the broadcast axes
    s = rng.standard_normal((5, 1)).astype(np.float32)
    vs = jt.array(s)
    close(jt.grad((vs.broadcast([6, 5, 4]) * v).sum(), vs).numpy(), X.sum(axis=(0, 2)).reshape(5, 1))


def test_grad_pool_reindex_reduce(gpu):
    """max / add pooling written with reindex_reduce and with reindex + reduce
    (test_reindex_reduce_op.py:13-77)."""
    rng = np.random.default_rng(4)
    N, C, H, W, k = 2, 3, 8, 8, 2
    x = rng.standard_normal((N, C, H, W)).astype(np.float32)
    r = rng.standard_normal((N, C, H // k, W // k)).astype(np.float32)
    X = x.astype(np.float64)
    blocks = X.reshape(N, C, H // k, k, W // k, k)
    up = lambda a: np.repeat(np.repeat(a, k, 2), k, 3)
    for op, ref in (("add", up(r)), ("maximum", (X == up(blocks.max(axis=(3, 5)))) * up(r)),
                    ("minimum", (X == up(blocks.min(axis=(3, 5)))) * up(r))):
        v = jt.array(x)
        y = v.reindex_reduce(op, [N, C, H // k, W // k], ["i0", "i1", "i2/%d" % k, "i3/%d" % k])
        close(jt.grad((y * jt.array(r)).sum(), v).numpy(), ref)
        v = jt.array(x)
        xx = v.reindex([N, C, H // k, W // k, k, k], ["i0", "i1", "i2*%d+i4" % k, "i3*%d+i5" % k])
        y = xx.reduce(op, [4, 5])
        close(jt.grad((y * jt.array(r)).sum(), v).numpy(), ref)


def test_grad_gather_with_extras(gpu):
    rng = np.random.default_rng(5)
    x = rng.standard_normal(50).astype(np.float32)
    idx = rng.integers(0, 50, 300).astype(np.int32)
    r = rng.standard_normal(300).astype(np.float32)
    v = jt.array(x)
    y = v.reindex([300], ["@e0(i0)"], extras=[jt.array(idx)])
    g = jt.grad((y * jt.array(r)).sum(), v).numpy()
    close(g, np.bincount(idx, weights=r.astype(np.float64), minlength=50))
    # scatter-add forward: the gradient gathers
    vals = rng.standard_normal(300).astype(np.float32)
    vv = jt.array(vals)
    h = vv.reindex_reduce("add", [50], ["@e0(i0)"], extras=[jt.array(idx)])
    g = jt.grad((h * jt.array(x)).sum(), vv).numpy()
    close(g, x.astype(np.float64)[idx])


def _conv_grads_ref(x, w, r, stride, pad, dil):
    N, C, H, W = x.shape
    K, _, R, S = w.shape
    OH, OW = r.shape[2], r.shape[3]
    X = np.pad(x.astype(np.float64), ((0, 0), (0, 0), (pad, pad), (pad, pad)))
    Wt, Rr = w.astype(np.float64), r.astype(np.float64)
    dX, dW = np.zeros_like(X), np.zeros_like(Wt)
    for kh in range(R):
        for kw in range(S):
            sl = (slice(None), slice(None), slice(kh * dil, kh * dil + (OH - 1) * stride + 1, stride),
                  slice(kw * dil, kw * dil + (OW - 1) * stride + 1, stride))
            dW[:, :, kh, kw] = np.einsum("nkhw,nchw->kc", Rr, X[sl])
            dX[sl] += np.einsum("nkhw,kc->nchw", Rr, Wt[:, :, kh, kw])
    return dX[:, :, pad:pad + H, pad:pad + W], dW


@pytest.mark.parametrize("case", [
    dict(x=(2, 3, 6, 6), w=(4, 3, 3, 3), stride=1, pad=1, dil=1, units=3),
    dict(x=(3, 8, 12, 10), w=(6, 8, 3, 3), stride=1, pad=2, dil=2, units=3),
    dict(x=(2, 4, 9, 9), w=(5, 4, 3, 3), stride=1, pad=0, dil=1, units=3),
    dict(x=(2, 4, 11, 11), w=(5, 4, 3, 3), stride=2, pad=1, dil=1, units=3),     # strided: input gradient over zero-spaced dy
    dict(x=(2, 4, 12, 10), w=(5, 4, 3, 3), stride=2, pad=1, dil=1, units=3),     # ... rows and columns the stride never reaches
    dict(x=(1, 3, 13, 13), w=(2, 3, 3, 3), stride=3, pad=0, dil=2, units=3),     # stride 3, dilation 2
    dict(x=(2, 6, 8, 8), w=(4, 6, 1, 1), stride=1, pad=0, dil=1, units=3),
])
def test_grad_meta_conv(gpu, case):
    """Gradients of the meta-op convolution (nn.py:1245-1262) with respect to input and weight against a
    direct float64 evaluation (test_conv_tuner.py:105-133 checks the same pair).  Forward, input gradient
    (stride 1) and weight gradient are each recognised and run as one convolution call, so the
    7-dimensional intermediates are never computed (the invariant of test_longest_dis_fuse.py:51-66)."""
    rng = np.random.default_rng(6)
    x = rng.standard_normal(case["x"]).astype(np.float32)
    w = rng.standard_normal(case["w"]).astype(np.float32)
    vx, vw = jt.array(x), jt.array(w)
    y = jt.nn.conv2d(vx, vw, stride=case["stride"], padding=case["pad"], dilation=case["dil"])
    r = rng.standard_normal(y.shape).astype(np.float32)
    gx, gw = jt.grad((y * jt.array(r)).sum(), [vx, vw])
    before = jt.executor_stats["conv_matches"]
    jt.sync([y, gx, gw])
    assert jt.executor_stats["conv_matches"] - before == case["units"]
    dX, dW = _conv_grads_ref(x, w, r, case["stride"], case["pad"], case["dil"])
    close(gx.numpy(), dX, rtol=1e-4, atol=1e-4)
    close(gw.numpy(), dW, rtol=1e-4, atol=1e-4)
    if case["units"] == 3:
        # nothing of rank 7 was materialised on the way
        seen, stack = set(), [gx, gw, y]
        while stack:
            v = stack.pop()
            if v.id in seen:
                continue
            seen.add(v.id)
            assert not (v.ndim == 7 and v._buf is not None)
            if v._history is not None:
                stack.extend(v._history[1])


@pytest.mark.parametrize("xs,ws,wgrad_kernel", [((2, 32, 16, 16), (64, 32, 3, 3), 0), ((2, 64, 16, 16), (64, 64, 3, 3), 1),
                                                    ((2, 128, 8, 16), (64, 128, 3, 3), 1), ((2, 64, 28, 28), (64, 64, 3, 3), 1)])
def test_grad_meta_conv_bfloat16(gpu, xs, ws, wgrad_kernel):
    """The same three units for bfloat16 operands (conv2d builds them under amp_reg | 36, so the sums keep
    16 bit without casts): the MFMA kernel runs forward and input gradient; the weight gradient runs on its
    own MFMA kernel where that applies (64 input channels: half a block of its workgroup; 128: a whole one; 28 columns: rows
    whose last piece is shared with the next row) and as
    a batched GEMM over shifted input planes otherwise (first case: 32 input channels); gradients keep the dtype of
    their variable."""
    rng = np.random.default_rng(8)
    x = rng.standard_normal(xs).astype(np.float32)
    w = (rng.standard_normal(ws) * 0.05).astype(np.float32)
    vx, vw = jt.array(x).bfloat16(), jt.array(w).bfloat16()
    jt.sync([vx, vw])
    xb = O.BF16(vx.raw()).to_f32()
    wb = O.BF16(vw.raw()).to_f32()
    y = jt.nn.conv2d(vx, vw, padding=1)
    r = (rng.integers(-2, 3, y.shape) * 0.5).astype(np.float32)            # exact in bfloat16
    gx, gw = jt.grad((y * jt.array(r).bfloat16()).sum(), [vx, vw])
    assert gx.dtype == "bfloat16" and gw.dtype == "bfloat16"
    before, before_k = jt.executor_stats["conv_matches"], jt.executor_stats["wgrad_kernel"]
    jt.sync([y, gx, gw])
    assert jt.executor_stats["conv_matches"] - before == 3
    assert jt.executor_stats["wgrad_kernel"] - before_k == wgrad_kernel
    dX, dW = _conv_grads_ref(xb, wb, r, 1, 1, 1)
    tol = 2.0 ** -7                                                         # results are rounded to bfloat16
    assert np.abs(gx.float32().numpy() - dX).max() <= tol * np.abs(dX).max()
    assert np.abs(gw.float32().numpy() - dW).max() <= tol * np.abs(dW).max()
    seen, stack = set(), [gx, gw, y]
    while stack:
        v = stack.pop()
        if v.id in seen:
            continue
        seen.add(v.id)
        assert not (v.ndim == 7 and v._buf is not None)
        if v._history is not None:
            stack.extend(v._history[1])


@pytest.mark.parametrize("xs,k,rs,stride,pad,dtype,chunked", [
    ((8, 32, 14, 14), 64, 3, 1, 1, "bfloat16", 1),      # 196-pixel planes: pairs of images make 16-byte multiples, four chunks
    ((16, 64, 7, 7), 96, 3, 1, 1, "float16", 1),        # 49 pixels: eight images per chunk
    ((64, 32, 7, 7), 64, 3, 1, 1, "bfloat16", 1),       # 64 images of 49 pixels: one chunk of 3136, the product is the result
    ((6, 32, 27, 27), 64, 3, 2, 1, "bfloat16", 1),      # stride 2 onto 14 x 14; three chunks
    ((8, 48, 13, 13), 40, 1, 1, 0, "bfloat16", 1),      # 1x1 taps on 169 pixels: all eight images in one chunk
    ((3, 32, 14, 14), 64, 3, 1, 1, "bfloat16", 0),      # three images never make a multiple of 8 elements: the product per image
])
def test_grad_conv_weight_16bit_maps_with_unaligned_planes(gpu, xs, k, rs, stride, pad, dtype, chunked):
    """Weight gradient of 16-bit convolutions on maps whose planes are no 16-byte multiples (14 x 14, 7 x 7, 13 x 13): one
    product over chunks of images laid side by side instead of one product per image on the kernel without MFMAs
    (executor.py, ConvBwdWeightUnit); against the float64 gradient of the exact 16-bit operands."""
    rng = np.random.default_rng(12)
    x = rng.standard_normal(xs).astype(np.float32)
    w = (rng.standard_normal((k, xs[1], rs, rs)) * 0.05).astype(np.float32)
    vx, vw = jt.array(x).cast(dtype), jt.array(w).cast(dtype)
    jt.sync([vx, vw])
    xe = vx.float32().numpy()
    we = vw.float32().numpy()
    y = jt.nn.conv2d(vx, vw, stride=stride, padding=pad)
    r = (rng.integers(-2, 3, y.shape) * 0.5).astype(np.float32)            # exact in both 16-bit types
    gw, = jt.grad((y * jt.array(r).cast(dtype)).sum(), [vw])
    assert gw.dtype == dtype
    before = jt.executor_stats["wgrad_chunked"]
    jt.sync([gw])
    assert jt.executor_stats["wgrad_chunked"] - before == chunked
    _, dW = _conv_grads_ref(xe, we, r, stride, pad, 1)
    tol = 2.0 ** -7 if dtype == "bfloat16" else 2.0 ** -10                 # results are rounded to the 16-bit type
    assert np.abs(gw.float32().numpy() - dW).max() <= tol * np.abs(dW).max()


def test_grad_stop_grad_and_no_grad(gpu):
    x = jt.array(np.arange(1, 7, dtype=np.float32))
    y = (x * 2).stop_grad()
    z = (y * x).sum()
    close(jt.grad(z, x).numpy(), 2 * np.arange(1, 7))          # only the direct use of x counts
    with jt.no_grad():
        q = x * x
    assert q._history is None
    assert not jt.grad(q.sum(), x).numpy().any()
    with pytest.raises(ValueError):
        jt.grad(jt.array([1, 2, 3]).sum(), x)


def test_grad_grouped_conv(gpu):
    """Gradients of the grouped convolution (nn.py:1272-1294): each group is an independent convolution, so the
    gradients of its channel slices are those of the plain convolution (float64 closed form per group)."""
    rng = np.random.default_rng(9)
    G, cg, kg = 3, 2, 2
    x = rng.standard_normal((2, G * cg, 7, 6)).astype(np.float32)
    w = rng.standard_normal((G * kg, cg, 3, 3)).astype(np.float32)
    vx, vw = jt.array(x), jt.array(w)
    y = jt.nn.conv2d(vx, vw, padding=1, groups=G)
    r = rng.standard_normal(y.shape).astype(np.float32)
    gx, gw = jt.grad((y * jt.array(r)).sum(), [vx, vw])
    jt.sync([gx, gw])
    for g in range(G):
        dX, dW = _conv_grads_ref(x[:, g * cg:(g + 1) * cg], w[g * kg:(g + 1) * kg], r[:, g * kg:(g + 1) * kg], 1, 1, 1)
        close(gx.numpy()[:, g * cg:(g + 1) * cg], dX, rtol=1e-4, atol=1e-4)
        close(gw.numpy()[g * kg:(g + 1) * kg], dW, rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("dtype,G,cg,kg,kw", [
    ("float32", 8, 1, 1, dict(padding=1)),                       # depthwise
    ("float32", 2, 3, 2, dict(stride=2, padding=1)),
    ("float32", 3, 2, 3, dict(padding=2, dilation=2)),
    ("bfloat16", 4, 2, 2, dict(padding=1)),
    ("float16", 2, 2, 3, dict(stride=(2, 1), padding=(0, 1))),
])
def test_grad_grouped_conv_runs_as_convolutions(gpu, dtype, G, cg, kg, kw):
    """Forward and both gradients of a grouped convolution are recognised over the 8-d product and run as
    convolution kernels (the weight gradient on the direct kernel, the input gradient as the grouped forward kernel
    on dy with the weights transposed per group and flipped); the 8-d tensors are never written.  Values against
    the plain execution of the same graph (which sums in the same float type but another order) and, for float32,
    the oracle's gradient graph."""
    rng = np.random.default_rng(14)
    x = rng.standard_normal((3, G * cg, 9, 8)).astype(np.float32)
    w = (rng.standard_normal((G * kg, cg, 3, 3)) * 0.3).astype(np.float32)
    results = {}
    for matched in (True, False):
        jt.flags["enable_conv_match"] = matched
        try:
            vx, vw = jt.array(x).cast(dtype), jt.array(w).cast(dtype)
            y = jt.nn.conv2d(vx, vw, groups=G, **kw)
            if "r" not in results:
                results["r"] = rng.standard_normal(y.shape).astype(np.float32)
            gx, gw = jt.grad((y * jt.array(results["r"]).cast(dtype)).sum(), [vx, vw])
            before = dict(jt.executor_stats)
            jt.sync([y, gx, gw])
            if matched:
                assert jt.executor_stats["conv_matches"] == before["conv_matches"] + 3
            results[matched] = [np.asarray(v.numpy(), dtype=np.float32) for v in (y, gx, gw)]
        finally:
            jt.flags["enable_conv_match"] = True
    # the plain path sums 16-bit products in 16 bits (bfloat16 truncates every partial sum: a few hundred terms lose
    # tens of percent), the kernels in float32: only float32 results are comparable between the two
    for a, b in zip(results[True], results[False]):
        assert a.shape == b.shape
        if dtype == "float32":
            assert np.abs(a - b).max() <= 1e-4 * np.abs(b).max()
    # against the oracle's gradient graph on the same (narrowed) operands: one rounding of a float32 sum
    def stored(a):
        return np.asarray(jt.array(a).cast(dtype).numpy(), dtype=np.float32)
    dx, dw = O.conv_meta_grouped_grads(stored(x), stored(w), stored(results["r"]), G, kw.get("stride", 1), kw.get("padding", 0),
                                       kw.get("dilation", 1))
    tol = {"float32": 1e-4, "float16": 2.0 ** -9, "bfloat16": 2.0 ** -7}[dtype]
    assert np.abs(results[True][1] - dx).max() <= tol * np.abs(dx).max()
    assert np.abs(results[True][2] - dw).max() <= tol * np.abs(dw).max()


def test_pooling_forward_and_backward_keep_rank_six_out_of_memory(gpu):
    """Pooling and its gradient run without the rank-6 window tensors ever being written (the invariant of
    test_longest_dis_fuse.py:51-66): forward = reindex fused with its reduce, backward = the element-wise group
    (equal / ternary over the window tensor, recomputed through the scatter's index program) fused into the
    scatter.  Values against the plain path and closed forms."""
    rng = np.random.default_rng(12)
    x = rng.standard_normal((2, 3, 9, 10)).astype(np.float32)
    for op in ("maximum", "mean"):
        results = {}
        for fused in (True, False):
            jt.flags["enable_gather_reduce"] = jt.flags["enable_scatter_fusion"] = fused
            try:
                vx = jt.array(x)
                y = jt.pool(vx, 3, op, 1, 2)
                r = jt.array(rng.standard_normal(y.shape).astype(np.float32)) if "r" not in results else results["r"]
                results["r"] = r
                g = jt.grad((y * r).sum(), vx)
                before = dict(jt.executor_stats)
                jt.sync([y, g])
                results[fused] = (y.numpy(), g.numpy())
                if fused:
                    assert jt.executor_stats["fused_scatters"] == before["fused_scatters"] + 1
                    seen, stack = set(), [y, g]
                    while stack:                                       # nothing of rank 6 has memory
                        v = stack.pop()
                        if v.id in seen:
                            continue
                        seen.add(v.id)
                        assert not (v.ndim == 6 and v._buf is not None)
                        if v._history is not None:
                            stack.extend(v._history[1])
            finally:
                jt.flags["enable_gather_reduce"] = jt.flags["enable_scatter_fusion"] = True
        close(results[True][0], results[False][0], rtol=1e-6, atol=1e-6)
        close(results[True][1], results[False][1], rtol=1e-5, atol=1e-6)
    # mean pooling without padding: every input element gets r / 9 from each window that covers it
    xs = rng.standard_normal((1, 2, 6, 6)).astype(np.float32)
    vx = jt.array(xs)
    g = jt.grad(jt.pool(vx, 3, "mean", 0, 3).sum(), vx)
    close(g.numpy(), np.full(xs.shape, 1.0 / 9, np.float32))


def test_small_cnn_step_with_and_without_the_executor_rewrites(gpu):
    """One training step of a small CNN (conv, relu, max pool, strided conv, global mean, linear, softmax
    cross-entropy): loss and all gradients with every executor rewrite on (convolution units, weight-gradient
    kernel, matrix products, reduce prologues, broadcast sinking, gather-reduce, scatter prologue) against the same
    graph run op by op through the generic kernels."""
    rng = np.random.default_rng(13)
    x = rng.standard_normal((4, 8, 12, 12)).astype(np.float32)
    w1 = (rng.standard_normal((16, 8, 3, 3)) * 0.2).astype(np.float32)
    w2 = (rng.standard_normal((16, 16, 3, 3)) * 0.2).astype(np.float32)
    wl, bl = (rng.standard_normal((5, 16)) * 0.3).astype(np.float32), rng.standard_normal(5).astype(np.float32)
    onehot = np.eye(5, dtype=np.float32)[rng.integers(0, 5, 4)]
    names = ["enable_conv_match", "enable_reduce_fusion", "enable_broadcast_sink", "enable_matmul_match", "enable_conv_wgrad_kernel",
             "enable_gather_reduce", "enable_scatter_fusion"]

    def step():
        vx, v1, v2, vl, vb = (jt.array(a) for a in (x, w1, w2, wl, bl))
        h = jt.nn.relu(jt.nn.conv2d(vx, v1, padding=1))
        h = jt.nn.max_pool2d(h, 3, 2, 1)
        h = jt.nn.relu(jt.nn.conv2d(h, v2, stride=2, padding=1))
        f = h.mean([2, 3])
        logits = jt.nn.linear(f, vl, vb)
        m = logits.max([1], keepdims=True)
        e = jt.unary(logits - m, "exp")
        logp = logits - m - jt.unary(e.sum([1], keepdims=True), "log")
        loss = (logp * jt.array(onehot)).sum() * (-1.0 / 4)
        grads = jt.grad(loss, [vx, v1, v2, vl, vb])
        jt.sync([loss] + grads)
        return [loss.numpy()] + [g.numpy() for g in grads]

    fast = step()
    saved = {n: jt.flags[n] for n in names}
    try:
        for n in names:
            jt.flags[n] = False
        plain = step()
    finally:
        for n, v in saved.items():
            jt.flags[n] = v
    for a, b in zip(fast, plain):
        assert a.shape == b.shape
        close(a, b, rtol=2e-4, atol=2e-5)
    assert np.isfinite(fast[0]).all() and float(fast[0][0]) > 0
