"""Pins the CPU oracle (oracle/oracle.py) against the known-answer vectors the
reference's tests hold, numpy/scipy closed forms and brute-force loops, chosen
so that a wrong sign, index or operand order fails one of them.  No GPU."""
import json
import os

import numpy as np
import pytest
from scipy import special

from oracle import oracle as O

G = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "vectors.json")))
rng = np.random.default_rng(1234)


# ---- golden vectors of the reference ---------------------------------------------
def test_golden_reindex_shift():
    g = G["reindex_shift"]
    y = O.reindex(np.array(g["x"], np.int32), g["shape"], g["indexes"], g["overflow_value"])
    assert y.tolist() == g["y"]


def test_golden_pad_with_overflow_value():
    # test/test_reindex_op.py:181-190: b = a.reindex([size+l+r], ["i0-l"], -1)
    size, l, r = 10, 3, 4
    a = rng.random(size).astype(np.float32)
    b = O.reindex(a, [size + l + r], ["i0-%d" % l], -1)
    assert (b[l:l + size] == a).all() and (b[:l] == -1).all() and (b[-r:] == -1).all()


def test_golden_reduce_and_broadcast():
    g = G["reduce_negative_dim"]
    x = np.array(g["x"], np.int32)
    assert O.reduce(x, "add", -1).tolist() == g["sum_m1"]
    assert O.reduce(x, "add", -2).tolist() == g["sum_m2"]
    g = G["broadcast_dims"]
    x = np.array(g["x"], np.int32)
    assert O.broadcast_to(x, g["shape"], [-1]).tolist() == g["dims_m1"]
    assert O.broadcast_to(x, g["shape"], [-2]).tolist() == g["dims_m2"]
    g = G["add_scalar"]
    assert O.binary(np.array(g["x"], np.int32), np.array([1], np.int32), "add", yscalar=True).tolist() == g["plus1"]


def test_golden_gather_scatter_tables():
    g = G["gather"]
    t, idx = np.array(g["t"], np.int32), np.array(g["index"], np.int32)
    assert O.reindex(t, idx.shape, ["i0", "@e0(i0,i1)"], extras=[idx]).tolist() == g["dim1"]
    assert O.reindex(t, idx.shape, ["@e0(i0,i1)", "i1"], extras=[idx]).tolist() == g["dim0"]
    g = G["scatter_void"]
    src = np.array(g["src"], np.int32)
    i0 = np.array(g["index0"], np.int32)
    out = O.reindex_reduce(src[:1, :4], "void", [3, 5], ["@e0(i0,i1)", "i1"], extras=[i0])
    assert out.tolist() == g["out0"]
    i1 = np.array(g["index1"], np.int32)
    out = O.reindex_reduce(src[:2, :3], "void", [3, 5], ["i0", "@e0(i0,i1)"], extras=[i1])
    assert out.tolist() == g["out1"]


def test_golden_dtype_table():
    for op, x, y, xs, ys, want in G["dtype_table"]["rows"]:
        assert O.binary_dtype_infer(op, x, y, xs, ys) == want
    # test/test_bf16.py:280: ternary(int cond, bf16, float32 scalar) -> bfloat16
    assert O.dtype_infer("bfloat16", "float32", False, True) == "bfloat16"
    # test/test_bf16.py:250-255: a**a on bfloat16 is float32 (white list)
    assert O.binary_dtype_infer("pow", "bfloat16", "bfloat16") == "float32"
    assert O.reduce_dtype_infer("add", "bfloat16") == "float32"
    assert O.unary_dtype_infer("sqrt", "int32") == "float32"
    assert O.unary_dtype_infer("exp", "float16") == "float32"
    assert O.binary_dtype_infer("divide", "int32", "int32") == "float32"
    assert O.binary_dtype_infer("floor_divide", "int32", "int32") == "int32"
    assert O.binary_dtype_infer("less", "float32", "float32") == "bool"
    assert O.reduce_dtype_infer("add", "bool") == "int32"


def test_golden_bool_reduce():
    g = G["bool_reduce"]
    a, b = np.array(g["a"], bool), np.array(g["b"], bool)
    assert bool(O.reduce(O.binary(a, b, "bitwise_or"), "logical_and")[0]) is g["or_all"]
    assert bool(O.reduce(O.binary(a, b, "bitwise_and"), "logical_or")[0]) is g["and_any"]


# ---- reindex: closed forms and brute force ----------------------------------------
def test_reindex_im2col_closed_form():
    x = rng.standard_normal((2, 3, 7, 6)).astype(np.float32)
    y = O.reindex(x, [2, 3, 7, 6, 3, 3], ["i0", "i1", "i2+i4-1", "i3+i5-1"], 0)
    ref = np.lib.stride_tricks.sliding_window_view(np.pad(x, ((0, 0), (0, 0), (1, 1), (1, 1))), (3, 3), axis=(2, 3))
    assert np.array_equal(y, ref)


def test_reindex_matmul_identity():
    # test/test_reindex_op.py:192-204: two reindexes, multiply, sum == np.matmul
    n = 6
    a, b = rng.random((n, n)).astype(np.float32), rng.random((n, n)).astype(np.float32)
    cc = O.binary(O.reindex(a, [n, n, n], ["i0", "i1"]), O.reindex(b, [n, n, n], ["i1", "i2"]), "multiply")
    c = O.reduce(cc, "add", 1)
    assert np.allclose(c, a @ b)


def test_reindex_brute_force_with_conditions():
    # transposed-convolution indices with C truncating division and overflow conditions
    x = rng.random((2, 4, 4, 2)).astype(np.float32)
    shape = [2, 10, 10, 3, 3, 2]
    idx = ["i0", "(i1-i3)/2", "(i2-i4)/2", "i5"]
    ofc = ["(i1-i3)%2", "(i2-i4)%2"]
    y = O.reindex(x, shape, idx, 0, ofc)
    ref = np.zeros(shape, np.float32)
    for c in np.ndindex(*shape):
        i0, i1, i2, i3, i4, i5 = c
        h, w = int((i1 - i3) / 2), int((i2 - i4) / 2)     # C division truncates toward zero
        if (i1 - i3) % 2 or (i2 - i4) % 2:
            continue
        if 0 <= h < 4 and 0 <= w < 4:
            ref[c] = x[i0, h, w, i5]
    assert np.array_equal(y, ref)


def test_reindex_nested_extras():
    # test/test_reindex_op.py:297-303 shape of expression: "@e0(0)", "@e1(0,i0 / @e0(0))"
    a = rng.random((10, 10)).astype(np.float32)
    b = np.array([2], np.int32)
    e1 = rng.integers(0, 10, (10, 10)).astype(np.float32)
    y = O.reindex(a, [8, 8], ["@e0(0)", "@e1(0,i0 / @e0(0))"], extras=[b, e1])
    ref = np.zeros((8, 8), np.float32)
    for i0 in range(8):
        for i1 in range(8):
            ref[i0, i1] = a[2, int(e1[0, i0 // 2])]
    assert np.array_equal(y, ref)


def test_reindex_errors():
    a = np.zeros((10, 10), np.float32)
    with pytest.raises(ValueError):
        O.reindex(a, [8, 8], ["@e0(0) // 1", "@e0(0)"], extras=[np.array([1]), np.array([1])])
    with pytest.raises(ValueError):
        O.reindex(a, [8, 8], ["i0"])


# ---- reindex_reduce ------------------------------------------------------------------
@pytest.mark.parametrize("op", ["maximum", "minimum", "multiply", "add"])
def test_reindex_reduce_pooling_brute_force(op):
    N, H, W, C, size = 2, 7, 7, 3, 3
    x = rng.random((N, H, W, C)).astype(np.float32)
    h, w = (H + size - 1) // size, (W + size - 1) // size
    y = O.reindex_reduce(x, op, [N, h, w, C], ["i0", "i1/%d" % size, "i2/%d" % size, "i3"])
    init = {"maximum": -1e100, "minimum": 1e100, "multiply": 1.0, "add": 0.0}[op]
    f = {"maximum": max, "minimum": min, "multiply": lambda a, b: a * b, "add": lambda a, b: a + b}[op]
    ref = np.full((N, h, w, C), init)
    for i0, i1, i2, i3 in np.ndindex(N, H, W, C):
        ref[i0, i1 // size, i2 // size, i3] = f(ref[i0, i1 // size, i2 // size, i3], float(x[i0, i1, i2, i3]))
    assert np.allclose(y, ref)


def test_reindex_reduce_histogram_closed_forms():
    n, bins = 5000, 37
    v = rng.random(n).astype(np.float32)
    idx = rng.integers(0, bins + 5, n).astype(np.int32) - 2      # some out of range on both sides
    ok = (idx >= 0) & (idx < bins)
    add = O.reindex_reduce(v, "add", [bins], ["@e0(i0)"], extras=[idx])
    assert np.allclose(add, np.bincount(idx[ok], weights=v[ok].astype(np.float64), minlength=bins), rtol=1e-5)
    mx = O.reindex_reduce(v, "maximum", [bins + 8], ["@e0(i0)"], extras=[idx])
    ok8 = (idx >= 0) & (idx < bins + 8)
    ref = np.full(bins + 8, np.finfo(np.float32).min, np.float32)
    np.maximum.at(ref, idx[ok8], v[ok8])
    assert np.array_equal(mx, ref)
    assert (mx[bins + 3:] == np.finfo(np.float32).min).all()      # empty bins keep lowest(), not -inf
    # invariants: total mass, permutation invariance (integers: exact)
    vi = rng.integers(0, 100, n).astype(np.int32)
    a1 = O.reindex_reduce(vi, "add", [bins], ["@e0(i0)"], extras=[idx])
    p = rng.permutation(n)
    a2 = O.reindex_reduce(vi[p], "add", [bins], ["@e0(i0)"], extras=[idx[p]])
    assert np.array_equal(a1, a2) and a1.sum() == vi[ok].sum()


def test_reindex_reduce_errors():
    v = np.zeros(3, np.float32)
    O.reindex_reduce(v, "add", [3], ["i0"])
    for bad in (lambda: O.reindex_reduce(v, "add", [3], []),
                lambda: O.reindex_reduce(v, "add", [3], ["i0", "i0"]),
                lambda: O.reindex_reduce(v, "???", [3], ["i0"]),
                lambda: O.reindex_reduce(v, "add", [-1], ["i0"])):
        with pytest.raises(ValueError):
            bad()


# ---- reduce ---------------------------------------------------------------------------
@pytest.mark.parametrize("keepdims", [False, True])
def test_reduce_integer_exact(keepdims):
    # test/test_reduce_op.py:12-50: arange data, 10 ops x 10 dim sets, exact
    a = np.arange(2 * 3 * 4 * 5).reshape(2, 3, 4, 5).astype(np.int32)
    ops = {"add": np.add, "multiply": np.multiply, "maximum": np.maximum, "minimum": np.minimum,
           "logical_and": np.logical_and, "logical_or": np.logical_or, "logical_xor": np.logical_xor,
           "bitwise_and": np.bitwise_and, "bitwise_or": np.bitwise_or, "bitwise_xor": np.bitwise_xor}
    for dims in [(), (0,), (1,), (2,), (3,), (0, 2), (1, 3), (1, 2, 3), 2, 3]:
        nd = tuple(range(4)) if dims == () else dims
        for name, uf in ops.items():
            ref = uf.reduce(a, nd, keepdims=keepdims)
            ref = np.array([ref]) if ref.ndim == 0 else ref
            got = O.reduce(a, name, dims, keepdims)
            assert got.shape == ref.shape and (got == ref.astype(np.int32)).all(), (name, dims)


def test_reduce_float_and_mean():
    x = rng.uniform(-1, 1, (64, 33, 5)).astype(np.float32)
    for dims in [(1,), (0, 2), ()]:
        nd = tuple(range(3)) if dims == () else dims
        ref = x.astype(np.float64).sum(nd)
        assert np.allclose(O.reduce(x, "add", dims).reshape(-1), np.reshape(ref, -1), rtol=1e-5, atol=1e-4)
        refm = x.astype(np.float64).mean(nd)
        assert np.allclose(O.reduce(x, "mean", dims).reshape(-1), np.reshape(refm, -1), rtol=1e-4, atol=1e-5)
    assert O.reduce(np.zeros((3, 0), np.float32), "maximum", 1).tolist() == [np.finfo(np.float32).min] * 3
    with pytest.raises(ValueError):
        O.reduce(np.array([1, 2, 3]), "add", 2)


# ---- element-wise -------------------------------------------------------------------------
def test_unary_closed_forms():
    x = rng.uniform(0.1, 3, 257).astype(np.float32)
    for op, f in [("log", np.log), ("exp", np.exp), ("sqrt", np.sqrt), ("sin", np.sin), ("tanh", np.tanh),
                  ("atan", np.arctan), ("erf", special.erf), ("floor", np.floor), ("ceil", np.ceil),
                  ("abs", np.abs), ("negative", np.negative)]:
        assert np.allclose(O.unary(x, op), f(x.astype(np.float64)), rtol=2e-6), op
    y = rng.uniform(-0.99, 0.99, 200).astype(np.float32)
    assert np.allclose(O.unary(y, "erfinv"), special.erfinv(y.astype(np.float64)), rtol=1e-5, atol=1e-6)
    # std::round is half away from zero (numpy rounds half to even)
    assert O.unary(np.array([0.5, 1.5, 2.5, -0.5, -2.5], np.float32), "round").tolist() == [1, 2, 3, -1, -3]
    assert O.unary(np.array([2.5, -2.5], np.float32), "round_int").dtype == np.int32
    assert np.signbit(O.unary(np.array([-0.3, -0.0], np.float32), "round")).all()      # C: round(-0.3) is -0.0
    # test/test_unary_op.py:68-73: no NaN for large |x|; clamp makes sigmoid(-150) = 1/(1+e^30)
    s = O.unary(np.arange(-150, 150, 10).astype(np.float32), "sigmoid")
    assert not np.isnan(s).any() and np.isclose(s[0], 1 / (1 + np.exp(30.0)), rtol=1e-6) and s[-1] == 1.0
    assert O.unary(np.array([1.7, -1.7], np.float32), "int32").tolist() == [1, -1]      # cast truncates
    assert O.unary(np.array([0.0, 0.3], np.float32), "bool").tolist() == [False, True]
    assert O.unary(np.array([1, 2], np.int32), "sqrt").dtype == np.float32


def test_binary_rules():
    a = np.array([7, -7, 7, -7], np.int32)
    b = np.array([2, 2, -2, -2], np.int32)
    assert O.binary(a, b, "floor_divide").tolist() == [3, -3, -3, 3]        # C division, not floor
    assert O.binary(a, b, "mod").tolist() == [1, -1, 1, -1]                  # C remainder
    af, bf = a.astype(np.float32), b.astype(np.float32)
    assert O.binary(af, bf, "mod").tolist() == [1.0, 1.0, -1.0, -1.0]        # x - floor(x/y)*y
    assert O.binary(a, b, "divide").dtype == np.float32
    assert np.allclose(O.binary(a, b, "divide"), a / b)
    assert O.binary(a, b, "less").dtype == np.bool_
    t, f = np.array([True, True, False]), np.array([True, False, False])
    assert O.binary(t, f, "add").tolist() == [True, True, False]             # bool arithmetic stays bool
    assert O.binary(t, f, "subtract").tolist() == [False, True, False]
    assert O.binary(t, f, "multiply").tolist() == [True, False, False]
    x = rng.uniform(0.5, 2, 64).astype(np.float32)
    y = rng.uniform(-2, 2, 64).astype(np.float32)
    assert np.allclose(O.binary(x, y, "pow"), np.power(x.astype(np.float64), y), rtol=1e-6)
    assert np.array_equal(O.binary(x, y, "maximum"), np.maximum(x, y))
    assert np.array_equal(O.ternary(x > 1, x, y), np.where(x > 1, x, y))
    # relu = ternary(x > 0, x, 0): NaN -> 0 (python/jittor/nn.py:182-183)
    z = np.array([np.nan, -1, 2], np.float32)
    assert O.ternary(O.binary(z, np.float32([0]), "greater"), z, np.zeros(3, np.float32)).tolist() == [0, 0, 2]


def test_bf16_truncation():
    f = np.array([1.0, 1.00390625, 1.0078125, -3.1415926], np.float32)
    bits = O.f32_to_bf16_bits(f)
    back = O.BF16(bits).to_f32()
    assert back[0] == 1.0 and back[1] == 1.0 and back[2] == 1.0078125          # 1+2^-8 truncates down
    assert abs(back[3]) <= abs(f[3])                                          # toward zero
    assert O.c_cast(f, "bfloat16").bits.tolist() == bits.tolist()


# ---- convolution -----------------------------------------------------------------------------
def _conv_f64(x, w, stride, pad, dil):
    N, C, H, W = x.shape
    K, _, R, S = w.shape
    oh = (H + 2 * pad - dil * (R - 1) - 1) // stride + 1
    ow = (W + 2 * pad - dil * (S - 1) - 1) // stride + 1
    xp = np.pad(x.astype(np.float64), ((0, 0), (0, 0), (pad, pad), (pad, pad)))
    y = np.zeros((N, K, oh, ow))
    for r in range(R):
        for s in range(S):
            patch = xp[:, :, r * dil:r * dil + (oh - 1) * stride + 1:stride, s * dil:s * dil + (ow - 1) * stride + 1:stride]
            y += np.einsum("nchw,kc->nkhw", patch, w[:, :, r, s].astype(np.float64))
    return y


@pytest.mark.parametrize("stride,pad,dil", [(1, 1, 1), (2, 1, 1), (1, 2, 2), (1, 0, 1)])
def test_conv_meta_vs_float64(stride, pad, dil):
    x = rng.standard_normal((2, 3, 9, 8)).astype(np.float32)
    w = rng.standard_normal((4, 3, 3, 3)).astype(np.float32)
    y = O.conv_meta(x, w, stride, pad, dil)
    assert np.allclose(y, _conv_f64(x, w, stride, pad, dil), rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("groups,stride,pad,dil", [(2, 1, 1, 1), (4, 2, 1, 1), (3, 1, 2, 2)])
def test_conv_meta_grouped_is_one_convolution_per_group(groups, stride, pad, dil):
    """A grouped convolution is `groups` independent convolutions over channel slices: the 8-d
    restatement against the float64 convolution of each slice (a wrong group stride in either
    reindex, or in the scatter back, mixes slices and fails this)."""
    cg, kg = 2, 3
    x = rng.standard_normal((2, groups * cg, 7, 6)).astype(np.float32)
    w = rng.standard_normal((groups * kg, cg, 3, 3)).astype(np.float32)
    y = O.conv_meta_grouped(x, w, groups, stride, pad, dil)
    for g in range(groups):
        want = _conv_f64(x[:, g * cg:(g + 1) * cg], w[g * kg:(g + 1) * kg], stride, pad, dil)
        assert np.allclose(y[:, g * kg:(g + 1) * kg], want, rtol=1e-5, atol=1e-5)
    one = O.conv_meta_grouped(x[:, :cg], w[:kg], 1, stride, pad, dil)                # one group = the plain form
    assert np.allclose(one, O.conv_meta(x[:, :cg], w[:kg], stride, pad, dil), rtol=1e-6, atol=1e-6)


def test_conv_meta_wgrad_against_finite_differences_of_the_forward():
    """dw is linear in dy and the convolution is linear in w, so <conv(x, w), dy> = <w, dw> for every w
    (a transposed or shifted tap, or a wrong reduced axis, breaks the identity), and dw equals the float64
    correlation of dy with the shifted input planes."""
    for stride, pad, dil in [(1, 1, 1), (2, 1, 1), (1, 2, 2), (1, 0, 1)]:
        x = rng.standard_normal((2, 3, 9, 8)).astype(np.float32)
        w = rng.standard_normal((4, 3, 3, 3)).astype(np.float32)
        y = _conv_f64(x, w, stride, pad, dil)
        dy = rng.standard_normal(y.shape).astype(np.float32)
        dw = O.conv_meta_wgrad(x, dy, 3, 3, stride, pad, dil)
        assert dw.shape == w.shape and dw.dtype == np.float32
        assert np.isclose((y * dy).sum(), (w.astype(np.float64) * dw).sum(), rtol=1e-5)
        xp = np.pad(x.astype(np.float64), ((0, 0), (0, 0), (pad, pad), (pad, pad)))
        oh, ow = dy.shape[2:]
        for r in range(3):
            for s_ in range(3):
                patch = xp[:, :, r * dil:r * dil + (oh - 1) * stride + 1:stride, s_ * dil:s_ * dil + (ow - 1) * stride + 1:stride]
                want = np.einsum("nkhw,nchw->kc", dy.astype(np.float64), patch)
                assert np.allclose(dw[:, :, r, s_], want, rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("groups,stride,pad,dil", [(2, 1, 1, 1), (3, 2, 1, 1), (4, 1, 2, 2), (2, 2, 0, 1)])
def test_conv_meta_grouped_grads_are_the_adjoints_of_the_forward(groups, stride, pad, dil):
    """The grouped convolution is linear in x and in w, so <conv(x, w), dy> = <x, dx> = <w, dw> with the pinned
    forward on the left (a wrong group stride, a flipped tap or a dropped padding row breaks one of them), and
    each group's slices equal the float64 gradients of that group's plain convolution."""
    cg, kg = 2, 3
    x = rng.standard_normal((2, groups * cg, 8, 7)).astype(np.float32)
    w = rng.standard_normal((groups * kg, cg, 3, 3)).astype(np.float32)
    y = O.conv_meta_grouped(x, w, groups, stride, pad, dil).astype(np.float64)
    dy = rng.standard_normal(y.shape).astype(np.float32)
    dx, dw = O.conv_meta_grouped_grads(x, w, dy, groups, stride, pad, dil)
    assert dx.shape == x.shape and dw.shape == w.shape and dx.dtype == np.float32 and dw.dtype == np.float32
    inner = (y * dy).sum()
    assert np.isclose(inner, (x.astype(np.float64) * dx).sum(), rtol=1e-4)
    assert np.isclose(inner, (w.astype(np.float64) * dw).sum(), rtol=1e-4)
    oh, ow = dy.shape[2:]
    for g in range(groups):
        xs, ds = x[:, g * cg:(g + 1) * cg].astype(np.float64), dy[:, g * kg:(g + 1) * kg].astype(np.float64)
        xp = np.pad(xs, ((0, 0), (0, 0), (pad, pad), (pad, pad)))
        dxp = np.zeros_like(xp)
        for r in range(3):
            for s_ in range(3):
                rows = slice(r * dil, r * dil + (oh - 1) * stride + 1, stride)
                cols = slice(s_ * dil, s_ * dil + (ow - 1) * stride + 1, stride)
                want = np.einsum("nkhw,nchw->kc", ds, xp[:, :, rows, cols])
                assert np.allclose(dw[g * kg:(g + 1) * kg, :, r, s_], want, rtol=1e-4, atol=1e-4)
                dxp[:, :, rows, cols] += np.einsum("nkhw,kc->nchw", ds, w[g * kg:(g + 1) * kg, :, r, s_].astype(np.float64))
        want_dx = dxp[:, :, pad:pad + x.shape[2], pad:pad + x.shape[3]]
        assert np.allclose(dx[:, g * cg:(g + 1) * cg], want_dx, rtol=1e-4, atol=1e-4)
    if groups == 2 and stride == 1:                      # one group: the plain weight gradient
        _, dw1 = O.conv_meta_grouped_grads(x[:, :cg], w[:kg], dy[:, :kg], 1, stride, pad, dil)
        assert np.allclose(dw1, O.conv_meta_wgrad(x[:, :cg], dy[:, :kg], 3, 3, stride, pad, dil), rtol=1e-5, atol=1e-5)


def test_conv_meta_one_hot_kernel_is_a_shift():
    x = O.BF16(O.f32_to_bf16_bits(rng.standard_normal((1, 2, 6, 6)).astype(np.float32)))
    w = np.zeros((2, 2, 3, 3), np.float32)
    w[0, 0, 0, 2] = 1.0       # y[0,0,h,w] = x[0,0,h-1,w+1]
    w[1, 1, 1, 1] = 1.0       # identity on channel 1
    y = O.conv_meta(x, O.BF16(O.f32_to_bf16_bits(w)), 1, 1, 1)
    xf = x.to_f32()
    ref0 = np.zeros((6, 6), np.float32)
    ref0[1:, :5] = xf[0, 0, :5, 1:]
    assert np.array_equal(y[0, 0], ref0) and np.array_equal(y[0, 1], xf[0, 1])


# ---- the index-expression evaluator: every operator of python/jittor/src/opt/expr.cc:16-52 ---------------------
_EXPR_VARS = {"a": 7, "b": -3, "i0": 5, "i1": 12}
# literal known answers (C semantics: division truncates towards zero, the remainder takes the dividend's sign,
# comparisons and logical operators give 0 / 1, << binds tighter than <, ?: is right-associative)
_EXPR_KNOWN = [
    ("10+2*6", 22), ("100 * 2 + 12", 212), ("100 * ( 2 + 12 )", 1400), ("100*(2+12)/14", 100), ("-1", -1), ("- 1", -1),
    ("a", 7), ("a+b", 4), ("-1 +a *b", -22),                          # python/jittor/test/test_op_compiler.py:33-46
    ("a/b", -2), ("a%b", 1), ("b/2", -1), ("b%2", -1), ("(-a)%4", -3), ("-a/2", -3),
    ("1+2*3<<1", 14), ("1<<2+1", 8), ("a<b", 0), ("a>b", 1), ("a<=7", 1), ("a>=8", 0), ("a==7", 1), ("a!=b", 1),
    ("a<b?a:b", -3), ("a>b?(b<0?1:2):3", 1), ("0?1:0?2:3", 3), ("1?1:0?2:3", 1),
    ("a>=7&&b<0", 1), ("a==8||b", 1), ("0||0", 0), ("!a", 0), ("!0", 1), ("~a", -8), ("a&b", 5), ("a|b", -1), ("a^b", -6),
    ("a<<2", 28), ("a>>1", 3), ("b>>1", -2), ("a&3|8", 11), ("a|2&1", 7), ("a^1&3", 6), ("1|2^3&4", 3),
    ("i0*3+i1%5-2", 15), ("i1/i0*i0+i1%i0", 12), ("0x1f+0b101", 36), ("2-3-4", -5), ("100/10/5", 2), ("1<2==1", 1),
    ("int(2.7)", 2), ("int(-2.7)", -2), ("int(float(a)/2)", 3), ("int(float(a)/2*2)", 7), ("bool(a)+bool(0)", 1),
]


def test_expression_evaluator_known_answers():
    env = {k: np.int64(v) for k, v in _EXPR_VARS.items()}
    for text, want in _EXPR_KNOWN:
        got = O.eval_expr(O.parse_expr(text), env, [])
        assert int(np.asarray(got)) == want, (text, got, want)
    assert float(np.asarray(O.eval_expr(O.parse_expr("float(a)/2"), env, []))) == 3.5
    for bad in ("*****", "a//b", "a+", "(a", "a b"):                  # test_op_compiler.py:47; loop_var_analyze_pass.cc:298-309
        with pytest.raises(ValueError):
            O.eval_expr(O.parse_expr(bad), env, [])


def test_expression_evaluator_against_the_c_compiler(tmp_path):
    """The expressions are C: compiled as C (gcc, 64-bit integers) they must give what the oracle's evaluator
    gives.  An independent evaluator for precedence, associativity, truncating division and the 0 / 1 results."""
    import shutil
    import subprocess
    if shutil.which("gcc") is None:
        pytest.skip("no C compiler")
    rng = np.random.default_rng(12)
    ops2 = ["+", "-", "*", "/", "%", "<<", ">>", "<", "<=", ">", ">=", "==", "!=", "&", "|", "^", "&&", "||"]
    texts = [t for t, _ in _EXPR_KNOWN if "int(" not in t and "float(" not in t and "bool(" not in t]
    names = list(_EXPR_VARS)
    for _ in range(200):                                              # random three-operator expressions without parentheses
        t = names[rng.integers(4)]
        for _k in range(3):
            op = ops2[rng.integers(len(ops2))]
            rhs = names[rng.integers(4)] if rng.random() < 0.6 else str(int(rng.integers(1, 6)))
            if op in ("<<", ">>"):
                rhs = str(int(rng.integers(0, 4)))
            if op in ("/", "%"):
                rhs = str(int(rng.integers(1, 6)))                    # no division by zero or by a negative shift count
            t = "%s%s%s" % (t, op, rhs)
        if "<<" in t and "b<<" in t:
            continue                                                  # shifting a negative value left is undefined in C
        texts.append(t)
    for _ in range(40):
        texts.append("%s%s%s?%s:%s" % (names[rng.integers(4)], ops2[rng.integers(7, 13)], names[rng.integers(4)],
                                       texts[rng.integers(len(texts))], texts[rng.integers(len(texts))]))
    src = ["#include <stdio.h>", "int main(void) {"]
    src += ["  long long %s = %d;" % kv for kv in _EXPR_VARS.items()]
    src += ['  printf("%%lld\\n", (long long)(%s));' % t for t in texts]
    src += ["  return 0;", "}"]
    c = tmp_path / "e.c"
    c.write_text("\n".join(src))
    subprocess.check_call(["gcc", "-O0", "-w", "-o", str(tmp_path / "e"), str(c)])
    want = [int(v) for v in subprocess.check_output([str(tmp_path / "e")]).split()]
    env = {k: np.int64(v) for k, v in _EXPR_VARS.items()}
    assert len(want) == len(texts)
    for t, w in zip(texts, want):
        got = int(np.asarray(O.eval_expr(O.parse_expr(t), env, [])))
        assert got == w, (t, got, w)
