"""GPU parity: the HIP path (through the C-ABI, via the ctypes front end)
against the CPU oracle on the same seeded inputs.  Bar: bit-exact for reindex
and integer work; 1e-5 relative for fp32 reduce / element-wise; 1e-4 relative
for atomic scatter-add.  Full-size benchmark shapes are checked through
closed forms and size-independent properties."""
import ctypes
import json
import os

import numpy as np
import pytest

import jittor_amd as jt
from jittor_amd import _lib as L
from oracle import oracle as O

pytestmark = pytest.mark.gpu
G = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "vectors.json")))


def bits(a):
    a = np.ascontiguousarray(a)
    return a.view({1: np.uint8, 2: np.uint16, 4: np.uint32, 8: np.uint64}[a.dtype.itemsize])


def exact(a, b):
    return a.shape == b.shape and a.dtype == b.dtype and np.array_equal(bits(a), bits(b))


# ---- golden vectors ------------------------------------------------------------------
def test_golden_vectors(gpu):
    g = G["reindex_shift"]
    assert jt.array(np.array(g["x"], np.int32)).reindex(g["shape"], g["indexes"]).data.tolist() == g["y"]
    g = G["reduce_negative_dim"]
    a = jt.array(g["x"])
    assert a.sum(-1).data.tolist() == g["sum_m1"] and a.sum(-2).data.tolist() == g["sum_m2"]
    g = G["broadcast_dims"]
    b = jt.array(g["x"])
    assert b.broadcast(g["shape"], [-1]).data.tolist() == g["dims_m1"]
    assert b.broadcast(g["shape"], [-2]).data.tolist() == g["dims_m2"]
    g = G["add_scalar"]
    assert (jt.array(g["x"]) + 1).data.tolist() == g["plus1"]
    g = G["gather"]
    t, idx = jt.array(g["t"]), jt.array(g["index"])
    assert t.reindex(idx.shape, ["i0", "@e0(i0,i1)"], extras=[idx]).data.tolist() == g["dim1"]
    assert t.reindex(idx.shape, ["@e0(i0,i1)", "i1"], extras=[idx]).data.tolist() == g["dim0"]
    g = G["scatter_void"]
    src = np.array(g["src"], np.int32)
    out = jt.array(src[:1, :4]).reindex_reduce("void", [3, 5], ["@e0(i0,i1)", "i1"], extras=[jt.array(g["index0"])])
    assert out.data.tolist() == g["out0"]
    out = jt.array(src[:2, :3]).reindex_reduce("void", [3, 5], ["i0", "@e0(i0,i1)"], extras=[jt.array(g["index1"])])
    assert out.data.tolist() == g["out1"]
    g = G["bool_reduce"]
    assert bool((jt.array(np.array(g["a"], bool)) | jt.array(np.array(g["b"], bool))).all().item()) is g["or_all"]
    assert bool((jt.array(np.array(g["a"], bool)) & jt.array(np.array(g["b"], bool))).any().item()) is g["and_any"]


# ---- reduce -------------------------------------------------------------------------------
@pytest.mark.parametrize("keepdims", [False, True])
def test_reduce_integer_exact(gpu, keepdims):
    a = np.arange(2 * 3 * 4 * 5).reshape(2, 3, 4, 5).astype(np.int32)
    ja = jt.array(a)
    for dims in [(), (0,), (1,), (2,), (3,), (0, 2), (1, 3), (1, 2, 3), 2, 3]:
        for op in ["add", "multiply", "maximum", "minimum", "logical_and", "logical_or", "logical_xor",
                   "bitwise_and", "bitwise_or", "bitwise_xor"]:
            if dims not in ((), (0,)) and op != "add":
                continue
            got = jt.reduce(ja, op, dims, keepdims).data
            ref = O.reduce(a, op, dims, keepdims)
            assert exact(got, ref), (op, dims, got, ref)


@pytest.mark.parametrize("shape,dims", [((64, 33, 5), (1,)), ((64, 33, 5), (0, 2)), ((64, 33, 5), ()),
                                        ((7, 1000), (1,)), ((1000, 7), (0,)), ((3, 5, 7, 9, 2), (1, 3)),
                                        ((2, 70000), (1,)), ((70000, 4), (0,)), ((5, 0), (1,)), ((4, 6, 8), (2,)),
                                        # column reduces whose rows are split among workgroups: few vectors of outputs (the
                                        # workgroup's other lanes take other slices), partial sums folded by the row kernel
                                        ((5000, 96), (0,)), ((3, 4000, 520), (0, 1)), ((2048, 1024), (0,)), ((40000, 20), (0,))])
def test_reduce_float(gpu, shape, dims):
    rng = np.random.default_rng(7)
    x = rng.uniform(-1, 1, shape).astype(np.float32)
    n_red = max(1, x.size // max(1, int(np.prod(O.reduce_shape(shape, dims, False)[0]))))
    for op in ["add", "maximum", "minimum", "mean"]:
        got = jt.reduce(jt.array(x), op, dims).data
        ref = O.reduce(x, op, dims)
        assert got.shape == ref.shape and got.dtype == ref.dtype
        if op in ("maximum", "minimum"):
            assert exact(got, ref), op
        else:
            # tolerance: 1e-5 relative, with the absolute floor a reordered fp32 sum of n terms needs
            assert np.allclose(got, ref, rtol=1e-5, atol=1e-5 * np.sqrt(n_red)), (op, np.abs(got - ref).max())


def test_reduce_other_dtypes(gpu):
    rng = np.random.default_rng(8)
    for dtype in ["int8", "uint8", "int16", "int64", "float64", "bool"]:
        x = (rng.integers(0, 2, (6, 40)) if dtype == "bool" else rng.integers(0, 5, (6, 40))).astype(L.NP_STORAGE[dtype])
        for op in ["add", "maximum"]:
            got = jt.reduce(jt.array(x, dtype), op, 1).data
            ref = O.reduce(x, op, 1)
            assert got.dtype == ref.dtype and np.array_equal(got, ref), (dtype, op)
    h = rng.standard_normal((4, 64)).astype(np.float32)
    got = jt.array(h).bfloat16().sum(1).data          # cast -> float32 sum -> cast (truncation)
    hb = O.BF16(O.f32_to_bf16_bits(h)).to_f32()
    want = O.BF16(O.f32_to_bf16_bits(O.reduce(hb, "add", 1))).to_f32()
    assert np.allclose(got, want, rtol=2 ** -7)


@pytest.mark.parametrize("lanes", [128, 256, 512, 1024])
def test_reduce_rows_shared_by_several_waves(gpu, lanes, monkeypatch):
    """The row kernel with a row given to several whole waves (what long streamed rows take by themselves, forced here
    on small inputs): every op family, ragged row lengths (lanes without an element, rows that end inside a vector
    batch), row counts that do not fill the last workgroup, two reduced axes, 16-bit and integer inputs -- against
    the oracle, exact for maximum / minimum / integers, 1e-5 for float sums."""
    monkeypatch.setenv("MJT_REDUCE_G", str(lanes))
    rng = np.random.default_rng(lanes)
    # (few rows are split into partial sums and folded by a second launch; 2100 rows keep the chip busy by themselves)
    for shape, dims in [((37, 5000), (1,)), ((5, 4096), (1,)), ((3, 7, 1031), (2,)), ((6, 3, 2048), (1, 2)), ((9, 640), (1,)),
                        ((2100, 1100), (1,))]:
        x = rng.uniform(-1, 1, shape).astype(np.float32)
        n_red = x.size // int(np.prod(O.reduce_shape(shape, dims, False)[0]))
        for op in ["add", "maximum", "minimum", "mean"]:
            got = jt.reduce(jt.array(x), op, dims).data
            assert ("g%d" % lanes) in L.last_kernel() or (shape[0] < 2100 and L.last_kernel().endswith("_fold")), L.last_kernel()
            ref = O.reduce(x, op, dims)
            if op in ("maximum", "minimum"):
                assert exact(got, ref), (shape, op)
            else:
                assert np.allclose(got, ref, rtol=1e-5, atol=1e-5 * np.sqrt(n_red)), (shape, op, np.abs(got - ref).max())
    xi = rng.integers(-1000, 1000, (11, 3000)).astype(np.int32)
    for op in ["add", "maximum", "bitwise_xor"]:
        assert exact(jt.reduce(jt.array(xi), op, 1).data, O.reduce(xi, op, 1)), op
    h = rng.standard_normal((6, 2500)).astype(np.float32)
    got = jt.array(h).bfloat16().sum(1).data          # cast -> float32 sum -> cast (truncation)
    hb = O.BF16(O.f32_to_bf16_bits(h)).to_f32()
    want = O.BF16(O.f32_to_bf16_bits(O.reduce(hb, "add", 1))).to_f32()
    assert np.allclose(got, want, rtol=2 ** -7)


def test_reduce_full_size_c1(gpu):
    x = np.random.default_rng(0).uniform(-1, 1, (8192, 4096)).astype(np.float32)
    got = jt.array(x).sum(1).data
    assert L.last_kernel().startswith("mjt_reduce_row_add_float32")
    ref = x.astype(np.float64).sum(1)
    assert np.allclose(got, ref, rtol=1e-5, atol=1e-5 * np.sqrt(4096))
    # linearity: sum(2x) == 2 sum(x) exactly (power-of-two scaling commutes with rounding)
    assert np.array_equal(jt.array(2 * x).sum(1).data, 2 * got)


# ---- reindex ----------------------------------------------------------------------------------
def test_reindex_pad_matmul_and_conditions(gpu):
    rng = np.random.default_rng(9)
    a = rng.random(10).astype(np.float32)
    assert exact(jt.array(a).reindex([17], ["i0-3"], -1).data, O.reindex(a, [17], ["i0-3"], -1))
    n = 10
    A, B = rng.random((n, n)).astype(np.float32), rng.random((n, n)).astype(np.float32)
    cc = jt.array(A).reindex([n, n, n], ["i0", "i1"]) * jt.array(B).reindex([n, n, n], ["i1", "i2"])
    assert np.allclose(cc.sum(1).data, A @ B, rtol=1e-5)
    x = rng.random((2, 4, 4, 2)).astype(np.float32)
    shape, idx, ofc = [2, 10, 10, 3, 3, 2], ["i0", "(i1-i3)/2", "(i2-i4)/2", "i5"], ["(i1-i3)%2", "(i2-i4)%2"]
    assert exact(jt.array(x).reindex(shape, idx, 0, ofc).data, O.reindex(x, shape, idx, 0, ofc))
    # reflect-style ternary expression and shape names
    e = ["i0<2 ? 2-i0 : (i0>=xshape0+2 ? 2*xshape0-i0 : i0-2)"]
    assert exact(jt.array(a).reindex([14], e).data, O.reindex(a, [14], e))


def test_reindex_extras_and_dtypes(gpu):
    rng = np.random.default_rng(10)
    a = rng.random((10, 10)).astype(np.float32)
    b = np.array([2], np.int32)
    e1 = rng.integers(0, 10, (10, 10)).astype(np.float32)
    idx = ["@e0(0)", "@e1(0,i0 / @e0(0))"]
    assert exact(jt.array(a).reindex([8, 8], idx, extras=[jt.array(b), jt.array(e1)]).data,
                 O.reindex(a, [8, 8], idx, extras=[b, e1]))
    iv = rng.integers(-3, 13, (6, 7)).astype(np.int64)          # out of range on both sides -> overflow value
    for dtype in ["int8", "int16", "int32", "int64", "uint8", "float64", "bool", "float16"]:
        x = (rng.random(10) * 10).astype(L.NP_STORAGE[dtype])
        got = jt.array(x, dtype).reindex_var([jt.array(iv, "int64")], 1).data
        assert exact(got, O.reindex(x, [6, 7], ["@e0(i0,i1)"], 1, extras=[iv])), dtype
    xb = jt.array(rng.standard_normal(10).astype(np.float32)).bfloat16()
    got = xb.reindex([6, 7], ["@e0(i0,i1)"], 1.5, extras=[jt.array(iv, "int64")]).raw()
    assert np.array_equal(got, O.reindex(O.BF16(xb.raw()), [6, 7], ["@e0(i0,i1)"], 1.5, extras=[iv]).bits)
    assert jt.array(a).reindex([0, 4], ["i0", "i1"]).data.shape == (0, 4)


@pytest.mark.parametrize("dtype", ["float32", "int8", "int16", "float64", "bfloat16"])
def test_reindex_rows_that_are_no_whole_vectors(gpu, dtype):
    """A gather whose innermost extent does not divide into 16-byte vectors while the whole result does: every lane
    still stores 16 bytes, its elements decoded one by one (they may lie in two rows).  Pads, crops with steps, a
    flipped axis, an overflow condition; bit-exact against the oracle and against the one-element-per-lane form."""
    rng = np.random.default_rng(12)
    x = (rng.standard_normal((3, 5, 14, 9)) * 40).astype(np.float32)
    xv = jt.array(x).cast(dtype)
    ref_in = O.BF16(xv.raw()) if dtype == "bfloat16" else xv.data
    for shape, idx, ov, ofc in [
            ([3, 5, 16, 11], ["i0", "i1", "i2-1", "i3-1"], 0.0, []),                  # pad 1: rows of 11
            ([3, 4, 8, 7], ["i0", "i1+1", "i2*2-1", "8-i3"], 2.0, []),                # steps, a flipped innermost axis
            ([2, 5, 14, 13], ["i0+1", "i1", "13-i2", "i3-2"], -3.0, ["i3>10"]),       # an overflow condition
            ([16, 1, 3, 5, 3], ["i2", "i3", "i0", "i4*4"], 1.0, []),                  # rows of 3, a permuted source
            ([3, 5, 14, 5], ["i0", "i1", "i2", "i3+2"], 0.0, [])]:                    # 1050 elements: no vector fits the whole
        want = O.reindex(ref_in, shape, idx, ov, ofc)
        want = want.bits if dtype == "bfloat16" else want
        got = xv.reindex(shape, idx, ov, ofc)
        got = got.raw() if dtype == "bfloat16" else got.data
        assert L.last_kernel().startswith("mjt_reindex_")
        assert np.array_equal(got, want), (dtype, shape)
        os.environ["MJT_REINDEX_NO_FLAT"] = "1"
        try:
            again = xv.reindex(shape, idx, ov, ofc)
            again = again.raw() if dtype == "bfloat16" else again.data
        finally:
            del os.environ["MJT_REINDEX_NO_FLAT"]
        assert np.array_equal(again, want), (dtype, shape)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16", "int8", "float64"])
def test_reindex_two_runs_woven_into_each_other(gpu, dtype):
    """A lane whose even and odd elements are each adjacent in x loads them as two half vectors: every source element
    taken twice (nearest-neighbour upsampling), columns interleaved from several sources (the stride phases of an input
    gradient), and the same with rows where only some waves qualify; bit-exact against the oracle."""
    rng = np.random.default_rng(14)
    x = (rng.standard_normal((4, 3, 5, 6, 8)) * 40).astype(np.float32)
    xv = jt.array(x).cast(dtype)
    ref_in = O.BF16(xv.raw()) if dtype == "bfloat16" else xv.data
    for shape, idx, ov in [
            ([3, 5, 12, 16], ["i2%2*2+i3%2", "i0", "i1", "i2/2", "i3/2"], 0.0),      # four sources woven by rows and columns
            ([4, 3, 5, 6, 16], ["i0", "i1", "i2", "i3", "i4/2"], 0.0),              # every element twice
            ([4, 3, 5, 6, 16], ["i0", "i1", "i2", "i3", "i4/2+1"], -2.0),            # the same, shifted: the last pair out of range
            ([2, 3, 5, 6, 16], ["i0*2+i4%2", "i1", "i2", "i3", "i4/2"], 0.0)]:       # two sources far apart
        want = O.reindex(ref_in, shape, idx, ov)
        want = want.bits if dtype == "bfloat16" else want
        got = xv.reindex(shape, idx, ov)
        got = got.raw() if dtype == "bfloat16" else got.data
        assert L.last_kernel().startswith("mjt_reindex_")
        assert np.array_equal(got, want), (dtype, shape, idx)


@pytest.mark.parametrize("case", [
    dict(x=(2, 3, 7, 6), k=(3, 3), s=(1, 1), d=(1, 1), p=(1, 1)),
    dict(x=(3, 9, 11), k=(3, 2), s=(2, 1), d=(1, 2), p=(0, 1)),
    dict(x=(13, 17), k=(5, 5), s=(1, 1), d=(1, 1), p=(2, 2)),
    dict(x=(2, 2, 70, 64), k=(3, 3), s=(1, 1), d=(1, 1), p=(1, 1)),
    dict(x=(1, 200, 8), k=(2, 2), s=(2, 2), d=(1, 1), p=(0, 0)),
])
@pytest.mark.parametrize("dtype", ["float32", "int16", "float64"])
def test_window_gather_fast_path_matches_oracle_and_generic(gpu, case, dtype):
    rng = np.random.default_rng(11)
    xs, (kh, kw), (sh, sw), (dh, dw), (ph, pw) = case["x"], case["k"], case["s"], case["d"], case["p"]
    H, W = xs[-2], xs[-1]
    oh = (H + 2 * ph - dh * (kh - 1) - 1) // sh + 1
    ow = (W + 2 * pw - dw * (kw - 1) - 1) // sw + 1
    nb = len(xs) - 2
    x = (rng.standard_normal(xs) * 50).astype(L.NP_STORAGE[dtype])
    shape = list(xs[:nb]) + [oh, ow, kh, kw]
    idx = ["i%d" % i for i in range(nb)] + ["i%d*%d+i%d*%d-%d" % (nb, sh, nb + 2, dh, ph),
                                            "i%d*%d+i%d*%d-%d" % (nb + 1, sw, nb + 3, dw, pw)]
    ref = O.reindex(x, shape, idx, 3)
    got = jt.array(x, dtype).reindex(shape, idx, 3).data
    fast = L.last_kernel()
    assert exact(got, ref)
    os.environ["MJT_NO_FASTPATH"] = "1"
    try:
        got2 = jt.array(x, dtype).reindex(shape, idx, 3).data
        assert L.last_kernel().startswith("mjt_reindex_")
    finally:
        del os.environ["MJT_NO_FASTPATH"]
    assert exact(got2, ref)
    assert fast.startswith("mjt_window_gather"), fast


@pytest.mark.parametrize("case", [
    # x [N, C, H, W],  taps,   stride, dilation, padding, images per chunk (None: one image per group; 0: the whole batch is one group)
    dict(x=(3, 5, 9, 10), k=(3, 3), s=(1, 1), d=(1, 1), p=(1, 1), nb=None),
    dict(x=(4, 3, 14, 14), k=(3, 3), s=(1, 1), d=(1, 1), p=(1, 1), nb=2),             # 196-pixel planes in pairs: vectors of 8 cross image borders
    dict(x=(8, 4, 7, 7), k=(3, 3), s=(1, 1), d=(1, 1), p=(1, 1), nb=0),               # 49-pixel planes, the whole batch side by side
    dict(x=(6, 2, 27, 27), k=(3, 3), s=(2, 2), d=(1, 1), p=(1, 1), nb=3),             # stride 2; three images: vectors of 4
    dict(x=(2, 3, 14, 13), k=(2, 3), s=(1, 2), d=(2, 1), p=(0, 2), nb=None),          # mixed stride / dilation, no vertical padding
    dict(x=(3, 2, 9, 9), k=(1, 2), s=(1, 1), d=(1, 1), p=(0, 0), nb=None),            # 1x2 taps, 72 pixels per run
    dict(x=(3, 2, 9, 9), k=(3, 3), s=(1, 1), d=(1, 1), p=(1, 1), nb=None),            # 81 pixels per run: single elements
    # (maps of up to 64 pixels read the other way round, taps as pixels and pixels as taps, are the sliding-window gather's)
    dict(x=(2, 2, 40, 56), k=(5, 5), s=(1, 1), d=(1, 1), p=(2, 2), nb=None),          # 25 taps on a larger plane
])
@pytest.mark.parametrize("dtype", ["bfloat16", "float32", "float16"])
def test_im2col_planes_fast_path_matches_oracle_and_generic(gpu, case, dtype):
    """The column matrices of a convolution with the pixels innermost (kernels/im2col_planes.h), per image, for the whole
    batch and per chunk of images: bit for bit against the oracle's reindex and against the generic gather."""
    rng = np.random.default_rng(14)
    (N, C, H, W), (kh, kw), (sh, sw), (dh, dw), (ph, pw), nb = case["x"], case["k"], case["s"], case["d"], case["p"], case["nb"]
    oh = (H + 2 * ph - dh * (kh - 1) - 1) // sh + 1
    ow = (W + 2 * pw - dw * (kw - 1) - 1) // sw + 1
    store = L.NP_STORAGE[dtype]
    x32 = (rng.standard_normal(case["x"]) * 4).astype(np.float32)
    x = O.f32_to_bf16_bits(x32) if dtype == "bfloat16" else x32.astype(store)
    if nb is None:
        shape, a = [N, C, kh, kw, oh, ow], 2
        idx = ["i0", "i1"]
    elif nb == 0:
        shape, a = [C, kh, kw, N, oh, ow], 1
        idx = ["i3", "i0"]
    else:
        shape, a = [N // nb, C, kh, kw, nb, oh, ow], 2
        idx = ["i0*%d+i4" % nb, "i1"]
    o = len(shape) - 2
    idx += ["i%d*%d-%d+i%d*%d" % (o, sh, ph, a, dh), "i%d*%d-%d+i%d*%d" % (o + 1, sw, pw, a + 1, dw)]
    ref = O.reindex(x, shape, idx, 0)
    vx = jt.from_storage(x, dtype) if dtype != "float32" else jt.array(x)
    got = vx.reindex(shape, idx, 0).raw()
    fast = L.last_kernel()
    assert exact(got, ref)
    os.environ["MJT_NO_FASTPATH"] = "1"
    try:
        got2 = vx.reindex(shape, idx, 0).raw()
        assert L.last_kernel().startswith("mjt_reindex_")
    finally:
        del os.environ["MJT_NO_FASTPATH"]
    assert exact(got2, ref)
    assert fast.startswith("mjt_im2col_planes"), fast


def test_reindex_full_size_c2_bit_exact(gpu):
    x = np.random.default_rng(0).standard_normal((32, 64, 56, 56)).astype(np.float32)
    y = jt.array(x).reindex([32, 64, 56, 56, 3, 3], ["i0", "i1", "i2+i4-1", "i3+i5-1"], 0).data
    assert L.last_kernel().startswith("mjt_window_gather")
    ref = np.lib.stride_tricks.sliding_window_view(np.pad(x, ((0, 0), (0, 0), (1, 1), (1, 1))), (3, 3), axis=(2, 3))
    assert np.array_equal(bits(y), bits(ref))


# ---- reindex_reduce ---------------------------------------------------------------------------------
@pytest.mark.parametrize("op", ["maximum", "minimum", "multiply", "add"])
def test_reindex_reduce_pool(gpu, op):
    x = np.random.default_rng(12).random((3, 10, 10, 4)).astype(np.float32)
    idx = ["i0", "i1/3", "i2/3", "i3"]
    got = jt.array(x).reindex_reduce(op, [3, 4, 4, 4], idx).data
    ref = O.reindex_reduce(x, op, [3, 4, 4, 4], idx)
    if op in ("maximum", "minimum"):
        assert exact(got, ref)
    else:
        assert np.allclose(got, ref, rtol=1e-4)


@pytest.mark.parametrize("case", [
    # y's loop shape,           indexes into x,                               x shape
    ([2, 3, 6, 7, 3, 3], ["i0", "i1", "i2*2+i4-1", "i3*2+i5-1"], [2, 3, 12, 14]),      # 3x3 stride 2 pad 1: windows overlap
    ([2, 3, 6, 7, 2, 2], ["i0", "i1", "i2*2+i4", "i3*2+i5"], [2, 3, 12, 14]),          # 2x2 stride 2: every element once
    ([4, 5, 5, 3, 2], ["i0", "i1*2+i3*2-2", "i2*3+i4-1"], [4, 11, 13]),               # one batch axis, dilation 2, elements no window reaches
    ([9, 8, 3, 2], ["i0+i2-2", "i1*1+i3*3"], [9, 12]),                                 # no batch axis, stride 1, horizontal dilation 3
    ([2, 4, 4, 3, 3], ["i0", "i1*4+i3", "i2*4+i4+1"], [2, 14, 20]),                    # stride beyond the window: gaps; rows the map never reaches
    ([1, 2, 3, 3, 7, 1], ["i0", "i1", "i2*3+i4-3", "i3+i5"], [1, 2, 8, 3]),            # a window taller than the image
])
@pytest.mark.parametrize("op,dtype", [("add", "float32"), ("maximum", "float32"), ("add", "int32"), ("minimum", "int16"),
                                      ("multiply", "float64"), ("add", "bfloat16")])
def test_window_scatter_runs_as_a_gather(gpu, case, op, dtype, monkeypatch):
    """reindex_reduce through a window pattern (the gradient of pooling): every element of x folds the windows that
    reach it, no atomic update.  Against the oracle, and against the atomic kernel on the same input; integers, maximum
    and minimum bit-exact, float sums within 1e-4 of the sum of magnitudes (another order of addition)."""
    shape, idx, xshape = case
    rng = np.random.default_rng(61)
    if dtype in ("float32", "float64", "bfloat16"):
        y = (rng.standard_normal(shape) * (0.2 if op == "multiply" else 2.0) + (1.0 if op == "multiply" else 0.0)).astype(np.float32)
    else:
        y = rng.integers(-3, 4, shape).astype(np.float32)
    vy = jt.array(y).cast(dtype)
    jt.sync([vy])
    ref_in = O.BF16(vy.raw()) if dtype == "bfloat16" else vy.data
    got_v = vy.reindex_reduce(op, xshape, idx)
    jt.sync([got_v])
    assert L.last_kernel().startswith("mjt_window_scatter_" + op), L.last_kernel()
    monkeypatch.setenv("MJT_NO_WINDOW_SCATTER", "1")
    atomic_v = vy.reindex_reduce(op, xshape, idx)
    jt.sync([atomic_v])
    assert L.last_kernel().startswith("mjt_reindex_reduce_" + op), L.last_kernel()
    monkeypatch.delenv("MJT_NO_WINDOW_SCATTER")
    if dtype == "bfloat16":
        # 16-bit sums: one rounding here (float32 accumulator), one per update in the atomic kernel and in the oracle
        ref = O.reindex_reduce(ref_in.to_f32(), op, xshape, idx)
        mag = O.reindex_reduce(np.abs(ref_in.to_f32()), op, xshape, idx)
        got = O.BF16(got_v.raw()).to_f32()
        assert (np.abs(got - ref) <= 2.0 ** -7 * mag + 1e-30).all()
        return
    ref = O.reindex_reduce(ref_in, op, xshape, idx)
    got, atomic = got_v.data, atomic_v.data
    assert got.dtype == ref.dtype
    if dtype in ("int32", "int16") or op in ("maximum", "minimum"):
        assert np.array_equal(got, ref) and np.array_equal(atomic, ref)
    elif op == "add":
        mag = O.reindex_reduce(np.abs(ref_in), op, xshape, idx)
        assert (np.abs(got - ref) <= 1e-4 * mag + 1e-30).all() and (np.abs(atomic - ref) <= 1e-4 * mag + 1e-30).all()
    else:
        assert np.allclose(got, ref, rtol=1e-9) and np.allclose(atomic, ref, rtol=1e-9)


def test_reindex_reduce_dtypes_and_overflow(gpu):
    rng = np.random.default_rng(13)
    n, bins = 4000, 50
    idx = (rng.integers(0, bins + 6, n) - 3).astype(np.int32)
    for dtype in ["int32", "int64", "uint32", "int8", "int16", "float64"]:
        v = rng.integers(0, 3, n).astype(L.NP_STORAGE[dtype])
        for op in ["add", "maximum", "minimum", "bitwise_or"]:
            if dtype == "float64" and op == "bitwise_or":
                continue
            got = jt.array(v, dtype).reindex_reduce(op, [bins], ["@e0(i0)"], extras=[jt.array(idx)]).data
            ref = O.reindex_reduce(v, op, [bins], ["@e0(i0)"], extras=[idx])
            assert got.dtype == ref.dtype and np.array_equal(got, ref), (dtype, op)
    # two-axis target, extras of another shape (test/test_reindex_reduce_op.py:79-90)
    a = np.array([1, 2, 3, 0], np.int32)
    b = rng.random((3, 3)).astype(np.float32)
    got = jt.array(b).reindex_reduce("add", [4, 4], ["@e0(i0)", "@e0(i1)"], extras=[jt.array(a)]).data
    assert np.allclose(got, O.reindex_reduce(b, "add", [4, 4], ["@e0(i0)", "@e0(i1)"], extras=[a]))


@pytest.mark.parametrize("n,bins", [(1 << 16, 300), (100003, 1 << 17), (5, 3), (1 << 18, 40000)])
def test_scatter_1d_fast_path(gpu, n, bins):
    rng = np.random.default_rng(14)
    v = rng.random(n).astype(np.float32)
    v[::97] = np.nan if n > 100 else v[::97]
    vi = np.nan_to_num(v)
    idx = np.minimum((rng.pareto(1.0, n) * 3).astype(np.int64), bins + 2).astype(np.int32) - 1   # skewed, some out of range
    ok = (idx >= 0) & (idx < bins)
    jv, ji = jt.array(vi), jt.array(idx)
    got = jv.reindex_reduce("add", [bins], ["@e0(i0)"], extras=[ji]).data
    assert L.last_kernel().startswith("mjt_scatter1d_add")
    ref = np.bincount(idx[ok], weights=vi[ok].astype(np.float64), minlength=bins)
    assert np.allclose(got, ref, rtol=1e-4, atol=1e-6)
    for op, at in (("maximum", np.maximum), ("minimum", np.minimum)):
        got = jt.array(v).reindex_reduce(op, [bins], ["@e0(i0)"], extras=[ji]).data      # NaN values never win
        assert exact(got, O.reindex_reduce(v, op, [bins], ["@e0(i0)"], extras=[idx])), op
    i64 = jt.array(idx.astype(np.int64), "int64")
    got = jt.array(np.ones(n, np.int32)).reindex_reduce("add", [bins], ["@e0(i0)"], extras=[i64]).data
    assert np.array_equal(got, np.bincount(idx[ok], minlength=bins).astype(np.int32))


def test_scatter_1d_add_propagates_nan(gpu):
    """The reference's loop is x[idx] = x[idx] + y (reindex_reduce_op.cc:123-130): one NaN update makes its bin
    NaN and leaves every other bin alone.  The bins are chosen so that NaNs pass through each route of the 1-d
    scatter: the LDS copy of the hot bucket, the lists of the other buckets (several list items combining in x
    through atomics for the well-filled bucket, a single storing item for the others), and a bin nobody else updates."""
    rng = np.random.default_rng(23)
    n, bins = 1 << 21, 1 << 18
    v = rng.random(n, dtype=np.float32)
    idx = np.where(rng.random(n) < 0.6, rng.integers(0, 3000, n),
                   np.where(rng.random(n) < 0.5, rng.integers(16384, 32768, n), rng.integers(0, bins - 1, n))).astype(np.int32)
    nan_bins = np.array([5, 2999, 20000, 32767, 100000, 200001, bins - 1], np.int64)
    where = rng.choice(n, nan_bins.size * 3, replace=False)
    idx[where] = np.repeat(nan_bins, 3)
    v[where] = np.nan
    got = jt.array(v).reindex_reduce("add", [bins], ["@e0(i0)"], extras=[jt.array(idx)]).data
    assert L.last_kernel().startswith("mjt_scatter1d_add")
    want = O.reindex_reduce(v, "add", [bins], ["@e0(i0)"], extras=[idx])
    assert np.array_equal(np.isnan(got), np.isnan(want)) and np.isnan(got).sum() == nan_bins.size
    assert np.isnan(got[nan_bins]).all()
    fin = ~np.isnan(want)
    ref = np.bincount(idx[~np.isnan(v)], weights=v[~np.isnan(v)].astype(np.float64), minlength=bins)
    assert np.allclose(got[fin], ref[fin], rtol=1e-4, atol=1e-6)


def _scatter_check(v, idx, bins, ops=("add", "maximum", "minimum")):
    ok = (idx >= 0) & (idx < bins)
    jv, ji = jt.array(v), jt.array(idx, "int64" if idx.dtype == np.int64 else "int32")
    for op in ops:
        got = jv.reindex_reduce(op, [bins], ["@e0(i0)"], extras=[ji]).data
        assert L.last_kernel().startswith("mjt_scatter1d_" + op), L.last_kernel()
        if op == "add":
            ref = np.bincount(idx[ok], weights=v[ok].astype(np.float64), minlength=bins)
            assert np.allclose(got, ref, rtol=1e-4, atol=1e-6), op
        else:
            ref = np.full(bins, np.finfo(np.float32).min if op == "maximum" else np.finfo(np.float32).max, np.float32)
            (np.maximum if op == "maximum" else np.minimum).at(ref, idx[ok], v[ok])
            assert np.array_equal(got, ref), op


def test_scatter_1d_index_distributions(gpu):
    """The routes of the 1-d scatter besides the Zipf head: no hot bucket at all (every update is listed, the
    staging areas overflow), two hot regions (lists overflow into the overflow lists), sorted indices (every
    workgroup has its own hot bucket), a single value, a ragged tail, indices far outside the bins."""
    rng = np.random.default_rng(17)
    n, bins = 1 << 21, 1 << 20
    v = (rng.random(n, dtype=np.float32) - 0.25).astype(np.float32)            # both signs
    _scatter_check(v, rng.integers(0, bins, n).astype(np.int32), bins)                       # uniform over 64 buckets
    two = np.where(rng.random(n) < 0.5, rng.integers(0, 9000, n), rng.integers(500000, 509000, n)).astype(np.int32)
    _scatter_check(v, two, bins)                                                             # two hot regions
    _scatter_check(v, np.sort(rng.integers(0, bins, n)).astype(np.int32), bins)              # sorted
    _scatter_check(v, np.full(n, 777777, np.int32), bins, ops=("add", "maximum"))            # one bin takes everything
    far = rng.integers(-(1 << 40), 1 << 40, 100003).astype(np.int64)                         # mostly out of range
    far[::3] = rng.integers(0, bins, far[::3].size)
    _scatter_check(v[:100003], far, bins)
    for m in (1, 2, 3, 6, 4097):                                                             # tails and tiny inputs
        _scatter_check(v[:m], rng.integers(0, 50, m).astype(np.int32), 50)
    big = 9_000_000                                                                          # more than 512 buckets: generic kernel
    got = jt.array(v[:4096]).reindex_reduce("add", [big], ["@e0(i0)"], extras=[jt.array(rng.integers(0, big, 4096).astype(np.int32))]).data
    assert not L.last_kernel().startswith("mjt_scatter1d_") and abs(got.sum() - v[:4096].astype(np.float64).sum()) < 1e-2


def test_window_gather_several_tiles_per_workgroup(gpu, monkeypatch):
    """MJT_WINDOW_TPW > 1: a workgroup walks several tiles of a plane and loads the next tile's input while it
    stores the current one; same bits as the oracle, also when the last workgroup of a plane has fewer tiles."""
    rng = np.random.default_rng(31)
    x = rng.standard_normal((3, 5, 41, 23)).astype(np.float32)
    idx = ["i0", "i1", "i2*2+i4-1", "i3+i5-2"]
    shape = [3, 5, 21, 24, 3, 4]
    want = O.reindex(x, shape, idx, -7.0)
    for tpw, th in ((3, 4), (2, 8), (50, 1)):
        monkeypatch.setenv("MJT_WINDOW_TPW", str(tpw))
        monkeypatch.setenv("MJT_WINDOW_TH", str(th))
        got = jt.array(x).reindex(shape, idx, -7.0).data
        assert L.last_kernel().startswith("mjt_window_gather") and L.last_kernel().endswith("x%d" % min(tpw, -(-21 // th))), L.last_kernel()
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (tpw, th)


def _zipf_indices(n, bins):
    w = np.arange(1, bins + 1, dtype=np.float64) ** -1.1
    cdf = np.cumsum(w) / w.sum()
    return np.minimum(np.searchsorted(cdf, np.random.default_rng(1).random(n)), bins - 1).astype(np.int32)


def test_scatter_full_size_c3(gpu):
    n, bins = 1 << 24, 1 << 20
    v = np.random.default_rng(0).random(n, dtype=np.float32)
    idx = _zipf_indices(n, bins)
    jv, ji = jt.array(v), jt.array(idx)
    got = jv.reindex_reduce("add", [bins], ["@e0(i0)"], extras=[ji]).data
    ref = np.bincount(idx, weights=v.astype(np.float64), minlength=bins)
    assert np.allclose(got, ref, rtol=1e-4, atol=0)                     # empty bins are exactly 0
    assert abs(got.astype(np.float64).sum() - ref.sum()) <= 1e-6 * ref.sum()
    got = jv.reindex_reduce("maximum", [bins], ["@e0(i0)"], extras=[ji]).data
    ref = np.full(bins, np.finfo(np.float32).min, np.float32)
    np.maximum.at(ref, idx, v)
    assert np.array_equal(got, ref)
    # a shifted hot region must give the same answer (the LDS window follows the data)
    shifted = ((idx.astype(np.int64) + 700001) % bins).astype(np.int32)
    got = jv.reindex_reduce("add", [bins], ["@e0(i0)"], extras=[jt.array(shifted)]).data
    ref = np.bincount(shifted, weights=v.astype(np.float64), minlength=bins)
    assert np.allclose(got, ref, rtol=1e-4, atol=0)


# ---- element-wise and fused chains ------------------------------------------------------------------------
UNARY_RANGES = {"log": (0.1, 5), "sqrt": (0, 5), "asin": (-1, 1), "acos": (-1, 1), "acosh": (1, 5), "atanh": (-0.99, 0.99),
                "erfinv": (-0.99, 0.99), "exp": (-5, 5), "sinh": (-5, 5), "cosh": (-5, 5)}


@pytest.mark.parametrize("op", L.UNARY_OPS)
def test_unary_ops(gpu, op):
    if op == "cast":
        pytest.skip("covered by test_casts")
    rng = np.random.default_rng(15)
    lo, hi = UNARY_RANGES.get(op, (-4, 4))
    x = rng.uniform(lo, hi, 1031).astype(np.float32)
    if op in ("logical_not", "bitwise_not"):
        xi = rng.integers(-5, 5, 1031).astype(np.int32)
        got, ref = jt.unary(jt.array(xi), op).data, O.unary(xi, op)
        assert exact(got, ref)
        return
    got, ref = jt.unary(jt.array(x), op).data, O.unary(x, op)
    assert got.dtype == ref.dtype
    if ref.dtype.kind != "f" or op in ("abs", "negative", "floor", "ceil", "round"):
        assert exact(got, ref), op
    else:
        assert np.allclose(got, ref, rtol=1e-5, atol=1e-6), (op, np.abs(got - ref).max())


@pytest.mark.parametrize("op", [o for o in L.BINARY_OPS if o != "mean"])
def test_binary_ops(gpu, op):
    rng = np.random.default_rng(16)
    if op in ("left_shift", "right_shift", "bitwise_and", "bitwise_or", "bitwise_xor"):
        pairs = [(rng.integers(0, 100, 515).astype(np.int32), rng.integers(0, 5, 515).astype(np.int32))]
    else:
        xf, yf = rng.uniform(0.5, 4, 515).astype(np.float32), rng.uniform(-3, 3, 515).astype(np.float32)
        yf[np.abs(yf) < 0.1] = 1.0
        if op == "floor_divide":
            yf[np.abs(yf) < 1] = 1.5          # int(y) == 0 would be an integer division by zero (undefined in C)
        xi, yi = rng.integers(-20, 20, 515).astype(np.int32), rng.integers(1, 7, 515).astype(np.int32) * rng.choice([-1, 1], 515).astype(np.int32)
        pairs = [(xf, yf), (xi, yi)] if op != "pow" else [(xf, yf)]
        if op in ("add", "multiply", "maximum", "less"):
            pairs.append((xi.astype(np.int8), yf))            # mixed widths / kinds
    for x, y in pairs:
        got, ref = jt.binary(jt.array(x), jt.array(y), op).data, O.binary(x, y, op)
        assert got.dtype == ref.dtype, (op, got.dtype, ref.dtype)
        if ref.dtype.kind == "f":
            assert np.allclose(got, ref, rtol=1e-5, atol=1e-6), (op, x.dtype)
        else:
            assert np.array_equal(got, ref), (op, x.dtype)


def test_casts(gpu):
    rng = np.random.default_rng(17)
    x = (rng.standard_normal(300) * 40).astype(np.float32)
    for dtype in ["bool", "int8", "int16", "int32", "int64", "uint8", "float16", "float64", "bfloat16"]:
        j = jt.array(x).cast(dtype)
        ref = O.c_cast(np.clip(x, 0, 100) if dtype == "uint8" else x, dtype)
        if dtype == "uint8":
            j = jt.array(np.clip(x, 0, 100)).cast(dtype)
        if dtype == "bfloat16":
            assert np.array_equal(j.raw(), ref.bits)           # truncation, not rounding
        else:
            assert exact(j.data, ref), dtype
    b = jt.array(x).bfloat16()
    assert np.array_equal(b.float32().data, O.BF16(b.raw()).to_f32())


def _c4(x, s, b):
    return jt.exp(-jt.nn.relu(x * s + b)) * jt.sigmoid(x)


def _c4_oracle(x, s, b):
    t = O.binary(O.binary(x, O.broadcast_to(s, x.shape), "multiply"), O.broadcast_to(b, x.shape), "add")
    zero = np.zeros(1, np.float32)
    r = O.ternary(O.binary(t, O.broadcast_to(zero, x.shape), "greater"), t, O.broadcast_to(zero, x.shape))
    return O.binary(O.unary(O.unary(r, "negative"), "exp"), O.unary(x, "sigmoid"), "multiply")


@pytest.mark.parametrize("shape", [(4, 6, 8), (3, 5, 7), (2, 512, 1024)])
def test_fused_chain_c4_small(gpu, shape):
    x = np.random.default_rng(0).standard_normal(shape).astype(np.float32)
    s = np.random.default_rng(1).standard_normal((shape[1], 1)).astype(np.float32)
    b = np.random.default_rng(2).standard_normal((1, shape[2])).astype(np.float32)
    before = jt.executor_stats["launches"]
    got = _c4(jt.array(x), jt.array(s), jt.array(b)).data
    assert jt.executor_stats["launches"] == before + 1            # one kernel for the whole chain
    assert L.last_kernel().startswith("mjt_fused_")
    ref = _c4_oracle(x, s, b)
    assert np.allclose(got, ref, rtol=1e-5, atol=0), np.abs(got / ref - 1).max()


def test_fused_chain_full_size_c4(gpu):
    shape = (64, 512, 1024)
    x = np.random.default_rng(0).standard_normal(shape).astype(np.float32)
    s = np.random.default_rng(1).standard_normal((512, 1)).astype(np.float32)
    b = np.random.default_rng(2).standard_normal((1, 1024)).astype(np.float32)
    got = _c4(jt.array(x), jt.array(s), jt.array(b)).data
    x64 = x.astype(np.float64)
    ref = np.exp(-np.maximum(x64 * s + b, 0)) / (1 + np.exp(np.minimum(-x64, 30)))
    assert np.abs(got / ref - 1).max() < 1e-5                     # all outputs are positive
    sl = (slice(0, 64, 9), slice(0, 512, 37), slice(None))
    assert np.allclose(got[sl], _c4_oracle(x[sl], s[sl[1]], b), rtol=1e-5, atol=0)


def test_fused_groups_outputs_scalars_and_bool(gpu):
    rng = np.random.default_rng(18)
    x = rng.standard_normal((33, 17)).astype(np.float32)
    y = rng.standard_normal((33, 17)).astype(np.float32)
    jx, jy = jt.array(x), jt.array(y)
    a = jx * 2.0 + jy                       # shared by both outputs
    m = a > 0.5
    z = jt.ternary(m, a, jy * 0.25)
    before = jt.executor_stats["launches"]
    jt.sync([a, m, z])
    assert jt.executor_stats["launches"] == before + 1
    ra = x * np.float32(2.0) + y
    assert np.allclose(a.data, ra, rtol=1e-6) and np.array_equal(m.data, ra > 0.5)
    assert np.allclose(z.data, np.where(ra > 0.5, ra, y * np.float32(0.25)), rtol=1e-6)
    # a [1]-shaped computed Var (a full reduce) broadcasts as a tensor input
    t = jx - jx.mean()
    assert np.allclose(t.data, x - x.mean(), rtol=1e-5, atol=1e-6)
    # relu(NaN) = 0 (python/jittor/nn.py:182-183)
    assert jt.nn.relu(jt.array(np.array([np.nan, -1.0, 2.0], np.float32))).data.tolist() == [0.0, 0.0, 2.0]
    # broadcast alone materialises through the same kernel family
    assert np.array_equal(jt.array(x[:, :1]).broadcast([33, 17]).data, np.broadcast_to(x[:, :1], (33, 17)))
    assert jt.zeros([0, 3]).exp().data.shape == (0, 3)


def test_lazy_graph_recomputes_fused_intermediates(gpu):
    x = np.random.default_rng(19).random(100).astype(np.float32)
    c = jt.array(x) * 3.0
    d = c + 1.0
    assert np.allclose(d.data, x * 3 + 1)
    assert np.allclose(c.data, x * 3)          # c was fused away; asking for it later still works
    s = (jt.array(x).reindex([100, 3], ["i0"]) * 2.0).sum(1)      # element group feeding a reduce
    assert np.allclose(s.data, x * 6, rtol=1e-6)
    h = jt.histc(jt.array(x), 10, 0.0, 1.0).data
    assert np.array_equal(h, np.histogram(x, 10, (0, 1))[0].astype(np.float32))


@pytest.mark.parametrize("shape,perm,dtype,tiled", [
    ((300, 400), (1, 0), "float32", True),
    ((7, 130, 97), (0, 2, 1), "float32", True),                  # ragged tiles in both directions
    ((5, 33, 20, 24), (0, 2, 3, 1), "float32", True),            # NCHW -> NHWC: the two trailing axes move as one
    ((5, 20, 24, 33), (0, 3, 1, 2), "bfloat16", True),           # NHWC -> NCHW, 2-byte elements
    ((40, 3, 50, 64), (2, 1, 0, 3), "float32", False),           # the innermost axis stays: rows move as rows
    ((64, 70, 1, 80), (3, 2, 1, 0), "int32", True),              # full reversal with an axis of extent 1
    ((6, 500, 8), (2, 1, 0), "float64", False),                  # a thin axis becomes innermost: generic kernel
    ((3, 200, 5, 300), (3, 2, 1, 0), "float64", False),          # y's innermost axis has extent 3
    ((30, 200, 5, 70), (3, 2, 1, 0), "float64", True),
    ((2, 3, 40, 50, 60), (0, 4, 2, 1, 3), "int16", True),
])
def test_permute_through_tiles(gpu, shape, perm, dtype, tiled):
    """Axis permutations (every index expression is one output coordinate) bit for bit against numpy.transpose; where
    x's innermost axis does not stay innermost and both tile axes are wide enough they run on the tile kernel."""
    rng = np.random.default_rng(11)
    if dtype == "bfloat16":
        host = O.f32_to_bf16_bits(rng.standard_normal(shape).astype(np.float32))
    elif dtype.startswith("float"):
        host = rng.standard_normal(shape).astype(dtype)
    else:
        host = rng.integers(-30000, 30000, shape).astype(dtype)
    x = jt.from_storage(host, dtype)
    yshape = [shape[a] for a in perm]
    # y[i0..] = x[...] : x's axis perm[j] is indexed by output coordinate j
    idx = [None] * len(shape)
    for j, a in enumerate(perm):
        idx[a] = "i%d" % j
    y = jt.zeros(yshape, dtype)
    tx, ty = L.tensor(x.raw_ptr(), dtype, x.shape), L.tensor(y.raw_ptr(), dtype, y.shape)
    L.check(L.load().mjt_reindex(ctypes.byref(tx), ctypes.byref(ty), len(shape), L.c_strings(idx), 0.0, 0, L.c_strings([]), 0, None))
    assert L.last_kernel().startswith("mjt_permute_") == tiled, L.last_kernel()
    got = L.d2h(y.raw_ptr(), y.shape, L.NP_STORAGE[dtype])
    assert np.array_equal(got, np.transpose(host, perm))


# ---- meta-op convolution ---------------------------------------------------------------------------------
def _bf16(a):
    return O.f32_to_bf16_bits(np.asarray(a, np.float32))


def _conv_call(xbits, wbits, params, out_dtype="float32", in_dtype="bfloat16"):
    import ctypes
    N, C, H, W = xbits.shape
    Kc, _, R, S = wbits.shape
    sh, sw, ph, pw, dh, dw = params
    oh = (H + 2 * ph - dh * (R - 1) - 1) // sh + 1
    ow = (W + 2 * pw - dw * (S - 1) - 1) // sw + 1
    x, w = jt.from_storage(xbits, in_dtype), jt.from_storage(wbits, in_dtype)
    y = jt.zeros([N, Kc, oh, ow], out_dtype)
    tx, tw = L.tensor(x.raw_ptr(), in_dtype, x.shape), L.tensor(w.raw_ptr(), in_dtype, w.shape)
    ty = L.tensor(y.raw_ptr(), out_dtype, y.shape)
    p = L.ConvParams(*params)
    L.check(L.load().mjt_conv2d_meta(ctypes.byref(tx), ctypes.byref(tw), ctypes.byref(ty), ctypes.byref(p)))
    return L.d2h(y.raw_ptr(), y.shape, L.NP_STORAGE[out_dtype]), L.last_kernel()


@pytest.mark.parametrize("case", [
    dict(x=(2, 64, 16, 16), w=(128, 64, 3, 3), p=(1, 1, 1, 1, 1, 1)),      # partial last row tile
    dict(x=(1, 128, 56, 56), w=(128, 128, 3, 3), p=(1, 1, 1, 1, 1, 1)),    # the benchmark geometry, fewer channels
    dict(x=(3, 64, 28, 24), w=(256, 64, 3, 3), p=(2, 2, 1, 1, 1, 1)),      # stride 2
    dict(x=(2, 64, 20, 32), w=(128, 64, 3, 3), p=(1, 1, 2, 2, 2, 2)),      # dilation 2
    dict(x=(2, 192, 14, 8), w=(128, 192, 1, 1), p=(1, 1, 0, 0, 1, 1), nogemm=True),     # 1x1, three channel blocks (kept off the matrix-product route)
    dict(x=(1, 64, 9, 40), w=(128, 64, 5, 3), p=(1, 1, 2, 1, 1, 1)),       # 5x3 taps, odd height
    dict(x=(2, 64, 12, 72), w=(64, 64, 3, 3), p=(1, 1, 1, 1, 1, 1)),       # 72 columns: two staging segments; 64 output channels
    dict(x=(2, 64, 10, 16), w=(128, 64, 3, 3), p=(1, 1, 0, 0, 1, 1)),      # output width 14: 4-byte store epilogue
    dict(x=(6, 64, 35, 16), w=(128, 64, 3, 3), p=(1, 1, 1, 1, 1, 1), rpw=35),   # two full tiles + a short tile whose last row is masked
    dict(x=(5, 64, 30, 16), w=(128, 64, 3, 3), p=(1, 1, 1, 1, 1, 1), rpw=20),   # second row range of an image is cut short
    dict(x=(3, 128, 24, 24), w=(128, 128, 3, 3), p=(1, 1, 1, 1, 1, 1), rpw=24, out="bfloat16"),   # bfloat16 output, several tiles
    dict(x=(3, 64, 28, 28), w=(128, 64, 3, 3), p=(1, 1, 1, 1, 1, 1), out="bfloat16"),   # width 28: the last group of 8 columns is half a group, rows 8-byte aligned
    dict(x=(2, 128, 14, 14), w=(64, 128, 3, 3), p=(1, 1, 1, 1, 1, 1)),      # width 14: 4-byte store epilogue too
    dict(x=(2, 64, 28, 28), w=(64, 64, 3, 3), p=(2, 2, 1, 1, 1, 1)),        # width 28, stride 2: output width 14
    dict(x=(2, 64, 9, 12), w=(64, 64, 1, 1), p=(1, 1, 0, 0, 1, 1)),         # width 12, 1x1: the last image row ends at the tensor's end
    dict(x=(1, 64, 11, 70), w=(64, 64, 3, 3), p=(1, 1, 1, 1, 1, 1)),        # 70 columns: a second staging segment of 6
    dict(x=(3, 64, 6, 6), w=(64, 64, 3, 3), p=(1, 1, 1, 1, 1, 1)),          # rows shorter than one group of 8 columns
    dict(x=(2, 64, 5, 2), w=(64, 64, 1, 1), p=(1, 1, 0, 0, 1, 1)),          # two columns: a load spans four rows
    dict(x=(2, 96, 12, 16), w=(64, 96, 3, 3), p=(1, 1, 1, 1, 1, 1)),        # 96 channels: three blocks of 32
    dict(x=(1, 64, 30, 112), w=(64, 64, 3, 3), p=(1, 1, 1, 1, 1, 1)),       # wide rows: one output row per wave, a short weight ring
    dict(x=(2, 64, 16, 16), w=(32, 64, 3, 3), p=(1, 1, 1, 1, 1, 1)),        # 32 output channels: workgroups of two waves that stage 32 items each, two channel blocks
    dict(x=(2, 128, 40, 16), w=(32, 128, 3, 3), p=(1, 1, 1, 1, 1, 1), rpw=40, out="bfloat16"),   # the same with two full tiles and a short one per workgroup, four blocks
    dict(x=(2, 64, 31, 10), w=(32, 64, 3, 3), p=(2, 2, 1, 1, 1, 1)),        # 32 output channels, stride 2, odd height
])
def test_conv_mfma_matches_oracle(gpu, case):
    from oracle import kernels as K
    rng = np.random.default_rng(20)
    xb = _bf16(rng.standard_normal(case["x"]))
    wb = _bf16(rng.standard_normal(case["w"]) * 0.05)
    sh, sw, ph, pw, dh, dw = case["p"]
    if "rpw" in case:
        os.environ["MJT_CONV_RPW"] = str(case["rpw"])      # rows per workgroup, forced: the heuristic would pick it only for large batches
    if case.get("nogemm"):
        os.environ["MJT_CONV_NO_GEMM"] = "1"
    try:
        got, kern = _conv_call(xb, wb, case["p"])
        if "out" in case:                                  # narrower output = truncation of the same accumulators
            got16, kern16 = _conv_call(xb, wb, case["p"], out_dtype=case["out"])
            assert kern16.startswith("mjt_conv_mfma_bf16") and np.array_equal(got16, O.f32_to_bf16_bits(got))
    finally:
        os.environ.pop("MJT_CONV_RPW", None)
        os.environ.pop("MJT_CONV_NO_GEMM", None)
    assert kern.startswith("mjt_conv_mfma_bf16"), kern
    if sh == sw and ph == pw and dh == dw:
        ref = K.conv_meta_bf16(xb, wb, sh, ph, dh, 8)
    else:
        ref = None
    xf, wf = O.BF16(xb).to_f32().astype(np.float64), O.BF16(wb).to_f32().astype(np.float64)
    R, S = wf.shape[2], wf.shape[3]
    oh, ow = got.shape[2], got.shape[3]
    xp = np.pad(xf, ((0, 0), (0, 0), (ph, ph), (pw, pw)))
    ref64, terms = np.zeros(got.shape), np.zeros(got.shape)      # the float64 result and the sum of |x * w| per output
    for r in range(R):
        for s in range(S):
            patch = xp[:, :, r * dh:r * dh + (oh - 1) * sh + 1:sh, s * dw:s * dw + (ow - 1) * sw + 1:sw]
            ref64 += np.einsum("nchw,kc->nkhw", patch, wf[:, :, r, s])
            terms += np.einsum("nchw,kc->nkhw", np.abs(patch), np.abs(wf[:, :, r, s]))
    if ref is None:
        ref = ref64
    # fp32 accumulation in a different order than the reference's (c, kh, kw) loop: every element within 1e-4 of
    # the sum of the magnitudes of its terms, against the float64 result and against the oracle's own fp32 loop
    bound = 1e-4 * terms + 1e-30
    assert (np.abs(got - ref64) <= bound).all(), float((np.abs(got - ref64) / bound).max())
    assert (np.abs(got - ref) <= 2 * bound).all(), float((np.abs(got - ref) / bound).max())
    scale = np.abs(ref).max()
    # the direct kernel follows the reference's loop order exactly
    os.environ["MJT_NO_FASTPATH"] = "1"
    try:
        got2, kern2 = _conv_call(xb, wb, case["p"])
    finally:
        del os.environ["MJT_NO_FASTPATH"]
    assert kern2.startswith("mjt_conv_direct")
    assert np.abs(got2 - ref).max() <= 1e-4 * scale


def test_conv_packed_weights_entry(gpu):
    """mjt_conv2d_meta_pack + mjt_conv2d_meta_packed (weights rearranged once, several calls on them) give the bits
    of mjt_conv2d_meta, which test_conv_mfma_matches_oracle holds against the oracle; the weights' own buffer may
    change after packing without effect; a convolution that takes another route is refused."""
    import ctypes
    lib = L.load()
    rng = np.random.default_rng(21)
    for xs, ws, params, out in (((3, 64, 28, 24), (256, 64, 3, 3), (2, 2, 1, 1, 1, 1), "float32"),
                                ((2, 128, 24, 24), (128, 128, 3, 3), (1, 1, 1, 1, 1, 1), "bfloat16")):
        wb = _bf16(rng.standard_normal(ws) * 0.05)
        w = jt.from_storage(wb, "bfloat16")
        packed = jt.zeros([int(np.prod(ws))], "bfloat16")
        p = L.ConvParams(*params)
        for trial in range(2):                              # two inputs on the same packed weights
            xb = _bf16(rng.standard_normal(xs))
            want, kern = _conv_call(xb, wb, params, out_dtype=out)
            assert kern.startswith("mjt_conv_mfma_bf16")
            x = jt.from_storage(xb, "bfloat16")
            y = jt.zeros(list(want.shape), out)
            tx, tw = L.tensor(x.raw_ptr(), "bfloat16", x.shape), L.tensor(w.raw_ptr(), "bfloat16", w.shape)
            ty = L.tensor(y.raw_ptr(), out, y.shape)
            if trial == 0:
                L.check(lib.mjt_conv2d_meta_pack(ctypes.byref(tx), ctypes.byref(tw), ctypes.byref(ty), ctypes.byref(p),
                                                 packed.raw_ptr(), int(np.prod(ws)) * 2))
                assert L.last_kernel().endswith("_pack")
                L.check(lib.mjt_fill_u32(w.raw_ptr(), 0x7fc07fc0, int(np.prod(ws)) // 2))      # w itself is not read any more
            L.check(lib.mjt_conv2d_meta_packed(ctypes.byref(tx), ctypes.byref(tw), packed.raw_ptr(), ctypes.byref(ty), ctypes.byref(p)))
            assert L.last_kernel() == kern
            got = L.d2h(y.raw_ptr(), y.shape, L.NP_STORAGE[out])
            assert np.array_equal(got.view(np.uint8), want.view(np.uint8)), (xs, trial)
    # float32 takes another route: no packed form
    x, w = jt.array(rng.standard_normal((1, 8, 6, 6)).astype(np.float32)), jt.array(rng.standard_normal((4, 8, 3, 3)).astype(np.float32))
    y, buf = jt.zeros([1, 4, 6, 6], "float32"), jt.zeros([4 * 8 * 9], "float32")
    tx, tw, ty = (L.tensor(v.raw_ptr(), "float32", v.shape) for v in (x, w, y))
    p = L.ConvParams(1, 1, 1, 1, 1, 1)
    assert lib.mjt_conv2d_meta_pack(ctypes.byref(tx), ctypes.byref(tw), ctypes.byref(ty), ctypes.byref(p), buf.raw_ptr(), 4 * 8 * 9 * 4) == -2
    assert lib.mjt_conv2d_meta_packed(ctypes.byref(tx), ctypes.byref(tw), buf.raw_ptr(), ctypes.byref(ty), ctypes.byref(p)) == -2


@pytest.mark.parametrize("seed,ks,at_least", [(77, [64, 128, 192], 8), (78, [32, 32, 64], 8)])
def test_conv_mfma_random_geometries(gpu, seed, ks, at_least):
    """Seeded sweep over geometries for the MFMA kernel (channel counts, map sizes with even widths, taps, stride,
    padding, dilation, 16-bit and float32 results): every case against a float64 sum of shifted products, per
    element within 1e-4 of the sum of its terms' magnitudes (plus the result type's own rounding).  The second sweep
    is mostly on 32 output channels (workgroups of two waves, each staging twice the input rows)."""
    rng = np.random.default_rng(seed)
    taken = 0
    for i in range(14):
        C, K = int(rng.choice([32, 64, 96, 128])), int(rng.choice(ks))
        R, S = int(rng.choice([1, 2, 3])), int(rng.choice([1, 3, 5]))
        sh, sw = int(rng.choice([1, 1, 2])), int(rng.choice([1, 1, 2]))
        dh, dw_ = int(rng.choice([1, 1, 2])), int(rng.choice([1, 1, 2]))
        ph, pw = int(rng.integers(0, 3)), int(rng.integers(0, 3))
        H, W = int(rng.integers(4, 30)), 2 * int(rng.integers(3, 40))
        N = int(rng.integers(1, 4))
        if H + 2 * ph < dh * (R - 1) + 1 or W + 2 * pw < dw_ * (S - 1) + 1:
            continue
        out = ("float32", "bfloat16")[i % 2]
        xb = O.f32_to_bf16_bits(rng.standard_normal((N, C, H, W)).astype(np.float32))
        wb = O.f32_to_bf16_bits((rng.standard_normal((K, C, R, S)) * 0.1).astype(np.float32))
        got, kern = _conv_call(xb, wb, (sh, sw, ph, pw, dh, dw_), out_dtype=out)
        taken += kern.startswith("mjt_conv_mfma_bf16")
        got = O.BF16(got).to_f32().astype(np.float64) if out == "bfloat16" else got.astype(np.float64)
        xf, wf = O.BF16(xb).to_f32().astype(np.float64), O.BF16(wb).to_f32().astype(np.float64)
        oh, ow = got.shape[2:]
        xp = np.pad(xf, ((0, 0), (0, 0), (ph, ph), (pw, pw)))
        ref, terms = np.zeros(got.shape), np.zeros(got.shape)
        for r in range(R):
            for s_ in range(S):
                patch = xp[:, :, r * dh:r * dh + (oh - 1) * sh + 1:sh, s_ * dw_:s_ * dw_ + (ow - 1) * sw + 1:sw]
                ref += np.einsum("nchw,kc->nkhw", patch, wf[:, :, r, s_])
                terms += np.einsum("nchw,kc->nkhw", np.abs(patch), np.abs(wf[:, :, r, s_]))
        bound = 1e-4 * terms + (np.abs(ref) * 2.0 ** -7 if out == "bfloat16" else 0.0) + 1e-30
        assert (np.abs(got - ref) <= bound).all(), (kern, (N, C, H, W), (K, C, R, S), (sh, sw, ph, pw, dh, dw_),
                                                    float((np.abs(got - ref) / bound).max()))
    assert taken >= at_least, taken   # most of the sweep runs on the MFMA kernel (the rest on the fallbacks, checked alike)


def _dgrad_reference(dy, w, H, W, params):
    """The definition, in float64: every product dy[n,k,oh,ow] * w[k,c,r,s] is added at the input position the forward
    window read (also returns the sum of the products' magnitudes, for the bound)."""
    sh, sw, ph, pw, dh, dw_ = params
    N, K, OH, OW = dy.shape
    C, R, S = w.shape[1:]
    dx, mag = np.zeros((N, C, H + 2 * ph, W + 2 * pw)), np.zeros((N, C, H + 2 * ph, W + 2 * pw))
    for r in range(R):
        for s_ in range(S):
            rows, cols = slice(r * dh, r * dh + (OH - 1) * sh + 1, sh), slice(s_ * dw_, s_ * dw_ + (OW - 1) * sw + 1, sw)
            dx[:, :, rows, cols] += np.einsum("nkhw,kc->nchw", dy, w[:, :, r, s_])
            mag[:, :, rows, cols] += np.einsum("nkhw,kc->nchw", np.abs(dy), np.abs(w[:, :, r, s_]))
    return dx[:, :, ph:ph + H, pw:pw + W], mag[:, :, ph:ph + H, pw:pw + W]


@pytest.mark.parametrize("case", [
    # x shape,         w shape,          (sh, sw, ph, pw, dh, dw), dtype,     result,    by phases
    ((2, 8, 10, 12), (6, 8, 3, 3), (1, 1, 1, 1, 1, 1), "float32", "float32", False),
    ((2, 8, 10, 12), (6, 8, 3, 3), (2, 2, 1, 1, 1, 1), "float32", "float32", True),
    ((2, 8, 10, 12), (6, 8, 1, 1), (2, 2, 0, 0, 1, 1), "float32", "float32", True),      # phases no tap reaches: zeros
    ((1, 4, 12, 12), (5, 4, 5, 5), (2, 2, 2, 2, 1, 1), "float32", "float32", True),
    ((1, 4, 12, 9), (5, 4, 3, 3), (2, 3, 1, 0, 1, 1), "float32", "float32", True),
    ((1, 4, 12, 12), (5, 4, 5, 3), (3, 2, 2, 1, 1, 1), "float32", "float32", True),
    ((1, 4, 12, 12), (5, 4, 3, 2), (3, 2, 1, 1, 1, 1), "float32", "float32", False),     # a phase that starts past dy's first row
    ((1, 4, 13, 12), (5, 4, 3, 3), (2, 2, 1, 1, 1, 1), "float32", "float32", False),     # 13 rows: dy spread out with zeros
    ((1, 4, 12, 12), (5, 4, 3, 3), (2, 2, 2, 2, 2, 2), "float32", "float32", False),     # dilation: likewise
    ((2, 64, 28, 28), (64, 64, 3, 3), (2, 2, 1, 1, 1, 1), "bfloat16", "bfloat16", True), # each phase on the MFMA kernel
    ((2, 64, 28, 28), (128, 64, 3, 3), (2, 2, 1, 1, 1, 1), "float16", "float32", True),
    ((2, 64, 28, 28), (64, 64, 3, 3), (1, 1, 1, 1, 1, 1), "bfloat16", "float32", False),
], ids=lambda c: "x%s_w%s_p%s_%s" % ("x".join(map(str, c[0])), "x".join(map(str, c[1])), "".join(map(str, c[2])), c[3]))
def test_conv_input_gradient_entry(gpu, case):
    """mjt_conv2d_meta_dgrad against the definition of the gradient in float64 (per element within 1e-4 of the sum of
    its terms' magnitudes, plus the result type's rounding), and for float32 against the oracle's gradient graph."""
    xshape, wshape, params, dtype, out_dtype, phased = case
    sh, sw, ph, pw, dh, dw_ = params
    N, C, H, W = xshape
    K, _, R, S = wshape
    OH, OW = (H + 2 * ph - dh * (R - 1) - 1) // sh + 1, (W + 2 * pw - dw_ * (S - 1) - 1) // sw + 1
    rng = np.random.default_rng(5)
    dyf = rng.standard_normal((N, K, OH, OW)).astype(np.float32)
    wf = (rng.standard_normal(wshape) * 0.2).astype(np.float32)
    if dtype == "bfloat16":
        dyb, wb = O.f32_to_bf16_bits(dyf), O.f32_to_bf16_bits(wf)
        dyf, wf = O.BF16(dyb).to_f32(), O.BF16(wb).to_f32()
    elif dtype == "float16":
        dyb, wb = dyf.astype(np.float16), wf.astype(np.float16)
        dyf, wf = dyb.astype(np.float32), wb.astype(np.float32)
    else:
        dyb, wb = dyf, wf
    dy, w = jt.from_storage(np.ascontiguousarray(dyb), dtype), jt.from_storage(np.ascontiguousarray(wb), dtype)
    dx = jt.zeros(list(xshape), out_dtype)
    td, tw = L.tensor(dy.raw_ptr(), dtype, dy.shape), L.tensor(w.raw_ptr(), dtype, w.shape)
    tx = L.tensor(dx.raw_ptr(), out_dtype, dx.shape)
    p = L.ConvParams(*params)
    L.check(L.load().mjt_conv2d_meta_dgrad(ctypes.byref(td), ctypes.byref(tw), ctypes.byref(tx), ctypes.byref(p)))
    kern = L.last_kernel()
    assert kern.startswith("conv_dgrad_phases:") == phased, kern
    if dtype != "float32" and phased:
        assert "mjt_conv_mfma" in kern, kern
    raw = L.d2h(dx.raw_ptr(), dx.shape, L.NP_STORAGE[out_dtype])
    got = (O.BF16(raw).to_f32() if out_dtype == "bfloat16" else raw).astype(np.float64)
    ref, mag = _dgrad_reference(dyf.astype(np.float64), wf.astype(np.float64), H, W, params)
    rounding = {"float32": 0.0, "bfloat16": 2.0 ** -7, "float16": 2.0 ** -10}[out_dtype]
    bound = 1e-4 * mag + np.abs(ref) * rounding + 1e-30
    assert (np.abs(got - ref) <= bound).all(), (kern, float((np.abs(got - ref) / bound).max()))
    # the oracle's restatement of the gradient graph jt.grad builds (sequential float32 sums; small cases only)
    if dtype == "float32":
        odx, _ = O.conv_meta_grouped_grads(np.zeros(xshape, np.float32), wf, dyf, 1, (sh, sw), (ph, pw), (dh, dw_))
        assert (np.abs(got - odx.astype(np.float64)) <= bound).all()


def test_conv_direct_small_shapes_and_fp32(gpu):
    rng = np.random.default_rng(21)
    for xs, ws, st, pd, dl in [((2, 3, 9, 8), (4, 3, 3, 3), 1, 1, 1), ((2, 3, 9, 8), (4, 3, 3, 3), 2, 1, 1),
                               ((1, 5, 11, 7), (2, 5, 3, 3), 1, 2, 2), ((1, 2, 6, 6), (3, 2, 1, 1), 1, 0, 1)]:
        x = rng.standard_normal(xs).astype(np.float32)
        w = rng.standard_normal(ws).astype(np.float32)
        got, kern = _conv_call(x, w, (st, st, pd, pd, dl, dl), in_dtype="float32")
        assert kern.startswith("mjt_conv_direct_float32")
        assert np.allclose(got, O.conv_meta(x, w, st, pd, dl), rtol=1e-5, atol=1e-5)
        got, _ = _conv_call(_bf16(x), _bf16(w), (st, st, pd, pd, dl, dl))
        assert np.allclose(got, O.conv_meta(O.BF16(_bf16(x)), O.BF16(_bf16(w)), st, pd, dl), rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("case", [
    dict(dt="float32", x=(4, 32, 28, 28), w=(48, 32, 3, 3), p=(1, 1, 1, 1, 1, 1)),
    dict(dt="float32", x=(3, 16, 30, 27), w=(48, 16, 3, 2), p=(2, 1, 1, 0, 1, 2), chunk=2),       # chunks of 2 + 1 images
    dict(dt="bfloat16", x=(2, 64, 27, 27), w=(128, 64, 3, 3), p=(2, 2, 1, 1, 1, 1), out="bfloat16"),   # odd width
    dict(dt="bfloat16", x=(2, 48, 14, 14), w=(64, 48, 3, 3), p=(1, 1, 1, 1, 1, 1)),                     # channels no multiple of 64
    dict(dt="float16", x=(4, 64, 14, 14), w=(96, 64, 1, 1), p=(1, 1, 0, 0, 1, 1), out="float16"),   # 196 pixels: rows of 392 bytes are padded
    dict(dt="float16", x=(4, 64, 16, 16), w=(96, 64, 1, 1), p=(1, 1, 0, 0, 1, 1), out="float16", plain=True),
    dict(dt="float32", x=(12, 24, 7, 7), w=(40, 24, 3, 3), p=(1, 1, 1, 1, 1, 1)),                      # 49 pixels: padded rows, k ends inside a stage
    dict(dt="bfloat16", x=(3, 72, 9, 11), w=(40, 72, 3, 3), p=(1, 1, 1, 1, 1, 1), out="bfloat16"),
    dict(dt="float32", x=(5, 40, 16, 16), w=(96, 40, 1, 1), p=(1, 1, 0, 0, 1, 1), plain=True, chunk=2),
    dict(dt="float32", x=(8, 3, 64, 64), w=(32, 3, 7, 7), p=(2, 2, 3, 3, 1, 1)),      # a stem: weight rows of 588 bytes are padded to 16-byte multiples
    dict(dt="float32", x=(8, 3, 64, 64), w=(32, 3, 7, 7), p=(2, 2, 3, 3, 1, 1), cols=True),      # the same through column matrices
    dict(dt="float32", x=(4, 32, 28, 28), w=(48, 32, 3, 3), p=(1, 1, 1, 1, 1, 1), cols=True),
    dict(dt="bfloat16", x=(2, 64, 27, 27), w=(128, 64, 3, 3), p=(2, 2, 1, 1, 1, 1), out="bfloat16", cols=True),
    dict(dt="float16", x=(4, 64, 14, 14), w=(96, 64, 1, 1), p=(1, 1, 0, 0, 1, 1), out="float16", cols=True),
    dict(dt="bfloat16", x=(3, 40, 13, 9), w=(72, 40, 5, 3), p=(1, 1, 2, 1, 1, 1)),                 # 40 channels, 13 x 9 maps, 5 x 3 taps: weight rows of 1200 bytes
    dict(dt="float16", x=(2, 16, 10, 130), w=(24, 16, 3, 3), p=(1, 1, 1, 1, 1, 1), out="float16"),   # rows of 130 outputs
    dict(dt="float32", x=(3, 80, 19, 23), w=(136, 80, 3, 3), p=(1, 2, 2, 0, 2, 1)),                 # 136 output channels: two row tiles, the second mostly empty; mixed strides
    dict(dt="float32", x=(70, 16, 7, 7), w=(24, 16, 3, 3), p=(1, 1, 1, 1, 1, 1)),                    # 7 x 7 maps: a tile of pixels spans several images
    dict(dt="float32", x=(2, 8, 40, 130), w=(16, 8, 1, 5), p=(1, 1, 0, 2, 1, 1)),                    # wide rows, taps along the row only
    # 16-bit with more than 64 output channels and enough tiles: 128 x 64 tiles (200 and 136 rows: part-filled row tiles)
    dict(dt="bfloat16", x=(50, 32, 13, 13), w=(200, 32, 3, 3), p=(1, 1, 1, 1, 1, 1), out="bfloat16", tile="128x64"),
    dict(dt="float16", x=(80, 24, 15, 17), w=(136, 24, 3, 3), p=(2, 1, 1, 1, 1, 1), tile="128x64"),
    # float32 with more than 64 output channels and enough tiles: 128 x 128 tiles (72 rows: a part-filled row tile)
    dict(dt="float32", x=(42, 8, 28, 28), w=(72, 8, 3, 3), p=(1, 1, 1, 1, 1, 1), tile="128x128"),
    # 16-bit with a long sum and few tiles: stays on the column matrices
    dict(dt="bfloat16", x=(2, 128, 7, 7), w=(128, 128, 3, 3), p=(1, 1, 1, 1, 1, 1), stays=True),
    # small maps with long sums and many output channels: one product for the whole batch on column matrices with the
    # images side by side, then a permutation (by the rule; asked for by name with strides, dilation and a float32 result)
    dict(dt="bfloat16", x=(48, 64, 7, 7), w=(512, 64, 3, 3), p=(1, 1, 1, 1, 1, 1), out="bfloat16", batch=True),
    dict(dt="float16", x=(48, 512, 7, 7), w=(512, 512, 1, 1), p=(1, 1, 0, 0, 1, 1), batch=True),
    dict(dt="bfloat16", x=(16, 32, 12, 10), w=(40, 32, 3, 3), p=(2, 1, 1, 0, 1, 2), batch=True, flat="1"),
    dict(dt="bfloat16", x=(48, 64, 7, 7), w=(512, 64, 3, 3), p=(1, 1, 1, 1, 1, 1), out="bfloat16", flat="0"),
    # the product on the direct-copy kernel (asked for by name: these shapes have too few tiles to get it by themselves):
    # weights shared across the batch, column matrices with the pixels innermost read with transposing reads
    dict(dt="bfloat16", x=(3, 64, 15, 15), w=(96, 64, 3, 3), p=(1, 1, 1, 1, 1, 1), dma=True, cols=True),
    dict(dt="float16", x=(4, 64, 16, 16), w=(96, 64, 1, 1), p=(1, 1, 0, 0, 1, 1), out="float16", plain=True, dma=True),
])
def test_conv_as_reindex_and_gemm(gpu, case, monkeypatch):
    """Shapes the MFMA kernel does not take and that are large enough to matter run as column matrices (one reindex)
    times the weights (the GEMM kernel, float32 accumulation): against a float64 closed form and, for float32, the
    oracle's own summation order; a bfloat16 result is truncated like everywhere else, a float16 one rounded."""
    rng = np.random.default_rng(41)
    dt = case["dt"]
    sh, sw, ph, pw, dh, dw_ = case["p"]
    narrow = {"float32": lambda a: a.astype(np.float32), "bfloat16": _bf16, "float16": lambda a: a.astype(np.float16)}[dt]
    widen = {"float32": lambda a: a, "bfloat16": lambda a: O.BF16(a).to_f32(), "float16": lambda a: a.astype(np.float32)}
    xb, wb = narrow(rng.standard_normal(case["x"])), narrow(rng.standard_normal(case["w"]) * 0.1)
    out = case.get("out", "float32")
    if "chunk" in case:
        monkeypatch.setenv("MJT_CONV_GEMM_CHUNK", str(case["chunk"]))
    if case.get("dma"):
        monkeypatch.setenv("MJT_GEMM_DMA", "1")
    if case.get("cols"):
        monkeypatch.setenv("MJT_CONV_NO_IGEMM", "1")
    if "flat" in case:
        monkeypatch.setenv("MJT_CONV_FLAT", case["flat"])
    got, kern = _conv_call(xb, wb, case["p"], out_dtype=out, in_dtype=dt)
    if case.get("batch"):
        assert kern == "conv_as_batch_gemm", kern
    elif not case.get("plain") and not case.get("cols") and not case.get("dma") and not case.get("stays"):
        assert kern.startswith("mjt_conv_igemm_" + dt), kern        # the product kernel gathers its operand from x itself
        assert kern.endswith(case.get("tile", "64x64")), kern
    else:
        assert kern == ("conv_as_gemm" if case.get("plain") else "conv_as_reindex_gemm"), kern
    got = widen[out](got)
    xf, wf = widen[dt](xb).astype(np.float64), widen[dt](wb).astype(np.float64)
    K, _, R, S = wf.shape
    oh, ow = got.shape[2:]
    xp = np.pad(xf, ((0, 0), (0, 0), (ph, ph), (pw, pw)))
    ref = np.zeros(got.shape)
    for r in range(R):
        for s in range(S):
            patch = xp[:, :, r * dh:r * dh + (oh - 1) * sh + 1:sh, s * dw_:s * dw_ + (ow - 1) * sw + 1:sw]
            ref += np.einsum("nchw,kc->nkhw", patch, wf[:, :, r, s])
    tol = {"float32": 1e-4, "bfloat16": 2.0 ** -7, "float16": 2.0 ** -10}[out]
    assert np.abs(got - ref).max() <= tol * np.abs(ref).max()
    if out == "bfloat16":                                    # truncated, never rounded up in magnitude
        assert np.all(np.abs(got) <= np.abs(ref) + 1e-5 * np.abs(ref).max())
    if dt == "float32" and sh == sw and ph == pw and dh == dw_:
        assert np.abs(got - O.conv_meta(xb, wb, sh, ph, dh)).max() <= 1e-4 * np.abs(ref).max()
    # the same call with that path off: the direct kernel, same values to the same bound
    monkeypatch.setenv("MJT_CONV_NO_GEMM", "1")
    got2, kern2 = _conv_call(xb, wb, case["p"], out_dtype=out, in_dtype=dt)
    assert kern2.startswith("mjt_conv_direct")
    assert np.abs(widen[out](got2) - ref).max() <= tol * np.abs(ref).max()


def test_conv_1x1_runs_as_a_product(gpu, monkeypatch):
    """A 1x1 convolution of stride 1 is handed to the matrix-product kernel although the MFMA convolution kernel would
    take it: always when a plane's rows are 16-byte multiples (the product then reads x as it lies, with tiles picked for
    a short sum); with other plane sizes the product kernel gathers x itself, when the input channels outnumber the output
    channels 4 : 1 or more with at most 64 output channels or a map of at most 256 pixels, or when there are more than 64
    output channels and enough 128 x 64 tiles for every compute unit.  Both kernels against a float64 product, same
    bound; 16-bit and float32 results."""
    rng = np.random.default_rng(43)
    for xs, ws, out, want in (((2, 256, 16, 16), (64, 256, 1, 1), "float32", "conv_as_gemm"),
                              ((3, 512, 14, 14), (128, 512, 1, 1), "float32", "mjt_conv_igemm_bfloat16_of32"),
                              ((48, 128, 14, 14), (256, 128, 1, 1), "bfloat16", "mjt_conv_igemm_bfloat16_c128_k256_14x14_r1x1_s1x1_p0x0_d1x1_128x64"),
                              ((20, 128, 14, 14), (256, 128, 1, 1), "bfloat16", "mjt_conv_mfma_bf16"),   # too few tiles: stays
                              ((3, 64, 24, 28), (256, 64, 1, 1), "bfloat16", "conv_as_gemm"),        # one step of the sum, tiles of 128
                              ((5, 128, 12, 20), (192, 128, 1, 1), "float32", "conv_as_gemm"),       # 240 pixels, 192 channels: edge tiles
                              ((2, 1024, 8, 8), (128, 1024, 1, 1), "bfloat16", "conv_as_gemm"),      # 64 pixels: narrow tiles
                              ((70, 64, 16, 16), (192, 64, 1, 1), "bfloat16", "conv_as_gemm"),       # more tiles than compute units
                              ((2, 64, 9, 12), (64, 64, 1, 1), "float32", "mjt_conv_mfma_bf16")):    # rows of 216 bytes: stays
        xb, wb = _bf16(rng.standard_normal(xs)), _bf16(rng.standard_normal(ws) * 0.1)
        ref = np.einsum("nchw,kc->nkhw", O.BF16(xb).to_f32().astype(np.float64), O.BF16(wb).to_f32().astype(np.float64)[:, :, 0, 0])
        mag = np.einsum("nchw,kc->nkhw", np.abs(O.BF16(xb).to_f32().astype(np.float64)), np.abs(O.BF16(wb).to_f32().astype(np.float64))[:, :, 0, 0])
        widen = (lambda a: O.BF16(a).to_f32().astype(np.float64)) if out == "bfloat16" else (lambda a: a.astype(np.float64))
        bound = 1e-4 * mag + (np.abs(ref) * 2.0 ** -7 if out == "bfloat16" else 0.0) + 1e-30
        got, kern = _conv_call(xb, wb, (1, 1, 0, 0, 1, 1), out_dtype=out)
        assert kern.startswith(want), (kern, xs)
        assert (np.abs(widen(got) - ref) <= bound).all(), (xs, ws)
        monkeypatch.setenv("MJT_CONV_NO_GEMM", "1")
        got2, kern2 = _conv_call(xb, wb, (1, 1, 0, 0, 1, 1), out_dtype=out)
        monkeypatch.delenv("MJT_CONV_NO_GEMM")
        assert kern2.startswith("mjt_conv_mfma_bf16"), kern2
        assert (np.abs(widen(got2) - ref) <= bound).all(), (xs, ws)


def test_conv_grouped_entry_and_front_end(gpu):
    """Grouped convolution (python/jittor/nn.py:1272-1294): the C entry point against the oracle's 8-d
    restatement, then nn.conv2d(groups=G) matched by the executor (one kernel, nothing of rank 8 in memory)
    and, with the matcher off, through the generic reindex / reindex_reduce kernels."""
    rng = np.random.default_rng(23)
    for xs, ws, G, st, pd, dl in [((2, 6, 9, 8), (4, 3, 3, 3), 2, 1, 1, 1), ((1, 8, 10, 10), (8, 1, 3, 3), 8, 2, 1, 1),
                                  ((2, 6, 7, 9), (9, 2, 3, 3), 3, 1, 2, 2)]:
        x = rng.standard_normal(xs).astype(np.float32)
        w = rng.standard_normal(ws).astype(np.float32)
        want = O.conv_meta_grouped(x, w, G, st, pd, dl)
        lib = L.load()
        vx, vw, vy = jt.from_storage(x, "float32"), jt.from_storage(w, "float32"), jt.zeros(list(want.shape), "float32")
        tx, tw = L.tensor(vx.raw_ptr(), "float32", vx.shape), L.tensor(vw.raw_ptr(), "float32", vw.shape)
        ty = L.tensor(vy.raw_ptr(), "float32", vy.shape)
        p = L.ConvParams(st, st, pd, pd, dl, dl)
        L.check(lib.mjt_conv2d_meta_grouped(ctypes.byref(tx), ctypes.byref(tw), ctypes.byref(ty), ctypes.byref(p), G))
        assert L.last_kernel().endswith("_g%d" % G)
        assert np.allclose(L.d2h(vy.raw_ptr(), vy.shape, np.float32), want, rtol=1e-5, atol=1e-5)
        before = jt.executor_stats["conv_matches"]
        v = jt.nn.conv2d(jt.array(x), jt.array(w), stride=st, padding=pd, dilation=dl, groups=G)
        got = v.data
        assert jt.executor_stats["conv_matches"] == before + 1 and L.last_kernel().endswith("_g%d" % G)
        assert np.allclose(got, want, rtol=1e-5, atol=1e-5)
        jt.flags["enable_conv_match"] = False
        try:
            got = jt.nn.conv2d(jt.array(x), jt.array(w), stride=st, padding=pd, dilation=dl, groups=G).data
        finally:
            jt.flags["enable_conv_match"] = True
        assert np.allclose(got, want, rtol=1e-4, atol=1e-4)          # scatter-add: order differs
    # wrong group count: an error, not a fault
    rc = lib.mjt_conv2d_meta_grouped(ctypes.byref(tx), ctypes.byref(tw), ctypes.byref(ty), ctypes.byref(p), 2)
    assert rc < 0 and "group" in lib.mjt_last_error().decode()
    with pytest.raises(ValueError):
        jt.nn.conv2d(jt.array(x), jt.array(w), groups=4)


@pytest.mark.parametrize("xs,ws,G,params,out", [
    ((2, 128, 12, 16), (256, 64, 3, 3), 2, (1, 1, 1, 1, 1, 1), "float32"),      # two groups of 64 -> 128 channels
    ((3, 128, 9, 24), (256, 32, 3, 3), 4, (1, 1, 1, 1, 1, 1), "bfloat16"),      # four groups of 32 -> 64, 16-bit result
    ((2, 192, 10, 12), (192, 64, 1, 1), 3, (2, 2, 0, 0, 1, 1), "float32"),      # 1x1 stride 2, three groups
    ((2, 128, 12, 16), (128, 32, 3, 3), 4, (1, 1, 1, 1, 1, 1), "float32"),      # four groups of 32 -> 32: workgroups of two waves, 16 channels each
    ((3, 256, 14, 14), (256, 32, 3, 3), 8, (2, 2, 1, 1, 1, 1), "bfloat16"),     # eight groups of 32 -> 32, stride 2
])
def test_conv_grouped_on_the_mfma_kernel(gpu, xs, ws, G, params, out):
    """Groups of at least 32 input and 32 output channels run on the MFMA kernel, all groups in one launch, each on its own
    channels (python/jittor/nn.py:1272-1294): against the oracle's grouped convolution of the exact 16-bit operands,
    per element within 1e-4 of the sum of its terms' magnitudes."""
    rng = np.random.default_rng(41)
    xb = O.f32_to_bf16_bits(rng.standard_normal(xs).astype(np.float32))
    wb = O.f32_to_bf16_bits((rng.standard_normal(ws) * 0.1).astype(np.float32))
    xf, wf = O.BF16(xb).to_f32(), O.BF16(wb).to_f32()
    sh, sw, ph, pw, dh, dw = params
    want = O.conv_meta_grouped(xf, wf, G, sh, ph, dh)
    terms = O.conv_meta_grouped(np.abs(xf), np.abs(wf), G, sh, ph, dh)
    x, w = jt.from_storage(xb, "bfloat16"), jt.from_storage(wb, "bfloat16")
    y = jt.zeros(list(want.shape), out)
    tx, tw, ty = L.tensor(x.raw_ptr(), "bfloat16", x.shape), L.tensor(w.raw_ptr(), "bfloat16", w.shape), L.tensor(y.raw_ptr(), out, y.shape)
    p = L.ConvParams(*params)
    L.check(L.load().mjt_conv2d_meta_grouped(ctypes.byref(tx), ctypes.byref(tw), ctypes.byref(ty), ctypes.byref(p), G))
    kern = L.last_kernel()
    assert kern.startswith("mjt_conv_mfma_bf16") and "_g%d_" % G in kern, kern
    got = L.d2h(y.raw_ptr(), y.shape, L.NP_STORAGE[out])
    got = O.BF16(got).to_f32().astype(np.float64) if out == "bfloat16" else got.astype(np.float64)
    bound = 1e-4 * terms + (np.abs(want) * 2.0 ** -7 if out == "bfloat16" else 0.0)
    assert (np.abs(got - want) <= bound).all(), float((np.abs(got - want) / np.maximum(bound, 1e-30)).max())


def _wgrad_call(xbits, dybits, R, S, params, out_dtype="float32", in_dtype="bfloat16"):
    x, dy = jt.from_storage(xbits, in_dtype), jt.from_storage(dybits, in_dtype)
    dw = jt.zeros([dybits.shape[1], xbits.shape[1], R, S], out_dtype)
    tx, td = L.tensor(x.raw_ptr(), in_dtype, x.shape), L.tensor(dy.raw_ptr(), in_dtype, dy.shape)
    tw = L.tensor(dw.raw_ptr(), out_dtype, dw.shape)
    p = L.ConvParams(*params)
    rc = L.load().mjt_conv2d_meta_wgrad(ctypes.byref(tx), ctypes.byref(td), ctypes.byref(tw), ctypes.byref(p))
    if rc != 0:
        return rc, None
    return 0, L.d2h(dw.raw_ptr(), dw.shape, L.NP_STORAGE[out_dtype])


@pytest.mark.parametrize("case", [
    dict(x=(2, 128, 6, 8), k=64, rs=(3, 3), p=(1, 1, 1, 1, 1, 1)),        # one partial chunk per row, rows in pairs
    dict(x=(1, 128, 1, 8), k=64, rs=(3, 3), p=(1, 1, 1, 1, 1, 1)),        # a single row: the last fragments end at the tensor's end
    dict(x=(3, 32, 7, 40), k=256, rs=(3, 3), p=(1, 1, 1, 1, 1, 1)),       # four channel groups; chunks of 32 + 8 columns; odd height
    dict(x=(2, 64, 9, 18), k=128, rs=(3, 3), p=(1, 1, 1, 1, 2, 2)),       # dilation 2: every column shift odd
    dict(x=(2, 128, 6, 10), k=64, rs=(3, 3), p=(1, 1, 0, 0, 1, 1)),       # no padding: shifts 0, 1, 2
    dict(x=(2, 128, 4, 8), k=64, rs=(1, 1), p=(1, 1, 0, 0, 1, 1)),        # 1x1
    dict(x=(2, 128, 9, 8), k=64, rs=(3, 3), p=(2, 1, 1, 1, 1, 1)),        # vertical stride 2
    dict(x=(5, 128, 5, 72), k=64, rs=(2, 3), p=(1, 1, 0, 1, 1, 1), ips=2),   # three chunks (odd), 2x3 taps, two images per slice, the last slice one
    dict(x=(2, 128, 5, 16), k=64, rs=(1, 5), p=(1, 1, 0, 2, 1, 1)),       # 1x5 taps, padding 2: shifts -2 .. 2
    dict(x=(2, 128, 8, 16), k=64, rs=(3, 3), p=(1, 1, 2, 2, 2, 2)),       # dilation 2, padding 2: shifts -2, 0, 2
    dict(x=(2, 128, 6, 12), k=64, rs=(2, 3), p=(1, 1, 0, 0, 1, 2)),       # horizontal dilation 2, no padding: shifts 0, 2, 4
    dict(x=(2, 32, 6, 16), k=256, rs=(3, 3), p=(1, 1, 1, 1, 1, 1), out="bfloat16"),
    dict(x=(3, 64, 10, 24), k=64, rs=(3, 3), p=(1, 1, 1, 1, 1, 1)),       # 64 of a block's 128 input channels: half of the waves idle
    dict(x=(2, 192, 5, 8), k=64, rs=(3, 3), p=(1, 1, 1, 1, 1, 1)),        # a full block of input channels and half a block
    dict(x=(2, 48, 6, 16), k=128, rs=(1, 1), p=(1, 1, 0, 0, 1, 1)),       # blocks of 64 channels: 48
    dict(x=(3, 128, 9, 8), k=64, rs=(3, 3), p=(1, 1, 1, 1, 1, 1), rps=5),    # slices of 5 output rows: they start and end inside images
    dict(x=(3, 128, 9, 40), k=64, rs=(3, 3), p=(2, 1, 1, 1, 1, 1), rps=4),   # 5 output rows per image (stride 2), slices of 4; two chunks
    dict(x=(2, 128, 7, 8), k=64, rs=(3, 3), p=(1, 1, 1, 1, 1, 1), rps=1),    # one row per slice
    dict(x=(3, 128, 28, 28), k=64, rs=(3, 3), p=(1, 1, 1, 1, 1, 1)),      # 28 output columns: the row's last piece of dy is half the next row's
    dict(x=(4, 64, 14, 14), k=128, rs=(3, 3), p=(1, 1, 1, 1, 1, 1)),      # 14 columns: six of the second piece
    dict(x=(2, 128, 9, 36), k=64, rs=(3, 3), p=(1, 1, 1, 1, 1, 1)),       # 36 columns: a second chunk of four
    dict(x=(2, 64, 12, 12), k=64, rs=(1, 3), p=(1, 1, 0, 1, 1, 1), out="bfloat16"),
    dict(x=(3, 128, 7, 6), k=64, rs=(3, 3), p=(1, 1, 1, 1, 1, 1)),        # six columns: rows shorter than a piece
    dict(x=(2, 128, 27, 30), k=64, rs=(3, 3), p=(2, 1, 1, 1, 1, 1)),      # vertical stride 2 onto 14 rows of 30 columns
    dict(x=(2, 128, 10, 22), k=64, rs=(3, 3), p=(1, 1, 2, 2, 2, 2)),      # dilation 2 on 22 columns
])
def test_conv_wgrad_mfma_matches_oracle(gpu, case, monkeypatch):
    """The weight gradient kernel through the C entry point against the oracle's restatement of the
    gradient graph (float32 accumulator; the kernel sums in another order: 1e-4 of the largest value)."""
    rng = np.random.default_rng(31)
    N, C, H, W = case["x"]
    K, (R, S) = case["k"], case["rs"]
    sh, sw, ph, pw, dh, dw_ = case["p"]
    OH = (H + 2 * ph - dh * (R - 1) - 1) // sh + 1
    OW = (W + 2 * pw - dw_ * (S - 1) - 1) // sw + 1
    xb = _bf16(rng.standard_normal((N, C, H, W)))
    db = _bf16(rng.standard_normal((N, K, OH, OW)))
    out = case.get("out", "float32")
    if "ips" in case:
        monkeypatch.setenv("MJT_WGRAD_IPS", str(case["ips"]))
    if "rps" in case:
        monkeypatch.setenv("MJT_WGRAD_RPS", str(case["rps"]))
    rc, got = _wgrad_call(xb, db, R, S, case["p"], out)
    assert rc == 0 and L.last_kernel().startswith("mjt_conv_wgrad_mfma_bf16")
    xf, df = O.BF16(xb).to_f32().astype(np.float64), O.BF16(db).to_f32().astype(np.float64)
    xp = np.pad(xf, ((0, 0), (0, 0), (ph, ph), (pw, pw)))
    want = np.zeros((K, C, R, S))
    for r in range(R):
        for s in range(S):
            patch = xp[:, :, r * dh:r * dh + (OH - 1) * sh + 1:sh, s * dw_:s * dw_ + (OW - 1) * sw + 1:sw]
            want[:, :, r, s] = np.einsum("nkhw,nchw->kc", df, patch)
    if out == "bfloat16":
        got = O.BF16(got).to_f32()
        assert np.abs(got - want).max() <= 2.0 ** -7 * np.abs(want).max()
    else:
        assert np.abs(got - want).max() <= 1e-4 * np.abs(want).max()
    if N * K * C * OH * OW * R * S <= 4e7 and sh == sw and ph == pw and dh == dw_:
        ref = O.conv_meta_wgrad(O.BF16(xb), O.BF16(db), R, S, sh, ph, dh)     # the reference's own summation order
        assert np.abs(got - ref).max() <= (1e-4 if out == "float32" else 2.0 ** -7) * np.abs(ref).max()


def test_conv_wgrad_mfma_keeps_an_infinite_dy_in_its_row(gpu):
    """With 28 output columns a row's last 16-byte piece of dy holds the first four values of the next row.  An infinity
    there must not reach the sums of the row before it (0 x inf is NaN): the non-finite entries of dw are exactly those of
    the float64 evaluation, with their signs, and the finite ones agree."""
    rng = np.random.default_rng(33)
    N, C, K, H = 2, 128, 64, 28
    xb = _bf16(rng.standard_normal((N, C, H, H)) + 3.0)        # no zeros and no sign changes: every product with inf is +inf or -inf
    d = rng.standard_normal((N, K, H, H)).astype(np.float32)
    d[0, 3, 5, 0] = np.inf                                     # first column of a row: in the tail of the piece that ends row 4
    d[1, 9, 0, 2] = -np.inf
    db = _bf16(d)
    rc, got = _wgrad_call(xb, db, 3, 3, (1, 1, 1, 1, 1, 1))
    assert rc == 0 and L.last_kernel().startswith("mjt_conv_wgrad_mfma_bf16")
    xf, df = O.BF16(xb).to_f32().astype(np.float64), O.BF16(db).to_f32().astype(np.float64)
    xp = np.pad(xf, ((0, 0), (0, 0), (1, 1), (1, 1)))
    want = np.zeros((K, C, 3, 3))
    with np.errstate(invalid="ignore"):
        for r in range(3):
            for s in range(3):
                want[:, :, r, s] = np.einsum("nkhw,nchw->kc", df, xp[:, :, r:r + H, s:s + H])
    assert np.array_equal(np.isnan(got), np.isnan(want))
    assert np.array_equal(np.isposinf(got), np.isposinf(want)) and np.array_equal(np.isneginf(got), np.isneginf(want))
    fin = np.isfinite(want)
    assert fin.sum() > 0.9 * want.size and not fin.all()
    assert np.abs(got[fin] - want[fin]).max() <= 1e-4 * np.abs(want[fin]).max()


@pytest.mark.parametrize("case", [
    dict(dt="float32", x=(2, 6, 9, 8), k=6, g=6, rs=(3, 3), p=(1, 1, 1, 1, 1, 1)),          # depthwise
    dict(dt="float32", x=(3, 12, 8, 9), k=4, g=2, rs=(3, 3), p=(2, 1, 1, 0, 1, 2)),         # 6 channels per group: a tile of 4 and a tile of 2
    dict(dt="bfloat16", x=(2, 8, 10, 7), k=8, g=4, rs=(3, 3), p=(2, 2, 1, 1, 1, 1)),        # stride 2
    dict(dt="float16", x=(2, 4, 9, 9), k=6, g=2, rs=(2, 3), p=(1, 1, 2, 2, 2, 2), out="float16"),
    dict(dt="float32", x=(1, 2, 12, 12), k=2, g=2, rs=(9, 9), p=(1, 1, 4, 4, 1, 1)),        # 81 taps: three chunks of 32, the last short
    dict(dt="float32", x=(8, 4, 16, 16), k=4, g=4, rs=(1, 1), p=(1, 1, 0, 0, 1, 1)),        # 1x1; several slices of images, folded by the reduce
    dict(dt="bfloat16", x=(9, 6, 17, 16), k=6, g=3, rs=(3, 3), p=(1, 1, 1, 1, 1, 1), out="bfloat16"),   # slices with a short last one, 16-bit result
    dict(dt="float32", x=(2, 3, 7, 6), k=5, g=1, rs=(3, 3), p=(1, 1, 1, 1, 1, 1)),          # one group, float32: the direct kernel
    dict(dt="bfloat16", x=(2, 128, 6, 8), k=64, g=1, rs=(3, 3), p=(1, 1, 1, 1, 1, 1)),      # one group the MFMA kernel covers
    dict(dt="float32", x=(2, 4, 5, 5), k=4, g=2, rs=(3, 3), p=(1, 1, 0, 0, 1, 1), empty=True),
])
def test_conv_wgrad_grouped_matches_oracle(gpu, case):
    """mjt_conv2d_meta_wgrad_grouped against the oracle's restatement of the gradient graph of the grouped
    convolution (scatter-add over the 8-d product) and a float64 closed form per group; the kernel sums in another
    order: 1e-4 of the largest value, 2^-7 for a 16-bit result."""
    rng = np.random.default_rng(33)
    dt, (N, C, H, W), K, G, (R, S) = case["dt"], case["x"], case["k"], case["g"], case["rs"]
    sh, sw, ph, pw, dh, dw_ = case["p"]
    if case.get("empty"):
        N = 0
    OH = (H + 2 * ph - dh * (R - 1) - 1) // sh + 1
    OW = (W + 2 * pw - dw_ * (S - 1) - 1) // sw + 1
    narrow = {"float32": lambda a: a.astype(np.float32), "bfloat16": _bf16, "float16": lambda a: a.astype(np.float16)}[dt]
    widen = {"float32": lambda a: a, "bfloat16": lambda a: O.BF16(a).to_f32(), "float16": lambda a: a.astype(np.float32)}
    xb, db = narrow(rng.standard_normal((N, C, H, W))), narrow(rng.standard_normal((N, K, OH, OW)))
    out = case.get("out", "float32")
    x, dy = jt.from_storage(xb, dt), jt.from_storage(db, dt)
    dw = jt.zeros([K, C // G, R, S], out) + 7.0                       # stale values must be overwritten, not added to
    jt.sync([dw], True)
    tx, td, tw = L.tensor(x.raw_ptr(), dt, x.shape), L.tensor(dy.raw_ptr(), dt, dy.shape), L.tensor(dw.raw_ptr(), out, dw.shape)
    p = L.ConvParams(*case["p"])
    L.check(L.load().mjt_conv2d_meta_wgrad_grouped(ctypes.byref(tx), ctypes.byref(td), ctypes.byref(tw), ctypes.byref(p), G))
    mfma = G == 1 and dt == "bfloat16"
    if N:
        assert L.last_kernel().startswith("mjt_conv_wgrad_mfma" if mfma else "mjt_conv_wgrad_direct_" + dt), L.last_kernel()
    got = widen[out](L.d2h(dw.raw_ptr(), dw.shape, L.NP_STORAGE[out]))
    xf, df = widen[dt](xb).astype(np.float64), widen[dt](db).astype(np.float64)
    xp = np.pad(xf, ((0, 0), (0, 0), (ph, ph), (pw, pw)))
    cg, kg = C // G, K // G
    want = np.zeros((K, cg, R, S))
    for g in range(G):
        for r in range(R):
            for s in range(S):
                patch = xp[:, g * cg:(g + 1) * cg, r * dh:r * dh + (OH - 1) * sh + 1:sh, s * dw_:s * dw_ + (OW - 1) * sw + 1:sw]
                want[g * kg:(g + 1) * kg, :, r, s] = np.einsum("nkhw,nchw->kc", df[:, g * kg:(g + 1) * kg], patch)
    tol = 1e-4 if out == "float32" else 2.0 ** -7
    assert np.abs(got - want).max() <= tol * max(np.abs(want).max(), 1e-30)
    if N and sh == sw and ph == pw and dh == dw_ and N * K * cg * OH * OW * R * S <= 2e7:
        w0 = np.zeros((K, cg, R, S), np.float32)
        _, ref = O.conv_meta_grouped_grads(widen[dt](xb), w0, widen[dt](db), G, sh, ph, dh)   # the reference's own summation order
        assert np.abs(got - ref).max() <= tol * np.abs(ref).max()


def test_conv_wgrad_grouped_entry_errors(gpu):
    rng = np.random.default_rng(34)
    x, dy = jt.array(rng.standard_normal((1, 6, 5, 5)).astype(np.float32)), jt.array(rng.standard_normal((1, 4, 5, 5)).astype(np.float32))
    dw = jt.zeros([4, 3, 3, 3])
    jt.sync([x, dy, dw], True)
    tx, td, tw = (L.tensor(v.raw_ptr(), "float32", v.shape) for v in (x, dy, dw))
    p = L.ConvParams(1, 1, 1, 1, 1, 1)
    lib = L.load()
    assert lib.mjt_conv2d_meta_wgrad_grouped(ctypes.byref(tx), ctypes.byref(td), ctypes.byref(tw), ctypes.byref(p), 4) == -1
    assert "groups" in lib.mjt_last_error().decode()
    assert lib.mjt_conv2d_meta_wgrad_grouped(ctypes.byref(tx), ctypes.byref(td), ctypes.byref(tw), ctypes.byref(p), 0) == -1
    tw2 = L.tensor(dw.raw_ptr(), "float32", [4, 2, 3, 3])
    assert lib.mjt_conv2d_meta_wgrad_grouped(ctypes.byref(tx), ctypes.byref(td), ctypes.byref(tw2), ctypes.byref(p), 2) == -1
    ti = L.tensor(x.raw_ptr(), "int32", x.shape)
    assert lib.mjt_conv2d_meta_wgrad_grouped(ctypes.byref(ti), ctypes.byref(td), ctypes.byref(tw), ctypes.byref(p), 2) == -2


def test_conv_wgrad_entry_rejects_what_the_kernel_does_not_cover(gpu):
    rng = np.random.default_rng(32)
    xb, db = _bf16(rng.standard_normal((1, 128, 9, 9))), _bf16(rng.standard_normal((1, 64, 5, 5)))
    rc, _ = _wgrad_call(xb, db, 3, 3, (2, 2, 1, 1, 1, 1))                       # horizontal stride 2
    assert rc == -2 and "stride" in L.load().mjt_last_error().decode()
    rc, _ = _wgrad_call(xb, _bf16(rng.standard_normal((1, 64, 9, 8))), 3, 3, (1, 1, 1, 1, 1, 1))   # dy does not follow from x
    assert rc == -1 and "does not follow" in L.load().mjt_last_error().decode()


def test_conv_float16_operands(gpu):
    """float16 operands take the same kernels as bfloat16 (the f16 MFMA; a float16 result is rounded to nearest
    even, type/fp16_compute.h:147-198): forward on the MFMA and the direct kernel, weight gradient, and the three
    units through the front end with float16 gradients."""
    rng = np.random.default_rng(33)
    x = rng.standard_normal((2, 64, 12, 16)).astype(np.float16)
    w = (rng.standard_normal((128, 64, 3, 3)) * 0.1).astype(np.float16)
    want = O.conv_meta(x.astype(np.float32), w.astype(np.float32), 1, 1, 1)
    got, kern = _conv_call(x, w, (1, 1, 1, 1, 1, 1), in_dtype="float16")
    assert kern.startswith("mjt_conv_mfma_f16") and np.allclose(got, want, rtol=1e-5, atol=1e-5)
    got16, kern = _conv_call(x, w, (1, 1, 1, 1, 1, 1), out_dtype="float16", in_dtype="float16")
    assert kern.endswith("_of16") and got16.dtype == np.float16
    assert np.all(np.abs(got16.astype(np.float32) - want) <= 2.0 ** -10 * np.abs(want) + 1e-5)   # rounding + summation order
    xs, ws = rng.standard_normal((2, 3, 9, 8)).astype(np.float16), rng.standard_normal((4, 3, 3, 3)).astype(np.float16)
    got, kern = _conv_call(xs, ws, (1, 1, 1, 1, 1, 1), in_dtype="float16")
    assert kern.startswith("mjt_conv_direct_float16")
    assert np.allclose(got, O.conv_meta(xs.astype(np.float32), ws.astype(np.float32), 1, 1, 1), rtol=1e-5, atol=1e-5)
    # weight gradient
    xg, dy = rng.standard_normal((2, 128, 6, 8)).astype(np.float16), rng.standard_normal((2, 64, 6, 8)).astype(np.float16)
    rc, dw = _wgrad_call(xg, dy, 3, 3, (1, 1, 1, 1, 1, 1), in_dtype="float16")
    assert rc == 0 and L.last_kernel().startswith("mjt_conv_wgrad_mfma_f16")
    ref = O.conv_meta_wgrad(xg.astype(np.float32), dy.astype(np.float32), 3, 3, 1, 1, 1)
    assert np.abs(dw - ref).max() <= 1e-4 * np.abs(ref).max()
    # front end
    vx, vw = jt.array(x), jt.array(w)
    assert vx.dtype == "float16"
    y = jt.nn.conv2d(vx, vw, padding=1)
    r = (rng.integers(-2, 3, y.shape) * 0.5).astype(np.float16)
    gx, gw = jt.grad((y * jt.array(r)).sum(), [vx, vw])
    before = jt.executor_stats["conv_matches"]
    jt.sync([y, gx, gw])
    assert jt.executor_stats["conv_matches"] - before == 3 and (y.dtype, gx.dtype, gw.dtype) == ("float16",) * 3
    assert np.abs(y.float32().data - want).max() <= 2.0 ** -10 * np.abs(want).max()
    ref_gw = O.conv_meta_wgrad(x.astype(np.float32), r.astype(np.float32), 3, 3, 1, 1, 1)
    assert np.abs(gw.float32().data - ref_gw).max() <= 2.0 ** -9 * np.abs(ref_gw).max()


def test_conv_front_end_pattern_match(gpu):
    rng = np.random.default_rng(22)
    x = jt.array(rng.standard_normal((2, 64, 14, 16)).astype(np.float32)).bfloat16()
    w = jt.array((rng.standard_normal((128, 64, 3, 3)) * 0.05).astype(np.float32)).bfloat16()
    before = dict(jt.executor_stats)
    y = jt.nn.conv2d(x, w, padding=1)              # reindex + broadcast + multiply + sum, bf16 output
    got = y.data
    assert jt.executor_stats["conv_matches"] == before["conv_matches"] + 1
    assert y.dtype == "bfloat16" and L.last_kernel().endswith("_obf16")           # the sum keeps 16 bit (amp_reg | 36, nn.py:1250)
    from oracle import kernels as K
    acc = K.conv_meta_bf16(x.raw(), w.raw(), 1, 1, 1, 8)
    want = O.BF16(O.f32_to_bf16_bits(acc)).to_f32()
    assert np.abs(got - want).max() <= 2 ** -7 * np.abs(want).max()
    # without the matcher the same graph runs through the generic kernels (7-d intermediate materialised)
    jt.flags["enable_conv_match"] = False
    try:
        xs = jt.array(rng.standard_normal((1, 2, 6, 6)).astype(np.float32))
        ws = jt.array(rng.standard_normal((3, 2, 3, 3)).astype(np.float32))
        got = jt.nn.conv2d(xs, ws, padding=1).data
    finally:
        jt.flags["enable_conv_match"] = True
    assert np.allclose(got, O.conv_meta(xs.data, ws.data, 1, 1, 1), rtol=1e-5, atol=1e-5)
    got = jt.nn.conv2d(xs, ws, padding=1).data      # matched, fp32 -> direct kernel
    assert L.last_kernel().startswith("mjt_conv_direct_float32")
    assert np.allclose(got, O.conv_meta(xs.data, ws.data, 1, 1, 1), rtol=1e-5, atol=1e-5)


def test_conv_full_size_c5_properties(gpu):
    rng = np.random.default_rng(0)
    xs, ws = (64, 256, 56, 56), (256, 256, 3, 3)
    xb = _bf16(rng.standard_normal(xs))
    wb = _bf16(np.random.default_rng(1).standard_normal(ws) * np.sqrt(2.0 / (256 * 9)))
    got, kern = _conv_call(xb, wb, (1, 1, 1, 1, 1, 1))
    assert kern.startswith("mjt_conv_mfma_bf16")
    xf, wf = O.BF16(xb).to_f32(), O.BF16(wb).to_f32().astype(np.float64)
    xp = np.pad(xf, ((0, 0), (0, 0), (1, 1), (1, 1)))
    # sampled outputs against float64 dot products
    pts = np.random.default_rng(2).integers(0, [64, 256, 56, 56], (4000, 4))
    err = 0.0
    mag = 0.0
    for n, k, h, w_ in pts:
        patch = xp[n, :, h:h + 3, w_:w_ + 3].astype(np.float64)
        ref = float((patch * wf[k]).sum())
        err = max(err, abs(ref - got[n, k, h, w_]))
        mag = max(mag, float(np.abs(patch * wf[k]).sum()))
    assert err <= 1e-4 * mag, (err, mag)
    # two whole images (the first and the last, all 256 output channels) against the float64 product of the
    # weights with the image's column matrix, every element held to 1e-4 of the sum of its |x * w| terms
    wm = wf.reshape(256, 256 * 9)
    for n in (0, 63):
        win = np.lib.stride_tricks.sliding_window_view(xp[n].astype(np.float64), (3, 3), axis=(1, 2))   # [c, oh, ow, kh, kw]
        cols = win.transpose(0, 3, 4, 1, 2).reshape(256 * 9, 56 * 56)
        want = (wm @ cols).reshape(256, 56, 56)
        bound = 1e-4 * (np.abs(wm) @ np.abs(cols)).reshape(256, 56, 56)
        assert (np.abs(got[n] - want) <= bound).all(), (n, float(np.abs(got[n] - want).max()))
    # padding taps contribute exactly 0 and a one-hot kernel is a shift (bit-exact)
    w1 = np.zeros(ws, np.float32)
    for k in range(256):
        w1[k, k, 0, 2] = 1.0                       # y[n,k,h,w] = x[n,k,h-1,w+1]
    got1, _ = _conv_call(xb[:8], _bf16(w1), (1, 1, 1, 1, 1, 1))
    ref1 = np.zeros((8, 256, 56, 56), np.float32)
    ref1[:, :, 1:, :55] = xf[:8, :, :55, 1:]
    assert np.array_equal(got1, ref1)
    # linearity in w: conv(x, 2w) == 2 conv(x, w) exactly
    got2, _ = _conv_call(xb[:4], _bf16(2 * O.BF16(wb).to_f32()), (1, 1, 1, 1, 1, 1))
    assert np.array_equal(got2, 2 * got[:4])


# ---- 64-bit index mode ------------------------------------------------------------------------------
def test_index64_mode_beyond_2g_elements(gpu):
    """A Var with 2^31 or more elements switches index arithmetic to 64 bit
    (python/jittor/src/op.cc:158-192): reindex, fused element-wise and reduce on a
    [2^31 + 4096] int8 tensor, checked at the far end and through closed-form sums."""
    n = (1 << 31) + 4096
    base = np.arange(251, dtype=np.int8)                       # values 0..250 as int8 (wraps above 127)
    x = jt.array(base)
    y = x.reindex([n], ["i0 % 251"])                           # 2 GiB of int8
    z = y + 1                                                  # fused kernel over >= 2^31 elements (int8 wraps like C)
    tail = z.reindex([4096], ["i0 + %d" % (1 << 31)]).data
    idx = (np.arange(4096, dtype=np.int64) + (1 << 31)) % 251
    assert np.array_equal(tail, (base[idx].astype(np.int16) + 1).astype(np.int8))
    # reduce: maximum over everything, and a sum of a 0/1 pattern (int32 accumulator would overflow int8)
    assert int(y.max().data[0]) == int(base.max())
    ones = (y == 7).int32().sum().data[0]
    want = n // 251 + (1 if n % 251 > 7 else 0)
    assert int(ones) == want


def test_reduce_with_16_bit_results(gpu):
    """With amp_reg's keep_reduce a 16-bit float reduce keeps its type (nano_string.h:268-277), and with bit 32
    add / mean are not routed through float32 casts (ops/reduce_op.cc:260): the kernel accumulates in float32
    and rounds once.  Against the float32 reduce of the same values rounded the same way; row, column,
    split and whole-tensor shapes."""
    rng = np.random.default_rng(41)
    for shape, dims in [((37, 129), [1]), ((37, 129), [0]), ((4, 70000), [1]), ((30000, 8), [0]), ((64, 96), [])]:
        host = rng.uniform(-1, 1, shape).astype(np.float32)
        for dtype in ("bfloat16", "float16"):
            a = jt.array(host).cast(dtype)
            exact = a.float32().data                                     # the 16-bit values
            with jt.flag_scope(amp_reg=4 + 32):
                got = {op: a.reduce(op, dims) for op in ("add", "maximum", "mean")}
                assert all(v.dtype == dtype and v._op.kind == "reduce" for v in got.values())
                jt.sync(list(got.values()))
            want = {"add": O.reduce(exact, "add", dims), "maximum": O.reduce(exact, "maximum", dims),
                    "mean": O.reduce(exact, "mean", dims)}
            ulp = 2.0 ** -8 if dtype == "bfloat16" else 2.0 ** -11
            assert np.array_equal(got["maximum"].float32().data, want["maximum"])          # exact
            for op in ("add", "mean"):
                g, w = got[op].float32().data, want[op]
                assert np.all(np.abs(g - w) <= 2 * ulp * np.abs(w) + 1e-4), (shape, dims, dtype, op)


# ---- reduce with an element-wise prologue -----------------------------------------------------------
def test_fused_reduce_prologue(gpu):
    """A group of element-wise ops whose only result feeds a reduce runs inside the reduce kernel
    (element, broadcast and reduce ops share a group, python/jittor/src/executor.cc:555); results must
    equal the two-kernel path and the oracle."""
    rng = np.random.default_rng(40)
    x = rng.standard_normal((37, 129)).astype(np.float32)
    y = rng.standard_normal((37, 129)).astype(np.float32)
    cases = [
        (lambda a, b: (a * a).sum(1), lambda X, Y: (X * X).sum(1)),                          # row kernel
        (lambda a, b: ((a - b) * (a - b)).sum(0), lambda X, Y: ((X - Y) ** 2).sum(0)),       # column kernel
        (lambda a, b: (a * 2.0 + 1.0).abs().max(), lambda X, Y: np.abs(X * 2 + 1).max(keepdims=True).reshape(1)),   # all axes, scalars by value
        (lambda a, b: (a > b).int32().sum(1), lambda X, Y: (X > Y).sum(1)),                  # bool -> int32 prologue
        (lambda a, b: (a * b).mean(1), lambda X, Y: (X * Y).mean(1)),
        (lambda a, b: a.exp().min(0), lambda X, Y: np.exp(X).min(0)),
    ]
    for f, ref in cases:
        before = dict(jt.executor_stats)
        got = f(jt.array(x), jt.array(y)).data
        assert jt.executor_stats["fused_reduces"] == before["fused_reduces"] + 1
        assert jt.executor_stats["fused_groups"] == before["fused_groups"]          # nothing was materialised on the way
        want = ref(x.astype(np.float64), y.astype(np.float64))
        assert np.allclose(got, want, rtol=1e-5, atol=1e-4), (got, want)
        jt.flags["enable_reduce_fusion"] = False
        try:
            two = f(jt.array(x), jt.array(y)).data
        finally:
            jt.flags["enable_reduce_fusion"] = True
        assert np.allclose(got, two, rtol=1e-6, atol=1e-5)
    # large input: split path (partials + fold) with a prologue; bf16 sum is cast -> reduce -> cast
    big = rng.standard_normal((4, 1 << 18)).astype(np.float32)
    got = (jt.array(big) * jt.array(big)).sum().data
    assert np.allclose(got, (big.astype(np.float64) ** 2).sum(), rtol=1e-5)
    xb = jt.array(x).bfloat16()
    before = jt.executor_stats["fused_reduces"]
    s = xb.sum(1)
    got = s.data
    assert jt.executor_stats["fused_reduces"] == before + 1 and s.dtype == "bfloat16"
    want = O.BF16(O.f32_to_bf16_bits(O.BF16(xb.raw()).to_f32().astype(np.float64).sum(1).astype(np.float32))).to_f32()
    assert np.abs(got - want).max() <= 2 ** -7 * np.abs(want).max()
    # a tensor broadcast along an axis that is kept is not taken as a prologue: two kernels, same result
    sc = rng.standard_normal((1, x.shape[1])).astype(np.float32)
    before = dict(jt.executor_stats)
    got = (jt.array(x) * jt.array(sc)).sum(1).data
    assert jt.executor_stats["fused_reduces"] == before["fused_reduces"]
    assert np.allclose(got, (x.astype(np.float64) * sc).sum(1), rtol=1e-5, atol=1e-4)


def test_fused_reduce_with_per_output_inputs(gpu):
    """Prologue inputs broadcast along exactly the reduced axes (the mean inside a variance, the maximum
    inside a softmax) are read once per output: the variance of a
    normalisation is one launch (the pattern of python/jittor/test/test_new_fused_op.py:24-40)."""
    rng = np.random.default_rng(41)
    x = rng.standard_normal((33, 7, 130)).astype(np.float32)
    X = x.astype(np.float64)
    for dims in ([2], [0], [1, 2], [0, 2]):
        v = jt.array(x)
        before = dict(jt.executor_stats)
        mean = v.mean(dims, keepdims=True)
        var = ((v - mean) * (v - mean)).mean(dims, keepdims=True)
        y = (v - mean) / (var + 1e-5).sqrt()
        got = y.data
        assert jt.executor_stats["fused_reduces"] - before["fused_reduces"] == 1          # the variance
        # mean, variance, and one kernel for the rest: + eps and sqrt run behind their broadcast
        assert jt.executor_stats["launches"] - before["launches"] == 3
        ax = tuple(dims)
        want = (X - X.mean(ax, keepdims=True)) / np.sqrt(X.var(ax, keepdims=True) + 1e-5)
        assert np.allclose(got, want, rtol=1e-4, atol=1e-5), dims
    # softmax over the last axis
    v = jt.array(x)
    m = v.max(2, keepdims=True)
    e = (v - m).exp()
    s = e.sum(2, keepdims=True)
    got = (e / s).data
    ex = np.exp(X - X.max(2, keepdims=True))
    assert np.allclose(got, ex / ex.sum(2, keepdims=True), rtol=1e-5, atol=1e-7)
    # the same chain with the broadcast sink switched off gives the same values from more launches
    jt.flags["enable_broadcast_sink"] = False
    try:
        v = jt.array(x)
        before = dict(jt.executor_stats)
        mean = v.mean([2], keepdims=True)
        var = ((v - mean) * (v - mean)).mean([2], keepdims=True)
        ref = ((v - mean) / (var + 1e-5).sqrt()).data
        assert jt.executor_stats["launches"] - before["launches"] > 3
    finally:
        jt.flags["enable_broadcast_sink"] = True
    v = jt.array(x)
    mean = v.mean([2], keepdims=True)
    var = ((v - mean) * (v - mean)).mean([2], keepdims=True)
    assert np.allclose(((v - mean) / (var + 1e-5).sqrt()).data, ref, rtol=1e-6, atol=1e-6)
    # an input broadcast along other axes than the reduced ones stays a separate kernel
    w = rng.standard_normal((1, 7, 1)).astype(np.float32)
    before = dict(jt.executor_stats)
    got = (jt.array(x) * jt.array(w)).sum(2).data
    assert jt.executor_stats["fused_reduces"] == before["fused_reduces"]
    assert np.allclose(got, (X * w).sum(2), rtol=1e-5, atol=1e-4)


def test_zz_shutdown_and_rebind_on_the_device(gpu):
    """mjt_shutdown followed by mjt_init: kernels, scratch buffers and the packed-weight buffer are rebuilt, results
    stay the same (buffers the caller allocated survive: they are the caller's)."""
    rng = np.random.default_rng(50)
    x = rng.standard_normal((300, 257)).astype(np.float32)
    xb, wb = _bf16(rng.standard_normal((2, 64, 16, 16))), _bf16(rng.standard_normal((128, 64, 3, 3)) * 0.1)
    a = jt.array(x)
    s1 = a.sum(1).data
    y1, _ = _conv_call(xb, wb, (1, 1, 1, 1, 1, 1))
    lib = L.load()
    lib.mjt_shutdown()
    L._device = None
    L.init(0)
    s2 = a.sum(1).data                                       # `a` was allocated before the shutdown
    y2, kern = _conv_call(xb, wb, (1, 1, 1, 1, 1, 1))
    assert kern.startswith("mjt_conv_mfma_bf16") and np.array_equal(s1, s2) and np.array_equal(y1, y2)
    assert np.allclose(s2, x.sum(1), rtol=1e-5, atol=1e-4)


def test_gather_fused_with_reduce(gpu):
    """mjt_reindex_then_reduce: a reindex whose only consumer is a reduce over its last axes runs as one kernel
    (pooling, pool.py:200-208).  Through the C entry point against the oracle's reindex + reduce, then the
    front end: same results as the two-kernel path, no rank-6 tensor in memory."""
    rng = np.random.default_rng(60)
    lib = L.load()
    x = rng.standard_normal((2, 3, 9, 10)).astype(np.float32)
    none, noex = L.c_strings([]), (L.Tensor * 1)()
    for op, shape, idx, ov, nred in [
            ("maximum", [2, 3, 4, 5, 3, 2], ["i0", "i1", "i2*2-1+i4", "i3*2-0+i5"], -1e30, 2),
            ("mean", [2, 3, 4, 5, 3, 2], ["i0", "i1", "i2*2-1+i4", "i3*2-0+i5"], 0.0, 2),
            ("add", [2, 9, 10, 3], ["i0", "i3", "i1", "i2"], 0.0, 1),                      # sum over channels, moved last
            ("minimum", [7, 2, 3, 9, 10], ["i1", "i2", "(i3+i0)%9", "i4"], 5.0, 4),        # keeps only the first axis
            ("multiply", [4, 2, 3, 3, 3], ["i1", "i2", "i0+i3", "i4*5"], 1.0, 2),
            ("add", [3, 5, 3, 2], ["i0%2", "i1%3", "i2*3+i0", "i3*6"], 0.5, 2),            # an odd number of outputs, two per lane
            ("add", [2, 3, 2, 2, 4, 5], ["i0", "i1", "i2*4+i4", "i3*5+i5"], 0.0, 2),       # window rows of 5, all in range: loaded as vectors
            ("maximum", [2, 3, 2, 2, 4, 5], ["i0", "i1", "i2*4+i4-1", "i3*5+i5"], -1e30, 2),  # the same with rows above the image
            ("minimum", [2, 3, 9, 2, 4], ["i0", "i1", "i2", "i3*4+i4+1"], 7.0, 1),          # rows of 4 at odd offsets
            ("maximum", [1, 1, 2, 3, 5, 3], ["i0", "i1", "i2*5+i4-1", "i3*3+i5"], -1e30, 4)]:  # 90 folded elements: the loop form
        want = O.reduce(O.reindex(x, shape, idx, ov), op, list(range(len(shape) - nred, len(shape))))
        vx, vz = jt.from_storage(x, "float32"), jt.zeros(list(want.shape), "float32")
        tx, ts = L.tensor(vx.raw_ptr(), "float32", vx.shape), L.tensor(0, "float32", shape)
        tz = L.tensor(vz.raw_ptr(), "float32", vz.shape)
        L.check(lib.mjt_reindex_then_reduce(ctypes.byref(tx), ctypes.byref(ts), ctypes.byref(tz), L.OP_CODE[op], nred, len(idx),
                                            L.c_strings(idx), ov, 0, none, 0, noex))
        assert L.last_kernel().startswith("mjt_reindex_then_" + op)
        got = L.d2h(vz.raw_ptr(), vz.shape, np.float32)
        assert np.allclose(got, want, rtol=1e-5, atol=1e-6), (op, shape)
    # integers with an overflow condition and an extra (a gather by an index tensor, then a sum): bit-exact
    xi = rng.integers(-50, 50, (6, 20)).astype(np.int32)
    e0 = rng.integers(0, 20, (6, 5, 4)).astype(np.int32)
    shape, idx, ofc = [6, 5, 4], ["i0", "@e0(i0,i1,i2)"], ["i2>2"]
    want = O.reduce(O.reindex(xi, shape, idx, 7, ofc, [e0]), "add", [1, 2])
    got = jt.array(xi).reindex(shape, idx, 7, ofc, [jt.array(e0)]).sum([1, 2])
    before = jt.executor_stats["gather_reduces"]
    assert np.array_equal(got.data, want) and jt.executor_stats["gather_reduces"] == before + 1
    # pooling through the front end, float32 and bfloat16 (the 16-bit mean's float32 casts are part of the group)
    xp = rng.standard_normal((3, 5, 11, 12)).astype(np.float32)
    for dtype in ("float32", "bfloat16"):                      # windows of 4 x 4 without padding: rows loaded as vectors
        v = jt.array(xp).cast(dtype)
        y4 = jt.pool(v, 4, "maximum", 0, 4)
        jt.sync([y4])
        assert L.last_kernel().startswith("mjt_reindex_then_maximum"), L.last_kernel()
        want = v.float32().data[:, :, :8, :12].reshape(3, 5, 2, 4, 3, 4).max(axis=(3, 5))
        assert np.array_equal(y4.float32().data, want), dtype
    for dtype in ("float32", "bfloat16"):
        for op in ("maximum", "mean"):
            v = jt.array(xp).cast(dtype)
            jt.sync([v])
            before, l0 = jt.executor_stats["gather_reduces"], jt.executor_stats["launches"]
            y = jt.pool(v, 3, op, 1, 2)
            jt.sync([y])
            l1 = jt.executor_stats["launches"]
            fused = y.float32().data
            assert jt.executor_stats["gather_reduces"] == before + 1 and y.dtype == ("float32" if op == "maximum" or dtype == "float32" else dtype)
            jt.flags["enable_gather_reduce"] = False
            try:
                l2 = jt.executor_stats["launches"]
                yp = jt.pool(v, 3, op, 1, 2)
                jt.sync([yp])
                assert jt.executor_stats["launches"] - l2 > l1 - l0            # the window tensor costs a launch of its own
                plain = yp.float32().data
            finally:
                jt.flags["enable_gather_reduce"] = True
            # a 16-bit mean is rounded after a float32 sum whose order differs between the two paths
            tol = 1e-5 if dtype == "float32" else 2.0 ** -7
            assert np.array_equal(fused, plain) if op == "maximum" else np.allclose(fused, plain, rtol=tol, atol=tol * 1e-1)


def test_scatter_with_element_wise_prologue(gpu):
    """mjt_fused_reindex_reduce through the C entry point: the scattered values are computed in the kernel from a
    full-shape tensor, a tensor broadcast along the window axes, a scalar, and a tensor read through the scatter's
    own index program; against the oracle's reindex / element-wise / reindex_reduce chain."""
    rng = np.random.default_rng(61)
    lib = L.load()
    xshape, yshape = [2, 3, 8, 9], [2, 3, 4, 4, 3, 3]
    idx = ["i0", "i1", "i2*2-1+i4", "i3*2-0+i5"]
    src = rng.standard_normal(xshape).astype(np.float32)          # read through the index program
    full = rng.standard_normal(yshape).astype(np.float32)
    small = rng.standard_normal(yshape[:4] + [1, 1]).astype(np.float32)
    # value = (gathered(src) * full + small) * 0.5
    want_y = (O.reindex(src, yshape, idx, 0.0) * full + small) * np.float32(0.5)
    want = O.reindex_reduce(want_y.astype(np.float32), "add", xshape, idx)
    vs, vf, vm, vx = jt.from_storage(src, "float32"), jt.from_storage(full, "float32"), jt.from_storage(small, "float32"), jt.zeros(xshape)
    V, F = L.FusedVar, L.FusedOp
    spec = [(L.VAR_GATHERED, vs.raw_ptr(), 0, 0.0), (L.VAR_INPUT, vf.raw_ptr(), 0, 0.0), (L.VAR_INPUT, vm.raw_ptr(), 0b110000, 0.0),
            (L.VAR_SCALAR, None, 0, 0.5), (L.VAR_INTERMEDIATE, None, 0, 0.0), (L.VAR_INTERMEDIATE, None, 0, 0.0),
            (L.VAR_OUTPUT, None, 0, 0.0)]
    va = (V * len(spec))()
    for i, (role, ptr, mask, f) in enumerate(spec):
        va[i].role, va[i].dtype, va[i].ptr, va[i].bcast_mask, va[i].fvalue = role, L.DTYPE_CODE["float32"], ptr, mask, f
    ops = [("multiply", [0, 1], 4), ("add", [4, 2], 5), ("multiply", [5, 3], 6)]
    oa = (F * len(ops))()
    for i, (name, ins, out) in enumerate(ops):
        oa[i].kind, oa[i].op, oa[i].out = L.FOP_BINARY, L.OP_CODE[name], out
        for j, v in enumerate(ins):
            oa[i].inp[j] = v
    d = L.FusedDesc()
    d.ndim = len(yshape)
    for i, s_ in enumerate(yshape):
        d.shape[i] = s_
    d.n_vars, d.vars, d.n_ops, d.ops = len(spec), va, len(ops), oa
    tx = L.tensor(vx.raw_ptr(), "float32", xshape)
    # the window pattern runs as a gather over x; with that path switched off, as atomic updates
    for env, kernel in ((None, "mjt_window_scatter_add_"), ("MJT_NO_WINDOW_SCATTER", "mjt_reindex_reduce_add_")):
        if env:
            os.environ[env] = "1"
        try:
            L.check(lib.mjt_fused_reindex_reduce(ctypes.byref(d), ctypes.byref(tx), L.OP_CODE["add"], 4, L.c_strings(idx), 0, L.c_strings([]),
                                                 0, (L.Tensor * 1)()))
        finally:
            if env:
                del os.environ[env]
        assert L.last_kernel().startswith(kernel), L.last_kernel()
        got = L.d2h(vx.raw_ptr(), xshape, np.float32)
        assert np.allclose(got, want, rtol=1e-4, atol=1e-5), kernel
    # a gathered var is refused where it has no meaning
    assert lib.mjt_fused_elementwise(ctypes.byref(d)) < 0 and "role" in lib.mjt_last_error().decode()
