"""mjt_reduce_static: the entry point that allocates nothing (partials of a two-pass reduction in a fixed
device array).  Checked through the C-ABI against mjt_reduce, the entry point it is a variant of, on two
calls in a row, the second with a smaller input; float32 sums to 1e-5 relative (here the two run the same
kernels over the same split, so they also agree bit for bit), integer results exactly."""
import ctypes

import numpy as np
import pytest

from jittor_amd import _lib as L

pytestmark = pytest.mark.gpu

STATIC_BYTES = 4 << 20


def _reduce(lib, fn, dx, dy, xshape, yshape, xdt, ydt, op, mask):
    tx, ty = L.tensor(dx, xdt, xshape), L.tensor(dy, ydt, yshape)
    return fn(ctypes.byref(tx), ctypes.byref(ty), L.OP_CODE[op], mask)


def test_reduce_static_matches_reduce_on_two_calls_in_a_row(gpu):
    lib = L.load()
    rng = np.random.default_rng(5)
    # few outputs and long reduced axes: both shapes take the two-pass route (row kernel: partials [O, S])
    big, small = (6, 1 << 21), (3, 300000)
    xs = {s: rng.uniform(-1, 1, s).astype(np.float32) for s in (big, small)}
    dx = {s: L.alloc(xs[s].nbytes) for s in xs}
    for s in xs:
        L.h2d(dx[s], xs[s])
    dy_ref, dy_new = L.alloc(256), L.alloc(256)
    try:
        # the allocating entry point first: reference results, and it loads the kernels both calls below need
        refs = {}
        for s in (big, small):
            L.check(_reduce(lib, lib.mjt_reduce, dx[s], dy_ref, s, [s[0]], "float32", "float32", "add", 0b10))
            assert "split" in L.last_kernel() or "fold" in L.last_kernel(), L.last_kernel()
            refs[s] = L.d2h(dy_ref, [s[0]], np.float32)
        # what the entry point exists for: between here and the end of its calls no kernel is built or loaded and
        # no device memory is taken (the free memory the runtime reports stays what it was)
        hip = ctypes.CDLL("libamdhip64.so")
        free0, free1, total = ctypes.c_size_t(), ctypes.c_size_t(), ctypes.c_size_t()
        L.sync()
        assert hip.hipMemGetInfo(ctypes.byref(free0), ctypes.byref(total)) == 0
        stats0 = L.jit_stats()
        # two calls in a row of the variant that allocates nothing, the second with the smaller input
        for s in (big, small):
            L.h2d(dy_new, np.full(64, np.nan, np.float32))
            L.check(_reduce(lib, lib.mjt_reduce_static, dx[s], dy_new, s, [s[0]], "float32", "float32", "add", 0b10))
            got = L.d2h(dy_new, [s[0]], np.float32)
            exact = xs[s].astype(np.float64).sum(1)
            assert np.allclose(got, refs[s], rtol=1e-5, atol=0), (s, got, refs[s])
            assert np.array_equal(got, refs[s]), (s, got, refs[s])
            assert np.allclose(got, exact, rtol=1e-5, atol=1e-5 * np.sqrt(s[1])), (s, got, exact)
        assert L.jit_stats() == stats0, (stats0, L.jit_stats())
        assert hip.hipMemGetInfo(ctypes.byref(free1), ctypes.byref(total)) == 0
        assert free1.value == free0.value, (free0.value, free1.value)
    finally:
        for p in list(dx.values()) + [dy_ref, dy_new]:
            L.free(p)


def test_reduce_static_column_route_and_integers(gpu):
    lib = L.load()
    rng = np.random.default_rng(6)
    for shape in ((40000, 96), (9000, 32)):                     # reduce axis 0: column kernel, partials [S, O]
        x = rng.integers(-1000, 1000, shape).astype(np.int32)
        dx, d1, d2 = L.alloc(x.nbytes), L.alloc(shape[1] * 4), L.alloc(shape[1] * 4)
        try:
            L.h2d(dx, x)
            for op, ref in (("add", x.sum(0, dtype=np.int32)), ("maximum", x.max(0))):
                L.check(_reduce(lib, lib.mjt_reduce, dx, d1, shape, [shape[1]], "int32", "int32", op, 0b01))
                L.check(_reduce(lib, lib.mjt_reduce_static, dx, d2, shape, [shape[1]], "int32", "int32", op, 0b01))
                a, b = L.d2h(d1, [shape[1]], np.int32), L.d2h(d2, [shape[1]], np.int32)
                assert np.array_equal(a, ref) and np.array_equal(b, ref), (shape, op)
        finally:
            for p in (dx, d1, d2):
                L.free(p)


def test_reduce_static_refuses_what_it_cannot_do_without_allocating(gpu):
    lib = L.load()
    shape = (64, 500000)             # reduce axis 0: split in 3, 500000 x 3 float32 partials = 6 MB > the 4 MiB array
    dx, dy = L.alloc(shape[0] * shape[1] * 4), L.alloc(shape[1] * 4)
    try:
        # a kernel nobody has loaded yet (float64 minimum over the middle axis of a rank-3 tensor)
        rc = _reduce(lib, lib.mjt_reduce_static, dx, dy, (4, 50000, 3), [4, 3], "float64", "float64", "minimum", 0b010)
        assert rc == -6 and b"not loaded" in lib.mjt_last_error(), (rc, lib.mjt_last_error())
        L.check(_reduce(lib, lib.mjt_reduce, dx, dy, shape, [shape[1]], "float32", "float32", "add", 0b01))
        assert "fold" in L.last_kernel(), L.last_kernel()
        rc = _reduce(lib, lib.mjt_reduce_static, dx, dy, shape, [shape[1]], "float32", "float32", "add", 0b01)
        assert rc == -2 and b"fixed scratch array holds" in lib.mjt_last_error(), (rc, lib.mjt_last_error())
    finally:
        L.free(dx)
        L.free(dy)
