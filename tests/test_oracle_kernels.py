"""The C++ oracle kernels (oracle/oracle_kernels.cc, the timed CPU baseline)
against the numpy oracle and closed forms.  No GPU."""
import numpy as np

from oracle import oracle as O
from oracle import kernels as K

rng = np.random.default_rng(5)


def test_reduce_and_reindex_kernels():
    x = rng.uniform(-1, 1, (37, 513)).astype(np.float32)
    for t in (1, 4):
        assert np.allclose(K.reduce_sum_axis1(x, t), x.astype(np.float64).sum(1), rtol=1e-5, atol=1e-4)
    x = rng.standard_normal((2, 3, 9, 7)).astype(np.float32)
    ref = O.reindex(x, [2, 3, 9, 7, 3, 3], ["i0", "i1", "i2+i4-1", "i3+i5-1"], 0)
    for t in (1, 4):
        assert np.array_equal(K.reindex_im2col3x3(x, t), ref)


def test_scatter_kernel():
    n, bins = 20000, 300
    v = rng.random(n).astype(np.float32)
    idx = (rng.integers(0, bins + 10, n) - 5).astype(np.int32)
    for op in ("add", "maximum"):
        ref = O.reindex_reduce(v, op, [bins], ["@e0(i0)"], extras=[idx])
        got = K.scatter_1d(v, idx, bins, op)
        assert np.allclose(got, ref, rtol=1e-6) if op == "add" else np.array_equal(got, ref)


def test_fused_chain_kernel():
    x = rng.standard_normal((3, 5, 16)).astype(np.float32)
    s, b = rng.standard_normal((5, 1)).astype(np.float32), rng.standard_normal((1, 16)).astype(np.float32)
    x64 = x.astype(np.float64)
    ref = np.exp(-np.maximum(x64 * s + b, 0)) / (1 + np.exp(np.minimum(-x64, 30)))
    for t in (1, 4):
        assert np.allclose(K.fused_chain(x, s, b, t), ref, rtol=1e-5)


def test_conv_kernel():
    xb = O.f32_to_bf16_bits(rng.standard_normal((2, 4, 7, 6)).astype(np.float32))
    wb = O.f32_to_bf16_bits(rng.standard_normal((5, 4, 3, 3)).astype(np.float32))
    ref = O.conv_meta(O.BF16(xb), O.BF16(wb), 1, 1, 1)
    for t in (1, 4):
        assert np.allclose(K.conv_meta_bf16(xb, wb, 1, 1, 1, t), ref, rtol=1e-5, atol=1e-5)
    ref = O.conv_meta(O.BF16(xb), O.BF16(wb), 2, 0, 1)
    assert np.allclose(K.conv_meta_bf16(xb, wb, 2, 0, 1), ref, rtol=1e-5, atol=1e-5)
