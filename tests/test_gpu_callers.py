"""GPU tests of the callers built on the path (gather, scatter, pad, pool,
permute, reshape, flip, slicing) against numpy, with the examples of the
reference's docstrings (python/jittor/misc.py:1575-1600,1628-1634) and its
tests of pooling and padding as cases."""
import numpy as np
import pytest

import jittor_amd as jt
from jittor_amd import _lib as L
from oracle import oracle as O

pytestmark = pytest.mark.gpu


def test_gather_scatter_docstring_examples(gpu):
    t = jt.array([[1, 2], [3, 4]])
    assert t.gather(1, jt.array([[0, 0], [1, 0]])).data.tolist() == [[1, 1], [4, 3]]
    assert t.gather(0, jt.array([[0, 0], [1, 0]])).data.tolist() == [[1, 2], [3, 2]]
    src = jt.array(np.arange(1, 11, dtype=np.int32).reshape(2, 5))
    x = jt.zeros((3, 5), "int32").scatter(0, jt.array([[0, 1, 2, 0]]), src)
    assert x.data.tolist() == [[1, 0, 0, 4, 0], [0, 2, 0, 0, 0], [0, 0, 3, 0, 0]]
    x = jt.zeros((3, 5), "int32").scatter(1, jt.array([[0, 1, 2], [0, 1, 4]]), src)
    assert x.data.tolist() == [[1, 2, 3, 0, 0], [6, 7, 0, 0, 8], [0, 0, 0, 0, 0]]
    full = jt.array(np.full((2, 4), 2.0, np.float32))
    x = full.scatter(1, jt.array([[2], [3]]), jt.array(1.23), reduce="multiply")
    assert np.allclose(x.data, [[2, 2, 2.46, 2], [2, 2, 2, 2.46]])
    x = full.scatter(1, jt.array([[2], [3]]), jt.array(1.23), reduce="add")
    assert np.allclose(x.data, [[2, 2, 3.23, 2], [2, 2, 2, 3.23]])


def test_gather_scatter_random(gpu):
    rng = np.random.default_rng(50)
    x = rng.standard_normal((7, 9, 5)).astype(np.float32)
    for dim in range(3):
        idx = rng.integers(0, x.shape[dim], (7, 9, 5)).astype(np.int32)
        assert np.array_equal(jt.array(x).gather(dim, jt.array(idx)).data, np.take_along_axis(x, idx, dim))
        src = rng.standard_normal((7, 9, 5)).astype(np.float32)
        want = x.astype(np.float64).copy()
        np.add.at(want, tuple(idx if d == dim else np.indices(idx.shape)[d] for d in range(3)), src)
        got = jt.array(x).scatter(dim, jt.array(idx), jt.array(src), reduce="add").data
        assert np.allclose(got, want, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("mode", ["constant", "replicate", "reflect", "circular"])
def test_pad_modes(gpu, mode):
    rng = np.random.default_rng(51)
    x = rng.standard_normal((2, 3, 6, 7)).astype(np.float32)
    padding = (2, 1, 3, 2)                                   # left, right of the last axis, then of the one before
    got = jt.pad(jt.array(x), padding, mode, 1.5).data
    widths = ((0, 0), (0, 0), (3, 2), (2, 1))
    np_mode = {"constant": "constant", "replicate": "edge", "reflect": "reflect", "circular": "wrap"}[mode]
    want = np.pad(x, widths, np_mode, **({"constant_values": 1.5} if mode == "constant" else {}))
    assert np.array_equal(got, want)


def test_pool_against_numpy(gpu):
    rng = np.random.default_rng(52)
    x = rng.standard_normal((2, 3, 12, 10)).astype(np.float32)
    for k, s, p in [(2, 2, 0), (3, 2, 1), (3, 1, 1)]:
        H = (12 + 2 * p - k) // s + 1
        W = (10 + 2 * p - k) // s + 1
        xp = np.pad(x, ((0, 0), (0, 0), (p, p), (p, p)))     # the reference's meta-operator pooling pads with 0
        win = np.stack([xp[:, :, i:i + (H - 1) * s + 1:s, j:j + (W - 1) * s + 1:s] for i in range(k) for j in range(k)], -1)
        for op, f in (("maximum", np.max), ("minimum", np.min), ("mean", np.mean), ("add", np.sum)):
            got = jt.pool(jt.array(x), k, op, p, s).data
            assert np.allclose(got, f(win.astype(np.float64), axis=-1), rtol=1e-5, atol=1e-6), (k, s, p, op)
    # gradient of max pooling: ones at the arg-max of every window
    v = jt.array(x)
    g = jt.grad(jt.nn.max_pool2d(v, 2).sum(), v).data
    blocks = x.reshape(2, 3, 6, 2, 5, 2)
    want = (blocks == blocks.max(axis=(3, 5), keepdims=True)).reshape(x.shape).astype(np.float32)
    assert np.array_equal(g, want)


def test_reshape_shares_its_input_bytes(gpu):
    """reshape launches nothing (python/jittor/src/ops/reshape_op.cc aliases the buffer); values, gradients and later
    assignments to either Var behave as with a copy."""
    from jittor_amd import executor as E
    rng = np.random.default_rng(59)
    x = rng.standard_normal((6, 8, 10)).astype(np.float32)
    v = jt.array(x)
    v.sync()
    before = E.stats["launches"]
    r = v.reshape(48, 10)
    r.sync()
    assert E.stats["launches"] == before and r._device_ptr() == v._device_ptr()
    assert np.array_equal(r.data, x.reshape(48, 10))
    # a computed input, a reshape in the middle of a chain, and a reduce over the reshaped axes
    w = ((v * 2.0 + 1.0).reshape(6, 80) - 0.5).reshape(12, 40)
    assert np.allclose(w.data, ((x * 2.0 + 1.0).reshape(6, 80) - 0.5).reshape(12, 40), rtol=1e-6, atol=1e-6)
    s = (v * v).reshape(6, 4, 20).sum(2)
    assert np.allclose(s.data, (x * x).reshape(6, 4, 20).sum(2), rtol=1e-5, atol=1e-5)
    # functional values: rebinding one Var leaves the other's contents alone
    v2 = jt.array(x)
    r2 = v2.reshape(-1)
    r2.sync()
    v2.assign(v2 + 1.0)
    v2.sync()
    assert np.array_equal(r2.data, x.reshape(-1)) and np.allclose(v2.data, x + 1.0)
    # gradient through a reshape
    p = jt.array(x)
    loss = (p.reshape(48, 10) * jt.array(np.arange(10, dtype=np.float32))).sum()
    g = jt.grad(loss, [p])[0]
    assert np.allclose(g.data, np.broadcast_to(np.arange(10, dtype=np.float32), (6, 8, 10)))
    with jt.flag_scope(reshape_shares_memory=False):
        before = E.stats["launches"]
        c = v.reshape(10, 48)
        c.sync()
        assert E.stats["launches"] == before + 1 and c._device_ptr() != v._device_ptr()
        assert np.array_equal(c.data, x.reshape(10, 48))


def test_layout_ops_and_slicing(gpu):
    rng = np.random.default_rng(53)
    x = rng.standard_normal((4, 5, 6, 7)).astype(np.float32)
    v = jt.array(x)
    assert np.array_equal(v.permute(0, 2, 3, 1).data, x.transpose(0, 2, 3, 1))
    assert np.array_equal(v.transpose().data, x.transpose())
    assert np.array_equal(v.reshape(20, -1).data, x.reshape(20, -1))
    assert np.array_equal(v.reshape(2, 2, 5, 42).data, x.reshape(2, 2, 5, 42))
    assert np.array_equal(v.flip([1, 3]).data, x[:, ::-1, :, ::-1])
    assert np.array_equal(v[1].data, x[1])
    assert np.array_equal(v[1:3, ::2, -1].data, x[1:3, ::2, -1])
    assert np.array_equal(v[..., ::-2].data, x[..., ::-2])
    assert np.array_equal(v[:, None, 2].data, x[:, None, 2])
    idx = np.array([3, 0, 3, 1], np.int32)
    assert np.array_equal(v[:, jt.array(idx)].data, x[:, idx])
    # integer Vars (lists, numpy arrays) of any rank; several of them index together, broadcast against each other into
    # one block of dims where the first of them stood (getitem_op.cc:76-113) -- numpy's result when they are adjacent
    i2 = np.array([[3, 0], [1, 2], [0, 0]], np.int32)
    assert np.array_equal(v[jt.array(i2)].data, x[i2])
    assert np.array_equal(v[:, jt.array(i2), 1].data, x[:, i2, 1])
    a, b = np.array([0, 3, 1], np.int32), np.array([4, 4, 2], np.int32)
    assert np.array_equal(v[jt.array(a), jt.array(b)].data, x[a, b])
    assert np.array_equal(v[:, jt.array(a), jt.array(b), ::2].data, x[:, a, b, ::2])
    col = np.array([[0], [3]], np.int32)
    assert np.array_equal(v[jt.array(col), jt.array(b)].data, x[col, b])          # [2,1] with [3] -> a [2,3] block
    assert np.array_equal(v[[1, 0, 1]].data, x[[1, 0, 1]])
    assert np.array_equal(v[:, np.array([4, 1])].data, x[:, [4, 1]])
    # separated by a slice: the block stays at the first index Var's place (numpy would move it to the front)
    got = v[jt.array(a), :, jt.array(b)].data
    assert np.array_equal(got, x[a, :, b])               # (the first one stands first here, so both agree)
    got = v[:, jt.array(a), :, jt.array(b)].data
    assert got.shape == (4, 3, 6) and np.array_equal(got, np.stack([x[:, a[i], :, b[i]] for i in range(3)], axis=1))
    with pytest.raises(IndexError):
        v[jt.array(a), jt.array(np.array([0, 1], np.int32))]                       # [3] and [2] do not broadcast
    with pytest.raises(IndexError):
        v[4]
    with pytest.raises(IndexError):
        v[0, 0, 0, 0, 0]
    # gradients flow through the layout ops: d/dx sum(x[1:3] * w) = w placed at the slice
    w = rng.standard_normal((2, 5, 6, 7)).astype(np.float32)
    g = jt.grad((v[1:3] * jt.array(w)).sum(), v).data
    want = np.zeros_like(x)
    want[1:3] = w
    assert np.array_equal(g, want)


def test_profile_scope_report(gpu):
    """jt.profile_scope: rows per kernel with count, times and byte rates (profiler.cc:374-470)."""
    rng = np.random.default_rng(54)
    a = jt.array(rng.standard_normal((512, 2048)).astype(np.float32))
    b = jt.array(rng.standard_normal((512, 2048)).astype(np.float32))
    jt.sync([a, b])
    with jt.profile_scope(warmup=1, rerun=4) as report:
        y = (a * b + 1.0).sum(1)
        z = a.reindex([512, 2048], ["i0", "2047-i1"])
        jt.sync([y, z])
    assert report[0] == ["Name", "FileName", "Count", "TotalTime", "AvgTime", "MinTime", "MaxTime", "Input", "Output", "InOut", "Compute"]
    rows = {r[0]: r for r in report[2:]}
    red = [r for n, r in rows.items() if n.startswith("mjt_reduce_row_add")]
    rei = [r for n, r in rows.items() if n.startswith("mjt_reindex")]
    assert len(red) == 1 and len(rei) == 1
    for r in red + rei:
        assert int(r[2]) == 5 and 0 < float(r[5]) <= float(r[4]) <= float(r[6])       # 1 + rerun launches; min <= avg <= max
    # byte accounting: external inputs and outputs of the group
    total_ns = float(red[0][3])
    assert abs(float(red[0][7]) - 5 * 2 * a.nbytes / (total_ns * 1e-9)) / float(red[0][7]) < 1e-3
    assert np.allclose(y.data, (a.data.astype(np.float64) * b.data + 1).sum(1), rtol=1e-5, atol=1e-3)


def test_matmul_forms_and_relay(gpu):
    """jt.matmul / nn.matmul_transpose / nn.linear build broadcast * broadcast -> sum; 2-d products are
    recognised (the three layouts of opt/tuner/matmul_tuner.cc:33-83) and run as one launch of the GEMM kernel, batched
    and vector forms run on the generic kernels.  Values against numpy in float64."""
    from jittor_amd import nn
    rng = np.random.default_rng(50)
    a = rng.standard_normal((70, 129)).astype(np.float32)
    b = rng.standard_normal((129, 45)).astype(np.float32)
    w = rng.standard_normal((45, 129)).astype(np.float32)
    A, B, W = a.astype(np.float64), b.astype(np.float64), w.astype(np.float64)

    def close(got, want, tol=1e-4):
        return np.allclose(got, want, rtol=tol, atol=tol * np.abs(want).max())

    before = dict(jt.executor_stats)
    assert close(jt.matmul(jt.array(a), jt.array(b)).data, A @ B)
    assert L.last_kernel().startswith("mjt_gemm_")
    assert close(nn.matmul_transpose(jt.array(a), jt.array(w)).data, A @ W.T)
    assert close((jt.array(a) @ jt.array(b)).data, A @ B)
    # the transposed-first layout appears in gradients: sum over axis 0 of [m, n, k]
    at = jt.array(a.T.copy())
    tn = (at.broadcast([129, 70, 45], [2]) * jt.array(b).broadcast([129, 70, 45], [1])).sum(0)
    assert close(tn.data, A @ B)
    assert jt.executor_stats["matmul_matches"] - before["matmul_matches"] == 4
    # bfloat16 operands: float32 accumulation, result narrowed by the cast that follows the sum
    ab, bb = jt.array(a).bfloat16(), jt.array(b).bfloat16()
    got = jt.matmul(ab, bb)
    assert got.dtype == "bfloat16"
    want = O.BF16(ab.raw()).to_f32().astype(np.float64) @ O.BF16(bb.raw()).to_f32().astype(np.float64)
    assert close(got.float32().data, want, 1e-2)
    # the flag switches the relay off: same values from the generic path
    jt.flags["enable_matmul_match"] = False
    try:
        assert close(jt.matmul(jt.array(a), jt.array(b)).data, A @ B)
        assert not L.last_kernel().startswith("mjt_gemm_")
    finally:
        jt.flags["enable_matmul_match"] = True
    # shape rules (python/jittor/nn.py:83-159)
    x = rng.standard_normal((2, 3, 70, 129)).astype(np.float32)
    assert close(jt.matmul(jt.array(x), jt.array(b)).data, x.astype(np.float64) @ B)
    b3 = rng.standard_normal((3, 129, 45)).astype(np.float32)
    assert close(jt.matmul(jt.array(x), jt.array(b3)).data, x.astype(np.float64) @ b3.astype(np.float64))
    assert not L.last_kernel().startswith("mjt_gemm_")                  # a broadcast batch axis: generic kernels
    b4 = rng.standard_normal((2, 3, 129, 45)).astype(np.float32)       # equal batch extents: one strided batched GEMM
    jx, jb4 = jt.array(x), jt.array(b4)
    y4 = jt.matmul(jx, jb4)
    assert close(y4.data, x.astype(np.float64) @ b4.astype(np.float64))
    assert L.last_kernel().startswith("mjt_gemm_")
    gx, gb = jt.grad((y4 * y4).sum(), [jx, jb4])
    Y = x.astype(np.float64) @ b4.astype(np.float64)
    assert close(gx.data, 2 * Y @ np.swapaxes(b4.astype(np.float64), -1, -2), 1e-3)
    assert close(gb.data, np.swapaxes(x.astype(np.float64), -1, -2) @ (2 * Y), 1e-3)
    v = rng.standard_normal(129).astype(np.float32)
    assert close(jt.matmul(jt.array(a), jt.array(v)).data, A @ v.astype(np.float64))
    assert close(jt.matmul(jt.array(v), jt.array(b)).data, v.astype(np.float64) @ B)
    bias = rng.standard_normal(45).astype(np.float32)
    assert close(nn.linear(jt.array(x), jt.array(w), jt.array(bias)).data, x.astype(np.float64) @ W.T + bias)
    # gradients of a product are products again (both are matched)
    ja, jb = jt.array(a), jt.array(b)
    before = dict(jt.executor_stats)
    loss = (jt.matmul(ja, jb) * jt.array(np.ones((70, 45), np.float32))).sum()
    da, db = jt.grad(loss, [ja, jb])
    assert close(da.data, np.ones((70, 45)) @ B.T) and close(db.data, A.T @ np.ones((70, 45)))
    assert jt.executor_stats["matmul_matches"] - before["matmul_matches"] >= 2


def test_histc_ranges(gpu):
    """jt.histc (python/jittor/misc.py:2212-2235): values outside [min, max] are not counted, a value equal
    to max lands in the last bin, N-d inputs are flattened; with min == max == 0 the range is the data's."""
    rng = np.random.default_rng(77)
    x = (rng.integers(-4, 40, (37, 50)) / 8.0 + 1.0 / 16).astype(np.float32)      # well inside the bins
    x[3, :5] = 4.0                                                                # == max
    h = jt.histc(jt.array(x), 8, 0.0, 4.0).data
    want = np.histogram(x, 8, (0.0, 4.0))[0].astype(np.float32)
    assert h.dtype == np.float32 and np.array_equal(h, want)
    assert h.sum() < x.size                                                       # some values were outside
    y = rng.integers(0, 16, 1000).astype(np.float32)                              # default range [0, 15]: 15 equal bins
    h = jt.histc(jt.array(y), 15).data
    want = np.bincount(np.minimum(y.astype(np.int64), 14), minlength=15).astype(np.float32)
    assert np.array_equal(h, want)
    with pytest.raises(RuntimeError):
        jt.histc(jt.array(y), 0)


def test_setitem_and_assign(gpu):
    """x[key] = value (python/jittor/src/ops/setitem_op.cc) for the keys getitem takes, against numpy; ops built
    from the old value keep the old value (lazy graph), gradients flow through the written and the kept part."""
    rng = np.random.default_rng(61)
    a = rng.standard_normal((6, 7, 5)).astype(np.float32)
    cases = [
        (np.s_[2], 1.5), (np.s_[1:4], rng.standard_normal((3, 7, 5)).astype(np.float32)),
        (np.s_[:, ::2, 1], rng.standard_normal((6, 4)).astype(np.float32)), (np.s_[..., -1], 0.0),
        (np.s_[::-2, 3:, :], rng.standard_normal((7 - 3, 5)).astype(np.float32)),          # broadcast along the first axis
        (np.s_[5, 6, 4], 9.0), (np.s_[:, None, 2, :], rng.standard_normal((6, 1, 5)).astype(np.float32)),
    ]
    for key, val in cases:
        want = a.copy()
        want[key] = val
        x = jt.array(a)
        y_before = x * 2                                         # built before the write, evaluated after it
        x[key] = jt.array(val) if isinstance(val, np.ndarray) else val
        assert np.array_equal(x.data, want), key
        assert np.array_equal(y_before.data, a * 2), key
    # one integer Var per axis (distinct positions)
    idx = np.array([4, 0, 2], np.int32)
    v = rng.standard_normal((3, 7, 5)).astype(np.float32)
    x = jt.array(a)
    x[jt.array(idx)] = jt.array(v)
    want = a.copy()
    want[idx] = v
    assert np.array_equal(x.data, want)
    # two index Vars zipped (distinct positions), with a slice behind them
    ia, ib = np.array([5, 0, 3], np.int32), np.array([6, 2, 2], np.int32)
    v2 = rng.standard_normal((3, 2)).astype(np.float32)
    x = jt.array(a)
    x[jt.array(ia), jt.array(ib), 1:3] = jt.array(v2)
    want = a.copy()
    want[ia, ib, 1:3] = v2
    assert np.array_equal(x.data, want)
    # integer data, and a chain of writes
    b = np.arange(24, dtype=np.int32).reshape(4, 6)
    x = jt.array(b)
    x[1:3, ::3] = -1
    x[0] = x[3] + 100
    want = b.copy()
    want[1:3, ::3] = -1
    want[0] = want[3] + 100
    assert np.array_equal(x.data, want)
    # gradients: d/dx of sum(w * x') where x' = x with a slice replaced by 3 * v
    xv, vv = jt.array(a), jt.array(v[0, :3])
    w = rng.standard_normal(a.shape).astype(np.float32)
    x2 = xv * 1.0
    x2[2, 1:4] = vv * 3
    loss = (x2 * jt.array(w)).sum()
    gx, gv = jt.grad(loss, [xv, vv])
    wx = w.copy()
    wx[2, 1:4] = 0
    assert np.allclose(gx.data, wx) and np.allclose(gv.data, 3 * w[2, 1:4])
    # assign: the object takes another Var's value; what was built from the old value keeps it
    p, q = jt.array(a), jt.array(a[::-1].copy())
    s_old = p + 1
    p.assign(q * 2)
    assert np.array_equal(p.data, a[::-1] * 2) and np.array_equal(s_old.data, a + 1)
    assert np.array_equal(jt.array(a)[jt.array(a > 0)].data, a[a > 0])      # a boolean mask: where(mask) as index Vars


def _conv_transpose_ref(x, w, stride, padding, output_padding, dilation):
    """Direct statement of the scatter python/jittor/nn.py:1556-1568 builds, in float64."""
    N, C, H, W = x.shape
    _, O_, kh, kw = w.shape
    ho = (H - 1) * stride + output_padding - 2 * padding + 1 + (kh - 1) * dilation
    wo = (W - 1) * stride + output_padding - 2 * padding + 1 + (kw - 1) * dilation
    full = np.zeros((N, O_, ho + 2 * padding + stride, wo + 2 * padding + stride))
    for r in range(kh):
        for s in range(kw):
            contrib = np.einsum("nihw,io->nohw", x.astype(np.float64), w[:, :, r, s].astype(np.float64))
            full[:, :, r * dilation:r * dilation + (H - 1) * stride + 1:stride, s * dilation:s * dilation + (W - 1) * stride + 1:stride] += contrib
    return full[:, :, padding:padding + ho, padding:padding + wo]


def test_conv_transpose_runs_as_the_input_gradient_pattern(gpu):
    """nn.conv_transpose builds the reference's graph (broadcast x, broadcast w, multiply, reindex_reduce.add); the
    executor takes it for the backward-data pattern and runs it on the convolution kernels: float32 (through the
    product kernel) and bfloat16 (MFMA convolution kernel, one convolution per stride phase), with bias."""
    rng = np.random.default_rng(61)
    for dt, xs, ws, st, pd, op, dl, tol in (("float32", (2, 8, 5, 7), (8, 6, 3, 3), 2, 1, 1, 1, 1e-4),
                                            ("float32", (3, 16, 9, 9), (16, 12, 3, 2), 1, 0, 0, 2, 1e-4),
                                            # bfloat16: the sum and the sum plus bias are each truncated to 8 bits
                                            ("bfloat16", (2, 64, 14, 14), (64, 64, 3, 3), 2, 1, 1, 1, 2.0 ** -6),
                                            ("bfloat16", (2, 64, 12, 16), (64, 128, 3, 3), 1, 1, 0, 1, 2.0 ** -6)):
        x = rng.standard_normal(xs).astype(np.float32)
        w = (rng.standard_normal(ws) * 0.1).astype(np.float32)
        b = rng.standard_normal(ws[1]).astype(np.float32)
        if dt == "bfloat16":
            x, w, b = (O.BF16(O.f32_to_bf16_bits(v)).to_f32() for v in (x, w, b))
        jx, jw, jb = jt.array(x), jt.array(w), jt.array(b)
        if dt == "bfloat16":
            jx, jw, jb = jx.bfloat16(), jw.bfloat16(), jb.bfloat16()
        before = jt.executor_stats["conv_matches"]
        y = jt.nn.conv_transpose(jx, jw, jb, stride=st, padding=pd, output_padding=op, dilation=dl)
        assert y.dtype == dt
        got = y.numpy().astype(np.float32)
        assert jt.executor_stats["conv_matches"] == before + 1, "not taken for the backward-data pattern"
        ref = _conv_transpose_ref(x, w, st, pd, op, dl) + b[None, :, None, None]
        assert got.shape == ref.shape and np.abs(got - ref).max() <= tol * np.abs(ref).max(), (dt, xs)


def test_concat_unfold_fold(gpu):
    rng = np.random.default_rng(62)
    parts = [rng.standard_normal((3, n, 5)).astype(np.float32) for n in (2, 4, 1)]
    assert np.array_equal(jt.concat([jt.array(p) for p in parts], 1).data, np.concatenate(parts, 1))
    assert np.array_equal(jt.concat([jt.array(p) for p in parts], -2).data, np.concatenate(parts, 1))
    assert jt.concat([jt.array([[1], [2]]), jt.array([[2], [2]])], dim=1).data.tolist() == [[1, 2], [2, 2]]    # contrib.py:33-35
    with pytest.raises(ValueError):
        jt.concat([jt.array(parts[0]), jt.array(parts[1])], 0)
    # unfold against windows cut with numpy; fold(unfold(x)) counts how many windows cover each element
    x = rng.standard_normal((2, 3, 9, 8)).astype(np.float32)
    for k, d, p, s in ((3, 1, 1, 2), ((2, 3), (2, 1), (0, 1), (1, 2))):
        kh, kw = (k, k) if isinstance(k, int) else k
        dh, dw = (d, d) if isinstance(d, int) else d
        ph, pw = (p, p) if isinstance(p, int) else p
        sh, sw = (s, s) if isinstance(s, int) else s
        u = jt.nn.unfold(jt.array(x), k, d, p, s)
        xp = np.pad(x, ((0, 0), (0, 0), (ph, ph), (pw, pw)))
        bh = (x.shape[2] + 2 * ph - dh * (kh - 1) - 1) // sh + 1
        bw = (x.shape[3] + 2 * pw - dw * (kw - 1) - 1) // sw + 1
        want = np.zeros((2, 3 * kh * kw, bh * bw), np.float32)
        for c in range(3):
            for r in range(kh):
                for t in range(kw):
                    want[:, (c * kh + r) * kw + t] = xp[:, c, r * dh:r * dh + (bh - 1) * sh + 1:sh, t * dw:t * dw + (bw - 1) * sw + 1:sw].reshape(2, -1)
        assert np.array_equal(u.data, want), (k, d, p, s)
        back = jt.nn.fold(u, (9, 8), k, d, p, s).data
        cover = np.zeros_like(xp)
        for r in range(kh):
            for t in range(kw):
                cover[:, :, r * dh:r * dh + (bh - 1) * sh + 1:sh, t * dw:t * dw + (bw - 1) * sw + 1:sw] += 1
        cover = cover[:, :, ph:ph + 9, pw:pw + 8]
        assert np.allclose(back, x * cover, rtol=1e-5, atol=1e-6), (k, d, p, s)


def test_where_and_boolean_masks(gpu):
    """jt.where(cond) against np.nonzero for several dtypes, ranks and sizes (tile edges of the compaction kernel,
    all-false and all-true inputs); x[mask] and x[mask] = v with boolean masks as the reference's tests use them
    (test/test_setitem.py:204-221)."""
    rng = np.random.default_rng(63)
    for shape, dtype, p in (((10,), "bool", 0.5), ((4096,), "int32", 0.3), ((4097,), "float32", 0.9), ((3, 5, 7), "bool", 0.5),
                            ((70, 300), "float32", 0.01), ((1 << 20,), "bool", 0.5), ((9, 1000), "int8", 1.0), ((5, 5), "bool", 0.0),
                            ((33, 129), "bfloat16", 0.5)):
        m = rng.random(shape) < p
        host = m.astype(np.float32)
        if dtype == "float32":
            host = np.where(m, rng.standard_normal(shape), 0.0).astype(np.float32)
            host.reshape(-1)[::7] *= -0.0                        # -0.0 counts as zero
            if m.any():
                host[tuple(i[0] for i in np.nonzero(m))] = np.nan      # NaN counts as non-zero
        v = jt.array(host.astype(np.float32) if dtype in ("float32", "bfloat16") else m.astype(L.NP_STORAGE[dtype]))
        if dtype == "bfloat16":
            v = v.bfloat16()
        got = jt.where(v)
        want = np.nonzero(host != 0) if dtype == "float32" else np.nonzero(m)
        assert len(got) == len(shape)
        for g, w in zip(got, want):
            assert g.dtype == "int32" and list(g.shape) == [w.size] and np.array_equal(g.numpy(), w.astype(np.int32)), (shape, dtype)
    # where(cond, x, y) is the ternary
    c = jt.array([True, False, True])
    assert jt.where(c, jt.array([1, 2, 3]), jt.array([7, 8, 9])).data.tolist() == [1, 8, 3]
    # masks as keys
    a = jt.array([1, 2, 3, 4])
    b = jt.array([True, False, True, False])
    a[b] = jt.array([-1, -2])
    assert a.data.tolist() == [-1, 2, -2, 4]
    a = jt.array([1, 2, 3, 4])
    a[b] = jt.array([-1])
    assert a.data.tolist() == [-1, 2, -1, 4]
    a = jt.array([1, 2, 3, 4])
    a[b] = -1
    assert a.data.tolist() == [-1, 2, -1, 4]
    x = rng.standard_normal((6, 5, 4)).astype(np.float32)
    jx = jt.array(x)
    assert np.array_equal(jx[jx > 0.5].data, x[x > 0.5])
    rows = x[:, 0, 0] > 0
    assert np.array_equal(jx[jt.array(rows)].data, x[rows])
    assert np.array_equal(jx[jt.array(rows), 1:3].data, x[rows, 1:3])
    m2 = x[0] > 0
    assert np.array_equal(jx[2, jt.array(m2)].data, x[2, m2])
    assert np.array_equal(jx[..., jt.array(m2[0])].data, x[..., m2[0]])
    assert list(jx[jx > 100.0].shape) == [0]
    with pytest.raises(IndexError):
        jx[jt.array(m2)]                                         # [5, 4] does not match axes 0..1 of [6, 5, 4]
    y = x.copy()
    y[y < 0] = 0.0
    jx[jx < 0] = 0.0
    assert np.array_equal(jx.data, y)
