"""A graph that was executed before is replayed from its recorded library calls (the executor's counterpart of the
reference's per-group cache, python/jittor/src/executor.cc:55-110): the results of replayed steps must be the results of
steps executed from scratch, bit for bit, on new data, new scalars and new buffers."""
import numpy as np
import pytest

import jittor_amd as jt
from jittor_amd import executor

pytestmark = pytest.mark.gpu


def _both_ways(step, nsteps=4):
    """step(seed) -> list of arrays; runs nsteps seeds without and with replay and returns (fresh, replayed, replays)"""
    saved = jt.flags["enable_replay"]
    try:
        jt.flags["enable_replay"] = False
        fresh = [step(s) for s in range(nsteps)]
        jt.flags["enable_replay"] = True
        executor._plans.clear()
        r0 = executor.stats["replays"]
        again = [step(s) for s in range(nsteps)]
        return fresh, again, executor.stats["replays"] - r0
    finally:
        jt.flags["enable_replay"] = saved


def _same(fresh, again):
    for s, (fa, ag) in enumerate(zip(fresh, again)):
        assert len(fa) == len(ag)
        for i, (a, b) in enumerate(zip(fa, ag)):
            assert a.shape == b.shape and a.dtype == b.dtype, (s, i)
            assert np.array_equal(a, b, equal_nan=True), (s, i, float(np.abs(a.astype(np.float64) - b.astype(np.float64)).max()))


def test_replayed_cnn_steps_equal_fresh_ones(gpu):
    """A small CNN step (convolution units, pooling and its scatter, strided convolution, matrix product, softmax
    cross-entropy, every gradient; a learning rate that changes from step to step as a by-value scalar)."""
    def step(seed):
        rng = np.random.default_rng(100 + seed)
        x = rng.standard_normal((4, 8, 12, 12)).astype(np.float32)
        w1 = (rng.standard_normal((16, 8, 3, 3)) * 0.2).astype(np.float32)
        w2 = (rng.standard_normal((16, 16, 3, 3)) * 0.2).astype(np.float32)
        wl, bl = (rng.standard_normal((5, 16)) * 0.3).astype(np.float32), rng.standard_normal(5).astype(np.float32)
        onehot = np.eye(5, dtype=np.float32)[rng.integers(0, 5, 4)]
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
        lr = jt.array(np.float32(0.1 / (1 + seed)))
        new_w1 = v1 - grads[1] * lr
        jt.sync([loss, new_w1] + grads)
        return [loss.numpy(), new_w1.numpy()] + [g.numpy() for g in grads]

    fresh, again, replays = _both_ways(step)
    _same(fresh, again)
    assert replays >= 2                                      # the second signature (weights already on the device) repeats
    assert not np.array_equal(again[1][1], again[2][1])      # and the steps did differ


def test_replayed_16bit_steps_with_library_made_buffers(gpu):
    """bfloat16 convolution with both gradients (the input gradient and the weight-gradient kernel make buffers of their own
    inside the library), a float16 matrix product with a reshape that shares memory, a normalisation chain."""
    def step(seed):
        rng = np.random.default_rng(200 + seed)
        x = jt.array(rng.standard_normal((2, 32, 16, 16)).astype(np.float32)).cast("bfloat16")
        w = jt.array((rng.standard_normal((64, 32, 3, 3)) * 0.1).astype(np.float32)).cast("bfloat16")
        y = jt.nn.conv2d(x, w, stride=2, padding=1)
        loss = (y * y).sum()
        gx, gw = jt.grad(loss, [x, w])
        a = jt.array(rng.standard_normal((6, 10, 64)).astype(np.float16))
        b = jt.array(rng.standard_normal((64, 24)).astype(np.float16))
        c = jt.nn.matmul(a, b)                               # rank 3 x rank 2: reshapes around a product
        mean = c.mean([2], keepdims=True)
        var = ((c - mean) * (c - mean)).mean([2], keepdims=True)
        nrm = (c - mean) / jt.unary(var + 1e-3, "sqrt")
        jt.sync([y, gx, gw, nrm])
        return [y.raw(), gx.raw(), gw.raw(), nrm.numpy()]

    fresh, again, replays = _both_ways(step)
    _same(fresh, again)
    assert replays >= 2


def test_replay_float32_weight_gradient_through_column_matrices(gpu):
    """The float32 weight gradient runs as column matrices x dy with buffers the executor makes on the way (column
    matrices, partial sums); getitem / setitem / concat / where results around it."""
    def step(seed):
        rng = np.random.default_rng(300 + seed)
        x = jt.array(rng.standard_normal((3, 6, 10, 10)).astype(np.float32))
        w = jt.array((rng.standard_normal((8, 6, 3, 3)) * 0.2).astype(np.float32))
        y = jt.nn.conv2d(x, w, padding=1)
        gw, = jt.grad((y * y).sum(), [w])
        z = jt.concat([y[:, :4], y[:, 4:] * 2.0], dim=1)
        z[:, 1] = z[:, 0] + 1.0
        pos = jt.where(z > 1.5, z, z * 0.0)
        jt.sync([gw, pos])
        return [gw.numpy(), pos.numpy()]

    fresh, again, replays = _both_ways(step)
    _same(fresh, again)
    assert replays >= 1


def test_replay_16bit_weight_gradient_over_chunks_of_images(gpu):
    """The weight gradient on 14 x 14 maps (planes that are no 16-byte multiples) is one product over chunks of images
    laid side by side: two reindexes into buffers of their own, a batched product, a sum over the chunks."""
    def step(seed):
        rng = np.random.default_rng(400 + seed)
        x = jt.array(rng.standard_normal((8, 32, 14, 14)).astype(np.float32)).cast("bfloat16")
        w = jt.array((rng.standard_normal((64, 32, 3, 3)) * 0.1).astype(np.float32)).cast("bfloat16")
        y = jt.nn.conv2d(x, w, padding=1)
        gx, gw = jt.grad((y * y).sum(), [x, w])
        jt.sync([y, gx, gw])
        return [y.raw(), gx.raw(), gw.raw()]

    before = executor.stats["wgrad_chunked"]
    fresh, again, replays = _both_ways(step)
    _same(fresh, again)
    assert replays >= 2 and executor.stats["wgrad_chunked"] > before


def test_replay_keeps_the_graph_bookkeeping(gpu):
    """After a replayed execution the vars are leaves with buffers of their own, exactly as after a fresh one: a result
    can be reused by a later graph, and two replays never share a result buffer."""
    def step(seed):
        a = jt.array(np.full((64, 64), float(seed + 1), np.float32))
        b = (a * 2.0 + 1.0).sum([1])
        b.sync()
        return a, b

    executor._plans.clear()
    outs = [step(s) for s in range(4)]
    assert executor.stats["replays"] >= 2
    ptrs = {b._device_ptr() for _, b in outs}
    assert len(ptrs) == 4
    for s, (a, b) in enumerate(outs):
        assert b._op is None and b.materialised
        assert np.array_equal(b.numpy(), np.full(64, 64 * (2.0 * (s + 1) + 1.0), np.float32))
        c = (b + 1.0).numpy()                                  # a later graph on a replayed result
        assert np.array_equal(c, b.numpy() + 1.0)
