"""Seeded random differential tests on the GPU: many small random cases of
reduce, reindex / reindex_reduce and fused element-wise chains against the CPU
oracle (oracle/oracle.py).  The shapes are chosen to hit the host-side axis
merging, vector-width selection, split reductions and the generic index
kernels with odd extents."""
import numpy as np
import pytest

import jittor_amd as jt
from oracle import oracle as O

pytestmark = pytest.mark.gpu


def _shape(rng, max_rank=5, max_elems=40000):
    while True:
        rank = int(rng.integers(1, max_rank + 1))
        s = [int(rng.choice([1, 2, 3, 4, 5, 7, 8, 16, 17, 31, 32, 64, 100])) for _ in range(rank)]
        if np.prod(s) <= max_elems:
            return s


def test_random_reduce(gpu):
    rng = np.random.default_rng(1000)
    ops_f = ["add", "maximum", "minimum", "mean", "multiply"]
    ops_i = ["add", "maximum", "minimum", "bitwise_and", "bitwise_or", "bitwise_xor"]
    for case in range(150):
        shape = _shape(rng)
        rank = len(shape)
        dims = sorted(set(int(d) for d in rng.integers(0, rank, int(rng.integers(0, rank + 1)))))
        keep = bool(rng.integers(0, 2))
        if rng.random() < 0.6:
            x = rng.uniform(0.5, 1.5, shape).astype(np.float32)
            op = ops_f[int(rng.integers(len(ops_f)))]
            if op == "multiply" and np.prod(shape) > 64:
                op = "add"
            got = jt.array(x).reduce(op, dims, keep).data
            want = O.reduce(x, op, dims, keep)
            assert got.shape == want.shape, (case, shape, dims, keep, op)
            assert np.allclose(got, want, rtol=2e-5, atol=1e-5), (case, shape, dims, keep, op)
        else:
            x = rng.integers(-50, 50, shape).astype(np.int32)
            op = ops_i[int(rng.integers(len(ops_i)))]
            got = jt.array(x).reduce(op, dims, keep).data
            want = O.reduce(x, op, dims, keep)
            assert got.dtype == want.dtype and np.array_equal(got, want), (case, shape, dims, keep, op)


def _random_index_expr(rng, yrank, xextent):
    """An integer expression of the output coordinates: affine with small coefficients, sometimes with
    division, remainder or a conditional; results may fall outside [0, xextent) (overflow)."""
    terms = []
    for k in range(yrank):
        c = int(rng.integers(-2, 3))
        if c:
            terms.append("%d*i%d" % (c, k) if c != 1 else "i%d" % k)
    e = "+".join(terms) if terms else "0"
    e = "(%s%+d)" % (e, int(rng.integers(-2, 3)))
    r = rng.random()
    if r < 0.2:
        e = "(%s)/%d" % (e, int(rng.integers(2, 4)))
    elif r < 0.4:
        e = "(%s)%%%d" % (e, max(1, xextent))
    elif r < 0.5:
        e = "(i0<%d ? %s : %d)" % (int(rng.integers(1, 4)), e, int(rng.integers(0, max(1, xextent))))
    return e


def test_random_reindex_and_reindex_reduce(gpu):
    rng = np.random.default_rng(2000)
    for case in range(120):
        xshape = _shape(rng, 3, 3000)
        yshape = _shape(rng, 4, 6000)
        idx = [_random_index_expr(rng, len(yshape), xshape[d]) for d in range(len(xshape))]
        ofc = ["i0>%d" % int(rng.integers(0, 6))] if rng.random() < 0.3 else []
        if rng.random() < 0.5:
            x = rng.integers(-1000, 1000, xshape).astype(np.int32)
        else:
            x = rng.standard_normal(xshape).astype(np.float32)
        ov = float(rng.integers(-3, 4))
        got = jt.array(x).reindex(yshape, idx, ov, ofc).data
        want = O.reindex(x, yshape, idx, ov, ofc)
        assert got.dtype == want.dtype and np.array_equal(got, want), (case, xshape, yshape, idx, ofc)
        # the same index program as a scatter: y (shape yshape) reduced into xshape
        y = rng.integers(-20, 20, yshape).astype(np.int32)
        op = ["add", "maximum", "minimum"][int(rng.integers(3))]
        got = jt.array(y).reindex_reduce(op, xshape, idx, ofc).data
        want = O.reindex_reduce(y, op, xshape, idx, ofc)
        assert np.array_equal(got, want), (case, op, xshape, yshape, idx, ofc)


def test_random_fused_chains(gpu):
    rng = np.random.default_rng(3000)
    un = ["negative", "abs", "exp", "sigmoid", "tanh", "sqrt", "floor", "sin"]
    bi = ["add", "subtract", "multiply", "maximum", "minimum", "divide"]
    for case in range(80):
        shape = _shape(rng, 4, 20000)
        n_in = int(rng.integers(1, 4))
        host, dev, ref = [], [], []
        for k in range(n_in):
            # full-shape inputs or inputs broadcast along a random subset of axes
            bshape = [s if rng.random() < 0.7 else 1 for s in shape]
            a = rng.uniform(0.5, 2.0, bshape).astype(np.float32)
            host.append(a)
            dev.append(jt.array(a))
            ref.append(a)
        vals, refs = list(dev), list(ref)
        for step in range(int(rng.integers(1, 7))):
            if rng.random() < 0.4:
                op = un[int(rng.integers(len(un)))]
                i = int(rng.integers(len(vals)))
                vals.append(vals[i].unary(op))
                refs.append(O.unary(refs[i], op))
            else:
                op = bi[int(rng.integers(len(bi)))]
                i, j = int(rng.integers(len(vals))), int(rng.integers(len(vals)))
                vals.append(jt.binary(vals[i], vals[j], op))
                a, b = np.broadcast_arrays(refs[i], refs[j])
                refs.append(O.binary(np.ascontiguousarray(a), np.ascontiguousarray(b), op))
        got = vals[-1].data
        want = refs[-1]
        assert got.shape == want.shape, (case, shape)
        assert np.allclose(got, want, rtol=3e-5, atol=1e-6, equal_nan=True), (case, shape, np.abs(got - want).max())


def test_random_graphs_of_element_reduce_and_broadcast_ops(gpu):
    """Random DAGs mixing element-wise ops, reduces with keepdims and the broadcasts that bring their results
    back to the full shape (normalisation-like chains), several results fetched at once: what the executor
    makes of them -- prologues, ops evaluated behind a broadcast, ops delayed to their consumers' stage -- must
    not change any value.  Checked against the same DAG evaluated by numpy in float64."""
    rng = np.random.default_rng(3000)
    before = dict(jt.executor_stats)
    unary = {"negative": np.negative, "abs": np.abs, "exp": lambda a: np.exp(np.clip(a, -20, 3)), "sigmoid": None,
             "sqrt": lambda a: np.sqrt(np.abs(a))}
    for case in range(60):
        rank = int(rng.integers(2, 4))
        shape = [int(rng.choice([2, 3, 5, 8, 17, 32, 65])) for _ in range(rank)]
        pairs = []                                                        # (Var, float64 array)
        for _ in range(int(rng.integers(1, 4))):
            a = rng.uniform(-1.5, 1.5, shape).astype(np.float32)
            pairs.append((jt.array(a), a.astype(np.float64)))

        def pick(full_only=False):
            cand = [p for p in pairs if not full_only or list(p[1].shape) == shape]
            return cand[int(rng.integers(len(cand)))]

        for step in range(int(rng.integers(4, 14))):
            r = rng.random()
            if r < 0.3:
                name = list(unary)[int(rng.integers(len(unary)))]
                v, a = pick()
                if name == "sigmoid":
                    pairs.append((jt.unary(v, "sigmoid"), 1.0 / (1.0 + np.exp(-a))))
                elif name == "exp":
                    pairs.append((jt.unary(v.minimum(3.0).maximum(-20.0), "exp"), unary[name](a)))
                elif name == "sqrt":
                    pairs.append((jt.unary(jt.unary(v, "abs"), "sqrt"), unary[name](a)))
                else:
                    pairs.append((jt.unary(v, name), unary[name](a)))
            elif r < 0.65:
                (v, a), (w, b) = pick(), pick()
                op = ["add", "subtract", "multiply", "maximum"][int(rng.integers(4))]
                f = {"add": np.add, "subtract": np.subtract, "multiply": np.multiply, "maximum": np.maximum}[op]
                pairs.append((jt.binary(v, w, op), f(a, b)))
            elif r < 0.8:
                v, a = pick()
                k = float(rng.uniform(0.5, 2.0))
                pairs.append((v * k + 0.25, a * np.float32(k) + 0.25))
            else:
                v, a = pick(full_only=True)
                dims = sorted(set(int(d) for d in rng.integers(0, rank, int(rng.integers(1, rank)))))
                op = ["add", "maximum", "mean"][int(rng.integers(3))]
                f = {"add": np.sum, "maximum": np.max, "mean": np.mean}[op]
                pairs.append((v.reduce(op, dims, True), f(a, axis=tuple(dims), keepdims=True)))
        nout = int(rng.integers(1, 4))
        chosen = [pairs[-1 - i] for i in range(min(nout, len(pairs)))]
        got = jt.fetch_sync([v for v, _ in chosen])
        for g, (_, want) in zip(got, chosen):
            assert list(g.shape) == list(want.shape), (case, g.shape, want.shape)
            scale = max(1.0, float(np.abs(want).max()))
            assert np.allclose(g, want, rtol=2e-4, atol=2e-4 * scale), (case, float(np.abs(g - want).max()), scale)
    assert jt.executor_stats["sunk_ops"] > before["sunk_ops"] and jt.executor_stats["fused_reduces"] > before["fused_reduces"]
