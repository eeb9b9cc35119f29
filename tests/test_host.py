"""Host-side logic without a GPU: the C-ABI library loads and exports every
symbol include/mjt.h declares, descriptors are validated, index expressions
parse as the reference's language, the front end reproduces the constructor
rewrites / dtype rules, and kernels specialise + compile for gfx950."""
import ctypes
import json
import os
import re

import numpy as np
import pytest

import jittor_amd as jt
from jittor_amd import _lib as L

G = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "vectors.json")))
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
P = 0x100000     # fake, aligned device pointer: nothing is launched in compile-only mode


def test_library_exports_every_declared_symbol():
    lib = L.load()
    header = open(os.path.join(ROOT, "include", "mjt.h")).read()
    declared = set(re.findall(r"\b(mjt_[a-z0-9_]+)\s*\(", header))
    assert declared == set(L.EXPORTS), declared ^ set(L.EXPORTS)
    for name in declared:
        assert hasattr(lib, name), name


def test_names_and_codes():
    lib = L.load()
    for i, n in enumerate(L.DTYPES):
        assert lib.mjt_dtype_name(i).decode() == n
    for i, n in enumerate(L.OPS):
        assert lib.mjt_op_name(i).decode() == n
    assert lib.mjt_op_from_name(b"add") == L.OP_CODE["add"]
    assert lib.mjt_op_from_name(b"nope") < 0
    assert lib.mjt_dtype_from_name(b"bfloat16") == L.DTYPE_CODE["bfloat16"]


def test_calls_fail_cleanly_without_init():
    L.shutdown()
    lib = L.load()
    x = L.tensor(P, "float32", [4])
    assert lib.mjt_reduce(ctypes.byref(x), ctypes.byref(x), 3, 1) == -5
    assert b"mjt_init" in lib.mjt_last_error()


def test_expr_affine_and_errors():
    assert L.expr_affine("i3*2-1+i5*3", (4, 5, 6, 7), (1, 2, 3, 4, 5, 6)) == (-1, [0, 0, 0, 2, 0, 3, 0, 0, 0, 0])
    assert L.expr_affine("xshape0-1-i0", (4,), (4,)) == (3, [-1] + [0] * 9)
    assert L.expr_affine("(i1-i3)/2", (4, 4), (4, 4, 4, 4)) is None
    assert L.expr_affine("7/2*i0 + (0-7)/2", (4,), (4,)) == (-3, [3] + [0] * 9)   # C division truncates
    assert L.expr_affine("0x10 + 0b11", (4,), (4,)) == (19, [0] * 10)
    assert L.expr_affine("@e0(i0)", (4,), (4,)) is None
    with pytest.raises(L.MjtError):
        L.expr_affine("i0 // 2", (4,), (4,))
    with pytest.raises(L.MjtError):
        L.expr_affine("i0 +", (4,), (4,))


def test_descriptor_validation(compile_only):
    lib = compile_only.load()
    e = L.c_strings([])
    x, y = L.tensor(P, "float32", [10, 10]), L.tensor(P, "float32", [8, 8])
    # number of indexes must equal x rank (ops/reindex_op.cc:83)
    assert lib.mjt_reindex(ctypes.byref(x), ctypes.byref(y), 1, L.c_strings(["i0"]), 0.0, 0, e, 0, None) == -1
    # '//' is rejected (opt/pass/loop_var_analyze_pass.cc:298-309)
    ex = (L.Tensor * 1)(L.tensor(P, "int32", [1]))
    assert lib.mjt_reindex(ctypes.byref(x), ctypes.byref(y), 2, L.c_strings(["@e0(0) // 1", "@e0(0)"]), 0.0, 0, e, 1, ex) == -1
    # unknown identifier, @eK arity, missing extra
    assert lib.mjt_reindex(ctypes.byref(x), ctypes.byref(y), 2, L.c_strings(["i5", "i0"]), 0.0, 0, e, 0, None) == -1
    assert lib.mjt_reindex(ctypes.byref(x), ctypes.byref(y), 2, L.c_strings(["@e0(i0,i1)", "i0"]), 0.0, 0, e, 1, ex) == -1
    assert lib.mjt_reindex(ctypes.byref(x), ctypes.byref(y), 2, L.c_strings(["@e1(0)", "i0"]), 0.0, 0, e, 1, ex) == -1
    # reindex_reduce: op must be binary and not mean; indexes == rank of the output
    v, o = L.tensor(P, "float32", [3]), L.tensor(P, "float32", [3])
    assert lib.mjt_reindex_reduce(ctypes.byref(v), ctypes.byref(o), L.OP_CODE["mean"], 1, L.c_strings(["i0"]), 0, e, 0, None) == -1
    assert lib.mjt_reindex_reduce(ctypes.byref(v), ctypes.byref(o), L.OP_CODE["exp"], 1, L.c_strings(["i0"]), 0, e, 0, None) == -1
    assert lib.mjt_reindex_reduce(ctypes.byref(v), ctypes.byref(o), L.OP_CODE["add"], 2, L.c_strings(["i0", "i0"]), 0, e, 0, None) == -1
    # reduce: mask must fit, element counts must agree, op must be associative
    big, small = L.tensor(P, "float32", [4, 5]), L.tensor(P, "float32", [4])
    assert lib.mjt_reduce(ctypes.byref(big), ctypes.byref(small), L.OP_CODE["add"], 0b100) == -1
    assert lib.mjt_reduce(ctypes.byref(big), ctypes.byref(small), L.OP_CODE["add"], 0b01) == -1
    assert lib.mjt_reduce(ctypes.byref(big), ctypes.byref(small), L.OP_CODE["subtract"], 0b10) == -1
    assert lib.mjt_reduce(ctypes.byref(big), ctypes.byref(small), L.OP_CODE["add"], 0b10) == 0


def _fused(lib, shape, vars_, ops_):
    va = (L.FusedVar * len(vars_))()
    for i, (role, dt_, mask) in enumerate(vars_):
        va[i].role, va[i].dtype, va[i].ptr, va[i].bcast_mask = role, L.DTYPE_CODE[dt_], P, mask
    oa = (L.FusedOp * len(ops_))()
    for i, (kind, op, ins, out) in enumerate(ops_):
        oa[i].kind, oa[i].op, oa[i].out = kind, L.OP_CODE[op] if op else 0, out
        for j, v in enumerate(ins):
            oa[i].inp[j] = v
    d = L.FusedDesc()
    d.ndim = len(shape)
    for i, s in enumerate(shape):
        d.shape[i] = s
    d.n_vars, d.vars, d.n_ops, d.ops = len(vars_), va, len(ops_), oa
    return lib.mjt_fused_elementwise(ctypes.byref(d))


def test_kernels_specialise_for_gfx950(compile_only):
    """Compile-only mode builds the same kernels a GPU run would launch."""
    lib = compile_only.load()
    e = L.c_strings([])
    before = L.jit_stats()[0]
    os.environ["MJT_NO_DISK_CACHE"] = "1"
    try:
        # the five benchmark shapes
        x, y = L.tensor(P, "float32", [8192, 4096]), L.tensor(P, "float32", [8192])
        assert lib.mjt_reduce(ctypes.byref(x), ctypes.byref(y), L.OP_CODE["add"], 0b10) == 0, lib.mjt_last_error()
        assert L.last_kernel().startswith("mjt_reduce_row_add")
        x, y = L.tensor(P, "float32", [32, 64, 56, 56]), L.tensor(P, "float32", [32, 64, 56, 56, 3, 3])
        assert lib.mjt_reindex(ctypes.byref(x), ctypes.byref(y), 4, L.c_strings(["i0", "i1", "i2+i4-1", "i3+i5-1"]),
                               0.0, 0, e, 0, None) == 0, lib.mjt_last_error()
        assert L.last_kernel().startswith("mjt_window_gather")
        v, o = L.tensor(P, "float32", [1 << 24]), L.tensor(P, "float32", [1 << 20])
        ex = (L.Tensor * 1)(L.tensor(P, "int32", [1 << 24]))
        for op in ("add", "maximum"):
            assert lib.mjt_reindex_reduce(ctypes.byref(v), ctypes.byref(o), L.OP_CODE[op], 1, L.c_strings(["@e0(i0)"]),
                                          0, e, 1, ex) == 0, lib.mjt_last_error()
            assert L.last_kernel().startswith("mjt_scatter1d_" + op)
        vars_ = [(0, "float32", 0), (0, "float32", 0b101), (0, "float32", 0b011), (3, "float32", 0),
                 (1, "float32", 0), (1, "float32", 0), (1, "bool", 0), (1, "float32", 0), (1, "float32", 0),
                 (1, "float32", 0), (1, "float32", 0), (2, "float32", 0)]
        ops_ = [(1, "multiply", [0, 1], 4), (1, "add", [4, 2], 5), (1, "greater", [5, 3], 6), (2, None, [6, 5, 3], 7),
                (0, "negative", [7], 8), (0, "exp", [8], 9), (0, "sigmoid", [0], 10), (1, "multiply", [9, 10], 11)]
        assert _fused(lib, [64, 512, 1024], vars_, ops_) == 0, lib.mjt_last_error()
        # a generic gather with extras and a generic scatter
        x, y = L.tensor(P, "float32", [10, 10]), L.tensor(P, "float32", [8, 8])
        ex2 = (L.Tensor * 2)(L.tensor(P, "int32", [1]), L.tensor(P, "float32", [10, 10]))
        assert lib.mjt_reindex(ctypes.byref(x), ctypes.byref(y), 2, L.c_strings(["@e0(0)", "@e1(0,i0 / @e0(0))"]),
                               0.0, 0, e, 2, ex2) == 0, lib.mjt_last_error()
        yy, xx = L.tensor(P, "int16", [3, 10, 10, 4]), L.tensor(P, "int16", [3, 4, 4, 4])
        assert lib.mjt_reindex_reduce(ctypes.byref(yy), ctypes.byref(xx), L.OP_CODE["multiply"], 4,
                                      L.c_strings(["i0", "i1/3", "i2/3", "i3"]), 0, e, 0, None) == 0, lib.mjt_last_error()
    finally:
        del os.environ["MJT_NO_DISK_CACHE"]
    assert L.jit_stats()[0] >= before + 7


def test_fused_graph_validation(compile_only):
    lib = compile_only.load()
    # op reads a var that is produced later
    assert _fused(lib, [8], [(0, "float32", 0), (1, "float32", 0), (2, "float32", 0)],
                  [(0, "exp", [1], 2), (0, "exp", [0], 1)]) == -1
    # output never produced
    assert _fused(lib, [8], [(0, "float32", 0), (2, "float32", 0), (2, "float32", 0)], [(0, "exp", [0], 1)]) == -1
    # binary op code in a unary slot
    assert _fused(lib, [8], [(0, "float32", 0), (2, "float32", 0)], [(0, "add", [0], 1)]) == -1


# ---- front end: constructor rewrites, shapes, dtypes, errors ---------------------------
def _count_ops(v, kind):
    seen, stack, n = set(), [v], 0
    while stack:
        u = stack.pop()
        if u._op is None or u._op.id in seen:
            continue
        seen.add(u._op.id)
        n += u._op.kind == kind
        stack.extend(u._op.inputs)
    return n


def test_binary_inserts_broadcasts_like_the_reference():
    # test/test_broadcast_to_op.py:64-101: 0, 1 or 2 broadcast ops
    a = jt.array([1, 2, 3])
    assert _count_ops(a + 1, "broadcast") == 1
    assert _count_ops(a + a, "broadcast") == 0
    x, y = jt.zeros([3, 1]), jt.zeros([1, 4])
    z = x + y
    assert z.shape == [3, 4] and _count_ops(z, "broadcast") == 2
    assert (jt.zeros([5, 4]) + jt.zeros([4])).shape == [5, 4]
    with pytest.raises(ValueError):
        jt.zeros([3, 4]) + jt.zeros([3, 5])


def test_broadcast_shapes_and_forwarding():
    a = jt.array([1, 2])
    assert a.broadcast([2, 2], [-1]).shape == [2, 2]
    assert a.broadcast([2]) is a                              # forward(x): nothing to broadcast
    assert jt.zeros([512, 1]).broadcast([64, 512, 1024])._op.bcast_mask == 0b101
    assert jt.zeros([1, 1024]).broadcast([64, 512, 1024])._op.bcast_mask == 0b011
    w = jt.zeros([256, 256, 3, 3]).broadcast([64, 256, 256, 56, 56, 3, 3], [0, 3, 4])
    assert w.shape == [64, 256, 256, 56, 56, 3, 3] and w._op.bcast_mask == 0b0011001
    with pytest.raises(ValueError):
        a.broadcast([2, 2], [5])


def test_reduce_shapes_rewrites_and_errors():
    a = jt.array([[1, 2], [3, 4]])
    assert a.sum(-1).shape == [2] and a.sum(-1)._op.reduce_mask == 0b10
    assert a.sum(-2)._op.reduce_mask == 0b01
    assert a.sum().shape == [1] and a.sum().is_scalar
    assert a.sum(1, keepdims=True).shape == [2, 1]
    assert jt.zeros([2, 3, 4, 5]).sum([1, 3]).shape == [2, 4]
    with pytest.raises(ValueError):
        jt.reduce_add(jt.array([1, 2, 3]), 2)                 # test/test_reduce_op.py:50
    h = jt.zeros([4, 4]).bfloat16().sum(1)                    # cast -> reduce(float32) -> cast
    assert h.dtype == "bfloat16" and h._op.kind == "unary" and h._op.inputs[0].dtype == "float32"
    assert jt.array([True, False]).sum().dtype == "int32"
    assert len([n for n in dir(jt) if n.startswith("reduce_")]) >= 10


def test_dtype_rules_of_the_front_end():
    for op, x, y, xs, ys, want in G["dtype_table"]["rows"]:
        assert jt.dtypes.binary_dtype_infer(op, x, y, xs, ys) == want
    a = jt.array([1.0, 2.0, 3.0]).bfloat16()
    assert (a * 1).dtype == "bfloat16"                        # test/test_bf16.py:275-281
    assert (a * jt.array([1.0, 2.0, 3.0])).dtype == "float32"
    assert (a * jt.array([1.0, 2.0, 3.0]).sum()).dtype == "bfloat16"
    assert jt.array([0, 1, 0]).ternary(a, jt.array(1.0)).dtype == "bfloat16"
    assert (a ** a).dtype == "float32"
    i = jt.array([1, 2, 3])
    assert i.dtype == "int32" and jt.array([1.5]).dtype == "float32" and jt.array(np.arange(4, dtype=np.uint8)).dtype == "uint8"
    assert (i / 2).dtype == "float32" and (i // 2).dtype == "int32" and (i < 2).dtype == "bool"
    assert i.sqrt().dtype == "float32" and i.float16().exp().dtype == "float32" and i.float32().round_int().dtype == "int32"
    assert (i.float64() + 1).dtype == "float64"
    assert i.int32() is i                                      # unary_op.cc:867-870 forwards


def test_amp_reg_controls_dtype_inference():
    """The mixed-precision register (nano_string.h:199-277, var.cc:65-71), with the cases the reference checks
    in test/test_fp16.py:208-300: reduce keeps 16 bit only with keep_reduce, white-list ops only with
    keep_white, prefer16 / prefer32 steer float results unless an operand is a scalar, array-like ops follow
    with array_prefer, and conv2d builds its sum under amp_reg | 36 (nn.py:1250)."""
    a = jt.array(np.ones((3, 4), np.float32)).float16()
    assert jt.flags.amp_reg == 0
    for reg in (0, 1, 2):
        with jt.flag_scope(amp_reg=reg):
            assert a.maximum(a).max().dtype == "float32"                  # reduce_dtype_infer
            assert (a ** a).dtype == "float32"                            # white list
    with jt.flag_scope(amp_reg=2 + 4):
        assert a.sum().dtype == "float16" and a.max().dtype == "float16"  # test_fp16.py:248-252
    with jt.flag_scope(amp_reg=4):
        s = a.sum()
        assert s.dtype == "float16" and s._op.kind == "unary"             # still cast -> reduce(float32) -> cast
        assert a.max().dtype == "float16" and a.max()._op.kind == "reduce"
    with jt.flag_scope(amp_reg=4 + 32):
        s = a.sum()
        assert s.dtype == "float16" and s._op.kind == "reduce" and s._op.amp == 36
    with jt.flag_scope(amp_reg=2 + 8):
        assert (a ** a).dtype == "float16" and a.exp().dtype == "float16"
    with jt.flag_scope(amp_reg=1):
        assert a.sqrt().dtype == "float32" and (a + a).dtype == "float32"
        assert (a * 2.0).dtype == "float16"                               # a scalar operand does not count
    f = jt.array(np.ones((3, 4), np.float32))
    with jt.flag_scope(amp_reg=2):
        assert (f + f).dtype == "float16" and f.sqrt().dtype == "float16"
    assert jt.array([1.0, 2.0]).dtype == "float32"
    with jt.flag_scope(amp_reg=2 + 16):
        assert jt.array([1.0, 2.0]).dtype == "float16" and jt.array([1.0]).dtype == "float32"
    with jt.flag_scope(amp_level=3):                                      # test_fp16.py:293-299
        assert jt.flags.amp_reg == 12
        assert a.sum().dtype == "float16" and a.mean().dtype == "float16"
        assert a.log().dtype == "float16" and a.exp().dtype == "float16"
    assert jt.flags.amp_reg == 0 and jt.flags.auto_mixed_precision_level == 0
    # conv2d: 16-bit operands give a 16-bit sum without casts; the gradient inherits the register
    x, w = jt.zeros([2, 3, 8, 8]).bfloat16(), jt.zeros([4, 3, 3, 3]).bfloat16()
    y = jt.nn.conv2d(x, w, padding=1)
    assert y.dtype == "bfloat16" and y._op.kind == "reduce" and y._op.amp & 36 == 36
    gw = jt.grad(y.sum(), w)
    assert gw.dtype == "bfloat16" and gw._op.kind == "reduce" and gw._op.reduce_mask == 0b0011001
    assert jt.flags.amp_reg == 0
    with pytest.raises(KeyError):
        jt.flags["no_such_flag"] = 1


def test_reindex_constructor_checks():
    x = jt.zeros([10, 10])
    with pytest.raises(ValueError):
        x.reindex([8, 8], ["i0"])
    y = x.reindex_var([jt.zeros([4, 5]).int32(), jt.zeros([4, 5]).int32()])
    assert y.shape == [4, 5] and y._op.indexes == ["@e0(i0,i1)", "@e1(i0,i1)"]
    v = jt.zeros([3])
    v.reindex_reduce("add", [3], ["i0"])
    for bad in (lambda: v.reindex_reduce("add", [3], []), lambda: v.reindex_reduce("add", [3], ["i0", "i0"]),
                lambda: v.reindex_reduce("???", [3], ["i0"]), lambda: v.reindex_reduce("add", [-1], ["i0"])):
        with pytest.raises(ValueError):
            bad()                                              # test/test_reindex_reduce_op.py:92-97


def test_conv2d_builds_the_meta_op_group():
    x, w = jt.zeros([2, 3, 8, 8]), jt.zeros([4, 3, 3, 3])
    y = jt.nn.conv2d(x, w, padding=1)
    assert y.shape == [2, 4, 8, 8] and y._op.kind == "reduce" and y._op.reduce_mask == 0b1100100
    mul = y._op.inputs[0]._op
    assert mul.kind == "binary" and {i._op.kind for i in mul.inputs} == {"reindex", "broadcast"}
    r = [i for i in mul.inputs if i._op.kind == "reindex"][0]._op
    assert r.indexes == ["i0", "i2", "i3*1-1+i5*1", "i4*1-1+i6*1"]
    assert jt.nn.conv2d(x, w, stride=2, padding=1).shape == [2, 4, 4, 4]


# ---- gradients: graph construction (no execution) -------------------------------------------
def test_grad_graph_is_built_from_path_ops():
    """The gradient of a meta-op is again a meta-op of the path
    (reindex_op.cc:76-80, reindex_reduce_op.cc:45-63, reduce_op.cc:339-362,
    broadcast_to_op.cc:112-117)."""
    import jittor_amd as jt
    from jittor_amd import core
    x = jt.array(np.zeros((2, 3, 8, 8), np.float32))
    xx = x.reindex([2, 3, 4, 4, 2, 2], ["i0", "i1", "i2*2+i4", "i3*2+i5"], overflow_conditions=["i2<0"])
    g = jt.grad(xx.sum(), x)
    assert isinstance(g._op, core.ReindexReduceOp) and g._op.op == "add" and g.shape == x.shape
    assert g._op.indexes == xx._history[0].indexes and g._op.overflow_conditions == ["i2<0"]
    y = x.reindex_reduce("add", [2, 3, 4, 4], ["i0", "i1", "i2/2", "i3/2"])
    g = jt.grad(y.sum(), x)
    assert isinstance(g._op, core.ReindexOp) and g.shape == x.shape and g._op.overflow_value == 0
    g = jt.grad(x.sum([1, 3]).sum(), x)                    # reduce -> broadcast (of the ones seed)
    assert g.shape == x.shape and isinstance(g._op, core.BroadcastOp)
    s = jt.array(np.zeros((3, 1, 1), np.float32))
    g = jt.grad((x * s).sum(), s)                          # broadcast -> reduce add
    assert g.shape == [3, 1, 1] and isinstance(g._op, core.ReduceOp) and g._op.op == "add"
    # only float targets and losses; untouched targets get zeros of their shape
    with pytest.raises(ValueError):
        jt.grad(x.sum(), jt.array([1, 2]))
    z = jt.grad(x.sum(), s)
    assert z.shape == s.shape
    # history is dropped by stop_grad and under no_grad
    assert (x * 2).stop_grad()._history is None
    with jt.no_grad():
        assert (x * 2)._history is None
    # the gradient of a reshape is the reshape back (ops/reshape_op.cc): again a reindex that shares memory, no scatter
    g = jt.grad((x.reshape([6, 64]) * 3.0).sum(), x)
    assert isinstance(g._op, core.ReindexOp) and getattr(g._op, "same_memory", False) and g.shape == x.shape


def test_assign_of_a_python_number_leaves_the_shared_scalar_alone():
    """Python numbers are kept as one host Var per value; x.assign(2.0) must rebind x to an array of its own and
    leave that shared Var a plain constant: a later `w * 2.0` does not depend on x (its gradient w.r.t. x is the
    zeros of an untouched target), and the constant stays a by-value scalar without a producing op."""
    import jittor_amd as jt
    from jittor_amd import core
    x = jt.array(np.ones(3, np.float32))
    w = jt.array(np.ones(3, np.float32))
    shared = core._as_var(2.0)
    x.assign(2.0)
    assert core._as_var(2.0) is shared and shared._op is None and shared._history is None
    assert x.shape == [1] and not any(v is x for v in (shared._op.inputs if shared._op else ()))
    loss = (w * 2.0).sum()
    g = jt.grad(loss, [x])[0]
    assert g.shape == x.shape and not isinstance(g._op, (core.ReindexReduceOp, core.ReindexOp))   # zeros, not a gradient path
    z = jt.array(np.zeros(2, np.float32))
    z.assign(2.0)
    assert z._op is None or z._op.inputs == []          # an array of its own, not an alias of x


def test_fused_reduce_descriptor_checks_and_specialisation(compile_only):
    """mjt_fused_reduce: one output var (the reduce input); inputs are full-shape or broadcast along exactly
    the reduced axes (one value per output); the kernel with the prologue compiles for gfx950."""
    L = compile_only
    lib = L.load()
    V, F = L.FusedVar, L.FusedOp

    def desc(mask=0, outputs=1):
        spec = [(0, "float32", 0x1000, 0), (0, "float32", 0x2000, mask), (3, "float32", None, 0), (1, "float32", None, 0),
                (2, "float32", None, 0)]
        if outputs == 2:
            spec[3] = (2, "float32", None, 0)
        va = (V * len(spec))()
        for i, (role, dt_, ptr, m) in enumerate(spec):
            va[i].role, va[i].dtype, va[i].ptr, va[i].bcast_mask = role, L.DTYPE_CODE[dt_], ptr, m
        va[2].fvalue = 0.5
        ops = [(1, "multiply", [0, 1], 3), (1, "add", [3, 2], 4)]
        oa = (F * len(ops))()
        for i, (kind, op, ins, out) in enumerate(ops):
            oa[i].kind, oa[i].op, oa[i].out = kind, L.OP_CODE[op], out
            for j, u in enumerate(ins):
                oa[i].inp[j] = u
        d = L.FusedDesc()
        d.ndim = 2
        d.shape[0], d.shape[1] = 64, 256
        d.n_vars, d.vars, d.n_ops, d.ops = len(spec), va, len(ops), oa
        return d, (va, oa)

    ty = L.tensor(0x3000, "float32", [64])
    d, keep = desc()
    assert lib.mjt_fused_reduce(ctypes.byref(d), ctypes.byref(ty), L.OP_CODE["add"], 0b10) == 0
    assert "_pro" in L.last_kernel() and L.last_kernel().startswith("mjt_reduce_row_add")
    ty0 = L.tensor(0x3000, "float32", [256])
    assert lib.mjt_fused_reduce(ctypes.byref(d), ctypes.byref(ty0), L.OP_CODE["maximum"], 0b01) == 0
    # (the column kernel; when it splits the rows among workgroups, its partial results are folded by the row kernel)
    assert L.last_kernel().startswith("mjt_reduce_col_maximum") or L.last_kernel().startswith("mjt_reduce_row_maximum") and L.last_kernel().endswith("_fold")
    d, keep = desc(mask=0b01)                                    # broadcast along a kept axis
    assert lib.mjt_fused_reduce(ctypes.byref(d), ctypes.byref(ty), L.OP_CODE["add"], 0b10) == -2
    d, keep = desc(mask=0b10)                                    # one value per output: row and column kernels
    assert lib.mjt_fused_reduce(ctypes.byref(d), ctypes.byref(ty), L.OP_CODE["add"], 0b10) == 0
    assert L.last_kernel().startswith("mjt_reduce_row_add") and "_pro" in L.last_kernel()
    d, keep = desc(mask=0b01)
    assert lib.mjt_fused_reduce(ctypes.byref(d), ctypes.byref(ty0), L.OP_CODE["add"], 0b01) == 0
    assert L.last_kernel().startswith("mjt_reduce_col_add") or L.last_kernel().endswith("_fold")
    d, keep = desc(outputs=2)
    assert lib.mjt_fused_reduce(ctypes.byref(d), ctypes.byref(ty), L.OP_CODE["add"], 0b10) == -1
    d, keep = desc()
    assert lib.mjt_fused_reduce(ctypes.byref(d), ctypes.byref(ty0), L.OP_CODE["add"], 0b10) == -1    # y has the wrong size
    assert lib.mjt_fused_reduce(ctypes.byref(d), ctypes.byref(ty), L.OP_CODE["subtract"], 0b10) == -1


def test_callers_build_path_graphs():
    """gather / pad / pool / slicing are one reindex (plus a reduce for pool) with the reference's index
    strings (misc.py:1617-1640, nn.py:1679-1700, pool.py:200-208)."""
    import jittor_amd as jt
    from jittor_amd import core
    x = jt.array(np.zeros((2, 3, 8, 8), np.float32))
    g = x.gather(1, jt.array(np.zeros((2, 3, 8, 8), np.int32)))
    assert isinstance(g._op, core.ReindexOp) and g._op.indexes == ["i0", "@e0(i0,i1,i2,i3)", "i2", "i3"]
    p = jt.pad(x, (1, 2), "reflect")
    assert p.shape == [2, 3, 8, 11] and p._op.indexes[3] == "i3<1 ? 1-i3 : i3 > 8 ? 15-i3 : i3-1"
    y = jt.pool(x, 3, "maximum", 1, 2)
    assert isinstance(y._op, core.ReduceOp) and y.shape == [2, 3, 4, 4]
    assert y._history[1][0]._op.indexes == ["i0", "i1", "i2*2-1+i4", "i3*2-1+i5"]
    s = x[1, :, ::2, 3]
    assert s.shape == [3, 4] and s._op.indexes == ["1", "0+i0*(1)", "0+i1*(2)", "3"]
    with pytest.raises(ValueError):
        x.reshape(5, -1)
    with pytest.raises(ValueError):
        jt.pad(x, (1, 2), "mirror")


def test_executor_partitions_a_normalisation_into_three_kernels(monkeypatch):
    """mean, variance (reduce with the subtraction and the square as prologue) and one element-wise kernel:
    `+ eps` and `sqrt` act on the small variance and are evaluated behind their broadcast, and the
    subtraction waits for the division's stage (python/jittor/test/test_new_fused_op.py:24-40 counts the same
    three kernels).  The launches are replaced by recorders: no device is needed."""
    import jittor_amd as jt
    from jittor_amd import executor
    log = []

    def run_group(members, consumers, target_ids, reduce=None, pre=None):
        ids = {m.id for m in members}
        log.append(("group", [getattr(m, "op", m.kind) for m in members], reduce is not None,
                    sorted(getattr(q, "op", q.kind) for m in members for q in (pre or {}).get(m.id, ()))))
        if reduce is not None:
            reduce.out._buf = object()
        for m in members:
            if m.out.id in target_ids or any(c.id not in ids for c in consumers.get(m.out.id, ())):
                m.out._buf = object()
        return True

    def run_single(op):
        log.append(("single", getattr(op, "op", op.kind)))
        op.out._buf = object()

    monkeypatch.setattr(executor, "_run_group", run_group)
    monkeypatch.setattr(executor, "_run_single", run_single)
    v = jt.array(np.zeros((33, 7, 130), np.float32))
    v._buf = object()
    mean = v.mean([2], keepdims=True)
    var = ((v - mean) * (v - mean)).mean([2], keepdims=True)
    y = (v - mean) / (var + 1e-5).sqrt()
    executor._execute(executor._pending_ops([y]), {y.id})
    assert log[0] == ("single", "mean")
    assert log[1][0] == "group" and log[1][2] and log[1][1].count("subtract") == 2 and "multiply" in log[1][1]
    assert log[2][0] == "group" and not log[2][2] and log[2][1][-1] == "divide" and "subtract" in log[2][1]
    assert log[2][3] == ["add", "broadcast", "sqrt"] and len(log) == 3
    # both rules can be switched off
    log.clear()
    monkeypatch.setitem(executor.flags, "enable_broadcast_sink", False)
    v2 = jt.array(np.zeros((4, 6), np.float32))
    v2._buf = object()
    s = v2.sum([1], keepdims=True)
    z = v2 / (s + 1.0)
    executor._execute(executor._pending_ops([z]), {z.id})
    assert [e[0] for e in log] == ["single", "group", "group"]      # sum, s + 1, division


def test_matmul_entry_checks(compile_only):
    """mjt_matmul validates like the reference's relay op (cublas_matmul_op.cc:34-52): 2-d float operands of one
    dtype, matching inner extents, result [n, k]."""
    L = compile_only
    lib = L.load()
    t = lambda dt, shape: L.tensor(0x1000, dt, shape)
    call = lambda a, b, c, ta=0, tb=0: lib.mjt_matmul(ctypes.byref(a), ctypes.byref(b), ctypes.byref(c), ta, tb)
    assert call(t("float32", [4, 8]), t("float32", [8, 5]), t("float32", [4, 5])) == 0
    assert call(t("float32", [8, 4]), t("float32", [8, 5]), t("float32", [4, 5]), 1, 0) == 0
    assert call(t("float32", [4, 8]), t("float32", [5, 8]), t("float32", [4, 5]), 0, 1) == 0
    assert call(t("bfloat16", [4, 8]), t("bfloat16", [8, 5]), t("float32", [4, 5])) == 0
    assert call(t("float32", [4, 8]), t("float32", [7, 5]), t("float32", [4, 5])) == -1
    assert call(t("float32", [4, 8]), t("float32", [8, 5]), t("float32", [5, 4])) == -1
    assert call(t("float32", [4, 8]), t("float16", [8, 5]), t("float32", [4, 5])) == -1
    assert call(t("int32", [4, 8]), t("int32", [8, 5]), t("int32", [4, 5])) == -1
    assert call(t("float32", [4, 8, 1]), t("float32", [8, 5]), t("float32", [4, 5])) == -1
    assert call(t("float32", [3, 4, 8]), t("float32", [3, 8, 5]), t("float32", [3, 4, 5])) == 0       # equal batch extents
    assert call(t("float32", [3, 4, 8]), t("float32", [2, 8, 5]), t("float32", [3, 4, 5])) == -1
    assert lib.mjt_matmul_available() in (0, 1)


def test_shutdown_forgets_kernels_and_rebinding_compiles_again(compile_only, monkeypatch):
    """mjt_shutdown unloads every kernel module; the per-op look-up tables must not keep pointers to them: the same
    calls after binding again have to find (compile or load) their kernels anew."""
    lib = L.load()
    P = 0x100000
    monkeypatch.setenv("MJT_NO_DISK_CACHE", "1")            # count real compilations
    lib.mjt_shutdown()                                       # start from empty tables whatever ran before
    L._device = None
    L.init(-1)

    def calls():
        x, y = L.tensor(P, "float32", (64, 128)), L.tensor(P, "float32", (64,))
        assert lib.mjt_reduce(ctypes.byref(x), ctypes.byref(y), L.OP_CODE["add"], 2) == 0
        xb, w = L.tensor(P, "bfloat16", (2, 64, 16, 16)), L.tensor(P, "bfloat16", (64, 64, 3, 3))
        yb, p = L.tensor(P, "float32", (2, 64, 16, 16)), L.ConvParams(1, 1, 1, 1, 1, 1)
        assert lib.mjt_conv2d_meta(ctypes.byref(xb), ctypes.byref(w), ctypes.byref(yb), ctypes.byref(p)) == 0
        assert L.last_kernel().startswith("mjt_conv_mfma_bf16")
        z = L.tensor(P, "float32", (128, 64))
        assert lib.mjt_reindex(ctypes.byref(x), ctypes.byref(z), 2, L.c_strings(["i1", "i0"]), 0.0, 0, L.c_strings([]), 0, None) == 0
        return L.jit_stats()

    before = L.jit_stats()[0]
    first = calls()[0]
    assert first >= before + 3                               # reduce, convolution (+ its repack), transpose
    assert calls()[0] == first                               # second time: everything from the look-up tables
    lib.mjt_shutdown()
    L._device = None
    L.init(-1)
    assert calls()[0] >= first + 3                           # compiled again, not taken from a stale table


def test_conv_input_gradient_entry_validates_and_picks_its_path(compile_only):
    """mjt_conv2d_meta_dgrad without a device: argument checks, and which of its three forms a geometry takes (one
    convolution per stride phase, transposed flipped weights for stride 1, dy spread out with zeros otherwise)."""
    lib = L.load()
    P = 0x100000

    def call(xs, ws, params, dys=None, dtype="bfloat16"):
        N, C, H, W = xs
        K, _, R, S = ws
        sh, sw, ph, pw, dh, dw = params
        oh, ow = (H + 2 * ph - dh * (R - 1) - 1) // sh + 1, (W + 2 * pw - dw * (S - 1) - 1) // sw + 1
        dy, w = L.tensor(P, dtype, dys or (N, K, oh, ow)), L.tensor(P, dtype, ws)
        dx, p = L.tensor(P, dtype, xs), L.ConvParams(*params)
        return lib.mjt_conv2d_meta_dgrad(ctypes.byref(dy), ctypes.byref(w), ctypes.byref(dx), ctypes.byref(p))

    assert call((2, 64, 28, 28), (64, 64, 3, 3), (2, 2, 1, 1, 1, 1)) == 0
    assert L.last_kernel().startswith("conv_dgrad_phases:mjt_conv_mfma_bf16"), L.last_kernel()
    assert call((2, 64, 28, 28), (64, 64, 3, 3), (1, 1, 1, 1, 1, 1)) == 0
    assert L.last_kernel().startswith("mjt_conv_mfma_bf16"), L.last_kernel()
    assert call((2, 64, 27, 28), (64, 64, 3, 3), (2, 2, 1, 1, 1, 1)) == 0          # 27 rows: no whole phases
    assert not L.last_kernel().startswith("conv_dgrad_phases"), L.last_kernel()
    assert call((2, 64, 28, 28), (64, 64, 3, 3), (2, 2, 1, 1, 1, 1), dys=(2, 64, 15, 14)) == -1
    assert b"dy shape" in lib.mjt_last_error()
    assert call((2, 64, 28, 28), (64, 32, 3, 3), (2, 2, 1, 1, 1, 1)) == -1         # weight channels != dx channels
    assert call((2, 64, 28, 28), (64, 64, 1, 1), (1, 1, 1, 1, 1, 1)) == -1         # padding no tap reaches
    assert b"padding" in lib.mjt_last_error()


def test_conv_builds_that_ran_out_of_registers_are_not_run(compile_only):
    """The MFMA convolution keeps loads under way in registers the compiler does not track, which is sound only while the
    compiler moves no register aside.  The library reads each build's register figures from the code object: a geometry
    whose build stays within a wave's registers runs on the kernel (among them 32 output channels on two waves and 4-column
    maps, whose builds once did not), one whose build needs more takes another route (the weight-gradient kernel on rows of
    104 columns).  That the first group names the MFMA kernel also shows that the figures are found at all: a build whose
    figures are missing is not run either."""
    lib = L.load()
    P = 0x100000

    def call(xs, ws, params=(1, 1, 1, 1, 1, 1)):
        N, C, H, W = xs
        K, _, R, S = ws
        sh, sw, ph, pw, dh, dw = params
        oh, ow = (H + 2 * ph - dh * (R - 1) - 1) // sh + 1, (W + 2 * pw - dw * (S - 1) - 1) // sw + 1
        x, w, y = L.tensor(P, "bfloat16", xs), L.tensor(P, "bfloat16", ws), L.tensor(P, "bfloat16", (N, K, oh, ow))
        p = L.ConvParams(*params)
        assert lib.mjt_conv2d_meta(ctypes.byref(x), ctypes.byref(w), ctypes.byref(y), ctypes.byref(p)) == 0
        return L.last_kernel()

    assert call((2, 64, 16, 16), (32, 64, 3, 3)).startswith("mjt_conv_mfma_bf16")
    assert call((2, 64, 16, 16), (64, 64, 3, 3)).startswith("mjt_conv_mfma_bf16")
    assert call((2, 32, 40, 4), (64, 32, 3, 3)).startswith("mjt_conv_mfma_bf16")
    # the weight gradient kernel likewise: rows of 104 columns need more registers than there are
    x, dy = L.tensor(P, "bfloat16", (4, 64, 10, 104)), L.tensor(P, "bfloat16", (4, 64, 10, 104))
    dw, p = L.tensor(P, "float32", (64, 64, 3, 3)), L.ConvParams(1, 1, 1, 1, 1, 1)
    assert lib.mjt_conv2d_meta_wgrad(ctypes.byref(x), ctypes.byref(dy), ctypes.byref(dw), ctypes.byref(p)) == -2
    assert b"registers" in lib.mjt_last_error()
    x, dy = L.tensor(P, "bfloat16", (4, 64, 16, 16)), L.tensor(P, "bfloat16", (4, 64, 16, 16))
    assert lib.mjt_conv2d_meta_wgrad(ctypes.byref(x), ctypes.byref(dy), ctypes.byref(dw), ctypes.byref(p)) == 0
    assert L.last_kernel().startswith("mjt_conv_wgrad_mfma_bf16")


def test_scatter_and_gather_entries_pick_their_kernels(compile_only, monkeypatch):
    """Without a device: which kernel skeleton a reindex_reduce, a reindex and a fused gather + reduce take.  A scatter
    through a window pattern is a gather over x unless it has overflow conditions, extras or too many candidate windows
    per element; a gather into rows that are no whole vectors keeps 16-byte stores; axis permutations go through tiles."""
    lib = L.load()
    P = 0x100000
    e, noex = L.c_strings([]), (L.Tensor * 1)()

    def scatter(ys, xs, idx, op="add", ofc=(), dtype="float32"):
        ty, tx = L.tensor(P, dtype, ys), L.tensor(P, dtype, xs)
        rc = lib.mjt_reindex_reduce(ctypes.byref(ty), ctypes.byref(tx), L.OP_CODE[op], len(idx), L.c_strings(idx), len(ofc),
                                    L.c_strings(list(ofc)), 0, noex)
        assert rc == 0, lib.mjt_last_error()
        return L.last_kernel()

    pool = ([4, 8, 16, 16, 3, 3], [4, 8, 32, 32], ["i0", "i1", "i2*2+i4-1", "i3*2+i5-1"])
    assert scatter(*pool).startswith("mjt_window_scatter_add_")
    assert scatter(*pool, op="maximum", dtype="bfloat16").startswith("mjt_window_scatter_maximum_")
    assert scatter(*pool, ofc=["i4>1"]).startswith("mjt_reindex_reduce_add_")                      # an overflow condition
    assert scatter(*pool, op="bitwise_or", dtype="int32").startswith("mjt_reindex_reduce_bitwise_or_")
    assert scatter([4, 8, 30, 30, 7, 7], [4, 8, 36, 36], ["i0", "i1", "i2+i4", "i3+i5"]).startswith("mjt_reindex_reduce_add_")   # 49 windows reach an element
    assert scatter([4, 8, 16, 16, 3, 3], [4, 8, 32, 32], ["i0", "i1", "i3*2+i4-1", "i2*2+i5-1"]).startswith("mjt_reindex_reduce_add_")  # rows from the column axis
    monkeypatch.setenv("MJT_NO_WINDOW_SCATTER", "1")
    assert scatter(*pool).startswith("mjt_reindex_reduce_add_")
    monkeypatch.delenv("MJT_NO_WINDOW_SCATTER")

    def gather(xs, ys, idx):
        tx, ty = L.tensor(P, "float32", xs), L.tensor(P, "float32", ys)
        assert lib.mjt_reindex(ctypes.byref(tx), ctypes.byref(ty), len(idx), L.c_strings(idx), 0.0, 0, e, 0, noex) == 0, lib.mjt_last_error()
        return L.last_kernel()

    assert gather([8, 16, 64, 64], [8, 64, 64, 16], ["i0", "i3", "i1", "i2"]).startswith("mjt_permute_b4_")
    flat = gather([8, 16, 64, 64], [8, 16, 66, 66], ["i0", "i1", "i2-1", "i3-1"])
    monkeypatch.setenv("MJT_REINDEX_NO_FLAT", "1")
    rows = gather([8, 16, 64, 64], [8, 16, 66, 66], ["i0", "i1", "i2-1", "i3-1"])
    monkeypatch.delenv("MJT_REINDEX_NO_FLAT")
    assert flat.startswith("mjt_reindex_") and rows.startswith("mjt_reindex_") and flat != rows      # four elements per lane, or two
    # column matrices with the pixels innermost: per image, the whole batch as one group, chunks of images; a stride the
    # pattern does not have (the image index times 3 for chunks of 2) stays on the generic kernel
    taps = ["i4-1+i2", "i5-1+i3"]
    assert gather([8, 16, 28, 28], [8, 16, 3, 3, 28, 28], ["i0", "i1"] + taps).startswith("mjt_im2col_planes_b4_28x28_k3x3")
    assert gather([8, 16, 7, 7], [16, 3, 3, 8, 7, 7], ["i3", "i0", "i4-1+i1", "i5-1+i2"]).endswith("_n8_v4")
    assert gather([8, 16, 29, 29], [4, 16, 3, 3, 2, 14, 14], ["i0*2+i4", "i1", "i5*2-1+i2", "i6*2-1+i3"]).endswith("_n2_v4")
    assert gather([12, 16, 14, 14], [4, 16, 3, 3, 2, 14, 14], ["i0*3+i4", "i1", "i5-1+i2", "i6-1+i3"]).startswith("mjt_reindex_")

    loop, z = L.tensor(0, "float32", [8, 16, 32, 32, 2, 2]), L.tensor(P, "float32", [8, 16, 32, 32])
    tx = L.tensor(P, "float32", [8, 16, 64, 64])
    assert lib.mjt_reindex_then_reduce(ctypes.byref(tx), ctypes.byref(loop), ctypes.byref(z), L.OP_CODE["maximum"], 2, 4,
                                       L.c_strings(["i0", "i1", "i2*2+i4", "i3*2+i5"]), 0.0, 0, e, 0, noex) == 0
    assert L.last_kernel().startswith("mjt_reindex_then_maximum_")


def test_compile_options_follow_the_flag_and_mark_grouped_convolutions():
    """Var.compile_options (var_holder.h:265-273): a dict name -> int, initialised from the flag's value when the var is
    created (var.cc:75); nn.conv2d marks the gathered input of a grouped convolution with {"G": groups} (nn.py:1278),
    and the mark does not stand in the way of the matcher."""
    import jittor_amd.executor as E
    assert jt.zeros([2]).compile_options == {}
    with jt.flag_scope(compile_options={"parallel": 0}):
        v = jt.zeros([2])
    assert v.compile_options == {"parallel": 0} and jt.zeros([2]).compile_options == {}
    v.compile_options = {"G": 4, "C": 8}
    assert v.compile_options == {"G": 4, "C": 8}
    got = v.compile_options
    got["G"] = 5                                       # a copy: the var keeps its own
    assert v.compile_options["G"] == 4
    with pytest.raises(TypeError):
        v.compile_options = {"G": 1.5}
    x, w = jt.zeros([1, 8, 6, 6]), jt.zeros([8, 2, 3, 3])
    y = jt.nn.conv2d(x, w, padding=1, groups=4)
    scatter = y._op
    product = scatter.inputs[0]._op
    assert product.inputs[0].compile_options == {"G": 4}
    unit = E._match_conv_grouped(scatter)
    assert unit is not None and unit.groups == 4


def test_conv_gradient_patterns_match_for_common_losses():
    """The two backward patterns are recognised whatever stands between the convolution and the loss: the loss may
    be the output itself (jt.grad seeds ones, test_conv_tuner.py:105-133), its sum or mean (for 16-bit outputs these
    put float32 casts around dy: the narrowing cast of dy stays, the identity casts are looked through) or a product."""
    from jittor_amd import executor as E
    for dtype in ("float32", "float16", "bfloat16"):
        x, w = jt.zeros([2, 3, 8, 8]).cast(dtype), jt.zeros([4, 3, 3, 3]).cast(dtype)
        y = jt.nn.conv2d(x, w, padding=1)
        r = jt.zeros(y.shape).cast(dtype)
        for loss in (y, y.sum(), y.mean(), (y * r).sum(), (y * y).sum()):
            gx, gw = jt.grad(loss, [x, w])
            ux, uw = E._match_conv_bwd(gx._op), E._match_conv_bwd(gw._op)
            assert isinstance(ux, E.ConvBwdDataUnit) and isinstance(uw, E.ConvBwdWeightUnit), (dtype, loss)
            assert ux.inputs[0].dtype == dtype and list(ux.inputs[0].shape) == [2, 4, 8, 8]
            assert uw.inputs[1].dtype == dtype and gx.dtype == dtype and gw.dtype == dtype


def test_grouped_conv_and_its_gradients_are_matched_by_role():
    """Over the grouped form's 8-d product each of x, w and y has its own index pattern; the scattered-into one names
    the unit.  Forward, input gradient and weight gradient of a grouped and of a depthwise convolution are recognised,
    with the geometry read back from the x pattern."""
    from jittor_amd import executor as E
    for dtype in ("float32", "bfloat16"):
        for groups, cin, cout, kw in ((2, 4, 6, dict(padding=1)), (4, 4, 4, dict(stride=2, padding=1)), (3, 6, 3, dict(padding=2, dilation=2))):
            x, w = jt.zeros([2, cin, 9, 8]).cast(dtype), jt.zeros([cout, cin // groups, 3, 3]).cast(dtype)
            y = jt.nn.conv2d(x, w, groups=groups, **kw)
            r = jt.zeros(y.shape).cast(dtype)
            fwd = E._match_conv_grouped(y._op)
            assert isinstance(fwd, E.ConvUnit) and fwd.groups == groups and fwd.inputs[0] is x and fwd.inputs[1] is w
            gx, gw = jt.grad((y * r).sum(), [x, w])
            ux, uw = E._match_conv_grouped(gx._op), E._match_conv_grouped(gw._op)
            assert isinstance(ux, E.ConvBwdDataUnit) and isinstance(uw, E.ConvBwdWeightUnit), (dtype, groups)
            assert ux.groups == groups and uw.groups == groups and ux.params == fwd.params and uw.params == fwd.params
            assert ux.inputs[1] is w and uw.inputs[0] is x
            assert list(ux.inputs[0].shape) == list(y.shape) and ux.inputs[0] is uw.inputs[1]
            assert gx.dtype == dtype and gw.dtype == dtype
    # an 8-d scatter-add that is none of the three stays what it is
    a = jt.zeros([2, 2, 3, 2, 4, 4, 3, 3])
    z = (a * a).reindex_reduce("add", [2, 6, 4, 4], ["i0", "i1*3+i2", "i5", "i4"])
    assert E._match_conv_grouped(z._op) is None


def test_executor_replays_a_graph_it_has_seen(compile_only, monkeypatch):
    """The second execution of a graph with the same signature re-issues the recorded library calls: same number of calls
    and the same counters, every pointer inside the recorded descriptors is the new graph's (input, result or a buffer
    made on the way), a by-value scalar is the new graph's value, computed vars become leaves; another shape, another
    wiring or a switched flag is another signature.  Compile-only mode with addresses handed out by a counter: no device."""
    from jittor_amd import core, executor
    nxt = [0x10000000]

    def fake_alloc(nbytes):
        size = core._Pool._round(nbytes)
        nxt[0] += size
        return nxt[0] - size, size

    monkeypatch.setattr(core.pool, "alloc", fake_alloc)
    monkeypatch.setattr(core.pool, "free", lambda ptr, size: None)
    monkeypatch.setattr(L, "h2d", lambda ptr, arr: None)
    monkeypatch.setitem(executor.flags, "enable_replay", True)
    executor._plans.clear()

    def step(lr, shape=(3, 6, 10, 10), twice=False):
        x = jt.array(np.ones(shape, np.float32))
        w = jt.array(np.ones((8, shape[1], 3, 3), np.float32))
        y = jt.nn.conv2d(x, w, padding=1)
        gw, = jt.grad((y * y).sum(), [w])                    # float32 weight gradient: column matrices and partial sums on the way
        new_w = w - gw * jt.array(np.float32(lr))            # a by-value scalar
        flat = jt.reshape(y, [shape[0], -1])                 # shares y's buffer
        out = (flat + flat) if twice else (flat + 1.0)
        before = dict(executor.stats)
        jt.sync([new_w, out, y])
        return {k: executor.stats[k] - before[k] for k in before}, (x, w, y, new_w, out, flat)

    d1, keep1 = step(0.5)
    assert d1["plans"] == 1 and d1["replays"] == 0
    plan = next(iter(executor._plans.values()))
    ncalls = len(plan.calls)
    d2, keep2 = step(0.25)
    assert d2["replays"] == 1 and d2["plans"] == 0
    for k in d1:
        if k not in ("plans", "replays"):
            assert d1[k] == d2[k], k
    assert len(plan.calls) == ncalls and ncalls == d1["launches"]
    # every recorded pointer now points into a buffer of the second graph (or one made during the replay), none into the first's
    x1, w1, y1, nw1, out1, flat1 = keep1
    x2, w2, y2, nw2, out2, flat2 = keep2
    first = {v._buf.ptr for v in keep1}
    second = {v._buf.ptr for v in keep2}
    assert not first & second and flat2._buf is y2._buf and flat1._buf is y1._buf
    seen = set()
    for obj, idx, slot, off in plan.ptrs:
        ptr = (obj if idx is None else obj[idx]).ptr
        assert ptr - off not in first
        seen.add(ptr - off)
    assert second - {flat2._buf.ptr} <= seen | {y2._buf.ptr}
    assert all(v._op is None for v in (y2, nw2, out2))
    vals = [arr[i].fvalue for arr, i, _ in plan.scalars]
    assert 0.25 in vals and 0.5 not in vals
    # other signatures: a shape, the wiring of a leaf, a flag
    assert step(0.5, shape=(3, 6, 12, 10))[0]["plans"] == 1
    assert step(0.5, twice=True)[0]["plans"] == 1
    monkeypatch.setitem(executor.flags, "enable_reduce_fusion", False)
    assert step(0.5)[0]["plans"] == 1
    monkeypatch.setitem(executor.flags, "enable_replay", False)
    d = step(0.5)[0]
    assert d["plans"] == 0 and d["replays"] == 0
