"""mjt_matmul on the library's own kernels (kernels/gemm_mfma.h, kernels/gemm_plain.h), called through the C-ABI.
What the reference relays to a library GEMM is by definition broadcast * broadcast -> sum
(python/jittor/src/opt/tuner/matmul_tuner.cc:16-104), so the oracle is that meta-op expression for small
operands and the float64 matrix product of the same (rounded) operands beyond; every element is held to
1e-4 * sum_k |a_ik * b_kj| (float32 accumulation in another order), plus one rounding of a 16-bit result."""
import ctypes

import numpy as np
import pytest

from jittor_amd import _lib as L
from jittor_amd.dtypes import f32_to_bf16_bits
from oracle import oracle as O

pytestmark = pytest.mark.gpu


def _to_dev(arr):
    p = L.alloc(max(arr.nbytes, 256))
    L.h2d(p, arr)
    return p


def _operand(rng, shape, dt):
    """(what goes to the device, its exact float64 value)"""
    v = rng.standard_normal(shape).astype(np.float32)
    if dt == "bfloat16":
        bits = f32_to_bf16_bits(v)
        return bits, (bits.astype(np.uint32) << 16).view(np.float32).astype(np.float64)
    if dt == "float16":
        h = v.astype(np.float16)
        return h, h.astype(np.float64)
    if dt == "float64":
        d = v.astype(np.float64) + 1e-9 * rng.standard_normal(shape)
        return d, d
    return v, v.astype(np.float64)


def _from_dev(ptr, shape, dt):
    if dt == "bfloat16":
        return (L.d2h(ptr, shape, np.uint16).astype(np.uint32) << 16).view(np.float32).astype(np.float64)
    return L.d2h(ptr, shape, {"float16": np.float16, "float32": np.float32, "float64": np.float64}[dt]).astype(np.float64)


def _run(lib, dt, odt, M, K, N, ta, tb, batch=(), seed=0):
    rng = np.random.default_rng(seed)
    ash, bsh = tuple(batch) + ((K, M) if ta else (M, K)), tuple(batch) + ((N, K) if tb else (K, N))
    a_dev, a64 = _operand(rng, ash, dt)
    b_dev, b64 = _operand(rng, bsh, dt)
    pa, pb = _to_dev(a_dev), _to_dev(b_dev)
    csh = tuple(batch) + (M, N)
    pc = L.alloc(max(int(np.prod(csh)) * 8, 256))
    try:
        ta_, tb_, tc_ = L.tensor(pa, dt, ash), L.tensor(pb, dt, bsh), L.tensor(pc, odt, csh)
        L.check(lib.mjt_matmul(ctypes.byref(ta_), ctypes.byref(tb_), ctypes.byref(tc_), ta, tb))
        kern = L.last_kernel()
        got = _from_dev(pc, csh, odt)
    finally:
        for p in (pa, pb, pc):
            L.free(p)
    A = np.swapaxes(a64, -1, -2) if ta else a64
    B = np.swapaxes(b64, -1, -2) if tb else b64
    want = A @ B
    bound = 1e-4 * (np.abs(A) @ np.abs(B))
    if odt == "bfloat16":
        bound = bound + np.abs(want) * 2.0 ** -7
    elif odt == "float16":
        bound = bound + np.abs(want) * 2.0 ** -10
    elif dt == "float64":
        bound = 1e-12 * (np.abs(A) @ np.abs(B))
    bad = np.abs(got - want) > bound
    assert not bad.any(), (kern, dt, odt, M, K, N, ta, tb, int(bad.sum()), float(np.abs(got - want).max()))
    return kern


SHAPES = [(256, 256, 256), (304, 200, 136), (64, 64, 64), (1000, 72, 520), (40, 24, 48), (520, 264, 328), (8, 520, 8)]


@pytest.mark.parametrize("dt", ["bfloat16", "float16", "float32"])
@pytest.mark.parametrize("ta,tb", [(0, 0), (0, 1), (1, 0), (1, 1)])
def test_gemm_mfma_layouts_and_edges(gpu, dt, ta, tb):
    """Row lengths that are multiples of 16 bytes take the MFMA kernel: all four layouts, tiles that hang over
    every edge, a k that ends inside a stage and inside a 16-byte chunk."""
    lib = L.load()
    for i, (M, K, N) in enumerate(SHAPES):
        kern = _run(lib, dt, dt, M, K, N, ta, tb, seed=i)
        assert kern.startswith("mjt_gemm_mfma_"), kern
    if dt != "float32":                                   # the float32 sum of 16-bit operands, before it is narrowed
        assert _run(lib, dt, "float32", 304, 200, 136, ta, tb).startswith("mjt_gemm_mfma_")


@pytest.mark.parametrize("tile", ["256", "128"])
@pytest.mark.parametrize("dt", ["bfloat16", "float16"])
@pytest.mark.parametrize("ta,tb", [(0, 1), (0, 0), (1, 0), (1, 1)])
def test_gemm_direct_copy_kernel(gpu, dt, ta, tb, tile, monkeypatch):
    """16-bit operands with K a multiple of 64 have a kernel of their own (operands go from memory to LDS without
    passing through registers; an operand whose memory has m or n innermost is read from LDS with transposing
    reads) once there are enough 256 x 256 tiles (two stage buffers) or 128 x 128 tiles (a ring of four); here it is
    asked for by name and tile so that small shapes reach it too: all four layouts, tiles that hang over both edges, fewer
    stages than buffers (K = 64, 128, 192), many stages, a float32 result, a batch."""
    lib = L.load()
    monkeypatch.setenv("MJT_GEMM_DMA", tile)
    for i, (M, K, N) in enumerate([(256, 64, 256), (512, 256, 256), (304, 128, 136), (1000, 192, 520), (8, 512, 8), (520, 2048, 264)]):
        kern = _run(lib, dt, dt, M, K, N, ta, tb, seed=20 + i)
        assert kern.endswith("%sx%s_%s%s_direct" % (tile, tile, "nt"[ta], "nt"[tb])), kern
    assert _run(lib, dt, "float32", 304, 128, 520, ta, tb, seed=30).endswith("_direct")
    assert _run(lib, dt, dt, 264, 64, 248, ta, tb, seed=31, batch=(3,)).endswith("_direct")
    # K = 96 is no multiple of 64: the general kernel
    assert not _run(lib, dt, dt, 256, 96, 256, ta, tb, seed=32).endswith("_direct")


@pytest.mark.parametrize("tile", ["256", "128"])
def test_gemm_direct_copy_kernel_random_shapes(gpu, tile, monkeypatch):
    """Seeded sweep over shapes, layouts, result types and batches for the direct-copy kernel: M and N anywhere
    between 1 and 700 (tiles cut on every side, operands whose last rows or columns end at the tensor's end),
    K a multiple of 64 up to 1024."""
    lib = L.load()
    monkeypatch.setenv("MJT_GEMM_DMA", tile)
    rng = np.random.default_rng(2024)
    for i in range(24):
        M, N = int(rng.integers(1, 88)) * 8, int(rng.integers(1, 88)) * 8       # rows of 16-byte multiples in every layout
        K = 64 * int(rng.integers(1, 17))
        ta, tb = int(rng.integers(0, 2)), int(rng.integers(0, 2))
        dt = ("bfloat16", "float16")[i % 2]
        odt = (dt, "float32")[int(rng.integers(0, 2))]
        batch = () if i % 3 else (int(rng.integers(2, 4)),)
        kern = _run(lib, dt, odt, M, K, N, ta, tb, seed=100 + i, batch=batch)
        assert kern.endswith("_direct"), (kern, M, K, N, ta, tb)


def test_gemm_k_tail_inside_a_chunk(gpu):
    """k-innermost operands whose K is no multiple of the chunk: the row length (leading dimension) is what has to
    be aligned, and a product's operands are dense, so this route is only reachable with a K that is aligned;
    K = 72 ends inside a 64-wide stage for 16-bit operands, K = 36 inside one for float32."""
    lib = L.load()
    assert _run(lib, "bfloat16", "bfloat16", 128, 72, 128, 0, 1).startswith("mjt_gemm_mfma_")
    assert _run(lib, "float32", "float32", 128, 36, 128, 0, 1).startswith("mjt_gemm_mfma_")
    assert _run(lib, "float16", "float32", 96, 8, 64, 0, 1).startswith("mjt_gemm_mfma_")


@pytest.mark.parametrize("ta,tb", [(0, 0), (0, 1), (1, 0), (1, 1)])
def test_gemm_single_stage_uses_one_staging_buffer(gpu, ta, tb, monkeypatch):
    """A sum that fits one stage of the k loop (64 elements of 16 bits, 32 of float32) runs on a variant of the kernel
    with one staging buffer; one element more and it is the two-buffer kernel again.  Tiles over every edge, a batch."""
    lib = L.load()
    for dt, K in (("bfloat16", 64), ("float16", 40), ("float32", 32), ("float32", 8)):
        assert _run(lib, dt, dt, 304, K, 264, ta, tb, seed=K).endswith("_k1")
        assert _run(lib, dt, "float32", 72, K, 520, ta, tb, seed=K + 1, batch=(3,)).endswith("_k1")
    assert not _run(lib, "bfloat16", "bfloat16", 304, 72, 264, ta, tb, seed=3).endswith("_k1")
    assert not _run(lib, "float32", "float32", 304, 36, 264, ta, tb, seed=4).endswith("_k1")
    monkeypatch.setenv("MJT_GEMM_TWO_BUFFERS", "1")
    assert not _run(lib, "bfloat16", "bfloat16", 304, 64, 264, ta, tb, seed=64).endswith("_k1")


@pytest.mark.parametrize("dt", ["bfloat16", "float32", "float64"])
def test_gemm_plain_unaligned_and_float64(gpu, dt):
    lib = L.load()
    for ta, tb in ((0, 0), (0, 1), (1, 0), (1, 1)):
        kern = _run(lib, dt, dt, 70, 129, 45, ta, tb)
        assert kern.startswith("mjt_gemm_plain_"), kern
    assert _run(lib, dt, dt, 1, 1, 1, 0, 0).startswith("mjt_gemm_plain_")
    assert _run(lib, dt, dt, 130, 3, 67, 0, 1).startswith("mjt_gemm_plain_")


def test_gemm_batched(gpu):
    lib = L.load()
    assert _run(lib, "bfloat16", "bfloat16", 136, 64, 200, 0, 0, batch=(3, 2)).startswith("mjt_gemm_mfma_")
    assert _run(lib, "float32", "float32", 100, 36, 52, 1, 0, batch=(5,)).startswith("mjt_gemm_mfma_")
    assert _run(lib, "float32", "float32", 33, 17, 9, 0, 0, batch=(4,)).startswith("mjt_gemm_plain_")


def test_gemm_is_the_meta_op_expression(gpu):
    """The product equals the expression the reference's tuner matches: broadcast(a,[n,m,k]) * broadcast(b,[n,m,k])
    summed over m, evaluated by the oracle's meta-ops in float32 (python/jittor/nn.py:118-158)."""
    lib = L.load()
    rng = np.random.default_rng(3)
    a = rng.standard_normal((24, 40)).astype(np.float32)
    b = rng.standard_normal((40, 16)).astype(np.float32)
    prod = O.binary(O.broadcast_to(a, [24, 40, 16], [2]), O.broadcast_to(b, [24, 40, 16], [0]), "multiply")
    want = O.reduce(prod, "add", 1)
    pa, pb, pc = _to_dev(a), _to_dev(b), L.alloc(24 * 16 * 4)
    try:
        ta_, tb_, tc_ = L.tensor(pa, "float32", a.shape), L.tensor(pb, "float32", b.shape), L.tensor(pc, "float32", (24, 16))
        L.check(lib.mjt_matmul(ctypes.byref(ta_), ctypes.byref(tb_), ctypes.byref(tc_), 0, 0))
        got = L.d2h(pc, (24, 16), np.float32)
    finally:
        for p in (pa, pb, pc):
            L.free(p)
    assert np.allclose(got, want, rtol=1e-5, atol=1e-5 * np.abs(want).max())


def test_gemm_2048_runs_on_128_tiles_of_the_direct_copy_kernel(gpu):
    """2048^3 has 64 tiles of 256 x 256 for 256 compute units: the direct-copy kernel takes it on 128 x 128 tiles (a ring
    of four stages), in every layout; 1536^3 (144 such tiles) too; the whole result against float64."""
    lib = L.load()
    for ta, tb in ((0, 1), (0, 0), (1, 0), (1, 1)):
        kern = _run(lib, "bfloat16", "bfloat16", 2048, 2048, 2048, ta, tb, seed=40 + 2 * ta + tb)
        assert kern.endswith("128x128_%s%s_direct" % ("nt"[ta], "nt"[tb])), kern
    assert _run(lib, "float16", "float32", 1536, 1536, 1536, 0, 1, seed=44).endswith("128x128_nt_direct")


def test_gemm_more_128_tiles_than_compute_units_run_two_workgroups_per_unit(gpu):
    """With more 128 x 128 tiles than compute units (and too few 256 x 256 ones, or a sum too short for those) the
    direct-copy kernel runs on two stage buffers, two workgroups per compute unit: every layout, one to five stages of
    the sum, tiles hanging over both edges, a batch; the whole result against float64."""
    lib = L.load()
    for i, (ta, tb) in enumerate(((0, 1), (0, 0), (1, 0), (1, 1))):
        kern = _run(lib, "bfloat16", "bfloat16", 2176, 128, 2120, ta, tb, seed=50 + i)
        assert kern.endswith("128x128_%s%s_direct2" % ("nt"[ta], "nt"[tb])), kern
    assert _run(lib, "float16", "float16", 2304, 320, 2200, 0, 1, seed=54).endswith("128x128_nt_direct2")
    assert _run(lib, "bfloat16", "float32", 2304, 64, 2304, 1, 0, seed=55).endswith("128x128_tn_direct2")
    assert _run(lib, "bfloat16", "bfloat16", 640, 192, 904, 0, 0, seed=56, batch=(9,)).endswith("128x128_nn_direct2")


def test_gemm_full_size_4096_bf16_properties(gpu):
    """4096^3 in bfloat16 (the shape the throughput figure is quoted on): rows of the result against float64 on a
    sample, and linearity in b, which holds exactly for power-of-two factors."""
    lib = L.load()
    n = 4096
    rng = np.random.default_rng(9)
    a_bits = f32_to_bf16_bits(rng.standard_normal((n, n)).astype(np.float32))
    b_bits = f32_to_bf16_bits(rng.standard_normal((n, n)).astype(np.float32))
    pa, pb, pc = _to_dev(a_bits), _to_dev(b_bits), L.alloc(n * n * 4)
    try:
        ta_, tb_, tc_ = L.tensor(pa, "bfloat16", (n, n)), L.tensor(pb, "bfloat16", (n, n)), L.tensor(pc, "float32", (n, n))
        for trans_b in (1, 0):
            L.check(lib.mjt_matmul(ctypes.byref(ta_), ctypes.byref(tb_), ctypes.byref(tc_), 0, trans_b))
            assert L.last_kernel().startswith("mjt_gemm_mfma_bfloat16_float32_256x256"), L.last_kernel()
            got = L.d2h(pc, (n, n), np.float32)
            A = (a_bits.astype(np.uint32) << 16).view(np.float32).astype(np.float64)
            B = (b_bits.astype(np.uint32) << 16).view(np.float32).astype(np.float64)
            Bm = B.T if trans_b else B
            for r in (0, 1, 255, 256, 2049, 4095):
                want = A[r] @ Bm
                bound = 1e-4 * (np.abs(A[r]) @ np.abs(Bm))
                assert (np.abs(got[r] - want) <= bound).all(), (trans_b, r)
        L.h2d(pb, (b_bits.astype(np.uint32) + (2 << 7)).astype(np.uint16))     # exponent + 2: b * 4, exactly
        L.check(lib.mjt_matmul(ctypes.byref(ta_), ctypes.byref(tb_), ctypes.byref(tc_), 0, 0))
        assert np.array_equal(L.d2h(pc, (n, n), np.float32), got * 4)
    finally:
        for p in (pa, pb, pc):
            L.free(p)
