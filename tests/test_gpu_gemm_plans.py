"""Products that the planner launches in parts (a block of whole rounds plus strips), with the tiles of the last round
cut into pieces along k, or with k cut over several workgroups per large tile: against float64 products in full,
bit-exact on integer-valued operands, with accumulation, and through the fused Linear entry points (bias, ReLU and gate
must land on the right strip or tile)."""
from __future__ import annotations

import numpy as np
import pytest

from conftest import run_op
from zigrad_amd.device import F32

pytestmark = pytest.mark.gpu
TOL = 1e-5


def _matmul(hip, A, B, C0, m, n, k, ta, tb, alpha, beta):
    a, b, c = hip.from_numpy(A), hip.from_numpy(B), hip.from_numpy(C0)
    hip.dispatch("matmul", A=a, B=b, C=c, m=m, n=n, k=k, trans_a=ta, trans_b=tb, lda=A.shape[1], ldb=B.shape[1], ldc=n,
                 alpha=alpha, beta=beta)
    out = hip.to_numpy(c).reshape(m, n)
    for x in (a, b, c):
        hip.mem_free(x)
    return out


# tail in pieces: (3072, 3072, 3072): 128 x 128 tiles, 4 pieces of 48 k-tiles; (1536, 1536, 1234): 64 x 64 tiles, a k that ends inside a
# k-tile, so the last piece is short and masked; (2560, 3328, 1024): 8 pieces of 8 k-tiles, the shortest range allowed
@pytest.mark.parametrize("shape,kind", [((4100, 4100, 1030), "parts"), ((3600, 2308, 1541), "parts"),
                                        ((3072, 3072, 3072), "tail_in_pieces"), ((1536, 1536, 1234), "tail_in_pieces"),
                                        ((2560, 3328, 1024), "tail_in_pieces"),
                                        # tiles that end inside C (the edge kernels), and a C that takes scalar stores
                                        ((1498, 1530, 1000), "tail_in_pieces"), ((1498, 1531, 1003), "tail_in_pieces")])
@pytest.mark.parametrize("ta,tb", [(False, False), (False, True), (True, False), (True, True)])
def test_products_launched_in_parts_or_with_the_tail_in_pieces_match_float64(hip, shape, kind, ta, tb):
    m, n, k = shape
    assert hip.gemm_plan(m, n, k)["kind"] == kind, hip.gemm_plan(m, n, k)
    r = np.random.default_rng(m + 3 * n + 7 * k + 2 * ta + tb)
    A = r.standard_normal((k, m) if ta else (m, k), dtype=np.float32)
    B = r.standard_normal((n, k) if tb else (k, n), dtype=np.float32)
    C0 = r.standard_normal((m, n), dtype=np.float32)
    opA = (A.T if ta else A).astype(np.float64)
    opB = (B.T if tb else B).astype(np.float64)
    prod = opA @ opB
    got = _matmul(hip, A, B, np.full((m, n), np.nan, np.float32), m, n, k, ta, tb, 1.0, 0.0)
    assert np.linalg.norm(got - prod) <= TOL * np.linalg.norm(prod)
    # every strip separately: an error confined to a few rows or columns must not hide in the whole-matrix norm
    # (the tiles cut into pieces are the last of the walk over C: its bottom rows)
    for sl in (np.s_[-4:, :], np.s_[:, -4:], np.s_[: m // 2, n // 2:], np.s_[m // 2:, : n // 2], np.s_[-256:, -128:],
               np.s_[-64:, :64]):
        assert np.linalg.norm(got[sl] - prod[sl]) <= TOL * np.linalg.norm(prod[sl])
    got = _matmul(hip, A, B, C0, m, n, k, ta, tb, 0.5, 2.0)
    want = 0.5 * prod + 2.0 * C0
    assert np.linalg.norm(got - want) <= TOL * np.linalg.norm(want)


def test_parts_and_split_products_are_exact_on_small_integers(hip):
    for (m, n, k) in ((3072, 3072, 3072), (4100, 4100, 1030), (1536, 1536, 1536)):
        r = np.random.default_rng(m)
        A = r.integers(-3, 4, (m, k)).astype(np.float32)
        B = r.integers(-3, 4, (n, k)).astype(np.float32)  # stored [n, k]: the forward layout of a Linear layer
        got = _matmul(hip, A, B, np.zeros((m, n), np.float32), m, n, k, False, True, 1.0, 0.0)
        want = (A.astype(np.int64) @ B.astype(np.int64).T).astype(np.float32)  # |entries| < 2^24: exact in fp32
        assert np.array_equal(got, want)


@pytest.mark.parametrize("Bt,I,wide,kind", [(2560, 1024, 3332, "parts"), (2560, 1024, 3328, "tail_in_pieces"),
                                            (1498, 1000, 1530, "tail_in_pieces"), (1498, 1003, 1531, "tail_in_pieces")])
def test_fused_linear_entry_points_on_a_product_launched_in_parts_or_with_the_tail_in_pieces(hip, Bt, I, wide, kind):
    O = wide  # batch Bt, fan_in I, fan_out O
    assert hip.gemm_plan(Bt, O, I)["kind"] == kind, hip.gemm_plan(Bt, O, I)
    r = np.random.default_rng(77)
    x = r.standard_normal((Bt, I)).astype(np.float32)
    w = (r.standard_normal((O, I)) / np.sqrt(I)).astype(np.float32)
    b = r.standard_normal(O).astype(np.float32)
    got = run_op(hip, "linear_fwd", {"x": x, "w": w, "bias": b, "y": np.full((Bt, O), np.nan, np.float32), "batch": Bt,
                                     "fan_in": I, "fan_out": O, "relu": True}, ["y"])["y"].reshape(Bt, O)
    y = run_op(hip, "matmul", {"A": x, "B": w, "C": np.zeros((Bt, O), np.float32), "m": Bt, "n": O, "k": I,
                               "trans_a": False, "trans_b": True, "lda": I, "ldb": I, "ldc": O, "alpha": 1.0, "beta": 0.0},
               ["C"])["C"]
    y = run_op(hip, "add", {"x": b, "y": y, "z": np.zeros_like(y)}, ["z"])["z"]
    y = run_op(hip, "relu_fwd", {"x": y, "y": np.zeros_like(y)}, ["y"])["y"].reshape(Bt, O)
    assert np.array_equal(got, y)
    want = np.maximum(x.astype(np.float64) @ w.astype(np.float64).T + b, 0.0)
    assert np.linalg.norm(got - want) <= TOL * np.linalg.norm(want)
    # input gradient with the ReLU gate of the layer below: gx = (gy W) where act > 0
    I2, O2 = wide, I
    assert hip.gemm_plan(Bt, I2, O2)["kind"] == kind
    gy = r.standard_normal((Bt, O2)).astype(np.float32)
    w2 = (r.standard_normal((O2, I2)) / np.sqrt(O2)).astype(np.float32)
    act = np.maximum(r.standard_normal((Bt, I2)), 0.0).astype(np.float32)
    got = run_op(hip, "linear_bwd_input", {"gy": gy, "w": w2, "act_in": act, "gx": np.full((Bt, I2), np.nan, np.float32),
                                            "batch": Bt, "fan_in": I2, "fan_out": O2, "accumulate": False}, ["gx"])["gx"]
    want = np.where(act > 0, gy.astype(np.float64) @ w2.astype(np.float64), 0.0)
    assert np.linalg.norm(got.reshape(Bt, I2) - want) <= TOL * np.linalg.norm(want)
    assert np.all(got.reshape(Bt, I2)[act <= 0] == 0.0)


@pytest.mark.parametrize("shape", [(2708, 16, 1433), (2708, 7, 1433), (1000, 1, 300), (513, 32, 257), (4096, 17, 1024),
                                   (600, 8, 2050), (515, 9, 4099), (2048, 24, 256)])
def test_tall_narrow_products_of_k_contiguous_operands(hip, shape):
    """[m, k] x [n, k]^T with n <= 32 (the graph convolution's first layer; k is cut over several workgroups per tile):
    against float64, with accumulation, with padded leading dimensions, and through linear_fwd (bias and ReLU in the
    same launch) against the three separate ops."""
    m, n, k = shape
    r = np.random.default_rng(m + n + k)
    A = r.standard_normal((m, k), dtype=np.float32)
    B = r.standard_normal((n, k), dtype=np.float32)
    C0 = r.standard_normal((m, n), dtype=np.float32)
    prod = A.astype(np.float64) @ B.astype(np.float64).T
    got = _matmul(hip, A, B, np.full((m, n), np.nan, np.float32), m, n, k, False, True, 1.0, 0.0)
    assert np.linalg.norm(got - prod) <= TOL * np.linalg.norm(prod)
    assert np.abs(got - prod).max() <= 8 * TOL * np.sqrt(k)
    got = _matmul(hip, A, B, C0, m, n, k, False, True, -0.5, 1.0)
    want = -0.5 * prod + C0
    assert np.linalg.norm(got - want) <= TOL * np.linalg.norm(want)
    # a row stride larger than k (a view into a wider matrix) and an output wider than n
    Aw = r.standard_normal((m, k + 3), dtype=np.float32)
    a, b, c = hip.from_numpy(Aw), hip.from_numpy(B), hip.from_numpy(np.full((m, n + 5), 7.0, np.float32))
    hip.dispatch("matmul", A=a, B=b, C=c, m=m, n=n, k=k, trans_a=False, trans_b=True, lda=k + 3, ldb=k, ldc=n + 5,
                 alpha=1.0, beta=0.0)
    out = hip.to_numpy(c).reshape(m, n + 5)
    want = Aw[:, :k].astype(np.float64) @ B.astype(np.float64).T
    assert np.linalg.norm(out[:, :n] - want) <= TOL * np.linalg.norm(want)
    assert np.all(out[:, n:] == 7.0)
    for x in (a, b, c):
        hip.mem_free(x)
    bias = r.standard_normal(n).astype(np.float32)
    fused = run_op(hip, "linear_fwd", {"x": A, "w": B, "bias": bias, "y": np.full((m, n), np.nan, np.float32), "batch": m,
                                       "fan_in": k, "fan_out": n, "relu": True}, ["y"])["y"].reshape(m, n)
    y = _matmul(hip, A, B, np.zeros((m, n), np.float32), m, n, k, False, True, 1.0, 0.0)
    y = run_op(hip, "add", {"x": bias, "y": y, "z": np.zeros_like(y)}, ["z"])["z"]
    y = run_op(hip, "relu_fwd", {"x": y, "y": np.zeros_like(y)}, ["y"])["y"].reshape(m, n)
    assert np.array_equal(fused, y)


@pytest.mark.parametrize("shape", [(64, 128, 784), (100, 30, 384), (100, 30, 383), (256, 256, 2048), (256, 256, 2049),
                                   (250, 251, 1000), (257, 256, 600), (17, 33, 2047), (16, 16, 400), (64, 128, 1433),
                                   # k of 384 to 512 on up to 16 blocks of 32 x 32, which the unstaged kernel would take too
                                   (64, 64, 512), (128, 128, 512), (100, 30, 385), (96, 96, 513), (16, 16, 512)])
def test_deep_products_of_k_contiguous_operands_either_side_of_the_one_launch_kernels_limits(hip, shape):
    """[m, k] x [n, k]^T with 384 <= k <= 2048 on at most 256 blocks of 16 x 16 takes one launch of a kernel of its own
    (a Linear layer's forward at a small batch); the shapes here sit on both sides of each limit, with edges inside a
    block, a k that ends inside a chunk of 16 and inside a 16-byte piece: against float64, accumulating, with padded
    leading dimensions, exact on small integers, and with bias and ReLU against the three separate ops."""
    m, n, k = shape
    r = np.random.default_rng(m * 7 + n * 3 + k)
    A = r.standard_normal((m, k), dtype=np.float32)
    B = r.standard_normal((n, k), dtype=np.float32)
    C0 = r.standard_normal((m, n), dtype=np.float32)
    prod = A.astype(np.float64) @ B.astype(np.float64).T
    got = _matmul(hip, A, B, np.full((m, n), np.nan, np.float32), m, n, k, False, True, 1.0, 0.0)
    assert np.linalg.norm(got - prod) <= TOL * np.linalg.norm(prod)
    assert np.abs(got - prod).max() <= 8 * TOL * np.sqrt(k)
    got = _matmul(hip, A, B, C0, m, n, k, False, True, 0.25, -2.0)
    want = 0.25 * prod - 2.0 * C0
    assert np.linalg.norm(got - want) <= TOL * np.linalg.norm(want)
    Ai = r.integers(-3, 4, (m, k)).astype(np.float32)
    Bi = r.integers(-3, 4, (n, k)).astype(np.float32)
    got = _matmul(hip, Ai, Bi, np.zeros((m, n), np.float32), m, n, k, False, True, 1.0, 0.0)
    assert np.array_equal(got, (Ai.astype(np.int64) @ Bi.astype(np.int64).T).astype(np.float32))
    # views into wider matrices: row strides k + 3 and k + 1 (rows that start at any 4-byte alignment), an output wider than n
    Aw, Bw = r.standard_normal((m, k + 3), dtype=np.float32), r.standard_normal((n, k + 1), dtype=np.float32)
    a, b, c = hip.from_numpy(Aw), hip.from_numpy(Bw), hip.from_numpy(np.full((m, n + 5), 7.0, np.float32))
    hip.dispatch("matmul", A=a, B=b, C=c, m=m, n=n, k=k, trans_a=False, trans_b=True, lda=k + 3, ldb=k + 1, ldc=n + 5,
                 alpha=1.0, beta=0.0)
    out = hip.to_numpy(c).reshape(m, n + 5)
    want = Aw[:, :k].astype(np.float64) @ Bw[:, :k].astype(np.float64).T
    assert np.linalg.norm(out[:, :n] - want) <= TOL * np.linalg.norm(want)
    assert np.all(out[:, n:] == 7.0)
    for x in (a, b, c):
        hip.mem_free(x)
    bias = r.standard_normal(n).astype(np.float32)
    fused = run_op(hip, "linear_fwd", {"x": A, "w": B, "bias": bias, "y": np.full((m, n), np.nan, np.float32), "batch": m,
                                       "fan_in": k, "fan_out": n, "relu": True}, ["y"])["y"].reshape(m, n)
    y = _matmul(hip, A, B, np.zeros((m, n), np.float32), m, n, k, False, True, 1.0, 0.0)
    y = run_op(hip, "add", {"x": bias, "y": y, "z": np.zeros_like(y)}, ["z"])["z"]
    y = run_op(hip, "relu_fwd", {"x": y, "y": np.zeros_like(y)}, ["y"])["y"].reshape(m, n)
    assert np.array_equal(fused, y)


def test_tall_narrow_product_is_exact_on_small_integers(hip):
    m, n, k = 2708, 16, 1433
    r = np.random.default_rng(4)
    A = r.integers(0, 2, (m, k)).astype(np.float32)       # binary features, as in the benchmark's graph
    B = r.integers(-4, 5, (n, k)).astype(np.float32)
    got = _matmul(hip, A, B, np.zeros((m, n), np.float32), m, n, k, False, True, 1.0, 0.0)
    assert np.array_equal(got, (A.astype(np.int64) @ B.astype(np.int64).T).astype(np.float32))


@pytest.mark.parametrize("shape", [(500, 64, 385), (256, 256, 4096), (100, 100, 4099), (500, 256, 2048), (64, 64, 4096),
                                   (1024, 64, 2050), (130, 70, 1000), (16, 16, 4096)])
@pytest.mark.parametrize("ta,tb", [(False, False), (True, False), (True, True)])
def test_products_on_few_tiles_cut_into_ranges_of_k(hip, shape, ta, tb):
    """Few 64 x 64 tiles over a long k (in the layouts the one-launch kernels do not take): ranges of k on separate
    workgroups and a reduction, the last range shorter than the others, against float64 and accumulating."""
    m, n, k = shape
    r = np.random.default_rng(m + 3 * n + 7 * k)
    A = r.standard_normal((k, m) if ta else (m, k), dtype=np.float32)
    B = r.standard_normal((n, k) if tb else (k, n), dtype=np.float32)
    C0 = r.standard_normal((m, n), dtype=np.float32)
    a64 = (A.T if ta else A).astype(np.float64)
    b64 = (B.T if tb else B).astype(np.float64)
    prod = a64 @ b64
    got = _matmul(hip, A, B, np.full((m, n), np.nan, np.float32), m, n, k, ta, tb, 1.0, 0.0)
    assert np.linalg.norm(got - prod) <= TOL * np.linalg.norm(prod)
    assert np.abs(got - prod).max() <= 8 * TOL * np.sqrt(k)
    got = _matmul(hip, A, B, C0, m, n, k, ta, tb, -0.5, 1.0)
    want = C0 - 0.5 * prod
    assert np.linalg.norm(got - want) <= TOL * np.linalg.norm(want)


@pytest.mark.parametrize("shape,ta,tb", [
    # a small layer's weight gradient over a very long batch: up to 256 ranges of k and the reduction that adds many
    # partial products (64 x 64 tiles in every layout, the 32-wide blocks of the skinny products in the k-strided one)
    ((64, 64, 65536), False, False), ((64, 64, 65536 + 40), True, False), ((128, 70, 40000), False, True),
    ((16, 16, 300000), True, False), ((10, 64, 100000), True, False), ((64, 10, 70001), True, False),
    ((100, 30, 50000), True, True),
    # leading dimensions of 2^21 values and more: rows of millions of columns
    ((32, 32, (1 << 21) + 40), False, False), ((24, 40, (1 << 21) + 8), False, True), ((16, 8, 1 << 21), True, True)])
def test_products_over_a_very_long_k(hip, shape, ta, tb):
    m, n, k = shape
    r = np.random.default_rng(m + 3 * n + 7 * k)
    A = r.standard_normal((k, m) if ta else (m, k), dtype=np.float32)
    B = r.standard_normal((n, k) if tb else (k, n), dtype=np.float32)
    C0 = r.standard_normal((m, n), dtype=np.float32)
    prod = (A.T if ta else A).astype(np.float64) @ (B.T if tb else B).astype(np.float64)
    got = _matmul(hip, A, B, np.full((m, n), np.nan, np.float32), m, n, k, ta, tb, 1.0, 0.0)
    assert np.linalg.norm(got - prod) <= TOL * np.linalg.norm(prod)
    got = _matmul(hip, A, B, C0, m, n, k, ta, tb, -0.5, 1.0)
    want = C0 - 0.5 * prod
    assert np.linalg.norm(got - want) <= TOL * np.linalg.norm(want)


@pytest.mark.parametrize("m,n", [(5000, 300), (70000, 33), (64, 64), (63, 1), (1, 700), (4096, 4096), (130, 257)])
def test_transposed_matvec_over_many_rows(oracle, hip, m, n):
    """y = alpha A^T x + beta y with the rows split over workgroups (src/device/host_device.zig:232-240)."""
    r = np.random.default_rng(m * 3 + n)
    A = r.standard_normal((m, n), dtype=np.float32)
    x = r.standard_normal(m, dtype=np.float32)
    y0 = r.standard_normal(n, dtype=np.float32)
    want = 0.75 * (A.astype(np.float64).T @ x.astype(np.float64)) + 0.5 * y0
    p = {"A": A, "x": x, "y": y0.copy(), "m": m, "n": n, "trans_a": True, "alpha": 0.75, "beta": 0.5}
    got = run_op(hip, "matvec", dict(p), ["y"])["y"]
    assert np.linalg.norm(got - want) <= TOL * np.linalg.norm(want)
    if m * n <= 1 << 22:
        ref = run_op(oracle, "matvec", dict(p), ["y"])["y"]
        assert np.linalg.norm(got - ref) <= TOL * np.linalg.norm(ref)
    got = run_op(hip, "matvec", {**p, "y": np.full(n, np.nan, np.float32), "beta": 0.0}, ["y"])["y"]  # y is not read
    want0 = 0.75 * (A.astype(np.float64).T @ x.astype(np.float64))
    assert np.linalg.norm(got - want0) <= TOL * np.linalg.norm(want0)


def test_more_batches_than_one_grid_dimension_holds(hip):
    """bmm_acc over 70000 batches (a grid's z dimension ends at 65535): per-batch operands, and one B for all."""
    nb, s = 70000, 4
    r = np.random.default_rng(12)
    A = r.integers(-3, 4, (nb, s, s)).astype(np.float32)
    B = r.integers(-3, 4, (nb, s, s)).astype(np.float32)
    for shared_b in (False, True):
        Bop = B[:1] if shared_b else B
        a, b, c = hip.from_numpy(A), hip.from_numpy(Bop), hip.mem_alloc(F32, nb * s * s)
        hip.dispatch("bmm_acc", A=a, B=b, C=c, A_shape=[nb, s, s], B_shape=[Bop.shape[0], s, s], C_shape=[nb, s, s],
                     trans_a=False, trans_b=False, lda=s, ldb=s, ldc=s, alpha=1.0, beta=0.0)
        got = hip.to_numpy(c).reshape(nb, s, s)
        want = np.matmul(A, Bop if not shared_b else np.broadcast_to(Bop, A.shape))
        assert np.array_equal(got, want)  # small integers: exact
        for x in (a, b, c):
            hip.mem_free(x)
