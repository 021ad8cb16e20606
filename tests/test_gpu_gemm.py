"""fp32 GEMM family on the matrix cores against the oracle (BLAS sgemm) and an fp64-accumulated GEMM.

Tolerance: relative Frobenius error <= 1e-5 against the fp64-accumulated result (the benchmark definition's per-op
bound); cases built from small integers or permutation matrices are exact in fp32 and compared bit for bit.
"""
from __future__ import annotations

import numpy as np
import pytest

from conftest import rel_fro

pytestmark = pytest.mark.gpu
TOL = 1e-5


def rng(seed):
    return np.random.default_rng(seed)


def stored(r, rows, cols, ld, ints=False):
    """A row-major matrix with leading dimension ld >= cols (padding filled with NaN to catch stray reads)."""
    a = np.full((rows, ld), np.nan, np.float32)
    a[:, :cols] = r.integers(-3, 4, (rows, cols)).astype(np.float32) if ints else r.standard_normal((rows, cols)).astype(np.float32)
    return a


def run_matmul(dev, A, B, C, m, n, k, ta, tb, lda, ldb, ldc, alpha, beta):
    a, b, c = dev.from_numpy(A), dev.from_numpy(B), dev.from_numpy(C)
    dev.dispatch("matmul", A=a, B=b, C=c, m=m, n=n, k=k, trans_a=ta, trans_b=tb, lda=lda, ldb=ldb, ldc=ldc, alpha=alpha,
                 beta=beta)
    dev.sync()
    out = dev.to_numpy(c).reshape(C.shape)
    for x in (a, b, c):
        dev.mem_free(x)
    return out


SHAPES = [
    # (m, n, k)                      the Linear layers of the configurations and awkward sizes
    (64, 128, 784), (64, 64, 128), (64, 10, 64), (64, 128, 4), (64, 2, 128), (128, 784, 64), (10, 64, 64),
    (2708, 16, 1433), (2708, 7, 16), (16, 1433, 2708), (1, 1, 1), (33, 65, 17), (129, 257, 31), (256, 128, 16),
    (512, 384, 160), (300, 500, 70), (1024, 1024, 256),
    # few C tiles and a deep k: the split-k path, whole tiles (fast kernels) and ragged
    (128, 64, 2048), (64, 64, 4096), (70, 50, 1000),
    # aligned but ragged in m and n (edge kernels: clamped loads, guarded stores), with and without a k remainder
    (2072, 1300, 1028), (4100, 2060, 100), (2072, 1300, 1024), (1000, 1000, 512), (100, 68, 64), (4, 4, 32),
    # nothing a multiple of anything: odd m, n, k and (with the padding rule below) odd leading dimensions, so pieces
    # of 16 bytes straddle the edges of the operands, C takes scalar stores and the last k-tiles are masked
    (1023, 1021, 1019), (515, 259, 1031), (258, 1026, 2050), (1025, 3, 1025), (5, 1027, 513),
    # tall with at most 16 columns and a k of 512 to 2048
    (512, 16, 512), (600, 1, 2048), (4096, 10, 1000), (513, 15, 577), (1000, 16, 2049), (511, 16, 600), (700, 17, 600),
    # at most 16 rows, wide, over a long k
    (16, 256, 512), (7, 1433, 2708), (1, 300, 5000), (16, 257, 32768), (15, 1000, 513), (16, 255, 600), (17, 300, 600),
]


@pytest.mark.parametrize("m,n,k", SHAPES)
@pytest.mark.parametrize("ta,tb", [(False, False), (False, True), (True, False), (True, True)])
def test_matmul_variants(oracle, hip, m, n, k, ta, tb):
    r = rng(m * 131 + n * 17 + k + 2 * ta + tb)
    pad = 0 if (m + n + k) % 2 == 0 else 3  # alternate between tight and padded leading dimensions
    lda = (m if ta else k) + pad
    ldb = (k if tb else n) + pad
    ldc = n + pad
    A = stored(r, k if ta else m, m if ta else k, lda)
    B = stored(r, n if tb else k, k if tb else n, ldb)
    C0 = stored(r, m, n, ldc)
    for alpha, beta in [(1.0, 0.0), (1.0, 1.0), (0.5, -2.0)]:
        Cin = C0.copy()
        if beta == 0.0:
            Cin[:, :n] = np.nan  # must not be read
        got = run_matmul(hip, A, B, Cin, m, n, k, ta, tb, lda, ldb, ldc, alpha, beta)
        A64 = A[:, : (m if ta else k)].astype(np.float64)
        B64 = B[:, : (k if tb else n)].astype(np.float64)
        opA = A64.T if ta else A64
        opB = B64.T if tb else B64
        truth = alpha * (opA @ opB) + (beta * C0[:, :n].astype(np.float64) if beta != 0.0 else 0.0)
        assert rel_fro(got[:, :n], truth) <= TOL, (alpha, beta)
        if pad:
            assert np.all(np.isnan(got[:, n:])), "padding of C was written"
        ref = run_matmul(oracle, np.nan_to_num(A), np.nan_to_num(B), np.nan_to_num(Cin), m, n, k, ta, tb, lda, ldb, ldc, alpha, beta)
        assert rel_fro(got[:, :n], ref[:, :n]) <= TOL


@pytest.mark.parametrize("ta,tb", [(False, True), (True, False)])
def test_matmul_with_a_leading_dimension_beyond_32_bit_offsets(hip, ta, tb):
    """lda = 2^21 floats: a 256-row tile no longer fits 32-bit byte offsets, so the checked kernels take over."""
    r = rng(77 + ta)
    m, n, k, ld = 24, 40, 72, 1 << 21
    if ta:  # A stored [k, lda] with m valid columns, B stored [k, ldb]
        A = np.zeros((k, ld), np.float32); A[:, :m] = r.standard_normal((k, m))
        B = np.zeros((k, ld), np.float32); B[:, :n] = r.standard_normal((k, n))
        truth = A[:, :m].astype(np.float64).T @ B[:, :n].astype(np.float64)
    else:   # A stored [m, lda] with k valid columns, B stored [n, ldb]
        A = np.zeros((m, ld), np.float32); A[:, :k] = r.standard_normal((m, k))
        B = np.zeros((n, ld), np.float32); B[:, :k] = r.standard_normal((n, k))
        truth = A[:, :k].astype(np.float64) @ B[:, :k].astype(np.float64).T
    got = run_matmul(hip, A, B, np.full((m, n), np.nan, np.float32), m, n, k, ta, tb, ld, ld, n, 1.0, 0.0)
    assert rel_fro(got, truth) <= TOL


@pytest.mark.parametrize("ta,tb", [(False, False), (False, True), (True, False), (True, True)])
def test_matmul_exact_on_integers(oracle, hip, ta, tb):
    """Small integers make every product and partial sum exact in fp32: results must agree bit for bit."""
    m, n, k = 384, 256, 320
    r = rng(99 + 2 * ta + tb)
    A = stored(r, k if ta else m, m if ta else k, m if ta else k, ints=True)
    B = stored(r, n if tb else k, k if tb else n, k if tb else n, ints=True)
    C0 = stored(r, m, n, n, ints=True)
    got = run_matmul(hip, A, B, C0.copy(), m, n, k, ta, tb, A.shape[1], B.shape[1], n, 2.0, 1.0)
    ref = run_matmul(oracle, A, B, C0.copy(), m, n, k, ta, tb, A.shape[1], B.shape[1], n, 2.0, 1.0)
    np.testing.assert_array_equal(got, ref)
    opA = A.T if ta else A
    opB = B.T if tb else B
    np.testing.assert_array_equal(got, (2.0 * (opA.astype(np.float64) @ opB.astype(np.float64)) + C0).astype(np.float32))


def test_matmul_permutation_is_exact(hip):
    n = 512
    r = rng(4)
    P = np.eye(n, dtype=np.float32)[r.permutation(n)]
    X = r.standard_normal((n, n)).astype(np.float32)
    got = run_matmul(hip, P, X, np.zeros((n, n), np.float32), n, n, n, False, False, n, n, n, 1.0, 0.0)
    np.testing.assert_array_equal(got, P @ X)


def test_matmul_large_tile_path(oracle, hip):
    """Big enough to take the 256x128 tile, all four layouts, against BLAS."""
    m = n = 2048
    k = 512
    r = rng(12)
    for ta, tb in [(False, False), (False, True), (True, False), (True, True)]:
        A = stored(r, k if ta else m, m if ta else k, m if ta else k)
        B = stored(r, n if tb else k, k if tb else n, k if tb else n)
        C0 = stored(r, m, n, n)
        got = run_matmul(hip, A, B, C0.copy(), m, n, k, ta, tb, A.shape[1], B.shape[1], n, 1.0, 1.0)
        ref = run_matmul(oracle, A, B, C0.copy(), m, n, k, ta, tb, A.shape[1], B.shape[1], n, 1.0, 1.0)
        assert rel_fro(got, ref) <= TOL


def test_matmul_degenerate(hip):
    C = np.full((4, 5), 3.0, np.float32)
    A = np.ones((4, 1), np.float32)
    B = np.ones((1, 5), np.float32)
    # alpha == 0 leaves beta * C
    got = run_matmul(hip, A, B, C.copy(), 4, 5, 1, False, False, 1, 5, 5, 0.0, 2.0)
    np.testing.assert_array_equal(got, 2.0 * C)
    from zigrad_amd import ZgHipError

    with pytest.raises(ZgHipError, match="ldc"):
        run_matmul(hip, A, B, C.copy(), 4, 5, 1, False, False, 1, 5, 4, 1.0, 0.0)


@pytest.mark.parametrize("nba,nbb,nbc", [(32, 32, 32), (1, 4, 4), (4, 1, 4), (2, 4, 4)])
def test_bmm_acc_batches(oracle, hip, nba, nbb, nbc):
    m, n, k = 96, 80, 48
    r = rng(nba * 100 + nbb * 10 + nbc)
    A = r.standard_normal((nba, m, k)).astype(np.float32)
    B = r.standard_normal((nbb, k, n)).astype(np.float32)
    C0 = r.standard_normal((nbc, m, n)).astype(np.float32)
    res = []
    for dev in (oracle, hip):
        a, b, c = dev.from_numpy(A), dev.from_numpy(B), dev.from_numpy(C0)
        dev.dispatch("bmm_acc", A=a, B=b, C=c, A_shape=[nba, m, k], B_shape=[nbb, k, n], C_shape=[nbc, m, n], trans_a=False,
                     trans_b=False, lda=k, ldb=n, ldc=n, alpha=1.0, beta=1.0)
        dev.sync()
        res.append(dev.to_numpy(c).reshape(nbc, m, n))
    assert rel_fro(res[1], res[0]) <= TOL
    truth = np.stack([A[i % nba].astype(np.float64) @ B[i % nbb].astype(np.float64) for i in range(nbc)]) + C0
    assert rel_fro(res[1], truth) <= TOL


@pytest.mark.parametrize("nb,m,n,k,nba,nbb,ta,tb", [(5000, 8, 8, 8, 5000, 5000, False, False), (4096, 8, 8, 64, 4096, 1, False, True),
                                                    (70000, 4, 4, 4, 70000, 70000, True, False), (4100, 3, 5, 7, 1, 4100, True, True),
                                                    (6000, 1, 8, 33, 6000, 6000, False, False),
                                                    # just outside: 16 x 16 blocks go a workgroup per product
                                                    (4096, 16, 16, 16, 4096, 1, False, True)])
def test_thousands_of_very_small_products(hip, nb, m, n, k, nba, nbb, ta, tb):
    """Batches of at least 4096 products of at most 8 x 8 x 64 take a thread per element of C: every layout, an operand
    shared by all products, alpha and beta."""
    r = rng(nb + m * 7 + n * 11 + k)
    A = r.standard_normal((nba, k, m) if ta else (nba, m, k)).astype(np.float32)
    B = r.standard_normal((nbb, n, k) if tb else (nbb, k, n)).astype(np.float32)
    C0 = r.standard_normal((nb, m, n)).astype(np.float32)
    a, b, c = hip.from_numpy(A), hip.from_numpy(B), hip.from_numpy(C0)
    hip.dispatch("bmm_acc", A=a, B=b, C=c, A_shape=[nba, m, k], B_shape=[nbb, k, n], C_shape=[nb, m, n], trans_a=ta,
                 trans_b=tb, lda=(m if ta else k), ldb=(k if tb else n), ldc=n, alpha=0.5, beta=-1.0)
    hip.sync()
    got = hip.to_numpy(c).reshape(nb, m, n)
    A64 = (A.transpose(0, 2, 1) if ta else A).astype(np.float64)
    B64 = (B.transpose(0, 2, 1) if tb else B).astype(np.float64)
    ia, ib = np.arange(nb) % nba, np.arange(nb) % nbb
    truth = 0.5 * np.einsum("bik,bkj->bij", A64[ia], B64[ib]) - C0
    assert rel_fro(got, truth) <= TOL
    for x in (a, b, c):
        hip.mem_free(x)


def test_bmm_acc_split_k_batches(oracle, hip):
    """Batched products with few C tiles and a deep k take the split-k path: partial products per batch and split."""
    nb, m, n, k = 3, 64, 48, 1536
    r = rng(7)
    A = r.standard_normal((nb, m, k)).astype(np.float32)
    B = r.standard_normal((1, n, k)).astype(np.float32)  # one B shared by all batches, stored transposed
    C0 = r.standard_normal((nb, m, n)).astype(np.float32)
    res = []
    for dev in (oracle, hip):
        a, b, c = dev.from_numpy(A), dev.from_numpy(B), dev.from_numpy(C0)
        dev.dispatch("bmm_acc", A=a, B=b, C=c, A_shape=[nb, m, k], B_shape=[1, k, n], C_shape=[nb, m, n], trans_a=False,
                     trans_b=True, lda=k, ldb=k, ldc=n, alpha=0.5, beta=1.0)
        dev.sync()
        res.append(dev.to_numpy(c).reshape(nb, m, n))
    truth = 0.5 * np.stack([A[i].astype(np.float64) @ B[0].astype(np.float64).T for i in range(nb)]) + C0
    assert rel_fro(res[1], truth) <= TOL
    assert rel_fro(res[1], res[0]) <= TOL


@pytest.mark.parametrize("m,n,k", [(64, 128, 784), (40, 40, 16384), (33, 31, 16392), (500, 500, 300), (16, 1433, 2708),
                                   (2708, 16, 1433), (1000, 7, 600)])
def test_small_products_with_a_long_k_repeat_bit_for_bit(hip, m, n, k):
    """A small C with a long k is cut into ranges of k over several workgroups per tile of C, and the partial tiles
    are added in range order by a second kernel: repeated launches give the same bits, and the values match float64
    to the tolerance."""
    r = rng(m + n + k)
    A = r.standard_normal((m, k)).astype(np.float32)
    B = r.standard_normal((n, k)).astype(np.float32)
    C0 = r.standard_normal((m, n)).astype(np.float32)
    outs = [run_matmul(hip, A, B, C0.copy(), m, n, k, False, True, k, k, n, 1.0, 1.0) for _ in range(4)]
    for o in outs[1:]:
        assert np.array_equal(o, outs[0])
    truth = A.astype(np.float64) @ B.astype(np.float64).T + C0
    assert rel_fro(outs[0], truth) <= TOL


def test_bmm_32x512_cubed(oracle, hip):
    """The microbenchmark shape: batch 32 of 512 x 512 x 512, transposed-B layout as well."""
    r = rng(77)
    A = r.standard_normal((32, 512, 512)).astype(np.float32)
    B = r.standard_normal((32, 512, 512)).astype(np.float32)
    for tb in (False, True):
        res = []
        for dev in (oracle, hip):
            a, b = dev.from_numpy(A), dev.from_numpy(B)
            c = dev.from_numpy(np.full((32, 512, 512), np.nan, np.float32))
            dev.dispatch("bmm_acc", A=a, B=b, C=c, A_shape=[32, 512, 512], B_shape=[32, 512, 512], C_shape=[32, 512, 512],
                         trans_a=False, trans_b=tb, lda=512, ldb=512, ldc=512, alpha=1.0, beta=0.0)
            dev.sync()
            res.append(dev.to_numpy(c))
            for x in (a, b, c):
                dev.mem_free(x)
        assert rel_fro(res[1], res[0]) <= TOL


@pytest.mark.parametrize("m,n", [(2, 2), (64, 784), (1000, 33), (5, 4097),
                                 # every lanes-per-row shape of the row kernel, rows cut into segments, a reduced axis cut
                                 # into many chunks, tiles of the transpose that end inside the matrix
                                 (3, 300000), (7, 20000), (300, 16384), (100000, 8), (5000, 64), (4096, 256), (70000, 12),
                                 (130, 5000), (64, 64), (256, 1000), (1000, 1024), (68, 132), (1, 70000), (70000, 1),
                                 # transposes whose tiles are numbered down the diagonals (wide, both sides multiples of 1024)
                                 # and the tall counterpart that is not
                                 (1024, 1024), (1024, 3072), (2048, 1024),
                                 # rows short enough for two lanes each
                                 (3000, 20), (3000, 17)])
def test_matvec_outer_transpose(oracle, hip, m, n):
    r = rng(m + n)
    A = r.standard_normal((m, n)).astype(np.float32)
    for ta in (False, True):
        x = r.standard_normal(m if ta else n).astype(np.float32)
        y0 = r.standard_normal(n if ta else m).astype(np.float32)
        res = []
        for dev in (oracle, hip):
            a, xx, yy = dev.from_numpy(A), dev.from_numpy(x), dev.from_numpy(y0)
            dev.dispatch("matvec", A=a, x=xx, y=yy, m=m, n=n, trans_a=ta, alpha=0.5, beta=2.0)
            dev.sync()
            res.append(dev.to_numpy(yy))
        truth = 0.5 * ((A.T if ta else A).astype(np.float64) @ x) + 2.0 * y0
        assert rel_fro(res[1], truth) <= TOL and rel_fro(res[0], truth) <= TOL
    # outer: A += alpha x y^T
    x, y = r.standard_normal(m).astype(np.float32), r.standard_normal(n).astype(np.float32)
    res = []
    for dev in (oracle, hip):
        a, xx, yy = dev.from_numpy(A), dev.from_numpy(x), dev.from_numpy(y)
        dev.dispatch("outer", x=xx, y=yy, A=a, alpha=0.25)
        dev.sync()
        res.append(dev.to_numpy(a))
    assert rel_fro(res[1], res[0]) <= 1e-6
    # transpose: B = A^T + alpha B, alpha = 0 must not read B
    for alpha in (0.0, 1.0):
        B0 = np.full((n, m), np.nan, np.float32) if alpha == 0.0 else r.standard_normal((n, m)).astype(np.float32)
        a, b = hip.from_numpy(A), hip.from_numpy(B0)
        hip.dispatch("transpose", A=a, B=b, m=m, n=n, alpha=alpha)
        hip.sync()
        want = A.T if alpha == 0.0 else A.T + B0
        np.testing.assert_array_equal(hip.to_numpy(b).reshape(n, m), want)
