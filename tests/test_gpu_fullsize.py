"""The op microbenchmark suite (configuration 2 of the benchmark definition) at its full sizes, checked through properties that do
not need a CPU pass over the whole problem: sampled entries against float64 dot products, exact elementwise
identities, row invariants of softmax cross-entropy, and doubling under accumulation."""
from __future__ import annotations

import numpy as np
import pytest

from zigrad_amd.device import F32, U64

pytestmark = pytest.mark.gpu
TOL = 1e-5


@pytest.mark.parametrize("ta,tb", [(False, False), (True, False), (False, True)])
def test_matmul_4096_cubed_sampled_entries(hip, ta, tb):
    n = 4096
    r = np.random.default_rng(5 + 2 * ta + tb)
    A = r.standard_normal((n, n), dtype=np.float32)
    B = r.standard_normal((n, n), dtype=np.float32)
    a, b, c = hip.from_numpy(A), hip.from_numpy(B), hip.mem_alloc(F32, n * n)
    hip.dispatch("matmul", A=a, B=b, C=c, m=n, n=n, k=n, trans_a=ta, trans_b=tb, lda=n, ldb=n, ldc=n, alpha=1.0, beta=0.0)
    C = hip.to_numpy(c).reshape(n, n)
    opA = (A.T if ta else A).astype(np.float64)
    opB = (B.T if tb else B).astype(np.float64)
    # 8 whole rows, 8 whole columns and 512 scattered entries: every tile row / column and both lane halves are hit
    rows = r.integers(0, n, 8)
    cols = r.integers(0, n, 8)
    want_rows = opA[rows] @ opB
    want_cols = opA @ opB[:, cols]
    assert np.abs(C[rows] - want_rows).max() <= 4 * TOL * np.sqrt(n)  # sqrt(n) = rms magnitude of an entry of C
    assert np.linalg.norm(C[rows] - want_rows) <= TOL * np.linalg.norm(want_rows)
    assert np.linalg.norm(C[:, cols] - want_cols) <= TOL * np.linalg.norm(want_cols)
    ii, jj = r.integers(0, n, 512), r.integers(0, n, 512)
    want = np.einsum("ik,ki->i", opA[ii], opB[:, jj])
    assert np.linalg.norm(C[ii, jj] - want) <= TOL * np.linalg.norm(want)
    # linearity in alpha and accumulation with beta: C2 = 0.5 * op(A) op(B) + 2 * C  ==  2.5 * C up to rounding
    hip.dispatch("matmul", A=a, B=b, C=c, m=n, n=n, k=n, trans_a=ta, trans_b=tb, lda=n, ldb=n, ldc=n, alpha=0.5, beta=2.0)
    C2 = hip.to_numpy(c).reshape(n, n)
    assert np.linalg.norm(C2[rows] - 2.5 * C[rows].astype(np.float64)) <= 2e-7 * np.linalg.norm(2.5 * C[rows])
    for x in (a, b, c):
        hip.mem_free(x)


def test_bmm_32_by_512_cubed_sampled_batches(hip):
    nb, s = 32, 512
    r = np.random.default_rng(9)
    A = r.standard_normal((nb, s, s), dtype=np.float32)
    B = r.standard_normal((nb, s, s), dtype=np.float32)
    a, b, c = hip.from_numpy(A), hip.from_numpy(B), hip.mem_alloc(F32, nb * s * s)
    hip.dispatch("bmm_acc", A=a, B=b, C=c, A_shape=[nb, s, s], B_shape=[nb, s, s], C_shape=[nb, s, s], trans_a=False,
                 trans_b=False, lda=s, ldb=s, ldc=s, alpha=1.0, beta=0.0)
    C = hip.to_numpy(c).reshape(nb, s, s)
    for i in (0, 13, 31):
        want = A[i].astype(np.float64) @ B[i].astype(np.float64)
        assert np.linalg.norm(C[i] - want) <= TOL * np.linalg.norm(want)
    for x in (a, b, c):
        hip.mem_free(x)


def test_broadcast_add_and_axis_reductions_8192x4096(hip):
    rows, cols = 8192, 4096
    r = np.random.default_rng(11)
    X = r.standard_normal((rows, cols), dtype=np.float32)
    bias = r.standard_normal(cols, dtype=np.float32)
    x, bb, z = hip.from_numpy(X), hip.from_numpy(bias), hip.mem_alloc(F32, rows * cols)
    hip.dispatch("add", x=x, y=bb, z=z)
    assert np.array_equal(hip.to_numpy(z).reshape(rows, cols), X + bias)  # one rounding per element: exact
    y = hip.mem_alloc(F32, rows)
    hip.dispatch("sum_along", x=x, x_shape=[rows, cols], y=y, dim=1)
    want = X.astype(np.float64).sum(axis=1)
    assert np.linalg.norm(hip.to_numpy(y) - want) <= TOL * np.linalg.norm(want)
    hip.mem_fill(y, 0.0)
    hip.dispatch("max_along", x=x, x_shape=[rows, cols], y=y, dim=1)
    assert np.array_equal(hip.to_numpy(y), X.max(axis=1))
    idx = hip.mem_alloc(U64, rows)
    hip.dispatch("argmax_along", x=x, x_shape=[rows, cols], y=idx, dim=1)
    assert np.array_equal(hip.to_numpy(idx), X.argmax(axis=1).astype(np.uint64))
    for b in (x, bb, z, y, idx):
        hip.mem_free(b)


def test_smce_label_8192x32000_invariants(hip):
    M, N, base = 8192, 32000, 64
    r = np.random.default_rng(13)
    block = r.standard_normal((base, N), dtype=np.float32)  # the logits repeat every 64 rows; the labels do not
    labels = r.integers(0, N, M).astype(np.uint64)
    logits, grad = hip.mem_alloc(F32, M * N), hip.mem_alloc(F32, M * N)
    blk = hip.from_numpy(block)
    for i in range(M // base):
        hip.mem_copy(blk, logits.sub(i * base * N, base * N))
    lab = hip.from_numpy(labels)
    lse, loss = hip.mem_alloc(F32, M), hip.mem_alloc(F32, 1)
    hip.dispatch("smce_label_fwd", logits=logits, labels=lab, lse=lse, loss=loss, rows=M, cols=N)
    b64 = block.astype(np.float64)
    mx = b64.max(axis=1, keepdims=True)
    want_lse = (mx[:, 0] + np.log(np.exp(b64 - mx).sum(axis=1)))
    got_lse = hip.to_numpy(lse).reshape(M // base, base)
    assert np.abs(got_lse - want_lse).max() <= 2e-5  # |lse| is about 11: 1e-5 relative with margin for float32 log
    x_lab = b64[np.arange(M) % base, labels.astype(np.int64)]
    p = np.clip(np.exp(x_lab - np.tile(want_lse, M // base)), 1e-7, 1 - 1e-7)
    want_loss = -np.log(p).mean()
    assert abs(hip.to_numpy(loss)[0] - want_loss) <= 1e-5 * want_loss

    hip.mem_fill(grad, 0.0)
    hip.dispatch("smce_label_bwd", logits=logits, labels=lab, lse=lse, grad=grad, rows=M, cols=N, accumulate=True)
    # every row of the gradient sums to (sum p - 1) / M = 0
    rs = hip.mem_alloc(F32, M)
    hip.dispatch("sum_along", x=grad, x_shape=[M, N], y=rs, dim=1)
    assert np.abs(hip.to_numpy(rs)).max() <= 1e-8  # entries are about 1 / (M N) in size
    # sampled rows against the closed form softmax - onehot, / M
    for row in (0, 63, 4097, M - 1):
        g = hip.to_numpy(grad.sub(row * N, N))
        want = np.exp(b64[row % base] - want_lse[row % base])
        want[int(labels[row])] -= 1.0
        want /= M
        assert np.linalg.norm(g - want) <= TOL * np.linalg.norm(want)
    # accumulate = False overwrites and gives the same values; accumulating once more doubles them exactly
    first = hip.to_numpy(grad.sub(5 * N, N)).copy()
    hip.dispatch("smce_label_bwd", logits=logits, labels=lab, lse=lse, grad=grad, rows=M, cols=N, accumulate=False)
    assert np.array_equal(hip.to_numpy(grad.sub(5 * N, N)), first)
    hip.dispatch("smce_label_bwd", logits=logits, labels=lab, lse=lse, grad=grad, rows=M, cols=N, accumulate=True)
    assert np.array_equal(hip.to_numpy(grad.sub(5 * N, N)), 2 * first)
    for b in (logits, grad, blk, lab, lse, loss, rs):
        hip.mem_free(b)
