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


def test_unary_ops_and_their_backward_8192x4096(oracle, hip):
    """The unary ops at the op suite's size against the oracle on the same data: relu exactly (no rounding), the
    transcendental ones to 1e-6 (the device's expf/tanhf and the host's are both within an ulp or two of the truth)."""
    from conftest import run_op

    rows, cols = 8192, 4096
    n = rows * cols
    r = np.random.default_rng(21)
    X = r.standard_normal(n, dtype=np.float32)
    YG = r.standard_normal(n, dtype=np.float32)
    G0 = r.standard_normal(n, dtype=np.float32)
    x, yg, g, y = hip.from_numpy(X), hip.from_numpy(YG), hip.from_numpy(G0), hip.mem_alloc(F32, n)
    for name in ("relu_fwd", "tanh_fwd", "sigm_fwd", "exp_fwd"):
        hip.dispatch(name, x=x, y=y)
        got = hip.to_numpy(y)
        want = run_op(oracle, name, {"x": X, "y": np.zeros(n, np.float32)}, ["y"])["y"]
        if name == "relu_fwd":
            assert np.array_equal(got, want)
        else:
            assert np.linalg.norm(got - want) <= 1e-6 * np.linalg.norm(want), name
    # backward: x_g += f'(.) * y_g on the same buffers the benchmark uses them on
    hip.dispatch("relu_bwd", x=x, x_g=g, y_g=yg)
    want = run_op(oracle, "relu_bwd", {"x": X, "x_g": G0.copy(), "y_g": YG}, ["x_g"])["x_g"]
    assert np.array_equal(hip.to_numpy(g), want)
    T = np.tanh(X)
    t = hip.from_numpy(T)
    for name in ("tanh_bwd", "sigm_bwd", "exp_bwd"):
        hip.mem_transfer(G0, g, "HtoD")
        hip.dispatch(name, x_g=g, y=t, y_g=yg)
        want = run_op(oracle, name, {"x_g": G0.copy(), "y": T, "y_g": YG}, ["x_g"])["x_g"]
        assert np.linalg.norm(hip.to_numpy(g) - want) <= 1e-6 * np.linalg.norm(want), name
    hip.mem_transfer(G0, g, "HtoD")
    hip.dispatch("relu_inplace_bwd", x=x, x_g=g)
    assert np.array_equal(hip.to_numpy(g), np.where(X > 0, G0, np.float32(0.0)))
    hip.dispatch("mul", x=x, y=yg, z=y)
    assert np.array_equal(hip.to_numpy(y), X * YG)          # one rounding per element: exact
    for b in (x, yg, g, y, t):
        hip.mem_free(b)


def test_reductions_along_the_other_axis_and_norms_8192x4096(hip):
    rows, cols = 8192, 4096
    r = np.random.default_rng(22)
    X = r.standard_normal((rows, cols), dtype=np.float32)
    x = hip.from_numpy(X)
    ycol = hip.mem_alloc(F32, cols)
    hip.dispatch("sum_along", x=x, x_shape=[rows, cols], y=ycol, dim=0)
    want = X.astype(np.float64).sum(axis=0)
    assert np.linalg.norm(hip.to_numpy(ycol) - want) <= TOL * np.linalg.norm(want)
    hip.dispatch("max_along", x=x, x_shape=[rows, cols], y=ycol, dim=0)
    assert np.array_equal(hip.to_numpy(ycol), X.max(axis=0))
    icol = hip.mem_alloc(U64, cols)
    hip.dispatch("argmax_along", x=x, x_shape=[rows, cols], y=icol, dim=0)
    assert np.array_equal(hip.to_numpy(icol), X.argmax(axis=0).astype(np.uint64))
    one = hip.mem_alloc(F32, 1)
    hip.dispatch("nrm2", x=x, y=one)
    truth = np.sqrt((X.astype(np.float64) ** 2).sum())
    assert abs(float(hip.to_numpy(one)[0]) - truth) <= 2e-6 * truth
    # the bias gradient of the wide MLP's layers: unbroadcast of [4096,4096] and [4096,1024] to a row, accumulated
    from zigrad_amd import host
    for c in (4096, 1024):
        G = r.standard_normal((4096, c), dtype=np.float32)
        b0 = r.standard_normal(c, dtype=np.float32)
        gb, bb = hip.from_numpy(G), hip.from_numpy(b0)
        host.unbroadcast_(hip, gb, [4096, c], bb, [c], alpha=1.0, beta=1.0)
        want = G.astype(np.float64).sum(axis=0) + b0
        assert np.linalg.norm(hip.to_numpy(bb) - want) <= TOL * np.linalg.norm(want)
        hip.mem_free(gb)
        hip.mem_free(bb)
    for b in (x, ycol, icol, one):
        hip.mem_free(b)


def test_optimizer_updates_of_a_4096x4096_weight(oracle, hip):
    """SGD and Adam on 16.8 M parameters, clip off and on, against the oracle on the same data."""
    from conftest import run_op

    n = 4096 * 4096
    r = np.random.default_rng(23)
    P = r.standard_normal(n, dtype=np.float32)
    G = (r.standard_normal(n, dtype=np.float32) * np.float32(0.01))
    M0 = (r.standard_normal(n, dtype=np.float32) * np.float32(0.01))
    V0 = (r.random(n, dtype=np.float32) * np.float32(1e-4))
    for clip in (False, True):
        p, g = hip.from_numpy(P), hip.from_numpy(G)
        hip.dispatch("sgd_step", param=p, grad=g, lr=0.01, clip=clip, max_norm=10.0, delta=1e-6)
        want = run_op(oracle, "sgd_step", {"param": P.copy(), "grad": G.copy(), "lr": 0.01, "clip": clip, "max_norm": 10.0,
                                           "delta": 1e-6}, ["param", "grad"])
        assert np.linalg.norm(hip.to_numpy(p) - want["param"]) <= 1e-6 * np.linalg.norm(want["param"])
        assert np.linalg.norm(hip.to_numpy(g) - want["grad"]) <= 1e-6 * np.linalg.norm(want["grad"])
        hip.mem_transfer(P, p, "HtoD")
        hip.mem_transfer(G, g, "HtoD")
        m, v = hip.from_numpy(M0), hip.from_numpy(V0)
        kw = dict(t=7, lr=1e-3, beta1=0.9, beta2=0.999, epsilon=1e-8, clip=clip, max_norm=10.0, delta=1e-6)
        hip.dispatch("adam_step", param=p, grad=g, m=m, v=v, **kw)
        want = run_op(oracle, "adam_step", {"param": P.copy(), "grad": G.copy(), "m": M0.copy(), "v": V0.copy(), **kw},
                      ["param", "m", "v"])
        for name, buf in (("param", p), ("m", m), ("v", v)):
            assert np.linalg.norm(hip.to_numpy(buf) - want[name]) <= 1e-6 * np.linalg.norm(want[name]), (clip, name)
        for b in (p, g, m, v):
            hip.mem_free(b)


def test_gather_of_random_rows_65536x256(hip):
    n_rows, stride, n_idx = 131072, 256, 65536
    r = np.random.default_rng(24)
    S = r.standard_normal((n_rows, stride), dtype=np.float32)
    idx = r.integers(0, n_rows, n_idx).astype(np.uint64)
    s, i, d = hip.from_numpy(S), hip.from_numpy(idx), hip.mem_alloc(F32, n_idx * stride)
    hip.dispatch("index_select_fwd", src=s, indices=i, stride=stride, dst=d)
    assert np.array_equal(hip.to_numpy(d).reshape(n_idx, stride), S[idx.astype(np.int64)])
    for b in (s, i, d):
        hip.mem_free(b)
