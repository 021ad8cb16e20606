"""Float fills wait in the context and go out as one launch with the next call that is not a fill
(src/device/host_device.zig:876-884 fills at once; callers zero gradients tensor by tensor).  Whatever the caller does
next must see every fill: later fills win over earlier ones on the same memory, a freed block's fill does not land on
its next owner, more fills than the queue holds, odd offsets and lengths, and fills recorded into a graph."""
from __future__ import annotations

import numpy as np
import pytest

from zigrad_amd.device import F32

pytestmark = pytest.mark.gpu


def test_many_fills_of_odd_pieces_then_a_read(hip):
    r = np.random.default_rng(0)
    n = 300_000
    buf = hip.from_numpy(np.full(n, -1.0, np.float32))
    want = np.full(n, -1.0, np.float32)
    pos = 0
    k = 0
    while pos < n and k < 40:  # 40 fills: the queue (16) is sent more than once
        length = int(r.integers(1, 20_000))
        off = pos + int(r.integers(0, 7))  # 4-byte aligned only
        if off + length > n:
            break
        hip.mem_fill(buf.sub(off, length), float(k))
        want[off:off + length] = k
        pos = off + length
        k += 1
    np.testing.assert_array_equal(hip.to_numpy(buf), want)  # the read comes after every fill
    hip.mem_free(buf)


def test_a_later_fill_wins_where_two_overlap(hip):
    buf = hip.mem_alloc(F32, 10_000)
    hip.mem_fill(buf, 1.0)
    hip.mem_fill(buf.sub(100, 5000), 2.0)
    hip.mem_fill(buf.sub(4000, 3000), 3.0)
    hip.mem_fill(buf.sub(0, 1), 4.0)
    want = np.full(10_000, 1.0, np.float32)
    want[100:5100] = 2.0
    want[4000:7000] = 3.0
    want[0] = 4.0
    np.testing.assert_array_equal(hip.to_numpy(buf), want)
    hip.mem_free(buf)


def test_a_fill_then_an_op_on_the_same_memory(hip):
    n = 5000
    a = hip.from_numpy(np.arange(n, dtype=np.float32))
    b = hip.mem_alloc(F32, n)
    hip.mem_fill(b, 0.5)
    hip.dispatch("add", x=a, y=b, z=b)  # reads the filled values, in place
    np.testing.assert_array_equal(hip.to_numpy(b), np.arange(n, dtype=np.float32) + 0.5)
    hip.mem_fill(a, 0.0)
    hip.dispatch("relu_fwd", x=b, y=a)  # overwrites what the waiting fill wrote: the fill must not come after it
    np.testing.assert_array_equal(hip.to_numpy(a), np.arange(n, dtype=np.float32) + 0.5)
    for x in (a, b):
        hip.mem_free(x)


def test_a_fill_of_a_block_that_is_freed_does_not_reach_its_next_owner(hip):
    n = 4096
    first = hip.mem_cache_alloc(F32, n)
    hip.mem_fill(first, 9.0)
    hip.mem_cache_free(first)                 # the fill is sent before the block returns to the pool
    second = hip.mem_cache_alloc(F32, n)      # most likely the same block
    hip.mem_transfer(np.full(n, 1.0, np.float32), second, "HtoD")
    hip.sync()
    np.testing.assert_array_equal(hip.to_numpy(second), np.full(n, 1.0, np.float32))
    # allocations in between leave fills waiting; they still all arrive
    bufs = []
    for i in range(20):
        b = hip.mem_cache_alloc(F32, 1000 + i)
        hip.mem_fill(b, float(i))
        bufs.append(b)
    for i, b in enumerate(bufs):
        np.testing.assert_array_equal(hip.to_numpy(b), np.full(1000 + i, float(i), np.float32))
        hip.mem_cache_free(b)
    hip.mem_cache_free(second)


def test_fills_recorded_into_a_graph_replay_with_it(hip):
    n = 3000
    a, b, out = hip.mem_alloc(F32, n), hip.mem_alloc(F32, n), hip.mem_alloc(F32, n)
    hip.mem_fill(a, 0.0)
    hip.mem_fill(b, 0.0)
    hip.mem_fill(out, 0.0)
    hip.sync()
    hip.mem_fill(a, 7.0)  # waiting when the recording starts: sent before it, not recorded
    hip.graph_open()
    hip.mem_fill(a, 2.0)
    hip.mem_fill(b, 3.0)
    hip.dispatch("add", x=a, y=b, z=out)
    hip.mem_fill(b, 1.0)  # waiting when the recording ends: recorded
    g = hip.graph_save()
    for _ in range(3):
        hip.mem_transfer(np.full(n, -5.0, np.float32), a, "HtoD")
        hip.mem_transfer(np.full(n, -5.0, np.float32), b, "HtoD")
        g.run()
        hip.sync()
        np.testing.assert_array_equal(hip.to_numpy(out), np.full(n, 5.0, np.float32))
        np.testing.assert_array_equal(hip.to_numpy(b), np.full(n, 1.0, np.float32))
        np.testing.assert_array_equal(hip.to_numpy(a), np.full(n, 2.0, np.float32))
    g.free()
    for x in (a, b, out):
        hip.mem_free(x)


def test_one_large_fill_and_its_tail(hip):
    n = (1 << 24) + 3
    buf = hip.mem_alloc(F32, n)
    hip.mem_fill(buf, 1.25)
    got = hip.to_numpy(buf)
    assert got[0] == 1.25 and got[-1] == 1.25 and np.all(got == 1.25)
    hip.mem_free(buf)


def test_an_accumulating_product_takes_over_a_waiting_zero_fill(hip):
    """ensure_grad(0) then `C += A B` (src/ndtensor.zig:221-228, :1092-1136): the product writes C instead of adding to
    zeros; any other fill value, a padded C or a refused product leaves the fill's effect in place."""
    from zigrad_amd._lib import ZgHipError

    r = np.random.default_rng(1)
    m, n, k = 96, 80, 64
    A = r.standard_normal((m, k), dtype=np.float32)
    B = r.standard_normal((k, n), dtype=np.float32)
    a, b = hip.from_numpy(A), hip.from_numpy(B)
    c = hip.from_numpy(np.full(m * n, np.nan, np.float32))
    prod = (A.astype(np.float64) @ B.astype(np.float64))

    def matmul(cbuf, ldc=n, lda=k, beta=1.0):
        hip.dispatch("matmul", A=a, B=b, C=cbuf, m=m, n=n, k=k, trans_a=False, trans_b=False, lda=lda, ldb=n, ldc=ldc,
                     alpha=1.0, beta=beta)

    hip.mem_fill(c, 0.0)
    matmul(c)
    got = hip.to_numpy(c).reshape(m, n)
    assert np.linalg.norm(got - prod) <= 1e-5 * np.linalg.norm(prod)
    matmul(c)  # nothing waiting now: a true accumulation
    assert np.linalg.norm(hip.to_numpy(c).reshape(m, n) - 2 * prod) <= 1e-5 * np.linalg.norm(2 * prod)
    hip.mem_fill(c, 1.0)  # not zero: stays a fill
    matmul(c)
    assert np.linalg.norm(hip.to_numpy(c).reshape(m, n) - (prod + 1.0)) <= 1e-5 * np.linalg.norm(prod + 1.0)
    hip.mem_fill(c, 0.0)  # batched form, one batch: the same rule
    hip.dispatch("bmm_acc", A=a, B=b, C=c, A_shape=[1, m, k], B_shape=[1, k, n], C_shape=[1, m, n], trans_a=False,
                 trans_b=False, lda=k, ldb=n, ldc=n, alpha=1.0, beta=1.0)
    assert np.linalg.norm(hip.to_numpy(c).reshape(m, n) - prod) <= 1e-5 * np.linalg.norm(prod)
    # a C with padding between rows: the fill covers the padding too and is launched as a fill
    wide = hip.from_numpy(np.full(m * (n + 8), np.nan, np.float32))
    hip.mem_fill(wide, 0.0)
    matmul(wide, ldc=n + 8)
    w = hip.to_numpy(wide).reshape(m, n + 8)
    assert np.linalg.norm(w[:, :n] - prod) <= 1e-5 * np.linalg.norm(prod) and np.all(w[:, n:] == 0.0)
    # a refused product (lda too small) after a zero fill: C holds the zeros
    hip.mem_transfer(np.full(m * n, np.nan, np.float32), c, "HtoD")
    hip.mem_fill(c, 0.0)
    with pytest.raises(ZgHipError):
        matmul(c, lda=k - 1)
    assert np.all(hip.to_numpy(c) == 0.0)
    for x in (a, b, c, wide):
        hip.mem_free(x)


def test_the_loss_backward_takes_over_a_waiting_zero_fill(oracle, hip):
    from conftest import run_op

    r = np.random.default_rng(2)
    rows, cols = 64, 10
    logits = r.standard_normal((rows, cols)).astype(np.float32)
    onehot = np.eye(cols, dtype=np.float32)[r.integers(0, cols, rows)]
    fw = run_op(oracle, "smce_fwd", {"logits": logits, "target": onehot, "probs": np.zeros_like(logits),
                                     "loss": np.zeros(1, np.float32), "rows": rows, "cols": cols}, ["probs"])
    probs = fw["probs"]
    want = run_op(oracle, "smce_bwd", {"probs": probs, "target": onehot, "grad": np.zeros_like(logits), "rows": rows,
                                       "cols": cols}, ["grad"])["grad"]
    p, t = hip.from_numpy(probs), hip.from_numpy(onehot)
    g = hip.from_numpy(np.full(rows * cols, np.nan, np.float32))
    hip.mem_fill(g, 0.0)
    hip.dispatch("smce_bwd", probs=p, target=t, grad=g, rows=rows, cols=cols)
    got = hip.to_numpy(g).reshape(rows, cols)
    assert np.array_equal(got, want)
    hip.dispatch("smce_bwd", probs=p, target=t, grad=g, rows=rows, cols=cols)  # now it accumulates
    assert np.array_equal(hip.to_numpy(g).reshape(rows, cols), want + want)
    for x in (p, t, g):
        hip.mem_free(x)


def test_a_waiting_fill_of_a_block_that_is_given_back_never_lands(hip):
    """The fill of a cache block that is freed while the fill still waits is dropped; whoever gets the block next must
    not see it arrive later.  Fills of other memory that waited beside it still happen."""
    n = 5000
    other = hip.mem_alloc(F32, 300)
    t = hip.mem_cache_alloc(F32, n)
    hip.mem_fill(t, 5.0)
    hip.mem_fill(other, 2.0)
    hip.mem_cache_free(t)
    u = hip.mem_cache_alloc(F32, n)              # the same block again, most likely
    data = np.arange(n, dtype=np.float32)
    hip.mem_transfer(data, u, "HtoD")
    hip.sync()
    assert np.array_equal(hip.to_numpy(u), data)
    assert np.all(hip.to_numpy(other) == 2.0)
    # a view into a live block is not the block: freeing the view's parent drops nothing that lies elsewhere
    v = hip.mem_cache_alloc(F32, n)
    hip.mem_fill(v.sub(0, 100), 9.0)
    hip.mem_fill(other, 3.0)
    hip.mem_cache_free(u)
    assert np.all(hip.to_numpy(v)[:100] == 9.0) and np.all(hip.to_numpy(other) == 3.0)
    hip.mem_cache_free(v)
    hip.mem_free(other)


def test_the_loss_backward_leaves_unrelated_fills_waiting_and_sees_related_ones(hip):
    rows, cols = 64, 10
    r = np.random.default_rng(2)
    p = r.random((rows, cols)).astype(np.float32)
    t = np.zeros((rows, cols), np.float32)
    t[np.arange(rows), r.integers(0, cols, rows)] = 1.0
    pb, tb = hip.from_numpy(p), hip.from_numpy(t)
    g = hip.mem_cache_alloc(F32, rows * cols)
    up = hip.mem_cache_alloc(F32, 1)
    hip.mem_fill(up, 1.0)                        # the upstream gradient: unrelated to the three operands
    hip.mem_fill(g, 0.0)
    hip.dispatch("smce_bwd", probs=pb, target=tb, grad=g, rows=rows, cols=cols)
    assert np.all(hip.to_numpy(up) == 1.0)       # still filled when somebody does read it
    want = ((p - t) / np.float32(rows)).astype(np.float32)
    assert np.array_equal(hip.to_numpy(g).reshape(rows, cols), want)
    # a fill of the probabilities that waits when the backward is asked for must be seen by it
    hip.mem_fill(pb, 0.5)
    hip.mem_fill(g, 0.0)
    hip.dispatch("smce_bwd", probs=pb, target=tb, grad=g, rows=rows, cols=cols)
    want = ((np.float32(0.5) - t) / np.float32(rows)).astype(np.float32)
    assert np.array_equal(hip.to_numpy(g).reshape(rows, cols), want)
    hip.mem_cache_free(g)
    hip.mem_cache_free(up)
    hip.mem_free(pb)
    hip.mem_free(tb)


def test_a_refused_call_still_owes_the_zeros_it_took_over(hip):
    """An op that takes over a waiting zero fill and is then refused (an argument error) must leave the zeros behind:
    the caller asked for them and the refused op wrote nothing."""
    from zigrad_amd._lib import ZgHipError

    m, n, k = 24, 16, 8
    a = hip.from_numpy(np.ones(m * k, np.float32))
    b = hip.from_numpy(np.ones(k * n, np.float32))
    c = hip.from_numpy(np.full(m * n, 7.0, np.float32))
    hip.mem_fill(c, 0.0)
    with pytest.raises(ZgHipError):      # lda smaller than k
        hip.dispatch("matmul", A=a, B=b, C=c, m=m, n=n, k=k, trans_a=False, trans_b=False, lda=k - 1, ldb=n, ldc=n,
                     alpha=1.0, beta=1.0)
    assert np.all(hip.to_numpy(c) == 0.0)
    # the graph-convolution aggregation and its backward
    n_nodes, stride, n_edge = 12, 4, 30
    r = np.random.default_rng(1)
    src = hip.from_numpy(r.integers(0, n_nodes, n_edge).astype(np.uint64))
    tgt = hip.from_numpy(r.integers(0, n_nodes, n_edge).astype(np.uint64))
    h = hip.from_numpy(r.standard_normal(n_nodes * stride).astype(np.float32))
    deg = hip.from_numpy(np.ones(n_nodes, np.float32))
    y = hip.from_numpy(np.full(n_nodes * stride, 3.0, np.float32))
    hip.mem_fill(y, 0.0)
    with pytest.raises(ZgHipError):      # no node features
        hip._call("zg_hip_scatter_gcn_deg_scaled", y.ptr, None, deg.ptr, src.ptr, tgt.ptr, stride, n_edge, n_nodes)
    assert np.all(hip.to_numpy(y) == 0.0)
    gh = hip.from_numpy(np.full(n_nodes * stride, 3.0, np.float32))
    gd = hip.from_numpy(np.full(n_nodes, 3.0, np.float32))
    hip.mem_fill(gh, 0.0)
    hip.mem_fill(gd, 0.0)
    with pytest.raises(ZgHipError):      # no upstream gradient
        hip._call("zg_hip_scatter_gcn_deg_scaled_bwd", None, h.ptr, deg.ptr, src.ptr, tgt.ptr, gh.ptr, gd.ptr, stride,
                  n_edge, n_nodes)
    assert np.all(hip.to_numpy(gh) == 0.0) and np.all(hip.to_numpy(gd) == 0.0)
    # the loss backward
    g = hip.from_numpy(np.full(40, 2.0, np.float32))
    p = hip.from_numpy(np.full(40, 0.1, np.float32))
    hip.mem_fill(g, 0.0)
    with pytest.raises(ZgHipError):      # no target
        hip._call("zg_hip_smce_bwd", p.ptr, None, g.ptr, 4, 10)
    assert np.all(hip.to_numpy(g) == 0.0)
    for t in (a, b, c, src, tgt, h, deg, y, gh, gd, g, p):
        hip.mem_free(t)


def test_a_refused_max_along_still_owes_the_fill_it_dropped(hip):
    """max_along overwrites its output without reading it, so a fill of the output that still waits is dropped
    (NDArray.max_along zero-fills first, src/ndarray.zig:567).  When the call is then refused after that point (more
    leading slices than a grid holds), nothing was overwritten and the fill must still land."""
    from zigrad_amd._lib import ZgHipError

    outer, R, inner = 70_000, 2, 3          # dim 1 of [70000, 2, 3]: 70000 leading slices exceed the grid's 65535
    x = hip.from_numpy(np.ones(outer * R * inner, np.float32))
    y = hip.from_numpy(np.full(outer * inner, 7.0, np.float32))
    hip.mem_fill(y, 0.5)
    with pytest.raises(ZgHipError):
        hip.dispatch("max_along", x=x, x_shape=[outer, R, inner], y=y, y_shape=[outer, inner], dim=1)
    assert np.all(hip.to_numpy(y) == 0.5)
    hip.mem_free(x)
    hip.mem_free(y)
