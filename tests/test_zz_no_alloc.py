"""The entry point that allocates nothing (zg_hip_smce_label_fwd_noalloc) against zg_hip_smce_label_fwd.

Both run the same kernels; the only difference is where the per-row loss terms and the partial sums live (a fixed
array in the library's device image instead of the context's workspace), so lse and loss must agree bit for bit.
Two calls in a row, the second on a smaller input: the array keeps the first call's contents, and nothing of
them may leak into the second result.  The oracle's value is checked as well (1e-5 on the loss).
"""
import numpy as np
import pytest

from conftest import run_op

pytestmark = pytest.mark.gpu


def _case(seed, rows, cols):
    rng = np.random.default_rng(seed)
    x = (rng.standard_normal((rows, cols)) * 3).astype(np.float32)
    lab = rng.integers(0, cols, rows).astype(np.uint64)
    return x, lab


def _run(dev, name, x, lab):
    rows, cols = x.shape
    out = run_op(dev, name, {"logits": x, "labels": lab, "lse": np.zeros(rows, np.float32),
                             "loss": np.zeros(1, np.float32), "rows": rows, "cols": cols}, ["lse", "loss"])
    return out["lse"], out["loss"]


# first call: more than 131072 rows, so the sum of the row terms takes the two-launch form and uses the partials
# part of the array; second call: few rows (single-launch sum) over stale contents
@pytest.mark.parametrize("shapes", [[(140001, 12), (300, 40)], [(4096, 1000), (17, 7)], [(262144, 8), (131073, 8)], [(70001, 24), (65537, 8)]])
def test_noalloc_matches_the_allocating_entry_point(hip, oracle, shapes):
    results = []
    for k, (rows, cols) in enumerate(shapes):
        x, lab = _case(100 + k, rows, cols)
        lse_a, loss_a = _run(hip, "smce_label_fwd", x, lab)
        lse_n, loss_n = _run(hip, "smce_label_fwd_noalloc", x, lab)
        assert np.array_equal(lse_a, lse_n), (rows, cols)
        assert np.array_equal(loss_a, loss_n), (rows, cols, loss_a, loss_n)
        results.append((x, lab, loss_n))
    # the oracle on the smaller case (seconds on the CPU)
    x, lab, loss_n = results[-1]
    if x.shape[0] <= 4096:
        _, loss_o = _run(oracle, "smce_label_fwd", x, lab)
        assert abs(float(loss_o[0]) - float(loss_n[0])) <= 1e-5 * max(1.0, abs(float(loss_o[0])))


def test_noalloc_rejects_more_rows_than_the_scratch_holds(hip):
    from zigrad_amd._lib import ZgHipError

    rows, cols = 262145, 4
    x = hip.from_numpy(np.zeros(rows * cols, np.float32))
    lab = hip.from_numpy(np.zeros(rows, np.uint64))
    lse = hip.from_numpy(np.zeros(rows, np.float32))
    loss = hip.from_numpy(np.zeros(1, np.float32))
    with pytest.raises(ZgHipError) as e:
        hip.dispatch("smce_label_fwd_noalloc", logits=x, labels=lab, lse=lse, loss=loss, rows=rows, cols=cols)
    assert e.value.code == 1 and "262144" in e.value.message
    for b in (x, lab, lse, loss):
        hip.mem_free(b)


def test_noalloc_makes_no_device_allocation(hip):
    """The library counts every hipMalloc it makes (workspace growth, pool segments, raw allocations): the
    allocation-free entry point must leave that counter where it was, on a context whose workspace is still empty."""
    from zigrad_amd import HipDevice

    dev = HipDevice(0)  # fresh context: no workspace yet
    try:
        rows, cols = 100000, 16
        x, lab = _case(7, rows, cols)
        bx, bl = dev.from_numpy(x), dev.from_numpy(lab)
        lse, loss = dev.from_numpy(np.zeros(rows, np.float32)), dev.from_numpy(np.zeros(1, np.float32))
        before = dev.cache_stats()["n_device_allocs"]
        dev.dispatch("smce_label_fwd_noalloc", logits=bx, labels=bl, lse=lse, loss=loss, rows=rows, cols=cols)
        dev.sync()
        assert dev.cache_stats()["n_device_allocs"] == before
        got = float(dev.to_numpy(loss)[0])
        m = x.astype(np.float64)
        lse64 = np.log(np.exp(m - m.max(1, keepdims=True)).sum(1)) + m.max(1)
        p_label = np.exp(m[np.arange(rows), lab.astype(np.int64)] - lse64)
        # the loss clamps the probability (src/nn/loss.zig:143), with fp32 bounds
        ref = np.mean(-np.log(np.clip(p_label, np.float32(1e-7), np.float32(1.0) - np.float32(1e-7))))
        assert abs(got - ref) <= 1e-5 * abs(ref)
        for b in (bx, bl, lse, loss):
            dev.mem_free(b)
    finally:
        dev.deinit()


def test_noalloc_launches_waiting_work_without_allocating():
    """A product whose k is cut over workgroups (its partial tiles live in the context's workspace) is queued and
    still waiting when the allocation-free entry point is called: the entry point launches it first.  The workspace
    the product needs was reserved by the call that queued it, so the allocation-free call makes no driver allocation
    (it reports one if it happens), and both results are right.  A context of its own: its workspace starts empty."""
    from zigrad_amd.device import F32, HipDevice

    dev = HipDevice(0)
    try:
        r = np.random.default_rng(5)
        m, n, k = 256, 1024, 16384          # eight large tiles: k is cut, tens of MB of partial tiles
        assert dev.gemm_plan(m, n, k, 1)["kind"] == "split_k"
        A = (r.standard_normal((m, k)) * 0.1).astype(np.float32)
        W = (r.standard_normal((n, k)) * 0.1).astype(np.float32)
        a, w = dev.from_numpy(A), dev.from_numpy(W)
        c = dev.mem_alloc(F32, m * n)
        rows, cols = 3000, 50
        x, lab = _case(7, rows, cols)
        xb, lb = dev.from_numpy(x.ravel()), dev.from_numpy(lab)
        lse, loss = dev.mem_alloc(F32, rows), dev.mem_alloc(F32, 1)
        dev.sync()
        before = dev.cache_stats()["n_device_allocs"]
        dev.dispatch("matmul", A=a, B=w, C=c, m=m, n=n, k=k, trans_a=False, trans_b=True, lda=k, ldb=k, ldc=n, alpha=1.0,
                     beta=0.0)                                  # a layer's forward product: waits for its bias add
        queued = dev.cache_stats()["n_device_allocs"]           # a host counter: the product keeps waiting
        dev.dispatch("smce_label_fwd_noalloc", logits=xb, labels=lb, lse=lse, loss=loss, rows=rows, cols=cols)
        after = dev.cache_stats()["n_device_allocs"]
        got = dev.to_numpy(c).reshape(m, n)
        want = A.astype(np.float64) @ W.astype(np.float64).T
        assert np.linalg.norm(got - want) <= 1e-5 * np.linalg.norm(want)
        x64 = x.astype(np.float64)
        lse64 = np.log(np.exp(x64 - x64.max(axis=1, keepdims=True)).sum(axis=1)) + x64.max(axis=1)
        assert np.allclose(dev.to_numpy(lse), lse64, rtol=1e-6, atol=1e-6)
        # the product's workspace was allocated by the matmul call (one growth), nothing by the allocation-free call
        # although it is the one that launched the product
        assert queued - before == 1
        assert after == queued
        for b in (a, w, c, xb, lb, lse, loss):
            dev.mem_free(b)
    finally:
        dev.deinit()
