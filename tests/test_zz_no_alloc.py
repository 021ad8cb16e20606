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


# first call: more than 65536 rows, so the sum of the row terms takes the two-launch form and uses the partials
# part of the array; second call: few rows (single-launch sum) over stale contents
@pytest.mark.parametrize("shapes", [[(70001, 24), (300, 40)], [(4096, 1000), (17, 7)], [(262144, 8), (65537, 8)]])
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
