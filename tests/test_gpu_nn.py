"""Losses, optimizers and indexing ops of the HIP device against the CPU oracle, through the C ABI."""
from __future__ import annotations

import numpy as np
import pytest
from scipy.special import logsumexp, softmax

from conftest import rel_fro, run_op
from zigrad_amd.device import F32

pytestmark = pytest.mark.gpu
TOL = 1e-5


def rng(seed):
    return np.random.default_rng(seed)


def both(oracle, hip, name, params, outputs):
    a = run_op(oracle, name, {k: (v.copy() if isinstance(v, np.ndarray) else v) for k, v in params.items()}, outputs)
    b = run_op(hip, name, params, outputs)
    return a, b


# ----------------------------------------------------------------------------------------------
# softmax / cross-entropy
# ----------------------------------------------------------------------------------------------
def _smce_fwd_hip(hip, x, t):
    rows, cols = x.shape
    xb, tb = hip.from_numpy(x), hip.from_numpy(t)
    pb, lb = hip.mem_alloc(F32, rows * cols), hip.mem_alloc(F32, 1)
    hip.dispatch("smce_fwd", logits=xb, target=tb, probs=pb, loss=lb, rows=rows, cols=cols)
    out = hip.to_numpy(pb).reshape(rows, cols), float(hip.to_numpy(lb)[0])
    for b in (xb, tb, pb, lb):
        hip.mem_free(b)
    return out


@pytest.mark.parametrize("rows,cols", [(64, 10), (256, 32), (140, 7), (64, 200), (16, 3000), (1, 4), (255, 2),
                                       # rows that a larger batch holds in registers: 4, 16 and 64 lanes per row
                                       (200, 8), (50, 28), (64, 256), (16, 260), (16, 1000), (3, 1024), (9, 36),
                                       # more than 1024 columns: the small batch takes the row kernels as well
                                       (16, 2048), (5, 4096), (7, 1030)])
def test_smce_fwd_small_batches_equal_the_two_launch_path(hip, rows, cols):
    """A batch that fits one workgroup takes one launch (rows and their mean); the same rows inside a batch too large
    for it take the row kernel and the reduction.  Per row the probabilities must be the same bits; the mean is held to
    the float64 closed form."""
    r = rng(rows + 31 * cols)
    x = (r.standard_normal((rows, cols)) * 3).astype(np.float32)
    t = np.zeros((rows, cols), np.float32)
    t[np.arange(rows), r.integers(0, cols, rows)] = 1.0
    p_small, loss_small = _smce_fwd_hip(hip, x, t)
    big = 1200 // rows + 2
    p_big, _ = _smce_fwd_hip(hip, np.tile(x, (big, 1)), np.tile(t, (big, 1)))
    np.testing.assert_array_equal(p_small, p_big[:rows])
    x64 = x.astype(np.float64)
    p_lab = np.exp((x64 * t).sum(axis=1) - logsumexp(x64, axis=1))
    want = float(np.mean(-np.log(np.clip(p_lab, np.float32(1e-7), np.float32(1.0) - np.float32(1e-7)))))
    assert abs(loss_small - want) <= 1e-5 * max(1.0, abs(want))


SMCE_SHAPES = [(1, 4), (64, 10), (140, 7), (64, 2), (4096, 1024), (33, 1001), (17, 32000), (300, 257), (5, 70001), (9, 4100),
               # rows held in registers by 4, 16 or 64 lanes, by a workgroup of 256 threads (4 or 8 pieces each) or of 1024
               (3000, 8), (3000, 32), (700, 36), (1500, 256), (40, 260), (300, 1024), (40, 1028), (21, 2048), (9, 4096),
               (7, 5000), (6, 8192), (5, 8196), (3, 20000), (2, 32768),
               # rows that start off a 16-byte boundary: heads and tails of one to three values, pieces that hold the end
               # of one row and the start of the next, rows too long for the registers
               (1000, 5), (999, 6), (501, 11), (40, 4099), (7, 33001), (3, 70002), (2, 131072), (2000, 3), (5000, 1),
               # a handful of very long rows, cut into segments: whole segments, a short last one, segments that start
               # off the 16-byte grid, a single row
               (40, 65536), (3, 200003), (1, 1000001), (255, 65540)]


@pytest.mark.parametrize("rows,cols", SMCE_SHAPES)
def test_smce_onehot_and_label(oracle, hip, rows, cols):
    r = rng(rows * 7 + cols)
    x = (r.standard_normal((rows, cols)) * 3).astype(np.float32)
    lab = r.integers(0, cols, rows).astype(np.uint64)
    t = np.zeros((rows, cols), np.float32)
    t[np.arange(rows), lab] = 1.0
    one = np.zeros(1, np.float32)
    a, b = both(oracle, hip, "smce_fwd", {"logits": x, "target": t, "probs": np.zeros_like(x), "loss": one, "rows": rows,
                                          "cols": cols}, ["probs", "loss"])
    x64 = x.astype(np.float64)
    sm = softmax(x64, axis=1)
    # the loss clamps the label's probability to [1e-7, 1 - 1e-7] (src/nn/loss.zig:143)
    p_lab = np.exp(x64[np.arange(rows), lab] - logsumexp(x64, axis=1))
    loss = float(np.mean(-np.log(np.clip(p_lab, np.float32(1e-7), np.float32(1.0) - np.float32(1e-7)))))
    # The host loop adds the exponentials of a row one after the other in fp32; for rows of tens of thousands
    # of columns that alone drifts past 1e-5 from the exact value.  The device result is held to 1e-5 against
    # fp64; the oracle is held to 1e-5 where its own summation error allows it, to 2e-4 up to rows of 70002 columns
    # to 1e-3 up to 200003 (3.3e-4 measured on rows of 131072) and to 5e-3 beyond (1.7e-3 on a row of 1000001).
    oracle_tol = TOL if cols <= 4096 else 2e-4 if cols <= 70002 else 1e-3 if cols <= 200003 else 5e-3
    assert rel_fro(b["probs"], sm) <= TOL and rel_fro(a["probs"], sm) <= oracle_tol
    assert rel_fro(b["probs"], a["probs"]) <= max(TOL, 1.1 * rel_fro(a["probs"], sm) + 1e-6)
    assert abs(b["loss"][0] - loss) <= 1e-5 * max(1.0, abs(loss))
    assert abs(b["loss"][0] - a["loss"][0]) <= oracle_tol * max(1.0, abs(loss))
    g0 = (r.standard_normal((rows, cols)) * 0.01).astype(np.float32)
    ga, gb = both(oracle, hip, "smce_bwd", {"probs": b["probs"], "target": t, "grad": g0, "rows": rows, "cols": cols}, ["grad"])
    np.testing.assert_array_equal(ga["grad"], gb["grad"])  # pure sub/div/add on identical inputs
    # integer labels
    a2, b2 = both(oracle, hip, "smce_label_fwd", {"logits": x, "labels": lab, "lse": np.zeros(rows, np.float32), "loss": one,
                                                  "rows": rows, "cols": cols}, ["lse", "loss"])
    assert rel_fro(b2["lse"], logsumexp(x64, axis=1)) <= 1e-6
    assert abs(b2["loss"][0] - loss) <= 1e-5 * max(1.0, abs(loss))
    assert abs(b2["loss"][0] - a2["loss"][0]) <= oracle_tol * max(1.0, abs(loss))
    want = g0 + (sm - t) / rows
    for acc in (True, False):
        g = run_op(hip, "smce_label_bwd", {"logits": x, "labels": lab, "lse": b2["lse"], "grad": g0.copy(), "rows": rows,
                                           "cols": cols, "accumulate": acc}, ["grad"])["grad"]
        assert rel_fro(g, want if acc else (sm - t) / rows) <= TOL
        # every row of the un-accumulated gradient sums to zero
        if not acc:
            assert np.abs(g.astype(np.float64).sum(axis=1)).max() <= 1e-6
    go = run_op(oracle, "smce_label_bwd", {"logits": x, "labels": lab, "lse": a2["lse"], "grad": g0.copy(), "rows": rows,
                                           "cols": cols}, ["grad"])["grad"]
    assert rel_fro(go, want) <= oracle_tol


@pytest.mark.parametrize("rows,cols", [(5, 5), (70, 10), (40, 130), (9, 1001), (3, 4099), (2000, 7)])
def test_rows_that_begin_with_minus_infinity(oracle, hip, rows, cols):
    """Masked logits: -inf in the first columns (and elsewhere) of rows that are read value by value or in pieces with a
    head.  The running maximum must not form exp(-inf - -inf) before it has seen a finite value."""
    r = rng(rows * 3 + cols)
    x = (r.standard_normal((rows, cols)) * 2).astype(np.float32)
    x[:, 0] = -np.inf
    x[::2, 1] = -np.inf
    x[1::3, cols - 1] = -np.inf
    lab = np.full(rows, 2, np.uint64)
    t = np.zeros((rows, cols), np.float32)
    t[:, 2] = 1.0
    one = np.zeros(1, np.float32)
    sm = softmax(x.astype(np.float64), axis=1)
    a, b = both(oracle, hip, "smce_fwd", {"logits": x, "target": t, "probs": np.zeros_like(x), "loss": one, "rows": rows,
                                          "cols": cols}, ["probs", "loss"])
    assert np.isfinite(b["probs"]).all() and np.isfinite(b["loss"]).all()
    assert rel_fro(b["probs"], sm) <= TOL and rel_fro(a["probs"], sm) <= TOL
    assert abs(b["loss"][0] - a["loss"][0]) <= TOL * max(1.0, abs(a["loss"][0]))
    a, b = both(oracle, hip, "softmax_fwd", {"x": x, "y": np.zeros_like(x), "rows": rows, "cols": cols}, ["y"])
    assert rel_fro(b["y"], sm) <= TOL
    a2, b2 = both(oracle, hip, "smce_label_fwd", {"logits": x, "labels": lab, "lse": np.zeros(rows, np.float32), "loss": one,
                                                  "rows": rows, "cols": cols}, ["lse", "loss"])
    assert rel_fro(b2["lse"], logsumexp(x.astype(np.float64), axis=1)) <= 1e-6
    assert abs(b2["loss"][0] - a2["loss"][0]) <= TOL * max(1.0, abs(a2["loss"][0]))


def test_smce_clamp_edge(oracle, hip):
    """A vanishing probability is clamped to 1e-7 in the loss only (src/nn/loss.zig:143)."""
    x = np.asarray([[100.0, 0.0, 0.0], [0.0, 0.0, 50.0]], np.float32)
    lab = np.asarray([1, 0], np.uint64)
    t = np.zeros((2, 3), np.float32)
    t[[0, 1], [1, 0]] = 1
    one = np.zeros(1, np.float32)
    a, b = both(oracle, hip, "smce_fwd", {"logits": x, "target": t, "probs": np.zeros_like(x), "loss": one, "rows": 2, "cols": 3},
                ["loss"])
    want = -np.log(np.float32(1e-7))
    assert abs(b["loss"][0] - want) <= 1e-5 * want and abs(a["loss"][0] - want) <= 1e-5 * want
    a, b = both(oracle, hip, "smce_label_fwd", {"logits": x, "labels": lab, "lse": np.zeros(2, np.float32), "loss": one,
                                                "rows": 2, "cols": 3}, ["loss"])
    assert abs(b["loss"][0] - want) <= 1e-5 * want and abs(a["loss"][0] - want) <= 1e-5 * want


@pytest.mark.parametrize("rows,cols", [(64, 10), (5, 3000), (1, 7), (3, 8192), (2, 32768), (2, 32772),
                                       # every shape of the kernels that hold a row in registers, and rows beside them
                                       (1000, 4), (700, 32), (300, 36), (1500, 256), (70, 260), (300, 1024), (33, 1028),
                                       (21, 4096), (9, 4100), (5, 8196), (3, 32764), (70, 1030), (500, 30),
                                       # rows that start off a 16-byte boundary, rows too long for the registers
                                       (999, 6), (501, 11), (40, 4099), (7, 33001), (3, 70002), (2000, 3),
                                       # a handful of very long rows, cut into segments
                                       (40, 65536), (3, 200003), (1, 1000001)])
def test_softmax_fwd_bwd(oracle, hip, rows, cols):
    r = rng(rows + cols)
    x = r.standard_normal((rows, cols)).astype(np.float32)
    a, b = both(oracle, hip, "softmax_fwd", {"x": x, "y": np.zeros_like(x), "rows": rows, "cols": cols}, ["y"])
    assert rel_fro(b["y"], softmax(x.astype(np.float64), axis=1)) <= TOL
    yg = r.standard_normal((rows, cols)).astype(np.float32)
    g0 = r.standard_normal((rows, cols)).astype(np.float32)
    a, b = both(oracle, hip, "softmax_bwd", {"y": b["y"], "y_g": yg, "x_g": g0, "rows": rows, "cols": cols}, ["x_g"])
    assert rel_fro(b["x_g"], a["x_g"]) <= TOL


@pytest.mark.parametrize("n", [6, 64, 100001])
def test_smooth_l1_and_mse(oracle, hip, n):
    r = rng(n)
    p, t = r.standard_normal(n).astype(np.float32) * 2, r.standard_normal(n).astype(np.float32)
    one = np.zeros(1, np.float32)
    g0 = r.standard_normal(n).astype(np.float32)
    # the host loops add n terms one after the other in fp32; both sides are held against the fp64 value, the
    # device (tree sum) to 1e-5 and the oracle to what a sequential fp32 sum of n terms allows
    d64 = p.astype(np.float64) - t
    sl1 = np.where(np.abs(d64) < 1.0, 0.5 * d64 * d64, np.abs(d64) - 0.5).mean()
    seq_tol = max(1e-5, 2e-9 * n)
    a, b = both(oracle, hip, "smooth_l1_fwd", {"pred": p, "target": t, "beta": 1.0, "loss": one}, ["loss"])
    assert abs(b["loss"][0] - sl1) <= 1e-5 * sl1 and abs(a["loss"][0] - sl1) <= seq_tol * sl1
    a, b = both(oracle, hip, "smooth_l1_bwd", {"pred": p, "target": t, "grad": g0, "beta": 1.0}, ["grad"])
    np.testing.assert_array_equal(a["grad"], b["grad"])
    a, b = both(oracle, hip, "mse_fwd", {"pred": p, "target": t, "loss": one}, ["loss"])
    mse = (d64 * d64).mean()
    assert abs(b["loss"][0] - mse) <= 1e-5 * mse and abs(a["loss"][0] - mse) <= seq_tol * mse
    a, b = both(oracle, hip, "mse_bwd", {"pred": p, "target": t, "grad": g0}, ["grad"])
    np.testing.assert_array_equal(a["grad"], b["grad"])


# ----------------------------------------------------------------------------------------------
# optimizers
# ----------------------------------------------------------------------------------------------
@pytest.mark.parametrize("n", [10, 640, 8192, 100352, (1 << 21) + 3])
@pytest.mark.parametrize("clip", [False, True])
def test_sgd_and_adam_steps(oracle, hip, n, clip):
    r = rng(n + clip)
    p0 = r.standard_normal(n).astype(np.float32)
    # with clip on, one gradient is large enough to be clipped (norm > 10) and one is not
    for gscale in ((5.0, 1e-3) if clip else (1.0,)):
        g0 = (r.standard_normal(n) * gscale).astype(np.float32)
        a, b = both(oracle, hip, "sgd_step", {"param": p0, "grad": g0, "lr": 0.01, "clip": clip, "max_norm": 10.0, "delta": 1e-6},
                    ["param", "grad"])
        if clip:
            assert rel_fro(b["param"], a["param"]) <= 1e-6 and rel_fro(b["grad"], a["grad"]) <= 1e-6
        else:
            np.testing.assert_array_equal(a["param"], b["param"])
            np.testing.assert_array_equal(a["grad"], b["grad"])
        # Adam: two consecutive steps with the per-tensor counter t
        state = {}
        for name, dev in (("o", oracle), ("h", hip)):
            P, G, M, V = (dev.from_numpy(x) for x in (p0, g0, np.zeros(n, np.float32), np.zeros(n, np.float32)))
            for t in (1, 2):
                dev.dispatch("adam_step", param=P, grad=G, m=M, v=V, t=t, lr=1e-3, beta1=0.9, beta2=0.999, epsilon=1e-8,
                             clip=clip, max_norm=10.0, delta=1e-6)
            dev.sync()
            state[name] = [dev.to_numpy(x) for x in (P, G, M, V)]
        for xo, xh in zip(state["o"], state["h"]):
            if clip:
                assert rel_fro(xh, xo) <= 1e-6
            else:
                np.testing.assert_array_equal(xo, xh)


def test_adam_closed_form(hip):
    """Two hand-traced steps: t increments per update, lr_t in fp32 (src/nn/optim.zig:189-191, 226-229)."""
    p, g = np.asarray([1.0, -2.0], np.float32), np.asarray([0.5, -0.25], np.float32)
    P, G, M, V = (hip.from_numpy(x) for x in (p, g, np.zeros(2, np.float32), np.zeros(2, np.float32)))
    m = v = np.zeros(2)
    want = p.astype(np.float64)
    for t in (1, 2):
        hip.dispatch("adam_step", param=P, grad=G, m=M, v=V, t=t, lr=0.01, beta1=0.9, beta2=0.999, epsilon=1e-8, clip=False,
                     max_norm=10.0, delta=1e-6)
        m = 0.9 * m + 0.1 * g
        v = 0.999 * v + 0.001 * g * g
        lr_t = 0.01 * np.sqrt(1 - 0.999 ** t) / (1 - 0.9 ** t)
        want = want - lr_t * m / (np.sqrt(v) + 1e-8)
    np.testing.assert_allclose(hip.to_numpy(P), want, rtol=1e-5)


# ----------------------------------------------------------------------------------------------
# indexing: gather offsets, scatter_add, index_select, GCN scatter
# ----------------------------------------------------------------------------------------------
def test_gather_offsets_bit_exact(oracle, hip):
    r = rng(1)
    for src_shape, idx_shape, dim in [([64, 2], [64, 1], 1), ([5, 6, 7], [5, 4, 7], 1), ([5, 6, 7], [3, 6, 2], 0), ([9], [4], 0)]:
        n = int(np.prod(idx_shape))
        idx = r.integers(0, src_shape[dim], n).astype(np.uint64)
        res = []
        for dev in (oracle, hip):
            I, O = dev.from_numpy(idx), dev.from_numpy(np.zeros(n, np.uint64))
            assert dev.gather_offsets(src_shape, idx_shape, I, dim, O) == 0
            dev.sync()
            res.append(dev.to_numpy(O))
        np.testing.assert_array_equal(res[0], res[1])
        # brute force: numpy take_along_axis over a tensor of flat positions
        pos = np.arange(int(np.prod(src_shape))).reshape(src_shape)
        sl = tuple(slice(0, s) for s in idx_shape)
        want = np.take_along_axis(pos[tuple(s if i != dim else slice(None) for i, s in enumerate(sl))],
                                  idx.reshape(idx_shape).astype(np.int64), axis=dim)
        np.testing.assert_array_equal(res[1], want.ravel().astype(np.uint64))


def test_gather_in_one_launch_equals_offsets_then_take(oracle, hip):
    """zg_hip_gather against gather_offsets + mem_take on the device and against the oracle's host loops, bit for bit;
    an index beyond the source's dim is reported when the status is asked for."""
    from zigrad_amd.device import F32, U64

    r = rng(2)
    for src_shape, idx_shape, dim in [([64, 2], [64, 1], 1), ([5, 6, 7], [5, 4, 7], 1), ([5, 6, 7], [3, 6, 2], 0), ([9], [4], 0),
                                       ([300, 40], [300, 40], 1)]:
        n = int(np.prod(idx_shape))
        idx = r.integers(0, src_shape[dim], n).astype(np.uint64)
        src = r.standard_normal(int(np.prod(src_shape))).astype(np.float32)
        res = []
        for dev in (oracle, hip):
            S, I = dev.from_numpy(src), dev.from_numpy(idx)
            O, D = dev.from_numpy(np.zeros(n, np.uint64)), dev.from_numpy(np.full(n, np.nan, np.float32))
            assert dev.gather(S, src_shape, idx_shape, I, dim, O, D, check=(n % 2 == 0)) == 0
            dev.sync()
            res.append((dev.to_numpy(O), dev.to_numpy(D)))
        O2, D2 = hip.from_numpy(np.zeros(n, np.uint64)), hip.from_numpy(np.full(n, np.nan, np.float32))
        S, I = hip.from_numpy(src), hip.from_numpy(idx)
        assert hip.gather_offsets(src_shape, idx_shape, I, dim, O2) == 0
        hip.mem_take(S, O2, D2)
        hip.sync()
        np.testing.assert_array_equal(res[1][0], hip.to_numpy(O2))
        np.testing.assert_array_equal(res[1][1], hip.to_numpy(D2))
        np.testing.assert_array_equal(res[0][0], res[1][0])
        np.testing.assert_array_equal(res[0][1], res[1][1])
        want = np.take_along_axis(src.reshape(src_shape)[tuple(slice(0, s) if i != dim else slice(None) for i, s in enumerate(idx_shape))],
                                  idx.reshape(idx_shape).astype(np.int64), axis=dim)
        np.testing.assert_array_equal(res[1][1], want.ravel())
    bad = np.array([0, 1, 7, 1], np.uint64)  # 7 >= 2
    S, I = hip.from_numpy(np.arange(8, dtype=np.float32)), hip.from_numpy(bad)
    O, D = hip.from_numpy(np.zeros(4, np.uint64)), hip.from_numpy(np.zeros(4, np.float32))
    assert hip.gather(S, [4, 2], [4, 1], I, 1, O, D, check=True) == 2
    assert hip.gather(S, [4, 2], [4, 1], I, 1, O, D, check=False) == 0  # unchecked: the bad entry is skipped silently
    hip.sync()


@pytest.mark.parametrize("n,dst_len", [(64, 128), (13264, 2708), (100000, 17), (5000, 300000), (1, 1), (40000, 5000),
                                        (256, 7), (257, 7), (200, 1), (255, 1000)])
def test_scatter_add_bit_exact(oracle, hip, n, dst_len):
    """Order of accumulation per destination equals the host loop's, so the floats agree bit for bit."""
    r = rng(n + dst_len)
    src = r.standard_normal(n).astype(np.float32)
    off = r.integers(0, dst_len, n).astype(np.uint64)
    if n > 100:
        off[: n // 4] = np.sort(off[: n // 4])  # runs of consecutive / repeated offsets
    dst0 = r.standard_normal(dst_len).astype(np.float32)
    a, b = both(oracle, hip, "scatter_add", {"src": src, "offsets": off, "dst": dst0}, ["dst"])
    np.testing.assert_array_equal(a["dst"], b["dst"])
    # invariant: total mass is conserved
    assert abs(b["dst"].astype(np.float64).sum() - (dst0.astype(np.float64).sum() + src.astype(np.float64).sum())) <= 1e-3 * (1 + np.abs(src).sum())


def test_scatter_add_heavy_hitter_is_deterministic(hip):
    r = rng(6)
    n = 200000
    src = r.standard_normal(n).astype(np.float32)
    off = np.where(r.random(n) < 0.5, 3, r.integers(0, 1000, n)).astype(np.uint64)
    outs = [run_op(hip, "scatter_add", {"src": src, "offsets": off, "dst": np.zeros(1000, np.float32)}, ["dst"])["dst"]
            for _ in range(3)]
    np.testing.assert_array_equal(outs[0], outs[1])
    np.testing.assert_array_equal(outs[0], outs[2])
    want = np.zeros(1000, np.float32)
    for i in range(n):
        want[off[i]] += src[i]
    np.testing.assert_array_equal(outs[0], want)


@pytest.mark.parametrize("rows,stride,n_idx", [(100, 16, 37), (2708, 7, 5000), (50, 300, 200), (10, 1, 10),
                                               # long rows, cut into spans of columns: whole spans, a partial last one,
                                               # a row length that is no multiple of four
                                               (9, 8192, 20), (7, 9220, 11), (5, 70000, 8), (6, 8195, 9)])
def test_index_select(oracle, hip, rows, stride, n_idx):
    r = rng(rows + stride)
    src = r.standard_normal(rows * stride).astype(np.float32)
    idx = r.integers(0, rows, n_idx).astype(np.uint64)
    a, b = both(oracle, hip, "index_select_fwd", {"src": src, "indices": idx, "stride": stride,
                                                  "dst": np.zeros(n_idx * stride, np.float32)}, ["dst"])
    np.testing.assert_array_equal(a["dst"], b["dst"])
    np.testing.assert_array_equal(b["dst"], src.reshape(rows, stride)[idx.astype(np.int64)].ravel())
    yg = r.standard_normal(n_idx * stride).astype(np.float32)
    xg = r.standard_normal(rows * stride).astype(np.float32)
    a, b = both(oracle, hip, "index_select_bwd", {"y_grad": yg, "indices": idx, "stride": stride, "x_grad": xg}, ["x_grad"])
    np.testing.assert_array_equal(a["x_grad"], b["x_grad"])


def random_graph(r, n_nodes, n_pairs):
    """Symmetrised random pairs plus self loops, [2, E] layout (src row then tgt row)."""
    u, v = r.integers(0, n_nodes, n_pairs), r.integers(0, n_nodes, n_pairs)
    loops = np.arange(n_nodes)
    src = np.concatenate([u, v, loops]).astype(np.uint64)
    tgt = np.concatenate([v, u, loops]).astype(np.uint64)
    return src, tgt


@pytest.mark.parametrize("n_nodes,n_pairs,stride", [(2708, 5278, 16), (2708, 5278, 7), (50, 400, 3), (300, 100, 70), (10, 0, 4)])
def test_scatter_gcn_fwd_bwd_bit_exact(oracle, hip, n_nodes, n_pairs, stride):
    r = rng(n_nodes + stride)
    src, tgt = random_graph(r, n_nodes, n_pairs)
    E = src.size
    h = r.standard_normal(n_nodes * stride).astype(np.float32)
    indeg = np.bincount(tgt.astype(np.int64), minlength=n_nodes).astype(np.float32)
    deg = (1.0 / np.sqrt(1.0 + indeg)).astype(np.float32)
    dst0 = np.zeros(n_nodes * stride, np.float32)
    a, b = both(oracle, hip, "scatter_gcn_deg_scaled", {"dst": dst0, "h": h, "deg": deg, "src_indices": src, "tgt_indices": tgt,
                                                        "stride": stride, "n_edge": E}, ["dst"])
    np.testing.assert_array_equal(a["dst"], b["dst"])
    # textbook cross-check: dense D^-1/2 A D^-1/2 H
    Aw = np.zeros((n_nodes, n_nodes))
    np.add.at(Aw, (tgt.astype(np.int64), src.astype(np.int64)), 1.0)
    dense = (deg[:, None].astype(np.float64) * Aw * deg[None, :].astype(np.float64)) @ h.reshape(n_nodes, stride).astype(np.float64)
    assert rel_fro(b["dst"], dense.ravel()) <= TOL
    go = r.standard_normal(n_nodes * stride).astype(np.float32)
    gh0 = r.standard_normal(n_nodes * stride).astype(np.float32)
    gd0 = r.standard_normal(n_nodes).astype(np.float32)
    a, b = both(oracle, hip, "scatter_gcn_deg_scaled_bwd", {"grad_output": go, "h": h, "deg": deg, "src_indices": src,
                                                            "tgt_indices": tgt, "grad_h": gh0, "grad_deg": gd0, "stride": stride,
                                                            "n_edge": E}, ["grad_h", "grad_deg"])
    np.testing.assert_array_equal(a["grad_h"], b["grad_h"])
    np.testing.assert_array_equal(a["grad_deg"], b["grad_deg"])


def test_scatter_gcn_indices_in_pinned_host_memory(oracle, hip):
    """The reference hands the device op index slices that live in host memory (examples/gcn/src/model.zig:204-205)."""
    r = rng(21)
    n_nodes, stride = 200, 16
    src, tgt = random_graph(r, n_nodes, 600)
    h = r.standard_normal(n_nodes * stride).astype(np.float32)
    deg = (r.random(n_nodes) + 0.5).astype(np.float32)
    want = run_op(oracle, "scatter_gcn_deg_scaled", {"dst": np.zeros(n_nodes * stride, np.float32), "h": h, "deg": deg,
                                                     "src_indices": src, "tgt_indices": tgt, "stride": stride, "n_edge": src.size},
                  ["dst"])["dst"]
    S, T = hip.mem_alloc_host(np.uint64, src.size), hip.mem_alloc_host(np.uint64, tgt.size)
    hip.mem_transfer(src, S, "HtoD")
    hip.mem_transfer(tgt, T, "HtoD")
    D, H, G = hip.from_numpy(np.zeros(n_nodes * stride, np.float32)), hip.from_numpy(h), hip.from_numpy(deg)
    hip.dispatch("scatter_gcn_deg_scaled", dst=D, h=H, deg=G, src_indices=S, tgt_indices=T, stride=stride, n_edge=src.size)
    hip.sync()
    np.testing.assert_array_equal(hip.to_numpy(D), want)


def test_smce_soft_targets_on_long_rows(oracle, hip):
    """Dense (not one-hot) targets: every column contributes a loss term; rows long enough for the register-cached kernel."""
    rows, cols = 6, 8192
    r = rng(77)
    x = (r.standard_normal((rows, cols)) * 2).astype(np.float32)
    t = softmax(r.standard_normal((rows, cols)), axis=1).astype(np.float32)
    one = np.zeros(1, np.float32)
    a, b = both(oracle, hip, "smce_fwd", {"logits": x, "target": t, "probs": np.zeros_like(x), "loss": one, "rows": rows,
                                          "cols": cols}, ["probs", "loss"])
    x64 = x.astype(np.float64)
    logp = x64 - logsumexp(x64, axis=1, keepdims=True)
    want = float(-(t.astype(np.float64) * np.log(np.clip(np.exp(logp), 1e-7, 1 - 1e-7))).sum() / rows)
    assert abs(b["loss"][0] - want) <= 1e-5 * want
    assert abs(a["loss"][0] - want) <= 1e-4 * want
    assert rel_fro(b["probs"], softmax(x64, axis=1)) <= TOL
