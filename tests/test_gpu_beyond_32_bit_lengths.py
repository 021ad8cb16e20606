"""Arrays of more than 2^32 elements (17 GB each; the device has 288 GB): element indices, byte offsets and grid sizes
must not wrap at 32 bits anywhere on the way.  Operands are made on the device (mem_sequence, mem_fill) and read back
at a few places either side of 2^24, 2^31 and 2^32 and at both ends; reductions are checked against their closed forms.
The reference's loops index with usize throughout (src/device/host_device.zig), so these are the sizes its interface
allows; ops whose interface here is limited to 2^32 - 1 entries say so in the header and are not called."""
from __future__ import annotations

import numpy as np
import pytest

from zigrad_amd.device import F32, U64

pytestmark = pytest.mark.gpu

N = (1 << 32) + 4099
POINTS = [0, 1, 4095, 1 << 24, (1 << 31) - 3, (1 << 31) + 5, (1 << 32) - 2, 1 << 32, N - 1]


def _at(hip, buf, points=POINTS):
    return np.array([hip.to_numpy(buf.sub(p, 1))[0] for p in points], np.float32)


def _index_as_f32(points=POINTS):
    return np.array(points, np.float64).astype(np.float32)      # what mem_sequence(0, 1) holds there


def test_elementwise_ops_copies_and_updates_over_more_than_2_32_elements(hip):
    x, y, z = (hip.mem_alloc(F32, N) for _ in range(3))
    try:
        hip.mem_sequence(x, 0.0, 1.0)
        hip.mem_fill(y, 2.0)
        np.testing.assert_array_equal(_at(hip, x), _index_as_f32())
        np.testing.assert_array_equal(_at(hip, y), np.full(len(POINTS), 2.0, np.float32))
        hip.dispatch("add", x=x, y=y, z=z)
        np.testing.assert_array_equal(_at(hip, z), _index_as_f32() + np.float32(2.0))
        hip.dispatch("mul", x=y, y=y, z=z)
        np.testing.assert_array_equal(_at(hip, z), np.full(len(POINTS), 4.0, np.float32))
        hip.dispatch("relu_fwd", x=y, y=z)
        hip.dispatch("scale", x=z, alpha=0.5)
        np.testing.assert_array_equal(_at(hip, z), np.full(len(POINTS), 1.0, np.float32))
        hip.dispatch("relu_bwd", x=y, x_g=z, y_g=y)             # x_g += y_g where x > 0: 1 + 2
        np.testing.assert_array_equal(_at(hip, z), np.full(len(POINTS), 3.0, np.float32))
        one = hip.from_numpy(np.full(1, 3.0, np.float32))
        hip.dispatch("add", x=one, y=y, z=z)                    # the one-float operand in device memory
        np.testing.assert_array_equal(_at(hip, z), np.full(len(POINTS), 5.0, np.float32))
        hip.dispatch("mul", x=y, y=0.25, z=z)                   # and by value
        np.testing.assert_array_equal(_at(hip, z), np.full(len(POINTS), 0.5, np.float32))
        row = hip.from_numpy(np.arange(4099 + 1, dtype=np.float32))   # the shorter operand restarts every 4100 elements
        n_rows = N // 4100
        hip.dispatch("add", x=row, y=y.sub(0, n_rows * 4100), z=z.sub(0, n_rows * 4100))
        assert n_rows * 4100 > (1 << 32) + 3
        pts = [0, 4099, 4100, (1 << 31) + 11, (1 << 32) + 1, n_rows * 4100 - 1]
        np.testing.assert_array_equal(_at(hip, z, pts), np.array([p % 4100 for p in pts], np.float32) + np.float32(2.0))
        hip.mem_copy(x, z)
        np.testing.assert_array_equal(_at(hip, z), _index_as_f32())
        hip.dispatch("sgd_step", param=z, grad=y, lr=0.5, clip=False, max_norm=1.0, delta=1e-6)
        np.testing.assert_array_equal(_at(hip, z), _index_as_f32() - np.float32(1.0))
        hip.mem_free(one)
        hip.mem_free(row)
    finally:
        for b in (x, y, z):
            hip.mem_free(b)


def test_reductions_over_more_than_2_32_elements(hip):
    y = hip.mem_alloc(F32, N)
    s = hip.mem_alloc(F32, 1)
    try:
        hip.mem_fill(y, 2.0)
        for op, kw, want in (("sum", dict(x=y, y=s), 2.0 * N), ("nrm2", dict(x=y, y=s), 2.0 * np.sqrt(N)),
                             ("dot", dict(x=y, y=y, z=s), 4.0 * N)):
            hip.dispatch(op, **kw)
            got = float(hip.to_numpy(s)[0])
            assert abs(got - want) <= 1e-6 * want, (op, got, want)
        # along either axis of [1048577, 4096] (2^32 + 4096 elements): column sums = 2 * rows, row sums = 2 * cols, both
        # exact in fp32
        rows, cols = (1 << 20) + 1, 4096
        assert (1 << 32) < rows * cols <= N
        v = y.sub(0, rows * cols)
        out_c, out_r = hip.mem_alloc(F32, cols), hip.mem_alloc(F32, rows)
        hip.dispatch("sum_along", x=v, x_shape=[rows, cols], y=out_c, dim=0)
        np.testing.assert_array_equal(hip.to_numpy(out_c), np.full(cols, 2.0 * rows, np.float32))
        hip.dispatch("sum_along", x=v, x_shape=[rows, cols], y=out_r, dim=1)
        np.testing.assert_array_equal(hip.to_numpy(out_r), np.full(rows, 2.0 * cols, np.float32))
        hip.dispatch("max_along", x=v, x_shape=[rows, cols], y=out_r, dim=1)
        np.testing.assert_array_equal(hip.to_numpy(out_r), np.full(rows, 2.0, np.float32))
        # a single larger element far beyond 2^32: the row maximum and its position must find it
        hip.mem_fill(y.sub(rows * cols - 7, 1), 9.0)
        hip.dispatch("max_along", x=v, x_shape=[rows, cols], y=out_r, dim=1)
        got = hip.to_numpy(out_r)
        assert got[-1] == 9.0 and np.all(got[:-1] == 2.0)
        arg = hip.mem_alloc(U64, rows)
        hip.dispatch("argmax_along", x=v, x_shape=[rows, cols], y=arg, dim=1)
        a = hip.to_numpy(arg)
        assert a[-1] == cols - 7 and np.all(a[:-1] == 0)
        for b in (out_c, out_r, arg):
            hip.mem_free(b)
    finally:
        hip.mem_free(y)
        hip.mem_free(s)


def test_gather_by_offsets_beyond_2_32(hip):
    x = hip.mem_alloc(F32, N)
    try:
        hip.mem_sequence(x, 0.0, 1.0)
        pts = np.array([N - 1, 5, (1 << 31) + 1, (1 << 32) + 7, 0, 1 << 24], np.uint64)
        idx = hip.from_numpy(pts)
        dst = hip.mem_alloc(F32, len(pts))
        hip.mem_take(x, idx, dst)
        np.testing.assert_array_equal(hip.to_numpy(dst), pts.astype(np.float64).astype(np.float32))
        hip.mem_free(idx)
        hip.mem_free(dst)
    finally:
        hip.mem_free(x)


ROWS, COLS = (1 << 20) + 1, 4096        # 2^32 + 4096 elements


def test_row_kernels_products_and_optimizer_over_more_than_2_32_elements(hip):
    x, y = hip.mem_alloc(F32, N), hip.mem_alloc(F32, N)
    try:
        n = ROWS * COLS
        xv, yv = x.sub(0, n), y.sub(0, n)
        # softmax of constant rows: 1 / cols everywhere, also in the last row
        hip.mem_fill(xv, 0.5)
        hip.dispatch("softmax_fwd", x=xv, y=yv, rows=ROWS, cols=COLS)
        pts = [0, COLS - 1, (1 << 31) + 9, (1 << 32) + 100, n - 1]
        np.testing.assert_allclose(_at(hip, yv, pts), np.full(len(pts), 1.0 / COLS, np.float32), rtol=1e-6)
        # softmax cross-entropy with integer labels: loss = log(cols) for constant logits; gradient (p - onehot) / rows
        labels = hip.from_numpy(np.full(ROWS, 3, np.uint64))
        lse, loss = hip.mem_alloc(F32, ROWS), hip.mem_alloc(F32, 1)
        hip.dispatch("smce_label_fwd", logits=xv, labels=labels, lse=lse, loss=loss, rows=ROWS, cols=COLS)
        assert abs(float(hip.to_numpy(loss)[0]) - np.log(COLS)) <= 1e-5 * np.log(COLS)
        hip.dispatch("smce_label_bwd", logits=xv, labels=labels, lse=lse, grad=yv, rows=ROWS, cols=COLS, accumulate=False)
        pts = [0, 3, (1 << 32) + 3 - ((1 << 32) % COLS), n - COLS + 3, n - 1]
        want = np.array([(1.0 / COLS - (1.0 if p % COLS == 3 else 0.0)) / ROWS for p in pts], np.float32)
        np.testing.assert_allclose(_at(hip, yv, pts), want, rtol=1e-5)
        for b in (labels, lse, loss):
            hip.mem_free(b)
        # matvec over [ROWS, COLS]: y = A 1 = row sums, and A^T 1 = column sums
        hip.mem_fill(xv, 2.0)
        ones_c, ones_r = hip.from_numpy(np.ones(COLS, np.float32)), hip.from_numpy(np.ones(ROWS, np.float32))
        out_r, out_c = hip.mem_alloc(F32, ROWS), hip.mem_alloc(F32, COLS)
        hip.dispatch("matvec", A=xv, x=ones_c, y=out_r, m=ROWS, n=COLS, trans_a=False, alpha=1.0, beta=0.0)
        np.testing.assert_array_equal(hip.to_numpy(out_r), np.full(ROWS, 2.0 * COLS, np.float32))
        hip.dispatch("matvec", A=xv, x=ones_r, y=out_c, m=ROWS, n=COLS, trans_a=True, alpha=1.0, beta=0.0)
        np.testing.assert_array_equal(hip.to_numpy(out_c), np.full(COLS, 2.0 * ROWS, np.float32))
        # a product whose C has more than 2^32 elements: [ROWS, 8] x [8, COLS], every entry 2 * 3 * 8 = 48
        a8, b8 = hip.mem_alloc(F32, ROWS * 8), hip.mem_alloc(F32, 8 * COLS)
        hip.mem_fill(a8, 2.0)
        hip.mem_fill(b8, 3.0)
        hip.dispatch("matmul", A=a8, B=b8, C=yv, m=ROWS, n=COLS, k=8, trans_a=False, trans_b=False, lda=8, ldb=COLS,
                     ldc=COLS, alpha=1.0, beta=0.0)
        pts = [0, COLS, (1 << 31) + 9, (1 << 32) - 1, (1 << 32) + 100, n - 1]
        np.testing.assert_array_equal(_at(hip, yv, pts), np.full(len(pts), 48.0, np.float32))
        # and a deeper one on the staged kernels: k = 64 -> 2 * 3 * 64 = 384
        a64 = hip.mem_alloc(F32, ROWS * 64)
        b64 = hip.mem_alloc(F32, 64 * COLS)
        hip.mem_fill(a64, 2.0)
        hip.mem_fill(b64, 3.0)
        hip.dispatch("matmul", A=a64, B=b64, C=yv, m=ROWS, n=COLS, k=64, trans_a=False, trans_b=True, lda=64, ldb=64,
                     ldc=COLS, alpha=1.0, beta=0.0)
        np.testing.assert_array_equal(_at(hip, yv, pts), np.full(len(pts), 384.0, np.float32))
        for b in (ones_c, ones_r, out_r, out_c, a8, b8, a64, b64):
            hip.mem_free(b)
        # rows picked from beyond 2^32 (index_select forward) and added back (backward)
        hip.mem_sequence(x, 0.0, 1.0)
        sel = np.array([ROWS - 1, 0, (1 << 19) + 5], np.uint64)
        idx, dst = hip.from_numpy(sel), hip.mem_alloc(F32, len(sel) * COLS)
        hip.dispatch("index_select_fwd", src=xv, indices=idx, stride=COLS, dst=dst)
        got = hip.to_numpy(dst).reshape(len(sel), COLS)
        want = (sel[:, None].astype(np.float64) * COLS + np.arange(COLS)).astype(np.float32)
        np.testing.assert_array_equal(got, want)
        hip.mem_free(idx)
        hip.mem_free(dst)
        # Adam over all N elements: with m = v = 0, g = 2: m = 0.2, v = 0.004 * ... ; every element moves by the same step
        m, v = hip.mem_alloc(F32, N), hip.mem_alloc(F32, N)
        hip.mem_fill(x, 1.0)
        hip.mem_fill(y, 2.0)
        hip.mem_fill(m, 0.0)
        hip.mem_fill(v, 0.0)
        hip.dispatch("adam_step", param=x, grad=y, m=m, v=v, t=1, lr=0.1, beta1=0.9, beta2=0.999, epsilon=1e-8, clip=False,
                     max_norm=1.0, delta=1e-6)
        px = _at(hip, x)
        assert np.all(px == px[0]) and abs(px[0] - 0.9) < 1e-5      # first Adam step moves by lr
        assert np.all(_at(hip, m) == np.float32(0.2)) or np.allclose(_at(hip, m), 0.2, rtol=1e-6)
        hip.mem_free(m)
        hip.mem_free(v)
    finally:
        hip.mem_free(x)
        hip.mem_free(y)
