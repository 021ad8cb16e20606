"""Checks of every device op against what the mathematics fixes, independent of the oracle's own code.

Each check takes a device (the CPU oracle or the HIP device) and compares an op with a float64 numpy closed form, a
brute-force loop written from the op's definition, or an invariant.  The inputs are chosen so that a plausible
mistake -- a dropped term, a wrong sign, swapped operands, a transposed index -- fails: operands are asymmetric,
shapes are non-square, indices repeat, branches are hit on both sides of their threshold.

`PINS` maps every routine the oracle declares to the checks (here or in golden_checks.py / the training tests) that
would fail if that routine were restated wrongly; tests/test_oracle_closed_forms.py asserts that the table is
complete.
"""
from __future__ import annotations

import numpy as np

from conftest import run_op
from zigrad_amd import host

RTOL = 2e-6  # fp32 libm against a float64 closed form: a couple of units in the last place


def f32(a):
    return np.asarray(a, dtype=np.float32)


def rng(seed):
    return np.random.default_rng(seed)


def close(got, want, rtol=RTOL, atol=0.0):
    np.testing.assert_allclose(np.asarray(got, np.float64), np.asarray(want, np.float64), rtol=rtol, atol=atol)


def exact(got, want):
    np.testing.assert_array_equal(got, f32(want))


def r64(a):
    """fp32 values as float64, so that a closed form is evaluated on exactly the numbers the device saw"""
    return np.asarray(a, np.float32).astype(np.float64)


# ---------------------------------------------------------------------------------------------------------------
# elementwise binary: z[i] = x[i % xl] o y[i % yl]  (src/device/host_device.zig:975-1019, src/device/opspec.zig:1-11)
# ---------------------------------------------------------------------------------------------------------------
def check_binary_all_regimes(dev):
    r = rng(1)
    ops = {"add": np.add, "sub": np.subtract, "mul": np.multiply, "div": np.divide}
    # (xl, yl): scalar on either side, equal lengths, the shorter operand first and second, odd periods
    for xl, yl in [(1, 7), (7, 1), (12, 12), (3, 12), (12, 3), (5, 35), (35, 7), (1, 1), (4, 4096), (4096, 8)]:
        x = f32(r.uniform(0.5, 3.0, xl) * r.choice([-1, 1], xl))
        y = f32(r.uniform(0.5, 3.0, yl) * r.choice([-1, 1], yl))
        n = max(xl, yl)
        i = np.arange(n)
        for name, fn in ops.items():
            want = fn(x[i % xl], y[i % yl])  # fp32 numpy: the same IEEE operation, so equality is exact
            out = run_op(dev, name, {"x": x, "y": y, "z": np.full(n, np.nan, np.float32)}, ["z"])
            exact(out["z"], want)
    # in place: z aliases the long operand (NDArray._add / add_: src/ndarray.zig:274-299)
    x, y = f32(r.standard_normal(6)), f32(r.standard_normal(24))
    out = run_op(dev, "sub", {"x": x, "y": y, "z": y}, ["z"])
    exact(out["z"], x[np.arange(24) % 6] - y)
    x2 = f32(r.standard_normal(24))
    out = run_op(dev, "div", {"x": x2, "y": x, "z": x2}, ["z"])
    exact(out["z"], x2 / x[np.arange(24) % 6])
    # a host scalar on either side (NDArray.add_scalar: `.y = &.{s}`, src/ndarray.zig:247-257): the same IEEE operation
    # as the one-float device operand; sizes either side of the vector path and of the small-op queue, in place too
    for n in (1, 3, 24, 4099, 70001):
        v = f32(r.uniform(0.5, 3.0, n) * r.choice([-1, 1], n))
        for s in (np.float32(-1.75), np.float32(0.3)):
            for name, fn in ops.items():
                out = run_op(dev, name, {"x": v, "y": float(s), "z": np.full(n, np.nan, np.float32)}, ["z"])
                exact(out["z"], fn(v, s))
                out = run_op(dev, name, {"x": float(s), "y": v, "z": np.full(n, np.nan, np.float32)}, ["z"])
                exact(out["z"], fn(s, v))
        out = run_op(dev, "sub", {"x": 2.5, "y": v, "z": v}, ["z"])
        exact(out["z"], np.float32(2.5) - v)


# ---------------------------------------------------------------------------------------------------------------
# BLAS-backed level 1/2 (src/device/host_device.zig:224-346): textbook definitions
# ---------------------------------------------------------------------------------------------------------------
def check_dot_axpy_scale_nrm2(dev):
    r = rng(2)
    x, y = f32(r.standard_normal(257)), f32(r.standard_normal(257))
    out = run_op(dev, "dot", {"x": x, "y": y, "z": np.zeros(1, np.float32)}, ["z"])
    close(out["z"][0], np.dot(r64(x), r64(y)), rtol=1e-5)
    # axpy: y += alpha * x -- asymmetric in x and y, alpha negative as in SGD (src/nn/optim.zig:114-118)
    out = run_op(dev, "axpy", {"x": x, "y": y.copy(), "alpha": -0.37}, ["y"])
    close(out["y"], r64(y) + np.float64(np.float32(-0.37)) * r64(x), rtol=1e-6, atol=1e-7)
    out = run_op(dev, "scale", {"x": x.copy(), "alpha": -2.5}, ["x"])
    exact(out["x"], x * np.float32(-2.5))
    out = run_op(dev, "nrm2", {"x": x, "y": np.zeros(1, np.float32)}, ["y"])
    close(out["y"][0], np.sqrt(np.sum(r64(x) ** 2)), rtol=1e-6)
    # sum is cblas_sasum: the sum of magnitudes
    out = run_op(dev, "sum", {"x": x, "y": np.zeros(1, np.float32)}, ["y"])
    close(out["y"][0], np.sum(np.abs(r64(x))), rtol=1e-6)
    # clip_nrm2: x *= max_norm / (norm + delta) only above the threshold (src/device/host_device.zig:339-346)
    norm = np.sqrt(np.sum(r64(x) ** 2))
    out = run_op(dev, "clip_nrm2", {"x": x.copy(), "max_norm": 3.0, "delta": 1e-6}, ["x"])
    close(out["x"], r64(x) * (3.0 / (norm + 1e-6)), rtol=1e-6)
    out = run_op(dev, "clip_nrm2", {"x": x.copy(), "max_norm": float(norm) + 1.0, "delta": 1e-6}, ["x"])
    exact(out["x"], x)


def check_matvec_outer_transpose(dev):
    r = rng(3)
    m, n = 5, 9
    A = f32(r.standard_normal((m, n)))
    # matvec, both orientations, alpha/beta (cblas_sgemv row-major, lda = n: src/device/host_device.zig:232-240)
    x, y0 = f32(r.standard_normal(n)), f32(r.standard_normal(m))
    out = run_op(dev, "matvec", {"A": A.ravel(), "x": x, "y": y0.copy(), "m": m, "n": n, "trans_a": False, "alpha": 1.5,
                                 "beta": -0.5}, ["y"])
    close(out["y"], 1.5 * (r64(A) @ r64(x)) - 0.5 * r64(y0), rtol=1e-5, atol=1e-6)
    xt, yt0 = f32(r.standard_normal(m)), f32(r.standard_normal(n))
    out = run_op(dev, "matvec", {"A": A.ravel(), "x": xt, "y": yt0.copy(), "m": m, "n": n, "trans_a": True, "alpha": 2.0,
                                 "beta": 1.0}, ["y"])
    close(out["y"], 2.0 * (r64(A).T @ r64(xt)) + r64(yt0), rtol=1e-5, atol=1e-6)
    # beta = 0 must not read y
    out = run_op(dev, "matvec", {"A": A.ravel(), "x": x, "y": np.full(m, np.nan, np.float32), "m": m, "n": n,
                                 "trans_a": False, "alpha": 1.0, "beta": 0.0}, ["y"])
    close(out["y"], r64(A) @ r64(x), rtol=1e-5, atol=1e-6)
    # outer: A += alpha * x y^T, row-major with lda = y.len (cblas_sger, :252-259); x and y of different lengths
    xo, yo = f32(r.standard_normal(4)), f32(r.standard_normal(7))
    A0 = f32(r.standard_normal((4, 7)))
    out = run_op(dev, "outer", {"x": xo, "y": yo, "A": A0.ravel().copy(), "alpha": -1.25}, ["A"])
    close(out["A"].reshape(4, 7), r64(A0) - 1.25 * np.outer(r64(xo), r64(yo)), rtol=1e-6, atol=1e-7)
    # transpose: B = A^T + alpha * B (:261-267).  With alpha = 0 the reference still forms 0 * B on the fresh output
    # (src/ndarray.zig:794-802); any finite content must leave a clean transpose.  The device goes further and does
    # not read B then, so a NaN there must not leak either.
    B0 = f32(r.standard_normal((n, m)))
    out = run_op(dev, "transpose", {"A": A.ravel(), "B": B0.ravel().copy(), "m": m, "n": n, "alpha": 1.0}, ["B"])
    exact(out["B"].reshape(n, m), A.T + B0)
    stale = 123.0 if dev.is_host() else np.nan
    out = run_op(dev, "transpose", {"A": A.ravel(), "B": np.full(m * n, stale, np.float32), "m": m, "n": n, "alpha": 0.0},
                 ["B"])
    exact(out["B"].reshape(n, m), A.T)


def check_matmul_layouts(dev):
    """All four transposes with padded leading dimensions, alpha and beta, against a float64 product; the operands
    hold small integers, so every fp32 partial sum is exact and the comparison is for equality."""
    r = rng(4)
    m, n, k = 7, 5, 11
    for ta in (False, True):
        for tb in (False, True):
            a_rows, a_cols = (k, m) if ta else (m, k)
            b_rows, b_cols = (n, k) if tb else (k, n)
            lda, ldb, ldc = a_cols + 3, b_cols + 2, n + 4
            A = np.zeros((a_rows, lda), np.float32)
            B = np.zeros((b_rows, ldb), np.float32)
            A[:, :a_cols] = r.integers(-4, 5, (a_rows, a_cols))
            B[:, :b_cols] = r.integers(-4, 5, (b_rows, b_cols))
            A[:, a_cols:] = 1000.0  # padding must never be read as data
            B[:, b_cols:] = 1000.0
            C0 = np.zeros((m, ldc), np.float32)
            C0[:, :n] = r.integers(-3, 4, (m, n))
            C0[:, n:] = -7.0
            opA = A[:, :a_cols].T if ta else A[:, :a_cols]
            opB = B[:, :b_cols].T if tb else B[:, :b_cols]
            want = C0.copy()
            want[:, :n] = 2.0 * (opA.astype(np.float64) @ opB.astype(np.float64)) - 1.0 * C0[:, :n]
            p = {"A": A.ravel(), "B": B.ravel(), "C": C0.ravel().copy(), "m": m, "n": n, "k": k, "trans_a": ta,
                 "trans_b": tb, "lda": lda, "ldb": ldb, "ldc": ldc, "alpha": 2.0, "beta": -1.0}
            out = run_op(dev, "matmul", p, ["C"])
            exact(out["C"].reshape(m, ldc), want)  # also: the padding columns of C are untouched
            if hasattr(dev, "matmul_f64acc"):  # the oracle's float64-accumulating product, the anchor for large GEMMs
                bufs = {k2: dev.from_numpy(p[k2]) for k2 in ("A", "B", "C")}
                dev.matmul_f64acc(bufs["A"], bufs["B"], bufs["C"], m, n, k, ta, tb, lda, ldb, ldc, 2.0, -1.0)
                exact(dev.to_numpy(bufs["C"]).reshape(m, ldc), want)
    # bmm_acc with operand batch index i % n_batches (src/device/host_device.zig:277-313)
    A = f32(r.integers(-3, 4, (2, 3, 4)))
    B = f32(r.integers(-3, 4, (1, 4, 5)))
    out = run_op(dev, "bmm_acc", {"A": A.ravel(), "B": B.ravel(), "C": np.full(4 * 3 * 5, np.nan, np.float32),
                                  "A_shape": [2, 3, 4], "B_shape": [1, 4, 5], "C_shape": [4, 3, 5], "trans_a": False,
                                  "trans_b": False, "lda": 4, "ldb": 5, "ldc": 5, "alpha": 1.0, "beta": 0.0}, ["C"])
    want = np.stack([A[i % 2].astype(np.float64) @ B[0].astype(np.float64) for i in range(4)])
    exact(out["C"].reshape(4, 3, 5), want)


# ---------------------------------------------------------------------------------------------------------------
# unary forward / backward (src/device/host_device.zig:353-598)
# ---------------------------------------------------------------------------------------------------------------
def check_unary_forward(dev):
    r = rng(5)
    x = f32(np.concatenate([r.uniform(-6, 6, 61), [0.0, -0.0, 1e-3, -1e-3]]))
    z = np.zeros_like(x)
    close(run_op(dev, "tanh_fwd", {"x": x, "y": z.copy()}, ["y"])["y"], np.tanh(r64(x)), atol=1e-7)
    close(run_op(dev, "sigm_fwd", {"x": x, "y": z.copy()}, ["y"])["y"], 1.0 / (1.0 + np.exp(-r64(x))))
    close(run_op(dev, "exp_fwd", {"x": x, "y": z.copy()}, ["y"])["y"], np.exp(r64(x)))
    exact(run_op(dev, "relu_fwd", {"x": x, "y": z.copy()}, ["y"])["y"], np.maximum(x, 0))
    # aliased forward, as nn.relu_ / tanh_ / sigm_ call them (src/nn/nn.zig:39-62)
    close(run_op(dev, "tanh_fwd", {"x": x, "y": x}, ["y"])["y"], np.tanh(r64(x)), atol=1e-7)
    xp = f32(r.uniform(0.05, 9.0, 50))
    close(run_op(dev, "pow_fwd", {"x": xp, "exp": 2.5, "y": np.zeros_like(xp)}, ["y"])["y"], r64(xp) ** 2.5)
    close(run_op(dev, "pow_fwd", {"x": xp, "exp": -1.5, "y": np.zeros_like(xp)}, ["y"])["y"], r64(xp) ** -1.5)
    close(run_op(dev, "pow_fwd_", {"x": xp.copy(), "exp": 0.5}, ["x"])["x"], np.sqrt(r64(xp)))
    exact(run_op(dev, "sqrt_fwd", {"x": xp, "y": np.zeros_like(xp)}, ["y"])["y"], np.sqrt(xp))
    exact(run_op(dev, "sqrt_fwd_", {"x": xp.copy()}, ["x"])["x"], np.sqrt(xp))
    # rsqrt: 1 / sqrt(max(x, eps)) -- inputs on both sides of eps
    xr = f32([4.0, 0.25, 1e-3, 1e-9, 0.0, 9.0])
    eps = 1e-6
    close(run_op(dev, "rsqrt_fwd", {"x": xr, "y": np.zeros_like(xr), "eps": eps}, ["y"])["y"],
          1.0 / np.sqrt(np.maximum(r64(xr), np.float64(np.float32(eps)))))
    # clamp
    xc = f32([-3, -1, -0.5, 0, 0.5, 1, 3])
    exact(run_op(dev, "clamp_fwd", {"x": xc, "y": np.zeros_like(xc), "min": -1.0, "max": 0.5}, ["y"])["y"],
          np.minimum(0.5, np.maximum(-1.0, xc)))


def check_unary_backward(dev):
    """Backward forms: the *_bwd ops ACCUMULATE into x_g (which starts non-zero here), the *_inplace_bwd ops
    MULTIPLY x_g (or zero it), and the saved operand is the OUTPUT y for tanh/sigm/exp but the INPUT x for the rest."""
    r = rng(6)
    n = 48
    y_g = f32(r.uniform(0.5, 2.0, n) * r.choice([-1, 1], n))
    g0 = f32(r.standard_normal(n))
    # tanh / sigm / exp: x_g += f'(y) * y_g with y the saved output
    yt = f32(np.tanh(r.uniform(-2, 2, n)))
    close(run_op(dev, "tanh_bwd", {"x_g": g0.copy(), "y": yt, "y_g": y_g}, ["x_g"])["x_g"],
          r64(g0) + (1.0 - r64(yt) ** 2) * r64(y_g), atol=1e-7)
    ys = f32(1.0 / (1.0 + np.exp(-r.uniform(-3, 3, n))))
    close(run_op(dev, "sigm_bwd", {"x_g": g0.copy(), "y": ys, "y_g": y_g}, ["x_g"])["x_g"],
          r64(g0) + r64(ys) * (1.0 - r64(ys)) * r64(y_g), atol=1e-7)
    ye = f32(np.exp(r.uniform(-2, 2, n)))
    close(run_op(dev, "exp_bwd", {"x_g": g0.copy(), "y": ye, "y_g": y_g}, ["x_g"])["x_g"],
          r64(g0) + r64(ye) * r64(y_g), atol=1e-7)
    # in-place forms: x_g *= f'(x) where x is the op's (in-place) output
    close(run_op(dev, "tanh_inplace_bwd", {"x": yt, "x_g": g0.copy()}, ["x_g"])["x_g"], r64(g0) * (1.0 - r64(yt) ** 2),
          atol=1e-7)
    close(run_op(dev, "sigm_inplace_bwd", {"x": ys, "x_g": g0.copy()}, ["x_g"])["x_g"],
          r64(g0) * (r64(ys) * (1.0 - r64(ys))), atol=1e-7)
    # relu: x_g += y_g where x > 0 (strictly); in place: x_g = 0 where x <= 0, untouched elsewhere
    xr = f32([-2, -0.0, 0.0, 1e-20, 3, -1e-20, 5, 0.5])
    yg8, g8 = y_g[:8], g0[:8]
    exact(run_op(dev, "relu_bwd", {"x": xr, "x_g": g8.copy(), "y_g": yg8}, ["x_g"])["x_g"],
          np.where(xr > 0, g8 + yg8, g8))
    exact(run_op(dev, "relu_inplace_bwd", {"x": xr, "x_g": g8.copy()}, ["x_g"])["x_g"], np.where(xr <= 0, 0.0, g8))
    # pow: x_g += e * x^(e-1) * y_g, nothing added where x < eps
    eps = 1e-3
    xp = f32([2.0, 0.5, 1e-4, 0.0, -1.0, 3.0, 1e-3, 7.5])
    want = r64(g8) + np.where(r64(xp) < np.float64(np.float32(eps)), 0.0,
                              2.5 * np.abs(r64(xp)) ** 1.5 * r64(yg8))
    close(run_op(dev, "pow_bwd", {"x": xp, "x_g": g8.copy(), "exp": 2.5, "y_g": yg8, "eps": eps}, ["x_g"])["x_g"], want,
          atol=1e-7)
    # sqrt: x_g += 0.5 / sqrt(x) * y_g, nothing where x < eps
    want = r64(g8) + np.where(r64(xp) < np.float64(np.float32(eps)), 0.0,
                              0.5 / np.sqrt(np.maximum(np.abs(r64(xp)), 1e-30)) * r64(yg8))
    close(run_op(dev, "sqrt_bwd", {"x": xp, "x_g": g8.copy(), "y_g": yg8, "eps": eps}, ["x_g"])["x_g"], want, atol=1e-7)
    # rsqrt: x_g += -0.5 * x^-1.5 * y_g, nothing where x < eps
    want = r64(g8) + np.where(r64(xp) < np.float64(np.float32(eps)), 0.0,
                              -0.5 * np.maximum(np.abs(r64(xp)), 1e-30) ** -1.5 * r64(yg8))
    close(run_op(dev, "rsqrt_bwd", {"x": xp, "x_g": g8.copy(), "y_g": yg8, "eps": eps}, ["x_g"])["x_g"], want, atol=1e-7)
    # clamp: x_g += y_g strictly inside (min, max)
    xc = f32([-3, -1, -0.5, 0, 0.5, 1, 3, 0.25])
    exact(run_op(dev, "clamp_bwd", {"x": xc, "x_g": g8.copy(), "y_g": yg8, "min": -1.0, "max": 0.5}, ["x_g"])["x_g"],
          np.where((xc > -1.0) & (xc < 0.5), g8 + yg8, g8))


def check_max_fwd_bwd(dev):
    # max_fwd = x[isamax]: largest magnitude, first occurrence; max_bwd: x_g += y_g wherever x == that value (ties)
    x = f32([1.0, -7.0, 3.0, 7.0, -7.0, 2.0])
    y = run_op(dev, "max_fwd", {"x": x, "y": np.zeros(1, np.float32)}, ["y"])["y"]
    assert y[0] == np.float32(-7.0)
    g0 = f32([10, 20, 30, 40, 50, 60])
    out = run_op(dev, "max_bwd", {"x": x, "x_g": g0.copy(), "y": y, "y_g": f32([0.5])}, ["x_g"])
    exact(out["x_g"], [10, 20.5, 30, 40, 50.5, 60])  # both -7 entries, not the +7


# ---------------------------------------------------------------------------------------------------------------
# reductions (src/device/host_device.zig:709-874, src/device/reduce.zig)
# ---------------------------------------------------------------------------------------------------------------
def check_axis_reductions(dev):
    r = rng(7)
    shape = [3, 4, 5]
    x = f32(r.integers(-9, 10, shape))  # integer values: sums are exact in any order
    x[1, 2, 3] = 9.0
    x[1, 2, 4] = 9.0  # a tie along the last axis, and
    x[0, 2, 3] = 9.0  # along the first
    for dim in range(3):
        n_out = int(np.prod(shape)) // shape[dim]
        y0 = f32(r.integers(-5, 6, n_out))
        out = run_op(dev, "sum_along", {"x": x.ravel(), "x_shape": shape, "y": y0.copy(), "dim": dim, "alpha": 2.0,
                                        "beta": -1.0}, ["y"])
        exact(out["y"], (2.0 * x.sum(axis=dim) - y0.reshape(x.sum(axis=dim).shape)).ravel())
        out = run_op(dev, "max_along", {"x": x.ravel(), "x_shape": shape, "y": np.zeros(n_out, np.float32), "dim": dim},
                     ["y"])
        exact(out["y"], x.max(axis=dim).ravel())
        out = run_op(dev, "argmax_along", {"x": x.ravel(), "x_shape": shape, "y": np.zeros(n_out, np.uint64), "dim": dim},
                     ["y"])
        np.testing.assert_array_equal(out["y"], x.argmax(axis=dim).ravel().astype(np.uint64))  # first maximum
    # flat: y of one element takes alpha * sum(x) + beta * y, a signed sum (not the sum of magnitudes)
    out = run_op(dev, "sum_along", {"x": x.ravel(), "x_shape": [x.size], "y": f32([4.0]), "dim": 0, "alpha": 0.5,
                                    "beta": 3.0}, ["y"])
    exact(out["y"], [0.5 * x.sum() + 12.0])
    # max_along of all-negative rows starts from -inf, not from the zeros the output was filled with
    xn = f32([[-3, -2, -8], [-1, -5, -4]])
    out = run_op(dev, "max_along", {"x": xn.ravel(), "x_shape": [2, 3], "y": np.zeros(2, np.float32), "dim": 1}, ["y"])
    exact(out["y"], [-2, -1])


def check_unbroadcast(dev):
    r = rng(8)
    cases = [([4, 3, 5], [3, 5]), ([4, 3, 5], [5]), ([4, 3, 5], [1, 3, 5]), ([4, 3, 5], [4, 1, 5]),
             ([3, 4, 2, 5], [4, 1, 5]), ([6, 2, 3], [1, 1, 3]), ([3, 5], [3, 5])]
    for xs, ys in cases:
        x = f32(r.integers(-6, 7, xs))
        # numpy: sum over the leading extra axes and over every axis where y has extent 1
        lead = len(xs) - len(ys)
        want = x.astype(np.float64).sum(axis=tuple(range(lead))) if lead else x.astype(np.float64)
        axes = tuple(i for i, s in enumerate(ys) if s == 1 and want.shape[i] != 1)
        if axes:
            want = want.sum(axis=axes, keepdims=True)
        # scratch rule of NDArray.unbroadcast_ (src/ndarray.zig:701-719)
        x_size, y_size = int(np.prod(xs)), int(np.prod(ys))
        if lead > 0:
            coef = int(np.prod(xs[:lead]))
        else:
            mm = [i for i in range(len(xs)) if xs[i] != ys[i]]
            coef = xs[mm[0]] if mm else None
        n_scratch = 0 if coef is None or y_size * coef == x_size else y_size * coef
        assert dev.unbroadcast_scratch_len(xs, ys) == n_scratch, (xs, ys)
        # beta acts at EVERY stage (src/device/host_device.zig:740-775), so with two stages and beta = 1 the first
        # one adds whatever the scratch held before: only a single-stage reduction is defined for beta != 0
        for beta in ((0.0, 1.0) if n_scratch == 0 else (0.0,)):
            y0 = f32(r.integers(-4, 5, ys))
            bx, by = dev.from_numpy(x.ravel()), dev.from_numpy(y0.ravel())
            host.unbroadcast_(dev, bx, xs, by, ys, alpha=1.0, beta=beta)
            dev.sync()
            exact(dev.to_numpy(by), (want + beta * y0.astype(np.float64)).ravel())
    # Two shapes the reference's own staging cannot handle (its host loops write past their buffers): [2,4,3,5] ->
    # [4,1,5], where the scratch rule yields 40 floats but the first fold produces 4*3*5 = 60, and [4,3,5] -> [4,3,1],
    # where the trailing 1 is trimmed and the fold over the leading dim writes 15 floats into an output of 12.  The
    # device must refuse such a call instead of launching.
    if not dev.is_host():
        from zigrad_amd._lib import ZgHipError

        for xs, ys in (([2, 4, 3, 5], [4, 1, 5]), ([4, 3, 5], [4, 3, 1])):
            bx = dev.from_numpy(np.zeros(int(np.prod(xs)), np.float32))
            by = dev.from_numpy(np.zeros(int(np.prod(ys)), np.float32))
            try:
                host.unbroadcast_(dev, bx, xs, by, ys, alpha=1.0, beta=0.0)
            except ZgHipError as e:
                assert e.code == 1
            else:
                raise AssertionError(f"unbroadcast {xs} -> {ys} overflows a stage buffer and was launched")
    # one stage only: general alpha and beta apply once
    x = f32(r.integers(-6, 7, [5, 4]))
    y0 = f32(r.integers(-4, 5, [4]))
    bx, by = dev.from_numpy(x.ravel()), dev.from_numpy(y0)
    host.unbroadcast_(dev, bx, [5, 4], by, [4], alpha=0.5, beta=-2.0)
    dev.sync()
    exact(dev.to_numpy(by), 0.5 * x.sum(axis=0) - 2.0 * y0)


def check_broadcast(dev):
    r = rng(9)
    a, b = 1.5, -0.5
    # x shorter than y: y[i] = alpha * x[i % xl] + beta * y[i]
    x, y0 = f32(r.integers(-5, 6, 3)), f32(r.integers(-5, 6, 12))
    out = run_op(dev, "broadcast", {"x": x, "y": y0.copy(), "alpha": a, "beta": b}, ["y"])
    exact(out["y"], a * x[np.arange(12) % 3] + b * y0)
    # equal lengths: the reference's scaled copy is followed by the modulo loop (no `return`,
    # src/device/host_device.zig:782-795), so alpha/beta act twice: y = a x + b (a x + b y)
    x, y0 = f32(r.integers(-5, 6, 8)), f32(r.integers(-5, 6, 8))
    out = run_op(dev, "broadcast", {"x": x, "y": y0.copy(), "alpha": a, "beta": b}, ["y"])
    exact(out["y"], a * x + b * (a * x + b * y0))
    assert not np.array_equal(out["y"], a * x + b * y0)


# ---------------------------------------------------------------------------------------------------------------
# memory-style and index ops
# ---------------------------------------------------------------------------------------------------------------
def check_mem_ops(dev):
    b = dev.mem_alloc(np.float32, 9)
    dev.mem_fill(b, -2.5)
    dev.sync()
    exact(dev.to_numpy(b), np.full(9, -2.5))
    dev.mem_sequence(b, 3.0, -2.0)  # initial, initial + step, ... (src/device/host_device.zig:947-953)
    dev.sync()
    exact(dev.to_numpy(b), 3.0 - 2.0 * np.arange(9))
    src = dev.from_numpy(f32(np.arange(10) * 1.5))
    idx = dev.from_numpy(np.asarray([9, 0, 3, 3, 7], np.uint64))
    dst = dev.mem_alloc(np.float32, 5)
    dev.mem_take(src, idx, dst)
    dev.sync()
    exact(dev.to_numpy(dst), [13.5, 0, 4.5, 4.5, 10.5])


# ---------------------------------------------------------------------------------------------------------------
# mem_random (src/device/host_device.zig:931-945 fixes WHAT is drawn: U[0,1), N(0,1), N(0,1) * sqrt(2 / fan)).
# The stream is the documented one: splitmix64 seeding -> xoshiro256++ -> top 24 bits -> Box-Muller (cosine branch).
# It is written here a further time, in Python integers, and that copy is first held to the published known-answer
# vectors of the two generators (Vigna's splitmix64.c from seed 0 and from 1234567; xoshiro256++ from state
# {1, 2, 3, 4}, the vector of the generator's reference implementation that Zig's std.Random.Xoshiro256 test and
# Rust's rand_xoshiro repeat), so a wrong constant, rotate or shift in every copy cannot pass.
# ---------------------------------------------------------------------------------------------------------------
_M64 = (1 << 64) - 1


def _splitmix64(seed, count):
    z, out = seed & _M64, []
    for _ in range(count):
        z = (z + 0x9E3779B97F4A7C15) & _M64
        v = z
        v = ((v ^ (v >> 30)) * 0xBF58476D1CE4E5B9) & _M64
        v = ((v ^ (v >> 27)) * 0x94D049BB133111EB) & _M64
        out.append(v ^ (v >> 31))
    return out


def _xoshiro256pp(state, count):
    def rotl(x, k):
        return ((x << k) | (x >> (64 - k))) & _M64

    s, out = list(state), []
    for _ in range(count):
        out.append((rotl((s[0] + s[3]) & _M64, 23) + s[0]) & _M64)
        t = (s[1] << 17) & _M64
        s[2] ^= s[0]
        s[3] ^= s[1]
        s[1] ^= s[2]
        s[0] ^= s[3]
        s[2] ^= t
        s[3] = rotl(s[3], 45)
    return out


def _documented_uniforms(seed, count):
    """float64 values of the documented stream's uniforms: every one is k * 2^-24, exact in fp32 and fp64"""
    return np.asarray([w >> 40 for w in _xoshiro256pp(_splitmix64(seed, 4), count)], np.float64) / 16777216.0


def check_mem_random(dev):
    assert _splitmix64(0, 5) == [0xE220A8397B1DCDAF, 0x6E789E6AA1B965F4, 0x06C45D188009454F, 0xF88BB8A8724C81EC,
                                 0x1B39896A51A8749B]
    assert _splitmix64(1234567, 5) == [6457827717110365317, 3203168211198807973, 9817491932198370423,
                                       4593380528125082431, 16408922859458223821]
    assert _xoshiro256pp([1, 2, 3, 4], 10) == [
        41943041, 58720359, 3588806011781223, 3591011842654386, 9228616714210784205, 9973669472204895162,
        14011001112246962877, 12406186145184390807, 15849039046786891736, 10450023813501588000]

    def draw(n, kind, seed, fan=0):
        b = dev.mem_alloc(np.float32, n)
        dev.mem_fill(b, np.nan)
        dev.mem_random(b, kind, seed=seed, fan=fan)
        dev.sync()
        out = dev.to_numpy(b).copy()
        dev.mem_free(b)
        return out

    fan = 784
    for seed in (0, 81761, 2**63 + 12345):
        for n in (16, 1, 257):
            u = _documented_uniforms(seed, 2 * n)
            exact(draw(n, "uniform", seed), u[:n])  # one word per uniform, in order
            # normal i takes words 2i and 2i+1: radius from 1 - u (so the logarithm never sees 0), angle from the
            # second; cos near its zeros keeps only absolute accuracy (the fp32 angle is rounded), hence atol
            want = np.sqrt(-2.0 * np.log(1.0 - u[0::2])) * np.cos(2.0 * np.pi * u[1::2])
            close(draw(n, "normal", seed), want, rtol=2e-6, atol=5e-6)
            close(draw(n, "kaiming", seed, fan), want * np.sqrt(2.0 / fan), rtol=3e-6, atol=5e-6 * np.sqrt(2.0 / fan))
    assert not np.array_equal(draw(16, "uniform", 1), draw(16, "uniform", 2))  # the seed is used
    # distribution (what the reference's contract fixes): moments, range and independence of neighbours on 10^6
    # draws; every bound is five or more standard errors wide
    n = 1_000_000
    u = r64(draw(n, "uniform", 7))
    assert u.min() >= 0.0 and u.max() < 1.0
    assert abs(u.mean() - 0.5) < 5 * np.sqrt(1 / 12 / n) and abs(u.var() - 1 / 12) < 5e-4
    assert np.all(np.abs(np.histogram(u, bins=16, range=(0, 1))[0] / n - 1 / 16) < 5 * np.sqrt(1 / 16 / n))
    for kind, sd in (("normal", 1.0), ("kaiming", np.sqrt(2.0 / fan))):
        z = r64(draw(n, kind, 11, fan)) / sd
        assert abs(z.mean()) < 5 / np.sqrt(n) and abs(z.var() - 1.0) < 5 * np.sqrt(2 / n)
        assert abs(np.mean(z ** 3)) < 5 * np.sqrt(15 / n) and abs(np.mean(z ** 4) - 3.0) < 5 * np.sqrt(96 / n)
        assert abs(np.mean(z[:-1] * z[1:])) < 5 / np.sqrt(n)
        assert abs(np.mean(np.abs(z) < 1.0) - 0.6826894921) < 5 * np.sqrt(0.2167 / n)


def check_gather_offsets(dev):
    """offsets[i] = flat position in src of the index tensor's coordinate i with coordinate `dim` replaced by the
    index value (src/ndarray.zig:607-624), brute force over a rank-3 case with an index tensor smaller than src."""
    r = rng(10)
    src_shape, idx_shape = [3, 4, 5], [2, 3, 4]
    for dim in range(3):
        idx = r.integers(0, src_shape[dim], idx_shape).astype(np.uint64)
        want = np.zeros(idx.size, np.uint64)
        for flat, pos in enumerate(np.ndindex(*idx_shape)):
            c = list(pos)
            c[dim] = int(idx[pos])
            want[flat] = (c[0] * src_shape[1] + c[1]) * src_shape[2] + c[2]
        bi, bo = dev.from_numpy(idx.ravel()), dev.mem_alloc(np.uint64, idx.size)
        assert dev.gather_offsets(src_shape, idx_shape, bi, dim, bo) == 0
        dev.sync()
        np.testing.assert_array_equal(dev.to_numpy(bo), want)
    # errors: an index tensor wider than src off `dim` (1), an index value out of range (2)
    bi, bo = dev.from_numpy(np.zeros(6, np.uint64)), dev.mem_alloc(np.uint64, 6)
    assert dev.gather_offsets([2, 2], [3, 2], bi, 1, bo) == 1
    bi = dev.from_numpy(np.asarray([0, 2, 0, 1], np.uint64))
    assert dev.gather_offsets([2, 2], [2, 2], bi, 1, bo) == 2


def check_scatter_and_select(dev):
    r = rng(11)
    # scatter_add: dst[off[i]] += src[i], sequential in i (src/device/host_device.zig:1039-1087); repeated offsets
    n, m = 40, 7
    src = f32(r.standard_normal(n))
    off = r.integers(0, m, n).astype(np.uint64)
    dst0 = f32(r.standard_normal(m))
    want = dst0.copy()
    for i in range(n):
        want[off[i]] = np.float32(want[off[i]] + src[i])
    out = run_op(dev, "scatter_add", {"src": src, "offsets": off, "dst": dst0.copy()}, ["dst"])
    exact(out["dst"], want)
    # index_select: row `indices[j]` of stride elements -> row j; backward adds row j of y_grad into row indices[j]
    # of x_grad, in order of j (src/ndtensor.zig:1437-1513); index 2 appears three times
    stride, rows = 3, 5
    x = f32(r.standard_normal(rows * stride))
    indices = np.asarray([2, 0, 2, 4, 2, 1], np.uint64)
    out = run_op(dev, "index_select_fwd", {"src": x, "indices": indices, "stride": stride,
                                           "dst": np.zeros(indices.size * stride, np.float32)}, ["dst"])
    exact(out["dst"], x.reshape(rows, stride)[indices.astype(np.int64)].ravel())
    yg = f32(r.standard_normal(indices.size * stride))
    xg0 = f32(r.standard_normal(rows * stride))
    want = xg0.copy().reshape(rows, stride)
    for j, i in enumerate(indices.astype(np.int64)):
        want[i] = (yg.reshape(-1, stride)[j] + want[i]).astype(np.float32)
    out = run_op(dev, "index_select_bwd", {"y_grad": yg, "indices": indices, "stride": stride, "x_grad": xg0.copy()},
                 ["x_grad"])
    exact(out["x_grad"], want.ravel())


def check_csr_ops(dev):
    # scatter_add_csr broadcasts src[i] over [row_ptr[i], row_ptr[i+1]); segment_sum_csr writes the segment sums
    # (src/device/host_device.zig:1325-1353); an empty segment in each
    src = f32([2.0, -1.0, 5.0, 0.5])
    row_ptr = np.asarray([0, 3, 3, 4, 9], np.uint64)
    dst0 = f32(np.arange(9))
    want = dst0.copy()
    for i in range(4):
        want[int(row_ptr[i]):int(row_ptr[i + 1])] += src[i]
    out = run_op(dev, "scatter_add_csr", {"src": src, "row_ptr": row_ptr, "dst": dst0.copy()}, ["dst"])
    exact(out["dst"], want)
    vals = f32(np.arange(1, 10))
    out = run_op(dev, "segment_sum_csr", {"src": vals, "row_offsets": row_ptr, "dst": np.full(4, np.nan, np.float32)},
                 ["dst"])
    exact(out["dst"], [6, 0, 4, 35])


def check_gcn_scatter(dev):
    """dst[t] += deg[s] deg[t] h[s] per edge is the dense product (D A^T D) h with A[s, t] = multiplicity of the edge;
    the backward ops are the gradients of sum(go * dst): checked against the dense forms in float64."""
    r = rng(12)
    n, e, f = 6, 17, 3
    s = r.integers(0, n, e).astype(np.uint64)
    t = r.integers(0, n, e).astype(np.uint64)
    s[0], t[0] = 2, 2  # a self-loop
    s[1], t[1], s[2], t[2] = 3, 4, 3, 4  # a repeated edge
    h = f32(r.standard_normal((n, f)))
    deg = f32(r.uniform(0.3, 1.0, n))
    dst0 = f32(r.standard_normal((n, f)))
    W = np.zeros((n, n))  # W[t, s]
    for a, b in zip(s.astype(int), t.astype(int)):
        W[b, a] += r64(deg)[a] * r64(deg)[b]
    out = run_op(dev, "scatter_gcn_deg_scaled", {"dst": dst0.ravel().copy(), "h": h.ravel(), "deg": deg, "src_indices": s,
                                                 "tgt_indices": t, "stride": f, "n_edge": e}, ["dst"])
    close(out["dst"].reshape(n, f), r64(dst0) + W @ r64(h), rtol=1e-5, atol=1e-6)
    go = f32(r.standard_normal((n, f)))
    gh0, gd0 = f32(r.standard_normal((n, f))), f32(r.standard_normal(n))
    out = run_op(dev, "scatter_gcn_deg_scaled_bwd",
                 {"grad_output": go.ravel(), "h": h.ravel(), "deg": deg, "src_indices": s, "tgt_indices": t,
                  "grad_h": gh0.ravel().copy(), "grad_deg": gd0.copy(), "stride": f, "n_edge": e}, ["grad_h", "grad_deg"])
    close(out["grad_h"].reshape(n, f), r64(gh0) + W.T @ r64(go), rtol=1e-5, atol=1e-6)
    gd = r64(gd0).copy()
    for a, b in zip(s.astype(int), t.astype(int)):
        dots = float(np.dot(r64(go)[b], r64(h)[a]))
        gd[a] += r64(deg)[b] * dots
        gd[b] += r64(deg)[a] * dots
    close(out["grad_deg"], gd, rtol=1e-5, atol=1e-6)


# ---------------------------------------------------------------------------------------------------------------
# losses (src/nn/loss.zig:94-305)
# ---------------------------------------------------------------------------------------------------------------
def _softmax64(x):
    x = r64(x)
    e = np.exp(x - x.max(axis=1, keepdims=True))
    return e / e.sum(axis=1, keepdims=True)


def check_softmax_and_smce(dev):
    from scipy.special import logsumexp

    r = rng(13)
    rows, cols = 5, 9
    x = f32(r.standard_normal((rows, cols)) * 3)
    p = _softmax64(x)
    out = run_op(dev, "softmax_fwd", {"x": x.ravel(), "y": np.zeros(rows * cols, np.float32), "rows": rows, "cols": cols},
                 ["y"])
    close(out["y"].reshape(rows, cols), p, rtol=1e-5)
    # softmax backward: x_g += y * (y_g - sum_j y_j y_g_j) per row (src/nn/loss.zig:223-246); x_g starts non-zero
    y32 = f32(p)
    yg = f32(r.standard_normal((rows, cols)))
    xg0 = f32(r.standard_normal((rows, cols)))
    want = r64(xg0) + r64(y32) * (r64(yg) - (r64(y32) * r64(yg)).sum(axis=1, keepdims=True))
    out = run_op(dev, "softmax_bwd", {"y": y32.ravel(), "y_g": yg.ravel(), "x_g": xg0.ravel().copy(), "rows": rows,
                                      "cols": cols}, ["x_g"])
    close(out["x_g"].reshape(rows, cols), want, rtol=1e-5, atol=1e-6)
    # cross-entropy with soft (non one-hot) targets: -(1/B) sum t log p; gradient accumulates (p - t) / B
    t = f32(r.dirichlet(np.ones(cols), rows))
    out = run_op(dev, "smce_fwd", {"logits": x.ravel(), "target": t.ravel(), "probs": np.zeros(rows * cols, np.float32),
                                   "loss": np.zeros(1, np.float32), "rows": rows, "cols": cols}, ["probs", "loss"])
    close(out["probs"].reshape(rows, cols), p, rtol=1e-5)
    close(out["loss"][0], -(r64(t) * np.log(np.clip(p, 1e-7, 1 - 1e-7))).sum() / rows, rtol=1e-5)
    g0 = f32(r.standard_normal((rows, cols)))
    pr = out["probs"]
    out = run_op(dev, "smce_bwd", {"probs": pr, "target": t.ravel(), "grad": g0.ravel().copy(), "rows": rows, "cols": cols},
                 ["grad"])
    close(out["grad"].reshape(rows, cols), r64(g0) + (r64(pr).reshape(rows, cols) - r64(t)) / rows, rtol=1e-5, atol=1e-7)
    # integer labels: loss = mean(logsumexp - x[label]); lse saved; gradient (softmax - onehot) / B
    lab = r.integers(0, cols, rows).astype(np.uint64)
    out = run_op(dev, "smce_label_fwd", {"logits": x.ravel(), "labels": lab, "lse": np.zeros(rows, np.float32),
                                         "loss": np.zeros(1, np.float32), "rows": rows, "cols": cols}, ["lse", "loss"])
    lse = logsumexp(r64(x), axis=1)
    close(out["lse"], lse, rtol=1e-6)
    close(out["loss"][0], np.mean(lse - r64(x)[np.arange(rows), lab.astype(int)]), rtol=1e-5)
    onehot = np.zeros((rows, cols))
    onehot[np.arange(rows), lab.astype(int)] = 1.0
    out = run_op(dev, "smce_label_bwd", {"logits": x.ravel(), "labels": lab, "lse": out["lse"],
                                         "grad": g0.ravel().copy(), "rows": rows, "cols": cols}, ["grad"])
    close(out["grad"].reshape(rows, cols), r64(g0) + (p - onehot) / rows, rtol=1e-5, atol=1e-7)
    # the clamp acts in the loss only: a label whose probability underflows costs -log(1e-7), and a row that is all
    # but certain costs -log(1 - 1e-7) in fp32 (src/nn/loss.zig:143)
    xe = f32([[40.0, 0.0, 0.0], [40.0, 0.0, 0.0]])
    out = run_op(dev, "smce_label_fwd", {"logits": xe.ravel(), "labels": np.asarray([1, 0], np.uint64),
                                         "lse": np.zeros(2, np.float32), "loss": np.zeros(1, np.float32), "rows": 2,
                                         "cols": 3}, ["loss"])
    hi = np.float64(np.float32(1.0) - np.float32(1e-7))
    close(out["loss"][0], 0.5 * (-np.log(np.float64(np.float32(1e-7))) - np.log(hi)), rtol=1e-5)


def check_regression_losses(dev):
    # smooth-L1 with beta = 0.5: quadratic inside |d| < beta, linear outside, d = 0 and |d| = beta (linear branch)
    beta = 0.5
    pred = f32([1.0, 2.0, 3.0, 4.0, 5.0, 6.0, 7.0])
    targ = f32([1.2, 2.0, 1.0, 4.5, 4.75, 9.0, 7.4])
    d = r64(pred) - r64(targ)
    n = d.size
    per = np.where(np.abs(d) < beta, 0.5 * d * d / beta, np.abs(d) - 0.5 * beta)
    out = run_op(dev, "smooth_l1_fwd", {"pred": pred, "target": targ, "beta": beta, "loss": np.zeros(1, np.float32)}, ["loss"])
    close(out["loss"][0], per.sum() / n, rtol=1e-6)
    g0 = f32(np.arange(n) * 0.1)
    want = r64(g0) + np.where(np.abs(d) < beta, d / (beta * n), np.sign(d) / n)
    out = run_op(dev, "smooth_l1_bwd", {"pred": pred, "target": targ, "grad": g0.copy(), "beta": beta}, ["grad"])
    close(out["grad"], want, rtol=1e-6, atol=1e-7)
    # MSE: mean squared difference; gradient accumulates 2 (p - t) / n
    out = run_op(dev, "mse_fwd", {"pred": pred, "target": targ, "loss": np.zeros(1, np.float32)}, ["loss"])
    close(out["loss"][0], np.mean(d * d), rtol=1e-6)
    out = run_op(dev, "mse_bwd", {"pred": pred, "target": targ, "grad": g0.copy()}, ["grad"])
    close(out["grad"], r64(g0) + 2.0 * d / n, rtol=1e-6, atol=1e-7)


# ---------------------------------------------------------------------------------------------------------------
# optimizers (src/nn/optim.zig:100-122, :177-234)
# ---------------------------------------------------------------------------------------------------------------
def check_optimizers(dev):
    r = rng(14)
    n = 33
    p0, g0 = f32(r.standard_normal(n)), f32(r.standard_normal(n) * 4)  # |g| ~ 23 > max_norm 10: the clip bites
    norm = np.sqrt(np.sum(r64(g0) ** 2))
    assert norm > 10
    for clip in (False, True):
        gc = r64(g0) * (10.0 / (norm + 1e-6)) if clip else r64(g0)
        out = run_op(dev, "sgd_step", {"param": p0.copy(), "grad": g0.copy(), "lr": 0.01, "clip": clip, "max_norm": 10.0,
                                       "delta": 1e-6}, ["param", "grad"])
        close(out["param"], r64(p0) - 0.01 * gc, rtol=1e-6, atol=1e-7)
        close(out["grad"], gc, rtol=1e-6)  # the clipped gradient stays in place
        # Adam, two updates of the same tensor with counter values 3 and 4 (the counter is per tensor update)
        # the hyper-parameters as the fp32 values the op receives
        lr, b1, b2, eps = (float(np.float32(v)) for v in (0.01, 0.9, 0.999, 1e-8))
        m, v, p = np.zeros(n), np.zeros(n), r64(p0).copy()
        bufs = {k: dev.from_numpy(a) for k, a in (("param", p0.copy()), ("grad", g0.copy()),
                                                  ("m", np.zeros(n, np.float32)), ("v", np.zeros(n, np.float32)))}
        g = gc.copy()
        for t in (3, 4):
            dev.dispatch("adam_step", t=t, lr=lr, beta1=b1, beta2=b2, epsilon=eps, clip=clip, max_norm=10.0, delta=1e-6,
                         **bufs)
            lr_t = lr * np.sqrt(1.0 - b2 ** t) / (1.0 - b1 ** t)
            m = b1 * m + (1 - b1) * g
            v = b2 * v + (1 - b2) * g * g
            p = p - lr_t * m / (np.sqrt(v) + eps)
            # after the first clip the gradient's norm is just under max_norm: the second update leaves it alone
        dev.sync()
        close(dev.to_numpy(bufs["param"]), p, rtol=2e-5, atol=1e-6)
        close(dev.to_numpy(bufs["m"]), m, rtol=1e-5, atol=1e-7)
        close(dev.to_numpy(bufs["v"]), v, rtol=1e-5, atol=1e-9)
    # lr_t = lr * sqrt(1 - beta2^t) / (1 - beta1^t), formed in fp32 (src/nn/optim.zig:190-191): 1 - beta2^t loses up to
    # five digits to cancellation for small t, hence the tolerance
    lr, b1, b2 = (float(np.float32(v)) for v in (0.01, 0.9, 0.999))
    for t in (1, 2, 7, 1000):
        close(dev.adam_lr_t(0.01, 0.9, 0.999, t), lr * np.sqrt(1 - b2 ** t) / (1 - b1 ** t), rtol=1e-4)


ALL_CHECKS = [
    check_binary_all_regimes, check_dot_axpy_scale_nrm2, check_matvec_outer_transpose, check_matmul_layouts,
    check_unary_forward, check_unary_backward, check_max_fwd_bwd, check_axis_reductions, check_unbroadcast,
    check_broadcast, check_mem_ops, check_mem_random, check_gather_offsets, check_scatter_and_select, check_csr_ops, check_gcn_scatter,
    check_softmax_and_smce, check_regression_losses, check_optimizers,
]

# Which checks pin which restated routine.  "golden:<name>" is a check of golden_checks.py (the reference's own test
# vectors); "train:<name>" a test of tests/test_oracle_train.py (independent float64 backprop of whole steps).
PINS = {
    "zo_add": ["check_binary_all_regimes", "golden:check_add_sub_scalar", "golden:check_add_broadcast_grad"],
    "zo_sub": ["check_binary_all_regimes", "golden:check_add_sub_scalar"],
    "zo_mul": ["check_binary_all_regimes", "golden:check_mul_div_backward"],
    "zo_div": ["check_binary_all_regimes", "golden:check_mul_div_backward"],
    "zo_dot": ["check_dot_axpy_scale_nrm2", "golden:check_dot", "golden:check_matvec_dot_backward"],
    "zo_matvec": ["check_matvec_outer_transpose", "golden:check_matvec", "golden:check_matvec_dot_backward"],
    "zo_matmul": ["check_matmul_layouts", "golden:check_bmm", "golden:check_matmul_backward"],
    "zo_matmul_f64acc": ["check_matmul_layouts"],
    "zo_bmm_acc": ["check_matmul_layouts", "golden:check_bmm"],
    "zo_outer": ["check_matvec_outer_transpose", "golden:check_matvec_dot_backward"],
    "zo_transpose": ["check_matvec_outer_transpose"],
    "zo_axpy": ["check_dot_axpy_scale_nrm2", "golden:check_matvec_dot_backward"],
    "zo_sum": ["check_dot_axpy_scale_nrm2", "golden:check_sum"],
    "zo_scale": ["check_dot_axpy_scale_nrm2"],
    "zo_nrm2": ["check_dot_axpy_scale_nrm2", "golden:check_clip_nrm2"],
    "zo_clip_nrm2": ["check_dot_axpy_scale_nrm2", "golden:check_clip_nrm2"],
    "zo_pow_fwd": ["check_unary_forward", "golden:check_pow_sqrt"],
    "zo_pow_bwd": ["check_unary_backward", "golden:check_pow_sqrt"],
    "zo_sqrt_fwd": ["check_unary_forward", "golden:check_pow_sqrt"],
    "zo_sqrt_bwd": ["check_unary_backward", "golden:check_pow_sqrt"],
    "zo_rsqrt_fwd": ["check_unary_forward"],
    "zo_rsqrt_bwd": ["check_unary_backward"],
    "zo_exp_fwd": ["check_unary_forward"],
    "zo_exp_bwd": ["check_unary_backward"],
    "zo_relu_fwd": ["check_unary_forward"],
    "zo_relu_bwd": ["check_unary_backward"],
    "zo_relu_inplace_bwd": ["check_unary_backward"],
    "zo_tanh_fwd": ["check_unary_forward"],
    "zo_tanh_bwd": ["check_unary_backward"],
    "zo_tanh_inplace_bwd": ["check_unary_backward"],
    "zo_sigm_fwd": ["check_unary_forward"],
    "zo_sigm_bwd": ["check_unary_backward"],
    "zo_sigm_inplace_bwd": ["check_unary_backward"],
    "zo_clamp_fwd": ["check_unary_forward", "golden:check_clamp"],
    "zo_clamp_bwd": ["check_unary_backward", "golden:check_clamp"],
    "zo_max_fwd": ["check_max_fwd_bwd", "golden:check_sum"],
    "zo_max_bwd": ["check_max_fwd_bwd"],
    "zo_sum_along": ["check_axis_reductions", "golden:check_sum_max_along"],
    "zo_max_along": ["check_axis_reductions", "golden:check_sum_max_along"],
    "zo_argmax_along": ["check_axis_reductions"],
    "zo_unbroadcast_scratch_len": ["check_unbroadcast"],
    "zo_unbroadcast": ["check_unbroadcast", "golden:check_add_broadcast_grad"],
    "zo_broadcast": ["check_broadcast"],
    "zo_mem_fill": ["check_mem_ops"],
    "zo_mem_sequence": ["check_mem_ops"],
    "zo_mem_random": ["check_mem_random"],
    "zo_mem_take": ["check_mem_ops", "golden:check_gather"],
    "zo_gather_offsets": ["check_gather_offsets", "golden:check_gather"],
    "zo_scatter_add": ["check_scatter_and_select"],
    "zo_scatter_add_csr": ["check_csr_ops"],
    "zo_segment_sum_csr": ["check_csr_ops"],
    "zo_index_select_fwd": ["check_scatter_and_select"],
    "zo_index_select_bwd": ["check_scatter_and_select"],
    "zo_scatter_gcn_deg_scaled": ["check_gcn_scatter", "train:test_gcn_gradients_match_dense_numpy"],
    "zo_scatter_gcn_deg_scaled_bwd": ["check_gcn_scatter", "train:test_gcn_gradients_match_dense_numpy"],
    "zo_smce_fwd": ["check_softmax_and_smce", "golden:check_losses"],
    "zo_smce_bwd": ["check_softmax_and_smce", "golden:check_losses"],
    "zo_smce_label_fwd": ["check_softmax_and_smce", "golden:check_losses"],
    "zo_smce_label_bwd": ["check_softmax_and_smce", "golden:check_losses"],
    "zo_softmax_fwd": ["check_softmax_and_smce"],
    "zo_softmax_bwd": ["check_softmax_and_smce"],
    "zo_smooth_l1_fwd": ["check_regression_losses", "golden:check_losses"],
    "zo_smooth_l1_bwd": ["check_regression_losses", "golden:check_losses"],
    "zo_mse_fwd": ["check_regression_losses"],
    "zo_mse_bwd": ["check_regression_losses"],
    "zo_sgd_step": ["check_optimizers", "train:test_mlp_gradients_match_numpy_backprop"],
    "zo_adam_step": ["check_optimizers", "train:test_adam_counter_is_per_tensor_and_clip_is_per_tensor"],
    "zo_adam_lr_t": ["check_optimizers"],
}

# declared but deliberately without a pin: none.  The zo_blas_* calls select a backend and compute nothing.
UNPINNED = set()
NOT_ARITHMETIC = {"zo_blas_name", "zo_blas_set_threads", "zo_blas_force_builtin"}
