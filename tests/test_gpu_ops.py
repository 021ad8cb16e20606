"""Parity of every HIP device op with the CPU oracle on identical seeded inputs, through the C ABI.

Tolerances: bit-exact (array_equal) for index / integer / copy-like work and for elementwise ops built
only from IEEE add/sub/mul/div/sqrt/compare; relative Frobenius error <= 1e-5 for ops that call
transcendental functions or change the summation order (the benchmark definition's bound per op).
"""
from __future__ import annotations

import numpy as np
import pytest

from conftest import rel_fro, run_op

pytestmark = pytest.mark.gpu

TOL = 1e-5
SIZES = [1, 3, 64, 1000, 4099, 262147]  # empty is covered separately; odd sizes exercise the tails


def both(oracle, hip, name, params, outputs):
    a = run_op(oracle, name, {k: (v.copy() if isinstance(v, np.ndarray) else v) for k, v in params.items()}, outputs)
    b = run_op(hip, name, params, outputs)
    return a, b


def rng(seed):
    return np.random.default_rng(seed)


# ----------------------------------------------------------------------------------------------
# elementwise binary, all broadcasting regimes
# ----------------------------------------------------------------------------------------------
@pytest.mark.parametrize("op", ["add", "sub", "mul", "div"])
@pytest.mark.parametrize("xl,yl", [(1, 1), (1, 777), (777, 1), (4096, 4096), (1001, 1001), (128, 128 * 64), (128 * 64, 128),
                                   (10, 640), (640, 10), (4096, 4096 * 33), (12, 12 * 1000), (300000, 300000),
                                   # periods that are no multiple of four: short and long ones, results that end in a
                                   # partial 16-byte piece, a period of two and of three values
                                   (7, 7 * 1001), (7 * 1001, 7), (3, 3 * 70000), (2, 2 * 5001), (10001, 10001 * 50),
                                   (5, 15), (3, 6), (8193, 8193 * 9)])
def test_binary_ops_bit_exact(oracle, hip, op, xl, yl):
    r = rng(xl * 7919 + yl)
    x = r.standard_normal(xl).astype(np.float32)
    y = (r.standard_normal(yl).astype(np.float32) + np.float32(3.0))  # keep div away from 0
    z = np.zeros(max(xl, yl), np.float32)
    a, b = both(oracle, hip, op, {"x": x, "y": y, "z": z}, ["z"])
    np.testing.assert_array_equal(a["z"], b["z"])


@pytest.mark.parametrize("op", ["add", "mul"])
def test_binary_inplace_alias(oracle, hip, op):
    r = rng(5)
    bias = r.standard_normal(128).astype(np.float32)
    y = r.standard_normal(128 * 64).astype(np.float32)
    # bias add as the Linear layer issues it: x = bias, y = z = activations
    a = run_op(oracle, op, {"x": bias, "y": (yo := y.copy()), "z": yo}, ["z"])
    b = run_op(hip, op, {"x": bias, "y": (yh := y.copy()), "z": yh}, ["z"])
    np.testing.assert_array_equal(a["z"], b["z"])


def test_binary_misaligned_subslices(oracle, hip):
    """Sub-slices taken by pointer arithmetic need not be 16-byte aligned."""
    r = rng(11)
    n = 4096 + 5
    xs, ys = r.standard_normal(n + 3).astype(np.float32), r.standard_normal(n + 3).astype(np.float32)
    res = []
    for dev in (oracle, hip):
        X, Y, Z = dev.from_numpy(xs), dev.from_numpy(ys), dev.from_numpy(np.zeros(n + 3, np.float32))
        dev.dispatch("add", x=X.sub(1, n), y=Y.sub(2, n), z=Z.sub(3, n))
        dev.sync()
        res.append(dev.to_numpy(Z))
    np.testing.assert_array_equal(res[0], res[1])
    assert np.all(res[1][:3] == 0)


def test_binary_rejects_bad_lengths(hip):
    from zigrad_amd import ZgHipError

    X, Y, Z = (hip.from_numpy(np.zeros(n, np.float32)) for n in (3, 7, 7))
    with pytest.raises(ZgHipError, match="do not broadcast"):
        hip.dispatch("add", x=X, y=Y, z=Z)


# ----------------------------------------------------------------------------------------------
# unary forward / backward
# ----------------------------------------------------------------------------------------------
EXACT_UNARY = {"relu_fwd", "relu_bwd", "relu_inplace_bwd", "clamp_fwd", "clamp_bwd", "sqrt_fwd", "sqrt_bwd", "rsqrt_fwd",
               "rsqrt_bwd", "exp_bwd", "tanh_bwd", "tanh_inplace_bwd", "sigm_bwd", "sigm_inplace_bwd"}


def unary_case(name, n, seed):
    r = rng(seed)
    x = r.standard_normal(n).astype(np.float32)
    pos = np.abs(x) + np.float32(0.01)
    g = r.standard_normal(n).astype(np.float32)
    yg = r.standard_normal(n).astype(np.float32)
    z = np.zeros(n, np.float32)
    cases = {
        "pow_fwd": ({"x": pos, "exp": 2.5, "y": z}, ["y"]),
        "pow_bwd": ({"x": pos, "x_g": g, "exp": 2.5, "y_g": yg, "eps": 1e-12}, ["x_g"]),
        "sqrt_fwd": ({"x": pos, "y": z}, ["y"]),
        "sqrt_bwd": ({"x": pos, "x_g": g, "y_g": yg, "eps": 1e-12}, ["x_g"]),
        "rsqrt_fwd": ({"x": pos, "y": z, "eps": 1e-12}, ["y"]),
        "rsqrt_bwd": ({"x": pos, "x_g": g, "y_g": yg, "eps": 1e-12}, ["x_g"]),
        "exp_fwd": ({"x": x, "y": z}, ["y"]),
        "exp_bwd": ({"x_g": g, "y": x, "y_g": yg}, ["x_g"]),
        "relu_fwd": ({"x": x, "y": z}, ["y"]),
        "relu_bwd": ({"x": x, "x_g": g, "y_g": yg}, ["x_g"]),
        "relu_inplace_bwd": ({"x": np.maximum(x, 0), "x_g": g}, ["x_g"]),
        "tanh_fwd": ({"x": x, "y": z}, ["y"]),
        "tanh_bwd": ({"x_g": g, "y": np.tanh(x), "y_g": yg}, ["x_g"]),
        "tanh_inplace_bwd": ({"x": np.tanh(x), "x_g": g}, ["x_g"]),
        "sigm_fwd": ({"x": x, "y": z}, ["y"]),
        "sigm_bwd": ({"x_g": g, "y": x, "y_g": yg}, ["x_g"]),
        "sigm_inplace_bwd": ({"x": x, "x_g": g}, ["x_g"]),
        "clamp_fwd": ({"x": x, "y": z, "min": -0.5, "max": 0.75}, ["y"]),
        "clamp_bwd": ({"x": x, "x_g": g, "y_g": yg, "min": -0.5, "max": 0.75}, ["x_g"]),
    }
    return cases[name]


@pytest.mark.parametrize("name", ["pow_fwd", "pow_bwd", "sqrt_fwd", "sqrt_bwd", "rsqrt_fwd", "rsqrt_bwd", "exp_fwd", "exp_bwd",
                                  "relu_fwd", "relu_bwd", "relu_inplace_bwd", "tanh_fwd", "tanh_bwd", "tanh_inplace_bwd",
                                  "sigm_fwd", "sigm_bwd", "sigm_inplace_bwd", "clamp_fwd", "clamp_bwd"])
@pytest.mark.parametrize("n", SIZES)
def test_unary_ops(oracle, hip, name, n):
    params, outs = unary_case(name, n, n + len(name))
    a, b = both(oracle, hip, name, params, outs)
    for o in outs:
        if name in EXACT_UNARY:
            np.testing.assert_array_equal(a[o], b[o])
        else:
            assert rel_fro(b[o], a[o]) <= TOL


def test_unary_inplace_and_empty(oracle, hip):
    x = rng(3).standard_normal(5000).astype(np.float32)
    a = run_op(oracle, "relu_fwd", {"x": (xo := x.copy()), "y": xo}, ["y"])
    b = run_op(hip, "relu_fwd", {"x": (xh := x.copy()), "y": xh}, ["y"])
    np.testing.assert_array_equal(a["y"], b["y"])
    # zero-length slices are legal and do nothing
    e = hip.mem_alloc(np.float32, 0)
    hip.dispatch("relu_fwd", x=e, y=e)
    hip.dispatch("scale", x=e, alpha=2.0)
    hip.sync()


# ----------------------------------------------------------------------------------------------
# BLAS level 1 style ops and flat reductions
# ----------------------------------------------------------------------------------------------
@pytest.mark.parametrize("n", [1, 5, 1000, 65536, 65537, 131072, 131073, 1 << 20, (1 << 22) + 13])
def test_flat_reductions(oracle, hip, n):
    r = rng(n)
    x = r.standard_normal(n).astype(np.float32)
    y = r.standard_normal(n).astype(np.float32)
    one = np.zeros(1, np.float32)
    x64, y64 = x.astype(np.float64), y.astype(np.float64)
    truth = {"sum": np.abs(x64).sum(), "nrm2": np.sqrt((x64 * x64).sum()), "dot": (x64 * y64).sum()}
    for name, params, out in [("sum", {"x": x, "y": one}, "y"), ("nrm2", {"x": x, "y": one}, "y"),
                              ("dot", {"x": x, "y": y, "z": one}, "z")]:
        a, b = both(oracle, hip, name, params, [out])
        # both sides against the fp64 value: the summation orders differ, the answers may not
        scale = max(abs(truth[name]), np.sqrt(n))
        assert abs(float(b[out][0]) - truth[name]) <= 2e-6 * scale + 1e-6, name
        assert abs(float(a[out][0]) - truth[name]) <= 1e-4 * scale + 1e-6, name
    # max_fwd picks one element: bit-exact
    a, b = both(oracle, hip, "max_fwd", {"x": x, "y": one}, ["y"])
    assert a["y"][0] == b["y"][0]
    # sum_along with a one-element output is the flat sum of the signed values, with alpha/beta
    yb = np.asarray([2.0], np.float32)
    a, b = both(oracle, hip, "sum_along", {"x": x, "x_shape": [n], "y": yb, "dim": 0, "alpha": 0.5, "beta": 2.0}, ["y"])
    assert abs(float(b["y"][0]) - (0.5 * x64.sum() + 4.0)) <= 2e-6 * np.sqrt(n) + 1e-5


def test_max_fwd_ties_and_bwd(oracle, hip):
    x = np.asarray([1, -9, 9, 3, -9], np.float32)
    one = np.zeros(1, np.float32)
    a, b = both(oracle, hip, "max_fwd", {"x": x, "y": one}, ["y"])
    assert a["y"][0] == b["y"][0] == -9
    g = np.zeros(5, np.float32)
    a, b = both(oracle, hip, "max_bwd", {"x": x, "x_g": g, "y": np.asarray([-9], np.float32),
                                         "y_g": np.asarray([2.5], np.float32)}, ["x_g"])
    np.testing.assert_array_equal(a["x_g"], b["x_g"])
    np.testing.assert_array_equal(b["x_g"], np.asarray([0, 2.5, 0, 0, 2.5], np.float32))


@pytest.mark.parametrize("n", [7, 4096, 100003, 1 << 21])
def test_axpy_scale_clip(oracle, hip, n):
    r = rng(n + 1)
    x = r.standard_normal(n).astype(np.float32)
    y = r.standard_normal(n).astype(np.float32)
    a, b = both(oracle, hip, "axpy", {"x": x, "y": y, "alpha": -0.01}, ["y"])
    np.testing.assert_array_equal(a["y"], b["y"])
    a, b = both(oracle, hip, "scale", {"x": x, "alpha": 0.37}, ["x"])
    np.testing.assert_array_equal(a["x"], b["x"])
    # clip: the norm differs in the last bits between BLAS and the tree sum, so compare to tolerance
    for max_norm in (0.5, 1e9):
        a, b = both(oracle, hip, "clip_nrm2", {"x": x, "max_norm": max_norm, "delta": 1e-6}, ["x"])
        assert rel_fro(b["x"], a["x"]) <= TOL
    # device-resident alpha (dot backward)
    res = []
    for dev in (oracle, hip):
        X, Y, A = dev.from_numpy(x), dev.from_numpy(y), dev.from_numpy(np.asarray([1.5], np.float32))
        dev.dispatch("axpy", x=X, y=Y, alpha=A)
        dev.sync()
        res.append(dev.to_numpy(Y))
    np.testing.assert_array_equal(res[0], res[1])


# ----------------------------------------------------------------------------------------------
# reductions along an axis, argmax, unbroadcast
# ----------------------------------------------------------------------------------------------
AXIS_SHAPES = [([64, 10], 1), ([64, 10], 0), ([64, 2], 1), ([2708, 16], 0), ([1000, 4096], 1), ([1000, 4096], 0),
               ([33, 1001], 1), ([33, 1001], 0), ([6, 50, 7], 1), ([3, 4, 5, 6], 2), ([2, 3, 4], 0), ([4, 20000], 1),
               ([5, 70000], 1), ([70000, 3], 0), ([1, 5, 8], 1),
               # few long rows, cut into segments and combined in a second launch: a single row, a row length that is
               # no multiple of four, rows that end inside a segment, a reduced first axis of a vector
               ([1, 300000], 1), ([3, 262145], 1), ([7, 140002], 1), ([64, 16384], 1), ([100, 20000], 1), ([300000], 0),
               ([300, 16388], 1), ([2, 3, 140000], 2),
               # rows whose last trip of loads is partial
               ([700, 1000], 1), ([300, 1028], 1), ([900, 260], 1), ([50, 2044], 1),
               # tall matrices of one column group: 128 chunks of rows from 64 MiB, 256 from 256 MiB
               ([262149, 64], 0), ([65541, 256], 0), ([1048581, 68], 0),
               # rows that start off a 16-byte boundary and are read in 16-byte pieces between a head and a tail
               ([600, 2051], 1), ([50, 4099], 1), ([9, 33001], 1), ([700, 513], 1), ([5, 300001], 1), ([2, 1000003], 1),
               # short rows on one, two, four and eight lanes, with and without heads and tails
               ([5000, 1], 1), ([5000, 3], 1), ([3000, 9], 1), ([3000, 11], 1), ([3000, 12], 1), ([2000, 17], 1),
               ([2000, 30], 1), ([1500, 35], 1), ([1500, 61], 1), ([1000, 70], 1), ([1000, 130], 1), ([700, 255], 1)]


@pytest.mark.parametrize("shape,dim", AXIS_SHAPES)
def test_sum_max_argmax_along(oracle, hip, shape, dim):
    r = rng(sum(shape) + dim)
    n = int(np.prod(shape))
    x = r.standard_normal(n).astype(np.float32)
    out_n = n // shape[dim]
    x64 = x.astype(np.float64).reshape(shape)
    y0 = r.standard_normal(out_n).astype(np.float32)
    a, b = both(oracle, hip, "sum_along", {"x": x, "x_shape": shape, "y": y0, "dim": dim, "alpha": 1.0, "beta": 1.0}, ["y"])
    truth = x64.sum(axis=dim).ravel() + y0
    # the host's running float sum over a million terms drifts further from the exact sum than 1e-5 (1.6e-5 measured);
    # the device's partial sums stay at 4e-7
    tol_host = TOL if shape[dim] <= (1 << 19) else 1e-4
    assert rel_fro(b["y"], truth) <= TOL and rel_fro(a["y"], truth) <= tol_host
    if out_n > 1:
        a, b = both(oracle, hip, "sum_along", {"x": x, "x_shape": shape, "y": np.full(out_n, 7.0, np.float32), "dim": dim}, ["y"])
        assert rel_fro(b["y"], x64.sum(axis=dim).ravel()) <= TOL
    a, b = both(oracle, hip, "max_along", {"x": x, "x_shape": shape, "y": np.zeros(out_n, np.float32), "dim": dim}, ["y"])
    np.testing.assert_array_equal(a["y"], b["y"])
    a, b = both(oracle, hip, "argmax_along", {"x": x, "x_shape": shape, "y": np.zeros(out_n, np.uint64), "dim": dim}, ["y"])
    np.testing.assert_array_equal(a["y"], b["y"])
    np.testing.assert_array_equal(b["y"], np.argmax(x.reshape(shape), axis=dim).ravel().astype(np.uint64))


def test_argmax_ties_across_the_segments_of_a_long_row_take_the_first(oracle, hip):
    cols = 200_000
    x = np.zeros((3, cols), np.float32)
    x[0, [5000, 70000, 199999]] = 2.0      # equal maxima in three segments
    x[1, [150000, 150001]] = 1.0
    x[2, :] = -np.inf                       # nothing to find: the host loop answers 0
    a, b = both(oracle, hip, "argmax_along", {"x": x.ravel(), "x_shape": [3, cols], "y": np.zeros(3, np.uint64), "dim": 1}, ["y"])
    np.testing.assert_array_equal(a["y"], b["y"])
    np.testing.assert_array_equal(b["y"], np.asarray([5000, 150000, 0], np.uint64))
    a, b = both(oracle, hip, "max_along", {"x": x.ravel(), "x_shape": [3, cols], "y": np.zeros(3, np.float32), "dim": 1}, ["y"])
    np.testing.assert_array_equal(a["y"], b["y"])
    # integer values: the sum is exact in any order, with alpha and beta applied once
    xi = rng(5).integers(-4, 5, (5, 131075)).astype(np.float32)
    y0 = np.arange(5, dtype=np.float32)
    out = run_op(hip, "sum_along", {"x": xi.ravel(), "x_shape": [5, 131075], "y": y0.copy(), "dim": 1, "alpha": 2.0, "beta": -1.0},
                 ["y"])["y"]
    np.testing.assert_array_equal(out, 2.0 * xi.astype(np.float64).sum(axis=1) - y0)


def test_argmax_ties_take_first(oracle, hip):
    x = np.zeros((8, 300), np.float32)
    x[:, 17] = 5
    x[:, 250] = 5
    x[3, :] = -np.inf
    a, b = both(oracle, hip, "argmax_along", {"x": x.ravel(), "x_shape": [8, 300], "y": np.zeros(8, np.uint64), "dim": 1}, ["y"])
    np.testing.assert_array_equal(a["y"], b["y"])
    assert b["y"][0] == 17 and b["y"][3] == 0
    a, b = both(oracle, hip, "argmax_along", {"x": x.ravel(), "x_shape": [8, 300], "y": np.zeros(300, np.uint64), "dim": 0}, ["y"])
    np.testing.assert_array_equal(a["y"], b["y"])


@pytest.mark.parametrize("xs,ys", [([64, 128], [128]), ([4096, 1024], [1024]), ([2, 3, 3], [3]), ([2, 3, 3], [2, 1, 3]),
                                   ([5, 7], [5, 7]), ([6, 4, 10], [4, 10]), ([3, 5, 1000], [3, 1, 1000]), ([64, 10], [10]),
                                   ([1, 64, 10], [10]), ([8, 6, 33], [1, 6, 33])])
@pytest.mark.parametrize("alpha,beta", [(1.0, 1.0), (1.0, 0.0), (-1.0, 1.0)])
def test_unbroadcast(oracle, hip, xs, ys, alpha, beta):
    from zigrad_amd import host

    r = rng(sum(xs) * 31 + len(ys))
    x = r.standard_normal(int(np.prod(xs))).astype(np.float32)
    y0 = r.standard_normal(int(np.prod(ys))).astype(np.float32)
    res = []
    for dev in (oracle, hip):
        X, Y = dev.from_numpy(x), dev.from_numpy(y0)
        host.unbroadcast_(dev, X, xs, Y, ys, alpha=alpha, beta=beta)
        dev.sync()
        res.append(dev.to_numpy(Y))
    assert rel_fro(res[1], res[0]) <= TOL
    # closed form: sum over the broadcast axes
    x64 = x.astype(np.float64).reshape(xs)
    ys_full = [1] * (len(xs) - len(ys)) + list(ys)
    axes = tuple(i for i, (a, b) in enumerate(zip(xs, ys_full)) if a != b)
    truth = alpha * x64.sum(axis=axes).ravel() + beta * y0 if axes else alpha * x64.ravel() + beta * y0
    assert rel_fro(res[1], truth) <= TOL


def test_broadcast_op(oracle, hip):
    r = rng(8)
    x = r.standard_normal(12).astype(np.float32)
    for n in (12, 12 * 50):
        y = r.standard_normal(n).astype(np.float32)
        a, b = both(oracle, hip, "broadcast", {"x": x, "y": y, "alpha": 0.5, "beta": 2.0}, ["y"])
        np.testing.assert_array_equal(a["y"], b["y"])
    # short operands of any length against results that end in a partial 16-byte piece or not
    for xl, reps in ((7, 1001), (3, 70000), (2, 5001), (10001, 50), (5, 3), (16, 4096), (1, 4097)):
        x = r.standard_normal(xl).astype(np.float32)
        y = r.standard_normal(xl * reps).astype(np.float32)
        for alpha, beta in ((0.5, 2.0), (1.0, 0.0)):
            a, b = both(oracle, hip, "broadcast", {"x": x, "y": y, "alpha": alpha, "beta": beta}, ["y"])
            np.testing.assert_array_equal(a["y"], b["y"])


# ----------------------------------------------------------------------------------------------
# memory-style ops
# ----------------------------------------------------------------------------------------------
def test_mem_ops(oracle, hip):
    for n in (1, 5, 4096, 100001):
        B = hip.mem_alloc(np.float32, n)
        hip.mem_fill(B, 3.25)
        assert np.all(hip.to_numpy(B) == np.float32(3.25))
        hip.mem_sequence(B, 2.0, 3.0)
        Bo = oracle.mem_alloc(np.float32, n)
        oracle.mem_sequence(Bo, 2.0, 3.0)
        np.testing.assert_array_equal(hip.to_numpy(B), oracle.to_numpy(Bo))  # integer-valued steps are exact
        for kind, fan in (("uniform", 0), ("normal", 0), ("kaiming", 784)):
            hip.mem_random(B, kind, seed=81761, fan=fan)
            oracle.mem_random(Bo, kind, seed=81761, fan=fan)
            np.testing.assert_array_equal(hip.to_numpy(B), oracle.to_numpy(Bo))
        C = hip.mem_dupe(B)
        np.testing.assert_array_equal(hip.to_numpy(B), hip.to_numpy(C))
        hip.mem_free(B)
        hip.mem_free(C)
    u = hip.mem_alloc(np.uint64, 10)
    hip.mem_fill(u, 7)
    assert np.all(hip.to_numpy(u) == 7)
    m = hip.mem_alloc_byte_mask(17)
    assert m.n == 3
    hip.mem_fill(m, 0xFF)
    assert np.all(hip.to_numpy(m) == 0xFF)


def test_mem_take_and_transfer(oracle, hip):
    r = rng(2)
    src = r.standard_normal(5000).astype(np.float32)
    idx = r.integers(0, 5000, 12345).astype(np.uint64)
    S, I = hip.from_numpy(src), hip.from_numpy(idx)
    D = hip.mem_alloc(np.float32, idx.size)
    hip.mem_take(S, I, D)
    np.testing.assert_array_equal(hip.to_numpy(D), src[idx])
    # indices in pinned host memory work as well (the reference fills index slices on the host)
    H = hip.mem_alloc_host(np.uint64, idx.size)
    hip.mem_transfer(idx, H, "HtoD")
    hip.mem_fill(D, 0.0)
    hip.mem_take(S, H, D)
    np.testing.assert_array_equal(hip.to_numpy(D), src[idx])
    out = np.empty(5000, np.float32)
    hip.mem_transfer(S, out, "DtoH")
    np.testing.assert_array_equal(out, src)


def test_caching_allocator(hip):
    st0 = hip.cache_stats()
    a = hip.mem_cache_alloc(np.float32, 1000)
    b = hip.mem_cache_alloc(np.float32, 3 << 20)
    z = hip.mem_cache_alloc(np.float32, 0)
    assert z.ptr == 0 and z.block == 0
    hip.mem_cache_free(z)
    assert a.ptr % 256 == 0 and b.ptr % 256 == 0
    hip.mem_fill(a, 1.0)
    hip.mem_fill(b, 2.0)
    assert hip.to_numpy(a).sum() == 1000
    pa, pb = a.ptr, b.ptr
    hip.mem_cache_free(a)
    hip.mem_cache_free(b)
    st1 = hip.cache_stats()
    assert st1["bytes_in_use"] == st0["bytes_in_use"]
    # steady state: the same requests are served from the pools without new device allocations
    for _ in range(50):
        a = hip.mem_cache_alloc(np.float32, 1000)
        b = hip.mem_cache_alloc(np.float32, 3 << 20)
        assert (a.ptr, b.ptr) == (pa, pb)
        hip.mem_cache_free(a)
        hip.mem_cache_free(b)
    assert hip.cache_stats()["n_device_allocs"] == st1["n_device_allocs"]
    # neighbours fuse again: after freeing everything one block of the whole size fits
    blocks = [hip.mem_cache_alloc(np.float32, 4096) for _ in range(64)]
    for blk in blocks[::2] + blocks[1::2]:
        hip.mem_cache_free(blk)
    big = hip.mem_cache_alloc(np.float32, 4096 * 60)
    hip.mem_cache_free(big)
    assert hip.cache_stats()["n_device_allocs"] == st1["n_device_allocs"]
    s1 = hip.mem_scratch(np.float32, 100)
    s2 = hip.mem_scratch(np.float32, 50)
    assert s1.ptr == s2.ptr
    from zigrad_amd import ZgHipError

    with pytest.raises(ZgHipError):
        hip._call("zg_hip_mem_cache_free", 12345, 1)
