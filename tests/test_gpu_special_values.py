"""NaN, infinities, signed zeros, subnormals and values at the edge of the float range through every elementwise op,
the reductions and the losses: the HIP device must propagate them exactly as the host's loops do (the oracle,
src/device/host_device.zig): the same NaN positions, the same infinities, finite values bit-equal for the ops built
from IEEE +, -, x, /, sqrt and compares, within 2e-6 for the transcendental ones."""
from __future__ import annotations

import numpy as np
import pytest

from conftest import run_op

pytestmark = pytest.mark.gpu

SPECIAL = np.array([np.nan, np.inf, -np.inf, 0.0, -0.0, 1e-42, -1e-42, 1e38, -1e38, 3.4e38, 1.0, -1.0, 88.8, -104.0, 1e-30,
                    0.5], np.float32)
N = len(SPECIAL)


def _same(a, b, exact, tol=2e-6):
    a, b = np.asarray(a).ravel(), np.asarray(b).ravel()
    if not np.array_equal(np.isnan(a), np.isnan(b)):
        return False
    ok = ~np.isnan(a)
    if exact:
        return np.array_equal(a[ok].view(np.uint32), b[ok].view(np.uint32))     # also tells -0.0 from 0.0
    if not np.array_equal(np.isinf(a[ok]), np.isinf(b[ok])):
        return False
    inf = np.isinf(a[ok])
    return np.array_equal(a[ok][inf], b[ok][inf]) and np.allclose(a[ok][~inf], b[ok][~inf], rtol=tol, atol=1e-37)


def _both(oracle, hip, name, params, outs):
    def cp():
        return {k: (v.copy() if isinstance(v, np.ndarray) else v) for k, v in params.items()}
    return run_op(oracle, name, cp(), outs), run_op(hip, name, cp(), outs)


@pytest.mark.parametrize("op", ["add", "sub", "mul", "div"])
def test_binary_ops_on_every_pair_of_special_values(oracle, hip, op):
    X, Y = np.meshgrid(SPECIAL, SPECIAL)
    x, y = X.ravel().copy(), Y.ravel().copy()
    want, got = _both(oracle, hip, op, dict(x=x, y=y, z=np.zeros_like(x)), ["z"])
    assert _same(want["z"], got["z"], exact=True)
    for s in SPECIAL:       # one-float operands, in device memory and by value, on either side
        for params in (dict(x=np.full(1, s, np.float32), y=SPECIAL.copy(), z=np.zeros(N, np.float32)),
                       dict(x=SPECIAL.copy(), y=np.full(1, s, np.float32), z=np.zeros(N, np.float32)),
                       dict(x=float(s), y=SPECIAL.copy(), z=np.zeros(N, np.float32)),
                       dict(x=SPECIAL.copy(), y=float(s), z=np.zeros(N, np.float32))):
            want, got = _both(oracle, hip, op, params, ["z"])
            assert _same(want["z"], got["z"], exact=True), (op, s)


G, XG = np.full(N, 0.75, np.float32), np.full(N, 0.25, np.float32)
UNARY = [
    ("relu_fwd", dict(x=SPECIAL, y=np.zeros(N, np.float32)), "y", True),
    ("tanh_fwd", dict(x=SPECIAL, y=np.zeros(N, np.float32)), "y", False),
    ("sigm_fwd", dict(x=SPECIAL, y=np.zeros(N, np.float32)), "y", False),
    ("exp_fwd", dict(x=SPECIAL, y=np.zeros(N, np.float32)), "y", False),
    ("sqrt_fwd", dict(x=SPECIAL, y=np.zeros(N, np.float32)), "y", True),
    ("rsqrt_fwd", dict(x=SPECIAL, y=np.zeros(N, np.float32), eps=1e-6), "y", True),
    ("pow_fwd", dict(x=SPECIAL, exp=2.0, y=np.zeros(N, np.float32)), "y", False),
    ("pow_fwd", dict(x=SPECIAL, exp=0.5, y=np.zeros(N, np.float32)), "y", False),
    ("pow_fwd", dict(x=SPECIAL, exp=-1.0, y=np.zeros(N, np.float32)), "y", False),
    ("clamp_fwd", dict(x=SPECIAL, y=np.zeros(N, np.float32), min=-1.0, max=1.0), "y", True),
    ("relu_bwd", dict(x=SPECIAL, x_g=XG, y_g=G), "x_g", True),
    ("relu_inplace_bwd", dict(x=SPECIAL, x_g=XG), "x_g", True),
    ("tanh_bwd", dict(x_g=XG, y=SPECIAL, y_g=G), "x_g", True),
    ("tanh_inplace_bwd", dict(x=SPECIAL, x_g=XG), "x_g", True),
    ("sigm_bwd", dict(x_g=XG, y=SPECIAL, y_g=G), "x_g", True),
    ("sigm_inplace_bwd", dict(x=SPECIAL, x_g=XG), "x_g", True),
    ("exp_bwd", dict(x_g=XG, y=SPECIAL, y_g=G), "x_g", True),
    ("sqrt_bwd", dict(x=SPECIAL, x_g=XG, y_g=G, eps=1e-6), "x_g", True),
    ("rsqrt_bwd", dict(x=SPECIAL, x_g=XG, y_g=G, eps=1e-6), "x_g", True),
    ("pow_bwd", dict(x=SPECIAL, x_g=XG, exp=2.0, y_g=G, eps=1e-6), "x_g", False),
    ("clamp_bwd", dict(x=SPECIAL, x_g=XG, y_g=G, min=-1.0, max=1.0), "x_g", True),
    ("relu_bwd", dict(x=np.ones(N, np.float32), x_g=XG, y_g=SPECIAL), "x_g", True),      # specials as the gradient
    ("smooth_l1_bwd", dict(pred=SPECIAL, target=np.zeros(N, np.float32), grad=np.zeros(N, np.float32), beta=1.0), "grad", True),
    ("mse_bwd", dict(pred=SPECIAL, target=np.zeros(N, np.float32), grad=np.zeros(N, np.float32)), "grad", True),
    ("scale", dict(x=SPECIAL, alpha=0.0), "x", True),
    ("scale", dict(x=SPECIAL, alpha=-2.0), "x", True),
]


@pytest.mark.parametrize("i", range(len(UNARY)))
def test_unary_ops_and_their_backward_passes_on_special_values(oracle, hip, i):
    name, params, out, exact = UNARY[i]
    want, got = _both(oracle, hip, name, params, [out])
    assert _same(want[out], got[out], exact), (name, want[out], got[out])


FIN = np.array([1.0, -2.0, 0.5, -0.0, 0.0, 3.0, 1e-42, -7.0], np.float32)
ROWS = np.stack([FIN, np.where(np.arange(8) == 2, np.nan, FIN), np.where(np.arange(8) == 5, np.inf, FIN),
                 np.where(np.arange(8) == 1, -np.inf, FIN), np.full(8, -np.inf), np.full(8, np.nan),
                 np.where(np.arange(8) % 2 == 0, np.inf, -np.inf), np.full(8, -0.0)]).astype(np.float32)


def test_reductions_along_rows_and_columns_of_special_values(oracle, hip):
    R, C = ROWS.shape
    for name, y_len, dim, exact in (("sum_along", R, 1, False), ("sum_along", C, 0, False), ("max_along", R, 1, True),
                                    ("max_along", C, 0, True)):
        p = dict(x=ROWS.ravel(), x_shape=[R, C], y=np.zeros(y_len, np.float32), dim=dim)
        if name == "sum_along":
            p.update(alpha=1.0, beta=0.0)
        want, got = _both(oracle, hip, name, p, ["y"])
        assert _same(want["y"], got["y"], exact), (name, dim, want["y"], got["y"])
    arg = []
    for dev in (oracle, hip):       # the first maximum; a NaN is never greater than anything
        b, o = dev.from_numpy(ROWS.ravel()), dev.from_numpy(np.zeros(R, np.uint64))
        dev.dispatch("argmax_along", x=b, x_shape=[R, C], y=o, dim=1)
        dev.sync()
        arg.append(dev.to_numpy(o))
        dev.mem_free(b)
        dev.mem_free(o)
    np.testing.assert_array_equal(arg[0], arg[1])
    for i in range(R):
        for op in ("sum", "nrm2"):
            want, got = _both(oracle, hip, op, dict(x=ROWS[i], y=np.zeros(1, np.float32)), ["y"])
            assert _same(want["y"], got["y"], exact=False), (op, ROWS[i], want["y"], got["y"])
        want, got = _both(oracle, hip, "dot", dict(x=ROWS[i], y=ROWS[(i + 1) % R], z=np.zeros(1, np.float32)), ["z"])
        assert _same(want["z"], got["z"], exact=False)


def test_the_element_of_largest_magnitude_with_nans_and_infinities(oracle, hip):
    """cblas_isamax on NaNs is the BLAS library's business; the one the reference names (mkl_rt) documents that the
    first NaN wins, and so do the kernel and the oracle's own loop."""
    oracle.force_builtin_blas(True)
    try:
        for i, row in enumerate(ROWS):
            want, got = _both(oracle, hip, "max_fwd", dict(x=row, y=np.zeros(1, np.float32)), ["y"])
            assert _same(want["y"], got["y"], exact=True), (row, want["y"], got["y"])
            if np.isnan(row).any():
                assert np.isnan(got["y"][0])
        # far enough apart for the two-stage form, the NaN in the second half, an infinity before it
        x = np.ones(300_000, np.float32)
        x[1000], x[200_000] = -np.inf, np.nan
        got = run_op(hip, "max_fwd", dict(x=x, y=np.zeros(1, np.float32)), ["y"])["y"]
        assert np.isnan(got[0])
        x[200_000] = 2.0
        got = run_op(hip, "max_fwd", dict(x=x, y=np.zeros(1, np.float32)), ["y"])["y"]
        assert got[0] == -np.inf
    finally:
        oracle.force_builtin_blas(False)


def test_softmax_and_the_losses_on_special_values(oracle, hip):
    R, C = ROWS.shape
    want, got = _both(oracle, hip, "softmax_fwd", dict(x=ROWS.ravel(), y=np.zeros(R * C, np.float32), rows=R, cols=C), ["y"])
    assert _same(want["y"], got["y"], exact=False)
    t = np.zeros((R, C), np.float32)
    t[:, 0] = 1
    p = dict(logits=ROWS.ravel(), target=t.ravel(), probs=np.zeros(R * C, np.float32), loss=np.zeros(1, np.float32), rows=R,
             cols=C)
    want, got = _both(oracle, hip, "smce_fwd", p, ["probs", "loss"])
    assert _same(want["probs"], got["probs"], exact=False) and _same(want["loss"], got["loss"], exact=False)
    finite = ROWS[[0, 7]]       # the rows without NaN or infinity: loss and gradient as usual beside rows that have them
    p = dict(logits=finite.ravel(), target=t[:2].ravel(), probs=np.zeros(2 * C, np.float32), loss=np.zeros(1, np.float32),
             rows=2, cols=C)
    want, got = _both(oracle, hip, "smce_fwd", p, ["probs", "loss"])
    assert np.isfinite(got["loss"][0]) and _same(want["loss"], got["loss"], exact=False)
    want, got = _both(oracle, hip, "smooth_l1_fwd", dict(pred=SPECIAL, target=np.zeros(N, np.float32), beta=1.0,
                                                          loss=np.zeros(1, np.float32)), ["loss"])
    assert _same(want["loss"], got["loss"], exact=False)
