"""Known-answer checks taken from the reference's own unit tests (tests/golden/reference_vectors.json).

Each check takes a device object (the CPU oracle or the HIP device) and asserts the reference's expected
values.  The oracle must pass these before it is trusted as the checker for the HIP kernels.
"""
from __future__ import annotations

import json
from pathlib import Path

import numpy as np

from conftest import run_op
from zigrad_amd import host
from zigrad_amd.device import F32, U64

G = json.loads((Path(__file__).parent / "golden" / "reference_vectors.json").read_text())


def f32(x):
    return np.asarray(x, dtype=np.float32)


def check_clip_nrm2(dev):
    c = G["clip_nrm2"]
    x = f32(c["x"])
    out = run_op(dev, "nrm2", {"x": x, "y": np.zeros(1, np.float32)}, ["y"])
    assert out["y"][0] == np.float32(c["norm"])
    out = run_op(dev, "clip_nrm2", {"x": x.copy(), "max_norm": c["max_norm"], "delta": c["delta"]}, ["x"])
    np.testing.assert_allclose(out["x"], x * c["expected_scale"], atol=c["abs_tol"])
    # below the threshold nothing changes
    out = run_op(dev, "clip_nrm2", {"x": x.copy(), "max_norm": 10.0, "delta": c["delta"]}, ["x"])
    np.testing.assert_array_equal(out["x"], x)


def check_clamp(dev):
    c = G["clamp_inplace"]
    x = f32(c["x"])
    out = run_op(dev, "clamp_fwd", {"x": x, "y": x, "min": float(c["min"]), "max": float(c["max"])}, ["y"])
    np.testing.assert_array_equal(out["y"], f32(c["expected"]))
    c = G["clamp_fwd_bwd"]
    x = f32(c["x"])
    out = run_op(dev, "clamp_fwd", {"x": x, "y": np.zeros_like(x), "min": c["min"], "max": c["max"]}, ["y"])
    np.testing.assert_array_equal(out["y"], f32(c["expected_output"]))
    out = run_op(dev, "clamp_bwd", {"x": x, "x_g": np.zeros_like(x), "y_g": np.ones_like(x), "min": c["min"],
                                    "max": c["max"]}, ["x_g"])
    np.testing.assert_array_equal(out["x_g"], f32(c["expected_grad"]))


def check_add_sub_scalar(dev):
    for c in G["add_sub_scalar"]["cases"]:
        x, y = f32(c["x"]), f32(c["y"])
        z = np.zeros(max(x.size, y.size), np.float32)
        out = run_op(dev, c["op"], {"x": x, "y": y, "z": z}, ["z"])
        np.testing.assert_array_equal(out["z"], f32(c["expected"]))


def check_dot(dev):
    c = G["dot"]
    out = run_op(dev, "dot", {"x": f32(c["x"]), "y": f32(c["y"]), "z": np.zeros(1, np.float32)}, ["z"])
    assert out["z"][0] == c["expected"]


def check_bmm(dev):
    for c in G["bmm"]["cases"]:
        A, B = dev.from_numpy(f32(c["A"])), dev.from_numpy(f32(c["B"]))
        n_out = int(np.prod(c["C_shape"]))
        C = dev.from_numpy(np.full(n_out, np.nan, np.float32))  # beta = 0 must not read C
        shape = host.bmm_acc_(dev, A, c["A_shape"], B, c["B_shape"], C)
        dev.sync()
        assert shape == c["C_shape"]
        np.testing.assert_array_equal(dev.to_numpy(C), f32(c["expected"]))
        for b in (A, B, C):
            dev.mem_free(b)
    c = G["bmm_acc_alpha_beta"]
    A, B, C = (dev.from_numpy(f32(c[k])) for k in ("A", "B", "C"))
    host.bmm_acc_(dev, A, c["shape"], B, c["shape"], C, alpha=c["alpha"], beta=c["beta"])
    dev.sync()
    np.testing.assert_array_equal(dev.to_numpy(C), f32(c["expected"]))


def check_matvec(dev):
    c = G["matvec"]
    out = run_op(dev, "matvec", {"A": f32(c["A"]), "x": f32(c["x"]), "y": np.full(2, np.nan, np.float32), "m": c["m"],
                                 "n": c["n"], "trans_a": False, "alpha": 1.0, "beta": 0.0}, ["y"])
    np.testing.assert_array_equal(out["y"], f32(c["expected"]))


def check_sum_max_along(dev):
    c = G["sum_along"]
    # beta = 0 with a finite, arbitrary y: the reference computes alpha*s + beta*y on the uninitialised output
    # (src/device/reduce.zig:119,126), so y must not influence the result
    out = run_op(dev, "sum_along", {"x": f32(c["x"]), "x_shape": c["shape"], "y": np.full(2, 123.0, np.float32),
                                    "dim": c["dim"]}, ["y"])
    np.testing.assert_array_equal(out["y"], f32(c["expected"]))
    m = G["max_along"]
    x = np.arange(1, 25, dtype=np.float32)
    for c in m["cases"]:
        y = np.zeros(len(c["expected"]), np.float32)
        out = run_op(dev, "max_along", {"x": x, "x_shape": m["shape"], "y": y, "dim": c["dim"]}, ["y"])
        np.testing.assert_array_equal(out["y"], f32(c["expected"]))
        # argmax: first index of the maximum; for an increasing arange that is the last position
        ya = np.zeros(len(c["expected"]), np.uint64)
        out = run_op(dev, "argmax_along", {"x": x, "x_shape": m["shape"], "y": ya, "dim": c["dim"]}, ["y"])
        np.testing.assert_array_equal(out["y"], np.full(ya.shape, m["shape"][c["dim"]] - 1, np.uint64))


def check_gather(dev):
    c = G["gather"]
    src = dev.from_numpy(f32(c["input"]))
    idx = dev.from_numpy(np.asarray(c["index"], np.uint64))
    vals, offs = host.gather(dev, src, c["input_shape"], idx, c["index_shape"], c["dim"], return_offsets=True)
    dev.sync()
    np.testing.assert_array_equal(dev.to_numpy(vals), f32(c["expected"]))
    np.testing.assert_array_equal(dev.to_numpy(offs), np.asarray([0, 1, 4, 5, 6, 8], np.uint64))
    # out-of-range index -> IndexOutOfBounds
    bad = dev.from_numpy(np.asarray([3, 1, 1, 2, 0, 2], np.uint64))
    try:
        host.gather(dev, src, c["input_shape"], bad, c["index_shape"], c["dim"])
    except IndexError:
        pass
    else:
        raise AssertionError("expected IndexOutOfBounds")


def check_sum(dev):
    c = G["sum"]
    out = run_op(dev, "sum", {"x": f32(c["x"]), "y": np.zeros(1, np.float32)}, ["y"])
    assert out["y"][0] == c["expected"]
    # documented quirk: the op is cblas_sasum, the sum of absolute values
    out = run_op(dev, "sum", {"x": f32([1, -2, 3, -4]), "y": np.zeros(1, np.float32)}, ["y"])
    assert out["y"][0] == 10
    # max_fwd is x[isamax(x)]: the element of largest magnitude, first one on ties
    out = run_op(dev, "max_fwd", {"x": f32([1, -7, 3, 7]), "y": np.zeros(1, np.float32)}, ["y"])
    assert out["y"][0] == -7


def check_add_broadcast_grad(dev):
    c = G["add_broadcast_grad"]
    t1 = f32(c["t1"])
    for case in c["cases"]:
        t2 = f32(case["t2"])
        out = run_op(dev, "add", {"x": t1, "y": t2, "z": np.zeros_like(t1)}, ["z"])
        np.testing.assert_array_equal(out["z"], f32(c["expected_sum"]))
        # backward of add: unbroadcast the all-ones output grad into t2.grad (alpha = beta = 1, grad starts at 0)
        g_out = dev.from_numpy(np.ones_like(t1))
        g_t2 = dev.from_numpy(np.zeros_like(t2))
        host.unbroadcast_(dev, g_out, c["t1_shape"], g_t2, case["t2_shape"], alpha=1.0, beta=1.0)
        dev.sync()
        np.testing.assert_array_equal(dev.to_numpy(g_t2), f32(case["t2_grad"]))


def _matmul_backward_case(dev, t1, s1, t2, s2, ta, tb, g1, g2):
    A, B = dev.from_numpy(f32(t1)), dev.from_numpy(f32(t2))
    c_shape = host.bmm_out_shape(s1, s2, ta, tb)
    n_c = int(np.prod(c_shape))
    C = dev.from_numpy(np.full(n_c, np.nan, np.float32))
    host.bmm_acc_(dev, A, s1, B, s2, C, ta, tb)
    Cg = dev.from_numpy(np.ones(n_c, np.float32))
    Ag, Bg = dev.from_numpy(np.zeros(len(t1), np.float32)), dev.from_numpy(np.zeros(len(t2), np.float32))
    host.bmm_acc_backward(dev, ta, tb, A, s1, B, s2, Cg, c_shape, Ag, Bg)
    dev.sync()
    np.testing.assert_array_equal(dev.to_numpy(Ag), f32(g1))
    np.testing.assert_array_equal(dev.to_numpy(Bg), f32(g2))


def check_matmul_backward(dev):
    c = G["matmul_backward_square"]
    for case in c["cases"]:
        _matmul_backward_case(dev, c["t1"], c["shape"], c["t2"], c["shape"], case["trans_a"], case["trans_b"],
                              case["grad_t1"], case["grad_t2"])
    for case in G["matmul_backward_nonsquare"]["cases"]:
        _matmul_backward_case(dev, case["t1"], case["t1_shape"], case["t2"], case["t2_shape"], case["trans_a"],
                              case["trans_b"], case["grad_t1"], case["grad_t2"])


def check_pow_sqrt(dev):
    c = G["pow"]
    x = f32(c["x"])
    out = run_op(dev, "pow_fwd", {"x": x, "exp": float(c["exp"]), "y": np.zeros_like(x)}, ["y"])
    np.testing.assert_array_equal(out["y"], f32(c["expected"]))
    out = run_op(dev, "pow_bwd", {"x": x, "x_g": np.zeros_like(x), "exp": float(c["exp"]), "y_g": np.ones_like(x),
                                  "eps": 1e-12}, ["x_g"])
    np.testing.assert_array_equal(out["x_g"], f32(c["grad"]))
    c = G["sqrt"]
    x = f32(c["x"])
    out = run_op(dev, "sqrt_fwd", {"x": x, "y": np.zeros_like(x)}, ["y"])
    np.testing.assert_array_equal(out["y"], f32(c["expected"]))
    out = run_op(dev, "sqrt_bwd", {"x": x, "x_g": np.zeros_like(x), "y_g": np.ones_like(x), "eps": 1e-12}, ["x_g"])
    np.testing.assert_array_equal(out["x_g"], f32(c["grad"]))


def check_losses(dev):
    c = G["smce_1d"]
    x, t = f32(c["logits"]), f32(c["target"])
    out = run_op(dev, "smce_fwd", {"logits": x, "target": t, "probs": np.zeros_like(x), "loss": np.zeros(1, np.float32),
                                   "rows": 1, "cols": 4}, ["probs", "loss"])
    np.testing.assert_allclose(out["loss"][0], c["expected_loss"], rtol=2e-6)
    sm = np.exp(x.astype(np.float64) - np.log(np.sum(np.exp(x.astype(np.float64)))))
    np.testing.assert_allclose(out["probs"], sm, rtol=2e-6)
    g = run_op(dev, "smce_bwd", {"probs": out["probs"], "target": t, "grad": np.zeros_like(x), "rows": 1, "cols": 4},
               ["grad"])["grad"]
    np.testing.assert_allclose(g, sm - t, rtol=2e-6, atol=1e-7)
    # integer-label form gives the same loss and gradient
    lab = np.asarray([1], np.uint64)
    o2 = run_op(dev, "smce_label_fwd", {"logits": x, "labels": lab, "lse": np.zeros(1, np.float32),
                                        "loss": np.zeros(1, np.float32), "rows": 1, "cols": 4}, ["lse", "loss"])
    np.testing.assert_allclose(o2["loss"][0], c["expected_loss"], rtol=2e-6)
    g2 = run_op(dev, "smce_label_bwd", {"logits": x, "labels": lab, "lse": o2["lse"], "grad": np.zeros_like(x), "rows": 1,
                                        "cols": 4}, ["grad"])["grad"]
    np.testing.assert_allclose(g2, sm - t, rtol=2e-6, atol=1e-7)

    c = G["smooth_l1"]
    p, t = f32(c["pred"]), f32(c["target"])
    out = run_op(dev, "smooth_l1_fwd", {"pred": p, "target": t, "beta": c["beta"], "loss": np.zeros(1, np.float32)},
                 ["loss"])
    assert out["loss"][0] == np.float32(c["expected_loss"])
    g = run_op(dev, "smooth_l1_bwd", {"pred": p, "target": t, "grad": np.zeros_like(p), "beta": c["beta"]}, ["grad"])
    np.testing.assert_allclose(g["grad"] * 6, f32(c["expected_grad_times_6"]), rtol=1e-6)


def check_mul_div_backward(dev):
    """t3 = t1 * t2 and t3 = t1 / t2 followed by backward() with an upstream gradient of ones: the op sequences of
    MulBwd / DivBwd (src/ndtensor.zig:836-907), gradient buffers zero-filled on first touch."""
    for key, op, bwd, fwd_key in (("mul_backward", "mul", host.mul_backward, "expected_product"),
                                  ("div_backward", "div", host.div_backward, "expected_quotient")):
        c = G[key]
        a, b = dev.from_numpy(f32(c["t1"])), dev.from_numpy(f32(c["t2"]))
        z, z_shape = host.elwise(dev, op, a, c["t1_shape"], b, c["t2_shape"])
        dev.sync()
        np.testing.assert_array_equal(dev.to_numpy(z), f32(c[fwd_key]))
        zg = dev.from_numpy(np.ones(len(c[fwd_key]), np.float32))
        ag, bg = dev.from_numpy(np.zeros(len(c["t1"]), np.float32)), dev.from_numpy(np.zeros(len(c["t2"]), np.float32))
        bwd(dev, a, c["t1_shape"], b, c["t2_shape"], zg, z_shape, ag, bg)
        dev.sync()
        want_a = np.float32(1.0) / f32(c["t2"]) if c.get("grad_t1_is_fp32_reciprocal_of_t2") else f32(c["grad_t1"])
        np.testing.assert_array_equal(dev.to_numpy(ag), want_a)
        np.testing.assert_array_equal(dev.to_numpy(bg), f32(c["grad_t2"]))
        dev.mem_cache_free(z)
    # broadcasting operands: the gradient of the short one is folded back (same closures, shapes (2,3) and (3,))
    a_np, b_np = f32([[1, 2, 3], [4, 5, 6]]), f32([2, 4, 8])
    a, b = dev.from_numpy(a_np.ravel()), dev.from_numpy(b_np)
    zg = dev.from_numpy(np.ones(6, np.float32))
    ag, bg = dev.from_numpy(np.zeros(6, np.float32)), dev.from_numpy(np.zeros(3, np.float32))
    host.mul_backward(dev, a, [2, 3], b, [3], zg, [2, 3], ag, bg)
    dev.sync()
    np.testing.assert_array_equal(dev.to_numpy(ag), np.tile(b_np, 2))
    np.testing.assert_array_equal(dev.to_numpy(bg), a_np.sum(axis=0))
    ag, bg = dev.from_numpy(np.zeros(6, np.float32)), dev.from_numpy(np.zeros(3, np.float32))
    host.div_backward(dev, a, [2, 3], b, [3], zg, [2, 3], ag, bg)
    dev.sync()
    np.testing.assert_array_equal(dev.to_numpy(ag), np.tile(1 / b_np, 2))
    np.testing.assert_array_equal(dev.to_numpy(bg), -(a_np / (b_np * b_np)).sum(axis=0))  # powers of two: exact


def check_matvec_dot_backward(dev):
    """y = A x and z = t1 . t2 followed by backward(): MatvecBwd issues outer + matvec, DotBwd two axpy whose alpha
    is read through a pointer to the result's one-element gradient in device memory (src/ndtensor.zig:1142-1252)."""
    c = G["matvec_backward"]
    A, x = dev.from_numpy(f32(c["A"])), dev.from_numpy(f32(c["x"]))
    rows, cols = c["A_shape"]
    y = dev.from_numpy(np.full(rows, np.nan, np.float32))
    dev.dispatch("matvec", A=A, x=x, y=y, m=rows, n=cols, trans_a=False, alpha=1.0, beta=0.0)
    dev.sync()
    np.testing.assert_array_equal(dev.to_numpy(y), f32(c["expected_y"]))
    yg = dev.from_numpy(np.ones(rows, np.float32))
    Ag, xg = dev.from_numpy(np.zeros(rows * cols, np.float32)), dev.from_numpy(np.zeros(cols, np.float32))
    host.matvec_backward(dev, A, c["A_shape"], x, yg, Ag, xg)
    dev.sync()
    np.testing.assert_array_equal(dev.to_numpy(Ag), f32(c["grad_A"]))
    np.testing.assert_array_equal(dev.to_numpy(xg), f32(c["grad_x"]))
    # an upstream gradient that is not all ones separates outer(dy, x) from outer(x, dy) and A^T dy from A dy
    yg = dev.from_numpy(f32([2, -1]))
    Ag, xg = dev.from_numpy(np.zeros(4, np.float32)), dev.from_numpy(np.zeros(2, np.float32))
    x2 = dev.from_numpy(f32([3, 5]))
    host.matvec_backward(dev, A, c["A_shape"], x2, yg, Ag, xg)
    dev.sync()
    np.testing.assert_array_equal(dev.to_numpy(Ag), f32([6, 10, -3, -5]))
    np.testing.assert_array_equal(dev.to_numpy(xg), f32([2 * 1 - 3, 2 * 2 - 4]))

    c = G["dot_backward"]
    t1, t2 = dev.from_numpy(f32(c["t1"])), dev.from_numpy(f32(c["t2"]))
    z = dev.from_numpy(np.zeros(1, np.float32))
    dev.dispatch("dot", x=t1, y=t2, z=z)
    dev.sync()
    assert dev.to_numpy(z)[0] == c["expected"]
    zg = dev.from_numpy(np.ones(1, np.float32))  # backward() of a scalar: gradient 1, resident on the device
    g1, g2 = dev.from_numpy(np.zeros(3, np.float32)), dev.from_numpy(np.zeros(3, np.float32))
    host.dot_backward(dev, t1, t2, zg, g1, g2)
    dev.sync()
    np.testing.assert_array_equal(dev.to_numpy(g1), f32(c["grad_t1"]))
    np.testing.assert_array_equal(dev.to_numpy(g2), f32(c["grad_t2"]))
    # alpha really is read from the gradient: a different upstream value scales both
    zg = dev.from_numpy(f32([-0.5]))
    host.dot_backward(dev, t1, t2, zg, g1, g2)
    dev.sync()
    np.testing.assert_array_equal(dev.to_numpy(g1), f32(c["grad_t1"]) * 0.5)
    np.testing.assert_array_equal(dev.to_numpy(g2), f32(c["grad_t2"]) * 0.5)


ALL_CHECKS = [
    check_clip_nrm2, check_clamp, check_add_sub_scalar, check_dot, check_bmm, check_matvec, check_sum_max_along,
    check_gather, check_sum, check_add_broadcast_grad, check_matmul_backward, check_pow_sqrt, check_losses,
    check_mul_div_backward, check_matvec_dot_backward,
]
