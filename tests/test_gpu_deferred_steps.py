"""Optimizer steps of small tensors wait while the calls that follow are more steps with the same settings and then leave
together in the parameter-list kernels (src/nn/optim.zig:100-122, :177-234: Optimizer.step() walks its parameter list).
Whatever the list looks like, parameters, moments and clipped gradients must equal, bit for bit, those of the same
calls launched one by one (a synchronisation after each)."""
from __future__ import annotations

import numpy as np
import pytest

from zigrad_amd.device import F32

pytestmark = pytest.mark.gpu

SIZES = [7, 640, 4096, 4097, 8192, 65536, 65537, 100_352, 131072, 131073, 1 << 20, (1 << 20) + 4, 128, 1]


def _run(hip, kind, sizes, eager, clip, vary_lr=False, repeat_first=False):
    r = np.random.default_rng(11)
    bufs = []
    for n in sizes:
        p = r.standard_normal(n).astype(np.float32)
        g = (r.standard_normal(n) * (30.0 if n % 2 else 0.01)).astype(np.float32)  # some norms above the clip, some below
        bufs.append([hip.from_numpy(p), hip.from_numpy(g), hip.from_numpy(np.zeros(n, np.float32)),
                     hip.from_numpy(np.zeros(n, np.float32))])
    step = hip.sync if eager else (lambda: None)
    order = list(range(len(sizes))) + ([0] if repeat_first else [])
    t = 0
    for rounds in range(2):
        for i in order:
            p, g, m, v = bufs[i]
            t += 1
            lr = 0.01 * (1 + (i % 3 if vary_lr else 0))
            if kind == "sgd":
                hip.dispatch("sgd_step", param=p, grad=g, lr=lr, clip=clip, max_norm=10.0, delta=1e-6)
            else:
                hip.dispatch("adam_step", param=p, grad=g, m=m, v=v, t=t, lr=lr, beta1=0.9, beta2=0.999, epsilon=1e-8,
                             clip=clip, max_norm=10.0, delta=1e-6)
            step()
    out = [[hip.to_numpy(b) for b in row] for row in bufs]
    for row in bufs:
        for b in row:
            hip.mem_free(b)
    return out


@pytest.mark.parametrize("kind", ["sgd", "adam"])
@pytest.mark.parametrize("clip", [True, False])
@pytest.mark.parametrize("vary_lr,repeat_first", [(False, False), (True, False), (False, True)])
def test_runs_of_optimizer_steps_equal_the_steps_launched_one_by_one(hip, kind, clip, vary_lr, repeat_first):
    got = _run(hip, kind, SIZES, False, clip, vary_lr, repeat_first)
    ref = _run(hip, kind, SIZES, True, clip, vary_lr, repeat_first)
    for i, (a, b) in enumerate(zip(got, ref)):
        for name, x, y in zip(("param", "grad", "m", "v"), a, b):
            assert np.array_equal(x, y), (kind, SIZES[i], name)


def test_a_read_or_a_fill_after_waiting_steps_sees_them(hip):
    n = 1000
    p = hip.from_numpy(np.ones(n, np.float32))
    g = hip.from_numpy(np.full(n, 0.5, np.float32))
    hip.dispatch("sgd_step", param=p, grad=g, lr=0.1, clip=False, max_norm=10.0, delta=1e-6)
    np.testing.assert_array_equal(hip.to_numpy(p), np.full(n, np.float32(1.0) + np.float32(-0.1) * np.float32(0.5)))
    hip.dispatch("sgd_step", param=p, grad=g, lr=0.1, clip=False, max_norm=10.0, delta=1e-6)
    hip.mem_fill(g, 0.0)     # zero_grad: after the step that reads the gradient
    hip.dispatch("sgd_step", param=p, grad=g, lr=0.1, clip=False, max_norm=10.0, delta=1e-6)   # a step on zeros
    want = np.float32(1.0) + np.float32(-0.1) * np.float32(0.5)
    want = want + np.float32(-0.1) * np.float32(0.5)
    np.testing.assert_array_equal(hip.to_numpy(p), np.full(n, want, np.float32))
    np.testing.assert_array_equal(hip.to_numpy(g), np.zeros(n, np.float32))
    for b in (p, g):
        hip.mem_free(b)


def _step_then_zero_grad(hip, kind, sizes, eager, fills, extra_fill=None):
    """optimizer.step() over the list, then zero_grad() as the reference issues it: a mem_fill per gradient
    (examples/mnist/src/model.zig:57-62).  `fills`: which gradients are zeroed, and with what value."""
    r = np.random.default_rng(17)
    bufs = []
    for n in sizes:
        p = r.standard_normal(n).astype(np.float32)
        g = (r.standard_normal(n) * (30.0 if n % 2 else 0.01)).astype(np.float32)
        bufs.append([hip.from_numpy(p), hip.from_numpy(g), hip.from_numpy(np.zeros(n, np.float32)),
                     hip.from_numpy(np.zeros(n, np.float32))])
    step = hip.sync if eager else (lambda: None)
    other = hip.from_numpy(np.ones(300, np.float32))
    for t, (p, g, m, v) in enumerate(bufs, start=1):
        if kind == "sgd":
            hip.dispatch("sgd_step", param=p, grad=g, lr=0.01, clip=True, max_norm=10.0, delta=1e-6)
        else:
            hip.dispatch("adam_step", param=p, grad=g, m=m, v=v, t=t, lr=0.01, beta1=0.9, beta2=0.999, epsilon=1e-8,
                         clip=True, max_norm=10.0, delta=1e-6)
        step()
    for i, value in fills:
        g = bufs[i][1]
        if value == "half":
            hip.mem_fill(g.sub(0, max(1, g.n // 2)), 0.0)
        else:
            hip.mem_fill(g, value)
        step()
        if extra_fill == i:
            hip.mem_fill(other, 4.0)
            step()
    out = [[hip.to_numpy(b) for b in row] for row in bufs] + [[hip.to_numpy(other)]]
    for row in bufs:
        for b in row:
            hip.mem_free(b)
    hip.mem_free(other)
    return out


ZERO_SIZES = [100_352, 128, 8192, 64, 640, 10]


@pytest.mark.parametrize("kind", ["sgd", "adam"])
@pytest.mark.parametrize("case", ["all", "some", "one_tensor", "reversed", "nonzero", "minus_zero", "half", "twice",
                                  "other_fill_between"])
def test_zero_grad_after_waiting_steps(hip, kind, case):
    sizes = ZERO_SIZES if case != "one_tensor" else [4096]
    idx = list(range(len(sizes)))
    extra = None
    if case in ("all", "one_tensor"):
        fills = [(i, 0.0) for i in idx]
    elif case == "some":
        fills = [(i, 0.0) for i in idx[::2]]
    elif case == "reversed":
        fills = [(i, 0.0) for i in reversed(idx)]
    elif case == "nonzero":
        fills = [(i, 0.0 if i % 2 else 3.5) for i in idx]
    elif case == "minus_zero":
        fills = [(i, -0.0 if i == 2 else 0.0) for i in idx]
    elif case == "half":
        fills = [(i, "half" if i == 1 else 0.0) for i in idx]
    elif case == "twice":
        fills = [(i, 0.0) for i in idx] + [(0, 0.0), (3, 0.0)]
    else:
        fills = [(i, 0.0) for i in idx]
        extra = 2
    got = _step_then_zero_grad(hip, kind, sizes, False, fills, extra)
    ref = _step_then_zero_grad(hip, kind, sizes, True, fills, extra)
    for i, (a, b) in enumerate(zip(got, ref)):
        for j, (x, y) in enumerate(zip(a, b)):
            assert np.array_equal(x, y) and np.array_equal(np.signbit(x), np.signbit(y)), (kind, case, i, j)
    if case == "all":
        for row in got[:-1]:
            assert np.all(row[1] == 0.0) and not np.any(np.signbit(row[1]))


def test_the_next_step_accumulates_into_gradients_zeroed_by_the_update_kernel(hip):
    """step(), zero_grad(), then a product that adds into a zeroed gradient: the zeros must be in place before it."""
    r = np.random.default_rng(23)
    O, I, B = 48, 40, 64
    gy, x = r.standard_normal((B, O)).astype(np.float32), r.standard_normal((B, I)).astype(np.float32)
    w = hip.from_numpy(r.standard_normal(O * I).astype(np.float32))
    b = hip.from_numpy(r.standard_normal(O).astype(np.float32))
    gw = hip.from_numpy(r.standard_normal(O * I).astype(np.float32))
    gb = hip.from_numpy(r.standard_normal(O).astype(np.float32))
    gyb, xb = hip.from_numpy(gy), hip.from_numpy(x)
    hip.dispatch("sgd_step", param=w, grad=gw, lr=0.01, clip=True, max_norm=10.0, delta=1e-6)
    hip.dispatch("sgd_step", param=b, grad=gb, lr=0.01, clip=True, max_norm=10.0, delta=1e-6)
    hip.mem_fill(gw, 0.0)
    hip.mem_fill(gb, 0.0)
    hip.dispatch("bmm_acc", A=gyb, B=xb, C=gw, A_shape=[1, O, B], B_shape=[1, B, I], C_shape=[1, O, I], trans_a=True,
                 trans_b=False, lda=O, ldb=I, ldc=I, alpha=1.0, beta=1.0)
    got = hip.to_numpy(gw).reshape(O, I)
    want = gy.astype(np.float64).T @ x.astype(np.float64)
    assert np.linalg.norm(got - want) <= 1e-5 * np.linalg.norm(want)
    assert np.all(hip.to_numpy(gb) == 0.0)
    for t in (w, b, gw, gb, gyb, xb):
        hip.mem_free(t)


def test_a_step_whose_tensors_overlap_a_waiting_steps_goes_after_it(hip):
    """The gradient of one step is the parameter of the next (or overlaps it): the two must not share a launch."""
    r = np.random.default_rng(29)
    n = 640
    init = [r.standard_normal(4096).astype(np.float32) for _ in range(3)]
    outs = []
    for eager in (False, True):
        a, b, c = (hip.from_numpy(x) for x in init)
        step = hip.sync if eager else (lambda: None)
        hip.dispatch("sgd_step", param=a.sub(0, n), grad=b.sub(0, n), lr=0.01, clip=True, max_norm=10.0, delta=1e-6)
        step()
        hip.mem_fill(b.sub(0, n), 0.0)
        step()
        hip.dispatch("sgd_step", param=b, grad=c, lr=0.01, clip=True, max_norm=10.0, delta=1e-6)      # writes what the first reads
        step()
        hip.dispatch("sgd_step", param=c.sub(100, n), grad=a.sub(8, n), lr=0.01, clip=True, max_norm=10.0, delta=1e-6)
        step()
        outs.append([hip.to_numpy(t) for t in (a, b, c)])
        for t in (a, b, c):
            hip.mem_free(t)
    for x, y in zip(*outs):
        assert np.array_equal(x, y)
