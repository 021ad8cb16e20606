"""Optimizer steps of small tensors wait while the calls that follow are more steps with the same settings and then leave
together in the parameter-list kernels (src/nn/optim.zig:100-122, :177-234: Optimizer.step() walks its parameter list).
Whatever the list looks like, parameters, moments and clipped gradients must equal, bit for bit, those of the same
calls launched one by one (a synchronisation after each)."""
from __future__ import annotations

import numpy as np
import pytest

from zigrad_amd.device import F32

pytestmark = pytest.mark.gpu

SIZES = [7, 640, 4096, 4097, 8192, 65536, 65537, 100_352, 1 << 20, (1 << 20) + 4, 128, 1]


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
