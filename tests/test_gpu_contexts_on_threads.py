"""Contexts used at the same time from different host threads, one context per thread (the reference's devices are
not shared between threads either: the caching allocator of src/device/host_device.zig:181-191 has no lock): every
thread must get, bit for bit, what it gets when it runs alone.  The jobs cover the state a context keeps between
calls: the caching allocator, work that waits in the context, kept destination orderings, recorded steps."""
from __future__ import annotations

import threading

import numpy as np
import pytest

from zigrad_amd import HipDevice
from zigrad_amd.device import F32
from zigrad_amd.trainers import GCNTrainer, MLPTrainer, gcn_inputs, mlp_inputs

pytestmark = pytest.mark.gpu

STEPS = 12


def _mlp(dev, dims, batch, seed, data, recorded):
    params, x, onehot, labels = mlp_inputs(dims, batch, seed_weights=seed, seed_data=seed + 1, data=data)
    tr = MLPTrainer(dev, dims, batch, optimizer="adam", lr=1e-3, clip=True)
    tr.load_params(params)
    tr.set_batch(x, onehot, labels)
    if recorded:
        losses = [tr.step() for _ in range(2)]
        tr.capture()
        losses += [tr.step_graph() for _ in range(STEPS - 2)]
        tr.free_graph()
    else:
        losses = [tr.step() for _ in range(STEPS)]
    return losses, [dev.to_numpy(p) for p in tr.param_buffers()]


def _gcn(dev, seed):
    tr = GCNTrainer(dev, gcn_inputs(seed=seed), lr=0.01, clip=True)
    losses = [tr.step() for _ in range(STEPS)]
    return losses, [dev.to_numpy(p) for p in tr.param_buffers()]


def _long_scatter(dev, seed):
    """300 000 entries: the ordering is kept under the array's address and checked against it by every call."""
    r = np.random.default_rng(seed)
    n, n_dst = 300_000, 50_000
    off = r.integers(0, n_dst, n).astype(np.uint64)
    src, a = dev.from_numpy(r.standard_normal(n).astype(np.float32)), dev.from_numpy(off)
    outs = []
    for k in range(6):
        if k == 3:      # rewritten in place between two calls
            dev.sync()
            dev.mem_transfer(np.roll(off, 1), a, "HtoD")
        dst = dev.mem_alloc(F32, n_dst)
        dev.mem_fill(dst, 0.0)
        dev.dispatch("scatter_add", src=src, offsets=a, dst=dst)
        outs.append(dev.to_numpy(dst))
        dev.mem_free(dst)
    return [], outs


JOBS = [
    lambda dev: _mlp(dev, [784, 128, 64, 10], 64, 0, "uniform", False),
    lambda dev: _mlp(dev, [512, 768, 256, 128], 256, 3, "normal", False),
    lambda dev: _gcn(dev, 5),
    lambda dev: _mlp(dev, [784, 128, 64, 10], 64, 7, "uniform", True),
    lambda dev: _long_scatter(dev, 9),
    lambda dev: _gcn(dev, 11),
]


def _run(job, out, i):
    try:
        dev = HipDevice(0)
        try:
            out[i] = job(dev)
            dev.sync()
        finally:
            dev.deinit()
    except BaseException as e:  # handed to the main thread, which fails the test
        out[i] = e


def test_every_thread_gets_what_it_gets_alone():
    alone = [None] * len(JOBS)
    for i, job in enumerate(JOBS):
        _run(job, alone, i)
        assert not isinstance(alone[i], BaseException), alone[i]
    for _ in range(2):
        together = [None] * len(JOBS)
        threads = [threading.Thread(target=_run, args=(job, together, i)) for i, job in enumerate(JOBS)]
        for t in threads:
            t.start()
        for t in threads:
            t.join(timeout=100)
            assert not t.is_alive()
        for i, (a, b) in enumerate(zip(alone, together)):
            assert not isinstance(b, BaseException), (i, b)
            assert a[0] == b[0], i
            for x, y in zip(a[1], b[1]):
                np.testing.assert_array_equal(x, y, err_msg=f"job {i}")
