"""What the calls may leave waiting in the context, and the two ways a caller that mixes in its own HIP calls gets rid
of it: zg_hip_flush launches what waits without waiting for the stream, zg_hip_set_holding(ctx, 0) makes every call
launch its own work before it returns.  Values are the same either way (the reference's devices hold nothing:
src/device/host_device.zig, src/device/cuda_device.zig)."""
from __future__ import annotations

import numpy as np
import pytest

from zigrad_amd import HipDevice
from zigrad_amd.device import F32
from zigrad_amd.trainers import DQNTrainer, MLPTrainer, dqn_inputs, mlp_inputs

pytestmark = pytest.mark.gpu


def test_flush_launches_what_waits_and_nothing_else(hip):
    n = 1000
    a, b = hip.from_numpy(np.ones(n, np.float32)), hip.mem_alloc(F32, n)
    hip.sync()
    base = hip.launch_count()
    hip.mem_fill(b, 2.0)                       # waits
    hip.dispatch("add", x=a, y=3.0, z=a)       # waits (a small elementwise op)
    assert hip.launch_count() == base
    hip.flush()
    assert hip.launch_count() == base + 2
    hip.flush()                                # nothing waits: nothing is launched
    assert hip.launch_count() == base + 2
    hip.sync()
    np.testing.assert_array_equal(hip.to_numpy(a), np.full(n, 4.0, np.float32))
    np.testing.assert_array_equal(hip.to_numpy(b), np.full(n, 2.0, np.float32))
    hip.mem_free(a)
    hip.mem_free(b)


def test_with_holding_off_every_call_launches_its_own_work():
    dev = HipDevice(0)
    try:
        dev.set_holding(False)
        n = 512
        x = dev.from_numpy(np.arange(n, dtype=np.float32))
        y = dev.mem_alloc(F32, n)
        dev.sync()
        base = dev.launch_count()
        dev.mem_fill(y, 1.5)
        assert dev.launch_count() == base + 1
        dev.dispatch("mul", x=x, y=2.0, z=x)
        assert dev.launch_count() == base + 2
        dev.dispatch("relu_fwd", x=x, y=y)
        assert dev.launch_count() == base + 3
        np.testing.assert_array_equal(dev.to_numpy(y), np.arange(n, dtype=np.float32) * 2)
        dev.set_holding(True)
        dev.mem_fill(y, 0.0)
        assert dev.launch_count() == base + 3 + 1   # the read above was one launch (a copy kernel); the fill waits again
        dev.mem_free(x)
        dev.mem_free(y)
    finally:
        dev.deinit()


@pytest.mark.parametrize("which", ["mlp", "dqn"])
def test_train_steps_are_bit_identical_with_holding_off(which):
    """The launches differ (one or more per call instead of shared ones), the values do not."""
    results = []
    for hold in (True, False):
        dev = HipDevice(0)
        try:
            dev.set_holding(hold)
            if which == "mlp":
                dims, batch = [784, 128, 64, 10], 64
                params, x, onehot, labels = mlp_inputs(dims, batch, seed_weights=0, seed_data=1, data="uniform")
                tr = MLPTrainer(dev, dims, batch, optimizer="sgd", lr=0.01, clip=True)
                tr.load_params(params)
                tr.set_batch(x, onehot, labels)
            else:
                dims, batch = [4, 128, 128, 2], 64
                params, _, _, _ = mlp_inputs(dims, batch)
                tr = DQNTrainer(dev, dims, batch, lr=1e-3, gamma=0.99, clip=True)
                tr.load_params(params)
                tr.set_batch(dqn_inputs(batch=batch))
            dev.sync()
            before = dev.launch_count()
            losses = [tr.step() for _ in range(5)]
            dev.sync()
            launches = dev.launch_count() - before
            results.append((losses, [dev.to_numpy(p) for p in tr.param_buffers()], launches))
        finally:
            dev.deinit()
    (l1, p1, n1), (l2, p2, n2) = results
    assert l1 == l2
    for a, b in zip(p1, p2):
        np.testing.assert_array_equal(a, b)
    assert n2 > n1   # holding is what saves the launches
