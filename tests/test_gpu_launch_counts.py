"""How many kernel launches one train step of the latency-bound configurations costs, from an unchanged caller's op
sequence and through the fused entry points.  The reference launches one kernel (or more) per device op
(src/device/cuda_device.zig); here fills, products, elementwise ops and optimizer steps that follow each other share
launches inside the library, and these counts are what that sharing was measured to come to.  A change that makes a
step cost more launches fails here before it shows in a profile."""
from __future__ import annotations

import pytest

from zigrad_amd.trainers import DQNTrainer, GCNTrainer, MLPTrainer, dqn_inputs, gcn_inputs, mlp_inputs

pytestmark = pytest.mark.gpu


def launches_per_step(hip, tr, steps=6):
    for _ in range(4):      # the allocator, the workspace and the bucket plans reach their final state
        tr.step()
    hip.sync()
    before = hip.launch_count()
    for _ in range(steps):
        tr.step()
    hip.sync()
    total = hip.launch_count() - before
    assert total % steps == 0, "every step costs the same launches"
    return total // steps


@pytest.mark.parametrize("fused,want", [(False, 11), (True, 10)])
def test_batch_64_mlp_step(hip, fused, want):
    dims, batch = [784, 128, 64, 10], 64
    params, x, onehot, labels = mlp_inputs(dims, batch, seed_weights=0, seed_data=1, data="uniform")
    tr = MLPTrainer(hip, dims, batch, optimizer="sgd", lr=0.01, clip=True, fused=fused)   # 42 op calls per step
    tr.load_params(params)
    tr.set_batch(x, onehot, labels)
    assert launches_per_step(hip, tr) == want


@pytest.mark.parametrize("device_scalars", [False, True], ids=["host_scalars", "device_scalars"])
@pytest.mark.parametrize("fused,want", [(False, 18), (True, 17)])
def test_dqn_update(hip, fused, want, device_scalars):
    dims, batch = [4, 128, 128, 2], 64
    params, _, _, _ = mlp_inputs(dims, batch)
    tr = DQNTrainer(hip, dims, batch, lr=1e-3, gamma=0.99, clip=True, fused=fused, device_scalars=device_scalars)
    tr.load_params(params)
    tr.set_batch(dqn_inputs(batch=batch))
    assert launches_per_step(hip, tr) == want


@pytest.mark.parametrize("fused,want", [(False, 22), (True, 19)])
def test_gcn_step(hip, fused, want):
    tr = GCNTrainer(hip, gcn_inputs(seed=0), lr=0.01, clip=True, fused=fused)
    assert launches_per_step(hip, tr) == want
