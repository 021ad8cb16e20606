"""Whole train steps on the HIP device against the oracle: relative error <= 1e-4 on loss, gradients and
updated parameters (the benchmark definition's bound for a full step)."""
from __future__ import annotations

import numpy as np
import pytest

from conftest import rel_fro
from zigrad_amd.trainers import MLPTrainer, mlp_inputs

pytestmark = pytest.mark.gpu
STEP_TOL = 1e-4


@pytest.mark.parametrize("dims,batch,optimizer,clip,data", [
    ([784, 128, 64, 10], 64, "sgd", True, "uniform"),    # config 1 (reference defaults: clip on)
    ([784, 128, 64, 10], 64, "sgd", False, "uniform"),   # config 1 as the example runs it
    ([4, 128, 128, 2], 64, "adam", True, "normal"),      # the DQN-sized network
    ([512, 768, 256, 128], 256, "adam", True, "normal"),  # a scaled-down wide MLP
])
@pytest.mark.parametrize("loss_mode", ["onehot", "label"])
def test_mlp_steps_match_oracle(oracle, hip, dims, batch, optimizer, clip, data, loss_mode):
    params, x, onehot, labels = mlp_inputs(dims, batch, seed_weights=0, seed_data=1, data=data)
    runs = {}
    for name, dev in (("oracle", oracle), ("hip", hip)):
        tr = MLPTrainer(dev, dims, batch, optimizer=optimizer, lr=0.01 if optimizer == "sgd" else 1e-3, clip=clip,
                        loss_mode=loss_mode)
        tr.load_params(params)
        tr.set_batch(x, onehot, labels)
        losses, grads = [], None
        for s in range(3):
            losses.append(tr.step(keep_grads=(s == 0)))
            if s == 0:
                grads = tr.last_grads
        dev.sync()
        runs[name] = (losses, grads, [dev.to_numpy(p) for p in tr.param_buffers()])
    (lo, go, po), (lh, gh, ph) = runs["oracle"], runs["hip"]
    for a, b in zip(lo, lh):
        assert abs(a - b) <= STEP_TOL * max(1.0, abs(a)), (lo, lh)
    for a, b in zip(go, gh):
        assert rel_fro(b, a) <= STEP_TOL
    for a, b in zip(po, ph):
        assert rel_fro(b, a) <= STEP_TOL
    assert lh[-1] < lh[0]  # the loss goes down on a fixed batch


def test_no_device_allocation_in_steady_state(hip):
    dims, batch = [784, 128, 64, 10], 64
    params, x, onehot, labels = mlp_inputs(dims, batch, data="uniform")
    tr = MLPTrainer(hip, dims, batch, optimizer="adam", lr=1e-3)
    tr.load_params(params)
    tr.set_batch(x, onehot, labels)
    for _ in range(3):
        tr.step()
    n0 = hip.cache_stats()["n_device_allocs"]
    for _ in range(20):
        tr.step()
    assert hip.cache_stats()["n_device_allocs"] == n0


def test_gcn_steps_match_oracle(oracle, hip):
    """Config 3 at its real size: 2708 nodes, 1433 features, 13264 edges, 140 labelled nodes, Adam."""
    from zigrad_amd.trainers import GCNTrainer, gcn_inputs

    inp = gcn_inputs(seed=0)
    runs = {}
    for name, dev in (("oracle", oracle), ("hip", hip)):
        tr = GCNTrainer(dev, inp, lr=0.01, clip=True)
        losses = [tr.step(keep_grads=(s == 0)) for s in range(5)]
        dev.sync()
        runs[name] = (losses, tr.last_grads, [dev.to_numpy(p) for p in tr.param_buffers()])
    (lo, go, po), (lh, gh, ph) = runs["oracle"], runs["hip"]
    for a, b in zip(lo, lh):
        assert abs(a - b) <= STEP_TOL * max(1.0, abs(a)), (lo, lh)
    for a, b in zip(go, gh):
        assert rel_fro(b, a) <= STEP_TOL
    for a, b in zip(po, ph):
        assert rel_fro(b, a) <= STEP_TOL
    assert lh[-1] < lh[0]


def test_dqn_steps_match_oracle(oracle, hip):
    """Config 4: 4 -> 128 -> 128 -> 2, batch 64, frozen target network, gather, smooth-L1, Adam lr 1e-3."""
    from zigrad_amd.trainers import DQNTrainer, dqn_inputs

    dims, batch = [4, 128, 128, 2], 64
    params, _, _, _ = mlp_inputs(dims, batch)
    b = dqn_inputs(batch=batch)
    runs = {}
    for name, dev in (("oracle", oracle), ("hip", hip)):
        tr = DQNTrainer(dev, dims, batch, lr=1e-3, gamma=0.99, clip=True)
        tr.load_params(params)
        tr.set_batch(b)
        losses = [tr.step(keep_grads=(s == 0)) for s in range(10)]
        dev.sync()
        runs[name] = (losses, tr.last_grads, [dev.to_numpy(p) for p in tr.param_buffers()])
    (lo, go, po), (lh, gh, ph) = runs["oracle"], runs["hip"]
    for a, b2 in zip(lo, lh):
        assert abs(a - b2) <= STEP_TOL * max(1.0, abs(a)), (lo, lh)
    for a, b2 in zip(go, gh):
        assert rel_fro(b2, a) <= STEP_TOL
    for a, b2 in zip(po, ph):
        assert rel_fro(b2, a) <= STEP_TOL


@pytest.mark.parametrize("fused", [False, True])
def test_dqn_with_host_scalars_equals_dqn_with_device_scalars(hip, fused):
    """gamma and 1 by value (NDArray's scalar ops, src/ndarray.zig:247-257) against gamma and 1 as one-element device
    tensors (examples/dqn/src/dqn_agent.zig:173-181): the same IEEE operations, so the same bits after ten updates."""
    from zigrad_amd.trainers import DQNTrainer, dqn_inputs

    dims, batch = [4, 128, 128, 2], 64
    params, _, _, _ = mlp_inputs(dims, batch)
    b = dqn_inputs(batch=batch)
    runs = []
    for device_scalars in (False, True):
        tr = DQNTrainer(hip, dims, batch, lr=1e-3, gamma=0.99, clip=True, fused=fused, device_scalars=device_scalars)
        tr.load_params(params)
        tr.set_batch(b)
        losses = [tr.step() for _ in range(10)]
        hip.sync()
        runs.append((losses, [hip.to_numpy(p) for p in tr.param_buffers()]))
    assert runs[0][0] == runs[1][0]
    for a, b2 in zip(runs[0][1], runs[1][1]):
        np.testing.assert_array_equal(a, b2)
