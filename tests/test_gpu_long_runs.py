"""The latency-bound configurations at the step counts the benchmark definition names (100 SGD steps of the batch-64
MLP, 200 Adam steps of the graph convolution network, 1000 updates of the DQN network), device against the CPU oracle:
every loss of the run and the parameters at its end within 1e-4 (measured: losses 4e-7, parameters 1e-5 and better),
so rounding differences do not build up over a run."""
from __future__ import annotations

import pytest

from conftest import rel_fro
from zigrad_amd.trainers import DQNTrainer, GCNTrainer, MLPTrainer, dqn_inputs, gcn_inputs, mlp_inputs

pytestmark = pytest.mark.gpu
TOL = 1e-4


def _compare(runs):
    (lo, po), (lh, ph) = runs["oracle"], runs["hip"]
    assert len(lo) == len(lh)
    for s, (a, b) in enumerate(zip(lo, lh)):
        assert abs(a - b) <= TOL * max(1.0, abs(a)), (s, a, b)
    for a, b in zip(po, ph):
        assert rel_fro(b, a) <= TOL
    return lo, lh


def test_batch_64_mlp_100_sgd_steps(oracle, hip):
    dims, batch = [784, 128, 64, 10], 64
    params, x, onehot, labels = mlp_inputs(dims, batch, seed_weights=0, seed_data=1, data="uniform")
    runs = {}
    for name, dev in (("oracle", oracle), ("hip", hip)):
        tr = MLPTrainer(dev, dims, batch, optimizer="sgd", lr=0.01, clip=True)
        tr.load_params(params)
        tr.set_batch(x, onehot, labels)
        losses = [tr.step() for _ in range(100)]
        runs[name] = (losses, [dev.to_numpy(p) for p in tr.param_buffers()])
    lo, lh = _compare(runs)
    assert lh[-1] < 0.5 * lh[0]


def test_gcn_200_adam_steps(oracle, hip):
    inp = gcn_inputs(seed=0)
    runs = {}
    for name, dev in (("oracle", oracle), ("hip", hip)):
        tr = GCNTrainer(dev, inp, lr=0.01, clip=True)
        losses = [tr.step() for _ in range(200)]
        runs[name] = (losses, [dev.to_numpy(p) for p in tr.param_buffers()])
    lo, lh = _compare(runs)
    assert lh[-1] < 1e-2 * lh[0]  # the 140 labelled nodes are fitted
    assert hip.plan_cache_stats()["hits"] > 0  # the edge list's orderings were computed once, not 1600 times


def test_dqn_1000_updates(oracle, hip):
    dims, batch = [4, 128, 128, 2], 64
    params, _, _, _ = mlp_inputs(dims, batch)
    b = dqn_inputs(batch=batch)
    runs = {}
    for name, dev in (("oracle", oracle), ("hip", hip)):
        tr = DQNTrainer(dev, dims, batch, lr=1e-3, gamma=0.99, clip=True)
        tr.load_params(params)
        tr.set_batch(b)
        losses = [tr.step() for _ in range(1000)]
        runs[name] = (losses, [dev.to_numpy(p) for p in tr.param_buffers()])
    _compare(runs)
