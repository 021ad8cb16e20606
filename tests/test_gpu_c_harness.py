"""The batch-64 MLP train step driven from plain C through the C ABI (examples/c_caller/mlp_step.c) gives, step for
step, the losses the Python trainer gives on the same parameters and batch: the boundary needs nothing from Python."""
from __future__ import annotations

import subprocess

import numpy as np
import pytest

from zigrad_amd.build import C_DQN_BIN, C_GCN_BIN, C_HARNESS_BIN
from zigrad_amd.trainers import DQNTrainer, GCNTrainer, MLPTrainer, dqn_inputs, gcn_inputs, mlp_inputs

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("fused", [False, True])
@pytest.mark.parametrize("dims,batch", [([784, 128, 64, 10], 64), ([100, 260, 130, 7], 50)])
def test_c_harness_matches_python_trainer(hip, tmp_path, dims, batch, fused):
    assert C_HARNESS_BIN.exists(), "build first: python -m zigrad_amd.build"
    steps = 6
    params, x, onehot, labels = mlp_inputs(dims, batch, seed_weights=5, seed_data=6, data="uniform")
    blob = tmp_path / "inputs.bin"
    with open(blob, "wb") as f:
        for a in (*params, x, onehot):
            f.write(np.ascontiguousarray(a, np.float32).tobytes())
    tr = MLPTrainer(hip, dims, batch, optimizer="sgd", lr=0.01, clip=True, fused=fused)
    tr.load_params(params)
    tr.set_batch(x, onehot, labels)
    want = [tr.step() for _ in range(steps)]
    run = subprocess.run([str(C_HARNESS_BIN), str(blob), str(steps), str(batch), *map(str, dims), *(["fused"] if fused else [])],
                         capture_output=True, text=True, timeout=120)
    assert run.returncode == 0, run.stderr
    got = [float(np.float32(line.split()[1])) for line in run.stdout.splitlines() if line.startswith("loss ")]
    assert got == want


@pytest.mark.parametrize("dims,batch", [([4, 128, 128, 2], 64), ([6, 40, 24, 3], 50)])
def test_c_dqn_update_matches_python_trainer(hip, tmp_path, dims, batch):
    """The DQN update (examples/c_caller/dqn_step.c): target network, max, the elementwise target chain, gather,
    smooth-L1, zero_grad before the backward pass, scatter, Adam with its per-tensor counter."""
    assert C_DQN_BIN.exists(), "build first: python -m zigrad_amd.build"
    steps = 6
    params, _, _, _ = mlp_inputs(dims, batch, seed_weights=7)
    b = dqn_inputs(batch=batch, state_dim=dims[0], n_actions=dims[-1], seed=8)
    b["dones"][::5] = 1.0
    blob = tmp_path / "inputs.bin"
    with open(blob, "wb") as f:
        for a in (*params, b["states"], b["next_states"], b["rewards"], b["dones"]):
            f.write(np.ascontiguousarray(a, np.float32).tobytes())
        f.write(np.ascontiguousarray(b["actions"], np.uint64).tobytes())
    tr = DQNTrainer(hip, dims, batch, lr=1e-3, gamma=0.99, clip=True, fused=False)
    tr.load_params(params)
    tr.set_batch(b)
    want = [tr.step() for _ in range(steps)]
    run = subprocess.run([str(C_DQN_BIN), str(blob), str(steps), str(batch), *map(str, dims)], capture_output=True, text=True,
                         timeout=120)
    assert run.returncode == 0, run.stderr
    got = [float(np.float32(line.split()[1])) for line in run.stdout.splitlines() if line.startswith("loss ")]
    assert got == want


def write_gcn_inputs(path, inp):
    with open(path, "wb") as f:
        for a in (*inp["params"], inp["x"], inp["onehot"][: inp["n_train"]]):
            f.write(np.ascontiguousarray(a, np.float32).tobytes())
        f.write(np.ascontiguousarray(inp["src"], np.uint64).tobytes())
        f.write(np.ascontiguousarray(inp["tgt"], np.uint64).tobytes())


def gcn_args(inp):
    return [inp["x"].shape[0], *inp["dims"], inp["src"].size, inp["n_train"]]


@pytest.mark.parametrize("shape", [dict(), dict(n_nodes=300, n_features=50, n_pairs=700, n_classes=5, n_train=33, hidden=8)])
def test_c_gcn_step_matches_python_trainer(hip, tmp_path, shape):
    """The GCN step (examples/c_caller/gcn_step.c): degree normalisation in every layer's forward, aggregation, the
    masked loss, both backward aggregations with the degree gradient freed unread, Adam, zero_grad."""
    assert C_GCN_BIN.exists(), "build first: python -m zigrad_amd.build"
    steps = 5
    inp = gcn_inputs(seed=3, **shape)
    blob = tmp_path / "inputs.bin"
    write_gcn_inputs(blob, inp)
    tr = GCNTrainer(hip, inp, lr=0.01, clip=True, fused=False)
    want = [tr.step() for _ in range(steps)]
    run = subprocess.run([str(C_GCN_BIN), str(blob), str(steps), *map(str, gcn_args(inp))], capture_output=True, text=True,
                         timeout=120)
    assert run.returncode == 0, run.stderr
    got = [float(np.float32(line.split()[1])) for line in run.stdout.splitlines() if line.startswith("loss ")]
    assert got == want
