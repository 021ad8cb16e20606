"""The batch-64 MLP train step driven from plain C through the C ABI (examples/c_caller/mlp_step.c) gives, step for
step, the losses the Python trainer gives on the same parameters and batch: the boundary needs nothing from Python."""
from __future__ import annotations

import subprocess

import numpy as np
import pytest

from zigrad_amd.build import C_HARNESS_BIN
from zigrad_amd.trainers import MLPTrainer, mlp_inputs

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
