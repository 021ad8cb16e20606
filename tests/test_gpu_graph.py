"""Execution graphs (open / save / run / free, the ExecutionGraph of src/device/cuda_device.zig:558-611): a
recorded train step replayed many times must give exactly what the same steps give when issued eagerly."""
from __future__ import annotations

import numpy as np
import pytest

from zigrad_amd._lib import ZgHipError
from zigrad_amd.device import F32
from zigrad_amd.trainers import DQNTrainer, MLPTrainer, dqn_inputs, mlp_inputs

pytestmark = pytest.mark.gpu


def _eager_noise(hip):
    """Unrelated eager work and a synchronisation between replays (other users of the same stream, workspace,
    scalar slots and allocator)."""
    a = hip.from_numpy(np.arange(1000, dtype=np.float32), cached=True)
    out = hip.mem_cache_alloc(F32, 1)
    hip.dispatch("nrm2", x=a, y=out)
    hip.sync()
    got = hip.to_numpy(out)[0]
    hip.mem_cache_free(a)
    hip.mem_cache_free(out)
    assert abs(got - np.linalg.norm(np.arange(1000, dtype=np.float64))) < 1e-2


@pytest.mark.parametrize("optimizer,loss_mode", [("sgd", "onehot"), ("adam", "label")])
def test_mlp_replays_equal_eager_steps(hip, optimizer, loss_mode):
    dims, batch, n_steps = [784, 128, 64, 10], 64, 12
    params, x, onehot, labels = mlp_inputs(dims, batch, data="uniform")

    def make():
        tr = MLPTrainer(hip, dims, batch, optimizer=optimizer, lr=0.01 if optimizer == "sgd" else 1e-3, clip=True,
                        loss_mode=loss_mode)
        tr.load_params(params)
        tr.set_batch(x, onehot, labels)
        return tr

    eager = make()
    want = [eager.step() for _ in range(n_steps)]
    want_params = [hip.to_numpy(p) for p in eager.param_buffers()]

    tr = make()
    got = [tr.step() for _ in range(2)]
    in_use_before = hip.cache_stats()["bytes_in_use"]
    tr.capture()
    assert hip.cache_stats()["bytes_in_use"] > in_use_before  # the step's temporaries stay with the graph
    for _ in range(n_steps - 2):
        got.append(tr.step_graph())
        _eager_noise(hip)
    assert got == want  # every replay, not just the last
    for a, b in zip(want_params, [hip.to_numpy(p) for p in tr.param_buffers()]):
        assert np.array_equal(a, b)
    tr.free_graph()
    assert hip.cache_stats()["bytes_in_use"] == in_use_before
    assert tr.step() is not None  # eager steps still work afterwards


def test_dqn_replays_equal_eager_steps(hip):
    dims, batch, n_steps = [4, 128, 128, 2], 64, 10
    params, _, _, _ = mlp_inputs(dims, batch)
    b = dqn_inputs(batch=batch)

    def make():
        tr = DQNTrainer(hip, dims, batch, lr=1e-3, gamma=0.99, clip=True)
        tr.load_params(params)
        tr.set_batch(b)
        return tr

    eager = make()
    want = [eager.step() for _ in range(n_steps)]
    tr = make()
    got = [tr.step() for _ in range(2)]
    tr.capture()
    for _ in range(n_steps - 2):
        got.append(tr.step_graph())
        _eager_noise(hip)
    assert got == want
    for p, q in zip(eager.param_buffers(), tr.param_buffers()):
        assert np.array_equal(hip.to_numpy(p), hip.to_numpy(q))
    tr.free_graph()


def test_gcn_replays_equal_eager_steps(hip):
    from zigrad_amd.trainers import GCNTrainer, gcn_inputs

    inp = gcn_inputs(n_nodes=600, n_features=200, n_pairs=1500, n_classes=7, n_train=60, hidden=16, seed=1)
    eager = GCNTrainer(hip, inp, lr=0.01, clip=True)
    want = [eager.step() for _ in range(8)]
    tr = GCNTrainer(hip, inp, lr=0.01, clip=True)
    got = [tr.step() for _ in range(2)]
    tr.capture()
    for _ in range(6):
        got.append(tr.step_graph())
        _eager_noise(hip)
    assert got == want
    for p, q in zip(eager.param_buffers(), tr.param_buffers()):
        assert np.array_equal(hip.to_numpy(p), hip.to_numpy(q))
    tr.free_graph()


def test_calls_that_cannot_be_recorded_are_refused(hip):
    a = hip.from_numpy(np.ones(16, np.float32), cached=True)
    hip.graph_open()
    try:
        for fn in (hip.sync, lambda: hip.to_numpy(a), lambda: hip.mem_alloc(F32, 4)):
            with pytest.raises(ZgHipError) as e:
                fn()
            assert e.value.code == 4  # ZG_HIP_ECAPTURE
        hip.dispatch("relu_fwd", x=a, y=a)  # ordinary ops are recorded
    finally:
        g = hip.graph_save()
    hip.mem_fill(a, -1.0)
    g.run()
    assert not hip.to_numpy(a).any()  # relu(-1) = 0: the recorded op ran on replay
    g.free()
    with pytest.raises(ZgHipError):
        hip.graph_save()  # no capture in progress
    hip.mem_cache_free(a)
