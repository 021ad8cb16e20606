"""SafeTensors checkpoints of device-resident parameters and optimizer state (D2H / H2D staging instead of the
host-pointer reads of src/utils/layer_map.zig:334-448)."""
from __future__ import annotations

import numpy as np
import pytest

from zigrad_amd.checkpoint import read_header
from zigrad_amd.trainers import MLPTrainer, mlp_inputs


def _round_trip(dev, tmp_path):
    dims, batch = [20, 33, 7], 16
    params, x, onehot, labels = mlp_inputs(dims, batch)

    def make():
        tr = MLPTrainer(dev, dims, batch, optimizer="adam", lr=1e-3, clip=True)
        tr.load_params(params)
        tr.set_batch(x, onehot, labels)
        return tr

    a = make()
    for _ in range(3):
        a.step()
    path = tmp_path / "mlp.safetensors"
    a.save_checkpoint(path)
    want = [a.step() for _ in range(3)]

    b = make()
    b.load_checkpoint(path)
    assert b.optim.t == 3 * 4  # Adam's counter advances once per parameter tensor
    got = [b.step() for _ in range(3)]
    assert got == want  # parameters, both moments and the counter came back exactly
    return path, a


def test_checkpoint_round_trip_and_library_interop(oracle, tmp_path):
    path, tr = _round_trip(oracle, tmp_path)
    header, _ = read_header(path)
    assert header["__metadata__"]["optim.kind"] == "adam"
    w0 = header["layers.0.weights"]
    assert (w0["dtype"], w0["shape"]) == ("F32", [33, 20])
    assert w0["data_offsets"][1] - w0["data_offsets"][0] == 33 * 20 * 4
    # the file is an ordinary SafeTensors container: the stock library reads it and agrees with our own reader
    from safetensors.numpy import load_file, save_file

    theirs = load_file(str(path))
    assert set(theirs) == {k for k in header if k != "__metadata__"}
    fresh = MLPTrainer(oracle, [20, 33, 7], 16, optimizer="adam", lr=1e-3)
    fresh.load_checkpoint(path)
    for key, (buf, shape) in fresh.named_tensors().items():
        assert np.array_equal(oracle.to_numpy(buf).reshape(shape), theirs[key])
    # and a file written by the stock library loads here
    other = tmp_path / "theirs.safetensors"
    save_file(theirs, str(other), metadata={"optim.kind": "adam", "optim.t": "12"})
    again = MLPTrainer(oracle, [20, 33, 7], 16, optimizer="adam", lr=1e-3)
    again.load_checkpoint(other)
    assert again.optim.t == 12
    for key, (buf, shape) in again.named_tensors().items():
        assert np.array_equal(oracle.to_numpy(buf).reshape(shape), theirs[key])


def test_checkpoint_rejects_mismatched_shapes(oracle, tmp_path):
    path, _ = _round_trip(oracle, tmp_path)
    wrong = MLPTrainer(oracle, [20, 32, 7], 16, optimizer="adam", lr=1e-3)
    with pytest.raises(ValueError):
        wrong.load_checkpoint(path)
    sgd = MLPTrainer(oracle, [20, 33, 7], 16, optimizer="sgd", lr=1e-3)
    with pytest.raises(ValueError):
        sgd.load_checkpoint(path)


@pytest.mark.gpu
def test_checkpoint_round_trip_on_the_device(hip, tmp_path):
    _round_trip(hip, tmp_path)
