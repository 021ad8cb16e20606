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


def test_checkpoint_keys_follow_the_layer_map_convention(oracle, tmp_path):
    """LayerMap builds a key from struct field names joined by "." (src/utils/layer_map.zig:91, :320-326) and its
    serialiser writes one SafeTensors entry per key with the element type's name (:346-354: f32 -> F32).  The leaf
    names are the fields of the reference's LinearLayer (examples/mnist/src/model.zig:70-71: `weights`, `bias`).
    The reference's own MLP example never serialises and LayerMap's struct walk has no rule for arrays, so the
    `layers.<index>` component is this build's; the test pins the rest."""
    path, tr = _round_trip(oracle, tmp_path)
    header, _ = read_header(path)
    keys = sorted(k for k in header if k != "__metadata__")
    params = [k for k in keys if not k.startswith("optim.")]
    assert params == sorted(f"layers.{l}.{leaf}" for l in range(2) for leaf in ("weights", "bias"))
    for k in keys:
        assert header[k]["dtype"] == "F32" and all(part for part in k.split("."))
    assert header["layers.1.weights"]["shape"] == [7, 33]   # [out, in], as LinearLayer stores it (model.zig:75)
    assert header["layers.1.bias"]["shape"] == [7]
    # Adam's state: one first and one second moment per parameter, same shapes (src/nn/optim.zig:126-130)
    state = [k for k in keys if k.startswith("optim.")]
    assert len(state) == 2 * len(params)
    for k in params:
        shapes = {tuple(header[s]["shape"]) for s in state if s.endswith(k)}
        assert shapes == {tuple(header[k]["shape"])}


def _trainer(dev, dims, batch, params, x, onehot, labels):
    tr = MLPTrainer(dev, dims, batch, optimizer="adam", lr=1e-3, clip=True)
    tr.load_params(params)
    tr.set_batch(x, onehot, labels)
    return tr


@pytest.mark.gpu
def test_checkpoint_round_trip_on_the_device(hip, tmp_path):
    _round_trip(hip, tmp_path)


@pytest.mark.gpu
@pytest.mark.parametrize("writer", ["oracle", "hip"])
def test_checkpoint_crosses_between_host_oracle_and_device(hip, oracle, tmp_path, writer):
    """A file written on one device continues the run on the other: the bytes in the file are the writer's
    parameters and moments exactly, and the next three losses are the writer's own to 1e-4."""
    dims, batch = [96, 160, 48, 12], 64
    params, x, onehot, labels = mlp_inputs(dims, batch)
    src_dev, dst_dev = (oracle, hip) if writer == "oracle" else (hip, oracle)
    a = _trainer(src_dev, dims, batch, params, x, onehot, labels)
    for _ in range(4):
        a.step()
    path = tmp_path / "cross.safetensors"
    a.save_checkpoint(path)
    from safetensors.numpy import load_file

    on_disk = load_file(str(path))
    for key, (buf, shape) in a.named_tensors().items():
        assert np.array_equal(src_dev.to_numpy(buf).reshape(shape), on_disk[key])
    want = [a.step() for _ in range(3)]

    b = _trainer(dst_dev, dims, batch, params, x, onehot, labels)
    b.load_checkpoint(path)
    assert b.optim.t == a.optim.t - 3 * 6
    for key, (buf, shape) in b.named_tensors().items():
        assert np.array_equal(dst_dev.to_numpy(buf).reshape(shape), on_disk[key])
    got = [b.step() for _ in range(3)]
    for w, g in zip(want, got):
        assert abs(w - g) <= 1e-4 * max(1.0, abs(w)), (want, got)
    for p, q in zip(a.param_buffers(), b.param_buffers()):
        pa, qa = src_dev.to_numpy(p).astype(np.float64), dst_dev.to_numpy(q).astype(np.float64)
        assert np.linalg.norm(pa - qa) <= 1e-4 * np.linalg.norm(pa)
