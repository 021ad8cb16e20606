"""The headline configuration at its real size: wide MLP 4096 -> 4096 -> 4096 -> 1024, batch 4096, Adam with the
per-tensor gradient clip on, on the HIP device (op by op as the reference's loop issues it, and through the fused
entry points; float one-hot targets and integer labels) against the same step on the CPU oracle.

Op sequence: examples/mnist/src/model.zig:34-110 (Linear = bmm_acc(trans_b) + bias add, ReLU between layers),
src/nn/loss.zig:130-171, src/ndtensor.zig:1092-1136 (the five backward products), src/nn/optim.zig:177-234.

What is held to the full-step bound of 1e-4 relative Frobenius error, and how:
  * the loss and every layer output of the forward pass (in fact to 1e-5);
  * every gradient, with the oracle's backward pass started from the device's layer outputs;
  * every updated parameter and both Adam moments, with the oracle's optimizer started from the device's gradients;
  * the loss of the second step, end to end with nothing shared.
The backward pass cannot be compared end to end at this size: of the 33.5 million ReLU outputs a handful (5 + 8 in
this configuration) lie within rounding distance of zero and come out as +1e-6 on one device and as 0 on the other
(two fp32 GEMMs that sum in different orders), and relu_inplace_bwd (src/device/host_device.zig:543-547) gates the
gradient on `x <= 0`.  Each such entry switches one element of a 4096 x 4096 gradient on or off, which alone is a
relative difference of about 1e-3 in the weight gradients below it, between ANY two GEMM implementations.  The test
therefore counts those entries, checks that every one of them is within 1e-5 of zero, and compares the backward
pass from identical layer outputs.
"""
from __future__ import annotations

import numpy as np
import pytest

from conftest import rel_fro
from zigrad_amd.trainers import MLPTrainer, mlp_inputs

pytestmark = pytest.mark.gpu
STEP_TOL = 1e-4
OP_TOL = 1e-5
DIMS, BATCH = [4096, 4096, 4096, 1024], 4096


@pytest.fixture(scope="module")
def inputs():
    return mlp_inputs(DIMS, BATCH, seed_weights=0, seed_data=1, data="normal")


def _trainer(dev, inputs, loss_mode, fused=False):
    params, x, onehot, labels = inputs
    tr = MLPTrainer(dev, DIMS, BATCH, optimizer="adam", lr=1e-3, clip=True, loss_mode=loss_mode, fused=fused)
    tr.load_params(params)
    tr.set_batch(x, onehot, labels)
    return tr


def _state(dev, tr):
    return {"params": [dev.to_numpy(p) for p in tr.param_buffers()], "m": [dev.to_numpy(m) for m, _ in tr.optim.state],
            "v": [dev.to_numpy(v) for _, v in tr.optim.state], "t": tr.optim.t}


def _release(dev, tr):
    for b in tr.param_buffers() + tr.grad_buffers() + [s for mv in tr.optim.state for s in mv] + [tr.x, tr.onehot, tr.labels]:
        dev.mem_free(b)


@pytest.fixture(scope="module")
def oracle_free_runs(oracle, inputs):
    """Two oracle steps with nothing shared, once per loss form (the box's BLAS on 16 threads: about a second each)."""
    oracle.set_threads(16)
    out = {}
    for mode in ("onehot", "label"):
        tr = _trainer(oracle, inputs, mode)
        losses = [tr.step(keep_acts=True), tr.step()]
        out[mode] = {"losses": losses, "acts": tr.last_acts}
        _release(oracle, tr)
    return out


@pytest.mark.parametrize("fused", [False, True], ids=["op_by_op", "fused"])
@pytest.mark.parametrize("loss_mode", ["onehot", "label"])
def test_wide_mlp_step_matches_oracle_at_full_size(hip, oracle, inputs, oracle_free_runs, loss_mode, fused):
    free = oracle_free_runs[loss_mode]
    tr = _trainer(hip, inputs, loss_mode, fused)
    loss1 = tr.step(keep_grads=True, keep_acts=True)
    acts, grads = tr.last_acts, tr.last_grads
    after1 = _state(hip, tr)
    loss2 = tr.step()
    _release(hip, tr)

    # forward pass and loss, end to end
    assert abs(loss1 - free["losses"][0]) <= OP_TOL * abs(free["losses"][0]), (loss1, free["losses"])
    flips = 0
    for a, b in zip(free["acts"], acts):
        assert rel_fro(b, a) <= OP_TOL
        differ = (a > 0) != (b > 0)
        flips += int(np.count_nonzero(differ))
        if differ.any():  # an output is positive on one side only: both values must be at rounding distance from zero
            assert float(np.maximum(np.abs(a[differ]), np.abs(b[differ])).max()) <= 1e-5
    assert flips <= 64, flips
    # second step, end to end: the few gated gradient elements above move the next loss far less than the bound
    assert abs(loss2 - free["losses"][1]) <= STEP_TOL * abs(free["losses"][1]), (loss2, free["losses"])
    assert loss2 < loss1

    # backward pass from the device's layer outputs, optimizer from the device's gradients
    forced = _trainer(oracle, inputs, loss_mode)
    loss_o = forced.step(keep_grads=True, force={"acts": acts, "grads": grads})
    want = _state(oracle, forced)
    want_grads = forced.last_grads
    _release(oracle, forced)
    assert abs(loss1 - loss_o) <= OP_TOL * abs(loss_o)
    for i, (a, b) in enumerate(zip(want_grads, grads)):
        assert np.isfinite(b).all(), i
        assert rel_fro(b, a) <= STEP_TOL, ("grad", i, rel_fro(b, a))
    assert after1["t"] == want["t"] == 6  # six parameter tensors: the counter moves once per tensor (src/nn/optim.zig:189)
    for key in ("params", "m", "v"):
        for i, (a, b) in enumerate(zip(want[key], after1[key])):
            assert np.isfinite(b).all(), (key, i)
            assert rel_fro(b, a) <= STEP_TOL, (key, i, rel_fro(b, a))
    # softmax minus one-hot sums to zero along every row, so the last bias gradient (its column sums) sums to zero
    assert abs(float(grads[5].astype(np.float64).sum())) <= 1e-5


def test_the_fifty_step_run_amplifies_a_one_ulp_difference(hip, inputs):
    """The benchmark definition runs this configuration for 50 steps on one batch.  Past the first few steps the losses of two
    fp32 implementations cannot be compared: 4096 samples with random labels are memorised within five steps and Adam
    at lr 1e-3 then overshoots, and in that regime the run multiplies any difference by about ten per step.  Shown here
    on the device alone: moving ONE of the 37.7 million weights by one unit in the last place changes the loss by more
    than 1e-4 (relative) within 12 steps.  Device and oracle differ by a rounding in every element of every product,
    so their losses agree to 1e-6 at step 2, 6e-5 at step 3 and 5e-4 at step 5 (measured); the end-to-end comparison above
    therefore stops at the second step, and the steps after it are covered op by op."""
    params, x, onehot, labels = inputs
    runs = []
    for perturb in (False, True):
        p2 = [q.copy() for q in params]
        if perturb:
            flat = p2[0].reshape(-1)
            flat[12345] = np.nextafter(flat[12345], np.float32(10.0))
        tr = _trainer(hip, (p2, x, onehot, labels), "onehot")
        runs.append([tr.step() for _ in range(12)])
        _release(hip, tr)
    rel = [abs(a - b) / abs(a) for a, b in zip(*runs)]
    assert rel[0] <= 1e-6 and rel[1] <= 1e-6  # the change is invisible at first
    assert max(rel) > 1e-4, rel
