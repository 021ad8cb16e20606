"""The fused Linear entry points against the ops they stand for (examples/mnist/src/model.zig:104-110 forward,
src/ndtensor.zig:1092-1136 + src/device/host_device.zig:543-547 backward): bit for bit against the separate device
ops on the same inputs, to 1e-5 against float64, on shapes that reach every GEMM path (tiny, split-k, fast, edge and
checked kernels of each tile size), and whole train steps with and without fusion."""
from __future__ import annotations

import numpy as np
import pytest

from conftest import run_op
from zigrad_amd.trainers import MLPTrainer, mlp_inputs

pytestmark = pytest.mark.gpu

# (batch, fan_in, fan_out)
SHAPES = [(64, 784, 128), (64, 128, 64), (64, 64, 10), (1, 5, 3), (33, 70, 129), (256, 512, 384), (250, 512, 380),
          (512, 96, 1024), (1024, 1024, 1024), (2048, 4096, 512), (130, 1433, 16), (300, 260, 7), (2048, 1000, 1024)]


def _unfused_fwd(dev, x, w, b, relu):
    B, I = x.shape
    O = w.shape[0]
    y = run_op(dev, "matmul", {"A": x, "B": w, "C": np.zeros((B, O), np.float32), "m": B, "n": O, "k": I, "trans_a": False,
                               "trans_b": True, "lda": I, "ldb": I, "ldc": O, "alpha": 1.0, "beta": 0.0}, ["C"])["C"]
    if b is not None:
        y = run_op(dev, "add", {"x": b, "y": y, "z": np.zeros_like(y)}, ["z"])["z"]
    if relu:
        y = run_op(dev, "relu_fwd", {"x": y, "y": np.zeros_like(y)}, ["y"])["y"]
    return y.reshape(B, O)


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("relu,with_bias", [(True, True), (False, True), (True, False)])
def test_linear_fwd_equals_the_three_ops(oracle, hip, shape, relu, with_bias):
    B, I, O = shape
    r = np.random.default_rng(B * 31 + I * 7 + O)
    x = r.standard_normal((B, I)).astype(np.float32)
    w = (r.standard_normal((O, I)) / np.sqrt(I)).astype(np.float32)
    b = r.standard_normal(O).astype(np.float32) if with_bias else None
    p = {"x": x, "w": w, "bias": b, "y": np.full((B, O), np.nan, np.float32), "batch": B, "fan_in": I, "fan_out": O,
         "relu": relu}
    got = run_op(hip, "linear_fwd", dict(p), ["y"])["y"].reshape(B, O)
    assert np.array_equal(got, _unfused_fwd(hip, x, w, b, relu)), shape
    want = x.astype(np.float64) @ w.astype(np.float64).T + (b.astype(np.float64) if with_bias else 0.0)
    if relu:
        want = np.maximum(want, 0.0)
    assert np.linalg.norm(got - want) <= 1e-5 * (np.linalg.norm(want) + 1e-3), shape
    if B * I * O <= 1 << 22:  # the CPU oracle's composition of the same three ops
        ref = run_op(oracle, "linear_fwd", dict(p), ["y"])["y"].reshape(B, O)
        assert np.linalg.norm(got - ref) <= 1e-5 * (np.linalg.norm(ref) + 1e-3), shape


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("accumulate,masked", [(False, True), (True, True), (False, False)])
def test_linear_bwd_input_equals_product_then_relu_backward(hip, shape, accumulate, masked):
    B, I, O = shape
    r = np.random.default_rng(B * 13 + I * 5 + O + 1)
    gy = r.standard_normal((B, O)).astype(np.float32)
    w = (r.standard_normal((O, I)) / np.sqrt(O)).astype(np.float32)
    act = np.maximum(r.standard_normal((B, I)), 0.0).astype(np.float32) if masked else None  # a ReLU output: half zeros
    gx0 = r.standard_normal((B, I)).astype(np.float32) if accumulate else np.full((B, I), np.nan, np.float32)
    got = run_op(hip, "linear_bwd_input", {"gy": gy, "w": w, "act_in": act, "gx": gx0.copy(), "batch": B, "fan_in": I,
                                            "fan_out": O, "accumulate": accumulate}, ["gx"])["gx"].reshape(B, I)
    base = gx0.copy() if accumulate else np.zeros((B, I), np.float32)
    ref = run_op(hip, "matmul", {"A": gy, "B": w, "C": base, "m": B, "n": I, "k": O, "trans_a": False, "trans_b": False,
                                 "lda": O, "ldb": I, "ldc": I, "alpha": 1.0, "beta": 1.0}, ["C"])["C"]
    if masked:
        ref = run_op(hip, "relu_inplace_bwd", {"x": act, "x_g": ref}, ["x_g"])["x_g"]
    assert np.array_equal(got, ref.reshape(B, I)), shape
    want = gy.astype(np.float64) @ w.astype(np.float64) + (gx0 if accumulate else 0.0)
    if masked:
        want = np.where(act > 0, want, 0.0)
    assert np.linalg.norm(got - want) <= 1e-5 * (np.linalg.norm(want) + 1e-3), shape


@pytest.mark.parametrize("shape", SHAPES + [(64, 4, 128), (64, 128, 2), (128, 128, 128), (256, 100, 64), (257, 100, 64),
                                            (10, 128, 1), (256, 38, 1), (1, 20, 30), (1, 1, 1)])
@pytest.mark.parametrize("with_gx,with_gb", [(True, True), (False, True), (True, False)])
def test_linear_bwd_equals_the_separate_ops(oracle, hip, shape, with_gx, with_gb):
    """One call against the weight-gradient product, the bias's unbroadcast and linear_bwd_input on the same device,
    bit for bit (small layers take one launch, the others the separate ops); against float64 and the CPU oracle's
    composition to 1e-5."""
    B, I, O = shape
    r = np.random.default_rng(B * 7 + I * 3 + O + 5)
    gy = r.standard_normal((B, O)).astype(np.float32)
    x = np.maximum(r.standard_normal((B, I)), 0.0).astype(np.float32)  # a ReLU output: layer input and mask
    w = (r.standard_normal((O, I)) / np.sqrt(O)).astype(np.float32)
    gw0 = r.standard_normal((O, I)).astype(np.float32)
    gb0 = r.standard_normal(O).astype(np.float32)
    p = {"gy": gy, "x": x, "w": w, "act_in": x if with_gx else None, "gw": gw0.copy(), "gb": gb0.copy() if with_gb else None,
         "gx": np.full((B, I), np.nan, np.float32) if with_gx else None, "batch": B, "fan_in": I, "fan_out": O}
    outs = ["gw"] + (["gb"] if with_gb else []) + (["gx"] if with_gx else [])
    got = run_op(hip, "linear_bwd", dict(p), outs)
    ref_gw = run_op(hip, "matmul", {"A": gy, "B": x, "C": gw0.copy(), "m": O, "n": I, "k": B, "trans_a": True,
                                    "trans_b": False, "lda": O, "ldb": I, "ldc": I, "alpha": 1.0, "beta": 1.0}, ["C"])["C"]
    assert np.array_equal(got["gw"], ref_gw), shape
    want_gw = gy.astype(np.float64).T @ x.astype(np.float64) + gw0
    assert np.linalg.norm(got["gw"] - want_gw) <= 1e-5 * (np.linalg.norm(want_gw) + 1e-3)
    if with_gb:
        ref_gb = run_op(hip, "unbroadcast", {"x": gy, "x_shape": [B, O], "y": gb0.copy(), "y_shape": [O], "alpha": 1.0,
                                             "beta": 1.0}, ["y"])["y"]
        assert np.array_equal(got["gb"], ref_gb), shape
        want_gb = gy.astype(np.float64).sum(axis=0) + gb0
        assert np.linalg.norm(got["gb"] - want_gb) <= 1e-5 * (np.linalg.norm(want_gb) + 1e-3)
    if with_gx:
        ref_gx = run_op(hip, "linear_bwd_input", {"gy": gy, "w": w, "act_in": x, "gx": np.full((B, I), np.nan, np.float32),
                                                  "batch": B, "fan_in": I, "fan_out": O, "accumulate": False}, ["gx"])["gx"]
        assert np.array_equal(got["gx"], ref_gx), shape
        want_gx = np.where(x > 0, gy.astype(np.float64) @ w.astype(np.float64), 0.0)
        assert np.linalg.norm(got["gx"] - want_gx) <= 1e-5 * (np.linalg.norm(want_gx) + 1e-3)
    if B * I * O <= 1 << 22:
        ref = run_op(oracle, "linear_bwd", dict(p), outs)
        for name in outs:
            assert np.linalg.norm(got[name] - ref[name]) <= 1e-5 * (np.linalg.norm(ref[name]) + 1e-3), (shape, name)


@pytest.mark.parametrize("dims,batch,optimizer", [([784, 128, 64, 10], 64, "sgd"), ([100, 260, 130, 7], 50, "adam"),
                                                  ([512, 768, 384, 32], 512, "adam")])
def test_train_steps_with_and_without_fusion_agree_exactly(hip, dims, batch, optimizer):
    params, x, onehot, labels = mlp_inputs(dims, batch, seed_weights=3, seed_data=4, data="normal")
    out = []
    for fused in (False, True):
        tr = MLPTrainer(hip, dims, batch, optimizer=optimizer, lr=0.01, clip=True, fused=fused)
        tr.load_params(params)
        tr.set_batch(x, onehot, labels)
        losses = [tr.step() for _ in range(4)]
        out.append((losses, [hip.to_numpy(b) for b in tr.param_buffers()]))
    assert out[0][0] == out[1][0]
    for a, b in zip(out[0][1], out[1][1]):
        assert np.array_equal(a, b)


def test_fused_step_replays_from_an_execution_graph(hip):
    dims, batch = [784, 128, 64, 10], 64
    params, x, onehot, labels = mlp_inputs(dims, batch, data="uniform")
    eager = MLPTrainer(hip, dims, batch, optimizer="sgd", lr=0.01, clip=True, fused=True)
    graph = MLPTrainer(hip, dims, batch, optimizer="sgd", lr=0.01, clip=True, fused=True)
    for tr in (eager, graph):
        tr.load_params(params)
        tr.set_batch(x, onehot, labels)
    graph.capture()
    for _ in range(5):
        assert eager.step() == graph.step_graph()
        hip.sync()
    for a, b in zip(eager.param_buffers(), graph.param_buffers()):
        assert np.array_equal(hip.to_numpy(a), hip.to_numpy(b))
    graph.free_graph()


@pytest.mark.parametrize("kind", ["sgd", "adam"])
@pytest.mark.parametrize("clip,zero", [(True, True), (True, False), (False, True)])
def test_optimizer_list_entry_points_equal_the_per_tensor_ops(hip, kind, clip, zero):
    """Sizes either side of every limit (update slices of 2048, Adam's one-workgroup path up to 4096, the one-launch
    norm up to 131072, the shared update launch up to 2^20), a list longer than one launch holds (16), gradients large
    enough that the clip is active for some tensors and not for others."""
    from zigrad_amd.device import F32

    r = np.random.default_rng(7)
    sizes = [1, 10, 128, 640, 2048, 2049, 4096, 4097, 8192, 65536, 65537, 100352, 131072, 131073, 3, 64, (1 << 20), (1 << 20) + 4] + [int(r.integers(1, 5000)) for _ in range(14)]
    host = [(r.standard_normal(n).astype(np.float32), (r.standard_normal(n) * r.choice([0.01, 3.0])).astype(np.float32),
             (r.standard_normal(n) * 0.1).astype(np.float32), (r.random(n) * 0.1).astype(np.float32)) for n in sizes]
    beta1, beta2, eps, lr = 0.9, 0.999, 1e-8, 0.01
    out = []
    for multi in (False, True):
        bufs = [[hip.from_numpy(a) for a in t] for t in host]
        if multi and kind == "sgd":
            hip.dispatch("sgd_step_multi", params=[b[0] for b in bufs], grads=[b[1] for b in bufs], lr=lr, clip=clip,
                         max_norm=10.0, delta=1e-6, zero_grads=zero)
        elif multi:
            hip.dispatch("adam_step_multi", params=[b[0] for b in bufs], grads=[b[1] for b in bufs], ms=[b[2] for b in bufs],
                         vs=[b[3] for b in bufs], lr=lr, t_first=5, beta1=beta1, beta2=beta2, epsilon=eps, clip=clip,
                         max_norm=10.0, delta=1e-6, zero_grads=zero)
        else:
            for i, (p, g, m, v) in enumerate(bufs):
                if kind == "sgd":
                    hip.dispatch("sgd_step", param=p, grad=g, lr=lr, clip=clip, max_norm=10.0, delta=1e-6)
                else:
                    hip.dispatch("adam_step", param=p, grad=g, m=m, v=v, t=5 + i, lr=lr, beta1=beta1, beta2=beta2,
                                 epsilon=eps, clip=clip, max_norm=10.0, delta=1e-6)
                if zero:
                    hip.mem_fill(g, 0.0)
        out.append([[hip.to_numpy(b) for b in t] for t in bufs])
        for t in bufs:
            for b in t:
                hip.mem_free(b)
    for i, (a, b) in enumerate(zip(*out)):
        for which, (x, y) in enumerate(zip(a, b)):
            if kind == "sgd" and which >= 2:
                continue
            assert np.array_equal(x, y), (sizes[i], which)


def test_optimizer_list_with_a_tensor_listed_twice_updates_it_twice(hip):
    """Shared weights that appear twice in the parameter list get two updates, the second on the result of the first,
    as the per-tensor loop gives them (src/nn/optim.zig:100-122)."""
    r = np.random.default_rng(11)
    n = 5000
    p0, g0 = r.standard_normal(n).astype(np.float32), (3.0 * r.standard_normal(n)).astype(np.float32)
    q0, h0 = r.standard_normal(77).astype(np.float32), r.standard_normal(77).astype(np.float32)
    out = []
    for multi in (False, True):
        p, g, q, h = (hip.from_numpy(a) for a in (p0, g0, q0, h0))
        if multi:
            hip.dispatch("sgd_step_multi", params=[p, q, p], grads=[g, h, g], lr=0.1, clip=True, max_norm=10.0, delta=1e-6,
                         zero_grads=False)
        else:
            for a, b in ((p, g), (q, h), (p, g)):
                hip.dispatch("sgd_step", param=a, grad=b, lr=0.1, clip=True, max_norm=10.0, delta=1e-6)
        out.append([hip.to_numpy(t) for t in (p, g, q, h)])
        for t in (p, g, q, h):
            hip.mem_free(t)
    for x, y in zip(*out):
        assert np.array_equal(x, y)


def test_dqn_and_gcn_steps_with_and_without_fusion_agree_exactly(hip):
    from zigrad_amd.trainers import DQNTrainer, GCNTrainer, dqn_inputs, gcn_inputs

    dims, batch = [4, 128, 128, 2], 64
    params, _, _, _ = mlp_inputs(dims, batch)
    inp = gcn_inputs(n_nodes=500, n_features=200, n_pairs=1500, n_train=40, hidden=16, seed=2)
    for make in (lambda f: DQNTrainer(hip, dims, batch, fused=f), lambda f: GCNTrainer(hip, inp, fused=f)):
        out = []
        for fused in (False, True):
            tr = make(fused)
            if isinstance(tr, DQNTrainer):
                tr.load_params(params)
                tr.set_batch(dqn_inputs(batch=batch))
            losses = [tr.step() for _ in range(4)]
            out.append((losses, [hip.to_numpy(b) for b in tr.param_buffers()]))
        assert out[0][0] == out[1][0]
        for a, b in zip(out[0][1], out[1][1]):
            assert np.array_equal(a, b)


def test_fused_adam_step_replays_from_an_execution_graph(hip):
    from zigrad_amd.trainers import DQNTrainer, dqn_inputs

    dims, batch = [4, 128, 128, 2], 64
    params, _, _, _ = mlp_inputs(dims, batch)
    eager, graph = DQNTrainer(hip, dims, batch, fused=True), DQNTrainer(hip, dims, batch, fused=True)
    for tr in (eager, graph):
        tr.load_params(params)
        tr.set_batch(dqn_inputs(batch=batch))
    graph.step()
    eager.step()
    graph.capture()
    for _ in range(5):
        assert eager.step() == graph.step_graph()
        hip.sync()
    for a, b in zip(eager.param_buffers(), graph.param_buffers()):
        assert np.array_equal(hip.to_numpy(a), hip.to_numpy(b))
    graph.free_graph()


def test_fused_gcn_step_with_an_edge_plan_replays_from_an_execution_graph(hip):
    from zigrad_amd.trainers import GCNTrainer, gcn_inputs

    inp = gcn_inputs(n_nodes=500, n_features=200, n_pairs=1500, n_train=40, hidden=16, seed=3)
    eager, graph = GCNTrainer(hip, inp, fused=True), GCNTrainer(hip, inp, fused=True)
    graph.step()
    eager.step()
    graph.capture()
    for _ in range(4):
        assert eager.step() == graph.step_graph()
        hip.sync()
    for a, b in zip(eager.param_buffers(), graph.param_buffers()):
        assert np.array_equal(hip.to_numpy(a), hip.to_numpy(b))
    graph.free_graph()


@pytest.mark.parametrize("rows,cols", [(64, 10), (140, 7), (256, 32), (257, 32), (1, 1), (64, 256), (65, 256), (16, 4096),
                                       (17, 4096), (3, 1000), (5, 33), (700, 1024), (2, 5000),
                                       # one pass over rows held in registers: a wave per row, a workgroup per row
                                       (1024, 1024), (1500, 260), (1100, 1000), (3, 8192), (2, 32768), (5, 4100),
                                       # 4, 16 and 64 lanes per row on either side of the one-launch limit; a workgroup of
                                       # 256 threads per row with 4 and with 8 pieces each
                                       (3000, 8), (300, 32), (700, 36), (65, 256), (1500, 256), (17, 1024), (40, 1028),
                                       (21, 2048), (9, 4096), (6, 8192), (5, 8196)])
@pytest.mark.parametrize("accumulate", [False, True])
def test_smce_fwd_bwd_equals_forward_then_backward(oracle, hip, rows, cols, accumulate):
    """One call against smce_fwd + smce_bwd (src/nn/loss.zig:130-159) on the same device, bit for bit, on both sides
    of the one-launch limit; against the CPU oracle's composition to 1e-5."""
    r = np.random.default_rng(rows * 131 + cols)
    logits = r.standard_normal((rows, cols)).astype(np.float32)  # label probabilities stay above the 1e-7 clamp
    target = np.zeros((rows, cols), np.float32)
    target[np.arange(rows), r.integers(0, cols, rows)] = 1.0
    g0 = r.standard_normal((rows, cols)).astype(np.float32)
    nan = np.full((rows, cols), np.nan, np.float32)
    p = {"logits": logits, "target": target, "probs": nan.copy(), "loss": np.full(1, np.nan, np.float32),
         "grad": g0.copy() if accumulate else nan.copy(), "rows": rows, "cols": cols, "accumulate": accumulate}
    got = run_op(hip, "smce_fwd_bwd", dict(p), ["probs", "loss", "grad"])
    fwd = run_op(hip, "smce_fwd", {"logits": logits, "target": target, "probs": nan.copy(), "loss": np.zeros(1, np.float32),
                                   "rows": rows, "cols": cols}, ["probs", "loss"])
    bwd = run_op(hip, "smce_bwd", {"probs": fwd["probs"], "target": target,
                                   "grad": g0.copy() if accumulate else np.zeros((rows, cols), np.float32),
                                   "rows": rows, "cols": cols}, ["grad"])
    assert np.array_equal(got["probs"], fwd["probs"])
    assert np.array_equal(got["loss"], fwd["loss"])
    assert np.array_equal(got["grad"], bwd["grad"])
    ref = run_op(oracle, "smce_fwd_bwd", dict(p), ["probs", "loss", "grad"])
    for name in ("probs", "loss", "grad"):
        assert np.linalg.norm(got[name].ravel() - ref[name].ravel()) <= 1e-5 * (np.linalg.norm(ref[name].ravel()) + 1e-6), name
    # closed form: rows of the written gradient sum to zero, the loss is the mean of -log clamp(p[label])
    if not accumulate:
        assert np.abs(got["grad"].reshape(rows, cols).astype(np.float64).sum(axis=1)).max() <= 1e-6
    x = logits.astype(np.float64)
    lse = np.log(np.exp(x - x.max(axis=1, keepdims=True)).sum(axis=1)) + x.max(axis=1)
    p_label = np.clip(np.exp((x * target).sum(axis=1) - lse), 1e-7, np.float64(np.float32(1.0 - 1e-7)))  # the clamp of loss.zig:143
    want = np.mean(-np.log(p_label))
    assert abs(float(got["loss"][0]) - want) <= 1e-5 * (abs(want) + 1e-3)


@pytest.mark.parametrize("n", [1, 64, 4096, 4097, 100001])
@pytest.mark.parametrize("accumulate", [False, True])
def test_smooth_l1_fwd_bwd_equals_forward_then_backward(oracle, hip, n, accumulate):
    """One call against smooth_l1_fwd + smooth_l1_bwd (src/nn/loss.zig:259-305) on the same device, bit for bit, on
    both sides of the one-launch limit; against the closed form and the CPU oracle's composition to 1e-5."""
    r = np.random.default_rng(n)
    pred = (2.0 * r.standard_normal(n)).astype(np.float32)
    target = r.standard_normal(n).astype(np.float32)
    g0 = r.standard_normal(n).astype(np.float32)
    p = {"pred": pred, "target": target, "grad": g0.copy() if accumulate else np.full(n, np.nan, np.float32), "beta": 1.0,
         "loss": np.full(1, np.nan, np.float32), "accumulate": accumulate}
    got = run_op(hip, "smooth_l1_fwd_bwd", dict(p), ["grad", "loss"])
    fwd = run_op(hip, "smooth_l1_fwd", {"pred": pred, "target": target, "beta": 1.0, "loss": np.zeros(1, np.float32)}, ["loss"])
    bwd = run_op(hip, "smooth_l1_bwd", {"pred": pred, "target": target, "grad": g0.copy() if accumulate else np.zeros(n, np.float32),
                                        "beta": 1.0}, ["grad"])
    assert np.array_equal(got["loss"], fwd["loss"])
    assert np.array_equal(got["grad"], bwd["grad"])
    d = pred.astype(np.float64) - target
    want_loss = np.mean(np.where(np.abs(d) < 1.0, 0.5 * d * d, np.abs(d) - 0.5))
    want_grad = np.where(np.abs(d) < 1.0, d, np.sign(d)) / n + (g0 if accumulate else 0.0)
    assert abs(float(got["loss"][0]) - want_loss) <= 1e-5 * (abs(want_loss) + 1e-6)
    assert np.linalg.norm(got["grad"] - want_grad) <= 1e-5 * (np.linalg.norm(want_grad) + 1e-9)
    ref = run_op(oracle, "smooth_l1_fwd_bwd", dict(p), ["grad", "loss"])
    assert np.linalg.norm(got["grad"] - ref["grad"]) <= 1e-5 * (np.linalg.norm(ref["grad"]) + 1e-9)
    assert abs(float(got["loss"][0]) - float(ref["loss"][0])) <= 1e-5 * (abs(float(ref["loss"][0])) + 1e-6)
