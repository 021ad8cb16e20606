"""The CPU oracle's compositions for the fused entry points (linear_fwd, linear_bwd_input, linear_bwd, smce_fwd_bwd,
the planned GCN aggregation with its bias / ReLU tail, the list optimizers) against closed forms written out in numpy
float64: the GPU tests compare the device with these compositions, so a composition that dropped a term, transposed
an operand or applied the mask to the wrong tensor has to fail here, without a GPU."""
from __future__ import annotations

import numpy as np
import pytest

from conftest import run_op


def _close(a, b, tol=1e-5):
    a, b = np.asarray(a, np.float64).ravel(), np.asarray(b, np.float64).ravel()
    return np.linalg.norm(a - b) <= tol * (np.linalg.norm(b) + 1e-6)


@pytest.mark.parametrize("B,I,O", [(5, 7, 3), (64, 128, 10), (33, 70, 129), (1, 4, 1)])
def test_oracle_linear_compositions(oracle, B, I, O):
    r = np.random.default_rng(B + 10 * I + 100 * O)
    x = np.maximum(r.standard_normal((B, I)), 0.0).astype(np.float32)
    w = r.standard_normal((O, I)).astype(np.float32)
    b = r.standard_normal(O).astype(np.float32)
    y = run_op(oracle, "linear_fwd", {"x": x, "w": w, "bias": b, "y": np.full((B, O), np.nan, np.float32), "batch": B,
                                      "fan_in": I, "fan_out": O, "relu": True}, ["y"])["y"]
    assert _close(y, np.maximum(x.astype(np.float64) @ w.astype(np.float64).T + b, 0.0))
    gy = r.standard_normal((B, O)).astype(np.float32)
    gw0, gb0 = r.standard_normal((O, I)).astype(np.float32), r.standard_normal(O).astype(np.float32)
    got = run_op(oracle, "linear_bwd", {"gy": gy, "x": x, "w": w, "act_in": x, "gw": gw0.copy(), "gb": gb0.copy(),
                                        "gx": np.full((B, I), np.nan, np.float32), "batch": B, "fan_in": I, "fan_out": O},
                 ["gw", "gb", "gx"])
    assert _close(got["gw"], gy.astype(np.float64).T @ x.astype(np.float64) + gw0)      # not x^T gy, and accumulated
    assert _close(got["gb"], gy.astype(np.float64).sum(axis=0) + gb0)                   # over the batch, accumulated
    assert _close(got["gx"], np.where(x > 0, gy.astype(np.float64) @ w.astype(np.float64), 0.0))  # masked by the input
    gx = run_op(oracle, "linear_bwd_input", {"gy": gy, "w": w, "act_in": None, "gx": x.copy(), "batch": B, "fan_in": I,
                                             "fan_out": O, "accumulate": True}, ["gx"])["gx"]
    assert _close(gx, gy.astype(np.float64) @ w.astype(np.float64) + x)


@pytest.mark.parametrize("rows,cols,accumulate", [(4, 5, False), (64, 10, True), (140, 7, False)])
def test_oracle_smce_fwd_bwd(oracle, rows, cols, accumulate):
    r = np.random.default_rng(rows * cols)
    logits = r.standard_normal((rows, cols)).astype(np.float32)
    target = np.zeros((rows, cols), np.float32)
    target[np.arange(rows), r.integers(0, cols, rows)] = 1.0
    g0 = r.standard_normal((rows, cols)).astype(np.float32)
    got = run_op(oracle, "smce_fwd_bwd", {"logits": logits, "target": target, "probs": np.full((rows, cols), np.nan, np.float32),
                                          "loss": np.full(1, np.nan, np.float32),
                                          "grad": g0.copy() if accumulate else np.full((rows, cols), np.nan, np.float32),
                                          "rows": rows, "cols": cols, "accumulate": accumulate}, ["probs", "loss", "grad"])
    x = logits.astype(np.float64)
    p = np.exp(x - x.max(axis=1, keepdims=True))
    p /= p.sum(axis=1, keepdims=True)
    assert _close(got["probs"], p)
    assert abs(float(got["loss"][0]) - np.mean(-np.log((p * target).sum(axis=1)))) <= 1e-5
    assert _close(got["grad"], (p - target) / rows + (g0 if accumulate else 0.0))


def test_oracle_planned_gcn_aggregation_with_tail(oracle):
    r = np.random.default_rng(3)
    n_nodes, n_edge, stride = 40, 300, 6
    src = r.integers(0, n_nodes, n_edge).astype(np.uint64)
    tgt = r.integers(0, n_nodes - 3, n_edge).astype(np.uint64)  # the last three nodes receive nothing
    h = r.standard_normal((n_nodes, stride)).astype(np.float32)
    deg = (r.random(n_nodes) + 0.5).astype(np.float32)
    bias = r.standard_normal(stride).astype(np.float32)
    plan = oracle.edge_plan(oracle.from_numpy(src), oracle.from_numpy(tgt), n_nodes)
    got = run_op(oracle, "scatter_gcn_deg_scaled_planned", {"dst": np.full((n_nodes, stride), np.nan, np.float32), "h": h,
                                                           "deg": deg, "plan": plan, "stride": stride, "accumulate": False,
                                                           "bias": bias, "relu": True}, ["dst"])["dst"]
    adj = np.zeros((n_nodes, n_nodes))
    for s, t in zip(src, tgt):
        adj[int(t), int(s)] += 1.0
    want = np.maximum((deg[:, None] * adj * deg[None, :]) @ h.astype(np.float64) + bias, 0.0)  # D A D h + b, then relu
    assert _close(got, want)
    assert np.array_equal(got[-3:], np.maximum(np.tile(bias, (3, 1)), 0.0))  # isolated rows: relu(bias) exactly


@pytest.mark.parametrize("kind", ["sgd", "adam"])
def test_oracle_list_optimizers_follow_the_per_tensor_recurrence(oracle, kind):
    """Two steps over three tensors, against the recurrences of src/nn/optim.zig:100-122 and :177-234 in float64,
    with the per-tensor step counter (tensor i of step s uses t = (s - 1) * 3 + i + 1) and the clip active on one
    tensor only."""
    r = np.random.default_rng(5)
    sizes = [7, 300, 33]
    p0 = [r.standard_normal(n).astype(np.float32) for n in sizes]
    g0 = [(r.standard_normal(n) * s).astype(np.float32) for n, s in zip(sizes, (0.1, 5.0, 0.1))]  # only the second is clipped
    lr, b1, b2, eps, max_norm, delta = 0.05, 0.9, 0.999, 1e-8, 10.0, 1e-6
    from zigrad_amd.device import F32

    P = [oracle.from_numpy(a) for a in p0]
    G = [oracle.from_numpy(a) for a in g0]
    M = [oracle.from_numpy(np.zeros(n, np.float32)) for n in sizes]
    V = [oracle.from_numpy(np.zeros(n, np.float32)) for n in sizes]
    p = [a.astype(np.float64) for a in p0]
    m = [np.zeros(n) for n in sizes]
    v = [np.zeros(n) for n in sizes]
    t = 0
    for step in range(2):
        if kind == "sgd":
            oracle.dispatch("sgd_step_multi", params=P, grads=G, lr=lr, clip=True, max_norm=max_norm, delta=delta, zero_grads=False)
        else:
            oracle.dispatch("adam_step_multi", params=P, grads=G, ms=M, vs=V, lr=lr, t_first=t + 1, beta1=b1, beta2=b2,
                            epsilon=eps, clip=True, max_norm=max_norm, delta=delta, zero_grads=False)
        for i in range(3):
            g = oracle.to_numpy(G[i]).astype(np.float64) if step else g0[i].astype(np.float64)
            if step == 0:
                nrm = np.linalg.norm(g)
                if nrm > max_norm:
                    g = g * (max_norm / (nrm + delta))
            t += 1
            if kind == "sgd":
                p[i] = p[i] - lr * g
            else:
                m[i] = b1 * m[i] + (1 - b1) * g
                v[i] = b2 * v[i] + (1 - b2) * g * g
                p[i] = p[i] - lr * np.sqrt(1 - b2 ** t) / (1 - b1 ** t) * m[i] / (np.sqrt(v[i]) + eps)
    for i in range(3):
        assert _close(oracle.to_numpy(P[i]), p[i], 1e-5), (kind, i)
    # the clip rescaled the second gradient in place to max_norm, and left the others alone
    assert abs(np.linalg.norm(oracle.to_numpy(G[1]).astype(np.float64)) - max_norm) <= 1e-3
    assert np.array_equal(oracle.to_numpy(G[0]), g0[0])


@pytest.mark.parametrize("accumulate", [False, True])
def test_oracle_smooth_l1_fwd_bwd(oracle, accumulate):
    r = np.random.default_rng(9)
    n = 200
    pred, target = (2.0 * r.standard_normal(n)).astype(np.float32), r.standard_normal(n).astype(np.float32)
    g0 = r.standard_normal(n).astype(np.float32)
    got = run_op(oracle, "smooth_l1_fwd_bwd", {"pred": pred, "target": target, "grad": g0.copy() if accumulate else np.full(n, np.nan, np.float32),
                                               "beta": 1.0, "loss": np.full(1, np.nan, np.float32), "accumulate": accumulate},
                 ["grad", "loss"])
    d = pred.astype(np.float64) - target
    assert abs(float(got["loss"][0]) - np.mean(np.where(np.abs(d) < 1.0, 0.5 * d * d, np.abs(d) - 0.5))) <= 1e-6
    assert _close(got["grad"], np.where(np.abs(d) < 1.0, d, np.sign(d)) / n + (g0 if accumulate else 0.0))


def test_oracle_gather_in_one_call(oracle):
    r = np.random.default_rng(4)
    src = r.standard_normal((5, 6, 7)).astype(np.float32)
    idx = r.integers(0, 6, (5, 4, 7)).astype(np.uint64)
    S, I = oracle.from_numpy(src), oracle.from_numpy(idx)
    O, D = oracle.from_numpy(np.zeros(idx.size, np.uint64)), oracle.from_numpy(np.full(idx.size, np.nan, np.float32))
    assert oracle.gather(S, [5, 6, 7], [5, 4, 7], I, 1, O, D) == 0
    want = np.take_along_axis(src[:, :, :], idx.astype(np.int64), axis=1)
    assert np.array_equal(oracle.to_numpy(D), want.ravel())
    assert np.array_equal(src.ravel()[oracle.to_numpy(O).astype(np.int64)], want.ravel())
