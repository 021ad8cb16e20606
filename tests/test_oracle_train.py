"""The MLP train-step op sequence, run on the CPU oracle, against an independent fp64 numpy backprop.

This pins the sequencing (which device ops backward issues, alpha/beta, the optimizer recurrences with
the per-tensor Adam counter, gradient clipping) without a GPU.
"""
from __future__ import annotations

import numpy as np
import pytest

from conftest import rel_fro
from zigrad_amd.trainers import MLPTrainer, mlp_inputs


def numpy_mlp_step(params, x, onehot):
    """Loss and gradients of Linear/ReLU/.../softmax-CE in float64."""
    p = [a.astype(np.float64) for a in params]
    n_layers = len(p) // 2
    acts = [x.astype(np.float64)]
    for l in range(n_layers):
        y = acts[-1] @ p[2 * l].T + p[2 * l + 1]
        if l + 1 < n_layers:
            y = np.maximum(y, 0)
        acts.append(y)
    z = acts[-1]
    z = z - z.max(axis=1, keepdims=True)
    sm = np.exp(z) / np.exp(z).sum(axis=1, keepdims=True)
    B = x.shape[0]
    loss = -np.sum(onehot * np.log(np.clip(sm, 1e-7, 1 - 1e-7))) / B
    g = (sm - onehot) / B
    grads = [None] * len(p)
    for l in reversed(range(n_layers)):
        if l + 1 < n_layers:
            g = g * (acts[l + 1] > 0)
        grads[2 * l + 1] = g.sum(axis=0)
        grads[2 * l] = g.T @ acts[l]
        g = g @ p[2 * l]
    return loss, grads


@pytest.mark.parametrize("dims,batch", [([784, 128, 64, 10], 64), ([20, 33, 7], 5)])
@pytest.mark.parametrize("loss_mode", ["onehot", "label"])
def test_mlp_gradients_match_numpy_backprop(oracle, dims, batch, loss_mode):
    params, x, onehot, labels = mlp_inputs(dims, batch, data="uniform")
    tr = MLPTrainer(oracle, dims, batch, optimizer="sgd", lr=0.01, clip=False, loss_mode=loss_mode)
    tr.load_params(params)
    tr.set_batch(x, onehot, labels)
    loss = tr.step(keep_grads=True)
    want_loss, want_grads = numpy_mlp_step(params, x, onehot)
    assert abs(loss - want_loss) <= 1e-5 * abs(want_loss)
    for got, want in zip(tr.last_grads, want_grads):
        assert rel_fro(got, want) <= 1e-5
    # SGD without clipping: p -= lr * g; gradients are zeroed afterwards
    for buf, p0, g in zip(tr.param_buffers(), params, want_grads):
        assert rel_fro(oracle.to_numpy(buf), p0.ravel() - 0.01 * g.ravel()) <= 1e-6
    for gb in tr.grad_buffers():
        assert not oracle.to_numpy(gb).any()


def test_adam_counter_is_per_tensor_and_clip_is_per_tensor(oracle):
    dims, batch = [12, 9, 4], 6
    params, x, onehot, labels = mlp_inputs(dims, batch, data="normal")
    params = [p * 40 for p in params]  # large weights -> gradients big enough for the clip to bite on some tensors
    tr = MLPTrainer(oracle, dims, batch, optimizer="adam", lr=1e-3, clip=True)
    tr.load_params(params)
    tr.set_batch(x * 30, onehot, labels)
    p = [a.astype(np.float64).ravel() for a in params]
    m = [np.zeros_like(a) for a in p]
    v = [np.zeros_like(a) for a in p]
    t = 0
    clipped = 0
    for _ in range(2):
        tr.step()
        _, grads = numpy_mlp_step([a.reshape(q.shape) for a, q in zip(p, params)], x * 30, onehot)
        for i, g in enumerate(grads):
            g = g.ravel()
            t += 1  # one increment per parameter tensor (src/nn/optim.zig:189)
            norm = np.linalg.norm(g)
            if norm > 10.0:
                g = g * (10.0 / (norm + 1e-6))
                clipped += 1
            lr_t = 1e-3 * np.sqrt(1 - 0.999 ** t) / (1 - 0.9 ** t)
            m[i] = 0.9 * m[i] + 0.1 * g
            v[i] = 0.999 * v[i] + 0.001 * g * g
            p[i] = p[i] - lr_t * m[i] / (np.sqrt(v[i]) + 1e-8)
    assert clipped > 0
    for buf, want in zip(tr.param_buffers(), p):
        assert rel_fro(oracle.to_numpy(buf), want) <= 1e-5


def test_allocator_traffic_is_balanced(oracle):
    dims, batch = [16, 8, 4], 4
    params, x, onehot, labels = mlp_inputs(dims, batch)
    tr = MLPTrainer(oracle, dims, batch)
    tr.load_params(params)
    tr.set_batch(x, onehot, labels)
    before = len(oracle._arrays)
    tr.step()
    assert len(oracle._arrays) == before  # every intermediate went back to the allocator


def numpy_gcn_step(inp):
    """Dense fp64 restatement of the two-layer GCN step: loss and gradients."""
    x = inp["x"].astype(np.float64)
    N = x.shape[0]
    src, tgt = inp["src"].astype(np.int64), inp["tgt"].astype(np.int64)
    A = np.zeros((N, N))
    np.add.at(A, (tgt, src), 1.0)
    deg = 1.0 + np.bincount(tgt, minlength=N)
    dn = 1.0 / np.sqrt(deg)
    Ah = dn[:, None] * A * dn[None, :]
    W1, b1, W2, b2 = [p.astype(np.float64) for p in inp["params"]]
    M = inp["n_train"]
    t = inp["onehot"][:M].astype(np.float64)
    z1 = Ah @ (x @ W1.T) + b1
    h1 = np.maximum(z1, 0)
    z2 = Ah @ (h1 @ W2.T) + b2
    zm = z2[:M] - z2[:M].max(axis=1, keepdims=True)
    sm = np.exp(zm) / np.exp(zm).sum(axis=1, keepdims=True)
    loss = -np.sum(t * np.log(np.clip(sm, 1e-7, 1 - 1e-7))) / M
    g2 = np.zeros_like(z2)
    g2[:M] = (sm - t) / M
    gb2 = g2.sum(axis=0)
    gh2 = Ah.T @ g2
    gW2 = gh2.T @ h1
    g1 = (gh2 @ W2) * (z1 > 0)
    gb1 = g1.sum(axis=0)
    gh1 = Ah.T @ g1
    gW1 = gh1.T @ x
    return loss, [gW1, gb1, gW2, gb2]


def test_gcn_gradients_match_dense_numpy(oracle):
    from zigrad_amd.trainers import GCNTrainer, gcn_inputs

    inp = gcn_inputs(n_nodes=300, n_features=40, n_pairs=700, n_classes=5, n_train=50, hidden=8, seed=3)
    tr = GCNTrainer(oracle, inp, lr=0.01, clip=False)
    loss = tr.step(keep_grads=True)
    want_loss, want = numpy_gcn_step(inp)
    assert abs(loss - want_loss) <= 1e-5 * abs(want_loss)
    for got, w in zip(tr.last_grads, want):
        assert rel_fro(got, w) <= 2e-5


def test_dqn_gradients_match_numpy(oracle):
    from zigrad_amd.trainers import DQNTrainer, dqn_inputs

    dims, batch = [4, 16, 16, 2], 32
    params, _, _, _ = mlp_inputs(dims, batch)
    params = [p + 0.05 for p in params]  # non-zero biases
    b = dqn_inputs(batch=batch)
    tr = DQNTrainer(oracle, dims, batch, lr=1e-3, gamma=0.99, clip=False)
    tr.load_params(params)
    tr.set_batch(b)
    loss = tr.step(keep_grads=True)

    def fwd(x, p):
        acts = [x.astype(np.float64)]
        for l in range(3):
            y = acts[-1] @ p[2 * l].astype(np.float64).T + p[2 * l + 1]
            acts.append(np.maximum(y, 0) if l < 2 else y)
        return acts

    qn = fwd(b["next_states"], params)[-1]
    target = b["rewards"] + 0.99 * qn.max(axis=1) * (1 - b["dones"])
    acts = fwd(b["states"], params)
    a = b["actions"].ravel().astype(np.int64)
    q = acts[-1][np.arange(batch), a]
    d = q - target
    want_loss = np.where(np.abs(d) < 1, 0.5 * d * d, np.abs(d) - 0.5).mean()
    assert abs(loss - want_loss) <= 1e-5 * abs(want_loss)
    g = np.zeros_like(acts[-1])
    g[np.arange(batch), a] = np.where(np.abs(d) < 1, d, np.sign(d)) / batch
    grads = [None] * 6
    for l in reversed(range(3)):
        if l < 2:
            g = g * (acts[l + 1] > 0)
        grads[2 * l + 1] = g.sum(axis=0)
        grads[2 * l] = g.T @ acts[l]
        g = g @ params[2 * l].astype(np.float64)
    for got, w in zip(tr.last_grads, grads):
        assert rel_fro(got, w) <= 1e-5
