"""Train-step op sequences of the benchmark configurations, issued against a device object.

Each trainer reproduces the order in which Zigrad's example programs reach the device for one
training step -- forward ops, the loss, every backward op the autograd graph issues (with the same
alpha/beta), the optimizer update per parameter tensor and zero_grad -- including the allocator
traffic (every intermediate and every non-parameter gradient is taken from and returned to the
caching allocator, as eager teardown does).  Nothing here computes: all arithmetic happens in device
ops, so the same code runs on any object with the HipDevice interface.

Reference call stacks: examples/mnist/src/model.zig:34-110 and main-simple.zig:55-86 (MLP),
src/ndtensor.zig:780-796, 1050-1136 (bias add and matmul backward), src/nn/nn.zig:39-62 (relu_),
src/nn/loss.zig:130-171 (softmax cross-entropy), src/nn/optim.zig:46-58, 100-122, 177-234 (optimizers).
"""
from __future__ import annotations

import numpy as np

from . import host
from .device import DevBuf, F32, U64

# defaults of the reference's Settings (src/zigrad.zig:62-65)
GRAD_CLIP_MAX_NORM = 10.0
GRAD_CLIP_DELTA = 1e-6


def mlp_inputs(dims, batch, seed_weights=0, seed_data=1, data="normal"):
    """Synthetic parameters and one batch for an MLP classifier.

    Weights follow the reference's `.kaiming` initialiser, N(0,1) * sqrt(2 / fan_in)
    (src/device/host_device.zig:939-943), biases are zero; inputs are U[0,1) or N(0,1); labels uniform.
    Returns (params list [W0, b0, W1, b1, ...], x [batch, dims[0]], onehot [batch, classes], labels u64).
    """
    rw = np.random.default_rng(seed_weights)
    params = []
    for fan_in, fan_out in zip(dims[:-1], dims[1:]):
        w = rw.standard_normal((fan_out, fan_in), dtype=np.float32) * np.float32(np.sqrt(2.0 / fan_in))
        params.append(w.astype(np.float32))
        params.append(np.zeros(fan_out, np.float32))
    rd = np.random.default_rng(seed_data)
    if data == "uniform":
        x = rd.random((batch, dims[0]), dtype=np.float32)
    else:
        x = rd.standard_normal((batch, dims[0]), dtype=np.float32)
    labels = rd.integers(0, dims[-1], batch).astype(np.uint64)
    onehot = np.zeros((batch, dims[-1]), np.float32)
    onehot[np.arange(batch), labels.astype(np.int64)] = 1.0
    return params, x, onehot, labels


class Optimizer:
    """SGD / Adam over a list of attached parameter tensors, one fused device op per tensor."""

    def __init__(self, dev, kind: str, lr: float, clip: bool = True, max_norm: float = GRAD_CLIP_MAX_NORM,
                 delta: float = GRAD_CLIP_DELTA, beta1: float = 0.9, beta2: float = 0.999, epsilon: float = 1e-8):
        if kind not in ("sgd", "adam"):
            raise ValueError(f"unknown optimizer {kind!r}")
        self.dev, self.kind, self.lr, self.clip = dev, kind, lr, clip
        self.max_norm, self.delta = max_norm, delta
        self.beta1, self.beta2, self.epsilon = beta1, beta2, epsilon
        self.params: list[tuple[DevBuf, DevBuf]] = []
        self.state: list[tuple[DevBuf, DevBuf]] = []
        self.t = 0  # Adam's counter: incremented once per parameter tensor update (src/nn/optim.zig:189)

    def attach(self, param: DevBuf, grad: DevBuf) -> None:
        self.params.append((param, grad))
        if self.kind == "adam":
            m, v = self.dev.mem_alloc(F32, param.n), self.dev.mem_alloc(F32, param.n)
            self.dev.mem_fill(m, 0.0)
            self.dev.mem_fill(v, 0.0)
            self.state.append((m, v))

    def step(self) -> None:
        d = self.dev
        for i, (p, g) in enumerate(self.params):
            if self.kind == "sgd":
                d.dispatch("sgd_step", param=p, grad=g, lr=self.lr, clip=self.clip, max_norm=self.max_norm, delta=self.delta)
            else:
                self.t += 1
                m, v = self.state[i]
                d.dispatch("adam_step", param=p, grad=g, m=m, v=v, t=self.t, lr=self.lr, beta1=self.beta1, beta2=self.beta2,
                           epsilon=self.epsilon, clip=self.clip, max_norm=self.max_norm, delta=self.delta)


class MLPTrainer:
    """Linear -> ReLU -> ... -> Linear -> softmax cross-entropy, one train step per `step()` call.

    loss_mode "onehot" is the reference's loss (float one-hot targets, probabilities kept for backward);
    "label" is the fused integer-label form (same values, one pass over the logits).
    """

    def __init__(self, dev, dims, batch, optimizer="sgd", lr=0.01, clip=True, loss_mode="onehot"):
        self.dev, self.dims, self.batch, self.loss_mode = dev, list(dims), batch, loss_mode
        self.n_layers = len(dims) - 1
        self.W, self.b, self.Wg, self.bg = [], [], [], []
        self.optim = Optimizer(dev, optimizer, lr, clip)
        for fan_in, fan_out in zip(dims[:-1], dims[1:]):
            w, wg = dev.mem_alloc(F32, fan_in * fan_out), dev.mem_alloc(F32, fan_in * fan_out)
            b, bg = dev.mem_alloc(F32, fan_out), dev.mem_alloc(F32, fan_out)
            for g in (wg, bg):
                dev.mem_fill(g, 0.0)
            self.W.append(w)
            self.b.append(b)
            self.Wg.append(wg)
            self.bg.append(bg)
            self.optim.attach(w, wg)  # attach order of LinearLayer.init: weights, then bias
            self.optim.attach(b, bg)
        self.x = dev.mem_alloc(F32, batch * dims[0])
        self.onehot = dev.mem_alloc(F32, batch * dims[-1])
        self.labels = dev.mem_alloc(U64, batch)
        self.loss_host = np.zeros(1, np.float32)
        self.last_grads = None

    # -- data ----------------------------------------------------------------------------------
    def load_params(self, params) -> None:
        for l in range(self.n_layers):
            self.dev.mem_transfer(params[2 * l], self.W[l], "HtoD")
            self.dev.mem_transfer(params[2 * l + 1], self.b[l], "HtoD")

    def param_buffers(self):
        out = []
        for l in range(self.n_layers):
            out += [self.W[l], self.b[l]]
        return out

    def grad_buffers(self):
        out = []
        for l in range(self.n_layers):
            out += [self.Wg[l], self.bg[l]]
        return out

    def set_batch(self, x, onehot, labels=None) -> None:
        self.dev.mem_transfer(x, self.x, "HtoD")
        self.dev.mem_transfer(onehot, self.onehot, "HtoD")
        if labels is None:
            labels = np.argmax(onehot, axis=1).astype(np.uint64)
        self.dev.mem_transfer(labels, self.labels, "HtoD")

    # -- one step --------------------------------------------------------------------------------
    def forward(self):
        d, B = self.dev, self.batch
        acts = [self.x]
        for l in range(self.n_layers):
            fan_in, fan_out = self.dims[l], self.dims[l + 1]
            y = d.mem_cache_alloc(F32, B * fan_out)
            host.bmm_acc_(d, acts[-1], [B, fan_in], self.W[l], [fan_out, fan_in], y, trans_a=False, trans_b=True)
            d.dispatch("add", x=self.b[l], y=y, z=y)  # bias.add_(y): shorter operand first
            if l + 1 < self.n_layers:
                d.dispatch("relu_fwd", x=y, y=y)
            acts.append(y)
        return acts

    def step(self, read_loss: bool = True, keep_grads: bool = False):
        d, B, C = self.dev, self.batch, self.dims[-1]
        acts = self.forward()
        logits = acts[-1]
        loss = d.mem_cache_alloc(F32, 1)
        if self.loss_mode == "onehot":
            saved = d.mem_cache_alloc(F32, B * C)  # sm_preds
            d.dispatch("smce_fwd", logits=logits, target=self.onehot, probs=saved, loss=loss, rows=B, cols=C)
        else:
            saved = d.mem_cache_alloc(F32, B)  # per-row log-sum-exp
            d.dispatch("smce_label_fwd", logits=logits, labels=self.labels, lse=saved, loss=loss, rows=B, cols=C)
        loss_val = None
        if read_loss:
            d.mem_transfer(loss, self.loss_host, "DtoH")  # loss.get(0): a blocking read before backward
            loss_val = float(self.loss_host[0])

        # backward
        loss_grad = d.mem_cache_alloc(F32, 1)
        d.mem_fill(loss_grad, 1.0)
        g = d.mem_cache_alloc(F32, B * C)
        d.mem_fill(g, 0.0)
        if self.loss_mode == "onehot":
            d.dispatch("smce_bwd", probs=saved, target=self.onehot, grad=g, rows=B, cols=C)
        else:
            d.dispatch("smce_label_bwd", logits=logits, labels=self.labels, lse=saved, grad=g, rows=B, cols=C, accumulate=True)
        d.mem_cache_free(saved)
        d.mem_cache_free(loss_grad)
        d.mem_cache_free(loss)
        for l in reversed(range(self.n_layers)):
            fan_in, fan_out = self.dims[l], self.dims[l + 1]
            y = acts[l + 1]
            if l + 1 < self.n_layers:
                d.dispatch("relu_inplace_bwd", x=y, x_g=g)
            host.unbroadcast_(d, g, [B, fan_out], self.bg[l], [fan_out], alpha=1.0, beta=1.0)
            g_prev = None
            if l > 0:  # the network input does not require a gradient
                g_prev = d.mem_cache_alloc(F32, B * fan_in)
                d.mem_fill(g_prev, 0.0)
            host.bmm_acc_backward(d, False, True, acts[l], [B, fan_in], self.W[l], [fan_out, fan_in], g, [B, fan_out],
                                  g_prev, self.Wg[l])
            d.mem_cache_free(y)
            d.mem_cache_free(g)
            g = g_prev
        if keep_grads:
            self.last_grads = [d.to_numpy(b) for b in self.grad_buffers()]
        self.optim.step()
        for gb in self.grad_buffers():  # model.zero_grad()
            d.mem_fill(gb, 0.0)
        return loss_val
