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

import ctypes

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
                 delta: float = GRAD_CLIP_DELTA, beta1: float = 0.9, beta2: float = 0.999, epsilon: float = 1e-8,
                 fused: bool = False):
        if kind not in ("sgd", "adam"):
            raise ValueError(f"unknown optimizer {kind!r}")
        self.dev, self.kind, self.lr, self.clip = dev, kind, lr, clip
        self.fused = fused  # step_and_zero_grad() through the list entry points: same values, fewer launches
        self.max_norm, self.delta = max_norm, delta
        self.beta1, self.beta2, self.epsilon = beta1, beta2, epsilon
        self.params: list[tuple[DevBuf, DevBuf]] = []
        self.state: list[tuple[DevBuf, DevBuf]] = []
        self.t = 0  # Adam's counter: incremented once per parameter tensor update (src/nn/optim.zig:189)
        self.capturing = False  # set while a trainer records its step into an execution graph
        self.lr_slots = None    # Adam under replay: one lr_t per tensor in pinned host memory the kernels read
        self._lr_view = None

    def attach(self, param: DevBuf, grad: DevBuf) -> None:
        self.params.append((param, grad))
        if self.kind == "adam":
            m, v = self.dev.mem_alloc(F32, param.n), self.dev.mem_alloc(F32, param.n)
            self.dev.mem_fill(m, 0.0)
            self.dev.mem_fill(v, 0.0)
            self.state.append((m, v))

    def state_tensors(self, names) -> dict:
        """{key: (buffer, shape)} of Adam's moments, keyed like the parameters they belong to."""
        out = {}
        if self.kind == "adam":
            for (name, shape), (m, v) in zip(names, self.state):
                out[f"optim.m.{name}"] = (m, shape)
                out[f"optim.v.{name}"] = (v, shape)
        return out

    def begin_capture(self) -> None:
        """Before recording a step: Adam's lr_t changes every step, so the recorded kernels read it from memory."""
        if self.kind == "adam" and self.lr_slots is None:
            n = len(self.params)
            self.lr_slots = self.dev.mem_alloc_host(F32, n)
            self._lr_view = np.ctypeslib.as_array((ctypes.c_float * n).from_address(self.lr_slots.ptr))
        self.capturing = True

    def prepare_replay(self) -> None:
        """Host part of one replayed step: advance the per-tensor counter and publish each tensor's lr_t.
        The previous replay must have finished (GraphSteps.step_graph waits for it when the loss was not read)."""
        if self.kind != "adam":
            return
        for i in range(len(self.params)):
            self.t += 1
            self._lr_view[i] = self.dev.adam_lr_t(self.lr, self.beta1, self.beta2, self.t)

    def step_and_zero_grad(self) -> bool:
        """optim.step() + model.zero_grad() through the list entry points; False when this optimizer is not fused
        (the caller then issues the two separately)."""
        if not self.fused:
            return False
        d = self.dev
        params, grads = [p for p, _ in self.params], [g for _, g in self.params]
        common = dict(clip=self.clip, max_norm=self.max_norm, delta=self.delta, zero_grads=True)
        if self.kind == "sgd":
            d.dispatch("sgd_step_multi", params=params, grads=grads, lr=self.lr, **common)
            return True
        d.dispatch("adam_step_multi", params=params, grads=grads, ms=[m for m, _ in self.state],
                   vs=[v for _, v in self.state], lr=self.lr, t_first=self.t + 1, beta1=self.beta1, beta2=self.beta2,
                   epsilon=self.epsilon, lr_t_mem=self.lr_slots if self.capturing else None, **common)
        if not self.capturing:
            self.t += len(params)  # once per tensor (src/nn/optim.zig:189)
        return True

    def step(self) -> None:
        d = self.dev
        for i, (p, g) in enumerate(self.params):
            if self.kind == "sgd":
                d.dispatch("sgd_step", param=p, grad=g, lr=self.lr, clip=self.clip, max_norm=self.max_norm, delta=self.delta)
            elif self.capturing:
                m, v = self.state[i]
                d.dispatch("adam_step_at", param=p, grad=g, m=m, v=v, lr_t=self.lr_slots.sub(i, 1), beta1=self.beta1,
                           beta2=self.beta2, epsilon=self.epsilon, clip=self.clip, max_norm=self.max_norm, delta=self.delta)
            else:
                self.t += 1
                m, v = self.state[i]
                d.dispatch("adam_step", param=p, grad=g, m=m, v=v, t=self.t, lr=self.lr, beta1=self.beta1, beta2=self.beta2,
                           epsilon=self.epsilon, clip=self.clip, max_norm=self.max_norm, delta=self.delta)


class GraphSteps:
    """capture() / step_graph() for trainers whose step() touches the host only to read the loss: the step is
    recorded once as an execution graph (src/device/cuda_device.zig:558-611) and replayed with one launch."""

    graph = None
    _capturing = False

    _loss_pinned = None
    _loss_view = None

    def _init_loss_slot(self) -> None:
        """One float of pinned host memory the device posts the loss into (allocated with the trainer: driver
        allocations are refused while a step is being recorded)."""
        self._loss_pinned = self.dev.mem_alloc_host(F32, 1)
        self._loss_view = self.dev.host_view(self._loss_pinned)

    def _read_loss(self, loss: DevBuf):
        """loss.get(0): the device posts the value into pinned host memory on its stream (a copy kernel when the step
        is being recorded) and the host waits for the stream; cheaper than a blocking driver copy of four bytes."""
        self.dev.mem_copy(loss, self._loss_pinned)
        if self._capturing:  # nothing executes while recording
            return None
        self.dev.sync()
        return float(self._loss_view[0])

    def capture(self) -> None:
        """Record one step.  Run at least one eager step first, so that the allocator and the library's internal
        workspace have reached their final size (growing either is refused while recording)."""
        self.optim.begin_capture()
        self.dev.graph_open()
        self._capturing = True
        try:
            self.step()
        finally:
            self._capturing = False
            self.optim.capturing = False
            self.graph = self.dev.graph_save()

    _replay_pending = False

    def step_graph(self, read_loss: bool = True):
        # Adam's recorded kernels read each tensor's lr_t from pinned host memory when they run: the slots may only
        # be rewritten once the previous replay has finished
        if self._replay_pending and self.optim.kind == "adam":
            self.dev.sync()
        self.optim.prepare_replay()
        self.graph.run()
        if not read_loss:
            self._replay_pending = True
            return None
        self.dev.sync()
        self._replay_pending = False
        return float(self._loss_view[0])

    def free_graph(self) -> None:
        if self.graph is not None:
            self.graph.free()
            self.graph = None


class BatchStager:
    """Double-buffered upload of training batches from pinned host memory on the device's copy stream, so the
    upload of batch k+1 overlaps the kernels of batch k.  (The reference uploads each batch with a blocking
    NDTensor.from_slice, examples/mnist/src/dataset.zig:51-52.)

    `specs` lists (dtype, element count) of the arrays that make up one batch.  Protocol per step:
        bufs = stager.current()        # device buffers holding batch k
        stager.prefetch(arrays_k1)     # start uploading batch k+1 into the other slot
        ... issue the ops of step k on bufs ...
        stager.advance()
    """

    def __init__(self, dev, specs):
        self.dev = dev
        self.pinned = [[dev.mem_alloc_host(dt, n) for dt, n in specs] for _ in range(2)]
        self.views = [[dev.host_view(b) for b in slot] for slot in self.pinned]
        self.device = [[dev.mem_alloc(dt, n) for dt, n in specs] for _ in range(2)]
        self.slot = 0

    def upload_first(self, arrays) -> None:
        for a, dst in zip(arrays, self.device[self.slot]):
            self.dev.mem_transfer(np.ascontiguousarray(a).ravel(), dst, "HtoD")

    def current(self):
        return self.device[self.slot]

    def prefetch(self, arrays=None) -> None:
        """Upload the next batch.  With `arrays` = None the pinned slot is sent as it is (a loader that writes
        straight into `views[slot ^ 1]` needs no extra host copy)."""
        d, nxt = self.dev, self.slot ^ 1
        d.staging_wait()  # the copy that last read pinned[nxt] (two steps ago) has long finished; make it certain
        if arrays is not None:
            for a, view in zip(arrays, self.views[nxt]):
                np.copyto(view, np.asarray(a).ravel())
        d.compute_after_staging()   # the ops issued next wait for the upload of the current batch
        d.staging_after_compute()   # the new upload waits for the ops already issued, which read device[nxt]
        for src, dst in zip(self.pinned[nxt], self.device[nxt]):
            d.staged_h2d(src, dst)

    def advance(self) -> None:
        self.slot ^= 1

    def free(self) -> None:
        self.dev.staging_wait()
        self.dev.sync()
        for slot in self.pinned + self.device:
            for b in slot:
                self.dev.mem_free(b)


class MLP:
    """Parameters, gradients and the forward/backward op sequences of a ReLU multi-layer perceptron whose
    Linear layers follow examples/mnist/src/model.zig:64-110 (weights [out, in], forward x . W^T + bias)."""

    def __init__(self, dev, dims, optim: Optimizer | None = None, fused: bool = False):
        self.dev, self.dims, self.fused = dev, list(dims), fused
        self.n_layers = len(dims) - 1
        self.W, self.b, self.Wg, self.bg = [], [], [], []
        for fan_in, fan_out in zip(dims[:-1], dims[1:]):
            w, wg = dev.mem_alloc(F32, fan_in * fan_out), dev.mem_alloc(F32, fan_in * fan_out)
            b, bg = dev.mem_alloc(F32, fan_out), dev.mem_alloc(F32, fan_out)
            for g in (wg, bg):
                dev.mem_fill(g, 0.0)
            self.W.append(w)
            self.b.append(b)
            self.Wg.append(wg)
            self.bg.append(bg)
            if optim is not None:
                optim.attach(w, wg)  # attach order of LinearLayer.init: weights, then bias
                optim.attach(b, bg)

    def load_params(self, params) -> None:
        for l in range(self.n_layers):
            self.dev.mem_transfer(params[2 * l], self.W[l], "HtoD")
            self.dev.mem_transfer(params[2 * l + 1], self.b[l], "HtoD")

    def copy_params_from(self, other: "MLP") -> None:
        for l in range(self.n_layers):
            self.dev.mem_copy(other.W[l], self.W[l])
            self.dev.mem_copy(other.b[l], self.b[l])

    def param_buffers(self):
        return [buf for l in range(self.n_layers) for buf in (self.W[l], self.b[l])]

    def grad_buffers(self):
        return [buf for l in range(self.n_layers) for buf in (self.Wg[l], self.bg[l])]

    def zero_grad(self) -> None:
        for gb in self.grad_buffers():
            self.dev.mem_fill(gb, 0.0)

    def forward(self, x: DevBuf, batch: int):
        """Returns the activations [x, y_1, ..., y_L]; y_l are cache allocations owned by the caller."""
        d = self.dev
        acts = [x]
        for l in range(self.n_layers):
            fan_in, fan_out = self.dims[l], self.dims[l + 1]
            y = d.mem_cache_alloc(F32, batch * fan_out)
            if self.fused:  # the same three ops in one launch
                d.dispatch("linear_fwd", x=acts[-1], w=self.W[l], bias=self.b[l], y=y, batch=batch, fan_in=fan_in,
                           fan_out=fan_out, relu=l + 1 < self.n_layers)
                acts.append(y)
                continue
            host.bmm_acc_(d, acts[-1], [batch, fan_in], self.W[l], [fan_out, fan_in], y, trans_a=False, trans_b=True)
            d.dispatch("add", x=self.b[l], y=y, z=y)  # bias.add_(y): shorter operand first
            if l + 1 < self.n_layers:
                d.dispatch("relu_fwd", x=y, y=y)
            acts.append(y)
        return acts

    def free_activations(self, acts) -> None:
        for y in acts[1:]:
            self.dev.mem_cache_free(y)

    def backward(self, acts, g: DevBuf, batch: int) -> None:
        """g is the gradient of the last activation (a cache allocation; consumed).  Every activation and
        intermediate gradient goes back to the allocator as soon as its backward ran (eager teardown)."""
        d = self.dev
        for l in reversed(range(self.n_layers)):
            fan_in, fan_out = self.dims[l], self.dims[l + 1]
            y = acts[l + 1]
            if self.fused:
                # g arrives with this layer's ReLU backward applied (by the product that made it); the input
                # gradient is written, not accumulated, so it needs no zero fill
                g_prev = d.mem_cache_alloc(F32, batch * fan_in) if l > 0 else None
                d.dispatch("linear_bwd", gy=g, x=acts[l], w=self.W[l], act_in=acts[l] if l > 0 else None, gw=self.Wg[l],
                           gb=self.bg[l], gx=g_prev, batch=batch, fan_in=fan_in, fan_out=fan_out)
                d.mem_cache_free(y)
                d.mem_cache_free(g)
                g = g_prev
                continue
            if l + 1 < self.n_layers:
                d.dispatch("relu_inplace_bwd", x=y, x_g=g)
            host.unbroadcast_(d, g, [batch, fan_out], self.bg[l], [fan_out], alpha=1.0, beta=1.0)
            g_prev = None
            if l > 0:  # the network input does not require a gradient
                g_prev = d.mem_cache_alloc(F32, batch * fan_in)
                d.mem_fill(g_prev, 0.0)
            host.bmm_acc_backward(d, False, True, acts[l], [batch, fan_in], self.W[l], [fan_out, fan_in], g,
                                  [batch, fan_out], g_prev, self.Wg[l])
            d.mem_cache_free(y)
            d.mem_cache_free(g)
            g = g_prev


class MLPTrainer(GraphSteps):
    """Linear -> ReLU -> ... -> Linear -> softmax cross-entropy, one train step per `step()` call.

    loss_mode "onehot" is the reference's loss (float one-hot targets, probabilities kept for backward);
    "label" is the fused integer-label form (same values, one pass over the logits).  fused=True issues every
    Linear layer through the fused entry points (bias and ReLU in the GEMM epilogue, ReLU backward in the epilogue
    of the input-gradient product): same arithmetic, fewer launches and passes over the activations.
    """

    def __init__(self, dev, dims, batch, optimizer="sgd", lr=0.01, clip=True, loss_mode="onehot", fused=False):
        self.dev, self.dims, self.batch, self.loss_mode = dev, list(dims), batch, loss_mode
        self.optim = Optimizer(dev, optimizer, lr, clip, fused=fused)
        self.net = MLP(dev, dims, self.optim, fused=fused)
        self.n_layers = self.net.n_layers
        self.x = dev.mem_alloc(F32, batch * dims[0])
        self.onehot = dev.mem_alloc(F32, batch * dims[-1])
        self.labels = dev.mem_alloc(U64, batch)
        self._init_loss_slot()
        self.last_grads = None

    def load_params(self, params) -> None:
        self.net.load_params(params)

    def param_buffers(self):
        return self.net.param_buffers()

    def grad_buffers(self):
        return self.net.grad_buffers()

    def set_batch(self, x, onehot, labels=None) -> None:
        self.dev.mem_transfer(x, self.x, "HtoD")
        self.dev.mem_transfer(onehot, self.onehot, "HtoD")
        if labels is None:
            labels = np.argmax(onehot, axis=1).astype(np.uint64)
        self.dev.mem_transfer(labels, self.labels, "HtoD")

    def named_tensors(self) -> dict:
        """Parameters and optimizer state under dotted keys (the LayerMap convention, src/utils/layer_map.zig)."""
        names, out = [], {}
        for l in range(self.n_layers):
            fan_in, fan_out = self.dims[l], self.dims[l + 1]
            for key, buf, shape in ((f"layers.{l}.weights", self.net.W[l], [fan_out, fan_in]),
                                    (f"layers.{l}.bias", self.net.b[l], [fan_out])):
                out[key] = (buf, shape)
                names.append((key, shape))
        out.update(self.optim.state_tensors(names))
        return out

    def save_checkpoint(self, path) -> None:
        from .checkpoint import save_tensors

        save_tensors(path, self.dev, self.named_tensors(),
                     {"optim.kind": self.optim.kind, "optim.t": self.optim.t, "optim.lr": repr(self.optim.lr)})

    def load_checkpoint(self, path) -> None:
        from .checkpoint import load_tensors

        meta = load_tensors(path, self.dev, self.named_tensors())
        if meta.get("optim.kind", self.optim.kind) != self.optim.kind:
            raise ValueError(f"checkpoint was written by {meta['optim.kind']}, this trainer uses {self.optim.kind}")
        self.optim.t = int(meta.get("optim.t", 0))

    def use_batch(self, x: DevBuf, onehot: DevBuf, labels: DevBuf) -> None:
        """Train on batch buffers owned by the caller (a BatchStager slot) from the next step on."""
        self.x, self.onehot, self.labels = x, onehot, labels

    def step(self, read_loss=True, keep_grads: bool = False, keep_acts: bool = False, force: dict | None = None):
        """One train step.  read_loss=True reads the loss where the reference's loop does (loss.get(0) before
        backward, examples/mnist/src/main-simple.zig:67): the host blocks there and the GPU idles until the backward
        launches arrive.  read_loss="late" moves the same read behind the optimizer step, so the queue never drains.

        keep_acts / keep_grads read the layer outputs / the gradients back into last_acts / last_grads.
        force = {"acts": [...], "grads": [...]} (host arrays, either key optional) overwrites the layer outputs after
        the forward pass and the gradients after the backward pass: two devices can then run the backward pass and
        the optimizer from identical inputs, which takes the ReLU's discontinuity at zero out of a comparison (an
        output that rounds to +1e-7 on one device and to 0 on the other gates a whole gradient row differently)."""
        d, B, C = self.dev, self.batch, self.dims[-1]
        acts = self.net.forward(self.x, B)
        if keep_acts:
            self.last_acts = [d.to_numpy(a) for a in acts[1:]]
        if force and "acts" in force:
            for buf, a in zip(acts[1:], force["acts"]):
                d.mem_transfer(a, buf, "HtoD")
        logits = acts[-1]
        loss = d.mem_cache_alloc(F32, 1)
        if self.optim.fused and self.loss_mode == "onehot":
            # forward and the loss's backward in one call; the gradient is written, so it needs no zero fill
            saved, g = d.mem_cache_alloc(F32, B * C), d.mem_cache_alloc(F32, B * C)
            d.dispatch("smce_fwd_bwd", logits=logits, target=self.onehot, probs=saved, loss=loss, grad=g, rows=B, cols=C,
                       accumulate=False)
            loss_val = self._read_loss(loss) if read_loss is True else None
            d.mem_cache_free(saved)
        else:
            if self.loss_mode == "onehot":
                saved = d.mem_cache_alloc(F32, B * C)  # sm_preds
                d.dispatch("smce_fwd", logits=logits, target=self.onehot, probs=saved, loss=loss, rows=B, cols=C)
            else:
                saved = d.mem_cache_alloc(F32, B)  # per-row log-sum-exp
                d.dispatch("smce_label_fwd", logits=logits, labels=self.labels, lse=saved, loss=loss, rows=B, cols=C)
            loss_val = self._read_loss(loss) if read_loss is True else None  # loss.get(0): a blocking read before backward

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
        self.net.backward(acts, g, B)
        if keep_grads:
            self.last_grads = [d.to_numpy(b) for b in self.grad_buffers()]
        if force and "grads" in force:
            for buf, g_host in zip(self.grad_buffers(), force["grads"]):
                d.mem_transfer(g_host, buf, "HtoD")
        if not self.optim.step_and_zero_grad():
            self.optim.step()
            self.net.zero_grad()  # model.zero_grad()
        if read_loss == "late":
            loss_val = self._read_loss(loss)
        d.mem_cache_free(loss)
        return loss_val


def dqn_inputs(batch=64, state_dim=4, n_actions=2, seed=0):
    """Synthetic replay batch: states / next states N(0,1), actions uniform, rewards U[0,1), done = 0."""
    r = np.random.default_rng(seed)
    return {
        "states": r.standard_normal((batch, state_dim), dtype=np.float32),
        "next_states": r.standard_normal((batch, state_dim), dtype=np.float32),
        "actions": r.integers(0, n_actions, (batch, 1)).astype(np.uint64),
        "rewards": r.random(batch, dtype=np.float32),
        "dones": np.zeros(batch, np.float32),
    }


class DQNTrainer(GraphSteps):
    """One DQN update per `step()`: TD target from a frozen copy of the network, Q(s,a) through gather,
    smooth-L1 loss, Adam.  Op order follows DQNAgent.train (examples/dqn/src/dqn_agent.zig:125-228) without
    its host-side clamps, on the network 4 -> 128 -> 128 -> 2."""

    def __init__(self, dev, dims=(4, 128, 128, 2), batch=64, lr=1e-3, gamma=0.99, clip=True, fused=False,
                 device_scalars=False):
        self.dev, self.dims, self.batch, self.gamma = dev, list(dims), batch, gamma
        self.optim = Optimizer(dev, "adam", lr, clip, fused=fused)
        self.policy = MLP(dev, dims, self.optim, fused=fused)
        self.target = MLP(dev, dims, None, fused=fused)
        B, S, A = batch, dims[0], dims[-1]
        self.states, self.next_states = dev.mem_alloc(F32, B * S), dev.mem_alloc(F32, B * S)
        self.actions = dev.mem_alloc(U64, B)
        self.rewards, self.dones = dev.mem_alloc(F32, B), dev.mem_alloc(F32, B)
        # gamma and 1: host scalars, as NDArray's scalar ops hand them over (`.y = &.{s}`, src/ndarray.zig:247-257);
        # with device_scalars they are one-element tensors in device memory, the form the example builds
        # (examples/dqn/src/dqn_agent.zig:173-181).  Same values either way.
        if device_scalars:
            self.gamma_t = dev.from_numpy(np.asarray([gamma], np.float32))
            self.one_t = dev.from_numpy(np.asarray([1.0], np.float32))
        else:
            self.gamma_t, self.one_t = float(np.float32(gamma)), 1.0
        self._init_loss_slot()
        self.last_grads = None

    def load_params(self, params) -> None:
        self.policy.load_params(params)
        self.target.copy_params_from(self.policy)

    def set_batch(self, b) -> None:
        d = self.dev
        d.mem_transfer(b["states"], self.states, "HtoD")
        d.mem_transfer(b["next_states"], self.next_states, "HtoD")
        d.mem_transfer(b["actions"].ravel(), self.actions, "HtoD")
        d.mem_transfer(b["rewards"], self.rewards, "HtoD")
        d.mem_transfer(b["dones"], self.dones, "HtoD")

    def param_buffers(self):
        return self.policy.param_buffers()

    def step(self, keep_grads: bool = False) -> float:
        d, B, A = self.dev, self.batch, self.dims[-1]
        # TD target, no gradient
        acts_t = self.target.forward(self.next_states, B)
        max_next = d.mem_cache_alloc(F32, B)
        d.mem_fill(max_next, 0.0)  # NDArray.max_along writes into a zero-filled output (src/ndarray.zig:567)
        d.dispatch("max_along", x=acts_t[-1], x_shape=[B, A], y=max_next, y_shape=[B], dim=1)
        self.target.free_activations(acts_t)
        disc = d.mem_cache_alloc(F32, B)
        d.dispatch("mul", x=max_next, y=self.gamma_t, z=disc)
        not_done = d.mem_cache_alloc(F32, B)
        d.dispatch("sub", x=self.one_t, y=self.dones, z=not_done)
        masked = d.mem_cache_alloc(F32, B)
        d.dispatch("mul", x=disc, y=not_done, z=masked)
        targets = d.mem_cache_alloc(F32, B)
        d.dispatch("add", x=self.rewards, y=masked, z=targets)
        for t in (max_next, disc, not_done, masked):
            d.mem_cache_free(t)
        # Q(s, a)
        acts = self.policy.forward(self.states, B)
        q_all = acts[-1]
        q, offsets = host.gather(d, q_all, [B, A], self.actions, [B, 1], 1, return_offsets=True, check=False)
        loss = d.mem_cache_alloc(F32, 1)
        loss_grad = d.mem_cache_alloc(F32, 1)
        g_q = d.mem_cache_alloc(F32, B)
        if self.optim.fused:
            # forward and the loss's backward in one call, the gradient written (no fills); the fused optimizer step
            # leaves the parameter gradients zero for the next step
            d.dispatch("smooth_l1_fwd_bwd", pred=q, target=targets, grad=g_q, beta=1.0, loss=loss, accumulate=False)
        else:
            d.dispatch("smooth_l1_fwd", pred=q, target=targets, beta=1.0, loss=loss)
            self.policy.zero_grad()
            # backward
            d.mem_fill(loss_grad, 1.0)
            d.mem_fill(g_q, 0.0)
            d.dispatch("smooth_l1_bwd", pred=q, target=targets, grad=g_q, beta=1.0)
        g_all = d.mem_cache_alloc(F32, B * A)
        d.mem_fill(g_all, 0.0)
        d.dispatch("scatter_add", src=g_q, offsets=offsets, dst=g_all)  # GatherBwd, src/ndtensor.zig:1367-1380
        d.mem_cache_free(offsets)
        for t in (g_q, loss_grad, q, targets):
            d.mem_cache_free(t)
        self.policy.backward(acts, g_all, B)
        if keep_grads:
            self.last_grads = [d.to_numpy(b) for b in self.policy.grad_buffers()]
        if not self.optim.step_and_zero_grad():
            self.optim.step()
        loss_val = self._read_loss(loss)
        d.mem_cache_free(loss)
        return loss_val


def gcn_inputs(n_nodes=2708, n_features=1433, n_pairs=5278, n_classes=7, n_train=140, hidden=16, seed=0):
    """Synthetic Cora-shaped graph: Bernoulli(0.0127) features, symmetrised uniform random pairs plus self
    loops in [2, E] layout (source row, then target row), uniform labels, the first n_train nodes labelled."""
    r = np.random.default_rng(seed)
    x = (r.random((n_nodes, n_features)) < 0.0127).astype(np.float32)
    u, v = r.integers(0, n_nodes, n_pairs), r.integers(0, n_nodes, n_pairs)
    loops = np.arange(n_nodes)
    src = np.concatenate([u, v, loops]).astype(np.uint64)
    tgt = np.concatenate([v, u, loops]).astype(np.uint64)
    labels = r.integers(0, n_classes, n_nodes)
    onehot = np.zeros((n_nodes, n_classes), np.float32)
    onehot[np.arange(n_nodes), labels] = 1.0
    params = []
    for fan_in, fan_out in ((n_features, hidden), (hidden, n_classes)):
        params.append((r.standard_normal((fan_out, fan_in)) * np.sqrt(2.0 / fan_in)).astype(np.float32))
        params.append(np.zeros(fan_out, np.float32))
    return {"x": x, "src": src, "tgt": tgt, "onehot": onehot, "n_train": n_train, "params": params,
            "dims": [n_features, hidden, n_classes]}


class GCNTrainer(GraphSteps):
    """Two GraphConv layers (GEMM, degree-scaled scatter, bias) with ReLU between, masked softmax
    cross-entropy, Adam: the op sequence of examples/gcn/src/model.zig:27-36, 100-224 and main.zig:68-84.
    The labelled nodes are the first `n_train` rows (MaskLayer.backward indexes the masked gradient by node
    id, examples/gcn/src/model.zig:343-348, which is only meaningful for a prefix mask)."""

    EPS = 1e-12  # Settings.eps, src/zigrad.zig:72

    def __init__(self, dev, inp, lr=0.01, clip=True, fused=False):
        d = self.dev = dev
        self.N = inp["x"].shape[0]
        self.dims = inp["dims"]
        self.E = inp["src"].size
        self.n_train = inp["n_train"]
        self.optim = Optimizer(dev, "adam", lr, clip, fused=fused)
        self.W, self.b, self.Wg, self.bg = [], [], [], []
        for fan_in, fan_out in zip(self.dims[:-1], self.dims[1:]):
            w, wg = d.mem_alloc(F32, fan_in * fan_out), d.mem_alloc(F32, fan_in * fan_out)
            b, bg = d.mem_alloc(F32, fan_out), d.mem_alloc(F32, fan_out)
            for g in (wg, bg):
                d.mem_fill(g, 0.0)
            self.W.append(w); self.b.append(b); self.Wg.append(wg); self.bg.append(bg)
            self.optim.attach(w, wg)
            self.optim.attach(b, bg)
        for l in range(2):
            d.mem_transfer(inp["params"][2 * l], self.W[l], "HtoD")
            d.mem_transfer(inp["params"][2 * l + 1], self.b[l], "HtoD")
        self.x = d.from_numpy(inp["x"])
        # the edge list lives where the host can write it and the kernels can read it
        self.edge_index = d.mem_alloc_host(U64, 2 * self.E)
        d.mem_transfer(np.concatenate([inp["src"], inp["tgt"]]), self.edge_index, "HtoD")
        self.src, self.tgt = self.edge_index.sub(0, self.E), self.edge_index.sub(self.E, self.E)
        # fused: the edge list is the dataset's and never changes, so its segment plans are built once
        self.plan = d.edge_plan(self.src, self.tgt, self.N) if fused else None
        self._deg_norm = None
        self.label_m = d.from_numpy(inp["onehot"][: self.n_train])
        self._init_loss_slot()
        self.last_grads = None

    def param_buffers(self):
        return [self.W[0], self.b[0], self.W[1], self.b[1]]

    def grad_buffers(self):
        return [self.Wg[0], self.bg[0], self.Wg[1], self.bg[1]]

    def _degree_norm(self) -> DevBuf:
        """deg^-1/2 with deg = 1 + in-degree, as GraphConvLayer.forward computes it on every call
        (examples/gcn/src/model.zig:116-224).  With an edge plan the graph is known not to change, so the fused
        trainer computes it once (during its first, eager step) and every layer reads that one buffer."""
        d, N, E = self.dev, self.N, self.E
        if self._deg_norm is not None:
            return self._deg_norm
        deg = d.mem_cache_alloc(F32, N)
        d.mem_fill(deg, 1.0)
        ones_edges = d.mem_cache_alloc(F32, E)
        d.mem_fill(ones_edges, 1.0)
        contrib = d.mem_cache_alloc(F32, N)
        d.mem_fill(contrib, 0.0)
        if self.plan is not None:
            d.dispatch("scatter_add_planned", src=ones_edges, plan=self.plan, dst=contrib)
        else:
            d.dispatch("scatter_add", src=ones_edges, offsets=self.tgt, dst=contrib)
        d.mem_cache_free(ones_edges)
        d.dispatch("add", x=contrib, y=deg, z=deg)  # deg._add(deg_contrib)
        d.mem_cache_free(contrib)
        deg_norm = d.mem_cache_alloc(F32, N)
        d.dispatch("rsqrt_fwd", x=deg, y=deg_norm, eps=self.EPS)
        d.mem_cache_free(deg)
        if self.plan is not None:
            self._deg_norm = d.mem_alloc(F32, N)
            d.mem_copy(deg_norm, self._deg_norm)
            d.mem_cache_free(deg_norm)
            return self._deg_norm
        return deg_norm

    def _conv_forward(self, l, x_in, relu=False):
        """h = x W^T, y = aggregate(h) + b (GraphConvLayer.forward, examples/gcn/src/model.zig:100-112); `relu` applies
        the model's relu_ to y as well (:36)."""
        d, N, E = self.dev, self.N, self.E
        fan_in, fan_out = self.dims[l], self.dims[l + 1]
        h = d.mem_cache_alloc(F32, N * fan_out)
        host.bmm_acc_(d, x_in, [N, fan_in], self.W[l], [fan_out, fan_in], h, trans_a=False, trans_b=True)
        deg_norm = self._degree_norm()
        y = d.mem_cache_alloc(F32, N * fan_out)
        if self.plan is not None:  # written, not accumulated (no zero fill); bias and relu in the same launch
            d.dispatch("scatter_gcn_deg_scaled_planned", dst=y, h=h, deg=deg_norm, plan=self.plan, stride=fan_out,
                       accumulate=False, bias=self.b[l], relu=relu)
        else:
            d.mem_fill(y, 0.0)
            d.dispatch("scatter_gcn_deg_scaled", dst=y, h=h, deg=deg_norm, src_indices=self.src, tgt_indices=self.tgt,
                       stride=fan_out, n_edge=E)
            d.dispatch("add", x=self.b[l], y=y, z=y)  # y._add(bias)
            if relu:
                d.dispatch("relu_fwd", x=y, y=y)
        return {"x": x_in, "h": h, "deg": deg_norm, "y": y}

    def _conv_backward(self, l, saved, g_y, need_input_grad, act_in=None):
        """`act_in` (fused trainer only): the ReLU output that fed this layer; its backward is then applied to the
        input gradient by the product that writes it."""
        d, N, E = self.dev, self.N, self.E
        fan_in, fan_out = self.dims[l], self.dims[l + 1]
        host.unbroadcast_(d, g_y, [N, fan_out], self.bg[l], [fan_out], alpha=1.0, beta=1.0)
        g_h = d.mem_cache_alloc(F32, N * fan_out)
        if self.plan is not None:
            # written, not accumulated (no zero fill), and without the degree gradient, which nobody reads: the
            # chain stops at rsqrt (src/ndtensor.zig:1009) and the degrees are data of the graph
            d.dispatch("scatter_gcn_deg_scaled_bwd_planned", grad_output=g_y, h=saved["h"], deg=saved["deg"], plan=self.plan,
                       grad_h=g_h, grad_deg=None, stride=fan_out, accumulate=False)
        else:
            d.mem_fill(g_h, 0.0)
            g_deg = d.mem_cache_alloc(F32, N)
            d.mem_fill(g_deg, 0.0)
            d.dispatch("scatter_gcn_deg_scaled_bwd", grad_output=g_y, h=saved["h"], deg=saved["deg"], src_indices=self.src,
                       tgt_indices=self.tgt, grad_h=g_h, grad_deg=g_deg, stride=fan_out, n_edge=E)
            d.mem_cache_free(g_deg)  # deg itself needs no gradient: the chain stops at rsqrt (src/ndtensor.zig:1009)
        d.mem_cache_free(g_y)
        d.mem_cache_free(saved["y"])
        if saved["deg"] is not self._deg_norm:
            d.mem_cache_free(saved["deg"])
        g_x = d.mem_cache_alloc(F32, N * fan_in) if need_input_grad else None
        if self.optim.fused:  # the input gradient is written (no zero fill) with the ReLU backward applied
            d.dispatch("linear_bwd", gy=g_h, x=saved["x"], w=self.W[l], act_in=act_in, gw=self.Wg[l], gb=None, gx=g_x,
                       batch=N, fan_in=fan_in, fan_out=fan_out)
        else:
            if need_input_grad:
                d.mem_fill(g_x, 0.0)
            host.bmm_acc_backward(d, False, True, saved["x"], [N, fan_in], self.W[l], [fan_out, fan_in], g_h, [N, fan_out],
                                  g_x, self.Wg[l])
        d.mem_cache_free(g_h)
        d.mem_cache_free(saved["h"])
        return g_x

    def step(self, keep_grads: bool = False) -> float:
        d, N, C, M = self.dev, self.N, self.dims[-1], self.n_train
        s1 = self._conv_forward(0, self.x, relu=True)
        s2 = self._conv_forward(1, s1["y"])
        out_m = d.mem_cache_alloc(F32, M * C)  # MaskLayer.forward: the labelled rows, here one contiguous prefix
        d.mem_copy(s2["y"].sub(0, M * C), out_m)
        probs, loss = d.mem_cache_alloc(F32, M * C), d.mem_cache_alloc(F32, 1)
        g_m = d.mem_cache_alloc(F32, M * C)
        loss_grad = d.mem_cache_alloc(F32, 1)
        if self.optim.fused:  # forward and the loss's backward in one call, the gradient written without a zero fill
            d.dispatch("smce_fwd_bwd", logits=out_m, target=self.label_m, probs=probs, loss=loss, grad=g_m, rows=M, cols=C,
                       accumulate=False)
            loss_val = self._read_loss(loss)
        else:
            d.dispatch("smce_fwd", logits=out_m, target=self.label_m, probs=probs, loss=loss, rows=M, cols=C)
            loss_val = self._read_loss(loss)
            # backward
            d.mem_fill(loss_grad, 1.0)
            d.mem_fill(g_m, 0.0)
            d.dispatch("smce_bwd", probs=probs, target=self.label_m, grad=g_m, rows=M, cols=C)
        g2 = d.mem_cache_alloc(F32, N * C)
        d.mem_fill(g2, 0.0)
        d.mem_copy(g_m, g2.sub(0, M * C))  # MaskLayer.backward
        for t in (probs, loss, loss_grad, g_m, out_m):
            d.mem_cache_free(t)
        if self.optim.fused:
            g1 = self._conv_backward(1, s2, g2, need_input_grad=True, act_in=s1["y"])
        else:
            g1 = self._conv_backward(1, s2, g2, need_input_grad=True)
            d.dispatch("relu_inplace_bwd", x=s1["y"], x_g=g1)
        self._conv_backward(0, s1, g1, need_input_grad=False)
        if keep_grads:
            self.last_grads = [d.to_numpy(b) for b in self.grad_buffers()]
        if not self.optim.step_and_zero_grad():
            self.optim.step()
            for gb in self.grad_buffers():
                d.mem_fill(gb, 0.0)
        return loss_val
