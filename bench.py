#!/usr/bin/env python3
"""Benchmark of the device-op hot path on one MI355X.

Headline workload: the wide-MLP train step (configuration 5 of the benchmark definition: 4096 -> 4096 -> 4096 -> 1024,
batch 4096, fp32, forward + backward + Adam), issued op by op through the C ABI exactly as the reference's
training loop reaches its device.  `value` is train steps per second with every operand resident in HBM.

The same JSON line also carries:
  roofline      the dominant kernel (the fp32 MFMA GEMM): algorithmic FLOPs of the step's eight GEMM launches
                divided by their summed duration, measured with HIP events on the stream they run on
  cpu_baseline  the CPU oracle (C restatement of HostDevice + the box's BLAS) running the same step
  ops           the op microbenchmark suite of configs[1] (GEMM variants, bmm, broadcast add, axis
                reductions, fused softmax cross-entropy), each with its own roofline fraction
  input_pipeline  the same step with a fresh 67 MB batch from pinned host memory every step (PCIe-inclusive rate):
                blocking upload as the reference does it, and double-buffered on the copy stream
  mlp_b64, gcn, dqn   the latency-bound configurations (configs[0], [2], [3]): step time, loss read every step
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

PEAK_FP32_MFMA_TFLOPS = 157.3
PEAK_HBM_GBS = 8000.0

WIDE_DIMS = [4096, 4096, 4096, 1024]
WIDE_BATCH = 4096


def gemm_flops_per_step(dims, batch):
    """2*m*n*k over the GEMMs of one train step: forward per layer, dX for layers > 0, dW per layer."""
    total = 0
    for l, (fi, fo) in enumerate(zip(dims[:-1], dims[1:])):
        total += 2 * batch * fo * fi  # forward
        total += 2 * fo * fi * batch  # dW
        if l > 0:
            total += 2 * batch * fi * fo  # dX
    return total


def gemm_bytes_per_step(dims, batch):
    """Algorithmic bytes of the same launches: both operands read once, C written, C also read where the
    reference accumulates (beta = 1 for every gradient GEMM, src/ndtensor.zig:1092-1136)."""
    total = 0
    for l, (fi, fo) in enumerate(zip(dims[:-1], dims[1:])):
        total += 4 * (batch * fi + fo * fi + batch * fo)          # forward: X, W -> Y
        total += 4 * (batch * fo + batch * fi + 2 * fo * fi)      # dW += dY^T X
        if l > 0:
            total += 4 * (batch * fo + fo * fi + 2 * batch * fi)  # dX += dY W
    return total


# HBM-side bytes per GEMM launch (average over the step's 8 launches): measured by two rocprofv3 counter runs of this
# script (FETCH_SIZE, then WRITE_SIZE), each scaled by what the counter reads for the copy_calibration kernel.  The
# figure is read from the committed summary of those runs, so it cannot drift from it; without the file it is null.
GEMM_TRAFFIC_PROFILE = Path(__file__).resolve().parent / "profiles" / "gemm_kernel_wide_mlp_step_hbm_traffic.txt"


def gemm_traffic_bytes_per_launch(path=GEMM_TRAFFIC_PROFILE):
    """The 'All N launches ...: X MB per launch on average (B bytes).' line of the traffic summary -> B, else None."""
    import re

    try:
        text = Path(path).read_text()
    except OSError:
        return None
    m = re.search(r"^All \d+ launches.*per launch on average \((\d+) bytes\)", text, re.M)
    return float(m.group(1)) if m else None


class GemmTimer:
    """The library's own product timing: event pairs around every product's launches, on the device's stream, recorded
    where the launches are queued (a product may wait one call for its bias add and ReLU, so events placed around the
    bmm_acc call from outside would bracket nothing, or cut the product off from what follows it)."""

    def __init__(self, dev):
        self.dev = dev
        self._on = False
        self.ms, self.count = 0.0, 0

    def install(self):
        pass

    @property
    def on(self):
        return self._on

    @on.setter
    def on(self, value):
        if value and not self._on:
            self.dev.gemm_timing(True)
        elif self._on and not value:
            self.dev.gemm_timing(False)
            self.ms, self.count = self.dev.gemm_timing_read()
        self._on = bool(value)

    def total_ms(self):
        return self.ms

    @property
    def pairs(self):
        return range(self.count)


OP_WARM_MS = 60.0  # --short-ops lowers it: under a profiler every warm-up call is a row of output


def time_op(dev, fn, iters, warm_ms=None, batches=10):
    """Median (and p10/p90) per-call time in ms over `batches` event-bracketed runs of `iters` back-to-back calls.

    The warm-up runs for at least `warm_ms` of wall time: the GPU raises its clock only under sustained load, and a
    kernel timed in the first tens of milliseconds after idle reads 10 % slower than in a training loop.
    """
    if dev.is_host():  # the CPU oracle: wall clock around synchronous calls
        ms = []
        for _ in range(batches):
            t0 = time.perf_counter()
            for _ in range(iters):
                fn()
            ms.append((time.perf_counter() - t0) * 1e3 / iters)
        ms.sort()
        pick = lambda q: ms[min(len(ms) - 1, int(q * len(ms)))]
        return {"ms": pick(0.5), "ms_p10": pick(0.1), "ms_p90": pick(0.9)}
    warm_ms = OP_WARM_MS if warm_ms is None else warm_ms
    t0 = time.perf_counter()
    while True:
        for _ in range(iters):
            fn()
        dev.sync()
        if (time.perf_counter() - t0) * 1e3 >= warm_ms:
            break
    pairs = []
    for _ in range(batches):
        e0 = dev.event().record()
        for _ in range(iters):
            fn()
        pairs.append((e0, dev.event().record()))
    dev.sync()
    ms = sorted(a.elapsed_ms(b) / iters for a, b in pairs)
    pick = lambda q: ms[min(len(ms) - 1, int(q * len(ms)))]
    return {"ms": pick(0.5), "ms_p10": pick(0.1), "ms_p90": pick(0.9)}


def copy_calibration(dev):
    """Three launches of a plain streaming kernel of known size (relu_fwd over 2^26 floats: 256 MiB read, 256 MiB
    written, grid found in a counter trace by its 64 Mi-element size).  HBM byte counters of other kernels are
    scaled by what they read for this one."""
    from zigrad_amd.device import F32

    n = 1 << 26
    x, y = dev.mem_alloc(F32, n), dev.mem_alloc(F32, n)
    dev.mem_fill(x, 1.0)
    for _ in range(3):
        dev.dispatch("relu_fwd", x=x, y=y)
    dev.sync()
    dev.mem_free(x)
    dev.mem_free(y)


def op_suite(dev, quick=False, cpu=False):
    """configs[1]: per-op time, achieved TFLOP/s or GB/s from the algorithmic work, fraction of roofline.

    With cpu=True `dev` is the CPU oracle: the same ops, one call per timing, three timings each, and the loss
    kernels on the first 1024 of the 8192 rows (rows are independent; the rate is what is reported)."""
    from zigrad_amd.device import F32, U64

    out = {}
    r = np.random.default_rng(0)
    iters = 5 if quick else 20
    timed = (lambda d, fn, it: time_op(d, fn, 1, batches=3)) if cpu else time_op

    def tfl(flops, t):
        tf = flops / (t["ms"] * 1e-3) / 1e12
        return {**t, "tflops": tf, "frac_mfma": tf / PEAK_FP32_MFMA_TFLOPS}

    def dev_normal(n):
        b = dev.mem_alloc(F32, n)
        dev.mem_random(b, "normal", seed=int(r.integers(1 << 30)))
        return b

    # GEMM 4096^3: NN, TN (A transposed), NT (B transposed)
    n = 4096
    big = n * n if cpu else 4100 * 4100  # the largest operand any product below takes
    A, B, C = dev_normal(big), dev_normal(big), dev_normal(big)
    for tag, ta, tb in (("matmul_4096_nn", False, False), ("matmul_4096_tn", True, False), ("matmul_4096_nt", False, True)):
        t = timed(dev, lambda: dev.dispatch("matmul", A=A, B=B, C=C, m=n, n=n, k=n, trans_a=ta, trans_b=tb, lda=n, ldb=n,
                                               ldc=n, alpha=1.0, beta=0.0), iters)
        out[tag] = tfl(2 * n ** 3, t)
    # bmm 32 x 512^3
    nb, s = 32, 512
    t = timed(dev, lambda: dev.dispatch("bmm_acc", A=A, B=B, C=C, A_shape=[nb, s, s], B_shape=[nb, s, s], C_shape=[nb, s, s],
                                           trans_a=False, trans_b=False, lda=s, ldb=s, ldc=s, alpha=1.0, beta=0.0), iters * 5)
    out["bmm_32x512"] = tfl(2 * nb * s ** 3, t)
    if not cpu:
        # products off the large tile's grid (not part of the named op suite: cubes whose tile count does not fill whole
        # rounds of compute units, and the graph convolution's skinny first layer, which is bound by reading X)
        for m_, n_, k_ in ((1536, 1536, 1536), (3072, 3072, 3072), (4100, 4100, 4100)):
            t = timed(dev, lambda: dev.dispatch("matmul", A=A, B=B, C=C, m=m_, n=n_, k=k_, trans_a=False, trans_b=True,
                                                   lda=k_, ldb=k_, ldc=n_, alpha=1.0, beta=0.0), iters * (4 if m_ < 2048 else 1))
            out[f"matmul_{m_}_nt"] = {**tfl(2 * m_ * n_ * k_, t), "plan": dev.gemm_plan(m_, n_, k_)["kind"]}
        m_, n_, k_ = 2708, 16, 1433
        t = timed(dev, lambda: dev.dispatch("matmul", A=A, B=B, C=C, m=m_, n=n_, k=k_, trans_a=False, trans_b=True, lda=k_,
                                               ldb=k_, ldc=n_, alpha=1.0, beta=0.0), iters * 10)
        nbytes = 4 * (m_ * k_ + n_ * k_ + m_ * n_)
        out["matmul_2708x16x1433_nt"] = {**tfl(2 * m_ * n_ * k_, t), "gbs": nbytes / (t["ms"] * 1e-3) / 1e9,
                                         "frac_hbm": nbytes / (t["ms"] * 1e-3) / 1e9 / PEAK_HBM_GBS,
                                         "bound": "hbm (0.25 FLOP per byte of X at N = 16)"}
    for b in (A, B, C):
        dev.mem_free(b)

    # memory-bound ops on [8192, 4096]
    rows, cols = 8192, 4096
    X, bias, Z = dev_normal(rows * cols), dev_normal(cols), dev.mem_alloc(F32, rows * cols)
    yrow = dev.mem_alloc(F32, rows)

    def gbs(nbytes, t):
        g = nbytes / (t["ms"] * 1e-3) / 1e9
        return {**t, "gbs": g, "frac_hbm": g / PEAK_HBM_GBS}

    ms = timed(dev, lambda: dev.dispatch("add", x=X, y=bias, z=Z), iters * 5)
    out["add_bcast_8192x4096"] = gbs((2 * rows * cols + cols) * 4, ms)
    ms = timed(dev, lambda: dev.dispatch("sum_along", x=X, x_shape=[rows, cols], y=yrow, dim=1), iters * 5)
    out["sum_axis1_8192x4096"] = gbs((rows * cols + rows) * 4, ms)
    ms = timed(dev, lambda: dev.dispatch("max_along", x=X, x_shape=[rows, cols], y=yrow, dim=1), iters * 5)
    out["max_axis1_8192x4096"] = gbs((rows * cols + rows) * 4, ms)
    if not cpu:
        # the rest of the op surface at the same size (not in the named suite): unary ops forward and backward, a
        # same-size binary op, reductions along the other axis, argmax, the optimizer updates of a [4096,4096] weight,
        # row gathers.  Bytes are the algorithmic ones: every operand read once, every result written once.
        n_el = rows * cols
        G, Y = dev_normal(n_el), dev_normal(n_el)
        extra = {}
        for name in ("relu_fwd", "tanh_fwd", "sigm_fwd", "exp_fwd"):
            ms = timed(dev, lambda: dev.dispatch(name, x=X, y=Z), iters * 5)
            extra[f"{name}_8192x4096"] = gbs(2 * n_el * 4, ms)
        ms = timed(dev, lambda: dev.dispatch("relu_bwd", x=X, x_g=G, y_g=Y), iters * 5)
        extra["relu_bwd_8192x4096"] = gbs(4 * n_el * 4, ms)
        for name in ("tanh_bwd", "sigm_bwd", "exp_bwd"):
            ms = timed(dev, lambda: dev.dispatch(name, x_g=G, y=Z, y_g=Y), iters * 5)
            extra[f"{name}_8192x4096"] = gbs(4 * n_el * 4, ms)
        ms = timed(dev, lambda: dev.dispatch("relu_inplace_bwd", x=X, x_g=G), iters * 5)
        extra["relu_inplace_bwd_8192x4096"] = gbs(3 * n_el * 4, ms)
        ms = timed(dev, lambda: dev.dispatch("mul", x=X, y=Y, z=Z), iters * 5)
        extra["mul_8192x4096"] = gbs(3 * n_el * 4, ms)
        ycol = dev.mem_alloc(F32, cols)
        ms = timed(dev, lambda: dev.dispatch("sum_along", x=X, x_shape=[rows, cols], y=ycol, dim=0), iters * 5)
        extra["sum_axis0_8192x4096"] = gbs((n_el + cols) * 4, ms)
        yarg = dev.mem_alloc(U64, rows)
        ms = timed(dev, lambda: dev.dispatch("argmax_along", x=X, x_shape=[rows, cols], y=yarg, dim=1), iters * 5)
        extra["argmax_axis1_8192x4096"] = gbs(n_el * 4 + rows * 8, ms)
        ysc = dev.mem_alloc(F32, 1)
        ms = timed(dev, lambda: dev.dispatch("nrm2", x=X, y=ysc), iters * 5)
        extra["nrm2_33M"] = gbs(n_el * 4, ms)
        n_w = 4096 * 4096
        P, Gw, M1, V1 = (X.sub(0, n_w), G.sub(0, n_w), Y.sub(0, n_w), Z.sub(0, n_w))
        dev.mem_fill(M1, 0.0)
        dev.mem_fill(V1, 0.0)
        ms = timed(dev, lambda: dev.dispatch("sgd_step", param=P, grad=Gw, lr=1e-6, clip=False, max_norm=10.0, delta=1e-6),
                   iters * 5)
        extra["sgd_step_16.8M"] = gbs(3 * n_w * 4, ms)
        ms = timed(dev, lambda: dev.dispatch("adam_step", param=P, grad=Gw, m=M1, v=V1, t=10, lr=1e-6, beta1=0.9, beta2=0.999,
                                             epsilon=1e-8, clip=False, max_norm=10.0, delta=1e-6), iters * 5)
        extra["adam_step_16.8M"] = gbs(7 * n_w * 4, ms)
        ms = timed(dev, lambda: dev.dispatch("adam_step", param=P, grad=Gw, m=M1, v=V1, t=10, lr=1e-6, beta1=0.9, beta2=0.999,
                                             epsilon=1e-8, clip=True, max_norm=10.0, delta=1e-6), iters * 5)
        extra["adam_step_clip_16.8M"] = gbs(8 * n_w * 4, ms)
        n_idx, stride = 65536, 256
        idx = dev.from_numpy(r.integers(0, n_el // stride, n_idx).astype(np.uint64))
        ms = timed(dev, lambda: dev.dispatch("index_select_fwd", src=X, indices=idx, stride=stride, dst=Z.sub(0, n_idx * stride)),
                   iters * 5)
        extra["index_select_fwd_65536x256"] = gbs(2 * n_idx * stride * 4 + n_idx * 8, ms)
        # the deterministic scatter ops on a graph larger than the GCN configuration's (100 k nodes, 1 M edges, 64
        # features): with the destination ordering computed on every call (bare index slices in device memory, as the
        # reference hands them over) and with an edge plan made once for a graph that does not change
        n_nodes, n_edge, feat = 100_000, 1_000_000, 64
        e_src = dev.from_numpy(r.integers(0, n_nodes, n_edge).astype(np.uint64))
        e_tgt = dev.from_numpy(r.integers(0, n_nodes, n_edge).astype(np.uint64))
        h_buf, y_buf = X.sub(0, n_nodes * feat), Z.sub(0, n_nodes * feat)
        deg = dev.mem_alloc(F32, n_nodes)
        dev.mem_fill(deg, 1.0)
        gcn_bytes = n_edge * feat * 4 + 2 * n_nodes * feat * 4 + n_edge * 16
        ms = timed(dev, lambda: dev.dispatch("scatter_gcn_deg_scaled", dst=y_buf, h=h_buf, deg=deg, src_indices=e_src,
                                             tgt_indices=e_tgt, stride=feat, n_edge=n_edge), iters)
        extra["scatter_gcn_1Medges_x64_ordering_per_call"] = {**gbs(gcn_bytes, ms), "edges_per_us": n_edge / (ms["ms"] * 1e3)}
        # the same with the target array rewritten before every call (a copy of 8 MB inside the timed region, about
        # 3 us): the ordering the library keeps for the array is found stale on the GPU and built again, and after a few
        # such calls the library stops keeping one for this array
        e_alt = [e_tgt, dev.from_numpy(r.integers(0, n_nodes, n_edge).astype(np.uint64))]
        e_cur, flip = dev.mem_alloc(U64, n_edge), [0]

        def rewritten(op, **kw):
            flip[0] ^= 1
            dev.mem_copy(e_alt[flip[0]], e_cur)
            dev.dispatch(op, **kw)

        ms = timed(dev, lambda: rewritten("scatter_gcn_deg_scaled", dst=y_buf, h=h_buf, deg=deg, src_indices=e_src,
                                          tgt_indices=e_cur, stride=feat, n_edge=n_edge), iters)
        extra["scatter_gcn_1Medges_x64_indices_rewritten_every_call"] = {**gbs(gcn_bytes, ms), "edges_per_us": n_edge / (ms["ms"] * 1e3)}
        plan = dev.edge_plan(e_src, e_tgt, n_nodes)
        ms = timed(dev, lambda: dev.dispatch("scatter_gcn_deg_scaled_planned", dst=y_buf, h=h_buf, deg=deg, plan=plan,
                                             stride=feat, accumulate=True), iters)
        extra["scatter_gcn_1Medges_x64_planned"] = {**gbs(gcn_bytes, ms), "edges_per_us": n_edge / (ms["ms"] * 1e3)}
        vals = Y.sub(0, n_edge)
        ms = timed(dev, lambda: dev.dispatch("scatter_add", src=vals, offsets=e_tgt, dst=y_buf.sub(0, n_nodes)), iters)
        extra["scatter_add_1M_into_100k_ordering_per_call"] = {**ms, "entries_per_us": n_edge / (ms["ms"] * 1e3)}
        ms = timed(dev, lambda: rewritten("scatter_add", src=vals, offsets=e_cur, dst=y_buf.sub(0, n_nodes)), iters)
        extra["scatter_add_1M_into_100k_indices_rewritten_every_call"] = {**ms, "entries_per_us": n_edge / (ms["ms"] * 1e3)}
        ms = timed(dev, lambda: dev.dispatch("scatter_add_planned", src=vals, plan=plan, dst=y_buf.sub(0, n_nodes)), iters * 5)
        extra["scatter_add_1M_into_100k_planned"] = {**ms, "entries_per_us": n_edge / (ms["ms"] * 1e3)}
        plan.free()
        out["other_ops"] = extra
        for b in (G, Y, ycol, yarg, ysc, idx, e_src, e_tgt, e_alt[1], e_cur, deg):
            dev.mem_free(b)
    for b in (X, bias, Z, yrow):
        dev.mem_free(b)

    # fused softmax cross-entropy, integer labels, logits [8192, 32000]
    M, N = (1024 if cpu else 8192), 32000
    logits, grad = dev_normal(M * N), dev.mem_alloc(F32, M * N)
    labels = dev.from_numpy(r.integers(0, N, M).astype(np.uint64))
    lse, loss = dev.mem_alloc(F32, M), dev.mem_alloc(F32, 1)
    ms = timed(dev, lambda: dev.dispatch("smce_label_fwd", logits=logits, labels=labels, lse=lse, loss=loss, rows=M, cols=N),
                 iters)
    out["smce_fwd_8192x32000"] = gbs(4 * M * N + 8 * M + 4, ms)
    ms = timed(dev, lambda: dev.dispatch("smce_label_bwd", logits=logits, labels=labels, lse=lse, grad=grad, rows=M, cols=N,
                                            accumulate=False), iters)
    out["smce_bwd_8192x32000"] = gbs(2 * 4 * M * N, ms)
    ms = timed(dev, lambda: dev.dispatch("smce_label_bwd", logits=logits, labels=labels, lse=lse, grad=grad, rows=M, cols=N,
                                            accumulate=True), iters)
    out["smce_bwd_accumulate_8192x32000"] = gbs(3 * 4 * M * N, ms)
    # the reference's own form of the loss: float one-hot targets, probabilities saved for backward
    # (src/nn/loss.zig:130-215): 3 passes of the matrix forward (read logits, read target, write probs), 4 backward
    target, probs = dev.mem_alloc(F32, M * N), dev.mem_alloc(F32, M * N)
    dev.mem_fill(target, 0.0)
    dev.mem_fill(grad, 0.0)
    ms = timed(dev, lambda: dev.dispatch("smce_fwd", logits=logits, target=target, probs=probs, loss=loss, rows=M, cols=N),
                 iters // 2)
    out["smce_onehot_fwd_8192x32000"] = gbs(3 * 4 * M * N, ms)
    ms = timed(dev, lambda: dev.dispatch("smce_bwd", probs=probs, target=target, grad=grad, rows=M, cols=N), iters // 2)
    out["smce_onehot_bwd_8192x32000"] = gbs(4 * 4 * M * N, ms)
    # forward and the loss's backward in one pass over rows held in registers (the fused entry point): logits and target
    # in, probabilities and the written gradient out
    ms = timed(dev, lambda: dev.dispatch("smce_fwd_bwd", logits=logits, target=target, probs=probs, loss=loss, grad=grad,
                                            rows=M, cols=N, accumulate=False), iters // 2)
    out["smce_onehot_fwd_bwd_one_pass_8192x32000"] = gbs(4 * 4 * M * N, ms)
    for b in (logits, grad, labels, lse, loss, target, probs):
        dev.mem_free(b)
    return out


def timed_steps(dev, step_fn, steps):
    dev.sync()
    t0 = time.perf_counter()
    loss = None
    for _ in range(steps):
        loss = step_fn()
    dev.sync()
    return time.perf_counter() - t0, loss


def run_mlp(dev, dims, batch, optimizer, steps, warmup, data, timer=None, loss_mode="onehot", lr=1e-3, graph=False,
            late_read=False, fused=False, clip=True, loss_log=None):
    """Returns (seconds, last loss) for `steps` eager steps; with graph=True also the same for `steps` replays of
    the step recorded as an execution graph (the loss is read back every step in both modes)."""
    from zigrad_amd.trainers import MLPTrainer, mlp_inputs

    params, x, onehot, labels = mlp_inputs(dims, batch, seed_weights=0, seed_data=1, data=data)
    tr = MLPTrainer(dev, dims, batch, optimizer=optimizer, lr=lr, clip=clip, loss_mode=loss_mode, fused=fused)
    tr.load_params(params)
    tr.set_batch(x, onehot, labels)
    for _ in range(warmup):
        l = tr.step()
        if loss_log is not None:  # the loss of every step from the first, for the cross-check against the oracle
            loss_log.append(l)
    dt, loss = timed_steps(dev, tr.step, steps)
    if timer is not None:
        # the same steps once more with an event pair around every product: the events cost a few microseconds each
        # on the stream (sixteen per step), so the throughput is taken from the pass without them
        timer.on = True
        timer.dt_with_events, _ = timed_steps(dev, tr.step, steps)
        timer.on = False
    if late_read:  # the same steps with the loss read moved behind the optimizer step (the queue never drains)
        late = lambda: tr.step(read_loss="late")
        late()
        dt_late, loss_late = timed_steps(dev, late, steps)
        return dt, loss, dt_late, loss_late
    if not graph:
        return dt, loss
    tr.capture()
    for _ in range(warmup):
        tr.step_graph()
    dt_g, loss_g = timed_steps(dev, tr.step_graph, steps)
    tr.free_graph()
    return dt, loss, dt_g, loss_g


def run_input_pipeline(dev, dims, batch, steps, warmup):
    """The wide-MLP step with a new batch arriving from host memory every step: uploaded with the reference's
    blocking transfer before the step, or double-buffered on the copy stream under the previous step.  Both read
    the batches from pinned host memory that a loader would fill in place."""
    from zigrad_amd.device import F32, U64
    from zigrad_amd.trainers import BatchStager, MLPTrainer, mlp_inputs

    params, x, onehot, labels = mlp_inputs(dims, batch, seed_weights=0, seed_data=1, data="normal")
    tr = MLPTrainer(dev, dims, batch, optimizer="adam", lr=1e-3, clip=True)
    tr.load_params(params)
    own = (tr.x, tr.onehot, tr.labels)
    st = BatchStager(dev, [(F32, batch * dims[0]), (F32, batch * dims[-1]), (U64, batch)])
    for slot in range(2):
        for a, view in zip((x, onehot, labels), st.views[slot]):
            np.copyto(view, np.asarray(a).ravel())
    st.upload_first((x, onehot, labels))
    batch_bytes = sum(b.nbytes for b in st.pinned[0])

    def blocking_step():
        for src, dst in zip(st.views[0], own):
            dev.mem_transfer(src, dst, "HtoD")
        return tr.step()

    def staged_step():
        tr.use_batch(*st.current())
        st.prefetch()
        loss = tr.step()
        st.advance()
        return loss

    out = {"batch_bytes": batch_bytes}
    for name, fn in (("blocking_upload", blocking_step), ("staged_upload", staged_step)):
        for _ in range(warmup):
            fn()
        dt, _ = timed_steps(dev, fn, steps)
        out[name] = {"steps_per_s": steps / dt, "ms_per_step": dt / steps * 1e3}
        tr.use_batch(*own)
    st.free()
    return out


def run_small(dev, kind, steps, graph=True, fused=False):
    """Step time of the GCN (2708 nodes, 1433 features, 13264 edges, 140 labelled, Adam) or DQN (4-128-128-2, batch
    64, Adam) train step; the loss is read back every step, as the reference's loops do."""
    from zigrad_amd.trainers import DQNTrainer, GCNTrainer, dqn_inputs, gcn_inputs, mlp_inputs

    if kind == "gcn":
        tr = GCNTrainer(dev, gcn_inputs(seed=0), lr=0.01, clip=True, fused=fused)
        what = "2-layer GCN 1433-16-7, 2708 nodes, 13264 edges, 140 labelled nodes, Adam lr 0.01"
    else:
        dims, batch = [4, 128, 128, 2], 64
        params, _, _, _ = mlp_inputs(dims, batch)
        tr = DQNTrainer(dev, dims, batch, lr=1e-3, gamma=0.99, clip=True, fused=fused)
        tr.load_params(params)
        tr.set_batch(dqn_inputs(batch=batch))
        what = "DQN update 4-128-128-2, batch 64, frozen target net, gather, smooth-L1, Adam lr 1e-3"
    for _ in range(10):
        tr.step()
    dev.sync()
    launches = dev.launch_count()
    dt, _ = timed_steps(dev, tr.step, steps)
    launches = (dev.launch_count() - launches) / steps
    out = {"steps_per_s": steps / dt, "ms_per_step": dt / steps * 1e3, "workload": what}
    if launches:  # the CPU oracle launches nothing
        out["launches_per_step"] = launches
    if graph and hasattr(tr, "capture"):
        tr.capture()
        for _ in range(10):
            tr.step_graph()
        dt_g, _ = timed_steps(dev, tr.step_graph, steps)
        tr.free_graph()
        out["graph_replay"] = {"steps_per_s": steps / dt_g, "ms_per_step": dt_g / steps * 1e3}
    return out


def run_c_harness(dims, batch, steps, fused=False):
    """The same eager batch-64 step issued from plain C (examples/c_caller/mlp_step.c): what the op-by-op path costs
    without an interpreter between the calls.  None when the binary has not been built."""
    import subprocess
    import tempfile

    from zigrad_amd.build import C_HARNESS_BIN
    from zigrad_amd.trainers import mlp_inputs

    if not C_HARNESS_BIN.exists():
        return None
    params, x, onehot, _ = mlp_inputs(dims, batch, seed_weights=0, seed_data=1, data="uniform")
    with tempfile.NamedTemporaryFile(suffix=".bin") as f:
        for a in (*params, x, onehot):
            f.write(np.ascontiguousarray(a, np.float32).tobytes())
        f.flush()
        run = subprocess.run([str(C_HARNESS_BIN), f.name, str(steps), str(batch), *map(str, dims), *(["fused"] if fused else [])],
                             capture_output=True, text=True, timeout=300)
    if run.returncode != 0:
        raise RuntimeError("examples/c_caller/mlp_step failed: " + run.stderr)
    us = float(run.stdout.strip().splitlines()[-1].split()[1])
    what = "eager, fused entry points, caller in C" if fused else "eager, same op sequence, caller in C"
    return {"steps_per_s": 1e6 / us, "ms_per_step": us / 1e3, "workload": what}


def run_c_dqn(dims, batch, steps):
    """The DQN update issued op by op from plain C (examples/c_caller/dqn_step.c).  None when the binary has not been
    built."""
    import subprocess
    import tempfile

    from zigrad_amd.build import C_DQN_BIN
    from zigrad_amd.trainers import dqn_inputs, mlp_inputs

    if not C_DQN_BIN.exists():
        return None
    params, _, _, _ = mlp_inputs(dims, batch)
    b = dqn_inputs(batch=batch)
    with tempfile.NamedTemporaryFile(suffix=".bin") as f:
        for a in (*params, b["states"], b["next_states"], b["rewards"], b["dones"]):
            f.write(np.ascontiguousarray(a, np.float32).tobytes())
        f.write(np.ascontiguousarray(b["actions"], np.uint64).tobytes())
        f.flush()
        run = subprocess.run([str(C_DQN_BIN), f.name, str(steps), str(batch), *map(str, dims)], capture_output=True, text=True,
                             timeout=300)
    if run.returncode != 0:
        raise RuntimeError("examples/c_caller/dqn_step failed: " + run.stderr)
    us = float(run.stdout.strip().splitlines()[-1].split()[1])
    return {"steps_per_s": 1e6 / us, "ms_per_step": us / 1e3, "workload": "eager, same op sequence, caller in C"}


def run_c_gcn(steps):
    """The GCN step issued op by op from plain C (examples/c_caller/gcn_step.c).  None when the binary has not been
    built."""
    import subprocess
    import tempfile

    from zigrad_amd.build import C_GCN_BIN
    from zigrad_amd.trainers import gcn_inputs

    if not C_GCN_BIN.exists():
        return None
    inp = gcn_inputs(seed=0)
    with tempfile.NamedTemporaryFile(suffix=".bin") as f:
        for a in (*inp["params"], inp["x"], inp["onehot"][: inp["n_train"]]):
            f.write(np.ascontiguousarray(a, np.float32).tobytes())
        f.write(np.ascontiguousarray(inp["src"], np.uint64).tobytes())
        f.write(np.ascontiguousarray(inp["tgt"], np.uint64).tobytes())
        f.flush()
        argv = [inp["x"].shape[0], *inp["dims"], inp["src"].size, inp["n_train"]]
        run = subprocess.run([str(C_GCN_BIN), f.name, str(steps), *map(str, argv)], capture_output=True, text=True, timeout=300)
    if run.returncode != 0:
        raise RuntimeError("examples/c_caller/gcn_step failed: " + run.stderr)
    us = float(run.stdout.strip().splitlines()[-1].split()[1])
    return {"steps_per_s": 1e6 / us, "ms_per_step": us / 1e3, "workload": "eager, same op sequence, caller in C"}


def cpu_baseline(dims, batch, budget_steps=2, threads=None, loss_mode="onehot"):
    """The oracle on the host cores: the same step sequence, BLAS threads = the box's CPU share (or `threads`)."""
    from oracle.oracle_device import OracleDevice

    odev = OracleDevice()
    cores = threads or min(16, os.cpu_count() or 1)
    cores = odev.set_threads(cores)
    log = []
    dt, _ = run_mlp(odev, dims, batch, "adam", steps=budget_steps, warmup=1, data="normal", loss_mode=loss_mode,
                    loss_log=log)
    return {
        "first_step_loss": log[0],
        "value": budget_steps / dt,
        "unit": "steps/s",
        "cores": cores,
        "kind": "port",
        "sample": f"{budget_steps} timed steps (+1 warm-up) of the same batch-{batch} wide-MLP train step; "
                  f"C restatement of HostDevice with BLAS={odev.blas_name()}",
    }


VENDOR_SHAPES = [(4096, 4096, 4096, 1), (512, 512, 512, 32), (4096, 1024, 4096, 1), (3072, 3072, 3072, 1), (4100, 4100, 4100, 1),
                 (3584, 3584, 3584, 1), (3000, 3000, 3000, 1), (2560, 2560, 2560, 1), (2048, 2048, 2048, 1), (1792, 1792, 1792, 1),
                 (1536, 1536, 1536, 1), (1024, 1024, 1024, 1), (768, 768, 768, 1), (64, 128, 784, 1), (2708, 16, 1433, 1)]


def vendor_gemm_child():
    """The vendor leg, in a process of its own (torch brings its own HIP runtime): one JSON list of ms per shape."""
    import torch

    torch.backends.cuda.matmul.allow_tf32 = False
    tdev = torch.device("cuda:0")
    out = []
    for m, n, k, nb in VENDOR_SHAPES:
        iters = max(5, min(200, int(3e11 / (2.0 * m * n * k * nb))))
        ta = torch.randn(nb, m, k, device=tdev) if nb > 1 else torch.randn(m, k, device=tdev)
        tb = torch.randn(nb, n, k, device=tdev) if nb > 1 else torch.randn(n, k, device=tdev)
        tc = torch.empty(nb, m, n, device=tdev) if nb > 1 else torch.empty(m, n, device=tdev)
        tfn = (lambda: torch.bmm(ta, tb.transpose(1, 2), out=tc)) if nb > 1 else (lambda: torch.matmul(ta, tb.t(), out=tc))
        t0 = time.perf_counter()
        while (time.perf_counter() - t0) * 1e3 < 60.0:
            for _ in range(iters):
                tfn()
            torch.cuda.synchronize()
        ms = []
        for _ in range(10):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(iters):
                tfn()
            e1.record()
            torch.cuda.synchronize()
            ms.append(e0.elapsed_time(e1) / iters)
        out.append(sorted(ms)[5])
        del ta, tb, tc
    print(json.dumps(out))


def vendor_gemm_table():
    """A yardstick, not part of the product: fp32 products through this library and through the vendor's GEMM (torch's
    matmul / bmm on the same GPU, TF32 off), same shapes (C = A B^T, B stored [n, k]), same timing method (60 ms of
    warm-up, median of 10 event-bracketed batches), one process each, run one after the other."""
    import subprocess

    from zigrad_amd import HipDevice
    from zigrad_amd.device import F32

    dev = HipDevice(0)
    ours = []
    for m, n, k, nb in VENDOR_SHAPES:
        iters = max(5, min(200, int(3e11 / (2.0 * m * n * k * nb))))
        A, B, C = dev.mem_alloc(F32, nb * m * k), dev.mem_alloc(F32, nb * n * k), dev.mem_alloc(F32, nb * m * n)
        dev.mem_random(A, "normal", seed=1)
        dev.mem_random(B, "normal", seed=2)
        if nb == 1:
            fn = lambda: dev.dispatch("matmul", A=A, B=B, C=C, m=m, n=n, k=k, trans_a=False, trans_b=True, lda=k, ldb=k,
                                      ldc=n, alpha=1.0, beta=0.0)
        else:
            fn = lambda: dev.dispatch("bmm_acc", A=A, B=B, C=C, A_shape=[nb, m, k], B_shape=[nb, k, n], C_shape=[nb, m, n],
                                      trans_a=False, trans_b=True, lda=k, ldb=k, ldc=n, alpha=1.0, beta=0.0)
        ours.append(time_op(dev, fn, iters)["ms"])
        for b in (A, B, C):
            dev.mem_free(b)
    dev.deinit()
    run = subprocess.run([sys.executable, str(Path(__file__).resolve()), "--vendor-gemm-child"], capture_output=True,
                         text=True, timeout=600)
    if run.returncode != 0:
        sys.exit("the vendor leg failed: " + run.stderr[-2000:])
    theirs = json.loads(run.stdout.strip().splitlines()[-1])
    print(f"{'m x n x k (batch)':>28} {'this library':>22} {'vendor (torch.matmul)':>26}")
    for (m, n, k, nb), a, b in zip(VENDOR_SHAPES, ours, theirs):
        frac = lambda t: 2.0 * m * n * k * nb / (t * 1e-3) / 1e12 / PEAK_FP32_MFMA_TFLOPS * 100
        print(f"{m:>6} x {n:>5} x {k:>5} ({nb:>2}) {a * 1e3:>12.1f} us {frac(a):5.1f} % {b * 1e3:>16.1f} us {frac(b):5.1f} %")


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-ops", action="store_true", help="skip the op microbenchmark suite")
    ap.add_argument("--short-ops", action="store_true",
                    help="op suite with a 2 ms warm-up and a quarter of the repetitions: for runs under a profiler, which "
                         "reads the kernels' durations itself and writes a row per launch")
    ap.add_argument("--loss-mode", default="onehot", choices=["onehot", "label"])
    ap.add_argument("--no-small", action="store_true", help="skip the latency-bound configurations (keeps profiler output small)")
    ap.add_argument("--trace-small", choices=["mlp_b64", "gcn", "dqn"],
                    help="run 30 eager steps of one latency-bound configuration and exit (for rocprofv3 --kernel-trace: "
                         "the profiler cannot trace graph replays, the eager steps launch the same kernels)")
    ap.add_argument("--trace-fused", action="store_true", help="with --trace-small: through the fused entry points")
    ap.add_argument("--no-graph", action="store_true",
                    help="skip the execution-graph replays (rocprofv3's kernel tracing crashes inside hipGraphLaunch)")
    ap.add_argument("--vendor-gemm", action="store_true",
                    help="print a table of fp32 products through this library and through the vendor GEMM (torch) and exit")
    ap.add_argument("--vendor-gemm-child", action="store_true", help=argparse.SUPPRESS)
    args = ap.parse_args()
    if args.vendor_gemm_child:
        vendor_gemm_child()
        return
    if args.vendor_gemm:
        vendor_gemm_table()
        return
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: the hot path is single-device and this build uses no second GPU "
                 "(run with --gpus 1)")

    from zigrad_amd import HipDevice

    dev = HipDevice(0)
    if args.trace_small:
        from zigrad_amd.trainers import DQNTrainer, GCNTrainer, MLPTrainer, dqn_inputs, gcn_inputs, mlp_inputs

        if args.trace_small == "mlp_b64":
            dims, batch = [784, 128, 64, 10], 64
            params, x, onehot, labels = mlp_inputs(dims, batch, data="uniform")
            tr = MLPTrainer(dev, dims, batch, optimizer="sgd", lr=0.01, clip=True, fused=args.trace_fused)
            tr.load_params(params)
            tr.set_batch(x, onehot, labels)
        elif args.trace_small == "gcn":
            tr = GCNTrainer(dev, gcn_inputs(seed=0), lr=0.01, clip=True, fused=args.trace_fused)
        else:
            dims, batch = [4, 128, 128, 2], 64
            params, _, _, _ = mlp_inputs(dims, batch)
            tr = DQNTrainer(dev, dims, batch, lr=1e-3, gamma=0.99, clip=True, fused=args.trace_fused)
            tr.load_params(params)
            tr.set_batch(dqn_inputs(batch=batch))
        for _ in range(30):
            tr.step()
        dev.sync()
        print(json.dumps({"traced": args.trace_small, "fused": args.trace_fused, "steps": 30}))
        return
    copy_calibration(dev)
    timer = GemmTimer(dev)
    timer.install()
    gpu_losses = []
    dt, loss, dt_late, _ = run_mlp(dev, WIDE_DIMS, WIDE_BATCH, "adam", args.steps, args.warmup, "normal", timer, args.loss_mode,
                                   late_read=True, loss_log=gpu_losses)
    ms_per_step = dt / args.steps * 1e3
    gemm_ms = timer.total_ms()
    n_launch = len(timer.pairs)
    flops = gemm_flops_per_step(WIDE_DIMS, WIDE_BATCH) * args.steps
    achieved = flops / (gemm_ms * 1e-3) / 1e12 if gemm_ms > 0 else 0.0

    result = {
        "metric": "MLP train steps/sec @ batch 4096 (wide MLP 4096-4096-4096-1024, fwd+bwd+Adam)",
        "value": args.steps / dt,
        "unit": "steps/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "wide MLP train step: 4096->4096->4096->1024, batch 4096, softmax-CE "
                               f"({args.loss_mode}), Adam lr 1e-3, per-tensor grad clip on", "final_loss": loss},
        "roofline": {
            "bound": "mfma",
            "achieved": achieved,
            "peak": PEAK_FP32_MFMA_TFLOPS,
            "unit": "TFLOP/s",
            "frac": achieved / PEAK_FP32_MFMA_TFLOPS,
            "traffic": gemm_traffic_bytes_per_launch(),
            "traffic_unit": "bytes per launch (L2 misses to the fabric, rocprofv3 FETCH_SIZE + WRITE_SIZE)",
            "algorithmic_bytes_per_launch": gemm_bytes_per_step(WIDE_DIMS, WIDE_BATCH) / 8,
            "kernel": "gemm_kernel (fp32 MFMA 32x32x2), 8 launches per step",
            "gemm_ms_per_step": gemm_ms / args.steps,
            "launches_timed": n_launch,
            "measured_in": "a second pass of the same steps, right after the timed one, with a HIP event pair around "
                           "every product on the device's stream; `value` comes from the pass without events",
            "ms_per_step_with_events": timer.dt_with_events / args.steps * 1e3,
        },
    }
    # `value` reads the loss where the reference's loop does (before backward: the host blocks and the GPU idles until
    # the backward launches arrive); the same step with that one read moved behind the optimizer step:
    result["late_loss_read"] = {"steps_per_s": args.steps / dt_late, "ms_per_step": dt_late / args.steps * 1e3}
    # the fused entry points: every Linear layer with bias + ReLU in the GEMM epilogue and ReLU backward in the epilogue
    # of the input-gradient product, optimizer step + zero_grad over the whole parameter list (same arithmetic,
    # bit-identical parameters): not the reference's op sequence, so reported beside `value`, never as it
    f = run_mlp(dev, WIDE_DIMS, WIDE_BATCH, "adam", args.steps, args.warmup, "normal", None, args.loss_mode, late_read=True,
                fused=True)
    result["fused"] = {"steps_per_s": args.steps / f[0], "ms_per_step": f[0] / args.steps * 1e3,
                              "late_loss_read": {"steps_per_s": args.steps / f[2], "ms_per_step": f[2] / args.steps * 1e3}}
    # the latency-bound configurations: batch-64 MLP (configs[0]), GCN (configs[2]), DQN update (configs[3])
    if not args.no_small:
        small = run_mlp(dev, [784, 128, 64, 10], 64, "sgd", 200, 20, "uniform", None, "onehot", lr=0.01, graph=not args.no_graph)
        result["mlp_b64"] = {"steps_per_s": 200 / small[0], "ms_per_step": small[0] / 200 * 1e3,
                             "workload": "784-128-64-10, batch 64, SGD lr 0.01, clip on, loss read every step; "
                                         "graph_replay = the same step recorded once as an execution graph"}
        if not args.no_graph:
            result["mlp_b64"]["graph_replay"] = {"steps_per_s": 200 / small[2], "ms_per_step": small[2] / 200 * 1e3}
        if not args.no_graph:
            fs = run_mlp(dev, [784, 128, 64, 10], 64, "sgd", 200, 20, "uniform", None, "onehot", lr=0.01, graph=True, fused=True)
            result["mlp_b64"]["fused"] = {"steps_per_s": 200 / fs[0], "ms_per_step": fs[0] / 200 * 1e3,
                                                 "graph_replay": {"steps_per_s": 200 / fs[2], "ms_per_step": fs[2] / 200 * 1e3}}
            # the example itself switches the gradient clip off (examples/mnist/src/main-simple.zig:29-34)
            nc = run_mlp(dev, [784, 128, 64, 10], 64, "sgd", 200, 20, "uniform", None, "onehot", lr=0.01, graph=True, clip=False)
            result["mlp_b64"]["clip_off"] = {"steps_per_s": 200 / nc[0], "ms_per_step": nc[0] / 200 * 1e3,
                                             "graph_replay": {"steps_per_s": 200 / nc[2], "ms_per_step": nc[2] / 200 * 1e3}}
        result["mlp_b64"]["c_caller"] = run_c_harness([784, 128, 64, 10], 64, 2000)
        if "fused" in result["mlp_b64"]:
            result["mlp_b64"]["fused"]["c_caller"] = run_c_harness([784, 128, 64, 10], 64, 2000, fused=True)
        result["input_pipeline"] = run_input_pipeline(dev, WIDE_DIMS, WIDE_BATCH, max(5, args.steps // 2), 2)
        result["gcn"] = run_small(dev, "gcn", 100, graph=not args.no_graph)
        result["gcn"]["c_caller"] = run_c_gcn(1000)
        result["dqn"] = run_small(dev, "dqn", 200, graph=not args.no_graph)
        result["dqn"]["c_caller"] = run_c_dqn([4, 128, 128, 2], 64, 2000)
        if not args.no_graph:
            for kind, n in (("gcn", 100), ("dqn", 200)):
                f = run_small(dev, kind, n, graph=True, fused=True)
                result[kind]["fused"] = {k: f[k] for k in ("steps_per_s", "ms_per_step", "graph_replay")}
    if not args.no_ops:
        if args.short_ops:
            global OP_WARM_MS
            OP_WARM_MS = 2.0
        result["ops"] = op_suite(dev, quick=args.short_ops)
        result["other_ops"] = result["ops"].pop("other_ops", None)  # the op surface outside the named suite
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(WIDE_DIMS, WIDE_BATCH, loss_mode=args.loss_mode)
        # the oracle ran the same first step from the same parameters and batch: its loss must be the device's
        if gpu_losses:
            o, g = result["cpu_baseline"]["first_step_loss"], gpu_losses[0]
            rel = abs(o - g) / max(1.0, abs(o))
            result["parity_check"] = {"what": "loss of the first train step, device against the CPU oracle",
                                      "device": g, "oracle": o, "rel_diff": rel, "bound": 1e-4, "ok": rel <= 1e-4}
        result["cpu_baseline"].pop("first_step_loss", None)
        result["cpu_baseline_1_thread"] = cpu_baseline(WIDE_DIMS, WIDE_BATCH, budget_steps=1, threads=1)
        result["cpu_baseline_1_thread"].pop("first_step_loss", None)
        # the same CPU oracle on the batch-64 MLP, the configuration the reference runs today
        from oracle.oracle_device import OracleDevice

        odev = OracleDevice()
        threads = odev.set_threads(min(16, os.cpu_count() or 1))
        dt_cpu, _ = run_mlp(odev, [784, 128, 64, 10], 64, "sgd", 200, 20, "uniform", None, "onehot", lr=0.01)
        result.setdefault("mlp_b64", {})["cpu_oracle"] = {"steps_per_s": 200 / dt_cpu, "ms_per_step": dt_cpu / 200 * 1e3, "cores": threads}
        if not args.no_small:
            for kind in ("gcn", "dqn"):
                c = run_small(odev, kind, 50, graph=False)
                result[kind]["cpu_oracle"] = {"steps_per_s": c["steps_per_s"], "ms_per_step": c["ms_per_step"], "cores": threads}
        if not args.no_ops:
            # the op suite on the host cores beside the GPU figures (BLAS on `threads` cores, everything else the
            # oracle's scalar loops on one core)
            strip = lambda d: {k: v for k, v in d.items() if not k.startswith("frac_")}
            for name, c in op_suite(odev, cpu=True).items():
                result["ops"][name]["cpu_oracle"] = strip(c)
                if name.startswith("smce"):
                    result["ops"][name]["cpu_oracle"]["rows_timed"] = 1024
            result["ops_cpu_oracle"] = {"cores_blas": threads, "cores_other": 1, "blas": odev.blas_name(),
                                        "sample": "one call per timing, median of 3; loss kernels on 1024 of the 8192 rows"}
    else:
        result["cpu_baseline"] = None
    dev.deinit()
    print(json.dumps(result))
    if result.get("parity_check") and not result["parity_check"]["ok"]:
        sys.exit("bench.py: the device's first-step loss differs from the CPU oracle's by more than 1e-4")


if __name__ == "__main__":
    main()
