"""The backward pass of a small Linear layer as an unchanged caller issues it (src/ndtensor.zig:780-796 for the bias's
unbroadcast, :1092-1136 for the two products, src/nn/nn.zig:44-50 for the ReLU node before the layer;
examples/mnist/src/model.zig:104-110): the bias gradient waits for the layer's products, the input-gradient product for
its mask, the weight-gradient product with it, and the three leave in one launch.  The results must be, bit for bit,
what the same calls give when each is launched on its own (forced by a synchronisation after every call), whatever the
caller does in between, and must agree with the float64 closed form."""
from __future__ import annotations

import numpy as np
import pytest

from zigrad_amd import host
from zigrad_amd.device import F32

pytestmark = pytest.mark.gpu

# (batch, fan_in, fan_out): the MNIST classifier's layers, the DQN net's, ragged sizes, one beyond the small kernels
SHAPES = [(64, 128, 10), (64, 784, 128), (64, 128, 64), (64, 64, 10), (64, 4, 128), (64, 128, 2), (33, 70, 29), (2, 5, 3),
          (100, 256, 160), (256, 300, 64), (512, 384, 96)]


def _layer_backward(hip, gy, w, x, mask, gw0, gb0, eager, with_input_grad=True, between=None):
    """One layer's backward in the reference's call order.  `between(stage)` lets a test do something after a stage."""
    B, O = gy.shape
    I = w.shape[1]
    step = hip.sync if eager else (lambda: None)
    wb, xb = hip.from_numpy(w), hip.from_numpy(x)
    mb = hip.from_numpy(mask) if mask is not None else None
    gwb, gbb = hip.from_numpy(gw0), hip.from_numpy(gb0)
    y = hip.mem_cache_alloc(F32, B * O)   # the layer's output: freed after the layer's backward
    g = hip.mem_cache_alloc(F32, B * O)   # its gradient
    hip.mem_transfer(gy, g, "HtoD")
    hip.sync()
    between = between or (lambda stage: None)
    host.unbroadcast_(hip, g, [B, O], gbb, [O], alpha=1.0, beta=1.0)
    step()
    between("bias")
    gx = None
    if with_input_grad:
        gx = hip.mem_cache_alloc(F32, B * I)
        hip.mem_fill(gx, 0.0)
        step()
        between("fill")
    # BmmAccBwd of y = x . w^T (host.bmm_acc_backward issues the same two calls): dX += dY . W, then dW += dY^T . X
    if gx is not None:
        host.bmm_acc_(hip, g, [B, O], wb, [O, I], gx, False, False, 1.0, 1.0)
        step()
    host.bmm_acc_(hip, g, [B, O], xb, [B, I], gwb, True, False, 1.0, 1.0)
    step()
    between("products")
    hip.mem_cache_free(y)
    hip.mem_cache_free(g)
    step()
    between("frees")
    if gx is not None and mb is not None:
        hip.dispatch("relu_inplace_bwd", x=mb, x_g=gx)
        step()
    out = (hip.to_numpy(gx).reshape(B, I) if gx is not None else None, hip.to_numpy(gwb).reshape(O, I), hip.to_numpy(gbb))
    if gx is not None:
        hip.mem_cache_free(gx)
    for b in (wb, xb, gwb, gbb) + ((mb,) if mb is not None else ()):
        hip.mem_free(b)
    return out


def _inputs(shape, seed=0):
    B, I, O = shape
    r = np.random.default_rng(seed + B + 3 * I + 7 * O)
    gy = r.standard_normal((B, O)).astype(np.float32)
    w = (r.standard_normal((O, I)) / np.sqrt(O)).astype(np.float32)
    x = np.maximum(r.standard_normal((B, I)), 0.0).astype(np.float32)
    gw0 = r.standard_normal((O, I)).astype(np.float32)
    gb0 = r.standard_normal(O).astype(np.float32)
    return gy, w, x, gw0, gb0


def _check_closed_form(shape, got, gy, w, x, gw0, gb0, masked):
    gx, gw, gb = got
    d = np.float64
    want_gw = gy.astype(d).T @ x.astype(d) + gw0
    want_gb = gy.astype(d).sum(axis=0) + gb0
    assert np.linalg.norm(gw - want_gw) <= 1e-5 * (np.linalg.norm(want_gw) + 1e-3), shape
    assert np.linalg.norm(gb - want_gb) <= 1e-5 * (np.linalg.norm(want_gb) + 1e-3), shape
    if gx is not None:
        want_gx = gy.astype(d) @ w.astype(d)
        if masked:
            want_gx = np.where(x > 0, want_gx, 0.0)
        assert np.linalg.norm(gx - want_gx) <= 1e-5 * (np.linalg.norm(want_gx) + 1e-3), shape


@pytest.mark.parametrize("shape", SHAPES)
def test_layer_backward_equals_the_ops_launched_one_by_one(hip, shape):
    gy, w, x, gw0, gb0 = _inputs(shape)
    in_use0 = hip.cache_stats()["bytes_in_use"]
    got = _layer_backward(hip, gy, w, x, x, gw0, gb0, eager=False)
    ref = _layer_backward(hip, gy, w, x, x, gw0, gb0, eager=True)
    for a, b in zip(got, ref):
        assert np.array_equal(a, b), shape
    _check_closed_form(shape, got, gy, w, x, gw0, gb0, masked=True)
    assert np.all(got[0][x <= 0] == 0.0)
    hip.sync()
    assert hip.cache_stats()["bytes_in_use"] == in_use0


@pytest.mark.parametrize("shape", SHAPES)
def test_first_layer_backward_without_an_input_gradient(hip, shape):
    gy, w, x, gw0, gb0 = _inputs(shape, seed=1)
    got = _layer_backward(hip, gy, w, x, None, gw0, gb0, eager=False, with_input_grad=False)
    ref = _layer_backward(hip, gy, w, x, None, gw0, gb0, eager=True, with_input_grad=False)
    assert np.array_equal(got[1], ref[1]) and np.array_equal(got[2], ref[2]), shape
    _check_closed_form(shape, got, gy, w, x, gw0, gb0, masked=False)


@pytest.mark.parametrize("shape", [(64, 128, 64), (33, 70, 29), (256, 300, 64)])
def test_last_layer_input_gradient_without_a_mask(hip, shape):
    """No ReLU before the layer: nothing follows the frees, and the next call of any kind sends the three out."""
    gy, w, x, gw0, gb0 = _inputs(shape, seed=2)
    got = _layer_backward(hip, gy, w, x, None, gw0, gb0, eager=False)
    ref = _layer_backward(hip, gy, w, x, None, gw0, gb0, eager=True)
    for a, b in zip(got, ref):
        assert np.array_equal(a, b), shape
    _check_closed_form(shape, got, gy, w, x, gw0, gb0, masked=False)


@pytest.mark.parametrize("stage", ["bias", "fill", "products", "frees"])
@pytest.mark.parametrize("what", ["sync", "alloc_fill", "other_product", "event"])
def test_a_caller_doing_something_else_between_the_calls(hip, stage, what):
    shape = (64, 128, 64)
    gy, w, x, gw0, gb0 = _inputs(shape, seed=3)
    r = np.random.default_rng(4)
    P = r.standard_normal((40, 24)).astype(np.float32)
    Q = r.standard_normal((24, 56)).astype(np.float32)
    seen = {}

    def between(at):
        if at != stage:
            return
        if what == "sync":
            hip.sync()
        elif what == "alloc_fill":
            t = hip.mem_cache_alloc(F32, 4096)
            hip.mem_fill(t, 7.0)
            seen["fill"] = hip.to_numpy(t)
            hip.mem_cache_free(t)
        elif what == "other_product":
            p, q = hip.from_numpy(P), hip.from_numpy(Q)
            c = hip.mem_alloc(F32, 40 * 56)
            hip.dispatch("matmul", A=p, B=q, C=c, m=40, n=56, k=24, trans_a=False, trans_b=False, lda=24, ldb=56, ldc=56,
                         alpha=1.0, beta=0.0)
            seen["prod"] = hip.to_numpy(c).reshape(40, 56)
            for b in (p, q, c):
                hip.mem_free(b)
        elif what == "event":
            seen["event"] = hip.event().record()

    got = _layer_backward(hip, gy, w, x, x, gw0, gb0, eager=False, between=between)
    ref = _layer_backward(hip, gy, w, x, x, gw0, gb0, eager=True)
    for a, b in zip(got, ref):
        assert np.array_equal(a, b), (stage, what)
    if "fill" in seen:
        assert np.all(seen["fill"] == 7.0)
    if "prod" in seen:
        want = P.astype(np.float64) @ Q.astype(np.float64)
        assert np.linalg.norm(seen["prod"] - want) <= 1e-5 * np.linalg.norm(want)


def test_reads_and_writes_of_the_waiting_bias_gradient_are_ordered(hip):
    B, O = 64, 48
    r = np.random.default_rng(6)
    gy = r.standard_normal((B, O)).astype(np.float32)
    gb0 = r.standard_normal(O).astype(np.float32)
    g, gb = hip.from_numpy(gy), hip.from_numpy(gb0)
    want = gy.astype(np.float64).sum(axis=0) + gb0
    host.unbroadcast_(hip, g, [B, O], gb, [O], alpha=1.0, beta=1.0)
    got = hip.to_numpy(gb)                                   # a read sends it out
    assert np.linalg.norm(got - want) <= 1e-5 * np.linalg.norm(want)
    host.unbroadcast_(hip, g, [B, O], gb, [O], alpha=1.0, beta=1.0)
    hip.mem_fill(gb, 0.0)                                    # zero_grad after it: the zeros win
    assert np.all(hip.to_numpy(gb) == 0.0)
    host.unbroadcast_(hip, g, [B, O], gb, [O], alpha=1.0, beta=1.0)
    hip.mem_fill(g, 1.0)                                     # its input overwritten after it: the old values count
    got = hip.to_numpy(gb)
    want0 = gy.astype(np.float64).sum(axis=0)
    assert np.linalg.norm(got - want0) <= 1e-5 * np.linalg.norm(want0)
    host.unbroadcast_(hip, g, [B, O], gb, [O], alpha=1.0, beta=1.0)
    host.unbroadcast_(hip, g, [B, O], gb, [O], alpha=1.0, beta=1.0)   # twice in a row: both count
    got = hip.to_numpy(gb)
    want2 = want0 + 2.0 * B
    assert np.linalg.norm(got - want2) <= 1e-5 * np.linalg.norm(want2)
    # the output gradient's block given back while the bias gradient waits alone: it is read before the block moves on
    gc = hip.mem_cache_alloc(F32, B * O)
    hip.mem_transfer(gy, gc, "HtoD")
    hip.mem_fill(gb, 0.0)
    hip.sync()
    host.unbroadcast_(hip, gc, [B, O], gb, [O], alpha=1.0, beta=1.0)
    hip.mem_cache_free(gc)
    t = hip.mem_cache_alloc(F32, B * O)
    hip.mem_fill(t, -5.0)
    got = hip.to_numpy(gb)
    assert np.linalg.norm(got - want0) <= 1e-5 * np.linalg.norm(want0)
    hip.mem_cache_free(t)
    for b in (g, gb):
        hip.mem_free(b)


def test_products_that_are_not_the_layers_own_send_the_bias_gradient_out_first(hip):
    """A product that writes what the waiting bias gradient reads, or reads what it writes, must find it done."""
    B, O, I = 64, 32, 48
    r = np.random.default_rng(8)
    gy = r.standard_normal((B, O)).astype(np.float32)
    g, gb = hip.from_numpy(gy), hip.from_numpy(np.zeros(O, np.float32))
    a = hip.from_numpy(r.standard_normal((B, I)).astype(np.float32))
    b = hip.from_numpy(r.standard_normal((I, O)).astype(np.float32))
    host.unbroadcast_(hip, g, [B, O], gb, [O], alpha=1.0, beta=1.0)
    # overwrites gy: the column sums must be of the old values
    hip.dispatch("matmul", A=a, B=b, C=g, m=B, n=O, k=I, trans_a=False, trans_b=False, lda=I, ldb=O, ldc=O, alpha=1.0, beta=0.0)
    got = hip.to_numpy(gb)
    want = gy.astype(np.float64).sum(axis=0)
    assert np.linalg.norm(got - want) <= 1e-5 * np.linalg.norm(want)
    # reads gb as an operand (a 1 x O row times O x ... ): must see the sums
    hip.mem_transfer(gy, g, "HtoD")
    hip.mem_fill(gb, 0.0)
    hip.sync()
    out = hip.mem_alloc(F32, B)
    host.unbroadcast_(hip, g, [B, O], gb, [O], alpha=1.0, beta=1.0)
    hip.dispatch("matmul", A=g, B=gb, C=out, m=B, n=1, k=O, trans_a=False, trans_b=False, lda=O, ldb=1, ldc=1, alpha=1.0, beta=0.0)
    got = hip.to_numpy(out)
    want = gy.astype(np.float64) @ gy.astype(np.float64).sum(axis=0)
    assert np.linalg.norm(got - want) <= 1e-5 * np.linalg.norm(want)
    for t in (g, gb, a, b, out):
        hip.mem_free(t)


def test_a_mask_that_lies_in_the_weight_gradient_is_read_after_the_weight_gradient_is_written(hip):
    """relu_inplace_bwd whose mask operand is the buffer the waiting weight-gradient product writes: the separate calls
    mask by the NEW weight gradient, so the three must not leave in one launch with that mask."""
    B = O = 32
    I = 48
    r = np.random.default_rng(12)
    gy = r.standard_normal((B, O)).astype(np.float32)
    w = r.standard_normal((O, I)).astype(np.float32)
    x = r.standard_normal((B, I)).astype(np.float32)
    gw0 = r.standard_normal((O, I)).astype(np.float32)
    outs = []
    for eager in (False, True):
        step = hip.sync if eager else (lambda: None)
        g, wb, xb, gwb = hip.from_numpy(gy), hip.from_numpy(w), hip.from_numpy(x), hip.from_numpy(gw0)
        gb = hip.from_numpy(np.zeros(O, np.float32))
        host.unbroadcast_(hip, g, [B, O], gb, [O], alpha=1.0, beta=1.0)
        step()
        gx = hip.mem_cache_alloc(F32, B * I)
        hip.mem_fill(gx, 0.0)
        step()
        host.bmm_acc_(hip, g, [B, O], wb, [O, I], gx, False, False, 1.0, 1.0)
        step()
        host.bmm_acc_(hip, g, [B, O], xb, [B, I], gwb, True, False, 1.0, 1.0)
        step()
        hip.dispatch("relu_inplace_bwd", x=gwb, x_g=gx)      # O * I == B * I: the weight gradient as the mask
        step()
        outs.append((hip.to_numpy(gx), hip.to_numpy(gwb), hip.to_numpy(gb)))
        hip.mem_cache_free(gx)
        for t in (g, wb, xb, gwb, gb):
            hip.mem_free(t)
    for a, b in zip(*outs):
        assert np.array_equal(a, b)
    new_gw = gy.astype(np.float64).T @ x.astype(np.float64) + gw0
    want = np.where(new_gw.ravel() > 0, (gy.astype(np.float64) @ w.astype(np.float64)).ravel(), 0.0)
    sure = np.abs(new_gw.ravel()) > 1e-4          # away from the mask's threshold, where rounding cannot flip it
    assert np.allclose(outs[0][0][sure], want[sure], rtol=1e-4, atol=1e-5)
