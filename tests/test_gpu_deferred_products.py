"""A layer's forward product waits one call for the bias add and the ReLU that follow it, an input-gradient product
for the mask that follows it (letting the weight-gradient product pass); what follows is then done in the product's
epilogue.  An unchanged caller's sequence (examples/mnist/src/model.zig:104-110, :38-46; src/ndtensor.zig:1092-1136;
src/nn/nn.zig:44-50) must give, bit for bit, what the same calls give when every one of them is launched on its own
(forced here by a synchronisation after each call), whatever comes next: the expected op, another op on the same
memory, a read, a free."""
from __future__ import annotations

import numpy as np
import pytest

from zigrad_amd._lib import ZgHipError
from zigrad_amd.device import F32

pytestmark = pytest.mark.gpu

SHAPES = [(64, 784, 128), (64, 64, 10), (33, 70, 129), (256, 512, 384), (250, 512, 380), (1024, 1024, 1024),
          (130, 1433, 16), (2048, 1000, 1024), (2560, 1024, 3328), (2560, 1024, 3332), (2, 5, 3)]


def _forward(hip, x, w, bias, relu, bias_first, eager):
    """bmm_acc(trans_b) -> add -> relu_fwd as the reference's Linear layer issues them; eager: a sync after each."""
    B, I = x.shape
    O = w.shape[0]
    xb, wb, bb = hip.from_numpy(x), hip.from_numpy(w), hip.from_numpy(bias)
    y = hip.mem_cache_alloc(F32, B * O)
    step = hip.sync if eager else (lambda: None)
    hip.dispatch("bmm_acc", A=xb, B=wb, C=y, A_shape=[1, B, I], B_shape=[1, I, O], C_shape=[1, B, O], trans_a=False,
                 trans_b=True, lda=I, ldb=I, ldc=O, alpha=1.0, beta=0.0)
    step()
    if bias_first:
        hip.dispatch("add", x=bb, y=y, z=y)   # bias.add_(y): the shorter operand first
    else:
        hip.dispatch("add", x=y, y=bb, z=y)
    step()
    if relu:
        hip.dispatch("relu_fwd", x=y, y=y)
        step()
    out = hip.to_numpy(y).reshape(B, O)
    for b in (xb, wb, bb):
        hip.mem_free(b)
    hip.mem_cache_free(y)
    return out


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("relu,bias_first", [(True, True), (False, True), (True, False)])
def test_linear_forward_sequence_equals_the_ops_launched_one_by_one(hip, shape, relu, bias_first):
    B, I, O = shape
    r = np.random.default_rng(B + 3 * I + 7 * O)
    x = r.standard_normal((B, I)).astype(np.float32)
    w = (r.standard_normal((O, I)) / np.sqrt(I)).astype(np.float32)
    bias = r.standard_normal(O).astype(np.float32)
    got = _forward(hip, x, w, bias, relu, bias_first, eager=False)
    ref = _forward(hip, x, w, bias, relu, bias_first, eager=True)
    assert np.array_equal(got, ref), shape
    want = x.astype(np.float64) @ w.astype(np.float64).T + bias
    if relu:
        want = np.maximum(want, 0.0)
    assert np.linalg.norm(got - want) <= 1e-5 * (np.linalg.norm(want) + 1e-3)


def _backward(hip, gy, w, x, act, eager):
    """ensure_grad(0) -> dX += dY W -> dW += dY^T X -> relu_inplace_bwd(act, dX), as BmmAccBwd and the ReLU node do."""
    B, O = gy.shape
    I = w.shape[1]
    gyb, wb, xb, ab = hip.from_numpy(gy), hip.from_numpy(w), hip.from_numpy(x), hip.from_numpy(act)
    gw = hip.from_numpy(np.full(O * I, 0.25, np.float32))  # an existing weight gradient: accumulated into
    gx = hip.mem_cache_alloc(F32, B * I)
    step = hip.sync if eager else (lambda: None)
    hip.mem_fill(gx, 0.0)
    step()
    hip.dispatch("bmm_acc", A=gyb, B=wb, C=gx, A_shape=[1, B, O], B_shape=[1, O, I], C_shape=[1, B, I], trans_a=False,
                 trans_b=False, lda=O, ldb=I, ldc=I, alpha=1.0, beta=1.0)
    step()
    hip.dispatch("bmm_acc", A=gyb, B=xb, C=gw, A_shape=[1, O, B], B_shape=[1, B, I], C_shape=[1, O, I], trans_a=True,
                 trans_b=False, lda=O, ldb=I, ldc=I, alpha=1.0, beta=1.0)
    step()
    hip.dispatch("relu_inplace_bwd", x=ab, x_g=gx)
    step()
    out = hip.to_numpy(gx).reshape(B, I), hip.to_numpy(gw).reshape(O, I)
    for b in (gyb, wb, xb, ab, gw):
        hip.mem_free(b)
    hip.mem_cache_free(gx)
    return out


@pytest.mark.parametrize("shape", SHAPES)
def test_layer_backward_sequence_equals_the_ops_launched_one_by_one(hip, shape):
    B, I, O = shape
    r = np.random.default_rng(5 * B + I + O)
    gy = r.standard_normal((B, O)).astype(np.float32)
    w = (r.standard_normal((O, I)) / np.sqrt(O)).astype(np.float32)
    x = np.maximum(r.standard_normal((B, I)), 0.0).astype(np.float32)  # the layer's input: a ReLU output, and the mask
    got_gx, got_gw = _backward(hip, gy, w, x, x, eager=False)
    ref_gx, ref_gw = _backward(hip, gy, w, x, x, eager=True)
    assert np.array_equal(got_gx, ref_gx) and np.array_equal(got_gw, ref_gw), shape
    want_gx = np.where(x > 0, gy.astype(np.float64) @ w.astype(np.float64), 0.0)
    want_gw = gy.astype(np.float64).T @ x.astype(np.float64) + 0.25
    assert np.linalg.norm(got_gx - want_gx) <= 1e-5 * (np.linalg.norm(want_gx) + 1e-3)
    assert np.linalg.norm(got_gw - want_gw) <= 1e-5 * (np.linalg.norm(want_gw) + 1e-3)
    assert np.all(got_gx[x <= 0] == 0.0)


def test_whatever_follows_a_waiting_product_sees_its_result(hip):
    r = np.random.default_rng(9)
    m, n, k = 200, 96, 80
    A = r.standard_normal((m, k)).astype(np.float32)
    W = r.standard_normal((n, k)).astype(np.float32)
    prod = (A.astype(np.float64) @ W.astype(np.float64).T)
    a, w = hip.from_numpy(A), hip.from_numpy(W)
    c = hip.mem_alloc(F32, m * n)

    def product():
        hip.dispatch("matmul", A=a, B=w, C=c, m=m, n=n, k=k, trans_a=False, trans_b=True, lda=k, ldb=k, ldc=n, alpha=1.0,
                     beta=0.0)

    def close(got, want):
        return np.linalg.norm(got - want) <= 1e-5 * np.linalg.norm(want)

    product()
    assert close(hip.to_numpy(c).reshape(m, n), prod)                      # a read
    product()
    hip.mem_fill(c, 3.0)                                                   # a fill of its output comes after it
    assert np.all(hip.to_numpy(c) == 3.0)
    product()
    other = hip.from_numpy(np.ones(m * n, np.float32))
    hip.dispatch("add", x=other, y=c, z=c)                                 # an add that is not a bias row
    assert close(hip.to_numpy(c).reshape(m, n), prod + 1.0)
    product()
    hip.dispatch("relu_fwd", x=c.sub(0, 50 * n), y=c.sub(0, 50 * n))       # a ReLU of a part of it only
    want = prod.copy()
    want[:50] = np.maximum(want[:50], 0.0)
    assert close(hip.to_numpy(c).reshape(m, n), want)
    product()
    d = hip.mem_alloc(F32, m * n)
    hip.dispatch("relu_fwd", x=c, y=d)                                     # a ReLU into another buffer
    assert close(hip.to_numpy(d).reshape(m, n), np.maximum(prod, 0.0)) and close(hip.to_numpy(c).reshape(m, n), prod)
    product()
    bias = hip.from_numpy(np.arange(n, dtype=np.float32))
    hip.dispatch("add", x=bias, y=c, z=c)
    hip.dispatch("add", x=bias, y=c, z=c)                                  # a second bias row: only the first is taken over
    assert close(hip.to_numpy(c).reshape(m, n), prod + 2.0 * np.arange(n))
    product()
    hip.dispatch("add", x=bias, y=c, z=c)
    c2 = hip.mem_alloc(F32, m * n)                                         # an allocation sends it out
    hip.dispatch("relu_fwd", x=c, y=c)
    assert close(hip.to_numpy(c).reshape(m, n), np.maximum(prod + np.arange(n), 0.0))
    # a second product that reads the waiting one's output goes after it
    product()
    e = hip.mem_alloc(F32, m * m)
    hip.dispatch("matmul", A=c, B=c, C=e, m=m, n=m, k=n, trans_a=False, trans_b=True, lda=n, ldb=n, ldc=m, alpha=1.0, beta=0.0)
    assert close(hip.to_numpy(e).reshape(m, m), prod @ prod.T)
    # a refused product is reported by the call itself
    with pytest.raises(ZgHipError):
        hip.dispatch("matmul", A=a, B=w, C=c, m=m, n=n, k=k, trans_a=False, trans_b=True, lda=k - 1, ldb=k, ldc=n, alpha=1.0,
                     beta=0.0)
    for b in (a, w, c, other, d, bias, c2, e):
        hip.mem_free(b)


def test_an_input_gradient_waits_only_for_products_that_leave_it_alone(hip):
    r = np.random.default_rng(10)
    B, I, O = 128, 96, 64
    gy = r.standard_normal((B, O)).astype(np.float32)
    w = r.standard_normal((O, I)).astype(np.float32)
    act = np.maximum(r.standard_normal((B, I)), 0.0).astype(np.float32)
    gyb, wb, ab = hip.from_numpy(gy), hip.from_numpy(w), hip.from_numpy(act)
    gx = hip.mem_alloc(F32, B * I)
    out = hip.mem_alloc(F32, I * I)
    hip.mem_fill(gx, 0.0)
    hip.dispatch("matmul", A=gyb, B=wb, C=gx, m=B, n=I, k=O, trans_a=False, trans_b=False, lda=O, ldb=I, ldc=I, alpha=1.0,
                 beta=1.0)
    # this product READS the waiting one's output: the waiting one must go first, unmasked
    hip.dispatch("matmul", A=gx, B=gx, C=out, m=I, n=I, k=B, trans_a=True, trans_b=False, lda=I, ldb=I, ldc=I, alpha=1.0,
                 beta=0.0)
    hip.dispatch("relu_inplace_bwd", x=ab, x_g=gx)
    full = gy.astype(np.float64) @ w.astype(np.float64)
    got_out = hip.to_numpy(out).reshape(I, I)
    assert np.linalg.norm(got_out - full.T @ full) <= 1e-5 * np.linalg.norm(full.T @ full)
    got = hip.to_numpy(gx).reshape(B, I)
    want = np.where(act > 0, full, 0.0)
    assert np.linalg.norm(got - want) <= 1e-5 * np.linalg.norm(want)
    for b in (gyb, wb, ab, gx, out):
        hip.mem_free(b)


@pytest.mark.parametrize("shape", [(64, 128, 64), (256, 512, 384), (1024, 1024, 1024)])
def test_frees_of_the_backward_pass_do_not_disturb_a_waiting_input_gradient(hip, shape):
    """The reference frees a layer's output and its gradient as soon as the layer's backward has run, which is before the
    mask of the input gradient arrives: blocks that hold an operand of the waiting product go back to the pool when the
    product has been launched, others at once; the pool ends where it started."""
    B, I, O = shape
    r = np.random.default_rng(B + I + O)
    gy = r.standard_normal((B, O)).astype(np.float32)
    w = (r.standard_normal((O, I)) / np.sqrt(O)).astype(np.float32)
    act = np.maximum(r.standard_normal((B, I)), 0.0).astype(np.float32)
    wb, ab = hip.from_numpy(w), hip.from_numpy(act)
    gw0 = r.standard_normal((O, I)).astype(np.float32)
    outs = []
    in_use0 = hip.cache_stats()["bytes_in_use"]
    for eager in (False, True):
        step = hip.sync if eager else (lambda: None)
        y = hip.mem_cache_alloc(F32, B * O)            # the layer's output: freed after the layer's backward
        g = hip.mem_cache_alloc(F32, B * O)            # its gradient: an operand of both products
        hip.mem_transfer(gy, g, "HtoD")
        gw = hip.from_numpy(gw0)
        gx = hip.mem_cache_alloc(F32, B * I)
        hip.mem_fill(gx, 0.0)
        step()
        hip.dispatch("bmm_acc", A=g, B=wb, C=gx, A_shape=[1, B, O], B_shape=[1, O, I], C_shape=[1, B, I], trans_a=False,
                     trans_b=False, lda=O, ldb=I, ldc=I, alpha=1.0, beta=1.0)
        step()
        hip.dispatch("bmm_acc", A=g, B=ab, C=gw, A_shape=[1, O, B], B_shape=[1, B, I], C_shape=[1, O, I], trans_a=True,
                     trans_b=False, lda=O, ldb=I, ldc=I, alpha=1.0, beta=1.0)
        step()
        hip.mem_cache_free(y)
        hip.mem_cache_free(g)
        step()
        hip.dispatch("relu_inplace_bwd", x=ab, x_g=gx)
        step()
        # memory handed out now must not be what the waiting product still had to read
        scratch = hip.mem_cache_alloc(F32, B * O)
        hip.mem_fill(scratch, 123.0)
        outs.append((hip.to_numpy(gx).reshape(B, I), hip.to_numpy(gw).reshape(O, I)))
        hip.mem_cache_free(scratch)
        hip.mem_cache_free(gx)
        hip.mem_free(gw)
    hip.sync()
    assert hip.cache_stats()["bytes_in_use"] == in_use0
    (gx_a, gw_a), (gx_b, gw_b) = outs
    assert np.array_equal(gx_a, gx_b) and np.array_equal(gw_a, gw_b)
    want = np.where(act > 0, gy.astype(np.float64) @ w.astype(np.float64), 0.0)
    assert np.linalg.norm(gx_a - want) <= 1e-5 * (np.linalg.norm(want) + 1e-3)
    for b in (wb, ab):
        hip.mem_free(b)


def test_giving_a_block_back_twice_while_its_free_waits_is_refused(hip):
    B, I, O = 64, 32, 48
    r = np.random.default_rng(3)
    g = hip.mem_cache_alloc(F32, B * O)
    hip.mem_transfer(r.standard_normal(B * O).astype(np.float32), g, "HtoD")
    wb = hip.from_numpy(r.standard_normal(O * I).astype(np.float32))
    gx = hip.mem_cache_alloc(F32, B * I)
    hip.mem_fill(gx, 0.0)
    hip.dispatch("bmm_acc", A=g, B=wb, C=gx, A_shape=[1, B, O], B_shape=[1, O, I], C_shape=[1, B, I], trans_a=False,
                 trans_b=False, lda=O, ldb=I, ldc=I, alpha=1.0, beta=1.0)
    ptr, block = g.ptr, g.block
    hip.mem_cache_free(g)
    with pytest.raises(ZgHipError):
        hip._call("zg_hip_mem_cache_free", ptr, block)
    hip.sync()
    hip.mem_cache_free(gx)
    hip.mem_free(wb)
