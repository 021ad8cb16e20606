"""A graph-convolution layer as an unchanged caller issues it (examples/gcn/src/model.zig:100-112, :36 for the
forward: a zeroed output, scatter_gcn_deg_scaled, y._add(bias), relu_; src/ndtensor.zig:221-228 and :1437-1513 for the
backward: two zeroed gradients, scatter_gcn_deg_scaled_bwd).  The zero fills are taken over by the op that would add
to them, and the aggregation's kernel waits for the bias add and the ReLU, which run as its tail.  Every sequence must
give, bit for bit, what the same calls give when each is launched on its own (a synchronisation after every call) and
what the host's sequential loops give (the oracle)."""
from __future__ import annotations

import numpy as np
import pytest

from conftest import run_op
from zigrad_amd.device import F32, U64

pytestmark = pytest.mark.gpu

GRAPHS = [(2708, 13264, 16), (2708, 13264, 7), (300, 2000, 5), (64, 40, 33), (1000, 1, 4), (50, 5000, 64)]


def _graph(n_nodes, n_edge, stride, seed=0):
    r = np.random.default_rng(seed + n_nodes + n_edge + stride)
    src = r.integers(0, n_nodes, n_edge).astype(np.uint64)
    tgt = r.integers(0, max(1, n_nodes - n_nodes // 10), n_edge).astype(np.uint64)   # a tenth of the nodes has no in-edge
    h = r.standard_normal((n_nodes, stride)).astype(np.float32)
    deg = (1.0 / np.sqrt(1.0 + r.integers(0, 9, n_nodes))).astype(np.float32)
    bias = r.standard_normal(stride).astype(np.float32)
    return src, tgt, h, deg, bias


def _index(hip, arr, pinned):
    if pinned:
        buf = hip.mem_alloc_host(U64, arr.size)
        hip.host_view(buf)[:] = arr
        return buf
    return hip.from_numpy(arr)


def _forward(hip, g, shape, eager, pinned, zero_first=True, bias_first=True, relu=True, add_bias=True, between=None):
    n_nodes, n_edge, stride = shape
    src, tgt, h, deg, bias = g
    step = hip.sync if eager else (lambda: None)
    sb, tb = _index(hip, src, pinned), _index(hip, tgt, pinned)
    hb, db, bb = hip.from_numpy(h), hip.from_numpy(deg), hip.from_numpy(bias)
    y = hip.mem_cache_alloc(F32, n_nodes * stride)
    if zero_first:
        hip.mem_fill(y, 0.0)
    else:
        hip.mem_transfer(np.full(n_nodes * stride, 0.5, np.float32), y, "HtoD")
    step()
    hip.dispatch("scatter_gcn_deg_scaled", dst=y, h=hb, deg=db, src_indices=sb, tgt_indices=tb, stride=stride, n_edge=n_edge)
    step()
    if between:
        between(hip, y)
    if add_bias:
        if bias_first:
            hip.dispatch("add", x=bb, y=y, z=y)
        else:
            hip.dispatch("add", x=y, y=bb, z=y)
        step()
    if relu:
        hip.dispatch("relu_fwd", x=y, y=y)
        step()
    out = hip.to_numpy(y).reshape(n_nodes, stride)
    hip.mem_cache_free(y)
    for b in (sb, tb, hb, db, bb):
        hip.mem_free(b)
    return out


def _forward_oracle(oracle, g, shape, zero_first, relu, add_bias):
    n_nodes, n_edge, stride = shape
    src, tgt, h, deg, bias = g
    dst = np.zeros((n_nodes, stride), np.float32) if zero_first else np.full((n_nodes, stride), 0.5, np.float32)
    out = run_op(oracle, "scatter_gcn_deg_scaled", {"dst": dst.ravel(), "h": h.ravel(), "deg": deg, "src_indices": src, "tgt_indices": tgt,
                                                    "stride": stride, "n_edge": n_edge}, ["dst"])["dst"].reshape(n_nodes, stride)
    if add_bias:
        out = out + bias            # fp32 + fp32, one rounding: the add op
    if relu:
        out = np.where(out > 0, out, np.float32(0.0)).astype(np.float32)
    return out.astype(np.float32)


@pytest.mark.parametrize("shape", GRAPHS)
@pytest.mark.parametrize("pinned", [True, False])
def test_layer_forward_equals_the_ops_launched_one_by_one(oracle, hip, shape, pinned):
    g = _graph(*shape)
    got = _forward(hip, g, shape, eager=False, pinned=pinned)
    ref = _forward(hip, g, shape, eager=True, pinned=pinned)
    np.testing.assert_array_equal(got, ref)
    np.testing.assert_array_equal(got, _forward_oracle(oracle, g, shape, True, True, True))


@pytest.mark.parametrize("zero_first,bias_first,relu,add_bias", [(False, True, True, True), (True, False, True, True),
                                                                 (True, True, False, True), (True, True, True, False),
                                                                 (False, False, False, False)])
def test_layer_forward_variants(oracle, hip, zero_first, bias_first, relu, add_bias):
    shape = (300, 2000, 5)
    g = _graph(*shape, seed=1)
    kw = dict(zero_first=zero_first, bias_first=bias_first, relu=relu, add_bias=add_bias)
    got = _forward(hip, g, shape, eager=False, pinned=True, **kw)
    ref = _forward(hip, g, shape, eager=True, pinned=True, **kw)
    np.testing.assert_array_equal(got, ref)
    np.testing.assert_array_equal(got, _forward_oracle(oracle, g, shape, zero_first, relu, add_bias))


@pytest.mark.parametrize("what", ["read", "fill_output", "alloc", "second_scatter", "other_add"])
def test_whatever_follows_a_waiting_aggregation_sees_its_result(oracle, hip, what):
    shape = (300, 2000, 8)
    g = _graph(*shape, seed=2)
    src, tgt, h, deg, bias = g
    plain = _forward_oracle(oracle, g, shape, True, False, False)
    seen = {}

    def between(hip, y):
        if what == "read":
            seen["y"] = hip.to_numpy(y).reshape(shape[0], shape[2])
        elif what == "fill_output":
            hip.mem_fill(y, 2.0)
        elif what == "alloc":
            t = hip.mem_cache_alloc(F32, 1000)
            hip.mem_fill(t, 1.0)
            hip.mem_cache_free(t)
        elif what == "second_scatter":
            sb, tb = hip.from_numpy(src), hip.from_numpy(tgt)
            hb, db = hip.from_numpy(h), hip.from_numpy(deg)
            hip.dispatch("scatter_gcn_deg_scaled", dst=y, h=hb, deg=db, src_indices=sb, tgt_indices=tb, stride=shape[2],
                         n_edge=shape[1])
            seen["twice"] = True
            hip.sync()
            for b in (sb, tb, hb, db):
                hip.mem_free(b)
        elif what == "other_add":
            ones = hip.from_numpy(np.ones(shape[0] * shape[2], np.float32))
            hip.dispatch("add", x=ones, y=y, z=y)       # not a bias row: an ordinary add after the aggregation
            hip.sync()
            hip.mem_free(ones)

    got = _forward(hip, g, shape, eager=False, pinned=False, between=between)
    ref = _forward(hip, g, shape, eager=True, pinned=False, between=between)
    np.testing.assert_array_equal(got, ref)
    if what == "read":
        np.testing.assert_array_equal(seen["y"], plain)
    if what == "fill_output":
        want = np.maximum(np.float32(2.0) + bias, 0).astype(np.float32)
        np.testing.assert_array_equal(got, np.broadcast_to(want, got.shape))
    if what == "alloc":
        np.testing.assert_array_equal(got, _forward_oracle(oracle, g, shape, True, True, True))


def _backward(hip, g, shape, go, eager, pinned, zero_h=True, zero_d=True):
    n_nodes, n_edge, stride = shape
    src, tgt, h, deg, _ = g
    step = hip.sync if eager else (lambda: None)
    sb, tb = _index(hip, src, pinned), _index(hip, tgt, pinned)
    hb, db, gob = hip.from_numpy(h), hip.from_numpy(deg), hip.from_numpy(go)
    gh = hip.mem_cache_alloc(F32, n_nodes * stride)
    gd = hip.mem_cache_alloc(F32, n_nodes)
    if zero_h:
        hip.mem_fill(gh, 0.0)
    else:
        hip.mem_transfer(np.full(n_nodes * stride, 0.25, np.float32), gh, "HtoD")
    step()
    if zero_d:
        hip.mem_fill(gd, 0.0)
    else:
        hip.mem_transfer(np.full(n_nodes, -0.5, np.float32), gd, "HtoD")
    step()
    hip.dispatch("scatter_gcn_deg_scaled_bwd", grad_output=gob, h=hb, deg=db, src_indices=sb, tgt_indices=tb, grad_h=gh,
                 grad_deg=gd, stride=stride, n_edge=n_edge)
    step()
    out = hip.to_numpy(gh).reshape(n_nodes, stride), hip.to_numpy(gd)
    hip.mem_cache_free(gh)
    hip.mem_cache_free(gd)
    for b in (sb, tb, hb, db, gob):
        hip.mem_free(b)
    return out


@pytest.mark.parametrize("shape", GRAPHS)
@pytest.mark.parametrize("pinned", [True, False])
@pytest.mark.parametrize("zero_h,zero_d", [(True, True), (True, False), (False, True), (False, False)])
def test_layer_backward_with_waiting_zero_fills(oracle, hip, shape, pinned, zero_h, zero_d):
    n_nodes, n_edge, stride = shape
    g = _graph(*shape, seed=3)
    src, tgt, h, deg, _ = g
    go = np.random.default_rng(5).standard_normal((n_nodes, stride)).astype(np.float32)
    got = _backward(hip, g, shape, go, False, pinned, zero_h, zero_d)
    ref = _backward(hip, g, shape, go, True, pinned, zero_h, zero_d)
    np.testing.assert_array_equal(got[0], ref[0])
    np.testing.assert_array_equal(got[1], ref[1])
    gh0 = np.zeros((n_nodes, stride), np.float32) if zero_h else np.full((n_nodes, stride), 0.25, np.float32)
    gd0 = np.zeros(n_nodes, np.float32) if zero_d else np.full(n_nodes, -0.5, np.float32)
    want = run_op(oracle, "scatter_gcn_deg_scaled_bwd", {"grad_output": go.ravel(), "h": h.ravel(), "deg": deg, "src_indices": src,
                                                         "tgt_indices": tgt, "grad_h": gh0.ravel(), "grad_deg": gd0, "stride": stride,
                                                         "n_edge": n_edge}, ["grad_h", "grad_deg"])
    np.testing.assert_array_equal(got[0], want["grad_h"].reshape(n_nodes, stride))
    np.testing.assert_array_equal(got[1], want["grad_deg"])


@pytest.mark.parametrize("shape", [(2708, 13264, 16), (300, 2000, 5), (50, 5000, 64)])
@pytest.mark.parametrize("pinned", [True, False])
def test_a_degree_gradient_that_is_given_back_unread_is_never_computed_and_changes_nothing(oracle, hip, shape, pinned):
    """The layer computes the degree gradient into a buffer it frees at once (the degrees are data of the graph,
    src/ndtensor.zig:1009).  The two launches that compute it wait for the next call; a free of their output drops
    them.  The feature gradient must be what it always was, a later owner of the freed block must not be written to,
    and a degree gradient that IS read later (after frees of other blocks) must be right."""
    n_nodes, n_edge, stride = shape
    g = _graph(*shape, seed=7)
    src, tgt, h, deg, _ = g
    go = np.random.default_rng(8).standard_normal((n_nodes, stride)).astype(np.float32)
    want = run_op(oracle, "scatter_gcn_deg_scaled_bwd", {"grad_output": go.ravel(), "h": h.ravel(), "deg": deg, "src_indices": src,
                                                         "tgt_indices": tgt, "grad_h": np.zeros(n_nodes * stride, np.float32),
                                                         "grad_deg": np.zeros(n_nodes, np.float32), "stride": stride,
                                                         "n_edge": n_edge}, ["grad_h", "grad_deg"])
    sb, tb = _index(hip, src, pinned), _index(hip, tgt, pinned)
    hb, db, gob = hip.from_numpy(h), hip.from_numpy(deg), hip.from_numpy(go)
    in_use0 = hip.cache_stats()["bytes_in_use"]
    for read_it in (False, True):
        gh = hip.mem_cache_alloc(F32, n_nodes * stride)
        gd = hip.mem_cache_alloc(F32, n_nodes)
        other = hip.mem_cache_alloc(F32, 64)
        hip.mem_fill(gh, 0.0)
        hip.mem_fill(gd, 0.0)
        hip.dispatch("scatter_gcn_deg_scaled_bwd", grad_output=gob, h=hb, deg=db, src_indices=sb, tgt_indices=tb, grad_h=gh,
                     grad_deg=gd, stride=stride, n_edge=n_edge)
        if read_it:
            hip.mem_cache_free(other)              # a free of another block: the waiting work goes out, nothing is lost
            np.testing.assert_array_equal(hip.to_numpy(gd), want["grad_deg"])
            hip.mem_cache_free(gd)
        else:
            hip.mem_cache_free(gd)                 # unread: dropped
            t = hip.mem_cache_alloc(F32, n_nodes)  # the same block again, most likely
            marker = np.arange(n_nodes, dtype=np.float32)
            hip.mem_transfer(marker, t, "HtoD")
            hip.sync()
            np.testing.assert_array_equal(hip.to_numpy(t), marker)
            hip.mem_cache_free(t)
            hip.mem_cache_free(other)
        np.testing.assert_array_equal(hip.to_numpy(gh), want["grad_h"])
        hip.mem_cache_free(gh)
    hip.sync()
    assert hip.cache_stats()["bytes_in_use"] == in_use0
    for b in (sb, tb, hb, db, gob):
        hip.mem_free(b)
