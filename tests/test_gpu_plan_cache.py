"""Destination orderings kept between calls for index arrays in pinned host memory: every call must give what the
host's sequential loop gives (src/device/host_device.zig:1039-1087, :1356-1403; src/ndtensor.zig:1437-1513), whether
its ordering was just computed, found again, found under another pointer, or replaced because the caller rewrote
the array; a recorded step refuses to replay over a rewritten array."""
from __future__ import annotations

import numpy as np
import pytest

from conftest import run_op
from zigrad_amd._lib import ZgHipError
from zigrad_amd.device import F32, U64

pytestmark = pytest.mark.gpu


def _pinned(hip, arr):
    buf = hip.mem_alloc_host(U64, arr.size)
    hip.host_view(buf)[:] = arr
    return buf


def _scatter(hip, src_np, off_buf, dst_np):
    s, d = hip.from_numpy(src_np), hip.from_numpy(dst_np)
    hip.dispatch("scatter_add", src=s, offsets=off_buf, dst=d)
    hip.sync()
    out = hip.to_numpy(d)
    hip.mem_free(s)
    hip.mem_free(d)
    return out


def test_scatter_add_reuses_and_replaces_kept_orderings(oracle, hip):
    r = np.random.default_rng(0)
    n, n_dst = 5000, 300
    off = r.integers(0, n_dst, n).astype(np.uint64)
    src = r.standard_normal(n).astype(np.float32)
    dst0 = r.standard_normal(n_dst).astype(np.float32)

    def want(o, s=src):
        return run_op(oracle, "scatter_add", {"src": s, "offsets": o, "dst": dst0.copy()}, ["dst"])["dst"]

    a = _pinned(hip, off)
    before = hip.plan_cache_stats()
    np.testing.assert_array_equal(_scatter(hip, src, a, dst0), want(off))
    mid = hip.plan_cache_stats()
    assert mid["builds"] == before["builds"] + 1
    # the same array again, other values to add: served from the kept ordering
    src2 = r.standard_normal(n).astype(np.float32)
    np.testing.assert_array_equal(_scatter(hip, src2, a, dst0), want(off, src2))
    # the same contents at another address
    b = _pinned(hip, off)
    np.testing.assert_array_equal(_scatter(hip, src, b, dst0), want(off))
    after = hip.plan_cache_stats()
    assert after["hits"] == mid["hits"] + 2 and after["builds"] == mid["builds"]
    # the caller rewrites the array in place: one changed entry must be seen
    off2 = off.copy()
    off2[n // 2] = (off2[n // 2] + 1) % n_dst
    hip.sync()
    hip.host_view(a)[:] = off2
    np.testing.assert_array_equal(_scatter(hip, src, a, dst0), want(off2))
    assert hip.plan_cache_stats()["builds"] == after["builds"] + 1
    # and back: the first ordering is still kept
    hip.sync()
    hip.host_view(a)[:] = off
    np.testing.assert_array_equal(_scatter(hip, src, a, dst0), want(off))
    assert hip.plan_cache_stats()["builds"] == after["builds"] + 1
    hip.mem_free(a)
    hip.mem_free(b)


def test_more_arrays_than_the_cache_keeps(oracle, hip):
    r = np.random.default_rng(1)
    n, n_dst = 1200, 97
    src = r.standard_normal(n).astype(np.float32)
    dst0 = np.zeros(n_dst, np.float32)
    arrays = [r.integers(0, n_dst, n).astype(np.uint64) for _ in range(20)]
    bufs = [_pinned(hip, a) for a in arrays]
    for rounds in range(2):  # the second round meets evicted and kept orderings alike
        for a, b in zip(arrays, bufs):
            want = run_op(oracle, "scatter_add", {"src": src, "offsets": a, "dst": dst0.copy()}, ["dst"])["dst"]
            np.testing.assert_array_equal(_scatter(hip, src, b, dst0), want)
    for b in bufs:
        hip.mem_free(b)


def _gcn_case(r, n_nodes, n_edge, f):
    src = r.integers(0, n_nodes, n_edge).astype(np.uint64)
    tgt = r.integers(0, n_nodes, n_edge).astype(np.uint64)
    h = r.standard_normal(n_nodes * f).astype(np.float32)
    deg = r.uniform(0.2, 1.0, n_nodes).astype(np.float32)
    go = r.standard_normal(n_nodes * f).astype(np.float32)
    return src, tgt, h, deg, go


def test_gcn_scatter_forward_and_backward_on_kept_orderings(oracle, hip):
    r = np.random.default_rng(2)
    n_nodes, n_edge, f = 700, 9000, 16
    src, tgt, h, deg, go = _gcn_case(r, n_nodes, n_edge, f)
    fw = {"dst": np.zeros(n_nodes * f, np.float32), "h": h, "deg": deg, "src_indices": src, "tgt_indices": tgt,
          "stride": f, "n_edge": n_edge}
    bw = {"grad_output": go, "h": h, "deg": deg, "src_indices": src, "tgt_indices": tgt,
          "grad_h": np.zeros(n_nodes * f, np.float32), "grad_deg": np.zeros(n_nodes, np.float32), "stride": f,
          "n_edge": n_edge}
    want_f = run_op(oracle, "scatter_gcn_deg_scaled", fw, ["dst"])["dst"]
    want_b = run_op(oracle, "scatter_gcn_deg_scaled_bwd", bw, ["grad_h", "grad_deg"])
    ps, pt = _pinned(hip, src), _pinned(hip, tgt)
    hb, db, gb = hip.from_numpy(h), hip.from_numpy(deg), hip.from_numpy(go)
    for attempt in range(3):  # computed, then found twice
        out = hip.from_numpy(np.zeros(n_nodes * f, np.float32))
        hip.dispatch("scatter_gcn_deg_scaled", dst=out, h=hb, deg=db, src_indices=ps, tgt_indices=pt, stride=f, n_edge=n_edge)
        gh = hip.from_numpy(np.zeros(n_nodes * f, np.float32))
        gd = hip.from_numpy(np.zeros(n_nodes, np.float32))
        hip.dispatch("scatter_gcn_deg_scaled_bwd", grad_output=gb, h=hb, deg=db, src_indices=ps, tgt_indices=pt, grad_h=gh,
                     grad_deg=gd, stride=f, n_edge=n_edge)
        hip.sync()
        np.testing.assert_array_equal(hip.to_numpy(out), want_f)
        np.testing.assert_array_equal(hip.to_numpy(gh), want_b["grad_h"])
        np.testing.assert_array_equal(hip.to_numpy(gd), want_b["grad_deg"])
        for b in (out, gh, gd):
            hip.mem_free(b)
    # index_select backward through the same mechanism
    rows, stride, n_idx = 90, 6, 4000
    idx = r.integers(0, rows, n_idx).astype(np.uint64)
    yg = r.standard_normal(n_idx * stride).astype(np.float32)
    xg0 = r.standard_normal(rows * stride).astype(np.float32)
    want = run_op(oracle, "index_select_bwd", {"y_grad": yg, "indices": idx, "stride": stride, "x_grad": xg0.copy()},
                  ["x_grad"])["x_grad"]
    pi, yb = _pinned(hip, idx), hip.from_numpy(yg)
    for attempt in range(2):
        xb = hip.from_numpy(xg0)
        hip.dispatch("index_select_bwd", y_grad=yb, indices=pi, stride=stride, x_grad=xb)
        hip.sync()
        np.testing.assert_array_equal(hip.to_numpy(xb), want)
        hip.mem_free(xb)
    for b in (ps, pt, hb, db, gb, pi, yb):
        hip.mem_free(b)


def test_a_recorded_step_refuses_to_replay_over_a_rewritten_index_array(oracle, hip):
    r = np.random.default_rng(3)
    n, n_dst = 3000, 128
    off = r.integers(0, n_dst, n).astype(np.uint64)
    src = r.standard_normal(n).astype(np.float32)
    a = _pinned(hip, off)
    s = hip.from_numpy(src)
    d = hip.mem_alloc(F32, n_dst)
    zero = np.zeros(n_dst, np.float32)
    hip.mem_transfer(zero, d, "HtoD")
    hip.dispatch("scatter_add", src=s, offsets=a, dst=d)  # eager first: the ordering is computed and kept
    hip.sync()
    want = run_op(oracle, "scatter_add", {"src": src, "offsets": off, "dst": zero.copy()}, ["dst"])["dst"]
    hip.graph_open()
    hip.dispatch("scatter_add", src=s, offsets=a, dst=d)
    g = hip.graph_save()
    for _ in range(2):
        hip.mem_transfer(zero, d, "HtoD")
        g.run()
        hip.sync()
        np.testing.assert_array_equal(hip.to_numpy(d), want)
    view = hip.host_view(a)
    view[7] = (view[7] + 1) % n_dst
    with pytest.raises(ZgHipError):
        g.run()
    view[7] = off[7]
    hip.mem_transfer(zero, d, "HtoD")
    g.run()
    hip.sync()
    np.testing.assert_array_equal(hip.to_numpy(d), want)
    g.free()
    for b in (a, s, d):
        hip.mem_free(b)


def test_long_pinned_index_arrays_are_analysed_every_call(oracle, hip):
    """Beyond 65536 entries the host comparison would cost more than the analysis: nothing is kept, results as ever."""
    r = np.random.default_rng(5)
    n, n_dst = 70_000, 900
    off = r.integers(0, n_dst, n).astype(np.uint64)
    src = r.standard_normal(n).astype(np.float32)
    dst0 = np.zeros(n_dst, np.float32)
    want = run_op(oracle, "scatter_add", {"src": src, "offsets": off, "dst": dst0.copy()}, ["dst"])["dst"]
    a = _pinned(hip, off)
    before = hip.plan_cache_stats()
    for _ in range(2):
        np.testing.assert_array_equal(_scatter(hip, src, a, dst0), want)
    assert hip.plan_cache_stats() == before
    hip.mem_free(a)
