"""Destination orderings of long index arrays (262144 entries and more), kept under the arrays' addresses and checked
against the arrays on the GPU by every call: whoever rewrites an array, and however, the next call must give what the
host's sequential loop gives on the new contents (src/device/host_device.zig:1039-1087, :1356-1403), and a call on
unchanged arrays must not build the ordering again.  Arrays in device memory and in pinned host memory alike."""
from __future__ import annotations

import numpy as np
import pytest

from conftest import run_op
from zigrad_amd.device import F32, U64

pytestmark = pytest.mark.gpu

N = 300_000


def _index_buffer(hip, arr, where):
    if where == "pinned":
        buf = hip.mem_alloc_host(U64, arr.size)
        hip.host_view(buf)[:] = arr
        return buf
    return hip.from_numpy(arr)


def _rewrite(hip, buf, arr, where):
    hip.sync()
    if where == "pinned":
        hip.host_view(buf)[:] = arr
    else:
        hip.mem_transfer(arr, buf, "HtoD")


def _scatter(hip, s, off_buf, dst_np):
    d = hip.from_numpy(dst_np)
    hip.dispatch("scatter_add", src=s, offsets=off_buf, dst=d)
    hip.sync()
    out = hip.to_numpy(d)
    hip.mem_free(d)
    return out


def _tally(hip):
    st = hip.plan_cache_stats()
    return st["builds"], st["hits"]


@pytest.mark.parametrize("where", ["device", "pinned"])
def test_scatter_add_follows_an_array_rewritten_in_place(oracle, hip, where):
    r = np.random.default_rng(3)
    n_dst = 70_000   # 17 bits of destination: two 9-bit passes
    off = r.integers(0, n_dst, N).astype(np.uint64)
    src = r.standard_normal(N).astype(np.float32)
    dst0 = r.standard_normal(n_dst).astype(np.float32)

    def want(o):
        keep = o < n_dst    # an offset outside the destination is skipped here (the host loop would write out of bounds)
        return run_op(oracle, "scatter_add", {"src": src[keep], "offsets": o[keep], "dst": dst0.copy()}, ["dst"])["dst"]

    a = _index_buffer(hip, off, where)
    s = hip.from_numpy(src)
    builds0, hits0 = _tally(hip)
    np.testing.assert_array_equal(_scatter(hip, s, a, dst0), want(off))
    # built now, or found under this address from an earlier owner of the memory and rebuilt in place
    builds1, hits1 = _tally(hip)
    assert (builds1, hits1) in ((builds0 + 1, hits0), (builds0, hits0 + 1))
    for _ in range(2):      # unchanged: the kept ordering, checked on the GPU
        np.testing.assert_array_equal(_scatter(hip, s, a, dst0), want(off))
    assert _tally(hip) == (builds1, hits1 + 2)
    # one changed entry at either end and in the middle of a tile, one key that leaves the range, one that comes back
    for pos, val in ((0, 5), (N - 1, n_dst - 1), (4096 * 17 + 5, 0), (9, n_dst + 3), (9, 11)):
        off = off.copy()
        off[pos] = val if off[pos] != val else (val + 1) % n_dst
        _rewrite(hip, a, off, where)
        np.testing.assert_array_equal(_scatter(hip, s, a, dst0), want(off))
        np.testing.assert_array_equal(_scatter(hip, s, a, dst0), want(off))     # and the rebuilt ordering is kept
    # two keys outside the range are the same key to the ordering: nothing to rebuild, same sums
    off = off.copy()
    off[9] = n_dst + 100
    _rewrite(hip, a, off, where)
    np.testing.assert_array_equal(_scatter(hip, s, a, dst0), want(off))
    off[9] = n_dst + 7
    _rewrite(hip, a, off, where)
    np.testing.assert_array_equal(_scatter(hip, s, a, dst0), want(off))
    # all new contents
    off = r.integers(0, n_dst, N).astype(np.uint64)
    _rewrite(hip, a, off, where)
    np.testing.assert_array_equal(_scatter(hip, s, a, dst0), want(off))
    assert _tally(hip)[0] == builds1    # one allocation of plan memory through all of it
    hip.mem_free(a)
    hip.mem_free(s)


def test_gcn_scatter_follows_either_edge_array(oracle, hip):
    """The payload (the other endpoint of an edge) is compared as well: a change in the sources only must be seen by the
    forward pass, whose ordering is by target."""
    r = np.random.default_rng(4)
    n_nodes, f = 2000, 4
    tgt = r.integers(0, n_nodes, N).astype(np.uint64)
    src = r.integers(0, n_nodes, N).astype(np.uint64)
    h = r.standard_normal(n_nodes * f).astype(np.float32)
    deg = r.uniform(0.2, 1.0, n_nodes).astype(np.float32)
    go = r.standard_normal(n_nodes * f).astype(np.float32)
    sb, tb = hip.from_numpy(src), hip.from_numpy(tgt)
    hb, db, gb = hip.from_numpy(h), hip.from_numpy(deg), hip.from_numpy(go)

    def check(src_np, tgt_np):
        fw = {"dst": np.zeros(n_nodes * f, np.float32), "h": h, "deg": deg, "src_indices": src_np, "tgt_indices": tgt_np,
              "stride": f, "n_edge": N}
        want = run_op(oracle, "scatter_gcn_deg_scaled", fw, ["dst"])["dst"]
        out = hip.from_numpy(np.zeros(n_nodes * f, np.float32))
        hip.dispatch("scatter_gcn_deg_scaled", dst=out, h=hb, deg=db, src_indices=sb, tgt_indices=tb, stride=f, n_edge=N)
        hip.sync()
        np.testing.assert_array_equal(hip.to_numpy(out), want)
        hip.mem_free(out)
        bw = {"grad_output": go, "h": h, "deg": deg, "src_indices": src_np, "tgt_indices": tgt_np,
              "grad_h": np.zeros(n_nodes * f, np.float32), "grad_deg": np.zeros(n_nodes, np.float32), "stride": f, "n_edge": N}
        want = run_op(oracle, "scatter_gcn_deg_scaled_bwd", bw, ["grad_h", "grad_deg"])
        gh, gd = hip.from_numpy(bw["grad_h"]), hip.from_numpy(bw["grad_deg"])
        hip.dispatch("scatter_gcn_deg_scaled_bwd", grad_output=gb, h=hb, deg=db, src_indices=sb, tgt_indices=tb, grad_h=gh,
                     grad_deg=gd, stride=f, n_edge=N)
        hip.sync()
        np.testing.assert_array_equal(hip.to_numpy(gh), want["grad_h"])
        np.testing.assert_array_equal(hip.to_numpy(gd), want["grad_deg"])
        hip.mem_free(gh)
        hip.mem_free(gd)

    check(src, tgt)
    builds = _tally(hip)[0]
    check(src, tgt)
    src = src.copy()
    src[12345] = (src[12345] + 1) % n_nodes
    _rewrite(hip, sb, src, "device")
    check(src, tgt)
    tgt = tgt.copy()
    tgt[N - 2] = (tgt[N - 2] + 7) % n_nodes
    _rewrite(hip, tb, tgt, "device")
    check(src, tgt)
    check(src, tgt)
    assert _tally(hip)[0] == builds
    for b in (sb, tb, hb, db, gb):
        hip.mem_free(b)


def test_a_recorded_scatter_follows_the_array_between_replays(oracle, hip):
    r = np.random.default_rng(6)
    n_dst = 200     # one pass
    off = r.integers(0, n_dst, N).astype(np.uint64)
    src = r.standard_normal(N).astype(np.float32)
    zero = np.zeros(n_dst, np.float32)

    def want(o):
        return run_op(oracle, "scatter_add", {"src": src, "offsets": o, "dst": zero.copy()}, ["dst"])["dst"]

    a, s, d = hip.from_numpy(off), hip.from_numpy(src), hip.from_numpy(zero)
    hip.dispatch("scatter_add", src=s, offsets=a, dst=d)    # eagerly once: the ordering is kept before the recording
    hip.sync()
    hip.mem_transfer(zero, d, "HtoD")
    hip.graph_open()
    try:
        hip.dispatch("scatter_add", src=s, offsets=a, dst=d)
    finally:
        g = hip.graph_save()
    for k in range(4):
        if k in (1, 3):
            off = off.copy()
            off[1000 * k: 1000 * k + 50] = (off[1000 * k: 1000 * k + 50] + 1) % n_dst
            _rewrite(hip, a, off, "device")
        hip.mem_transfer(zero, d, "HtoD")
        g.run()
        hip.sync()
        np.testing.assert_array_equal(hip.to_numpy(d), want(off))
        # eager work between the replays, on the same kept ordering
        hip.mem_transfer(zero, d, "HtoD")
        hip.dispatch("scatter_add", src=s, offsets=a, dst=d)
        hip.sync()
        np.testing.assert_array_equal(hip.to_numpy(d), want(off))
    g.free()
    for b in (a, s, d):
        hip.mem_free(b)


def test_arrays_that_change_every_call_are_given_up(oracle, hip):
    r = np.random.default_rng(7)
    n_dst = 5000
    src = r.standard_normal(N).astype(np.float32)
    dst0 = np.zeros(n_dst, np.float32)
    off = r.integers(0, n_dst, N).astype(np.uint64)
    a, s = hip.from_numpy(off), hip.from_numpy(src)
    hits_at = []
    for k in range(14):
        off = np.roll(off, 1)
        _rewrite(hip, a, off, "device")
        want = run_op(oracle, "scatter_add", {"src": src, "offsets": off, "dst": dst0.copy()}, ["dst"])["dst"]
        np.testing.assert_array_equal(_scatter(hip, s, a, dst0), want)
        hits_at.append(_tally(hip)[1])
    assert hits_at[-1] == hits_at[-2] == hits_at[-3]    # no longer looked up: analysed in the workspace like any new array
    assert hits_at[5] > hits_at[0]                      # but it was, to begin with
    hip.mem_free(a)
    hip.mem_free(s)
