"""Scatter ops on skewed index sets: one destination that receives a hundred thousand contributions, buckets on
both sides of the limits the plan uses (256 entries: a wave instead of a thread adds them; 1024: the bucket is put
back into input order by a pass over the input instead of all-pairs ranking), through the short build and through
the radix build (262144 entries and more, or 64 entries and more per destination).  The sums must still equal the host's
sequential loop bit for bit (src/device/host_device.zig:1039-1087, :1356-1403; src/ndtensor.zig:1437-1513)."""
from __future__ import annotations

import numpy as np
import pytest

from conftest import run_op

pytestmark = pytest.mark.gpu


def _skewed_offsets(r, n, n_dst, hubs):
    """`hubs` = [(destination, entries)]; the remaining entries are spread uniformly; everything shuffled."""
    parts = [np.full(cnt, d, np.uint64) for d, cnt in hubs]
    rest = n - sum(cnt for _, cnt in hubs)
    parts.append(r.integers(0, n_dst, rest).astype(np.uint64))
    off = np.concatenate(parts)
    r.shuffle(off)
    return off


@pytest.mark.parametrize("n,n_dst,hubs", [
    (200_000, 1000, [(3, 100_000)]),                                   # the single huge bucket
    (60_000, 50, [(0, 257), (1, 256), (2, 1024), (3, 1025), (49, 20_000)]),  # either side of both limits
    (5_000, 3, []),                                                    # every bucket long, none huge
    (300_000, 200_000, [(199_999, 3000), (7, 1500)]),                  # mostly tiny buckets, two long ones
    (400_000, 1000, [(3, 200_000)]),                                   # the same through the radix build (>= 262144 entries)
    (300_000, 50, [(0, 257), (1, 256), (2, 1024), (3, 1025), (49, 100_000)]),
    (270_000, 3, []),
    # few destinations for the entries (64 and more each on average): the radix build from 512 entries on
    (600, 3, []), (1000, 1, []), (4097, 17, [(16, 3000)]), (512, 8, []), (511, 7, []),
    # hubs among many destinations below 262144 entries: the short build with its long buckets
    (200_000, 4000, [(3, 100_000)]),
    (60_000, 1000, [(0, 257), (1, 256), (2, 1024), (3, 1025), (999, 20_000)]),
    (130_000, 100_000, [(99_999, 3000), (7, 1500)]),
])
def test_scatter_add_with_hub_destinations_equals_the_host_loop(oracle, hip, n, n_dst, hubs):
    r = np.random.default_rng(n + n_dst)
    off = _skewed_offsets(r, n, n_dst, hubs)
    src = r.standard_normal(n).astype(np.float32)
    dst0 = r.standard_normal(n_dst).astype(np.float32)
    p = {"src": src, "offsets": off, "dst": dst0.copy()}
    want = run_op(oracle, "scatter_add", p, ["dst"])["dst"]
    got = run_op(hip, "scatter_add", {**p, "dst": dst0.copy()}, ["dst"])["dst"]
    np.testing.assert_array_equal(got, want)


def test_planned_scatter_add_with_a_hub_equals_the_host_loop(oracle, hip):
    r = np.random.default_rng(9)
    n, n_nodes = 50_000, 300
    tgt = _skewed_offsets(r, n, n_nodes, [(5, 30_000), (6, 600)])
    srcs = r.integers(0, n_nodes, n).astype(np.uint64)
    vals = r.standard_normal(n).astype(np.float32)
    want = run_op(oracle, "scatter_add", {"src": vals, "offsets": tgt, "dst": np.zeros(n_nodes, np.float32)}, ["dst"])["dst"]
    s, t = hip.from_numpy(srcs), hip.from_numpy(tgt)
    plan = hip.edge_plan(s, t, n_nodes)
    v, d = hip.from_numpy(vals), hip.from_numpy(np.full(n_nodes, np.nan, np.float32))
    hip.dispatch("scatter_add_planned", src=v, plan=plan, dst=d, accumulate=False)
    hip.sync()
    np.testing.assert_array_equal(hip.to_numpy(d), want)
    plan.free()
    for b in (s, t, v, d):
        hip.mem_free(b)


def test_index_select_bwd_and_gcn_with_a_hub_equal_the_host_loops(oracle, hip):
    r = np.random.default_rng(10)
    # index_select backward: 40000 selected rows, 25000 of them row 2
    rows, stride, n_idx = 64, 5, 40_000
    indices = _skewed_offsets(r, n_idx, rows, [(2, 25_000)])
    p = {"y_grad": r.standard_normal(n_idx * stride).astype(np.float32), "indices": indices, "stride": stride,
         "x_grad": r.standard_normal(rows * stride).astype(np.float32)}
    want = run_op(oracle, "index_select_bwd", {**p, "x_grad": p["x_grad"].copy()}, ["x_grad"])["x_grad"]
    got = run_op(hip, "index_select_bwd", {**p, "x_grad": p["x_grad"].copy()}, ["x_grad"])["x_grad"]
    np.testing.assert_array_equal(got, want)
    # graph convolution scatter, forward and backward, with a node of in-degree 6000 and one of out-degree 3000
    n_nodes, n_edge, f = 500, 30_000, 7
    tgt = _skewed_offsets(r, n_edge, n_nodes, [(11, 6000)])
    src = _skewed_offsets(r, n_edge, n_nodes, [(12, 3000)])
    h = r.standard_normal(n_nodes * f).astype(np.float32)
    deg = r.uniform(0.2, 1.0, n_nodes).astype(np.float32)
    fw = {"dst": np.zeros(n_nodes * f, np.float32), "h": h, "deg": deg, "src_indices": src, "tgt_indices": tgt,
          "stride": f, "n_edge": n_edge}
    want = run_op(oracle, "scatter_gcn_deg_scaled", fw, ["dst"])["dst"]
    got = run_op(hip, "scatter_gcn_deg_scaled", {**fw, "dst": np.zeros(n_nodes * f, np.float32)}, ["dst"])["dst"]
    np.testing.assert_array_equal(got, want)
    bw = {"grad_output": r.standard_normal(n_nodes * f).astype(np.float32), "h": h, "deg": deg, "src_indices": src,
          "tgt_indices": tgt, "grad_h": np.zeros(n_nodes * f, np.float32), "grad_deg": np.zeros(n_nodes, np.float32),
          "stride": f, "n_edge": n_edge}
    want = run_op(oracle, "scatter_gcn_deg_scaled_bwd", bw, ["grad_h", "grad_deg"])
    got = run_op(hip, "scatter_gcn_deg_scaled_bwd", {**bw, "grad_h": np.zeros(n_nodes * f, np.float32),
                                                     "grad_deg": np.zeros(n_nodes, np.float32)}, ["grad_h", "grad_deg"])
    np.testing.assert_array_equal(got["grad_h"], want["grad_h"])
    np.testing.assert_array_equal(got["grad_deg"], want["grad_deg"])


@pytest.mark.parametrize("rows,stride,n_idx,hubs", [
    (64, 1, 40_000, [(2, 25_000)]), (300, 16, 20_000, [(7, 257), (8, 256), (299, 9000)]), (5000, 70, 9_000, [(0, 3000)]),
    (30, 300, 9_000, []), (100_000, 3, 300_000, [(5, 100_000), (99_999, 300)]),
])
def test_index_select_bwd_of_rows_selected_many_times(oracle, hip, rows, stride, n_idx, hubs):
    """Rows that more than 256 entries select are added up by a wave per column (the entries' loads in flight 64 at a
    time), the others by a thread group per row; through the short and the radix build.  Bit for bit the host's loop
    (src/ndtensor.zig:1461-1465)."""
    r = np.random.default_rng(rows + stride + n_idx)
    indices = _skewed_offsets(r, n_idx, rows, hubs)
    p = {"y_grad": r.standard_normal(n_idx * stride).astype(np.float32), "indices": indices, "stride": stride,
         "x_grad": r.standard_normal(rows * stride).astype(np.float32)}
    want = run_op(oracle, "index_select_bwd", {**p, "x_grad": p["x_grad"].copy()}, ["x_grad"])["x_grad"]
    got = run_op(hip, "index_select_bwd", {**p, "x_grad": p["x_grad"].copy()}, ["x_grad"])["x_grad"]
    np.testing.assert_array_equal(got, want)


@pytest.mark.parametrize("n", [262143, 262144, 262145, 266241, 300000])
@pytest.mark.parametrize("n_dst", [1, 255, 256, 257, 511, 512, 65535, 65536, 262143, 262144, 1 << 20])
def test_scatter_add_either_side_of_the_radix_build_limits(oracle, hip, n, n_dst):
    """From 262144 entries on the destination ordering is built by a stable radix sort, 8 bits a pass, or 9 where that
    saves a pass: one pass of 8 (n_dst up to 255) or of 9 (up to 511), two of 8 (up to 65535) or of 9 (up to 262143),
    three beyond; tiles that end inside the input, the shortest input that takes this build and the longest that does
    not.  Equal to the host's sequential loop bit for bit."""
    r = np.random.default_rng(n * 31 + n_dst)
    off = r.integers(0, n_dst, n).astype(np.uint64)
    src = r.standard_normal(n).astype(np.float32)
    dst0 = r.standard_normal(n_dst).astype(np.float32)
    p = {"src": src, "offsets": off, "dst": dst0.copy()}
    want = run_op(oracle, "scatter_add", p, ["dst"])["dst"]
    got = run_op(hip, "scatter_add", {**p, "dst": dst0.copy()}, ["dst"])["dst"]
    np.testing.assert_array_equal(got, want)


def test_gcn_scatter_through_the_radix_build_equals_the_host_loops(oracle, hip):
    """An edge list long enough for the radix build (>= 262144 edges), with hubs: the payload (the other endpoint of an
    edge) travels with its entry, forward and backward, and the incidence ordering of the degree gradient (2 x edges)."""
    r = np.random.default_rng(12)
    n_nodes, n_edge, f = 3000, 280_000, 5
    tgt = _skewed_offsets(r, n_edge, n_nodes, [(11, 60_000), (5, 300)])
    src = _skewed_offsets(r, n_edge, n_nodes, [(12, 30_000)])
    h = r.standard_normal(n_nodes * f).astype(np.float32)
    deg = r.uniform(0.2, 1.0, n_nodes).astype(np.float32)
    fw = {"dst": np.zeros(n_nodes * f, np.float32), "h": h, "deg": deg, "src_indices": src, "tgt_indices": tgt,
          "stride": f, "n_edge": n_edge}
    want = run_op(oracle, "scatter_gcn_deg_scaled", fw, ["dst"])["dst"]
    got = run_op(hip, "scatter_gcn_deg_scaled", {**fw, "dst": np.zeros(n_nodes * f, np.float32)}, ["dst"])["dst"]
    np.testing.assert_array_equal(got, want)
    bw = {"grad_output": r.standard_normal(n_nodes * f).astype(np.float32), "h": h, "deg": deg, "src_indices": src,
          "tgt_indices": tgt, "grad_h": np.zeros(n_nodes * f, np.float32), "grad_deg": np.zeros(n_nodes, np.float32),
          "stride": f, "n_edge": n_edge}
    want = run_op(oracle, "scatter_gcn_deg_scaled_bwd", bw, ["grad_h", "grad_deg"])
    got = run_op(hip, "scatter_gcn_deg_scaled_bwd", {**bw, "grad_h": np.zeros(n_nodes * f, np.float32),
                                                     "grad_deg": np.zeros(n_nodes, np.float32)}, ["grad_h", "grad_deg"])
    np.testing.assert_array_equal(got["grad_h"], want["grad_h"])
    np.testing.assert_array_equal(got["grad_deg"], want["grad_deg"])
    # index_select backward through the same build
    rows, stride, n_idx = 64, 3, 270_000
    indices = _skewed_offsets(r, n_idx, rows, [(2, 100_000)])
    p = {"y_grad": r.standard_normal(n_idx * stride).astype(np.float32), "indices": indices, "stride": stride,
         "x_grad": r.standard_normal(rows * stride).astype(np.float32)}
    want = run_op(oracle, "index_select_bwd", {**p, "x_grad": p["x_grad"].copy()}, ["x_grad"])["x_grad"]
    got = run_op(hip, "index_select_bwd", {**p, "x_grad": p["x_grad"].copy()}, ["x_grad"])["x_grad"]
    np.testing.assert_array_equal(got, want)
