"""Seeded random sweeps over shapes, transposes, leading dimensions and scalars.  Every GEMM path (tiny, split-k,
fast / edge / checked kernels of each tile size), the broadcasting regimes and the axis reductions are hit many
times with sizes nobody picked by hand; results are compared with float64 numpy."""
from __future__ import annotations

import numpy as np
import pytest

from conftest import rel_fro
from zigrad_amd.device import F32

pytestmark = pytest.mark.gpu
TOL = 1e-5


def _dim(r, hi):
    """Sizes biased towards tile edges: multiples of 32/64/128 and their neighbours as well as arbitrary values."""
    kind = r.integers(0, 4)
    if kind == 0:
        return int(r.integers(1, hi + 1))
    base = int(r.choice([32, 64, 128, 256])) * int(r.integers(1, max(2, hi // 256 + 1)))
    return max(1, min(hi, base + int(r.choice([-1, 0, 0, 1, 4]))))


@pytest.mark.parametrize("seed", range(16))
def test_matmul_random_cases(hip, seed):
    r = np.random.default_rng(1000 + seed)
    for case in range(30):
        m, n, k = _dim(r, 700), _dim(r, 700), _dim(r, 1500)
        ta, tb = bool(r.integers(0, 2)), bool(r.integers(0, 2))
        pa, pb, pc = (int(r.choice([0, 0, 4, 3])) for _ in range(3))
        lda, ldb, ldc = (m if ta else k) + pa, (k if tb else n) + pb, n + pc
        alpha = float(r.choice([1.0, 0.5, -1.25]))
        beta = float(r.choice([0.0, 1.0, -0.5]))
        A = np.full((k if ta else m, lda), np.nan, np.float32)
        B = np.full((n if tb else k, ldb), np.nan, np.float32)
        C0 = np.full((m, ldc), np.nan, np.float32)
        A[:, : (m if ta else k)] = r.standard_normal((A.shape[0], m if ta else k))
        B[:, : (k if tb else n)] = r.standard_normal((B.shape[0], k if tb else n))
        if beta != 0.0:
            C0[:, :n] = r.standard_normal((m, n))
        a, b, c = hip.from_numpy(A), hip.from_numpy(B), hip.from_numpy(C0)
        hip.dispatch("matmul", A=a, B=b, C=c, m=m, n=n, k=k, trans_a=ta, trans_b=tb, lda=lda, ldb=ldb, ldc=ldc,
                     alpha=alpha, beta=beta)
        got = hip.to_numpy(c).reshape(m, ldc)
        for x in (a, b, c):
            hip.mem_free(x)
        A64 = A[:, : (m if ta else k)].astype(np.float64)
        B64 = B[:, : (k if tb else n)].astype(np.float64)
        want = alpha * ((A64.T if ta else A64) @ (B64.T if tb else B64))
        if beta != 0.0:
            want = want + beta * C0[:, :n].astype(np.float64)
        what = (seed, case, m, n, k, ta, tb, lda, ldb, ldc, alpha, beta)
        assert not np.isnan(got[:, :n]).any(), what
        scale = np.linalg.norm(want) + np.sqrt(m * n) * 1e-3  # products that cancel to nearly nothing stay meaningful
        assert np.linalg.norm(got[:, :n] - want) <= TOL * scale, what
        if pc:
            assert np.isnan(got[:, n:]).all(), what  # padding of C untouched


@pytest.mark.parametrize("seed", range(4))
def test_bmm_random_cases(hip, seed):
    r = np.random.default_rng(2000 + seed)
    for case in range(10):
        nbc = int(r.integers(1, 7))
        nba, nbb = (int(r.choice([1, nbc])) for _ in range(2))
        m, n, k = _dim(r, 200), _dim(r, 200), _dim(r, 600)
        ta, tb = bool(r.integers(0, 2)), bool(r.integers(0, 2))
        A = r.standard_normal((nba, k, m) if ta else (nba, m, k)).astype(np.float32)
        B = r.standard_normal((nbb, n, k) if tb else (nbb, k, n)).astype(np.float32)
        C0 = r.standard_normal((nbc, m, n)).astype(np.float32)
        a, b, c = hip.from_numpy(A), hip.from_numpy(B), hip.from_numpy(C0)
        hip.dispatch("bmm_acc", A=a, B=b, C=c, A_shape=[nba, m, k], B_shape=[nbb, k, n], C_shape=[nbc, m, n], trans_a=ta,
                     trans_b=tb, lda=A.shape[2], ldb=B.shape[2], ldc=n, alpha=1.0, beta=1.0)
        got = hip.to_numpy(c).reshape(nbc, m, n)
        for x in (a, b, c):
            hip.mem_free(x)
        want = np.stack([(A[i % nba].astype(np.float64).T if ta else A[i % nba].astype(np.float64))
                         @ (B[i % nbb].astype(np.float64).T if tb else B[i % nbb].astype(np.float64)) for i in range(nbc)]) + C0
        assert rel_fro(got, want) <= TOL, (seed, case, nbc, nba, nbb, m, n, k, ta, tb)


@pytest.mark.parametrize("seed", range(4))
def test_axis_reductions_random_shapes(hip, seed):
    r = np.random.default_rng(3000 + seed)
    for case in range(15):
        rank = int(r.integers(1, 5))
        shape = [int(r.integers(1, 40)) for _ in range(rank)]
        if r.integers(0, 3) == 0:
            shape[int(r.integers(0, rank))] = int(r.integers(200, 3000))
        dim = int(r.integers(0, rank))
        X = r.standard_normal(shape).astype(np.float32)
        n_out = X.size // shape[dim]
        x = hip.from_numpy(X)
        y = hip.mem_alloc(F32, n_out)
        hip.mem_fill(y, 2.0)
        alpha, beta = float(r.choice([1.0, 0.5])), float(r.choice([0.0, 1.0]))
        hip.dispatch("sum_along", x=x, x_shape=shape, y=y, dim=dim, alpha=alpha, beta=beta)
        want = alpha * X.astype(np.float64).sum(axis=dim).ravel() + beta * 2.0
        assert np.linalg.norm(hip.to_numpy(y) - want) <= TOL * (np.linalg.norm(want) + 1e-3), (seed, case, shape, dim)
        hip.mem_fill(y, 0.0)
        hip.dispatch("max_along", x=x, x_shape=shape, y=y, dim=dim)
        assert np.array_equal(hip.to_numpy(y), X.max(axis=dim).ravel()), (seed, case, shape, dim)
        idx = hip.mem_alloc(np.uint64, n_out)
        hip.dispatch("argmax_along", x=x, x_shape=shape, y=idx, dim=dim)
        assert np.array_equal(hip.to_numpy(idx), X.argmax(axis=dim).ravel().astype(np.uint64)), (seed, case, shape, dim)
        for b in (x, y, idx):
            hip.mem_free(b)


@pytest.mark.parametrize("seed", range(4))
def test_elementwise_broadcast_random_lengths(hip, seed):
    """z = x op y with the shorter operand restarting every min(len) elements (src/device/host_device.zig:975-1019)."""
    r = np.random.default_rng(4000 + seed)
    ops = {"add": np.add, "sub": np.subtract, "mul": np.multiply, "div": np.divide}
    for case in range(25):
        short = int(r.choice([1, 3, 4, 7, 64, 100, 128, 1000, 4096]))
        reps = int(r.integers(1, 60))
        long_n = short * reps
        name = str(r.choice(list(ops)))
        swap = bool(r.integers(0, 2))
        S = (r.standard_normal(short) + 3.0).astype(np.float32)
        L = (r.standard_normal(long_n) + 3.0).astype(np.float32)
        X, Y = (S, L) if swap else (L, S)
        x, y, z = hip.from_numpy(X), hip.from_numpy(Y), hip.mem_alloc(F32, long_n)
        hip.dispatch(name, x=x, y=y, z=z)
        want = ops[name](np.resize(X, long_n), np.resize(Y, long_n))  # one IEEE operation per element: exact
        assert np.array_equal(hip.to_numpy(z), want), (seed, case, name, short, reps, swap)
        for b in (x, y, z):
            hip.mem_free(b)


@pytest.mark.parametrize("seed", range(4))
def test_scatter_ops_random_graphs_bit_exact(oracle, hip, seed):
    """Random edge lists with isolated nodes, hubs and strides that are not powers of two: scatter_add, the GCN
    scatter and its backward, index_select backward -- bit for bit against the sequential host loops."""
    from conftest import run_op

    r = np.random.default_rng(5000 + seed)
    for case in range(6):
        n_nodes = int(r.integers(1, 4000))
        n_edge = int(r.integers(0, 6000))
        stride = int(r.choice([1, 3, 7, 16, 20, 33, 64]))
        hub = int(r.integers(0, n_nodes))
        src = r.integers(0, n_nodes, n_edge).astype(np.uint64)
        tgt = np.where(r.random(n_edge) < 0.2, hub, r.integers(0, n_nodes, n_edge)).astype(np.uint64)
        what = (seed, case, n_nodes, n_edge, stride)
        if n_edge:
            vals = r.standard_normal(n_edge).astype(np.float32)
            d0 = r.standard_normal(n_nodes).astype(np.float32)
            p = {"src": vals, "offsets": tgt, "dst": d0}
            assert np.array_equal(run_op(oracle, "scatter_add", dict(p), ["dst"])["dst"], run_op(hip, "scatter_add", dict(p), ["dst"])["dst"]), what
        h = r.standard_normal(n_nodes * stride).astype(np.float32)
        deg = (r.random(n_nodes) + 0.25).astype(np.float32)
        p = {"dst": r.standard_normal(n_nodes * stride).astype(np.float32), "h": h, "deg": deg, "src_indices": src,
             "tgt_indices": tgt, "stride": stride, "n_edge": n_edge}
        assert np.array_equal(run_op(oracle, "scatter_gcn_deg_scaled", dict(p), ["dst"])["dst"],
                              run_op(hip, "scatter_gcn_deg_scaled", dict(p), ["dst"])["dst"]), what
        p = {"grad_output": r.standard_normal(n_nodes * stride).astype(np.float32), "h": h, "deg": deg, "src_indices": src,
             "tgt_indices": tgt, "grad_h": r.standard_normal(n_nodes * stride).astype(np.float32),
             "grad_deg": r.standard_normal(n_nodes).astype(np.float32), "stride": stride, "n_edge": n_edge}
        a = run_op(oracle, "scatter_gcn_deg_scaled_bwd", dict(p), ["grad_h", "grad_deg"])
        b = run_op(hip, "scatter_gcn_deg_scaled_bwd", dict(p), ["grad_h", "grad_deg"])
        assert np.array_equal(a["grad_h"], b["grad_h"]) and np.array_equal(a["grad_deg"], b["grad_deg"]), what
        n_idx = int(r.integers(1, 3000))
        idx = r.integers(0, n_nodes, n_idx).astype(np.uint64)
        p = {"y_grad": r.standard_normal(n_idx * stride).astype(np.float32), "indices": idx, "stride": stride,
             "x_grad": r.standard_normal(n_nodes * stride).astype(np.float32)}
        assert np.array_equal(run_op(oracle, "index_select_bwd", dict(p), ["x_grad"])["x_grad"],
                              run_op(hip, "index_select_bwd", dict(p), ["x_grad"])["x_grad"]), what


@pytest.mark.parametrize("n_nodes,n_edge", [(8191, 16384), (8192, 16384), (8191, 16385), (1, 16384), (300, 16000),
                                            (20000, 40000), (5, 40000)])
def test_scatter_ops_large_and_skewed_bit_exact(oracle, hip, n_nodes, n_edge):
    """Edge lists around powers of two, a single destination, a few very long segments (30 % of all edges on one
    node) and sizes that need the multi-tile scan: bit for bit against the sequential host loops."""
    from conftest import run_op

    r = np.random.default_rng(n_nodes * 7 + n_edge)
    stride = 5
    src = r.integers(0, n_nodes, n_edge).astype(np.uint64)
    tgt = np.where(r.random(n_edge) < 0.3, n_nodes // 2, r.integers(0, n_nodes, n_edge)).astype(np.uint64)
    p = {"src": r.standard_normal(n_edge).astype(np.float32), "offsets": tgt, "dst": r.standard_normal(n_nodes).astype(np.float32)}
    assert np.array_equal(run_op(oracle, "scatter_add", dict(p), ["dst"])["dst"], run_op(hip, "scatter_add", dict(p), ["dst"])["dst"])
    h = r.standard_normal(n_nodes * stride).astype(np.float32)
    deg = (r.random(n_nodes) + 0.25).astype(np.float32)
    p = {"grad_output": r.standard_normal(n_nodes * stride).astype(np.float32), "h": h, "deg": deg, "src_indices": src,
         "tgt_indices": tgt, "grad_h": r.standard_normal(n_nodes * stride).astype(np.float32),
         "grad_deg": r.standard_normal(n_nodes).astype(np.float32), "stride": stride, "n_edge": n_edge}
    a = run_op(oracle, "scatter_gcn_deg_scaled_bwd", dict(p), ["grad_h", "grad_deg"])
    b = run_op(hip, "scatter_gcn_deg_scaled_bwd", dict(p), ["grad_h", "grad_deg"])
    assert np.array_equal(a["grad_h"], b["grad_h"]) and np.array_equal(a["grad_deg"], b["grad_deg"])
    p = {"dst": r.standard_normal(n_nodes * stride).astype(np.float32), "h": h, "deg": deg, "src_indices": src,
         "tgt_indices": tgt, "stride": stride, "n_edge": n_edge}
    assert np.array_equal(run_op(oracle, "scatter_gcn_deg_scaled", dict(p), ["dst"])["dst"],
                          run_op(hip, "scatter_gcn_deg_scaled", dict(p), ["dst"])["dst"])


@pytest.mark.parametrize("n_nodes,n_edge,where", [(2708, 13264, "host"), (2708, 13264, "device"), (1, 50, "device"),
                                                  (300, 16000, "host"), (20000, 40000, "device"), (977, 3, "host")])
def test_planned_scatter_ops_equal_the_unplanned_ones(oracle, hip, n_nodes, n_edge, where):
    """An edge plan built once from index arrays in pinned host or device memory, used twice: scatter_add,
    scatter_gcn_deg_scaled and its backward return exactly what the ops that take the bare index arrays return
    (and what the sequential host loops return)."""
    from conftest import run_op
    from zigrad_amd.device import F32, U64

    r = np.random.default_rng(n_nodes + 3 * n_edge)
    src = r.integers(0, n_nodes, n_edge).astype(np.uint64)
    tgt = np.where(r.random(n_edge) < 0.2, n_nodes // 3, r.integers(0, n_nodes, n_edge)).astype(np.uint64)
    if where == "host":
        s_buf, t_buf = hip.mem_alloc_host(U64, n_edge), hip.mem_alloc_host(U64, n_edge)
    else:
        s_buf, t_buf = hip.mem_alloc(U64, n_edge), hip.mem_alloc(U64, n_edge)
    hip.mem_transfer(src, s_buf, "HtoD")
    hip.mem_transfer(tgt, t_buf, "HtoD")
    plan = hip.edge_plan(s_buf, t_buf, n_nodes)
    hip.mem_transfer(np.zeros(n_edge, np.uint64), s_buf, "HtoD")  # the plan keeps its own copy of the indices
    for rep, stride in enumerate((5, 16, 40)):  # 40: rows of more than 64 bytes reach the degree-gradient terms through LDS
        vals = r.standard_normal(n_edge).astype(np.float32)
        d0 = r.standard_normal(n_nodes).astype(np.float32)
        got = run_op(hip, "scatter_add_planned", {"src": vals, "plan": plan, "dst": d0.copy()}, ["dst"])["dst"]
        want = run_op(oracle, "scatter_add", {"src": vals, "offsets": tgt, "dst": d0.copy()}, ["dst"])["dst"]
        assert np.array_equal(got, want), (rep, "scatter_add")
        h = r.standard_normal(n_nodes * stride).astype(np.float32)
        deg = (r.random(n_nodes) + 0.25).astype(np.float32)
        y0 = r.standard_normal(n_nodes * stride).astype(np.float32)
        got = run_op(hip, "scatter_gcn_deg_scaled_planned", {"dst": y0.copy(), "h": h, "deg": deg, "plan": plan,
                                                              "stride": stride}, ["dst"])["dst"]
        want = run_op(oracle, "scatter_gcn_deg_scaled", {"dst": y0.copy(), "h": h, "deg": deg, "src_indices": src,
                                                         "tgt_indices": tgt, "stride": stride, "n_edge": n_edge}, ["dst"])["dst"]
        assert np.array_equal(got, want), (rep, "fwd")
        go = r.standard_normal(n_nodes * stride).astype(np.float32)
        gh0, gd0 = r.standard_normal(n_nodes * stride).astype(np.float32), r.standard_normal(n_nodes).astype(np.float32)
        got = run_op(hip, "scatter_gcn_deg_scaled_bwd_planned", {"grad_output": go, "h": h, "deg": deg, "plan": plan,
                                                                  "grad_h": gh0.copy(), "grad_deg": gd0.copy(),
                                                                  "stride": stride}, ["grad_h", "grad_deg"])
        want = run_op(oracle, "scatter_gcn_deg_scaled_bwd", {"grad_output": go, "h": h, "deg": deg, "src_indices": src,
                                                             "tgt_indices": tgt, "grad_h": gh0.copy(), "grad_deg": gd0.copy(),
                                                             "stride": stride, "n_edge": n_edge}, ["grad_h", "grad_deg"])
        assert np.array_equal(got["grad_h"], want["grad_h"]) and np.array_equal(got["grad_deg"], want["grad_deg"]), rep
        # written instead of accumulated: outputs start as NaN and must come out as if they had started as zeros
        # (every element, also where no edge arrives); the degree gradient may be left out
        nan_n, nan_ns = np.full(n_nodes, np.nan, np.float32), np.full(n_nodes * stride, np.nan, np.float32)
        got = run_op(hip, "scatter_add_planned", {"src": vals, "plan": plan, "dst": nan_n.copy(), "accumulate": False}, ["dst"])["dst"]
        want = run_op(oracle, "scatter_add", {"src": vals, "offsets": tgt, "dst": np.zeros(n_nodes, np.float32)}, ["dst"])["dst"]
        assert np.array_equal(got, want), (rep, "scatter_add fresh")
        got = run_op(hip, "scatter_gcn_deg_scaled_planned", {"dst": nan_ns.copy(), "h": h, "deg": deg, "plan": plan,
                                                              "stride": stride, "accumulate": False}, ["dst"])["dst"]
        want = run_op(oracle, "scatter_gcn_deg_scaled", {"dst": np.zeros(n_nodes * stride, np.float32), "h": h, "deg": deg,
                                                         "src_indices": src, "tgt_indices": tgt, "stride": stride,
                                                         "n_edge": n_edge}, ["dst"])["dst"]
        assert np.array_equal(got, want), (rep, "fwd fresh")
        # the layer's tail in the same launch: + bias per column, then relu (isolated nodes get relu(bias))
        bias = r.standard_normal(stride).astype(np.float32)
        for relu in (False, True):
            got = run_op(hip, "scatter_gcn_deg_scaled_planned", {"dst": nan_ns.copy(), "h": h, "deg": deg, "plan": plan,
                                                                  "stride": stride, "accumulate": False, "bias": bias,
                                                                  "relu": relu}, ["dst"])["dst"]
            tail = want.reshape(n_nodes, stride) + bias[None, :]
            tail = np.where(tail > 0, tail, np.float32(0)) if relu else tail
            assert np.array_equal(got, tail.ravel()), (rep, "fwd tail", relu)
            ref = run_op(oracle, "scatter_gcn_deg_scaled_planned", {"dst": nan_ns.copy(), "h": h, "deg": deg,
                                                                    "plan": oracle.edge_plan(oracle.from_numpy(src), oracle.from_numpy(tgt), n_nodes),
                                                                    "stride": stride, "accumulate": False, "bias": bias,
                                                                    "relu": relu}, ["dst"])["dst"]
            assert np.array_equal(got, ref), (rep, "fwd tail against the oracle's three ops", relu)
        want = run_op(oracle, "scatter_gcn_deg_scaled_bwd", {"grad_output": go, "h": h, "deg": deg, "src_indices": src,
                                                             "tgt_indices": tgt, "grad_h": np.zeros(n_nodes * stride, np.float32),
                                                             "grad_deg": np.zeros(n_nodes, np.float32), "stride": stride,
                                                             "n_edge": n_edge}, ["grad_h", "grad_deg"])
        got = run_op(hip, "scatter_gcn_deg_scaled_bwd_planned", {"grad_output": go, "h": h, "deg": deg, "plan": plan,
                                                                  "grad_h": nan_ns.copy(), "grad_deg": nan_n.copy(),
                                                                  "stride": stride, "accumulate": False}, ["grad_h", "grad_deg"])
        assert np.array_equal(got["grad_h"], want["grad_h"]) and np.array_equal(got["grad_deg"], want["grad_deg"]), rep
        got = run_op(hip, "scatter_gcn_deg_scaled_bwd_planned", {"grad_output": go, "h": h, "deg": deg, "plan": plan,
                                                                  "grad_h": nan_ns.copy(), "grad_deg": None, "stride": stride,
                                                                  "accumulate": False}, ["grad_h"])
        assert np.array_equal(got["grad_h"], want["grad_h"]), (rep, "no degree gradient")
    plan.free()
    hip.mem_free(s_buf)
    hip.mem_free(t_buf)
