"""Random call sequences against the work that waits inside the context (fills, products, bias gradients, optimizer
steps, graph-convolution aggregations).  Whatever the order of calls and however their operands overlap, the memory a
caller can observe must be what the same calls leave behind when every one of them is launched on its own, which a
synchronisation after each call forces.  Seeded; every buffer is compared bit for bit at the end of a sequence and at
random points inside it."""
from __future__ import annotations

import numpy as np
import pytest

from zigrad_amd import host
from zigrad_amd.device import F32

pytestmark = pytest.mark.gpu

N_BUF = 10
BUF_LEN = 64 * 64   # every buffer can hold a 64 x 64 matrix
DIMS = [1, 7, 16, 32, 33, 64]


class _Run:
    def __init__(self, hip, seed, eager, reads=True):
        self.hip, self.eager, self.seed, self.with_reads = hip, eager, seed, reads
        self.r = np.random.default_rng(seed)             # the same stream of choices in both runs
        init = np.random.default_rng(seed + 10_000)
        self.bufs = [hip.from_numpy((init.standard_normal(BUF_LEN) * 0.1).astype(np.float32)) for _ in range(N_BUF)]
        # Adam's moments live in buffers of their own (the second moment must stay non-negative)
        self.moments = [(hip.from_numpy(np.zeros(BUF_LEN, np.float32)), hip.from_numpy(np.zeros(BUF_LEN, np.float32)))
                        for _ in range(3)]
        self.temps = []                                   # cache allocations that are alive
        n_nodes, n_edge = 40, 150
        self.graph = (n_nodes, n_edge)
        self.src = hip.from_numpy(init.integers(0, n_nodes, n_edge).astype(np.uint64))
        self.tgt = hip.from_numpy(init.integers(0, n_nodes, n_edge).astype(np.uint64))
        # scatter_add, one-launch and planned forms; in pinned host memory, where the library keeps the buckets it sorted
        # the offsets into from call to call (what lets a count of a constant wait with the elementwise ops)
        self.offs = hip.mem_alloc_host(np.uint64, 1000)
        hip.mem_transfer(init.integers(0, 300, 1000).astype(np.uint64), self.offs, "HtoD")
        # index arrays in device memory for the ops that take them: values below 64 (rows), sorted bounds for the CSR forms
        self.idx = hip.from_numpy(init.integers(0, 64, 256).astype(np.uint64))
        self.row_ptr = hip.from_numpy(np.arange(65, dtype=np.uint64))                      # 64 segments of one element
        self.seg_bounds = hip.from_numpy(np.concatenate([[0], np.sort(init.integers(0, 257, 61)), [256]]).astype(np.uint64))
        self.lr_slot = hip.mem_alloc(F32, 1)
        self.u64_out = hip.mem_alloc(np.uint64, 4096)
        self.plan = hip.edge_plan(self.src, self.tgt, n_nodes)
        self.long = None    # index arrays long enough for the orderings kept by address (made on first use)
        self.reads = []
        self.t = 0
        self.last_c = None

    def done(self):
        if self.eager:
            self.hip.sync()

    def picks(self, *sizes):
        """One view per size, each in a different buffer (or live temp), so the operands of one call never overlap;
        calls that follow each other meet on the same buffers all the time."""
        pool = list(self.bufs) + list(self.temps)
        order = self.r.permutation(len(pool))
        out, used = [], set()
        for n in sizes:
            for j in order:
                if int(j) not in used and pool[int(j)].n >= n:
                    used.add(int(j))
                    b = pool[int(j)]
                    off = int(self.r.integers(0, b.n - n + 1)) if self.r.random() < 0.3 else 0
                    off -= off % 4
                    out.append(b.sub(off, n))
                    break
            else:
                raise AssertionError("no buffer left")
        return out

    def pick(self, n):
        return self.picks(n)[0]

    # ---- the calls -------------------------------------------------------------------------------------------------
    def op_fill(self):
        n = int(self.r.choice([1, 10, 64, 1024, BUF_LEN]))
        v = float(self.r.choice([0.0, 0.0, 0.125, -0.0, 0.5]))
        self.hip.mem_fill(self.pick(n), v)

    def op_matmul(self):
        m, n, k = (int(self.r.choice(DIMS)) for _ in range(3))
        ta, tb = bool(self.r.integers(0, 2)), bool(self.r.integers(0, 2))
        beta = float(self.r.choice([0.0, 1.0, 1.0]))
        a, b, c = self.picks(m * k, k * n, m * n)
        if self.r.random() < 0.5:
            self.hip.mem_fill(c, 0.0)      # ensure_grad(0) before an accumulating product
            self.done()
        self.hip.dispatch("matmul", A=a, B=b, C=c, m=m, n=n, k=k, trans_a=ta, trans_b=tb, lda=(m if ta else k),
                          ldb=(k if tb else n), ldc=n, alpha=1.0, beta=beta)
        self.last_c = (c, m, n)

    def op_add_row(self):
        """A bias row onto the last product's output, or onto something else."""
        m, n = int(self.r.choice(DIMS)), int(self.r.choice(DIMS))
        c, row = self.picks(m * n, n)
        if self.last_c is not None and self.r.random() < 0.7:
            c, m, n = self.last_c
            row = self.pick(n)
            if row.ptr < c.ptr + 4 * c.n and c.ptr < row.ptr + 4 * row.n:
                return
        if self.r.random() < 0.5:
            self.hip.dispatch("add", x=row, y=c, z=c)
        else:
            self.hip.dispatch("add", x=c, y=row, z=c)

    def op_relu(self):
        if self.last_c is not None and self.r.random() < 0.7:
            c = self.last_c[0]
        else:
            c = self.pick(int(self.r.choice([64, 1024])))
        other = self.pick(c.n)
        if self.r.random() < 0.8 or (other.ptr < c.ptr + 4 * c.n and c.ptr < other.ptr + 4 * other.n):
            self.hip.dispatch("relu_fwd", x=c, y=c)
        else:
            self.hip.dispatch("relu_fwd", x=c, y=other)

    def op_relu_mask(self):
        if self.last_c is not None and self.r.random() < 0.7:
            g = self.last_c[0]
        else:
            g = self.pick(int(self.r.choice([64, 1024])))
        x = self.pick(g.n)
        if x.ptr < g.ptr + 4 * g.n and g.ptr < x.ptr + 4 * x.n:
            return
        self.hip.dispatch("relu_inplace_bwd", x=x, x_g=g)

    def op_layer_backward(self):
        """unbroadcast, zero fill, dX, dW, frees, mask: the reference's order, on random buffers."""
        B, I, O = (int(self.r.choice([2, 16, 33, 64])) for _ in range(3))
        g, w, x, gw, gb = self.picks(B * O, O * I, B * I, O * I, O)
        g_temp = None
        if self.r.random() < 0.5:          # the output gradient in a cache block that is freed before the mask arrives
            g_temp = self.hip.mem_cache_alloc(F32, B * O)
            self.hip.mem_copy(g, g_temp)
            self.done()
            g = g_temp
        if self.r.random() < 0.5:          # zero_grad() before the backward pass: the fills wait for the ops that add
            for t in (gw, gb, self.pick(int(self.r.choice([16, 640])))):
                if self.r.random() < 0.8:
                    self.hip.mem_fill(t, 0.0)
                    self.done()
        host.unbroadcast_(self.hip, g, [B, O], gb, [O], alpha=1.0, beta=1.0)
        self.done()
        gx = self.hip.mem_cache_alloc(F32, B * I)
        self.hip.mem_fill(gx, 0.0)
        self.done()
        if self.r.random() < 0.8:
            host.bmm_acc_(self.hip, g, [B, O], w, [O, I], gx, False, False, 1.0, 1.0)
            self.done()
        host.bmm_acc_(self.hip, g, [B, O], x, [B, I], gw, True, False, 1.0, 1.0)
        self.done()
        if g_temp is not None:
            self.forget_if_in(g_temp)
            self.hip.mem_cache_free(g_temp)
            self.done()
        if self.r.random() < 0.7:
            self.hip.dispatch("relu_inplace_bwd", x=x, x_g=gx)
            self.done()
        self.temps.append(gx)

    def op_unbroadcast(self):
        R, inner = int(self.r.choice([2, 16, 64])), int(self.r.choice([2, 10, 64]))
        x, y = self.picks(R * inner, inner)
        how = self.r.random()
        if how < 0.4:
            self.hip.mem_fill(y, 0.0)
        elif how < 0.5:
            self.hip.mem_fill(y.sub(0, inner // 2), 0.0)
        elif how < 0.6:
            self.hip.mem_fill(y, 0.25)
        self.done()
        host.unbroadcast_(self.hip, x, [R, inner], y, [inner], alpha=1.0, beta=1.0)

    def op_step(self):
        n = int(self.r.choice([10, 640, BUF_LEN]))
        i, j = (int(v) for v in self.r.choice(N_BUF, 2, replace=False))
        p, g = self.bufs[i].sub(0, n), self.bufs[j].sub(0, n)
        if self.r.random() < 0.5:
            self.hip.dispatch("sgd_step", param=p, grad=g, lr=0.01, clip=True, max_norm=10.0, delta=1e-6)
        else:
            m, v = self.moments[int(self.r.integers(0, len(self.moments)))]
            self.t += 1
            self.hip.dispatch("adam_step", param=p, grad=g, m=m.sub(0, n), v=v.sub(0, n), t=self.t, lr=0.01, beta1=0.9,
                              beta2=0.999, epsilon=1e-8, clip=True, max_norm=10.0, delta=1e-6)
        if self.r.random() < 0.6:
            self.done()
            self.hip.mem_fill(g, 0.0)      # zero_grad() after step()

    def op_scatter(self):
        n_nodes, n_edge = self.graph
        stride = int(self.r.choice([4, 7, 16]))
        y, h, deg, bias = self.picks(n_nodes * stride, n_nodes * stride, n_nodes, stride)
        if self.r.random() < 0.6:
            self.hip.mem_fill(y, 0.0)
            self.done()
        self.hip.dispatch("scatter_gcn_deg_scaled", dst=y, h=h, deg=deg, src_indices=self.src, tgt_indices=self.tgt,
                          stride=stride, n_edge=n_edge)
        self.done()
        if self.r.random() < 0.7:
            self.hip.dispatch("add", x=bias, y=y, z=y)
            self.done()
        if self.r.random() < 0.5:
            self.hip.dispatch("relu_fwd", x=y, y=y)

    def op_scatter_bwd(self):
        n_nodes, n_edge = self.graph
        stride = int(self.r.choice([4, 7, 16]))
        go, h, deg, gh, gd = self.picks(n_nodes * stride, n_nodes * stride, n_nodes, n_nodes * stride, n_nodes)
        gd_temp = None
        if self.r.random() < 0.5:          # the degree gradient in a block of its own that is given back unread
            gd_temp = gd = self.hip.mem_cache_alloc(F32, n_nodes)
        if self.r.random() < 0.6:
            self.hip.mem_fill(gh, 0.0)
            self.done()
        if self.r.random() < 0.6 or gd_temp is not None:
            self.hip.mem_fill(gd, 0.0)
            self.done()
        self.hip.dispatch("scatter_gcn_deg_scaled_bwd", grad_output=go, h=h, deg=deg, src_indices=self.src,
                          tgt_indices=self.tgt, grad_h=gh, grad_deg=gd, stride=stride, n_edge=n_edge)
        if gd_temp is not None:
            self.done()
            if self.r.random() < 0.3:
                self.hip.mem_fill(self.pick(16), 0.5)     # something else first: the degree gradient is computed after all
                self.done()
            self.hip.mem_cache_free(gd_temp)

    def op_scatter_add(self):
        """GatherBwd: a zero fill of the gradient, then the scatter into it (small and planned forms), sometimes with
        another fill or a fill of only part of the destination before it."""
        n = int(self.r.choice([64, 200, 1000]))
        nb = int(self.r.choice([150, 300]))                     # some offsets past the end: skipped
        src, dst = self.picks(n, nb)
        how = self.r.random()
        if how < 0.5:
            self.hip.mem_fill(dst, 0.0)
        elif how < 0.65:
            self.hip.mem_fill(dst.sub(0, nb // 2), 0.0)
        elif how < 0.75:
            self.hip.mem_fill(dst, 0.25)
        self.done()
        if self.r.random() < 0.3:
            self.hip.mem_fill(self.pick(16), 0.5)
            self.done()
        if self.r.random() < 0.3:                                # a buffer of ones scattered to count (the GCN's degrees)
            self.hip.mem_fill(src if self.r.random() < 0.7 else src.sub(0, n // 2), 1.0)
            self.done()
        self.hip.dispatch("scatter_add", src=src, offsets=self.offs.sub(0, n), dst=dst)
        if self.r.random() < 0.4:                                # deg + count, then a unary op, as the GCN's layers go on
            self.done()
            other = self.pick(nb)
            self.hip.dispatch("add", x=dst, y=other, z=other)
            self.done()
            self.hip.dispatch("tanh_fwd", x=other, y=other)      # (rsqrt of arbitrary data would bring NaNs in)

    def op_scatter_long(self):
        """Index arrays of 270000 entries in device memory: their orderings are kept under the arrays' addresses and
        checked on the GPU by every call; the arrays are rewritten in place now and then (a device copy), and what waits
        in the context when the ordering is rebuilt (an aggregation waiting for its bias, a count) must not be lost."""
        n_nodes, n = self.graph[0], 270_000
        if self.long is None:
            init = np.random.default_rng(self.seed + 20_000)
            mk = lambda hi: self.hip.from_numpy(init.integers(0, hi, n).astype(np.uint64))
            self.long = {"offs": mk(300), "offs_alt": [mk(300), mk(300)], "src": mk(n_nodes), "tgt": mk(n_nodes),
                         "tgt_alt": [mk(n_nodes), mk(n_nodes)],
                         "vals": self.hip.from_numpy((init.standard_normal(n) * 0.01).astype(np.float32))}
        L = self.long
        if self.r.random() < 0.35:
            which = int(self.r.integers(0, 2))
            if self.r.random() < 0.5:
                self.hip.mem_copy(L["offs_alt"][which], L["offs"])
            else:
                self.hip.mem_copy(L["tgt_alt"][which], L["tgt"])
            self.done()
        if self.r.random() < 0.5:
            nb = int(self.r.choice([150, 300]))
            dst = self.pick(nb)
            if self.r.random() < 0.6:
                self.hip.mem_fill(dst, 0.0)
                self.done()
            self.hip.dispatch("scatter_add", src=L["vals"], offsets=L["offs"], dst=dst)
        else:
            stride = 4
            y, h, deg, bias = self.picks(n_nodes * stride, n_nodes * stride, n_nodes, stride)
            self.hip.dispatch("scale", x=h, alpha=0.01)      # 270000 edges into 40 nodes: keep the sums small
            self.done()
            if self.r.random() < 0.6:
                self.hip.mem_fill(y, 0.0)
                self.done()
            self.hip.dispatch("scatter_gcn_deg_scaled", dst=y, h=h, deg=deg, src_indices=L["src"], tgt_indices=L["tgt"],
                              stride=stride, n_edge=n)
            self.done()
            if self.r.random() < 0.7:
                self.hip.dispatch("add", x=bias, y=y, z=y)
                self.done()
            if self.r.random() < 0.4:       # the next long call finds the aggregation still waiting
                self.hip.dispatch("scatter_add", src=L["vals"], offsets=L["offs"], dst=self.pick(300))

    def op_max_along(self):
        rows, cols = int(self.r.choice([8, 64])), int(self.r.choice([2, 7, 33]))
        x, y = self.picks(rows * cols, rows)
        how = self.r.random()
        if how < 0.5:
            self.hip.mem_fill(y, 0.0)                           # NDArray.max_along zero-fills its output
        elif how < 0.65:
            self.hip.mem_fill(y.sub(0, rows // 2), 0.5)
        elif how < 0.75:
            room = [b for b in self.bufs + self.temps if b.ptr <= y.ptr < b.ptr + 4 * b.n][0]
            off = (y.ptr - room.ptr) // 4
            if off + rows + 4 <= room.n:
                self.hip.mem_fill(room.sub(off, rows + 4), 0.75)  # sticks out of the output: must be seen
        self.done()
        self.hip.dispatch("max_along", x=x, x_shape=[rows, cols], y=y, y_shape=[rows], dim=1)

    def op_loss(self):
        rows, cols = int(self.r.choice([8, 64])), int(self.r.choice([7, 10]))
        logits, target, probs, loss, grad = self.picks(rows * cols, rows * cols, rows * cols, 1, rows * cols)
        self.hip.dispatch("smce_fwd", logits=logits, target=target, probs=probs, loss=loss, rows=rows, cols=cols)
        self.done()
        self.hip.mem_fill(self.pick(1), 1.0)         # the upstream gradient of the loss
        self.done()
        if self.r.random() < 0.7:
            self.hip.mem_fill(grad, 0.0)
            self.done()
        self.hip.dispatch("smce_bwd", probs=probs, target=target, grad=grad, rows=rows, cols=cols)

    def op_alloc(self):
        n = int(self.r.choice([16, 1024, BUF_LEN]))
        t = self.hip.mem_cache_alloc(F32, n)
        self.hip.mem_fill(t, float(self.r.choice([0.0, 0.25])))
        self.temps.append(t)

    def forget_if_in(self, t):
        """The last product's output may lie in a temporary: once that is given back it must not be used again."""
        c = self.last_c
        if c is not None and t.ptr <= c[0].ptr < t.ptr + 4 * t.n:
            self.last_c = None

    def op_free(self):
        if self.temps:
            t = self.temps.pop(int(self.r.integers(0, len(self.temps))))
            self.forget_if_in(t)
            self.hip.mem_cache_free(t)

    def op_copy(self):
        n = int(self.r.choice([16, 1000, BUF_LEN]))
        a, b = self.picks(n, n)
        if self.r.random() < 0.4:                   # MaskLayer.backward: a zero-filled gradient, then rows copied into it
            room = [t for t in self.bufs + self.temps if t.ptr <= b.ptr < t.ptr + 4 * t.n][0]
            lo = (b.ptr - room.ptr) // 4
            lo0 = max(0, lo - int(self.r.integers(0, 40)))
            hi0 = min(room.n, lo + n + int(self.r.integers(0, 40)))
            self.hip.mem_fill(room.sub(lo0, hi0 - lo0), float(self.r.choice([0.0, 0.5])))
            self.done()
        self.hip.mem_copy(a, b)

    def op_elementwise(self):
        n = int(self.r.choice([64, 1024, BUF_LEN]))
        a, b = self.picks(n, n)
        which = int(self.r.integers(0, 3))
        if which == 0:
            self.hip.dispatch("add", x=a, y=b, z=b)
        elif which == 1:
            self.hip.dispatch("mul", x=a, y=b, z=b)
        else:
            self.hip.dispatch("tanh_fwd", x=a, y=b)

    def op_map_run(self):
        """A run of small elementwise ops of one length over a few buffers: results feeding later ops, in-place forms,
        one-float operands, and now and then a view shifted against one an earlier op of the run wrote."""
        n = int(self.r.choice([1, 64, 1000, 4096]))
        picked = self.picks(n, n, n, n, 1, 1)     # six different buffers: a one-float operand never lies in an output
        views, scalars = picked[:4], picked[4:]
        fresh = []                                        # outputs allocated inside the run, as a caller's op chain does
        for _ in range(int(self.r.integers(2, 6))):
            x, y, z = (views[int(v)] for v in self.r.integers(0, len(views), 3))
            if fresh and self.r.random() < 0.3:           # given back while the ops that use it may still wait
                t = fresh.pop(int(self.r.integers(0, len(fresh))))
                views = [v for v in views if v.ptr != t.ptr]
                self.hip.mem_cache_free(t)
                continue
            if self.r.random() < 0.3:
                z = self.hip.mem_cache_alloc(F32, n)
                fresh.append(z)
                views = views + [z]
                kind = int(self.r.integers(0, 3))         # a new block holds nothing: ops that only write it
                if kind == 0:
                    self.hip.dispatch(str(self.r.choice(["add", "sub", "mul"])), x=x, y=y, z=z)
                elif kind == 1:
                    self.hip.dispatch("mul", x=x, y=scalars[0], z=z)
                else:
                    self.hip.dispatch("tanh_fwd", x=x, y=z)
                self.done()
                continue
            if self.r.random() < 0.15 and n > 8:          # shifted against a buffer of the run
                base = views[int(self.r.integers(0, len(views)))]
                room = [b for b in self.bufs + self.temps + fresh if b.ptr <= base.ptr < b.ptr + 4 * b.n][0]
                off = (base.ptr - room.ptr) // 4 + 4
                if off + n <= room.n:
                    x = room.sub(off, n)
            if x.ptr != z.ptr and x.ptr < z.ptr + 4 * n and z.ptr < x.ptr + 4 * n:
                continue                                  # an op that reads a shifted view of its own output races with itself
            if self.r.random() < 0.3:                     # ensure_grad(0), or any other fill, right before the op
                f = self.r.random()
                target = z if f < 0.7 else (z.sub(0, n // 2) if n > 1 and f < 0.85 else x)
                self.hip.mem_fill(target, float(self.r.choice([0.0, 0.0, 0.25, -0.0])))
                self.done()
            kind = int(self.r.integers(0, 8))
            if kind == 0:
                self.hip.dispatch(str(self.r.choice(["add", "sub", "mul"])), x=x, y=y, z=z)
            elif kind == 1:
                s = scalars[int(self.r.integers(0, 2))]
                if self.r.random() < 0.5:
                    self.hip.dispatch(str(self.r.choice(["add", "mul", "sub"])), x=s, y=y, z=z)
                else:
                    self.hip.dispatch(str(self.r.choice(["add", "mul", "sub"])), x=x, y=s, z=z)
            elif kind == 2:
                self.hip.dispatch(str(self.r.choice(["relu_fwd", "tanh_fwd", "sigm_fwd"])), x=x, y=z)
            elif kind == 3:
                self.hip.dispatch("relu_fwd", x=z, y=z)
            elif kind == 4 and x.ptr != z.ptr and y.ptr != z.ptr:
                self.hip.dispatch(str(self.r.choice(["relu_bwd"])), x=x, x_g=z, y_g=y)
            elif kind == 5 and x.ptr != z.ptr and y.ptr != z.ptr:
                self.hip.dispatch(str(self.r.choice(["tanh_bwd", "sigm_bwd"])), x_g=z, y=x, y_g=y)
            elif kind == 6 and x.ptr != z.ptr:
                self.hip.dispatch(str(self.r.choice(["relu_inplace_bwd", "tanh_inplace_bwd"])), x=x, x_g=z)
            elif kind == 7:
                self.hip.dispatch("scale", x=z, alpha=0.5)
            self.done()
        for t in fresh:
            self.hip.mem_cache_free(t)

    def op_plain(self):
        """One of the ops that neither wait nor take over waiting work (they launch what waits, then themselves) and the
        by-value scalar forms: operands land on buffers other calls left work waiting on."""
        r, hip = self.r, self.hip
        which = int(r.integers(0, 40))
        n = int(r.choice([16, 64, 1000]))
        if which == 0:
            x, y = self.picks(n, 1); hip.dispatch("sum", x=x, y=y)
        elif which == 1:
            x, y = self.picks(n, 1); hip.dispatch("nrm2", x=x, y=y)
        elif which == 2:
            x, y, z = self.picks(n, n, 1); hip.dispatch("dot", x=x, y=y, z=z)
        elif which == 3:
            x, y, g, yg = self.picks(n, 1, n, 1)
            hip.dispatch("max_fwd", x=x, y=y); self.done()
            hip.dispatch("max_bwd", x=x, x_g=g, y=y, y_g=yg)
        elif which == 4:
            x, y = self.picks(n, n); hip.dispatch("axpy", x=x, y=y, alpha=0.25)
        elif which == 5:
            x, y, a = self.picks(n, n, 1); hip.dispatch("axpy", x=x, y=y, alpha=a)
        elif which == 6:
            hip.dispatch("clip_nrm2", x=self.pick(n), max_norm=0.5, delta=1e-6)
        elif which == 7:
            x, y = self.picks(n, n)
            if r.random() < 0.3:                                   # square roots and quotients of known values only
                hip.mem_fill(x, 0.25); self.done()
                hip.dispatch("sqrt_fwd", x=x, y=y)
            elif r.random() < 0.5:
                hip.mem_fill(y, 2.0); self.done()
                hip.dispatch("div", x=x, y=y, z=y)
            else:
                hip.dispatch(str(r.choice(["exp_fwd", "sigm_fwd"])), x=x, y=y)
        elif which == 8:
            x, y = self.picks(n, n); hip.dispatch("pow_fwd", x=x, exp=2.0, y=y)
        elif which == 9:
            x, y = self.picks(n, n); hip.dispatch("rsqrt_fwd", x=x, y=y, eps=0.5)
        elif which == 10:
            x, y = self.picks(n, n); hip.dispatch("clamp_fwd", x=x, y=y, min=-0.05, max=0.05)
        elif which == 11:
            x, g, yg = self.picks(n, n, n)
            name = str(r.choice(["pow_bwd", "sqrt_bwd", "rsqrt_bwd", "clamp_bwd"]))
            extra = {"pow_bwd": {"exp": 2.0, "eps": 1e-3}, "sqrt_bwd": {"eps": 0.05}, "rsqrt_bwd": {"eps": 0.05},
                     "clamp_bwd": {"min": -0.05, "max": 0.05}}[name]
            hip.dispatch(name, x=x, x_g=g, y_g=yg, **extra)
        elif which == 12:
            g, y, yg = self.picks(n, n, n)
            if r.random() < 0.6:
                hip.dispatch("exp_bwd", x_g=g, y=y, y_g=yg)
            else:
                hip.dispatch("sigm_inplace_bwd", x=y, x_g=g)
        elif which == 13:
            m, k = int(r.choice([7, 16, 33])), int(r.choice([5, 32]))
            A, B = self.picks(m * k, m * k); hip.dispatch("transpose", A=A, B=B, m=m, n=k, alpha=1.0)
        elif which == 14:
            m, k = int(r.choice([7, 16])), int(r.choice([5, 32]))
            x, y, A = self.picks(m, k, m * k); hip.dispatch("outer", x=x, y=y, A=A, alpha=0.5)
        elif which == 15:
            m, k = int(r.choice([7, 33])), int(r.choice([5, 64]))
            ta = bool(r.integers(0, 2))
            A, x, y = self.picks(m * k, m if ta else k, k if ta else m)
            hip.dispatch("matvec", A=A, x=x, y=y, m=m, n=k, trans_a=ta, alpha=1.0, beta=float(r.choice([0.0, 1.0])))
        elif which == 16:
            x, y = self.picks(16, 64); hip.dispatch("broadcast", x=x, y=y, alpha=0.5, beta=1.0)
        elif which == 17:
            rows, cols = int(r.choice([8, 33])), int(r.choice([7, 64]))
            dim = int(r.integers(0, 2))
            x, y = self.picks(rows * cols, cols if dim == 0 else rows)
            hip.dispatch("sum_along", x=x, x_shape=[rows, cols], y=y, dim=dim, alpha=1.0, beta=float(r.choice([0.0, 1.0])))
        elif which == 18:
            rows, cols = 16, 33
            hip.dispatch("argmax_along", x=self.pick(rows * cols), x_shape=[rows, cols], y=self.u64_out.sub(0, rows), dim=1)
        elif which == 19:
            rows, cols = int(r.choice([8, 64])), int(r.choice([7, 10]))
            x, y, g = self.picks(rows * cols, rows * cols, rows * cols)
            hip.dispatch("softmax_fwd", x=x, y=y, rows=rows, cols=cols); self.done()
            hip.dispatch("softmax_bwd", y=y, y_g=x, x_g=g, rows=rows, cols=cols)
        elif which == 20:
            rows, cols = 64, 64
            lg, lse, loss, g = self.picks(rows * cols, rows, 1, rows * cols)
            lab = self.idx.sub(0, rows)
            hip.dispatch("smce_label_fwd", logits=lg, labels=lab, lse=lse, loss=loss, rows=rows, cols=cols); self.done()
            hip.dispatch("smce_label_bwd", logits=lg, labels=lab, lse=lse, grad=g, rows=rows, cols=cols,
                         accumulate=bool(r.integers(0, 2)))
        elif which == 21:
            p_, t_, g, loss = self.picks(n, n, n, 1)
            if r.random() < 0.5:
                hip.dispatch("smooth_l1_fwd", pred=p_, target=t_, beta=1.0, loss=loss); self.done()
                hip.dispatch("smooth_l1_bwd", pred=p_, target=t_, grad=g, beta=1.0)
            else:
                hip.dispatch("smooth_l1_fwd_bwd", pred=p_, target=t_, grad=g, beta=1.0, loss=loss,
                             accumulate=bool(r.integers(0, 2)))
        elif which == 22:
            p_, t_, g, loss = self.picks(n, n, n, 1)
            hip.dispatch("mse_fwd", pred=p_, target=t_, loss=loss); self.done()
            hip.dispatch("mse_bwd", pred=p_, target=t_, grad=g)
        elif which == 23:
            stride, n_idx = int(r.choice([4, 16])), int(r.choice([10, 200]))
            src, dst = self.picks(64 * stride, n_idx * stride)
            hip.dispatch("index_select_fwd", src=src, indices=self.idx.sub(0, n_idx), stride=stride, dst=dst); self.done()
            hip.dispatch("index_select_bwd", y_grad=dst, indices=self.idx.sub(0, n_idx), stride=stride, x_grad=src)
        elif which == 24:
            src, dst = self.picks(64 * 8, 16 * 8)        # gather along dim 0 of [64, 8] with an index tensor [16, 8]
            offs = self.u64_out.sub(0, 128)
            if r.random() < 0.5:
                hip.gather_offsets([64, 8], [16, 8], self.idx.sub(0, 128), 0, offs, check=False); self.done()
                hip.mem_take(src, offs, dst)
            else:
                hip.gather(src, [64, 8], [16, 8], self.idx.sub(0, 128), 0, offs, dst, check=False)
        elif which == 25:
            hip.mem_sequence(self.pick(n), 0.0, 0.001)
        elif which == 26:
            hip.mem_fill(self.u64_out.sub(256, 64), 3)
            room = self.pick(64)
            hip._call("zg_hip_mem_fill_u8", room.ptr, 64, 0)      # 16 floats set to +0.0 byte by byte
        elif which == 27:
            src, dst = self.picks(64, 64); hip.dispatch("scatter_add_csr", src=src, row_ptr=self.row_ptr, dst=dst)
        elif which == 28:
            src, dst = self.picks(256, 62)
            hip.dispatch("segment_sum_csr", src=src, row_offsets=self.seg_bounds, dst=dst)
        elif which == 29:
            B, I, O = (int(r.choice([2, 16, 33])) for _ in range(3))
            x, w, b, y = self.picks(B * I, O * I, O, B * O)
            hip.dispatch("linear_fwd", x=x, w=w, bias=b if r.random() < 0.7 else None, y=y, batch=B, fan_in=I, fan_out=O,
                         relu=bool(r.integers(0, 2)))
        elif which == 30:
            B, I, O = (int(r.choice([2, 16, 33])) for _ in range(3))
            gy, w, act, gx = self.picks(B * O, O * I, B * I, B * I)
            hip.dispatch("linear_bwd_input", gy=gy, w=w, act_in=act if r.random() < 0.7 else None, gx=gx, batch=B, fan_in=I,
                         fan_out=O, accumulate=bool(r.integers(0, 2)))
        elif which == 31:
            B, I, O = (int(r.choice([2, 16, 33])) for _ in range(3))
            gy, x, w, gw, gb, gx = self.picks(B * O, B * I, O * I, O * I, O, B * I)
            hip.dispatch("linear_bwd", gy=gy, x=x, w=w, act_in=x if r.random() < 0.5 else None, gw=gw,
                         gb=gb if r.random() < 0.7 else None, gx=gx, batch=B, fan_in=I, fan_out=O)
        elif which == 32:
            sizes = [int(v) for v in r.choice([10, 640, 1024], 3)]
            ids = [int(v) for v in r.choice(N_BUF, 6, replace=False)]
            ps = [self.bufs[i].sub(0, k) for i, k in zip(ids[:3], sizes)]
            gs = [self.bufs[i].sub(0, k) for i, k in zip(ids[3:], sizes)]
            if r.random() < 0.5:
                hip.dispatch("sgd_step_multi", params=ps, grads=gs, lr=0.01, clip=True, max_norm=10.0, delta=1e-6,
                             zero_grads=bool(r.integers(0, 2)))
            else:
                ms = [self.moments[i][0].sub(0, k) for i, k in enumerate(sizes)]
                vs = [self.moments[i][1].sub(0, k) for i, k in enumerate(sizes)]
                hip.dispatch("adam_step_multi", params=ps, grads=gs, ms=ms, vs=vs, lr=0.01, t_first=self.t + 1, beta1=0.9,
                             beta2=0.999, epsilon=1e-8, clip=True, max_norm=10.0, delta=1e-6, zero_grads=bool(r.integers(0, 2)))
                self.t += 3
        elif which == 33:
            k = int(r.choice([10, 640]))
            i, j = (int(v) for v in r.choice(N_BUF, 2, replace=False))
            m, v = self.moments[0]
            lr_t = self.lr_slot
            hip.mem_fill(lr_t, 0.001); self.done()
            hip.dispatch("adam_step_at", param=self.bufs[i].sub(0, k), grad=self.bufs[j].sub(0, k), m=m.sub(0, k), v=v.sub(0, k),
                         lr_t=lr_t, beta1=0.9, beta2=0.999, epsilon=1e-8, clip=True, max_norm=10.0, delta=1e-6)
        elif which == 34:
            n_nodes, n_edge = self.graph
            stride = int(r.choice([4, 7]))
            y, h, deg, bias, gh = self.picks(n_nodes * stride, n_nodes * stride, n_nodes, stride, n_nodes * stride)
            hip.dispatch("scatter_gcn_deg_scaled_planned", dst=y, h=h, deg=deg, plan=self.plan, stride=stride,
                         accumulate=bool(r.integers(0, 2)), bias=bias if r.random() < 0.5 else None, relu=bool(r.integers(0, 2)))
            self.done()
            hip.dispatch("scatter_gcn_deg_scaled_bwd_planned", grad_output=y, h=h, deg=deg, plan=self.plan, grad_h=gh,
                         grad_deg=None, stride=stride, accumulate=bool(r.integers(0, 2)))
        elif which == 35:
            n_nodes, n_edge = self.graph
            src, dst = self.picks(n_edge, n_nodes)
            hip.dispatch("scatter_add_planned", src=src, plan=self.plan, dst=dst, accumulate=bool(r.integers(0, 2)))
        elif which == 36:
            rows, cols = int(r.choice([8, 64])), int(r.choice([7, 10]))
            lg, tg, pr, loss, g = self.picks(rows * cols, rows * cols, rows * cols, 1, rows * cols)
            hip.dispatch("smce_fwd_bwd", logits=lg, target=tg, probs=pr, loss=loss, grad=g, rows=rows, cols=cols,
                         accumulate=bool(r.integers(0, 2)))
        elif which == 37:
            m, k2, k = (int(r.choice([7, 16, 33])) for _ in range(3))
            a, b, c = self.picks(2 * m * k, k * k2, 2 * m * k2)    # two batches of A against one B
            host.bmm_acc_(hip, a, [2, m, k], b, [k, k2], c, False, False, 1.0, float(r.choice([0.0, 1.0])))
        elif which == 38:
            x, z = self.picks(n, n)                                # host scalars: by value
            name = str(r.choice(["add", "sub", "mul", "div"]))
            if r.random() < 0.5:
                hip.dispatch(name, x=x, y=2.0, z=z if r.random() < 0.5 else x)
            else:
                hip.dispatch(name if name != "div" else "sub", x=0.5, y=x, z=z)
        elif which == 39:
            hip.flush()

    def op_read(self):
        if not self.with_reads:
            return
        self.reads.append(self.hip.to_numpy(self.bufs[int(self.r.integers(0, N_BUF))]).view(np.uint32).copy())

    def ops(self, n_ops):
        """The sequence of this run's seed, from the start: every call of ops() makes the same choices."""
        self.r = np.random.default_rng(self.seed)
        self.t = 0
        self.last_c = None
        ops = [self.op_fill, self.op_matmul, self.op_add_row, self.op_relu, self.op_relu_mask, self.op_layer_backward,
               self.op_unbroadcast, self.op_step, self.op_scatter, self.op_alloc, self.op_free, self.op_read, self.op_copy,
               self.op_elementwise, self.op_scatter_bwd, self.op_loss, self.op_map_run, self.op_scatter_add,
               self.op_max_along, self.op_plain, self.op_scatter_long]
        weights = np.array([3, 4, 3, 3, 2, 2, 2, 3, 2, 1, 2, 1, 1, 1, 1, 1, 3, 1, 1, 6, 0.5], float)
        self.trace = []
        for _ in range(n_ops):
            op = ops[int(self.r.choice(len(ops), p=weights / weights.sum()))]
            self.trace.append(op.__name__)
            op()
            self.done()
        self.kept = list(self.temps)

    def free_temps(self):
        for t in self.temps:
            self.hip.mem_cache_free(t)
        self.temps = []

    def finish(self):
        out = [self.hip.to_numpy(b).view(np.uint32).copy() for b in self.bufs]
        for t in self.temps:
            out.append(self.hip.to_numpy(t).view(np.uint32).copy())
        self.free_temps()
        for m, v in self.moments:
            out += [self.hip.to_numpy(m).view(np.uint32).copy(), self.hip.to_numpy(v).view(np.uint32).copy()]
        self.plan.free()
        if self.long is not None:
            for v in self.long.values():
                for b in (v if isinstance(v, list) else [v]):
                    self.hip.mem_free(b)
        for b in self.bufs + [self.src, self.tgt, self.offs, self.idx, self.row_ptr, self.seg_bounds, self.u64_out, self.lr_slot] + \
                [x for mv in self.moments for x in mv]:
            self.hip.mem_free(b)
        return out, self.reads

    def run(self, n_ops):
        self.ops(n_ops)
        return self.finish()


def _first_divergence(hip, seed, n_ops):
    """The shortest prefix of the sequence after which the two ways differ, and the call that ends it."""
    for k in range(1, n_ops + 1):
        a = _Run(hip, seed, eager=False, reads=False)
        lazy, _ = a.run(k)
        want, _ = _Run(hip, seed, eager=True, reads=False).run(k)
        bad = [i for i, (x, y) in enumerate(zip(lazy, want)) if not np.array_equal(x, y)]
        if bad:
            return f"first difference after call {k} ({a.trace[-1]}; the calls before it: {a.trace[-6:-1]}), buffers {bad}"
    return "no prefix of the sequence differs (the difference needs the reads in between)"


@pytest.mark.parametrize("seed", range(1000))
def test_random_sequences_leave_what_one_launch_per_call_leaves(hip, seed):
    in_use0 = hip.cache_stats()["bytes_in_use"]
    lazy, lazy_reads = _Run(hip, seed, eager=False).run(80)
    want, want_reads = _Run(hip, seed, eager=True).run(80)
    assert len(lazy) == len(want) and len(lazy_reads) == len(want_reads)
    if not all(np.all(np.isfinite(b.view(np.float32))) for b in want):
        pytest.skip("the sequence overflowed: NaN payloads are not part of the contract")
    same = all(np.array_equal(a, b) for a, b in zip(lazy_reads, want_reads)) and \
        all(np.array_equal(a, b) for a, b in zip(lazy, want))
    if not same:
        pytest.fail(f"seed {seed}: {_first_divergence(hip, seed, 80)}")
    hip.sync()
    assert hip.cache_stats()["bytes_in_use"] == in_use0


# Entry points that are no device op of a call sequence: set-up and tear-down, queries, allocation from the driver, host
# copies (they wait for the stream), recording, staging, timing.  Everything else the header declares must be called
# by the random sequences above, so a new entry point cannot stay outside them unnoticed.
NOT_IN_SEQUENCES = {
    "zg_hip_last_error", "zg_hip_device_count", "zg_hip_init", "zg_hip_deinit", "zg_hip_total_memory", "zg_hip_stream",
    "zg_hip_event_create", "zg_hip_event_record", "zg_hip_event_elapsed_ms", "zg_hip_event_destroy", "zg_hip_page_size",
    "zg_hip_pool_map", "zg_hip_pool_unmap", "zg_hip_cache_configure", "zg_hip_clear_cache", "zg_hip_is_device_ptr",
    "zg_hip_mem_scratch", "zg_hip_launch_count", "zg_hip_gemm_timing", "zg_hip_gemm_timing_read", "zg_hip_gemm_plan",
    "zg_hip_plan_cache_stats", "zg_hip_unbroadcast_scratch_len", "zg_hip_adam_lr_t", "zg_hip_set_holding",
    "zg_hip_graph_open", "zg_hip_graph_save", "zg_hip_graph_run", "zg_hip_graph_free", "zg_hip_staged_h2d",
    "zg_hip_staging_after_compute", "zg_hip_compute_after_staging", "zg_hip_staging_wait", "zg_hip_mem_random",
    "zg_hip_smce_label_fwd_noalloc", "zg_hip_edge_plan_free", "zg_hip_host_free", "zg_hip_sync", "zg_hip_cache_stats",
}


def test_the_sequences_call_every_op_entry_point_the_header_declares(hip, monkeypatch):
    from zigrad_amd._lib import parse_header

    called = set()
    real = hip._lib.call

    def recording(name, *args):
        called.add(name)
        return real(name, *args)

    monkeypatch.setattr(hip._lib, "call", recording)
    for seed in range(200):
        _Run(hip, seed, eager=False).run(80)
    declared = set(parse_header())
    missing = declared - NOT_IN_SEQUENCES - called
    assert not missing, f"entry points no random sequence calls: {sorted(missing)}"
    assert not (NOT_IN_SEQUENCES - declared), f"not declared any more: {sorted(NOT_IN_SEQUENCES - declared)}"


@pytest.mark.parametrize("seed", range(40))
def test_recorded_random_sequences_replay_what_the_eager_calls_leave(hip, seed):
    """The same sequences recorded as an execution graph (nothing runs while recording; waiting work is launched into
    the recording) and replayed three times, against the same calls issued three times with one launch per call."""
    n_ops, reps = 50, 3
    in_use0 = hip.cache_stats()["bytes_in_use"]
    eager = _Run(hip, seed, eager=True, reads=False)
    for _ in range(reps):
        eager.ops(n_ops)
        eager.free_temps()
    want, _ = eager.finish()
    rec = _Run(hip, seed, eager=False, reads=False)
    rec.ops(n_ops)          # once eagerly: the allocator and the workspace reach their final size
    rec.free_temps()
    hip.sync()
    hip.graph_open()
    try:
        rec.ops(n_ops)
        rec.free_temps()
    finally:
        graph = hip.graph_save()
    for _ in range(reps - 1):
        graph.run()
    hip.sync()
    got, _ = rec.finish()
    graph.free()
    if not all(np.all(np.isfinite(b.view(np.float32))) for b in want):
        pytest.skip("the sequence overflowed: NaN payloads are not part of the contract")
    for i, (a, b) in enumerate(zip(got, want)):
        assert np.array_equal(a, b), f"seed {seed}: buffer {i} differs in {np.count_nonzero(a != b)} elements"
    hip.sync()
    assert hip.cache_stats()["bytes_in_use"] == in_use0
