"""Small elementwise ops of one length wait in the context and go out as one launch (the reference launches each at
once: src/device/host_device.zig:300-420).  Every result must be bit-identical to the ops run one launch each, which
is what the same calls with a synchronisation after each of them give."""
from __future__ import annotations

import numpy as np
import pytest

from zigrad_amd.device import F32

pytestmark = pytest.mark.gpu


def both_ways(hip, body):
    """body(step) issues the calls and returns the buffers to compare; step() is called after every call."""
    outs = []
    for sync_each in (False, True):
        step = hip.sync if sync_each else (lambda: None)
        bufs = body(step)
        outs.append([hip.to_numpy(b).view(np.uint32).copy() for b in bufs])
        for b in bufs:
            hip.mem_free(b)
    for lazy, eager in zip(*outs):
        np.testing.assert_array_equal(lazy, eager)
    return outs[0]


def test_td_target_chain_with_allocations_and_frees_between(hip):
    """The op chain of a DQN target (examples/dqn/src/dqn_agent.zig:173-186): every op's output is allocated just
    before it and the temporaries are given back afterwards."""
    r = np.random.default_rng(0)
    B = 64
    q = r.standard_normal(B).astype(np.float32)
    done = (r.random(B) < 0.3).astype(np.float32)
    rew = r.standard_normal(B).astype(np.float32)

    def body(step):
        qd, dd, rd = hip.from_numpy(q), hip.from_numpy(done), hip.from_numpy(rew)
        gamma, one = hip.from_numpy(np.float32([0.99])), hip.from_numpy(np.float32([1.0]))
        out = hip.mem_alloc(F32, B)
        disc = hip.mem_cache_alloc(F32, B); step()
        hip.dispatch("mul", x=qd, y=gamma, z=disc); step()
        nd = hip.mem_cache_alloc(F32, B); step()
        hip.dispatch("sub", x=one, y=dd, z=nd); step()
        masked = hip.mem_cache_alloc(F32, B); step()
        hip.dispatch("mul", x=disc, y=nd, z=masked); step()
        tgt = hip.mem_cache_alloc(F32, B); step()
        hip.dispatch("add", x=rd, y=masked, z=tgt); step()
        for t in (disc, nd, masked):
            hip.mem_cache_free(t); step()
        again = hip.mem_cache_alloc(F32, B); step()       # receives a block the waiting ops still use
        hip.dispatch("relu_fwd", x=tgt, y=again); step()
        hip.mem_copy(again, out); step()
        hip.mem_cache_free(again); hip.mem_cache_free(tgt)
        for t in (qd, dd, rd, gamma, one):
            hip.mem_free(t)
        return [out]

    got = both_ways(hip, body)[0].view(np.float32)
    want = np.maximum(rew + (q * np.float32(0.99)) * (np.float32(1.0) - done), 0)
    np.testing.assert_array_equal(got, want)


def test_td_target_chain_with_host_scalars_is_one_launch_and_can_be_recorded(hip):
    """gamma and 1 as host scalars (NDArray's scalar ops pass `&.{s}`, src/ndarray.zig:247-257): they travel by value, so
    the chain still leaves as one launch, equals the chain with one-float device operands bit for bit, and a recording
    accepts it (a copy of the scalar to the device would not be recordable)."""
    r = np.random.default_rng(5)
    B = 64
    q = r.standard_normal(B).astype(np.float32)
    done = (r.random(B) < 0.3).astype(np.float32)
    rew = r.standard_normal(B).astype(np.float32)
    qd, dd, rd = hip.from_numpy(q), hip.from_numpy(done), hip.from_numpy(rew)
    gamma_d, one_d = hip.from_numpy(np.float32([0.99])), hip.from_numpy(np.float32([1.0]))
    disc, nd, masked, tgt = (hip.mem_alloc(F32, B) for _ in range(4))

    def chain(gamma, one):
        hip.dispatch("mul", x=qd, y=gamma, z=disc)
        hip.dispatch("sub", x=one, y=dd, z=nd)
        hip.dispatch("mul", x=disc, y=nd, z=masked)
        hip.dispatch("add", x=rd, y=masked, z=tgt)

    chain(gamma_d, one_d)
    want = hip.to_numpy(tgt).copy()
    np.testing.assert_array_equal(want, rew + (q * np.float32(0.99)) * (np.float32(1.0) - done))
    hip.mem_fill(tgt, np.nan)
    hip.sync()
    before = hip.launch_count()
    chain(0.99, 1.0)
    hip.sync()
    assert hip.launch_count() - before == 1
    np.testing.assert_array_equal(hip.to_numpy(tgt), want)
    # recorded and replayed, with eager work and a synchronisation between the replays
    hip.graph_open()
    chain(0.99, 1.0)
    g = hip.graph_save()
    for _ in range(3):
        hip.mem_fill(tgt, np.nan)
        hip.sync()
        g.run()
        np.testing.assert_array_equal(hip.to_numpy(tgt), want)
    g.free()
    for b in (qd, dd, rd, gamma_d, one_d, disc, nd, masked, tgt):
        hip.mem_free(b)


def test_host_scalar_ops_alone_and_in_runs_match_a_launch_each(hip):
    n = 1000
    x0 = np.linspace(-3, 3, n).astype(np.float32)

    def body(step):
        x, y = hip.from_numpy(x0), hip.mem_alloc(F32, n)
        hip.dispatch("div", x=2.0, y=x, z=y); step()
        hip.dispatch("add", x=y, y=-0.5, z=y); step()
        hip.dispatch("mul", x=3.0, y=y, z=x); step()
        hip.dispatch("sub", x=x, y=0.125, z=x); step()
        hip.dispatch("div", x=x, y=7.0, z=x); step()
        return [x, y]

    x, y = (v.view(np.float32) for v in both_ways(hip, body))
    want_y = np.float32(2.0) / x0 + np.float32(-0.5)
    np.testing.assert_array_equal(y, want_y)
    np.testing.assert_array_equal(x, (np.float32(3.0) * want_y - np.float32(0.125)) / np.float32(7.0))


def test_in_place_ops_and_results_feeding_later_ops(hip):
    r = np.random.default_rng(1)
    n = 1000
    a0, b0 = r.standard_normal(n).astype(np.float32), r.standard_normal(n).astype(np.float32)

    def body(step):
        a, b, c = hip.from_numpy(a0), hip.from_numpy(b0), hip.mem_alloc(F32, n)
        hip.dispatch("add", x=a, y=b, z=c); step()
        hip.dispatch("mul", x=c, y=c, z=c); step()
        hip.dispatch("tanh_fwd", x=c, y=a); step()        # overwrites an operand of the first op
        hip.dispatch("sub", x=a, y=b, z=b); step()
        hip.dispatch("scale", x=b, alpha=0.25); step()
        hip.dispatch("relu_fwd", x=b, y=b); step()
        hip.dispatch("sigm_fwd", x=c, y=c); step()
        return [a, b, c]

    a, b, c = (x.view(np.float32) for x in both_ways(hip, body))
    s = (a0 + b0) * (a0 + b0)
    np.testing.assert_allclose(a, np.tanh(s), rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(b, np.maximum((a - b0) * np.float32(0.25), 0), rtol=0, atol=0)
    np.testing.assert_allclose(c, 1 / (1 + np.exp(-s.astype(np.float64))), rtol=1e-5, atol=1e-6)


def test_more_ops_than_the_queue_holds_and_a_change_of_length(hip):
    n = 777
    x0 = np.linspace(-2, 2, n).astype(np.float32)

    def body(step):
        x, y = hip.from_numpy(x0), hip.from_numpy(np.ones(n, np.float32))
        for _ in range(21):
            hip.dispatch("add", x=x, y=y, z=x); step()
        hip.dispatch("mul", x=x.sub(0, 100), y=x.sub(0, 100), z=y.sub(0, 100)); step()   # another length: a new run
        hip.dispatch("add", x=x, y=y, z=y); step()
        return [x, y]

    x, y = (v.view(np.float32) for v in both_ways(hip, body))
    want_x = x0.copy()
    for _ in range(21):
        want_x = want_x + np.float32(1)
    np.testing.assert_array_equal(x, want_x)
    want_y = np.ones(n, np.float32)
    want_y[:100] = x[:100] * x[:100]
    np.testing.assert_array_equal(y, x + want_y)


def test_views_that_overlap_out_of_step_do_not_share_a_launch(hip):
    """Element i of the second op reads what the first wrote at i + 4: two launches, or thread i would read before
    thread i + 4 has written."""
    n = 4096
    x0 = np.arange(n + 8, dtype=np.float32)

    def body(step):
        buf, one = hip.from_numpy(x0), hip.from_numpy(np.ones(n, np.float32))
        out = hip.mem_alloc(F32, n)
        hip.dispatch("add", x=buf.sub(4, n), y=one, z=buf.sub(4, n)); step()
        hip.dispatch("mul", x=buf.sub(0, n), y=one, z=out); step()       # reads the shifted view
        hip.dispatch("add", x=out, y=one, z=buf.sub(8, n)); step()       # writes over what the ops before read
        return [buf, out, one]

    buf, out, _ = (v.view(np.float32) for v in both_ways(hip, body))
    mid = x0.copy()
    mid[4:4 + n] += 1
    np.testing.assert_array_equal(out, mid[:n])
    mid[8:8 + n] = out + 1
    np.testing.assert_array_equal(buf, mid)


def test_a_one_float_operand_written_by_an_op_of_the_run(hip):
    n = 64
    v0 = np.arange(n, dtype=np.float32)

    def body(step):
        v, s, w = hip.from_numpy(v0), hip.from_numpy(np.float32([2.0, 0, 0, 0])), hip.mem_alloc(F32, n)
        hip.dispatch("mul", x=v, y=s.sub(0, 1), z=w); step()
        hip.dispatch("add", x=s.sub(0, 1), y=s.sub(0, 1), z=s.sub(0, 1)); step()   # the scalar doubles: length 1
        hip.dispatch("mul", x=w, y=s.sub(0, 1), z=w); step()
        hip.dispatch("scale", x=s, alpha=0.5); step()                               # length 4, covers the scalar
        hip.dispatch("add", x=s.sub(0, 1), y=w, z=w); step()
        return [w, s]

    w, s = (x.view(np.float32) for x in both_ways(hip, body))
    np.testing.assert_array_equal(w, v0 * 2 * 4 + 2)
    np.testing.assert_array_equal(s, np.float32([2, 0, 0, 0]))


def test_long_operands_and_other_calls_between(hip):
    """Ops past the waiting length take their own launches; a call of another kind (a fill, a reduction, a read) sends
    the waiting ops out first."""
    n = 70_000
    x0 = np.linspace(0, 1, n).astype(np.float32)

    def body(step):
        x, y = hip.from_numpy(x0), hip.mem_alloc(F32, n)
        small = hip.mem_alloc(F32, 256)
        hip.dispatch("add", x=x, y=x, z=y); step()                       # too long to wait
        hip.dispatch("mul", x=y.sub(0, 256), y=y.sub(0, 256), z=small); step()
        hip.mem_fill(y.sub(0, 256), 3.0); step()                         # overwrites an operand of the waiting op
        hip.dispatch("add", x=small, y=y.sub(0, 256), z=small); step()
        total = hip.mem_alloc(F32, 1)
        hip.dispatch("sum", x=small, y=total); step()
        hip.dispatch("mul", x=small, y=total, z=small); step()
        return [y, small, total]

    y, small, total = (v.view(np.float32) for v in both_ways(hip, body))
    want_small = (2 * x0[:256]) ** 2 + 3
    np.testing.assert_array_equal(y[256:], 2 * x0[256:])
    np.testing.assert_array_equal(y[:256], np.full(256, 3, np.float32))
    np.testing.assert_allclose(total[0], want_small.sum(dtype=np.float64), rtol=1e-6)
    np.testing.assert_array_equal(small, want_small * total[0])


def test_a_run_recorded_into_a_graph_replays(hip):
    n = 512
    x0 = np.linspace(-1, 1, n).astype(np.float32)
    x, y = hip.from_numpy(x0), hip.from_numpy(np.zeros(n, np.float32))
    half = hip.from_numpy(np.float32([0.5]))

    def calls():
        t = hip.mem_cache_alloc(F32, n)
        hip.dispatch("mul", x=x, y=half, z=t)
        hip.dispatch("add", x=t, y=y, z=y)
        hip.dispatch("relu_fwd", x=y, y=y)
        hip.mem_cache_free(t)

    calls()                                   # eager once: the pool grows outside the recording
    hip.graph_open()
    calls()
    g = hip.graph_save()
    want = np.maximum(x0 * np.float32(0.5), 0)
    for k in range(2, 6):
        g.run()
        hip.sync()
        want = np.maximum(x0 * np.float32(0.5) + want, 0)
        np.testing.assert_array_equal(hip.to_numpy(y), want)
    g.free()
    for b in (x, y, half):
        hip.mem_free(b)


@pytest.mark.parametrize("value", [0.0, -0.0, 0.25])
def test_a_fill_of_exactly_the_output_is_taken_over(hip, value):
    """ensure_grad(0) followed by an accumulating backward op (src/ndtensor.zig:221-228): the op takes the fill's value
    where it would have read the output, whatever the value, and other waiting fills are left alone."""
    r = np.random.default_rng(3)
    n = 300
    x0, g0 = r.standard_normal(n).astype(np.float32), r.standard_normal(n).astype(np.float32)
    g0[::7] = -0.0
    x0[::7] = 1.0

    def body(step):
        x, yg = hip.from_numpy(x0), hip.from_numpy(g0)
        xg, other, z = hip.from_numpy(np.ones(n, np.float32)), hip.from_numpy(np.ones(n, np.float32)), hip.mem_alloc(F32, n)
        hip.mem_fill(other, 7.0); step()
        hip.mem_fill(xg, value); step()
        hip.dispatch("relu_bwd", x=x, x_g=xg, y_g=yg); step()          # xg = fill + (x > 0 ? yg : 0)
        hip.mem_fill(z, value); step()
        hip.dispatch("mul", x=x, y=yg, z=z); step()                     # overwrites the filled output
        hip.mem_fill(xg.sub(0, n // 2), value); step()                  # only part of the output: must be seen
        hip.dispatch("tanh_inplace_bwd", x=x, x_g=xg); step()
        hip.dispatch("add", x=other, y=z, z=z); step()                  # reads the fill that kept waiting
        return [xg, z, other, x, yg]

    xg, z, other = (v.view(np.float32) for v in both_ways(hip, body)[:3])
    want = np.float32(value) + np.where(x0 > 0, g0, np.float32(0))
    want[:n // 2] = np.float32(value)
    want = want * (np.float32(1) - x0 * x0)
    np.testing.assert_array_equal(xg.view(np.uint32), want.astype(np.float32).view(np.uint32))
    np.testing.assert_array_equal(other, np.full(n, 7, np.float32))
    np.testing.assert_array_equal(z, np.float32(7) + x0 * g0)


def test_max_along_over_a_filled_output(hip):
    """NDArray.max_along zero-fills its output and then writes every element (src/ndarray.zig:567): the fill is never
    launched; a fill that reaches past the output is."""
    r = np.random.default_rng(4)
    rows, cols = 64, 2
    q0 = r.standard_normal(rows * cols).astype(np.float32)

    def body(step):
        q, room = hip.from_numpy(q0), hip.from_numpy(np.full(rows + 8, -1, np.float32))
        hip.mem_fill(room.sub(0, rows), 0.0); step()
        hip.dispatch("max_along", x=q, x_shape=[rows, cols], y=room.sub(0, rows), y_shape=[rows], dim=1); step()
        first = hip.mem_alloc(F32, rows)
        hip.mem_copy(room.sub(0, rows), first); step()
        hip.mem_fill(room.sub(4, rows + 4), 2.0); step()               # sticks out of the output
        hip.dispatch("max_along", x=q, x_shape=[rows, cols], y=room.sub(0, rows), y_shape=[rows], dim=1); step()
        return [first, room, q]

    first, room = (v.view(np.float32) for v in both_ways(hip, body)[:2])
    want = q0.reshape(rows, cols).max(axis=1)
    np.testing.assert_array_equal(first, want)
    np.testing.assert_array_equal(room[:rows], want)
    np.testing.assert_array_equal(room[rows:], np.float32([2, 2, 2, 2, 2, 2, 2, 2]))


@pytest.mark.parametrize("n,nb", [(64, 128), (200, 50), (1000, 300), (5000, 20000)])
def test_scatter_add_into_a_destination_whose_zero_fill_waits(hip, n, nb):
    """GatherBwd (src/ndtensor.zig:1367-1380): the gradient is zero-filled, then scattered into; the zeros of the
    untouched elements come from the scatter's own launch.  Other fills are not taken over."""
    r = np.random.default_rng(n)
    src0 = r.standard_normal(n).astype(np.float32)
    off0 = r.integers(0, nb + nb // 8, n).astype(np.uint64)               # a few past the end: skipped

    def body(step):
        src, off = hip.from_numpy(src0), hip.from_numpy(off0)
        a, b, c = (hip.from_numpy(np.full(nb, 9, np.float32)) for _ in range(3))
        hip.mem_fill(a, 0.0); step()
        hip.dispatch("scatter_add", src=src, offsets=off, dst=a); step()
        hip.mem_fill(b, 0.5); step()
        hip.dispatch("scatter_add", src=src, offsets=off, dst=b); step()
        hip.mem_fill(c.sub(0, nb // 2), 0.0); step()
        hip.dispatch("scatter_add", src=src, offsets=off, dst=c); step()
        return [a, b, c, src, off]

    a, b, c = (v.view(np.float32) for v in both_ways(hip, body)[:3])

    def scattered(start):
        out = start.copy()
        for i in range(n):
            if off0[i] < nb:
                out[off0[i]] = np.float32(out[off0[i]] + src0[i])
        return out

    half = np.full(nb, 9, np.float32)
    half[:nb // 2] = 0
    np.testing.assert_array_equal(a, scattered(np.zeros(nb, np.float32)))
    np.testing.assert_array_equal(b, scattered(np.full(nb, 0.5, np.float32)))
    np.testing.assert_array_equal(c, scattered(half))


@pytest.mark.parametrize("rows,cols", [(64, 10), (3000, 16), (2708, 7)])
def test_a_bias_gradient_takes_over_the_zero_fill_of_zero_grad(hip, rows, cols):
    """zero_grad(), then the backward pass: the bias gradient's column sums (src/ndtensor.zig:780-796) are written
    instead of added to zeros, in the one-launch and in the two-launch form; the fills of other gradients keep waiting
    and are seen by whoever reads them."""
    from zigrad_amd import host
    r = np.random.default_rng(rows)
    g0 = r.standard_normal((rows, cols)).astype(np.float32)

    def body(step):
        g = hip.from_numpy(g0.ravel())
        gb, gb2, other = (hip.from_numpy(np.full(cols, 5, np.float32)) for _ in range(3))
        hip.mem_fill(other, 0.0); step()
        hip.mem_fill(gb, 0.0); step()
        host.unbroadcast_(hip, g, [rows, cols], gb, [cols], alpha=1.0, beta=1.0); step()
        hip.mem_fill(gb2, 0.5); step()                                   # not zero: added to
        host.unbroadcast_(hip, g, [rows, cols], gb2, [cols], alpha=1.0, beta=1.0); step()
        hip.dispatch("add", x=gb, y=other, z=other); step()
        return [gb, gb2, other, g]

    gb, gb2, other = (v.view(np.float32) for v in both_ways(hip, body)[:3])
    np.testing.assert_allclose(gb, g0.sum(axis=0, dtype=np.float64), rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(gb2, 0.5 + g0.sum(axis=0, dtype=np.float64), rtol=1e-5, atol=1e-5)
    np.testing.assert_array_equal(other, gb)


def test_a_fill_that_waits_past_a_product_is_seen_by_the_bias_row_and_the_mask_it_takes_later(hip):
    """Fills that meet none of a product's operands keep waiting while the product waits for its bias add or its mask;
    when that call names memory such a fill covers, the fill goes out first."""
    from zigrad_amd import host
    r = np.random.default_rng(9)
    B, I, O = 16, 32, 8
    x0 = r.standard_normal((B, I)).astype(np.float32)
    w0 = r.standard_normal((O, I)).astype(np.float32)
    g0 = r.standard_normal((B, O)).astype(np.float32)

    def body(step):
        x, w, g = hip.from_numpy(x0.ravel()), hip.from_numpy(w0.ravel()), hip.from_numpy(g0.ravel())
        bias, mask = hip.from_numpy(np.full(O, 3, np.float32)), hip.from_numpy(np.full(B * I, -1, np.float32))
        y, gx = hip.from_numpy(np.full(B * O, 7, np.float32)), hip.from_numpy(np.full(B * I, 7, np.float32))
        hip.mem_fill(bias, 0.5); step()                                   # waits past the product below
        hip.mem_fill(y, 0.0); step()
        host.bmm_acc_(hip, x, [B, I], w, [O, I], y, False, True, 1.0, 1.0); step()    # y = x w^T, waits for its bias
        hip.dispatch("add", x=bias, y=y, z=y); step()
        hip.mem_fill(mask, 1.0); step()                                   # waits past the product below
        hip.mem_fill(gx, 0.0); step()
        host.bmm_acc_(hip, g, [B, O], w, [O, I], gx, False, False, 1.0, 1.0); step()  # gx = g w, waits for its mask
        hip.dispatch("relu_inplace_bwd", x=mask, x_g=gx); step()
        return [y, gx, x, w, g, bias, mask]

    y, gx = (v.view(np.float32) for v in both_ways(hip, body)[:2])
    np.testing.assert_allclose(y.reshape(B, O), x0 @ w0.T + 0.5, rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(gx.reshape(B, I), g0 @ w0, rtol=1e-5, atol=1e-5)   # the mask is all ones: nothing zeroed


@pytest.mark.parametrize("n,nb", [(100, 40), (3000, 500)])
def test_scatter_add_of_a_source_whose_fill_waits(hip, n, nb):
    """Counting with a buffer of ones (the GCN's degrees, examples/gcn/src/model.zig:116-224): the source's fill need
    not be launched for the scatter, but whoever reads the source afterwards finds it filled."""
    r = np.random.default_rng(n)
    off0 = r.integers(0, nb, n).astype(np.uint64)

    def body(step):
        # the offsets in pinned host memory: from the second round on the library has their buckets, and the count
        # waits with the add and the rsqrt that follow it
        off = hip.mem_alloc_host(np.uint64, n)
        hip.mem_transfer(off0, off, "HtoD")
        ones, counts, deg = hip.from_numpy(np.full(n, 9, np.float32)), hip.from_numpy(np.full(nb, 9, np.float32)), hip.mem_alloc(F32, nb)
        later = hip.mem_alloc(F32, n)
        for _ in range(3):
            hip.mem_fill(deg, 1.0); step()
            hip.mem_fill(ones, 1.0); step()
            hip.mem_fill(counts, 0.0); step()
            hip.dispatch("scatter_add", src=ones, offsets=off, dst=counts); step()
            hip.dispatch("add", x=counts, y=deg, z=deg); step()
            hip.dispatch("rsqrt_fwd", x=deg, y=deg, eps=1e-12); step()
            hip.dispatch("scale", x=ones, alpha=3.0); step()            # reads the source after all
            hip.mem_copy(ones, later); step()
        return [deg, counts, later, ones, off]

    deg, counts, later = (v.view(np.float32) for v in both_ways(hip, body)[:3])
    want = np.bincount(off0.astype(np.int64), minlength=nb).astype(np.float32)
    np.testing.assert_array_equal(counts, want)
    np.testing.assert_allclose(deg, 1 / np.sqrt(1 + want.astype(np.float64)), rtol=1e-6)
    np.testing.assert_array_equal(later, np.full(n, 3, np.float32))


@pytest.mark.parametrize("total,off,n", [(18956, 0, 980), (5000, 1234, 77), (300, 299, 1), (4096, 0, 4096)])
def test_rows_copied_into_a_gradient_whose_zero_fill_waits(hip, total, off, n):
    """MaskLayer.backward (examples/gcn/src/model.zig:343-348): the full gradient is zero-filled, then the labelled rows
    are copied into it; fill and copy leave in one launch, and a fill that waits elsewhere is left alone."""
    r = np.random.default_rng(total)
    rows0 = r.standard_normal(n).astype(np.float32)

    def body(step):
        rows, full, other = hip.from_numpy(rows0), hip.from_numpy(np.full(total, 9, np.float32)), hip.mem_alloc(F32, 64)
        hip.mem_fill(other, 2.0); step()
        hip.mem_fill(full, 0.0); step()
        hip.mem_copy(rows, full.sub(off, n)); step()
        hip.dispatch("scale", x=full, alpha=2.0); step()
        return [full, other, rows]

    full, other = (v.view(np.float32) for v in both_ways(hip, body)[:2])
    want = np.zeros(total, np.float32)
    want[off:off + n] = rows0
    np.testing.assert_array_equal(full, want * 2)
    np.testing.assert_array_equal(other, np.full(64, 2, np.float32))
