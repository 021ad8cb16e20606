"""The library's caching allocator through the C ABI (the counterpart of src/allocators/caching_allocator.zig:15-162
and block_pool.zig:103-412): no two live blocks overlap, neighbours fuse, the working set of a loop is served without
new device allocations, and memory named by a recorded execution graph stays out of circulation."""
from __future__ import annotations

import numpy as np
import pytest

from zigrad_amd import HipDevice
from zigrad_amd._lib import ZgHipError
from zigrad_amd.device import F32

pytestmark = pytest.mark.gpu


def test_random_alloc_free_never_overlaps_and_keeps_contents(hip):
    r = np.random.default_rng(3)
    live = []  # (buffer, tag)
    for it in range(3000):
        if live and (r.random() < 0.45 or len(live) > 200):
            buf, tag = live.pop(int(r.integers(len(live))))
            got = hip.to_numpy(buf)
            assert np.all(got == np.float32(tag)), (it, tag)  # nobody else wrote into the block while it was live
            hip.mem_cache_free(buf)
        else:
            n = int(r.integers(1, 70000)) if r.random() < 0.9 else int(r.integers(1 << 18, 1 << 20))
            buf = hip.mem_cache_alloc(F32, n)
            assert buf.ptr % 256 == 0 and buf.block != 0
            hip.mem_fill(buf, float(it))
            live.append((buf, it))
    spans = sorted((b.ptr, b.ptr + b.nbytes) for b, _ in live)
    for (_, hi), (lo, _) in zip(spans, spans[1:]):
        assert hi <= lo
    for buf, tag in live:
        assert np.all(hip.to_numpy(buf) == np.float32(tag))
        hip.mem_cache_free(buf)


def test_stale_and_foreign_handles_are_refused(hip):
    a = hip.mem_cache_alloc(F32, 100)
    ptr, block = a.ptr, a.block
    hip.mem_cache_free(a)
    for p, b in ((ptr, block), (ptr, 1), (ptr + 256, block), (12345, 0xdeadbeef)):
        with pytest.raises(ZgHipError) as e:
            hip._call("zg_hip_mem_cache_free", p, b)
        assert e.value.code == 1


def test_is_device_ptr(hip):
    c = hip.mem_cache_alloc(F32, 1000)
    raw = hip.mem_alloc(F32, 1000)
    s = hip.mem_scratch(F32, 64)
    host = np.zeros(4, np.float32)
    pinned = hip.mem_alloc_host(F32, 16)
    assert hip.is_device_ptr(c.ptr) and hip.is_device_ptr(c.ptr + 3996)
    assert hip.is_device_ptr(raw.ptr) and hip.is_device_ptr(raw.ptr + 3996) and not hip.is_device_ptr(raw.ptr + 4000)
    assert hip.is_device_ptr(s.ptr)
    assert not hip.is_device_ptr(host.ctypes.data)  # a host stack / heap scalar, as add_scalar passes (src/ndarray.zig:251)
    assert not hip.is_device_ptr(pinned.ptr)
    assert not hip.is_device_ptr(0)
    hip.mem_cache_free(c)
    hip.mem_free(raw)
    hip.mem_free(pinned)


def test_recording_reuses_blocks_freed_in_the_same_recording():
    """A recorded sequence whose allocations add up to four times the pool's segment but peak at one block: blocks
    freed while recording serve later allocations of the same recording, so the pool does not have to grow (it
    could not: growing is refused while recording).  After the recording the graph keeps the memory it names:
    eager allocations get other addresses, replays still compute the right values."""
    dev = HipDevice(0)
    try:
        seg = 8 << 20
        dev.cache_configure(1 << 20, seg)
        n = (5 << 20) // 4  # 5 MiB blocks: two do not fit one 8 MiB segment
        result = dev.mem_cache_alloc(F32, 4)
        dev.mem_fill(result, 0.0)

        def sequence():
            for k in range(4):
                t = dev.mem_cache_alloc(F32, n)
                dev.mem_fill(t, float(k + 1))
                dev.dispatch("sum", x=t, y=result.sub(k, 1))
                dev.mem_cache_free(t)

        sequence()  # eager warm-up: workspace and pool reach their final size
        dev.sync()
        allocs = dev.cache_stats()["n_device_allocs"]
        in_use = dev.cache_stats()["bytes_in_use"]
        dev.graph_open()
        sequence()
        g = dev.graph_save()
        assert dev.cache_stats()["n_device_allocs"] == allocs
        held = dev.cache_stats()["bytes_in_use"] - in_use
        assert 5 << 20 <= held < 8 << 20  # one block's worth stays with the graph, not four
        # an eager allocation of the same size must not land on the graph's memory: the segment has no room left
        # beside the held block, so the pool grows
        other = dev.mem_cache_alloc(F32, n)
        assert dev.cache_stats()["n_device_allocs"] == allocs + 1
        dev.mem_fill(other, -1.0)
        for _ in range(3):
            dev.mem_fill(result, 0.0)
            g.run()
            dev.sync()
            np.testing.assert_array_equal(dev.to_numpy(result), np.float32(n) * np.arange(1, 5, dtype=np.float32))
            assert np.all(dev.to_numpy(other) == -1.0)
        g.free()
        dev.mem_cache_free(other)
        assert dev.cache_stats()["bytes_in_use"] == in_use
        dev.mem_cache_free(result)
    finally:
        dev.deinit()


def test_scratch_may_grow_while_a_graph_is_alive(hip):
    s0 = hip.mem_scratch(F32, 256)
    x = hip.from_numpy(np.ones(256, np.float32), cached=True)
    hip.sync()
    hip.graph_open()
    hip.dispatch("add", x=x, y=x, z=s0)
    g = hip.graph_save()
    bigger = hip.mem_scratch(F32, (hip.cache_stats()["bytes_mapped"] // 4) + (1 << 20))  # forces growth
    assert bigger.ptr != 0
    g.run()  # still writes the old buffer, which must still exist
    hip.sync()
    g.free()
    hip.mem_cache_free(x)


def test_pinned_host_blocks_are_kept_and_reused_in_stream_order(hip):
    """A binding serves every `usize` tensor from pinned host memory (the reference's callers fill index tensors with
    host loops, src/ndarray.zig:607-624): a block given back is handed out again for the same size class, the next
    owner's host writes cannot reach a kernel that was queued before the block was given back, and every take reads the
    indices its own call was given."""
    U64 = np.uint64
    n, m = 3000, 50000
    src0 = np.arange(m, dtype=np.float32) * 0.5
    src = hip.from_numpy(src0)
    r = np.random.default_rng(9)
    seen, outs, wants = set(), [], []
    for it in range(40):
        idx = hip.mem_alloc_host(U64, n)
        seen.add(idx.ptr)
        want = r.integers(0, m, n).astype(U64)
        hip.host_view(idx)[:] = want            # a host loop writes the indices
        out = hip.mem_alloc(F32, n)
        hip.mem_take(src, idx, out)             # queued, not waited for
        hip.mem_free(idx)                       # given back while the kernel may still be running
        outs.append(out)
        wants.append(want)
    assert len(seen) <= 2, "blocks of one size class are reused, not obtained from the driver every time"
    for out, want in zip(outs, wants):
        np.testing.assert_array_equal(hip.to_numpy(out), src0[want])
        hip.mem_free(out)
    # another size class does not get the kept block; a larger request than the block's class neither
    a = hip.mem_alloc_host(U64, 8)
    b = hip.mem_alloc_host(U64, n * 4)
    assert a.ptr not in seen and b.ptr not in seen
    hip.mem_free(a)
    hip.mem_free(b)
    hip.mem_free(src)
    with pytest.raises(ZgHipError):
        hip._call("zg_hip_host_free", 12345)    # not a pointer of this context
