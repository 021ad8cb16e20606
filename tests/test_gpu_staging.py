"""Input staging: batches uploaded from pinned host memory on the copy stream while the previous step computes
must give exactly the run that uploads every batch with the reference's blocking transfer."""
from __future__ import annotations

import numpy as np
import pytest

from zigrad_amd._lib import ZgHipError
from zigrad_amd.device import F32, U64
from zigrad_amd.trainers import BatchStager, MLPTrainer, mlp_inputs

pytestmark = pytest.mark.gpu


def test_double_buffered_batches_equal_blocking_uploads(hip):
    dims, batch, n_steps = [256, 512, 128, 16], 512, 12
    params, _, _, _ = mlp_inputs(dims, batch)
    batches = [mlp_inputs(dims, batch, seed_data=100 + i)[1:] for i in range(4)]  # (x, onehot, labels)

    def make():
        tr = MLPTrainer(hip, dims, batch, optimizer="adam", lr=1e-3, clip=True)
        tr.load_params(params)
        return tr

    ref = make()
    want = []
    for k in range(n_steps):
        ref.set_batch(*batches[k % 4])
        want.append(ref.step())

    tr = make()
    own = (tr.x, tr.onehot, tr.labels)
    st = BatchStager(hip, [(F32, batch * dims[0]), (F32, batch * dims[-1]), (U64, batch)])
    st.upload_first(batches[0])
    got = []
    for k in range(n_steps):
        tr.use_batch(*st.current())
        st.prefetch(batches[(k + 1) % 4])
        got.append(tr.step())
        st.advance()
    assert got == want
    for p, q in zip(ref.param_buffers(), tr.param_buffers()):
        assert np.array_equal(hip.to_numpy(p), hip.to_numpy(q))
    tr.use_batch(*own)
    st.free()


def test_staged_batches_hold_the_host_bytes_and_train_like_the_oracle(hip, oracle):
    """What the copy stream delivers is compared with the host arrays themselves, and the staged run's losses with
    the CPU oracle's for the same batch sequence (1e-4), so an error common to both upload paths cannot pass."""
    dims, batch, n_steps = [128, 192, 64, 10], 96, 8
    params, _, _, _ = mlp_inputs(dims, batch)
    batches = [mlp_inputs(dims, batch, seed_data=200 + i)[1:] for i in range(3)]

    ref = MLPTrainer(oracle, dims, batch, optimizer="adam", lr=1e-3, clip=True)
    ref.load_params(params)
    want = []
    for k in range(n_steps):
        ref.set_batch(*batches[k % 3])
        want.append(ref.step())

    tr = MLPTrainer(hip, dims, batch, optimizer="adam", lr=1e-3, clip=True)
    tr.load_params(params)
    own = (tr.x, tr.onehot, tr.labels)
    st = BatchStager(hip, [(F32, batch * dims[0]), (F32, batch * dims[-1]), (U64, batch)])
    st.upload_first(batches[0])
    got = []
    for k in range(n_steps):
        cur = st.current()
        tr.use_batch(*cur)
        st.prefetch(batches[(k + 1) % 3])
        got.append(tr.step())
        for buf, host in zip(cur, batches[k % 3]):   # the slot the step just used still holds batch k, bit for bit
            assert np.array_equal(hip.to_numpy(buf), np.asarray(host).reshape(-1))
        st.advance()
    for w, g in zip(want, got):
        assert abs(w - g) <= 1e-4 * max(1.0, abs(w)), (want, got)
    for p, q in zip(ref.param_buffers(), tr.param_buffers()):
        a, b = oracle.to_numpy(p).astype(np.float64), hip.to_numpy(q).astype(np.float64)
        assert np.linalg.norm(a - b) <= 1e-4 * np.linalg.norm(a)
    tr.use_batch(*own)
    st.free()


def test_staged_copy_moves_exactly_the_bytes_asked_for(hip):
    """zg_hip_staged_h2d copies `bytes` bytes and nothing after them (guard values either side stay)."""
    n = 1000
    dst = hip.mem_alloc(F32, n + 64)
    hip.mem_transfer(np.full(n + 64, -7.0, np.float32), dst, "HtoD")
    pinned = hip.mem_alloc_host(F32, n)
    src = np.arange(n, dtype=np.float32) * 0.5 + 1.0
    hip.host_view(pinned)[:] = src
    hip.sync()
    hip._call("zg_hip_staged_h2d", dst.ptr + 32 * 4, pinned.ptr, 4 * (n - 100))
    hip.compute_after_staging()
    out = hip.to_numpy(dst)
    assert np.array_equal(out[32:32 + n - 100], src[:n - 100])
    assert np.all(out[:32] == -7.0) and np.all(out[32 + n - 100:] == -7.0)
    hip.staging_wait()
    hip.mem_free(dst)
    hip.mem_free(pinned)


def test_staged_copy_needs_a_pinned_source(hip):
    dst = hip.mem_alloc(F32, 16)
    src = hip.mem_alloc(F32, 16)  # device memory, not pinned host memory
    with pytest.raises(ValueError):
        hip.staged_h2d(src, dst)
    pinned = hip.mem_alloc_host(F32, 16)
    hip.host_view(pinned)[:] = np.arange(16, dtype=np.float32)
    hip.staged_h2d(pinned, dst)
    hip.compute_after_staging()
    assert np.array_equal(hip.to_numpy(dst), np.arange(16, dtype=np.float32))
    # the C entry point itself refuses a source outside zg_hip_host_alloc memory
    with pytest.raises(ZgHipError):
        hip._call("zg_hip_staged_h2d", dst.ptr, src.ptr, 64)
    hip.staging_wait()
    for b in (dst, src, pinned):
        hip.mem_free(b)
