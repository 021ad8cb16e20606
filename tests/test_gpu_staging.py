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
