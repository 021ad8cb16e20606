"""scatter_add_csr and segment_sum_csr (src/device/host_device.zig:1325-1353): the oracle against the definition
written out in numpy (CPU), the device against the oracle (GPU).  Empty segments, one long segment, boundaries that
stop short of the end of the data."""
from __future__ import annotations

import numpy as np
import pytest

from conftest import run_op


def _cases():
    r = np.random.default_rng(11)
    for n_seg, max_len in [(1, 5), (7, 0), (50, 9), (300, 40), (5, 20000), (2000, 3)]:
        lens = r.integers(0, max_len + 1, n_seg)
        if max_len == 20000:
            lens[2] = 70001  # one segment far longer than a wave's trip
        row_ptr = np.concatenate([[0], np.cumsum(lens)]).astype(np.uint64)
        total = int(row_ptr[-1])
        yield n_seg, row_ptr, total, r


def _check(dev, exact):
    for n_seg, row_ptr, total, r in _cases():
        src = r.standard_normal(n_seg).astype(np.float32)
        dst0 = r.standard_normal(total + 3).astype(np.float32)  # three elements past the last boundary stay as they are
        got = run_op(dev, "scatter_add_csr", {"src": src, "row_ptr": row_ptr, "dst": dst0.copy()}, ["dst"])["dst"]
        want = dst0.copy()
        for i in range(n_seg):
            want[int(row_ptr[i]): int(row_ptr[i + 1])] += src[i]
        assert np.array_equal(got, want), n_seg
        data = r.standard_normal(total + 2).astype(np.float32)[: max(total, 1)]
        if total == 0:
            data = np.zeros(1, np.float32)
        got = run_op(dev, "segment_sum_csr", {"src": data, "row_offsets": row_ptr, "dst": np.full(n_seg, np.nan, np.float32)},
                     ["dst"])["dst"]
        want = np.array([data[int(row_ptr[i]): int(row_ptr[i + 1])].astype(np.float64).sum() for i in range(n_seg)])
        scale = np.array([np.abs(data[int(row_ptr[i]): int(row_ptr[i + 1])]).astype(np.float64).sum() for i in range(n_seg)])
        assert np.all(np.abs(got - want) <= 1e-5 * scale + 1e-30), n_seg
        if exact:  # integer-valued data sum exactly in any order
            ints = r.integers(-8, 9, data.size).astype(np.float32)
            got = run_op(dev, "segment_sum_csr", {"src": ints, "row_offsets": row_ptr, "dst": np.zeros(n_seg, np.float32)},
                         ["dst"])["dst"]
            want = np.array([ints[int(row_ptr[i]): int(row_ptr[i + 1])].sum() for i in range(n_seg)], np.float32)
            assert np.array_equal(got, want), n_seg


def test_oracle_csr_ops_match_the_definition(oracle):
    _check(oracle, exact=True)


@pytest.mark.gpu
def test_device_csr_ops_match_the_definition(hip):
    _check(hip, exact=True)
