"""Shared fixtures.  GPU tests are marked `gpu`; everything else runs on the CPU only."""
from __future__ import annotations

import sys
from pathlib import Path

import numpy as np
import pytest

ROOT = Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def oracle():
    from oracle.oracle_device import OracleDevice

    return OracleDevice()


@pytest.fixture(scope="session")
def hip():
    """The HIP device.  Fails (does not skip) when the library is missing or no GPU answers:
    a GPU test that silently ran on something else would prove nothing."""
    from zigrad_amd import HipDevice

    dev = HipDevice(0)
    yield dev
    dev.deinit()


def run_op(dev, name, params, outputs):
    """Dispatch `name` on `dev`.  `params` maps opspec field names to numpy arrays (uploaded as buffers),
    or plain scalars / lists (passed through).  Returns {output name: numpy array read back}."""
    bufs, kw = {}, {}
    for k, v in params.items():
        if isinstance(v, np.ndarray):
            # aliases: the same array object passed under two names shares one buffer
            for k2, b2 in bufs.items():
                if params[k2] is v:
                    bufs[k] = b2
                    break
            else:
                bufs[k] = dev.from_numpy(v)
            kw[k] = bufs[k]
        else:
            kw[k] = v
    dev.dispatch(name, **kw)
    dev.sync()
    out = {o: dev.to_numpy(bufs[o]).reshape(params[o].shape) for o in outputs}
    seen = set()
    for b in bufs.values():
        if id(b) not in seen:
            seen.add(id(b))
            dev.mem_free(b)
    return out


def rel_fro(a, b):
    a = np.asarray(a, dtype=np.float64).ravel()
    b = np.asarray(b, dtype=np.float64).ravel()
    d = np.linalg.norm(a - b)
    n = np.linalg.norm(b)
    return d / n if n > 0 else d
