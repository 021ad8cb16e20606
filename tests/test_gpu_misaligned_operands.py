"""Every op with every operand starting 4, 8 and 12 bytes past a 16-byte boundary (sub-slices by pointer arithmetic are
legal everywhere in the reference, src/ndtensor.zig:581, :1462-1464): the values are those of the oracle on the same
data, and the elements either side of each operand stay what they were."""
from __future__ import annotations

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

r = np.random.default_rng(0)
GUARD = 77


def run_offset(dev, name, params, outs, k):
    """Dispatch with every array operand at offset k inside a longer buffer; returns (outputs, guards intact)."""
    bufs, kw, base = {}, {}, []
    for key, v in params.items():
        if isinstance(v, np.ndarray):
            padded = np.concatenate([np.full(k, GUARD, v.dtype), v.ravel(), np.full(3, GUARD, v.dtype)])
            b = dev.from_numpy(padded)
            base.append((b, v.size))
            bufs[key] = b.sub(k, v.size)
            kw[key] = bufs[key]
        else:
            kw[key] = v
    dev.dispatch(name, **kw)
    dev.sync()
    out = {o: dev.to_numpy(bufs[o]).reshape(params[o].shape) for o in outs}
    intact = True
    for b, n in base:
        full = dev.to_numpy(b)
        intact = intact and bool(np.all(full[:k] == GUARD) and np.all(full[k + n:] == GUARD))
        dev.mem_free(b)
    return out, intact


def f(*s):
    return r.standard_normal(s).astype(np.float32)


def pos(*s):
    return (np.abs(r.standard_normal(s)) + 0.1).astype(np.float32)


def idx(hi, n):
    return r.integers(0, hi, n).astype(np.uint64)


def _matmul(m, n, k, ta, tb, alpha, beta):
    return ("matmul", dict(A=f(m * k), B=f(n * k), C=f(m * n), m=m, n=n, k=k, trans_a=ta, trans_b=tb, lda=m if ta else k,
                           ldb=k if tb else n, ldc=n, alpha=alpha, beta=beta), ["C"])


def _adam(n):
    return ("adam_step", dict(param=f(n), grad=f(n), m=f(n), v=pos(n), t=3, lr=0.1, beta1=0.9, beta2=0.999, epsilon=1e-8,
                              clip=True, max_norm=1.0, delta=1e-6), ["param", "grad", "m", "v"])


def _smce(rows, cols):
    return ("smce_fwd", dict(logits=f(rows * cols), target=np.eye(rows, cols, dtype=np.float32).ravel(),
                             probs=f(rows * cols), loss=f(1), rows=rows, cols=cols), ["probs", "loss"])


R, C = 33, 71
CASES = [
    ("add", dict(x=f(1000), y=f(1000), z=f(1000)), ["z"]),
    ("mul", dict(x=f(50), y=f(1000), z=f(1000)), ["z"]),
    ("sub", dict(x=f(1000), y=f(1), z=f(1000)), ["z"]),
    ("relu_fwd", dict(x=f(1000), y=f(1000)), ["y"]),
    ("tanh_bwd", dict(x_g=f(1000), y=f(1000), y_g=f(1000)), ["x_g"]),
    ("sqrt_fwd", dict(x=pos(1000), y=f(1000)), ["y"]),
    ("sum", dict(x=f(5000), y=f(1)), ["y"]),
    ("nrm2", dict(x=f(5000), y=f(1)), ["y"]),
    ("dot", dict(x=f(5000), y=f(5000), z=f(1)), ["z"]),
    ("max_fwd", dict(x=f(5000), y=f(1)), ["y"]),
    ("nrm2", dict(x=f(300000), y=f(1)), ["y"]),             # the two-launch form
    ("sum", dict(x=f(300000), y=f(1)), ["y"]),
    ("scale", dict(x=f(5000), alpha=0.5), ["x"]),
    ("clip_nrm2", dict(x=f(5000), max_norm=1.0, delta=1e-6), ["x"]),
    ("axpy", dict(x=f(5000), y=f(5000), alpha=0.5), ["y"]),
    ("sum_along", dict(x=f(R * C), x_shape=[R, C], y=f(C), dim=0, alpha=1.0, beta=0.5), ["y"]),
    ("sum_along", dict(x=f(R * C), x_shape=[R, C], y=f(R), dim=1, alpha=1.0, beta=0.5), ["y"]),
    ("sum_along", dict(x=f(2000 * 260), x_shape=[2000, 260], y=f(260), dim=0, alpha=1.0, beta=0.0), ["y"]),
    ("sum_along", dict(x=f(2000 * 260), x_shape=[2000, 260], y=f(2000), dim=1, alpha=1.0, beta=0.0), ["y"]),
    ("max_along", dict(x=f(R * C), x_shape=[R, C], y=f(R), dim=1), ["y"]),
    ("max_along", dict(x=f(R * C), x_shape=[R, C], y=f(C), dim=0), ["y"]),
    _matmul(37, 29, 45, False, True, 1.0, 0.5),             # the unstaged kernel
    _matmul(300, 260, 500, False, False, 1.0, 0.0),         # the staged kernels, edge tiles
    _matmul(300, 260, 500, True, True, 1.0, 1.0),
    _matmul(64, 128, 784, False, True, 1.0, 0.0),           # the one-launch kernel for deep products
    ("matvec", dict(A=f(R * C), x=f(C), y=f(R), m=R, n=C, trans_a=False, alpha=1.0, beta=0.5), ["y"]),
    ("matvec", dict(A=f(R * C), x=f(R), y=f(C), m=R, n=C, trans_a=True, alpha=1.0, beta=0.5), ["y"]),
    ("outer", dict(x=f(R), y=f(C), A=f(R * C), alpha=0.5), ["A"]),
    ("transpose", dict(A=f(R * C), B=f(R * C), m=R, n=C, alpha=1.0), ["B"]),
    ("softmax_fwd", dict(x=f(R * C), y=f(R * C), rows=R, cols=C), ["y"]),
    ("softmax_fwd", dict(x=f(1100 * 300), y=f(1100 * 300), rows=1100, cols=300), ["y"]),     # a wave per row
    ("softmax_fwd", dict(x=f(5 * 5000), y=f(5 * 5000), rows=5, cols=5000), ["y"]),           # a workgroup per row
    _smce(R, C),
    _smce(1100, 300),
    ("smce_bwd", dict(probs=pos(R * C), target=np.eye(R, C, dtype=np.float32).ravel(), grad=f(R * C), rows=R, cols=C),
     ["grad"]),
    ("smce_label_fwd", dict(logits=f(R * C), labels=idx(C, R), lse=f(R), loss=f(1), rows=R, cols=C), ["lse", "loss"]),
    ("smooth_l1_fwd", dict(pred=f(500), target=f(500), beta=1.0, loss=f(1)), ["loss"]),
    ("smooth_l1_bwd", dict(pred=f(500), target=f(500), grad=f(500), beta=1.0), ["grad"]),
    ("mse_fwd", dict(pred=f(500), target=f(500), loss=f(1)), ["loss"]),
    ("sgd_step", dict(param=f(5000), grad=f(5000), lr=0.1, clip=True, max_norm=1.0, delta=1e-6), ["param", "grad"]),
    _adam(5000),
    _adam(200000),
    ("scatter_add", dict(src=f(3000), offsets=idx(100, 3000), dst=f(100)), ["dst"]),
    ("index_select_fwd", dict(src=f(50 * 12), indices=idx(50, 40), stride=12, dst=f(40 * 12)), ["dst"]),
    ("index_select_bwd", dict(y_grad=f(40 * 12), indices=idx(50, 40), stride=12, x_grad=f(50 * 12)), ["x_grad"]),
    ("scatter_gcn_deg_scaled", dict(dst=f(30 * 8), h=f(30 * 8), deg=pos(30), src_indices=idx(30, 200),
                                    tgt_indices=idx(30, 200), stride=8, n_edge=200), ["dst"]),
]


@pytest.mark.parametrize("k", [1, 2, 3])
@pytest.mark.parametrize("i", range(len(CASES)))
def test_operands_at_any_four_byte_alignment(oracle, hip, i, k):
    name, p, outs = CASES[i]
    copy = lambda: {key: (v.copy() if isinstance(v, np.ndarray) else v) for key, v in p.items()}
    want, _ = run_offset(oracle, name, copy(), outs, 0)
    got, intact = run_offset(hip, name, copy(), outs, k)
    assert intact, f"{name}: wrote outside an operand"
    for o in outs:
        err = np.linalg.norm(got[o].astype(np.float64) - want[o]) / (np.linalg.norm(want[o]) + 1e-30)
        assert err <= 1e-5, (name, o, err)
