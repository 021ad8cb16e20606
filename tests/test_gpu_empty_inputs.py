"""Empty operands.  The host's loops over no elements do nothing, and its BLAS calls on no elements return zero
(src/device/host_device.zig:224, :315-331, :975-1019; src/nn/loss.zig:157-171): every op of the surface is called with
empty operands on the oracle and on the HIP device, outputs that have elements must come out equal and nothing else
may be touched.  What the reference leaves undefined on empty input (an axis of length zero under a reduction, the
mean of no elements, the maximum of nothing) is refused with an error instead."""
from __future__ import annotations

import numpy as np
import pytest

from conftest import run_op
from zigrad_amd import ZgHipError

pytestmark = pytest.mark.gpu


def f0():
    return np.zeros(0, np.float32)


def u0():
    return np.zeros(0, np.uint64)


def full(n, v):
    return np.full(n, v, np.float32)


CASES = {
    "add": ("add", dict(x=f0(), y=f0(), z=f0())),
    "sub": ("sub", dict(x=f0(), y=f0(), z=f0())),
    "mul": ("mul", dict(x=f0(), y=f0(), z=f0())),
    "div": ("div", dict(x=f0(), y=f0(), z=f0())),
    "add_scalar_lhs": ("add", dict(x=full(1, 2.0), y=f0(), z=f0())),
    "mul_scalar_rhs": ("mul", dict(x=f0(), y=full(1, 2.0), z=f0())),
    "dot": ("dot", dict(x=f0(), y=f0(), z=full(1, 7.0))),
    "sum": ("sum", dict(x=f0(), y=full(1, 7.0))),
    "nrm2": ("nrm2", dict(x=f0(), y=full(1, 7.0))),
    "scale": ("scale", dict(x=f0(), alpha=2.0)),
    "clip_nrm2": ("clip_nrm2", dict(x=f0(), max_norm=1.0, delta=1e-6)),
    "axpy": ("axpy", dict(x=f0(), y=f0(), alpha=2.0)),
    "matmul_k0": ("matmul", dict(A=f0(), B=f0(), C=full(6, 2.0), m=2, n=3, k=0, trans_a=False, trans_b=False, lda=1,
                                 ldb=3, ldc=3, alpha=1.0, beta=0.5)),
    "matmul_m0": ("matmul", dict(A=f0(), B=full(6, 1.0), C=f0(), m=0, n=3, k=2, trans_a=False, trans_b=False, lda=2,
                                 ldb=3, ldc=3, alpha=1.0, beta=0.0)),
    "transpose": ("transpose", dict(A=f0(), B=f0(), m=0, n=0, alpha=0.0)),
    "relu_fwd": ("relu_fwd", dict(x=f0(), y=f0())),
    "relu_bwd": ("relu_bwd", dict(x=f0(), x_g=f0(), y_g=f0())),
    "relu_inplace_bwd": ("relu_inplace_bwd", dict(x=f0(), x_g=f0())),
    "tanh_fwd": ("tanh_fwd", dict(x=f0(), y=f0())),
    "tanh_bwd": ("tanh_bwd", dict(x_g=f0(), y=f0(), y_g=f0())),
    "sigm_fwd": ("sigm_fwd", dict(x=f0(), y=f0())),
    "sigm_bwd": ("sigm_bwd", dict(x_g=f0(), y=f0(), y_g=f0())),
    "exp_fwd": ("exp_fwd", dict(x=f0(), y=f0())),
    "exp_bwd": ("exp_bwd", dict(x_g=f0(), y=f0(), y_g=f0())),
    "pow_fwd": ("pow_fwd", dict(x=f0(), exp=2.0, y=f0())),
    "pow_bwd": ("pow_bwd", dict(x=f0(), x_g=f0(), exp=2.0, y_g=f0(), eps=1e-6)),
    "sqrt_fwd": ("sqrt_fwd", dict(x=f0(), y=f0())),
    "sqrt_bwd": ("sqrt_bwd", dict(x=f0(), x_g=f0(), y_g=f0(), eps=1e-6)),
    "rsqrt_fwd": ("rsqrt_fwd", dict(x=f0(), y=f0(), eps=1e-6)),
    "rsqrt_bwd": ("rsqrt_bwd", dict(x=f0(), x_g=f0(), y_g=f0(), eps=1e-6)),
    "clamp_fwd": ("clamp_fwd", dict(x=f0(), y=f0(), min=-1.0, max=1.0)),
    "clamp_bwd": ("clamp_bwd", dict(x=f0(), x_g=f0(), y_g=f0(), min=-1.0, max=1.0)),
    "scatter_add": ("scatter_add", dict(src=f0(), offsets=u0(), dst=full(5, 1.0))),
    "index_select_fwd": ("index_select_fwd", dict(src=full(8, 1.0), indices=u0(), stride=2, dst=f0())),
    "index_select_bwd": ("index_select_bwd", dict(y_grad=f0(), indices=u0(), stride=2, x_grad=full(8, 1.0))),
    "scatter_gcn": ("scatter_gcn_deg_scaled", dict(dst=full(8, 1.0), h=full(8, 1.0), deg=full(4, 1.0), src_indices=u0(),
                                                   tgt_indices=u0(), stride=2, n_edge=0)),
    "scatter_gcn_bwd": ("scatter_gcn_deg_scaled_bwd", dict(grad_output=full(8, 1.0), h=full(8, 1.0), deg=full(4, 1.0),
                                                           src_indices=u0(), tgt_indices=u0(), grad_h=full(8, 1.0),
                                                           grad_deg=full(4, 1.0), stride=2, n_edge=0)),
    "smooth_l1_bwd": ("smooth_l1_bwd", dict(pred=f0(), target=f0(), grad=f0(), beta=1.0)),
    "mse_bwd": ("mse_bwd", dict(pred=f0(), target=f0(), grad=f0())),
    "smce_bwd": ("smce_bwd", dict(probs=f0(), target=f0(), grad=f0(), rows=0, cols=4)),
    "softmax_fwd": ("softmax_fwd", dict(x=f0(), y=f0(), rows=0, cols=4)),
    "softmax_bwd": ("softmax_bwd", dict(y=f0(), y_g=f0(), x_g=f0(), rows=0, cols=4)),
    "sgd_step": ("sgd_step", dict(param=f0(), grad=f0(), lr=0.1, clip=True, max_norm=1.0, delta=1e-6)),
    "adam_step": ("adam_step", dict(param=f0(), grad=f0(), m=f0(), v=f0(), t=1, lr=0.1, beta1=0.9, beta2=0.999,
                                    epsilon=1e-8, clip=True, max_norm=1.0, delta=1e-6)),
}


def _copy(p):
    return {k: (v.copy() if isinstance(v, np.ndarray) else v) for k, v in p.items()}


@pytest.mark.parametrize("case", sorted(CASES))
def test_empty_operands_do_what_the_host_loops_do(oracle, hip, case):
    name, p = CASES[case]
    outs = [k for k, v in p.items() if isinstance(v, np.ndarray) and v.dtype == np.float32]
    want = run_op(oracle, name, _copy(p), outs)
    got = run_op(hip, name, _copy(p), outs)
    for k in outs:
        np.testing.assert_array_equal(got[k], want[k], err_msg=f"{case}: {k}")


def test_empty_calls_leave_waiting_work_alone(hip):
    """A call with nothing to do between a fill and the op that takes the fill over: the values are those of the calls
    without it."""
    x = hip.from_numpy(np.arange(8, dtype=np.float32))
    e = hip.mem_alloc(np.float32, 0)
    hip.mem_fill(x, 0.5)
    hip.dispatch("add", x=e, y=e, z=e)
    hip.dispatch("smce_bwd", probs=e, target=e, grad=e, rows=0, cols=3)
    hip.dispatch("relu_fwd", x=x, y=x)
    assert np.all(hip.to_numpy(x) == 0.5)
    hip.mem_free(x)


REFUSED = {
    "sum_along_over_no_rows": ("sum_along", dict(x=f0(), x_shape=[0, 4], y=full(4, 3.0), dim=0, alpha=1.0, beta=0.0)),
    "max_along_over_no_columns": ("max_along", dict(x=f0(), x_shape=[4, 0], y=full(4, 3.0), dim=1)),
    "max_fwd_of_nothing": ("max_fwd", dict(x=f0(), y=full(1, 3.0))),
    "mse_of_nothing": ("mse_fwd", dict(pred=f0(), target=f0(), loss=full(1, 3.0))),
    "smooth_l1_of_nothing": ("smooth_l1_fwd", dict(pred=f0(), target=f0(), beta=1.0, loss=full(1, 3.0))),
    "smce_over_no_rows": ("smce_fwd", dict(logits=f0(), target=f0(), probs=f0(), loss=full(1, 3.0), rows=0, cols=4)),
    "add_empty_to_longer": ("add", dict(x=f0(), y=full(4, 1.0), z=full(4, 3.0))),
}


@pytest.mark.parametrize("case", sorted(REFUSED))
def test_what_the_reference_leaves_undefined_on_empty_input_is_refused(hip, case):
    name, p = REFUSED[case]
    outs = [k for k, v in p.items() if isinstance(v, np.ndarray) and v.size]
    bufs = {k: hip.from_numpy(v) if isinstance(v, np.ndarray) else v for k, v in p.items()}
    with pytest.raises(ZgHipError):
        hip.dispatch(name, **bufs)
    hip.sync()
    for k in outs:       # and nothing was written
        np.testing.assert_array_equal(hip.to_numpy(bufs[k]), p[k])
    for v in bufs.values():
        if not isinstance(v, (int, float, bool, list)):
            hip.mem_free(v)
