"""OracleDevice -- TEST INFRASTRUCTURE ONLY.

Presents the CPU oracle (oracle/libzg_oracle.so, the C restatement of Zigrad's HostDevice) behind the
same `dispatch` / `mem_*` interface as zigrad_amd.HipDevice, so a test can run one op or one whole
op sequence on both and compare.  Buffers are numpy arrays in host memory.  Only tests/,
__graft_entry__.smoke() and bench.py's cpu_baseline leg may import this module; the shipped package
never does.
"""
from __future__ import annotations

import ctypes
import re
import subprocess
from pathlib import Path

import numpy as np

from zigrad_amd.device import DevBuf, HipDevice
from zigrad_amd._lib import _ctype

ORACLE_DIR = Path(__file__).resolve().parent
LIB_PATH = ORACLE_DIR / "libzg_oracle.so"
HEADER = ORACLE_DIR / "zg_oracle.h"


def build_oracle() -> Path:
    subprocess.run(["make", "-C", str(ORACLE_DIR), "-s"], check=True)
    return LIB_PATH


def _parse(path: Path):
    text = path.read_text()
    text = re.sub(r"/\*.*?\*/", " ", text, flags=re.S)
    protos = {}
    for m in re.finditer(r"(?m)^[ \t]*([A-Za-z_][\w \t\*]*?)\b(zo_\w+)\s*\(([^;{}]*?)\)\s*;", text):
        ret, name, params = m.group(1).strip(), m.group(2), m.group(3).strip()
        plist = []
        if params and params != "void":
            for p in params.split(","):
                pm = re.match(r"(.*?)(\w+)$", p.strip())
                plist.append(_ctype(pm.group(1)))
        protos[name] = (_ctype(ret), plist)
    return protos


class _OracleLib:
    def __init__(self):
        if not LIB_PATH.exists():
            build_oracle()
        self.cdll = ctypes.CDLL(str(LIB_PATH))
        for name, (restype, argtypes) in _parse(HEADER).items():
            fn = getattr(self.cdll, name)
            fn.restype = restype
            fn.argtypes = argtypes


_LIB = None


def oracle_lib() -> _OracleLib:
    global _LIB
    if _LIB is None:
        _LIB = _OracleLib()
    return _LIB


class OracleDevice(HipDevice):
    """Same op glue as HipDevice, but every call lands in the C oracle and memory is host memory."""

    def __init__(self):  # noqa: D107 - deliberately does not call HipDevice.__init__ (no GPU involved)
        self._o = oracle_lib()
        self._arrays: dict[int, np.ndarray] = {}
        self._scratch = None
        self.device_id = -1
        self.n_allocs = 0

    # -- plumbing ----------------------------------------------------------------------------
    def _call(self, name: str, *args):
        fn = getattr(self, "_x_" + name, None)
        if fn is not None:
            return fn(*args)
        assert name.startswith("zg_hip_"), name
        return getattr(self._o.cdll, "zo_" + name[len("zg_hip_"):])(*args)

    def deinit(self):
        self._arrays.clear()

    def is_host(self):
        return True

    def is_compatible(self, other):
        return isinstance(other, OracleDevice)

    def sync(self):
        pass

    def blas_name(self) -> str:
        return self._o.cdll.zo_blas_name().decode()

    def set_threads(self, n: int) -> int:
        return int(self._o.cdll.zo_blas_set_threads(int(n)))

    def force_builtin_blas(self, on: bool) -> None:
        self._o.cdll.zo_blas_force_builtin(int(on))

    # the by-value scalar forms: HostDevice reads the caller's one-element slice in place
    # (src/ndarray.zig:247-257, src/device/host_device.zig:975-1019), so the oracle gets a one-element array
    def _scalar_form(self, op, x, n, s, scalar_is_lhs, z):
        one = np.asarray([s], np.float32)
        fn = getattr(self._o.cdll, "zo_" + op)
        if scalar_is_lhs:
            return fn(one.ctypes.data, 1, x, n, z, n)
        return fn(x, n, one.ctypes.data, 1, z, n)

    def _x_zg_hip_add_scalar(self, *a): return self._scalar_form("add", *a)
    def _x_zg_hip_sub_scalar(self, *a): return self._scalar_form("sub", *a)
    def _x_zg_hip_mul_scalar(self, *a): return self._scalar_form("mul", *a)
    def _x_zg_hip_div_scalar(self, *a): return self._scalar_form("div", *a)

    # -- memory --------------------------------------------------------------------------------
    def _new(self, dtype, n, kind):
        dtype = np.dtype(dtype)
        a = np.empty(max(n, 1), dtype=dtype)
        self._arrays[a.ctypes.data] = a
        self.n_allocs += 1
        return DevBuf(a.ctypes.data, n, dtype, 1 if kind == "cache" else 0, kind)

    def mem_alloc(self, dtype, n):
        return self._new(dtype, n, "raw")

    def mem_alloc_host(self, dtype, n):
        return self._new(dtype, n, "raw")

    def host_view(self, buf):
        return self._view(buf)  # all of the oracle's memory is host memory

    def mem_cache_alloc(self, dtype, n):
        return self._new(dtype, n, "cache")

    def mem_free(self, buf):
        self._arrays.pop(buf.ptr, None)
        buf.ptr, buf.n = 0, 0

    def mem_cache_free(self, buf):
        if buf.block == 0:
            return
        self._arrays.pop(buf.ptr, None)
        buf.ptr, buf.n, buf.block = 0, 0, 0

    def mem_scratch(self, dtype, n):
        dtype = np.dtype(dtype)
        if self._scratch is None or self._scratch.nbytes < n * dtype.itemsize:
            self._scratch = np.empty(max(n * dtype.itemsize, 1), dtype=np.uint8)
        return DevBuf(self._scratch.ctypes.data, n, dtype, 0, "view")

    def clear_cache(self):
        pass

    def launch_count(self) -> int:
        return 0  # nothing is launched: every op runs on the host when it is called

    def cache_stats(self):
        return {"bytes_in_use": 0, "bytes_mapped": 0, "n_device_allocs": self.n_allocs}

    def _view(self, buf: DevBuf) -> np.ndarray:
        return np.ctypeslib.as_array(ctypes.cast(buf.ptr, ctypes.POINTER(ctypes.c_uint8)), (buf.nbytes,)).view(buf.dtype)

    def mem_fill(self, buf, value):
        if buf.n:
            self._view(buf)[:] = value

    def mem_copy(self, src, dst):
        if src.n:
            ctypes.memmove(dst.ptr, src.ptr, src.nbytes)

    def mem_transfer(self, src, dst, direction):
        if direction == "HtoD":
            a = np.ascontiguousarray(src, dtype=dst.dtype)
            ctypes.memmove(dst.ptr, a.ctypes.data, a.nbytes)
        elif direction == "DtoH":
            ctypes.memmove(dst.ctypes.data, src.ptr, src.nbytes)
        else:
            self.mem_copy(src, dst)

    def from_numpy(self, a, cached=False):
        a = np.ascontiguousarray(a)
        buf = self._new(a.dtype, a.size, "cache" if cached else "raw")
        if a.size:
            ctypes.memmove(buf.ptr, a.ctypes.data, a.nbytes)
        return buf

    def to_numpy(self, buf, shape=None):
        out = self._view(buf).copy() if buf.n else np.empty(0, dtype=buf.dtype)
        return out.reshape(shape) if shape is not None else out

    def event(self):
        raise NotImplementedError("the oracle is timed with time.perf_counter")

    # -- entry points whose oracle signature differs from the C ABI ----------------------------------
    # -- planned scatter ops: the plan is just the index arrays, the ops are the sequential host loops ------
    def edge_plan(self, src_indices, tgt_indices, n_nodes):
        from zigrad_amd.device import EdgePlan

        return EdgePlan(self, None, src_indices, tgt_indices, n_nodes)

    def _op_scatter_add_planned(self, src, plan, dst, accumulate=True):
        if not accumulate:
            self.mem_fill(dst, 0.0)
        self.dispatch("scatter_add", src=src, offsets=plan.tgt_indices, dst=dst)

    def _op_scatter_gcn_deg_scaled_planned(self, dst, h, deg, plan, stride, accumulate=True, bias=None, relu=False):
        if not accumulate:
            self.mem_fill(dst, 0.0)
        self.dispatch("scatter_gcn_deg_scaled", dst=dst, h=h, deg=deg, src_indices=plan.src_indices,
                      tgt_indices=plan.tgt_indices, stride=stride, n_edge=plan.src_indices.n)
        if bias is not None:  # y._add(self.bias), examples/gcn/src/model.zig:110
            self.dispatch("add", x=bias, y=dst, z=dst)
        if relu:              # relu_ on the layer's output, examples/gcn/src/model.zig:36
            self.dispatch("relu_fwd", x=dst, y=dst)

    def _op_scatter_gcn_deg_scaled_bwd_planned(self, grad_output, h, deg, plan, grad_h, grad_deg, stride, accumulate=True):
        unused = grad_deg is None
        if unused:
            grad_deg = self.mem_alloc(grad_h.dtype, plan.n_nodes)
        if not accumulate or unused:
            self.mem_fill(grad_deg, 0.0)
        if not accumulate:
            self.mem_fill(grad_h, 0.0)
        self.dispatch("scatter_gcn_deg_scaled_bwd", grad_output=grad_output, h=h, deg=deg, src_indices=plan.src_indices,
                      tgt_indices=plan.tgt_indices, grad_h=grad_h, grad_deg=grad_deg, stride=stride,
                      n_edge=plan.src_indices.n)
        if unused:
            self.mem_free(grad_deg)

    # -- the list entry points are the per-tensor ops in a loop --------------------------------------------
    def _op_sgd_step_multi(self, params, grads, lr, clip, max_norm, delta, zero_grads):
        for p, g in zip(params, grads):
            self.dispatch("sgd_step", param=p, grad=g, lr=lr, clip=clip, max_norm=max_norm, delta=delta)
            if zero_grads:
                self.mem_fill(g, 0.0)

    def _op_adam_step_multi(self, params, grads, ms, vs, lr, t_first, beta1, beta2, epsilon, clip, max_norm, delta,
                            zero_grads, lr_t_mem=None):
        assert lr_t_mem is None, "the oracle has no recorded steps"
        for i, (p, g, m, v) in enumerate(zip(params, grads, ms, vs)):
            self.dispatch("adam_step", param=p, grad=g, m=m, v=v, t=t_first + i, lr=lr, beta1=beta1, beta2=beta2,
                          epsilon=epsilon, clip=clip, max_norm=max_norm, delta=delta)
            if zero_grads:
                self.mem_fill(g, 0.0)

    def _x_zg_hip_linear_fwd(self, x, w, bias, y, batch, fan_in, fan_out, relu):
        # the three ops the fused entry point stands for (examples/mnist/src/model.zig:104-110, :38-46)
        c = self._o.cdll
        c.zo_matmul(x, w, y, batch, fan_out, fan_in, 0, 1, fan_in, fan_in, fan_out, 1.0, 0.0)
        if bias:
            c.zo_add(bias, fan_out, y, batch * fan_out, y, batch * fan_out)
        if relu:
            c.zo_relu_fwd(y, y, batch * fan_out)

    def _x_zg_hip_linear_bwd_input(self, gy, w, act_in, gx, batch, fan_in, fan_out, accumulate):
        # dA of BmmAccBwd (src/ndtensor.zig:1092-1136) followed by relu_inplace_bwd (src/device/host_device.zig:543-547)
        c = self._o.cdll
        c.zo_matmul(gy, w, gx, batch, fan_in, fan_out, 0, 0, fan_out, fan_in, fan_in, 1.0, 1.0 if accumulate else 0.0)
        if act_in:
            c.zo_relu_inplace_bwd(act_in, gx, batch * fan_in)

    def _x_zg_hip_linear_bwd(self, gy, x, w, act_in, gw, gb, gx, batch, fan_in, fan_out):
        # dB and dA of BmmAccBwd for MATMUL_ABt (src/ndtensor.zig:1092-1136), the bias's fold over the batch
        # (src/device/host_device.zig:709-780) and relu_inplace_bwd of the layer before (:543-547)
        c = self._o.cdll
        c.zo_matmul(gy, x, gw, fan_out, fan_in, batch, 1, 0, fan_out, fan_in, fan_in, 1.0, 1.0)
        if gb:
            shape_x, shape_y = (ctypes.c_uint64 * 2)(batch, fan_out), (ctypes.c_uint64 * 1)(fan_out)
            c.zo_unbroadcast(gy, shape_x, 2, gb, shape_y, 1, None, 0, 1.0, 1.0)
        if gx:
            c.zo_matmul(gy, w, gx, batch, fan_in, fan_out, 0, 0, fan_out, fan_in, fan_in, 1.0, 0.0)
            if act_in:
                c.zo_relu_inplace_bwd(act_in, gx, batch * fan_in)

    def _x_zg_hip_axpy(self, x, y, n, alpha, alpha_on_device):
        return self._o.cdll.zo_axpy(x, y, n, alpha)  # host memory either way

    def _x_zg_hip_scatter_gcn_deg_scaled(self, dst, h, deg, s, t, stride, n_edge, n_nodes):
        return self._o.cdll.zo_scatter_gcn_deg_scaled(dst, h, deg, s, t, stride, n_edge)

    def _x_zg_hip_scatter_gcn_deg_scaled_bwd(self, go, h, deg, s, t, gh, gd, stride, n_edge, n_nodes):
        return self._o.cdll.zo_scatter_gcn_deg_scaled_bwd(go, h, deg, s, t, gh, gd, stride, n_edge)

    def _x_zg_hip_smooth_l1_fwd_bwd(self, pred, target, grad, n, beta, loss, accumulate):
        # the forward followed by the loss's backward with an upstream gradient of 1 (src/nn/loss.zig:259-305)
        if not accumulate:
            ctypes.memset(grad, 0, n * 4)
        self._o.cdll.zo_smooth_l1_fwd(pred, target, n, beta, loss)
        self._o.cdll.zo_smooth_l1_bwd(pred, target, grad, n, beta)

    def _x_zg_hip_smce_fwd_bwd(self, logits, target, probs, loss, grad, rows, cols, accumulate):
        # the forward followed by CceBwd with an upstream gradient of 1 (src/nn/loss.zig:130-159)
        if not accumulate:
            ctypes.memset(grad, 0, rows * cols * 4)
        self._o.cdll.zo_smce_fwd(logits, target, probs, loss, rows, cols)
        self._o.cdll.zo_smce_bwd(probs, target, grad, rows, cols)

    def _x_zg_hip_smce_label_bwd(self, logits, labels, lse, grad, rows, cols, accumulate):
        if not accumulate:
            ctypes.memset(grad, 0, rows * cols * 4)
        return self._o.cdll.zo_smce_label_bwd(logits, labels, lse, grad, rows, cols)

    def gather_offsets(self, src_shape, idx_shape, indices, dim, offsets, check=True):
        from zigrad_amd.device import _shape

        ss, r = _shape(src_shape)
        ish, _ = _shape(idx_shape)
        return int(self._o.cdll.zo_gather_offsets(ss, ish, r, indices.ptr, dim, offsets.ptr))

    def gather(self, src, src_shape, idx_shape, indices, dim, offsets, dst, check=True):
        # NDArray.gather (src/ndarray.zig:593-633): the offsets loop, then mem_take
        status = self.gather_offsets(src_shape, idx_shape, indices, dim, offsets, check=check)
        if status == 0:
            self.mem_take(src, offsets, dst)
        return status

    def unbroadcast_scratch_len(self, x_shape, y_shape):
        from zigrad_amd.device import _shape

        xs, xr = _shape(x_shape)
        ys, yr = _shape(y_shape)
        return int(self._o.cdll.zo_unbroadcast_scratch_len(xs, xr, ys, yr))

    def _x_zg_hip_mem_sequence(self, x, n, initial, step):
        return self._o.cdll.zo_mem_sequence(x, n, initial, step)

    def mem_sequence(self, buf, initial, step):
        self._o.cdll.zo_mem_sequence(buf.ptr, buf.n, float(initial), float(step))

    def mem_random(self, buf, kind, seed, fan=0):
        code = {"uniform": 0, "normal": 1, "kaiming": 2}[kind]
        self._o.cdll.zo_mem_random(buf.ptr, buf.n, code, int(fan), int(seed))

    def adam_lr_t(self, lr, beta1, beta2, t) -> float:
        return float(self._o.cdll.zo_adam_lr_t(int(t), lr, beta1, beta2))

    def mem_take(self, src, idxs, dst):
        self._o.cdll.zo_mem_take(src.ptr, src.n, idxs.ptr, idxs.n, dst.ptr)

    def matmul_f64acc(self, A, B, C, m, n, k, trans_a, trans_b, lda, ldb, ldc, alpha, beta):
        self._o.cdll.zo_matmul_f64acc(A.ptr, B.ptr, C.ptr, m, n, k, int(trans_a), int(trans_b), lda, ldb, ldc, alpha, beta)
