"""HipDevice: the host-side face of the gfx950 backend.

It mirrors the device interface Zigrad's upper layers program against
(reference: src/device/device_reference.zig:15-131): `dispatch(name, **params)` takes the op name and
the field names of the matching parameter struct in src/device/opspec.zig, and the `mem_*` methods
keep the names and meaning of the reference's memory API.  Every call goes through the C ABI in
include/zg_hip.h; nothing is computed in Python and nothing falls back to the CPU.

Slices of the reference (`[]T`) are `DevBuf` objects here: a device pointer, an element count and a
dtype.  `DevBuf.sub(offset, n)` is the pointer-arithmetic sub-slice the reference takes freely
(src/ndtensor.zig:581, :1462-1464).
"""
from __future__ import annotations

import ctypes
from dataclasses import dataclass

import numpy as np

from ._lib import ZgHipError, lib

F32 = np.dtype(np.float32)
U64 = np.dtype(np.uint64)


@dataclass
class DevBuf:
    ptr: int
    n: int
    dtype: np.dtype = F32
    block: int = 0  # DeviceData.ctx of the reference: 0 for views / raw allocations
    kind: str = "raw"  # "raw" (mem_alloc), "cache" (mem_cache_alloc), "view", "host" (pinned host)

    def __len__(self) -> int:
        return self.n

    @property
    def nbytes(self) -> int:
        return self.n * self.dtype.itemsize

    def sub(self, offset: int, n: int) -> "DevBuf":
        if offset < 0 or n < 0 or offset + n > self.n:
            raise IndexError(f"sub-slice [{offset}:{offset + n}] outside a buffer of {self.n} elements")
        return DevBuf(self.ptr + offset * self.dtype.itemsize, n, self.dtype, 0, "view")


def _host_scalar(v):
    """The float value of a host-side scalar operand, None for a device buffer."""
    if isinstance(v, DevBuf):
        return None
    a = np.asarray(v, dtype=np.float32)
    if a.size != 1:
        raise ValueError("a host operand of an elementwise op must be a single value")
    return float(a.reshape(())[()])


def _shape(shape) -> tuple[ctypes.Array, int]:
    arr = (ctypes.c_uint64 * len(shape))(*[int(s) for s in shape])
    return arr, len(shape)


class HipDevice:
    """One MI355X device context: a single in-order stream plus the caching allocator."""

    def __init__(self, device_id: int = 0):
        self._lib = lib()
        ctx = ctypes.c_void_p()
        self._lib.call("zg_hip_init", int(device_id), ctypes.byref(ctx))
        self._ctx = ctx
        self.device_id = device_id

    # -- lifecycle ---------------------------------------------------------------------------
    def deinit(self) -> None:
        if self._ctx is not None:
            self._lib.call("zg_hip_deinit", self._ctx)
            self._ctx = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.deinit()

    def is_host(self) -> bool:
        return False

    def is_compatible(self, other) -> bool:
        return isinstance(other, HipDevice) and other.device_id == self.device_id

    def sync(self) -> None:
        self._call("zg_hip_sync")

    def flush(self) -> None:
        """Launch what earlier calls left waiting in the context, without waiting for the stream."""
        self._call("zg_hip_flush")

    def set_holding(self, enable: bool) -> None:
        """False: every call launches its own work before it returns (for callers that mix in their own HIP calls)."""
        self._call("zg_hip_set_holding", int(bool(enable)))

    def _call(self, name: str, *args) -> None:
        self._lib.call(name, self._ctx, *args)

    # -- timing ------------------------------------------------------------------------------
    def event(self) -> "Event":
        return Event(self)

    # -- input staging: upload the next batch on a second stream while the current one computes -------
    def staged_h2d(self, src_host: DevBuf, dst: DevBuf) -> None:
        """Asynchronous copy from pinned host memory (mem_alloc_host) on the copy stream."""
        if src_host.kind != "host":
            raise ValueError("staged_h2d needs a pinned source from mem_alloc_host")
        self._call("zg_hip_staged_h2d", dst.ptr, src_host.ptr, min(src_host.nbytes, dst.nbytes))

    def staging_after_compute(self) -> None:
        self._call("zg_hip_staging_after_compute")

    def compute_after_staging(self) -> None:
        self._call("zg_hip_compute_after_staging")

    def staging_wait(self) -> None:
        self._call("zg_hip_staging_wait")

    def host_view(self, buf: DevBuf) -> np.ndarray:
        """numpy view of a pinned host allocation (for the host code that fills it)."""
        if buf.kind != "host":
            raise ValueError("host_view needs a buffer from mem_alloc_host")
        ctype = np.ctypeslib.as_ctypes_type(buf.dtype)
        return np.ctypeslib.as_array((ctype * buf.n).from_address(buf.ptr))

    # -- execution graphs (src/device/cuda_device.zig:558-611: open / save / run / free) -----------
    def graph_open(self) -> None:
        """Start recording: until graph_save() every op call is captured instead of executed."""
        self._call("zg_hip_graph_open")

    def graph_save(self) -> "Graph":
        h = ctypes.c_void_p()
        self._call("zg_hip_graph_save", ctypes.byref(h))
        return Graph(self, h)

    # -- memory API (src/device/device_reference.zig:29-123) -----------------------------------
    def mem_alloc(self, dtype, n: int) -> DevBuf:
        dtype = np.dtype(dtype)
        p = ctypes.c_void_p()
        self._call("zg_hip_alloc", n * dtype.itemsize, ctypes.byref(p))
        return DevBuf(p.value or 0, n, dtype, 0, "raw")

    def mem_free(self, buf: DevBuf) -> None:
        if buf.n == 0 or buf.ptr == 0:
            return
        if buf.kind == "host":
            self._call("zg_hip_host_free", buf.ptr)
        else:
            self._call("zg_hip_free", buf.ptr)
        buf.ptr, buf.n = 0, 0

    def mem_alloc_host(self, dtype, n: int) -> DevBuf:
        """Pinned host memory the kernels can read: for index arrays the caller fills on the host."""
        dtype = np.dtype(dtype)
        p = ctypes.c_void_p()
        self._call("zg_hip_host_alloc", n * dtype.itemsize, ctypes.byref(p))
        return DevBuf(p.value or 0, n, dtype, 0, "host")

    def mem_alloc_byte_mask(self, n: int) -> DevBuf:
        return self.mem_alloc(np.uint8, (n - 1) // 8 + 1)

    def mem_cache_alloc(self, dtype, n: int) -> DevBuf:
        dtype = np.dtype(dtype)
        p, blk = ctypes.c_void_p(), ctypes.c_uint64()
        self._call("zg_hip_mem_cache_alloc", n * dtype.itemsize, ctypes.byref(p), ctypes.byref(blk))
        return DevBuf(p.value or 0, n, dtype, blk.value, "cache")

    def mem_cache_free(self, buf: DevBuf) -> None:
        if buf.block == 0:
            return
        self._call("zg_hip_mem_cache_free", buf.ptr, buf.block)
        buf.ptr, buf.n, buf.block = 0, 0, 0

    def mem_cache_dupe(self, src: DevBuf) -> DevBuf:
        dst = self.mem_cache_alloc(src.dtype, src.n)
        self.mem_copy(src, dst)
        return dst

    def mem_dupe(self, src: DevBuf) -> DevBuf:
        dst = self.mem_alloc(src.dtype, src.n)
        self.mem_copy(src, dst)
        return dst

    def mem_scratch(self, dtype, n: int) -> DevBuf:
        dtype = np.dtype(dtype)
        p = ctypes.c_void_p()
        self._call("zg_hip_mem_scratch", n * dtype.itemsize, ctypes.byref(p))
        return DevBuf(p.value or 0, n, dtype, 0, "view")

    def clear_cache(self) -> None:
        self._call("zg_hip_clear_cache")

    def cache_configure(self, small_pool_bytes: int, large_pool_bytes: int) -> None:
        """Segment sizes of the two block pools (CachingAllocator.Options, src/allocators/caching_allocator.zig:41-44);
        only before the first cache allocation or after clear_cache()."""
        self._call("zg_hip_cache_configure", int(small_pool_bytes), int(large_pool_bytes))

    def is_device_ptr(self, ptr: int) -> bool:
        yes = ctypes.c_int(0)
        self._call("zg_hip_is_device_ptr", ctypes.c_void_p(ptr), ctypes.byref(yes))
        return bool(yes.value)

    def cache_stats(self) -> dict:
        u, m, a = ctypes.c_size_t(), ctypes.c_size_t(), ctypes.c_uint64()
        self._call("zg_hip_cache_stats", ctypes.byref(u), ctypes.byref(m), ctypes.byref(a))
        return {"bytes_in_use": u.value, "bytes_mapped": m.value, "n_device_allocs": a.value}

    def launch_count(self) -> int:
        """Kernels the library has launched in this process so far (device-to-device copies included); work that
        still waits in the context is not counted."""
        n = ctypes.c_uint64()
        self._call("zg_hip_launch_count", ctypes.byref(n))
        return n.value

    def mem_fill(self, buf: DevBuf, value) -> None:
        if buf.dtype == F32:
            self._call("zg_hip_mem_fill", buf.ptr, buf.n, float(value))
        elif buf.dtype == U64:
            self._call("zg_hip_mem_fill_u64", buf.ptr, buf.n, int(value))
        elif buf.dtype.itemsize == 1:
            self._call("zg_hip_mem_fill_u8", buf.ptr, buf.n, int(value))
        else:
            raise TypeError(f"mem_fill: unsupported dtype {buf.dtype}")

    def mem_copy(self, src: DevBuf, dst: DevBuf) -> None:
        if dst.n < src.n:
            raise ValueError("mem_copy: destination shorter than source")
        self._call("zg_hip_memcpy_d2d", dst.ptr, src.ptr, src.nbytes)

    def mem_sequence(self, buf: DevBuf, initial: float, step: float) -> None:
        self._call("zg_hip_mem_sequence", buf.ptr, buf.n, float(initial), float(step))

    def mem_random(self, buf: DevBuf, kind: str, seed: int, fan: int = 0) -> None:
        code = {"uniform": 0, "normal": 1, "kaiming": 2}[kind]
        self._call("zg_hip_mem_random", buf.ptr, buf.n, code, int(fan), int(seed))

    def mem_take(self, src: DevBuf, idxs: DevBuf, dst: DevBuf) -> None:
        if dst.n < idxs.n:
            raise ValueError("mem_take: dst.len < idxs.len")
        self._call("zg_hip_mem_take", src.ptr, src.n, idxs.ptr, idxs.n, dst.ptr)

    def mem_transfer(self, src, dst, direction: str) -> None:
        """direction: 'HtoD' (src numpy array), 'DtoH' (dst numpy array, blocking), 'DtoD'."""
        if direction == "HtoD":
            a = np.ascontiguousarray(src, dtype=dst.dtype)
            if a.size > dst.n:
                raise ValueError("mem_transfer: destination too small")
            self._call("zg_hip_memcpy_h2d", dst.ptr, a.ctypes.data, a.nbytes)
        elif direction == "DtoH":
            if not (isinstance(dst, np.ndarray) and dst.flags.c_contiguous and dst.dtype == src.dtype):
                raise ValueError("mem_transfer: DtoH needs a contiguous numpy array of the buffer's dtype")
            if dst.size < src.n:
                raise ValueError("mem_transfer: destination too small")
            self._call("zg_hip_memcpy_d2h", dst.ctypes.data, src.ptr, src.nbytes)
        elif direction == "DtoD":
            self.mem_copy(src, dst)
        else:
            raise ValueError(f"unknown transfer direction {direction!r}")

    # conveniences built on the above (not part of the reference interface)
    def from_numpy(self, a: np.ndarray, cached: bool = False) -> DevBuf:
        a = np.ascontiguousarray(a)
        buf = (self.mem_cache_alloc if cached else self.mem_alloc)(a.dtype, a.size)
        if a.size:
            self._call("zg_hip_memcpy_h2d", buf.ptr, a.ctypes.data, a.nbytes)
        return buf

    def to_numpy(self, buf: DevBuf, shape=None) -> np.ndarray:
        out = np.empty(buf.n, dtype=buf.dtype)
        if buf.n:
            self._call("zg_hip_memcpy_d2h", out.ctypes.data, buf.ptr, buf.nbytes)
        return out.reshape(shape) if shape is not None else out

    # -- op dispatch (src/device/device_reference.zig:15-27) -----------------------------------
    def dispatch(self, name: str, **p) -> None:
        """Run device op `name` with the field names of opspec.<name>; unknown names raise like the
        reference's @panic("Unimplemented")."""
        fn = getattr(self, "_op_" + name, None)
        if fn is None:
            raise NotImplementedError(f"Unimplemented: {name} for HipDevice")
        fn(**p)

    # elementwise binary
    def _bin(self, cname, x, y, z):
        """x or y may be a host scalar (a Python / numpy number or a one-element numpy array): what NDArray.add_scalar
        hands the op as `.y = &.{s}` (src/ndarray.zig:247-257).  It goes to the by-value entry point."""
        xs, ys = _host_scalar(x), _host_scalar(y)
        if xs is None and ys is None:
            self._call(cname, x.ptr, x.n, y.ptr, y.n, z.ptr, z.n)
        elif xs is not None and ys is not None:
            raise ValueError(f"{cname}: both operands are host scalars")
        elif ys is not None:
            self._call(cname + "_scalar", x.ptr, x.n, ys, 0, z.ptr)
        else:
            self._call(cname + "_scalar", y.ptr, y.n, xs, 1, z.ptr)

    def _op_add(self, x, y, z): self._bin("zg_hip_add", x, y, z)
    def _op_sub(self, x, y, z): self._bin("zg_hip_sub", x, y, z)
    def _op_mul(self, x, y, z): self._bin("zg_hip_mul", x, y, z)
    def _op_div(self, x, y, z): self._bin("zg_hip_div", x, y, z)

    # linear algebra
    def _op_dot(self, x, y, z):
        if x.n != y.n:
            raise ValueError("dot: length mismatch")
        self._call("zg_hip_dot", x.ptr, y.ptr, x.n, z.ptr)

    def _op_matvec(self, A, x, y, m, n, trans_a, alpha, beta):
        self._call("zg_hip_matvec", A.ptr, x.ptr, y.ptr, m, n, int(trans_a), alpha, beta)

    def _op_matmul(self, A, B, C, m, n, k, trans_a, trans_b, lda, ldb, ldc, alpha, beta):
        self._call("zg_hip_matmul", A.ptr, B.ptr, C.ptr, m, n, k, int(trans_a), int(trans_b), lda, ldb, ldc,
                   alpha, beta)

    def _op_bmm_acc(self, A, B, C, A_shape, B_shape, C_shape, trans_a, trans_b, lda, ldb, ldc, alpha, beta):
        a, _ = _shape(A_shape)
        b, _ = _shape(B_shape)
        c, _ = _shape(C_shape)
        self._call("zg_hip_bmm_acc", A.ptr, a, B.ptr, b, C.ptr, c, int(trans_a), int(trans_b), lda, ldb, ldc,
                   alpha, beta)

    def _op_linear_fwd(self, x, w, bias, y, batch, fan_in, fan_out, relu):
        """y = act(x . w^T + bias) in one launch; bias may be None."""
        self._call("zg_hip_linear_fwd", x.ptr, w.ptr, bias.ptr if bias is not None else None, y.ptr, batch, fan_in,
                   fan_out, int(relu))

    def _op_linear_bwd_input(self, gy, w, act_in, gx, batch, fan_in, fan_out, accumulate):
        """gx = (gx if accumulate else 0) + gy . w, zeroed where act_in <= 0 (act_in None: no mask)."""
        self._call("zg_hip_linear_bwd_input", gy.ptr, w.ptr, act_in.ptr if act_in is not None else None, gx.ptr, batch,
                   fan_in, fan_out, int(accumulate))

    def _op_linear_bwd(self, gy, x, w, act_in, gw, gb, gx, batch, fan_in, fan_out):
        """gw += gy^T . x; gb += column sums of gy (None: none); gx = gy . w, zeroed where act_in <= 0 (None: none)."""
        opt = lambda b: b.ptr if b is not None else None
        self._call("zg_hip_linear_bwd", gy.ptr, x.ptr, opt(w), opt(act_in), gw.ptr, opt(gb), opt(gx), batch, fan_in,
                   fan_out)

    def _op_outer(self, x, y, A, alpha):
        self._call("zg_hip_outer", x.ptr, x.n, y.ptr, y.n, A.ptr, alpha)

    def _op_transpose(self, A, B, m, n, alpha):
        self._call("zg_hip_transpose", A.ptr, B.ptr, m, n, alpha)

    def _op_axpy(self, x, y, alpha):
        """alpha: a Python float (the host pointer of SGD) or a 1-element DevBuf (dot backward)."""
        if isinstance(alpha, DevBuf):
            self._call("zg_hip_axpy", x.ptr, y.ptr, x.n, alpha.ptr, 1)
        else:
            a = ctypes.c_float(alpha)
            self._call("zg_hip_axpy", x.ptr, y.ptr, x.n, ctypes.byref(a), 0)

    def _op_sum(self, x, y): self._call("zg_hip_sum", x.ptr, x.n, y.ptr)
    def _op_scale(self, x, alpha): self._call("zg_hip_scale", x.ptr, x.n, alpha)
    def _op_nrm2(self, x, y): self._call("zg_hip_nrm2", x.ptr, x.n, y.ptr)
    def _op_clip_nrm2(self, x, max_norm, delta): self._call("zg_hip_clip_nrm2", x.ptr, x.n, max_norm, delta)

    # unary
    def _op_pow_fwd(self, x, exp, y): self._call("zg_hip_pow_fwd", x.ptr, y.ptr, x.n, exp)
    def _op_pow_fwd_(self, x, exp): self._call("zg_hip_pow_fwd", x.ptr, x.ptr, x.n, exp)
    def _op_pow_bwd(self, x, x_g, exp, y_g, eps): self._call("zg_hip_pow_bwd", x.ptr, x_g.ptr, y_g.ptr, x.n, exp, eps)
    def _op_sqrt_fwd(self, x, y): self._call("zg_hip_sqrt_fwd", x.ptr, y.ptr, x.n)
    def _op_sqrt_fwd_(self, x): self._call("zg_hip_sqrt_fwd", x.ptr, x.ptr, x.n)
    def _op_sqrt_bwd(self, x, x_g, y_g, eps): self._call("zg_hip_sqrt_bwd", x.ptr, x_g.ptr, y_g.ptr, x.n, eps)
    def _op_rsqrt_fwd(self, x, y, eps): self._call("zg_hip_rsqrt_fwd", x.ptr, y.ptr, x.n, eps)
    def _op_rsqrt_bwd(self, x, x_g, y_g, eps): self._call("zg_hip_rsqrt_bwd", x.ptr, x_g.ptr, y_g.ptr, x.n, eps)
    def _op_exp_fwd(self, x, y): self._call("zg_hip_exp_fwd", x.ptr, y.ptr, x.n)
    def _op_exp_bwd(self, x_g, y, y_g): self._call("zg_hip_exp_bwd", x_g.ptr, y.ptr, y_g.ptr, x_g.n)
    def _op_relu_fwd(self, x, y): self._call("zg_hip_relu_fwd", x.ptr, y.ptr, x.n)
    def _op_relu_bwd(self, x, x_g, y_g): self._call("zg_hip_relu_bwd", x.ptr, x_g.ptr, y_g.ptr, x.n)
    def _op_relu_inplace_bwd(self, x, x_g): self._call("zg_hip_relu_inplace_bwd", x.ptr, x_g.ptr, x.n)
    def _op_tanh_fwd(self, x, y): self._call("zg_hip_tanh_fwd", x.ptr, y.ptr, x.n)
    def _op_tanh_bwd(self, x_g, y, y_g): self._call("zg_hip_tanh_bwd", x_g.ptr, y.ptr, y_g.ptr, x_g.n)
    def _op_tanh_inplace_bwd(self, x, x_g): self._call("zg_hip_tanh_inplace_bwd", x.ptr, x_g.ptr, x.n)
    def _op_sigm_fwd(self, x, y): self._call("zg_hip_sigm_fwd", x.ptr, y.ptr, x.n)
    def _op_sigm_bwd(self, x_g, y, y_g): self._call("zg_hip_sigm_bwd", x_g.ptr, y.ptr, y_g.ptr, x_g.n)
    def _op_sigm_inplace_bwd(self, x, x_g): self._call("zg_hip_sigm_inplace_bwd", x.ptr, x_g.ptr, x.n)
    def _op_clamp_fwd(self, x, y, min, max): self._call("zg_hip_clamp_fwd", x.ptr, y.ptr, x.n, min, max)
    def _op_clamp_bwd(self, x, x_g, y_g, min, max): self._call("zg_hip_clamp_bwd", x.ptr, x_g.ptr, y_g.ptr, x.n, min, max)
    def _op_max_fwd(self, x, y): self._call("zg_hip_max_fwd", x.ptr, x.n, y.ptr)
    def _op_max_bwd(self, x, x_g, y, y_g): self._call("zg_hip_max_bwd", x.ptr, x_g.ptr, x.n, y.ptr, y_g.ptr)

    # reductions
    def _op_sum_along(self, x, x_shape, y, y_shape=None, dim=0, alpha=1.0, beta=0.0):
        s, r = _shape(x_shape)
        self._call("zg_hip_sum_along", x.ptr, s, r, y.ptr, y.n, dim, alpha, beta)

    def _op_max_along(self, x, x_shape, y, y_shape=None, dim=0, alpha=1.0, beta=0.0):
        s, r = _shape(x_shape)
        self._call("zg_hip_max_along", x.ptr, s, r, y.ptr, y.n, dim)

    def _op_argmax_along(self, x, x_shape, y, dim):
        s, r = _shape(x_shape)
        self._call("zg_hip_argmax_along", x.ptr, s, r, y.ptr, y.n, dim)

    def unbroadcast_scratch_len(self, x_shape, y_shape) -> int:
        xs, xr = _shape(x_shape)
        ys, yr = _shape(y_shape)
        return int(self._lib.cdll.zg_hip_unbroadcast_scratch_len(xs, xr, ys, yr))

    def _op_unbroadcast(self, x, x_shape, y, y_shape, scratch=None, alpha=1.0, beta=0.0):
        xs, xr = _shape(x_shape)
        ys, yr = _shape(y_shape)
        sp, sn = (scratch.ptr, scratch.n) if scratch is not None else (None, 0)
        self._call("zg_hip_unbroadcast", x.ptr, xs, xr, y.ptr, ys, yr, sp, sn, alpha, beta)

    def _op_broadcast(self, x, y, x_shape=None, y_shape=None, alpha=1.0, beta=0.0):
        self._call("zg_hip_broadcast", x.ptr, x.n, y.ptr, y.n, alpha, beta)

    # indexing
    def gather_offsets(self, src_shape, idx_shape, indices: DevBuf, dim: int, offsets: DevBuf, check: bool = True) -> int:
        ss, r = _shape(src_shape)
        ish, _ = _shape(idx_shape)
        st = ctypes.c_int(0)
        try:
            self._call("zg_hip_gather_offsets", ss, ish, r, indices.ptr, dim, offsets.ptr,
                       ctypes.byref(st) if check else None)
        except ZgHipError:
            if st.value:
                return st.value
            raise
        return st.value

    def gather(self, src: DevBuf, src_shape, idx_shape, indices: DevBuf, dim: int, offsets: DevBuf, dst: DevBuf,
               check: bool = True) -> int:
        """Offsets and values of NDArray.gather in one launch; returns the status gather_offsets returns."""
        ss, r = _shape(src_shape)
        ish, _ = _shape(idx_shape)
        st = ctypes.c_int(0)
        try:
            self._call("zg_hip_gather", src.ptr, ss, ish, r, indices.ptr, dim, offsets.ptr, dst.ptr,
                       ctypes.byref(st) if check else None)
        except ZgHipError:
            if st.value:
                return st.value
            raise
        return st.value

    def _op_scatter_add(self, src, offsets, dst):
        if offsets.n != src.n:
            raise ValueError("scatter_add: offsets.len != src.len")
        self._call("zg_hip_scatter_add", src.ptr, offsets.ptr, src.n, dst.ptr, dst.n)

    def _op_scatter_add_csr(self, src, row_ptr, dst):
        if row_ptr.n != src.n + 1:
            raise ValueError("scatter_add_csr: row_ptr.len != src.len + 1")
        self._call("zg_hip_scatter_add_csr", src.ptr, row_ptr.ptr, src.n, dst.ptr, dst.n)

    def _op_segment_sum_csr(self, src, row_offsets, dst):
        if row_offsets.n != dst.n + 1:
            raise ValueError("segment_sum_csr: row_offsets.len != dst.len + 1")
        self._call("zg_hip_segment_sum_csr", src.ptr, src.n, row_offsets.ptr, dst.n, dst.ptr)

    def _op_index_select_fwd(self, src, indices, stride, dst):
        self._call("zg_hip_index_select_fwd", src.ptr, src.n, indices.ptr, indices.n, stride, dst.ptr)

    def _op_index_select_bwd(self, y_grad, indices, stride, x_grad):
        self._call("zg_hip_index_select_bwd", y_grad.ptr, indices.ptr, indices.n, stride, x_grad.ptr, x_grad.n)

    def _op_scatter_gcn_deg_scaled(self, dst, h, deg, src_indices, tgt_indices, stride, n_edge):
        self._call("zg_hip_scatter_gcn_deg_scaled", dst.ptr, h.ptr, deg.ptr, src_indices.ptr, tgt_indices.ptr,
                   stride, n_edge, deg.n)

    def _op_scatter_gcn_deg_scaled_bwd(self, grad_output, h, deg, src_indices, tgt_indices, grad_h, grad_deg, stride,
                                       n_edge):
        self._call("zg_hip_scatter_gcn_deg_scaled_bwd", grad_output.ptr, h.ptr, deg.ptr, src_indices.ptr,
                   tgt_indices.ptr, grad_h.ptr, grad_deg.ptr, stride, n_edge, deg.n)

    def gemm_plan(self, m: int, n: int, k: int, batches: int = 1) -> dict:
        """How the staged GEMM kernels would launch this product (see zg_hip_gemm_plan)."""
        return gemm_plan(m, n, k, batches, self)

    def gemm_timing(self, on: bool) -> None:
        """Start (clearing the count) or stop bracketing every product's launches with events on the stream."""
        self._call("zg_hip_gemm_timing", int(bool(on)))

    def gemm_timing_read(self) -> tuple[float, int]:
        """(summed milliseconds between the event pairs, number of products) since timing was last started."""
        ms, cnt = ctypes.c_double(), ctypes.c_uint64()
        self._call("zg_hip_gemm_timing_read", ctypes.byref(ms), ctypes.byref(cnt))
        return ms.value, cnt.value

    def plan_cache_stats(self) -> dict:
        """Calls served from a kept destination ordering / orderings computed and kept (pinned index arrays only)."""
        h, b = ctypes.c_uint64(), ctypes.c_uint64()
        self._call("zg_hip_plan_cache_stats", ctypes.byref(h), ctypes.byref(b))
        return {"hits": h.value, "builds": b.value}

    # the same three ops on an edge plan built once for an edge list that does not change
    def edge_plan(self, src_indices: DevBuf, tgt_indices: DevBuf, n_nodes: int) -> "EdgePlan":
        h = ctypes.c_void_p()
        self._call("zg_hip_edge_plan_create", src_indices.ptr, tgt_indices.ptr, src_indices.n, n_nodes, ctypes.byref(h))
        return EdgePlan(self, h, src_indices, tgt_indices, n_nodes)

    def _op_scatter_add_planned(self, src, plan, dst, accumulate=True):
        self._call("zg_hip_scatter_add_planned", src.ptr, plan.handle, dst.ptr, int(accumulate))

    def _op_scatter_gcn_deg_scaled_planned(self, dst, h, deg, plan, stride, accumulate=True, bias=None, relu=False):
        self._call("zg_hip_scatter_gcn_deg_scaled_planned", dst.ptr, h.ptr, deg.ptr, plan.handle,
                   bias.ptr if bias is not None else None, int(bool(relu)), stride, int(accumulate))

    def _op_scatter_gcn_deg_scaled_bwd_planned(self, grad_output, h, deg, plan, grad_h, grad_deg, stride, accumulate=True):
        """grad_deg may be None: the degree gradient is then not computed."""
        self._call("zg_hip_scatter_gcn_deg_scaled_bwd_planned", grad_output.ptr, h.ptr, deg.ptr, plan.handle, grad_h.ptr,
                   grad_deg.ptr if grad_deg is not None else None, stride, int(accumulate))

    # losses
    def _op_smce_fwd(self, logits, target, probs, loss, rows, cols):
        self._call("zg_hip_smce_fwd", logits.ptr, target.ptr, probs.ptr, loss.ptr, rows, cols)

    def _op_smce_bwd(self, probs, target, grad, rows, cols):
        self._call("zg_hip_smce_bwd", probs.ptr, target.ptr, grad.ptr, rows, cols)

    def _op_smce_fwd_bwd(self, logits, target, probs, loss, grad, rows, cols, accumulate=True):
        self._call("zg_hip_smce_fwd_bwd", logits.ptr, target.ptr, probs.ptr, loss.ptr, grad.ptr, rows, cols,
                   int(bool(accumulate)))

    def _op_smce_label_fwd(self, logits, labels, lse, loss, rows, cols):
        self._call("zg_hip_smce_label_fwd", logits.ptr, labels.ptr, lse.ptr, loss.ptr, rows, cols)

    def _op_smce_label_fwd_noalloc(self, logits, labels, lse, loss, rows, cols):
        """smce_label_fwd without any allocation: fixed scratch in the library's device image, at most 262144 rows."""
        self._call("zg_hip_smce_label_fwd_noalloc", logits.ptr, labels.ptr, lse.ptr, loss.ptr, rows, cols)

    def _op_smce_label_bwd(self, logits, labels, lse, grad, rows, cols, accumulate=True):
        self._call("zg_hip_smce_label_bwd", logits.ptr, labels.ptr, lse.ptr, grad.ptr, rows, cols, int(accumulate))

    def _op_softmax_fwd(self, x, y, rows, cols): self._call("zg_hip_softmax_fwd", x.ptr, y.ptr, rows, cols)
    def _op_softmax_bwd(self, y, y_g, x_g, rows, cols): self._call("zg_hip_softmax_bwd", y.ptr, y_g.ptr, x_g.ptr, rows, cols)

    def _op_smooth_l1_fwd(self, pred, target, beta, loss):
        self._call("zg_hip_smooth_l1_fwd", pred.ptr, target.ptr, pred.n, beta, loss.ptr)

    def _op_smooth_l1_bwd(self, pred, target, grad, beta):
        self._call("zg_hip_smooth_l1_bwd", pred.ptr, target.ptr, grad.ptr, pred.n, beta)

    def _op_smooth_l1_fwd_bwd(self, pred, target, grad, beta, loss, accumulate=True):
        self._call("zg_hip_smooth_l1_fwd_bwd", pred.ptr, target.ptr, grad.ptr, pred.n, beta, loss.ptr, int(bool(accumulate)))

    def _op_mse_fwd(self, pred, target, loss): self._call("zg_hip_mse_fwd", pred.ptr, target.ptr, pred.n, loss.ptr)
    def _op_mse_bwd(self, pred, target, grad): self._call("zg_hip_mse_bwd", pred.ptr, target.ptr, grad.ptr, pred.n)

    # optimizers
    def _op_sgd_step(self, param, grad, lr, clip, max_norm, delta):
        self._call("zg_hip_sgd_step", param.ptr, grad.ptr, param.n, lr, int(clip), max_norm, delta)

    def _op_adam_step(self, param, grad, m, v, t, lr, beta1, beta2, epsilon, clip, max_norm, delta):
        self._call("zg_hip_adam_step", param.ptr, grad.ptr, m.ptr, v.ptr, param.n, int(t), lr, beta1, beta2, epsilon,
                   int(clip), max_norm, delta)

    def _op_adam_step_at(self, param, grad, m, v, lr_t, beta1, beta2, epsilon, clip, max_norm, delta):
        """Adam update whose lr_t is read from `lr_t` (a one-float buffer) when the kernel runs."""
        self._call("zg_hip_adam_step_at", param.ptr, grad.ptr, m.ptr, v.ptr, param.n, lr_t.ptr, beta1, beta2, epsilon,
                   int(clip), max_norm, delta)

    @staticmethod
    def _ptr_list(bufs):
        return (ctypes.c_void_p * len(bufs))(*[b.ptr for b in bufs])

    def _op_sgd_step_multi(self, params, grads, lr, clip, max_norm, delta, zero_grads):
        """SGD over a parameter list in as few launches as possible; optionally leaves the gradients zero."""
        lens = (ctypes.c_size_t * len(params))(*[p.n for p in params])
        self._call("zg_hip_sgd_step_multi", len(params), self._ptr_list(params), self._ptr_list(grads), lens, lr, int(clip),
                   max_norm, delta, int(zero_grads))

    def _op_adam_step_multi(self, params, grads, ms, vs, lr, t_first, beta1, beta2, epsilon, clip, max_norm, delta,
                            zero_grads, lr_t_mem=None):
        """Adam over a parameter list.  Tensor i is updated with counter value t_first + i (the reference counts
        once per tensor, src/nn/optim.zig:189); with lr_t_mem (a DevBuf of one float per tensor in device or pinned
        memory) the kernels read each lr_t from there when they run instead."""
        lens = (ctypes.c_size_t * len(params))(*[p.n for p in params])
        if lr_t_mem is not None:
            lr_arg, in_memory = lr_t_mem.ptr, 1
        else:
            lr_arg = (ctypes.c_float * len(params))(*[self.adam_lr_t(lr, beta1, beta2, t_first + i) for i in range(len(params))])
            in_memory = 0
        self._call("zg_hip_adam_step_multi", len(params), self._ptr_list(params), self._ptr_list(grads), self._ptr_list(ms),
                   self._ptr_list(vs), lens, lr_arg, in_memory, beta1, beta2, epsilon, int(clip), max_norm, delta,
                   int(zero_grads))

    def adam_lr_t(self, lr, beta1, beta2, t) -> float:
        out = ctypes.c_float()
        self._lib.call("zg_hip_adam_lr_t", lr, beta1, beta2, int(t), ctypes.byref(out))
        return out.value


def gemm_plan(m: int, n: int, k: int, batches: int = 1, dev: "HipDevice | None" = None) -> dict:
    """zg_hip_gemm_plan as a dict; without a device the planner assumes 256 compute units (no GPU needed)."""
    from ._lib import lib

    out = (ctypes.c_int64 * 7)()
    lib().call("zg_hip_gemm_plan", dev._ctx if dev is not None else None, m, n, k, batches, out)
    kinds, tiles = ("single", "split_k", "parts", "tail_in_pieces"), ((256, 128), (128, 128), (64, 64))
    tail = kinds[out[0]] == "tail_in_pieces"
    return {"kind": kinds[out[0]], "tile": tiles[out[1]], "splits": out[2], "k_tiles_per_split": out[3],
            "main_tiles": (0, 0) if tail else (out[4], out[5]), "whole_tiles": out[4] if tail else 0,
            "estimate_us": out[6]}


class Graph:
    """A captured op sequence; run() replays it on the device's stream."""

    def __init__(self, dev: HipDevice, handle):
        self._dev, self._h = dev, handle

    def run(self) -> None:
        self._dev._call("zg_hip_graph_run", self._h)

    def free(self) -> None:
        if self._h is not None:
            self._dev._call("zg_hip_graph_free", self._h)
            self._h = None


class EdgePlan:
    """Both destination orderings of an edge list, built once (zg_hip_edge_plan_create)."""

    def __init__(self, dev, handle, src_indices, tgt_indices, n_nodes):
        self._dev, self.handle = dev, handle
        self.src_indices, self.tgt_indices, self.n_nodes = src_indices, tgt_indices, n_nodes

    def free(self) -> None:
        if self.handle is not None:
            self._dev._call("zg_hip_edge_plan_free", self.handle)
            self.handle = None


class Event:
    """A HIP event on the device's stream (timing only)."""

    def __init__(self, dev: HipDevice):
        self._dev = dev
        h = ctypes.c_void_p()
        dev._call("zg_hip_event_create", ctypes.byref(h))
        self._h = h

    def record(self) -> "Event":
        self._dev._call("zg_hip_event_record", self._h)
        return self

    def elapsed_ms(self, later: "Event") -> float:
        ms = ctypes.c_float()
        self._dev._lib.call("zg_hip_event_elapsed_ms", self._h, later._h, ctypes.byref(ms))
        return ms.value

    def __del__(self):
        try:
            if self._h is not None:
                self._dev._lib.cdll.zg_hip_event_destroy(self._h)
                self._h = None
        except Exception:
            pass
