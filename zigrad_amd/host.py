"""Host-side shape logic that sits between Zigrad's tensors and the device ops.

These functions restate, for `DevBuf` operands, what the reference's NDArray / NDTensor layers do on
the host before they dispatch to a device: work out batch shapes and leading dimensions for bmm,
size the scratch for unbroadcast, turn gather indices into flat offsets, and issue the device GEMMs a
matmul's backward needs.  They run unchanged on any device object with `dispatch` and the `mem_*` API.
"""
from __future__ import annotations

import math


from .device import DevBuf, F32, U64


def _prod(xs) -> int:
    return int(math.prod(int(x) for x in xs))


def _broadcast_batch(a: list[int], b: list[int]) -> list[int]:
    """Right-aligned broadcast of two batch-dim lists (reference: src/ndarray/shape.zig:247-264)."""
    n = max(len(a), len(b))
    a = [1] * (n - len(a)) + list(a)
    b = [1] * (n - len(b)) + list(b)
    out = []
    for x, y in zip(a, b):
        if x != y and x != 1 and y != 1:
            raise ValueError(f"batch dims {a} and {b} do not broadcast")
        out.append(max(x, y))
    return out


def bmm_out_shape(a_shape, b_shape, trans_a: bool, trans_b: bool) -> list[int]:
    a_shape, b_shape = list(a_shape), list(b_shape)
    if len(a_shape) < 2:
        a_shape = [1] + a_shape
    if len(b_shape) < 2:
        b_shape = [1] + b_shape
    a_batch = a_shape[:-2] if len(a_shape) > 2 else [1]
    b_batch = b_shape[:-2] if len(b_shape) > 2 else [1]
    batch = [] if (len(a_shape) == 2 and len(b_shape) == 2) else _broadcast_batch(a_batch, b_batch)
    a_rows, a_cols = a_shape[-2:]
    b_rows, b_cols = b_shape[-2:]
    M = a_cols if trans_a else a_rows
    N = b_rows if trans_b else b_cols
    return batch + [M, N]


def bmm_acc_(dev, A: DevBuf, a_shape, B: DevBuf, b_shape, C: DevBuf, trans_a=False, trans_b=False, alpha=1.0,
             beta=0.0) -> list[int]:
    """C = alpha * op(A) op(B) + beta * C with batch broadcasting.  Reference: bmm_acc_impl,
    src/ndarray.zig:817-899 (shape logic, lda/ldb/ldc = physical column counts)."""
    a_shape, b_shape = list(a_shape), list(b_shape)
    if len(a_shape) < 2:
        a_shape = [1] + a_shape
    if len(b_shape) < 2:
        b_shape = [1] + b_shape
    a_batch = a_shape[:-2] if len(a_shape) > 2 else [1]
    b_batch = b_shape[:-2] if len(b_shape) > 2 else [1]
    batch = [] if (len(a_shape) == 2 and len(b_shape) == 2) else _broadcast_batch(a_batch, b_batch)
    a_rows, a_cols = a_shape[-2:]
    b_rows, b_cols = b_shape[-2:]
    M = a_cols if trans_a else a_rows
    K = a_rows if trans_a else a_cols
    N = b_rows if trans_b else b_cols
    if K != (b_cols if trans_b else b_rows):
        raise ValueError(f"incompatible matrix dimensions {a_rows}x{a_cols} and {b_rows}x{b_cols}")
    c_shape = batch + [M, N]
    if C.n < _prod(c_shape):
        raise ValueError("bmm_acc_: output buffer too small")
    dev.dispatch(
        "bmm_acc", A=A, B=B, C=C,
        A_shape=[_prod(a_batch), M, K], B_shape=[_prod(b_batch), K, N], C_shape=[_prod(batch), M, N],
        trans_a=trans_a, trans_b=trans_b, lda=a_cols, ldb=b_cols, ldc=N, alpha=alpha, beta=beta,
    )
    return c_shape


def bmm_acc_backward(dev, trans_a: bool, trans_b: bool, A: DevBuf, a_shape, B: DevBuf, b_shape, C_grad: DevBuf, c_shape,
                     A_grad: DevBuf | None, B_grad: DevBuf | None) -> None:
    """The device GEMMs BmmAccBwd issues (src/ndtensor.zig:1092-1136); grads are accumulated (beta = 1)."""
    if A_grad is not None:
        if not trans_a and not trans_b:      # MATMUL_AB:   dA += dC . B^T
            bmm_acc_(dev, C_grad, c_shape, B, b_shape, A_grad, False, True, 1.0, 1.0)
        elif trans_a and not trans_b:        # MATMUL_AtB:  dA += B . dC^T
            bmm_acc_(dev, B, b_shape, C_grad, c_shape, A_grad, False, True, 1.0, 1.0)
        elif not trans_a and trans_b:        # MATMUL_ABt:  dA += dC . B
            bmm_acc_(dev, C_grad, c_shape, B, b_shape, A_grad, False, False, 1.0, 1.0)
        else:                                # MATMUL_AtBt: dA += B^T . dC^T
            bmm_acc_(dev, B, b_shape, C_grad, c_shape, A_grad, True, True, 1.0, 1.0)
    if B_grad is not None:
        if not trans_a and not trans_b:      # dB += A^T . dC
            bmm_acc_(dev, A, a_shape, C_grad, c_shape, B_grad, True, False, 1.0, 1.0)
        elif trans_a and not trans_b:        # dB += A . dC
            bmm_acc_(dev, A, a_shape, C_grad, c_shape, B_grad, False, False, 1.0, 1.0)
        elif not trans_a and trans_b:        # dB += dC^T . A
            bmm_acc_(dev, C_grad, c_shape, A, a_shape, B_grad, True, False, 1.0, 1.0)
        else:                                # dB += dC^T . A^T
            bmm_acc_(dev, C_grad, c_shape, A, a_shape, B_grad, True, True, 1.0, 1.0)


def unbroadcast_(dev, x: DevBuf, x_shape, out: DevBuf, out_shape, alpha=1.0, beta=0.0) -> None:
    """Reduce a broadcast gradient back to an operand's shape.  Reference: NDArray.unbroadcast_,
    src/ndarray.zig:687-730 (scratch sizing) + the device op."""
    x_shape, out_shape = list(x_shape), list(out_shape)
    if len(x_shape) < len(out_shape) or _prod(x_shape) % _prod(out_shape) != 0:
        raise ValueError(f"cannot unbroadcast {x_shape} to {out_shape}")
    n = dev.unbroadcast_scratch_len(x_shape, out_shape)
    scratch = dev.mem_scratch(F32, n) if n else None
    dev.dispatch("unbroadcast", x=x, x_shape=x_shape, y=out, y_shape=out_shape, scratch=scratch, alpha=alpha, beta=beta)


def gather(dev, src: DevBuf, src_shape, indices: DevBuf, idx_shape, dim: int, return_offsets: bool = False,
           check: bool = True):
    """values[i] = src[coord(i) with coord[dim] := indices[i]].  Reference: NDArray.gather,
    src/ndarray.zig:593-633; the offsets are computed by a device op instead of a host loop.  `check` reads the
    out-of-bounds status back (one blocking 4-byte copy); without it out-of-range indices are skipped silently."""
    src_shape, idx_shape = list(src_shape), list(idx_shape)
    if len(src_shape) != len(idx_shape):
        raise ValueError("gather: rank mismatch")
    n = _prod(idx_shape)
    # the reference takes the offsets from the raw allocator (its own "TODO: cache?"); on a GPU that would be a
    # hipMalloc/hipFree pair per call, so they come from the caching allocator (free with mem_cache_free)
    offsets = dev.mem_cache_alloc(U64, n)
    values = dev.mem_cache_alloc(F32, n)
    status = dev.gather(src, src_shape, idx_shape, indices, dim, offsets, values, check=check)
    if status:
        dev.mem_cache_free(values)
        dev.mem_cache_free(offsets)
        raise ValueError("InvalidIndexShape") if status == 1 else IndexError("IndexOutOfBounds")
    if return_offsets:
        return values, offsets
    dev.mem_cache_free(offsets)
    return values, None


def broadcast_shape(a, b) -> list[int]:
    """Right-aligned broadcast of two shapes (reference: Shape.broadcast, src/ndarray/shape.zig:247-264)."""
    return _broadcast_batch(list(a), list(b))


def elwise(dev, op: str, x: DevBuf, x_shape, y: DevBuf, y_shape):
    """z = x op y into a fresh buffer of the broadcast shape.  Reference: NDArray.elwise_alloc,
    src/ndarray.zig:231-246 (the device op does the modulo broadcasting).  Returns (z, z_shape); free z with
    mem_cache_free."""
    z_shape = broadcast_shape(x_shape, y_shape)
    z = dev.mem_cache_alloc(F32, _prod(z_shape))
    dev.dispatch(op, x=x, y=y, z=z)
    return z, z_shape


def mul_backward(dev, a: DevBuf, a_shape, b: DevBuf, b_shape, c_grad: DevBuf, c_shape, a_grad: DevBuf | None,
                 b_grad: DevBuf | None) -> None:
    """The device ops MulBwd issues (src/ndtensor.zig:836-868): a.grad += unbroadcast(b * dc),
    b.grad += unbroadcast(a * dc)."""
    for own_grad, own_shape, other, other_shape in ((a_grad, a_shape, b, b_shape), (b_grad, b_shape, a, a_shape)):
        if own_grad is None:
            continue
        t, t_shape = elwise(dev, "mul", other, other_shape, c_grad, c_shape)
        unbroadcast_(dev, t, t_shape, own_grad, own_shape, alpha=1.0, beta=1.0)
        dev.mem_cache_free(t)


def div_backward(dev, a: DevBuf, a_shape, b: DevBuf, b_shape, c_grad: DevBuf, c_shape, a_grad: DevBuf | None,
                 b_grad: DevBuf | None) -> None:
    """The device ops DivBwd issues (src/ndtensor.zig:871-907): a.grad += unbroadcast(dc / b);
    b.grad -= unbroadcast((dc * a) / (b * b))  (alpha = -1, beta = 1)."""
    if a_grad is not None:
        t, t_shape = elwise(dev, "div", c_grad, c_shape, b, b_shape)
        unbroadcast_(dev, t, t_shape, a_grad, a_shape, alpha=1.0, beta=1.0)
        dev.mem_cache_free(t)
    if b_grad is not None:
        num, num_shape = elwise(dev, "mul", c_grad, c_shape, a, a_shape)
        bsq, bsq_shape = elwise(dev, "mul", b, b_shape, b, b_shape)
        t, t_shape = elwise(dev, "div", num, num_shape, bsq, bsq_shape)
        dev.mem_cache_free(num)
        dev.mem_cache_free(bsq)
        unbroadcast_(dev, t, t_shape, b_grad, b_shape, alpha=-1.0, beta=1.0)
        dev.mem_cache_free(t)


def dot_backward(dev, a: DevBuf, b: DevBuf, c_grad: DevBuf, a_grad: DevBuf | None, b_grad: DevBuf | None) -> None:
    """DotBwd (src/ndtensor.zig:1142-1160): two axpy whose alpha is the one-element gradient of the result, read
    through a pointer into device memory."""
    if a_grad is not None:
        dev.dispatch("axpy", x=b, y=a_grad, alpha=c_grad)
    if b_grad is not None:
        dev.dispatch("axpy", x=a, y=b_grad, alpha=c_grad)


def matvec_backward(dev, A: DevBuf, a_shape, x: DevBuf, y_grad: DevBuf, A_grad: DevBuf | None, x_grad: DevBuf | None,
                    trans_a: bool = False) -> None:
    """MatvecBwd (src/ndtensor.zig:1225-1252): A.grad += outer(dy, x) (operands swapped when trans_a);
    x.grad += op(A)^T . dy, issued with the reference's own m / n (the matrix's dimensions exchanged and the
    transpose flag flipped), which describes the stored matrix correctly only when it is square."""
    rows, cols = int(a_shape[0]), int(a_shape[1])
    if A_grad is not None:
        dev.dispatch("outer", x=(x if trans_a else y_grad), y=(y_grad if trans_a else x), A=A_grad, alpha=1.0)
    if x_grad is not None:
        m, n = (cols, rows) if not trans_a else (rows, cols)
        dev.dispatch("matvec", A=A, x=y_grad, y=x_grad, m=m, n=n, trans_a=not trans_a, alpha=1.0, beta=1.0)
