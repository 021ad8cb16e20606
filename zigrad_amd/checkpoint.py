"""Checkpoints of device-resident tensors in the SafeTensors format.

The reference serialises a LayerMap by reading each tensor's host pointer (`tensor.get_data()`,
src/utils/layer_map.zig:334-378) and rebuilds tensors with `NDTensor.from_slice` (:381-448); neither step
works for memory the host cannot dereference.  Here every tensor is staged through a blocking device-to-host copy on
the way out and a host-to-device copy on the way in, one tensor at a time, so the peak host footprint is one tensor.
Optimizer state (Adam's m and v per parameter, the per-tensor-update counter t, src/nn/optim.zig:126-130, 189)
travels in the same file: m and v as tensors, scalars in the `__metadata__` string map.

File layout (the SafeTensors container): 8-byte little-endian header length, a JSON header
{name: {"dtype", "shape", "data_offsets": [begin, end]}, "__metadata__": {str: str}} padded with spaces to a
multiple of 8 bytes, then the tensors' bytes back to back in name order.
"""
from __future__ import annotations

import json
import struct
from pathlib import Path

import numpy as np

_DTYPES = {"F32": np.float32, "F64": np.float64, "I32": np.int32, "I64": np.int64, "U32": np.uint32, "U64": np.uint64,
           "U8": np.uint8}
_NAMES = {np.dtype(v): k for k, v in _DTYPES.items()}


def save_tensors(path, dev, tensors: dict, metadata: dict | None = None) -> None:
    """tensors: {key: (buffer, shape)} with dotted keys such as "layers.0.weights"."""
    header, offset = {}, 0
    names = sorted(tensors)
    for name in names:
        buf, shape = tensors[name]
        if int(np.prod(shape, dtype=np.int64)) != buf.n:
            raise ValueError(f"{name}: shape {list(shape)} does not match {buf.n} elements")
        if np.dtype(buf.dtype) not in _NAMES:
            raise ValueError(f"{name}: dtype {buf.dtype} has no SafeTensors name")
        header[name] = {"dtype": _NAMES[np.dtype(buf.dtype)], "shape": [int(s) for s in shape],
                        "data_offsets": [offset, offset + buf.nbytes]}
        offset += buf.nbytes
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    blob = json.dumps(header, separators=(",", ":")).encode()
    blob += b" " * (-len(blob) % 8)
    tmp = Path(str(path) + ".tmp")
    with open(tmp, "wb") as f:
        f.write(struct.pack("<Q", len(blob)))
        f.write(blob)
        for name in names:
            f.write(dev.to_numpy(tensors[name][0]).tobytes())  # blocking device-to-host copy, one tensor at a time
    tmp.replace(path)


def read_header(path) -> tuple[dict, int]:
    with open(path, "rb") as f:
        (n,) = struct.unpack("<Q", f.read(8))
        if n > 100 << 20:
            raise ValueError("implausible SafeTensors header length")
        header = json.loads(f.read(n))
    return header, 8 + n


def load_tensors(path, dev, tensors: dict) -> dict:
    """Fills the given buffers from the file (dtype and shape must match) and returns the metadata map."""
    header, base = read_header(path)
    meta = header.pop("__metadata__", {})
    missing = sorted(set(tensors) - set(header))
    if missing:
        raise KeyError(f"checkpoint lacks {missing}")
    with open(path, "rb") as f:
        for name, (buf, shape) in tensors.items():
            h = header[name]
            if _DTYPES[h["dtype"]] != np.dtype(buf.dtype).type or list(h["shape"]) != [int(s) for s in shape]:
                raise ValueError(f"{name}: file has {h['dtype']}{h['shape']}, expected {buf.dtype}{list(shape)}")
            begin, end = h["data_offsets"]
            f.seek(base + begin)
            host = np.frombuffer(f.read(end - begin), dtype=buf.dtype)
            dev.mem_transfer(host, buf, "HtoD")
    return meta
