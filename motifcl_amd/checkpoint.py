"""MCLTEN1/2 single-tensor files of MotifCL (src/serialization.cpp:21-63,121-136) for numpy arrays.

The same layout as motifcl_amd/host/src/serialization.cpp writes: magic, int32 dtype, uint64 ndim,
int64 dims, uint64 nbytes, (version 2) float quant_scale, int32 has_quant_scales, int32
quant_scale_axis, int64 quant_block_size, payload.  Only the unquantized dtypes of the counter
path are handled (F32 = 0, F16 = 1, I32 = 2, U8 = 3).
"""
import os
import struct

import numpy as np

MAGIC_V1 = b"MCLTEN1\0"
MAGIC_V2 = b"MCLTEN2\0"
_DTYPES = {0: np.dtype("<f4"), 1: np.dtype("<f2"), 2: np.dtype("<i4"), 3: np.dtype("u1")}
_CODES = {v: k for k, v in _DTYPES.items()}
MAX_RANK = 8


class CheckpointError(ValueError):
    pass


def save_tensor(array, path):
    a = np.ascontiguousarray(array)
    if a.dtype.newbyteorder("<") not in _CODES and a.dtype not in _CODES:
        raise CheckpointError("dtype %s is not storable in a MotifCL tensor file" % a.dtype)
    a = a.astype(a.dtype.newbyteorder("<"), copy=False)
    head = MAGIC_V2 + struct.pack("<iQ", _CODES[a.dtype], a.ndim)
    head += b"".join(struct.pack("<q", d) for d in a.shape)
    head += struct.pack("<QfiiQ", a.nbytes, 1.0, 0, -1, 0)
    with open(path, "wb") as f:
        f.write(head)
        f.write(a.tobytes())


def load_tensor(path):
    with open(path, "rb") as f:
        data = f.read()
    pos = 0

    def take(fmt):
        nonlocal pos
        size = struct.calcsize(fmt)
        if pos + size > len(data):
            raise CheckpointError("failed to read serialization stream")
        out = struct.unpack_from(fmt, data, pos)
        pos += size
        return out[0] if len(out) == 1 else out

    magic = data[:8]
    pos = 8
    if len(data) < 8 or magic not in (MAGIC_V1, MAGIC_V2):
        raise CheckpointError("serialization magic mismatch")
    code = take("<i")
    if code not in _DTYPES:
        raise CheckpointError("serialized tensor has a dtype the counter path does not store")
    ndim = take("<Q")
    if ndim > MAX_RANK:
        raise CheckpointError("serialized tensor rank is implausible")
    dims = [take("<q") for _ in range(ndim)]
    if any(d < 0 for d in dims):
        raise CheckpointError("serialized tensor has a negative dimension")
    nbytes = take("<Q")
    if magic == MAGIC_V2:
        take("<f")
        if take("<i") != 0:
            raise CheckpointError("serialized tensor carries quantization scales (not supported)")
        take("<i")
        take("<q")
    dt = _DTYPES[code]
    numel = int(np.prod(dims, dtype=np.int64)) if dims else 1
    if numel * dt.itemsize != nbytes:
        raise CheckpointError("serialized tensor byte size does not match dtype/shape")
    if pos + nbytes > len(data):
        raise CheckpointError("failed to read tensor payload")
    return np.frombuffer(data, dtype=dt, count=numel, offset=pos).reshape(dims).copy()


def save_counter_layer(prefix, state, scale, v):
    """<prefix>_state.mt / _scale.mt / _v.mt as tools/train_ternary15m.cpp:204-228 names them."""
    save_tensor(np.asarray(state, dtype=np.uint8), prefix + "_state.mt")
    save_tensor(np.asarray(scale, dtype=np.float32), prefix + "_scale.mt")
    save_tensor(np.asarray(v, dtype=np.float32), prefix + "_v.mt")


def load_counter_layer(prefix, in_features, out_features):
    state, scale, v = (load_tensor(prefix + s) for s in ("_state.mt", "_scale.mt", "_v.mt"))
    if state.dtype != np.uint8 or state.size != out_features * (in_features // 4) * 3:
        raise CheckpointError("counter checkpoint: state does not fit the layer")
    if scale.dtype != np.float32 or v.dtype != np.float32 or scale.size != out_features or v.size != out_features:
        raise CheckpointError("counter checkpoint: scale / v do not fit the layer")
    return state.reshape(-1), scale.reshape(-1), v.reshape(-1)
