"""Writers for the constant files ``allocConstantNVGPUF16/F32(idx)`` load from
``$HOM_CONSTANT_DIR``: the reference's text format (first line the three extents,
then the values in decimal; lib/WeightsEngine/WeightsEngine.cpp:22-62 writes it,
lib/ExecutionEngine/HandsOnNVGPURunnerUtils.cu:224-298 reads it) and the binary
format the library prefers when ``<idx>.bin`` exists (40-byte header: magic
``HOMW``, version 1, bytes per element, rank 3, three int64 extents; then the
values, row-major, little endian)."""
import os
import struct

import numpy as np


def _as3d(array):
    a = np.asarray(array)
    if a.ndim > 3:
        raise ValueError("constants are rank <= 3")
    return a.reshape((1,) * (3 - a.ndim) + a.shape)


def write_text(directory, idx, array):
    a = _as3d(array)
    path = os.path.join(directory, f"{idx}.txt")
    with open(path, "w") as f:
        f.write(" ".join(str(d) for d in a.shape) + "\n")
        # repr of the float32 value: shortest text that reads back to the same value
        f.write(" ".join(repr(float(v)) for v in a.astype(np.float32).ravel()))
        f.write("\n")
    return path


def write_binary(directory, idx, array):
    a = _as3d(array)
    if a.dtype not in (np.float16, np.float32):
        raise ValueError("binary constants hold fp16 or fp32 values")
    path = os.path.join(directory, f"{idx}.bin")
    with open(path, "wb") as f:
        f.write(struct.pack("<4sIIIqqq", b"HOMW", 1, a.dtype.itemsize, 3, *a.shape))
        f.write(np.ascontiguousarray(a).astype(a.dtype.newbyteorder("<"), copy=False).tobytes())
    return path
