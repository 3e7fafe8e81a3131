"""Minimal reader and writer of the reference's .mllm parameter container (mllm/Engine/ParameterReader.hpp:27-57):
268-byte head (u64 magic, char[256] model name, u32 count), then `count` 416-byte descriptors
(u32 id, u32 dtype, u64 size, u64 offset, u64 shape_len, u64 shape[16], char[256] name), then raw data."""
import struct

import numpy as np

MAGIC = 0x519ACE0519ACE000
DTYPES = {2: np.int8, 4: np.int32, 5: np.int64, 8: np.float16, 9: np.float32}


def read(path):
    raw = open(path, "rb").read()
    magic, name, count = struct.unpack_from("<Q256sI", raw, 0)
    assert magic == MAGIC, hex(magic)
    out = {}
    for i in range(count):
        off = 268 + 416 * i
        pid, dtype, size, data_off, shape_len = struct.unpack_from("<IIQQQ", raw, off)
        shape = struct.unpack_from("<16Q", raw, off + 32)[:shape_len]
        pname = struct.unpack_from("<256s", raw, off + 160)[0].split(b"\0", 1)[0].decode()
        arr = np.frombuffer(raw, dtype=DTYPES[dtype], count=size // np.dtype(DTYPES[dtype]).itemsize,
                            offset=data_off)
        out[pname] = arr.reshape(shape)
    return name.split(b"\0", 1)[0].decode(), out


def write(path, model_name, params):
    """params: name -> numpy array. Unpadded, as the C++ writer lays a file out
    (mllm/Engine/ParameterReader.cpp:114-181)."""
    codes = {np.dtype(v): k for k, v in DTYPES.items()}
    items = [(n, np.ascontiguousarray(a)) for n, a in params.items()]
    head = struct.pack("<Q256sI", MAGIC, model_name.encode(), len(items))
    off = 268 + 416 * len(items)
    descs, blobs = [], []
    for i, (n, a) in enumerate(items):
        shape = list(a.shape) + [0] * (16 - a.ndim)
        descs.append(struct.pack("<IIQQQ16Q256s", i, codes[a.dtype], a.nbytes, off, a.ndim, *shape, n.encode()))
        blobs.append(a.tobytes())
        off += a.nbytes
    with open(path, "wb") as f:
        f.write(head + b"".join(descs) + b"".join(blobs))
