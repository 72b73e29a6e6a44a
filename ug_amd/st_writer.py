"""Writer for safetensors files (synthetic checkpoints for the tests and the benchmark; the format is 8 bytes of little-endian header
length, a JSON header, then the raw tensor bytes): a hand-written one that can store bf16, which
numpy has no type for, next to the `safetensors` package's own writer where that is enough."""
import json
import struct

import numpy as np

NP_OF = {"F32": np.float32, "F16": np.float16, "I32": np.int32, "I64": np.int64, "BF16": np.uint16, "U8": np.uint8, "F64": np.float64}


def write_safetensors(path, tensors, metadata=None, pad_header_to=8):
    """tensors: [(name, dtype string, shape, numpy array of raw elements (uint16 bits for BF16))]."""
    header, blobs, at = {}, [], 0
    if metadata is not None:
        header["__metadata__"] = metadata
    for name, dt, shape, arr in tensors:
        raw = np.ascontiguousarray(arr, dtype=NP_OF[dt]).tobytes()
        assert len(raw) == int(np.prod(shape, dtype=np.int64)) * np.dtype(NP_OF[dt]).itemsize, (name, len(raw), shape)
        header[name] = {"dtype": dt, "shape": list(shape), "data_offsets": [at, at + len(raw)]}
        blobs.append(raw)
        at += len(raw)
    h = json.dumps(header, separators=(",", ":")).encode()
    h += b" " * ((-len(h)) % pad_header_to)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(h)))
        f.write(h)
        for b in blobs:
            f.write(b)
