"""Writes GGUF v3 files for the reader / loader tests: the public container layout (magic, version, counts,
metadata key-values, tensor table, aligned data section).  Test infrastructure only."""
import struct

import numpy as np

U8, I8, U16, I16, U32, I32, F32, BOOL, STR, ARR, U64, I64, F64 = range(13)
_FMT = {U8: "<B", I8: "<b", U16: "<H", I16: "<h", U32: "<I", I32: "<i", F32: "<f", BOOL: "<B", U64: "<Q", I64: "<q", F64: "<d"}


def _s(text: str) -> bytes:
    b = text.encode()
    return struct.pack("<Q", len(b)) + b


def _scalar(vt: int, v) -> bytes:
    return _s(v) if vt == STR else struct.pack(_FMT[vt], v)


def write(path, metadata, tensors, version=3, alignment=32, magic=0x46554747):
    """metadata: list of (key, value type, value) or (key, ARR, (element type, values)).
    tensors: list of (name, ggml type, dims with dims[0] the contiguous one, raw bytes)."""
    head = struct.pack("<IIQQ", magic, version, len(tensors), len(metadata))
    for key, vt, v in metadata:
        head += _s(key) + struct.pack("<I", vt)
        if vt == ARR:
            et, vals = v
            head += struct.pack("<IQ", et, len(vals)) + b"".join(_scalar(et, x) for x in vals)
        else:
            head += _scalar(vt, v)
    blobs, off = [], 0
    for name, ty, dims, raw in tensors:
        raw = np.ascontiguousarray(raw).view(np.uint8).reshape(-1)
        head += _s(name) + struct.pack("<I", len(dims)) + b"".join(struct.pack("<Q", d) for d in dims) + struct.pack("<IQ", ty, off)
        blobs.append((off, raw))
        off = (off + raw.size + alignment - 1) // alignment * alignment
    data_off = (len(head) + alignment - 1) // alignment * alignment
    with open(path, "wb") as f:
        f.write(head + b"\0" * (data_off - len(head)))
        for o, raw in blobs:
            f.seek(data_off + o)
            f.write(raw.tobytes())
        f.truncate(data_off + off)
    return data_off
