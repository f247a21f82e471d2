"""A minimal GGUF v3 writer for the tests: metadata of the scalar, string and array kinds and
tensors given as raw block bytes (the layout ggml/docs/gguf.md describes)."""
import struct

import numpy as np


def _s(b):
    b = b.encode("utf-8")
    return struct.pack("<Q", len(b)) + b


def _value(v):
    if isinstance(v, bool):
        return 7, struct.pack("<B", 1 if v else 0)
    if isinstance(v, int):
        return (4, struct.pack("<I", v)) if 0 <= v < 2 ** 32 else (11, struct.pack("<q", v))
    if isinstance(v, float):
        return 6, struct.pack("<f", v)
    if isinstance(v, str):
        return 8, _s(v)
    if isinstance(v, (list, tuple)):
        et = _value(v[0])[0] if v else 4
        return 9, struct.pack("<IQ", et, len(v)) + b"".join(_value(x)[1] for x in v)
    raise TypeError(type(v))


def write_gguf(path, metadata, tensors, version=3, alignment=None):
    """TENSORS: list of (name, dims in ggml order, ggml type code, uint8 array of the blocks)."""
    md = dict(metadata)
    if alignment is not None:
        md["general.alignment"] = alignment
    a = md.get("general.alignment", 32)
    head = struct.pack("<IIQQ", 0x46554747, version, len(tensors), len(md))
    for k, v in md.items():
        t, b = _value(v)
        head += _s(k) + struct.pack("<I", t) + b
    off, infos = 0, b""
    for name, dims, code, raw in tensors:
        infos += _s(name) + struct.pack("<I", len(dims)) + b"".join(struct.pack("<Q", d) for d in dims) + struct.pack("<IQ", code, off)
        off += (np.asarray(raw).size + a - 1) // a * a
    head += infos
    pad = (-len(head)) % a
    with open(path, "wb") as f:
        f.write(head + b"\0" * pad)
        for _, _, _, raw in tensors:
            raw = np.ascontiguousarray(raw, np.uint8).ravel()
            f.write(raw.tobytes() + b"\0" * ((-raw.size) % a))
