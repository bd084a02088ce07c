"""Writes MKIM files for the loader tests: the layout rules of BinWriter (src/weights.rs:70-170), restated.

Blob offsets in write order: routed-expert tensors (name contains ".block_sparse_moe.experts." and ends in .w1/.w2/.w3,
src/weights.rs:417-419) start on an `expert_align` boundary (4096 by default), everything else on 64; padding is zeros.
The loader is checked against three things: tests/golden/mkim_ref.bin, a file written by the reference's own exporter
(nano/export.py), files made here by these rules, and a header assembled byte by byte in the test itself.
"""
import json
import struct

import numpy as np

F32, MXFP4, I32, VQ1, MXFP4SQ = 0, 1, 2, 3, 4


def is_expert_tensor(name):
    return ".block_sparse_moe.experts." in name and name.endswith((".w1", ".w2", ".w3"))


def blob_bytes(dtype, value):
    if dtype == F32:
        return np.ascontiguousarray(value, dtype="<f4").tobytes()
    if dtype == I32:
        return np.ascontiguousarray(value, dtype="<i4").tobytes()
    if dtype == MXFP4:
        packed, scales = value
        return np.ascontiguousarray(packed, np.uint8).tobytes() + np.ascontiguousarray(scales, np.uint8).tobytes()
    return bytes(value)  # VQ1 / MXFP4SQ: raw bytes supplied by the test


def write(path, tensors, config=None, expert_align=4096):
    """tensors: list of (name, dtype, dims, value).  config: dict -> MKIM0002, None -> MKIM0001.  Returns {name: offset}."""
    blobs = [blob_bytes(dt, v) for _, dt, _, v in tensors]
    cfg = json.dumps(config).encode("utf-8") if config is not None else None
    prefix = 8 if cfg is None else 8 + 4 + len(cfg)
    dir_size = sum(2 + len(n.encode("utf-8")) + 1 + 1 + 4 * len(dims) + 8 + 8 for n, _, dims, _ in tensors)
    pos = prefix + 4 + dir_size
    offsets = []
    for (name, _, _, _), b in zip(tensors, blobs):
        align = expert_align if is_expert_tensor(name) else 64
        pos = (pos + align - 1) // align * align
        offsets.append(pos)
        pos += len(b)
    out = bytearray()
    if cfg is None:
        out += b"MKIM0001"
    else:
        out += b"MKIM0002" + struct.pack("<I", len(cfg)) + cfg
    out += struct.pack("<I", len(tensors))
    for (name, dt, dims, _), b, off in zip(tensors, blobs, offsets):
        nb = name.encode("utf-8")
        out += struct.pack("<H", len(nb)) + nb + struct.pack("<BB", dt, len(dims))
        out += b"".join(struct.pack("<I", d) for d in dims) + struct.pack("<QQ", off, len(b))
    for b, off in zip(blobs, offsets):
        out += b"\0" * (off - len(out))
        out += b
    with open(path, "wb") as f:
        f.write(out)
    return {t[0]: o for t, o in zip(tensors, offsets)}
