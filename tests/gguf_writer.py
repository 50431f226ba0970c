"""Writes small GGUF v3 files for the tests (header, key/value table, tensor table, aligned data), following the
format the reference's loader reads (src/graph/gguf/loader.cpp:577-770)."""
import struct

import numpy as np

GGML_TYPE = {"f32": 0, "f16": 1, "q4_0": 2, "q4_1": 3, "q5_0": 6, "q5_1": 7, "q8_0": 8, "q8_1": 9, "q2_k": 10,
             "q3_k": 11, "q4_k": 12, "q5_k": 13, "q6_k": 14, "q8_k": 15, "i32": 26}


def _string(s: str) -> bytes:
    b = s.encode()
    return struct.pack("<Q", len(b)) + b


def _value(v) -> bytes:
    if isinstance(v, bool):
        return struct.pack("<IB", 7, int(v))
    if isinstance(v, int):
        return struct.pack("<II", 4, v)
    if isinstance(v, float):
        return struct.pack("<If", 6, v)
    if isinstance(v, str):
        return struct.pack("<I", 8) + _string(v)
    if isinstance(v, (list, tuple)) and v and isinstance(v[0], str):
        return struct.pack("<IIQ", 9, 8, len(v)) + b"".join(_string(x) for x in v)
    if isinstance(v, (list, tuple)):
        return struct.pack("<IIQ", 9, 5, len(v)) + struct.pack(f"<{len(v)}i", *v)
    raise TypeError(type(v))


def write_gguf(path, tensors, kv=None, alignment=32, version=3, declare_alignment=True):
    """tensors: list of (name, type name, ne: GGUF dimensions innermost first, payload bytes / array)."""
    kv = dict(kv or {})
    if declare_alignment:
        kv["general.alignment"] = alignment
    head = struct.pack("<IIQQ", 0x46554747, version, len(tensors), len(kv))
    for k, v in kv.items():
        head += _string(k) + _value(v)
    payloads, infos, off = [], b"", 0
    for name, tname, ne, data in tensors:
        raw = np.ascontiguousarray(data).tobytes()
        infos += _string(name) + struct.pack("<I", len(ne)) + struct.pack(f"<{len(ne)}Q", *ne)
        infos += struct.pack("<IQ", GGML_TYPE[tname], off)
        pad = (-len(raw)) % alignment
        payloads.append(raw + b"\0" * pad)
        off += len(raw) + pad
    body = head + infos
    body += b"\0" * ((-len(body)) % alignment)
    with open(path, "wb") as f:
        f.write(body + b"".join(payloads))
    return path
