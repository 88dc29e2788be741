"""A minimal GGUF writer for the tests: header, metadata of every scalar kind plus arrays,
tensor index, aligned data.  Layout per the container the reference parses
(crates/ojas-formats/src/gguf.rs:100-206)."""
import struct

import numpy as np

U8, I8, U16, I16, U32, I32, F32, BOOL, STR, ARR, U64, I64, F64 = range(13)
_FMT = {U8: "<B", I8: "<b", U16: "<H", I16: "<h", U32: "<I", I32: "<i", F32: "<f", BOOL: "<B", U64: "<Q", I64: "<q", F64: "<d"}


def _s(x: str) -> bytes:
    b = x.encode()
    return struct.pack("<Q", len(b)) + b


def _val(t: int, v) -> bytes:
    if t == STR:
        return _s(v)
    if t == ARR:
        et, items = v
        return struct.pack("<IQ", et, len(items)) + b"".join(_val(et, i) for i in items)
    return struct.pack(_FMT[t], v)


def write_gguf(path, meta: list, tensors: list, version: int = 3, alignment: int | None = None,
               truncate: int | None = None) -> dict:
    """meta: [(key, type, value)], tensors: [(name, dims, ggml_type, bytes)].
    Returns {name: absolute data offset}."""
    if alignment is not None:
        meta = meta + [("general.alignment", U32, alignment)]
    align = alignment or 32
    head = b"GGUF" + struct.pack("<IQQ", version, len(tensors), len(meta))
    for k, t, v in meta:
        head += _s(k) + struct.pack("<I", t) + _val(t, v)
    rel, blobs, infos = 0, [], b""
    rels = {}
    for name, dims, ty, data in tensors:
        data = np.ascontiguousarray(data).view(np.uint8).tobytes()
        infos += _s(name) + struct.pack("<I", len(dims)) + b"".join(struct.pack("<Q", d) for d in dims) + struct.pack("<IQ", ty, rel)
        rels[name] = rel
        blobs.append(data)
        rel += (len(data) + align - 1) // align * align
    head += infos
    start = (len(head) + align - 1) // align * align
    body = b""
    for data in blobs:
        body += data + b"\0" * ((len(data) + align - 1) // align * align - len(data))
    blob = head + b"\0" * (start - len(head)) + body
    if truncate is not None:
        blob = blob[:truncate]
    with open(path, "wb") as f:
        f.write(blob)
    return {n: start + r for n, r in rels.items()}
