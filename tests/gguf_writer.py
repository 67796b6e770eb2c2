"""A minimal GGUF writer for the loader tests: header, typed metadata, tensor directory, aligned
data region, as gguf.h lays them out.  Knobs exist to write the malformed files the tests need."""
import struct

# metadata value types
U8, I8, U16, I16, U32, I32, F32, BOOL, STR, ARR, U64, I64, F64 = range(13)
_FMT = {U8: "<B", I8: "<b", U16: "<H", I16: "<h", U32: "<I", I32: "<i", F32: "<f", BOOL: "<B", U64: "<Q", I64: "<q",
        F64: "<d"}
GGML = {"F32": 0, "F16": 1, "Q4_0": 2, "Q4_1": 3, "Q5_0": 6, "Q5_1": 7, "Q8_0": 8, "Q2K": 10, "Q3K": 11, "Q4K": 12,
        "Q5K": 13, "Q6K": 14, "IQ4_NL": 20, "IQ4_XS": 23, "I32": 26, "BF16": 30, "TQ1_0": 34, "TQ2_0": 35, "I2S": 36,
        "MXFP4": 39, "NVFP4": 40, "Q2_0": 42}


def gstr(s) -> bytes:
    b = s if isinstance(s, bytes) else s.encode()
    return struct.pack("<Q", len(b)) + b


def value(vtype, v) -> bytes:
    if vtype == STR:
        return gstr(v)
    if vtype == ARR:
        et, items = v
        return struct.pack("<IQ", et, len(items)) + b"".join(value(et, it) for it in items)
    return struct.pack(_FMT[vtype], v)


def build(meta, tensors, version=3, alignment=32, magic=0x46554747, declared_tensors=None, dims_override=None) -> bytes:
    """meta: [(key, vtype, value)]; tensors: [(name, shape in file order, ggml type, data bytes)]."""
    head = struct.pack("<IIQQ", magic, version, len(tensors) if declared_tensors is None else declared_tensors, len(meta))
    for key, vtype, v in meta:
        head += gstr(key) + struct.pack("<I", vtype) + value(vtype, v)
    off, offsets = 0, []
    for _, _, _, data in tensors:
        offsets.append(off)
        off = (off + len(data) + alignment - 1) // alignment * alignment if alignment else off + len(data)
    for (name, shape, gt, _), o in zip(tensors, offsets):
        nd = len(shape) if dims_override is None else dims_override
        head += gstr(name) + struct.pack("<I", nd) + b"".join(struct.pack("<Q", d) for d in shape)
        head += struct.pack("<IQ", gt, o)
    a = alignment if alignment and alignment & (alignment - 1) == 0 and alignment <= (16 << 20) else 32
    body = head + b"\0" * (-len(head) % a)
    for (_, _, _, data), o in zip(tensors, offsets):
        body += b"\0" * (o - (len(body) - len(head) - (-len(head) % a)))
        body += bytes(data)
    return body


def write(path, *args, **kw) -> None:
    with open(path, "wb") as f:
        f.write(build(*args, **kw))
