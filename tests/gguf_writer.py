"""Test helper: writes a small GGUF v3 file with real payloads (tensor data aligned to 32 bytes, as gguf-py does)."""
import struct


def write_gguf(path, tensors, kvs=(), alignment=32):
    """tensors: [(name, shape, ggml_type, payload bytes)]; kvs: [(key, value_type, encoded value)]."""
    def s(x):
        b = x.encode()
        return struct.pack("<Q", len(b)) + b

    offsets, cursor = [], 0
    for _, _, _, payload in tensors:
        offsets.append(cursor)
        cursor = (cursor + len(payload) + alignment - 1) // alignment * alignment
    head = struct.pack("<IIQQ", 0x46554747, 3, len(tensors), len(kvs))
    for k, t, v in kvs:
        head += s(k) + struct.pack("<I", t) + v
    for (name, shape, typ, _), off in zip(tensors, offsets):
        head += s(name) + struct.pack("<I", len(shape)) + b"".join(struct.pack("<Q", d) for d in shape)
        head += struct.pack("<IQ", typ, off)
    data_start = (len(head) + alignment - 1) // alignment * alignment
    blob = bytearray(head + b"\0" * (data_start - len(head)))
    for (_, _, _, payload), off in zip(tensors, offsets):
        blob += b"\0" * (data_start + off - len(blob))
        blob += payload
    with open(path, "wb") as f:
        f.write(bytes(blob))
    return str(path)
