"""Test helper: writes GGUF files the way `gguf_file::write` does (candle-core/src/quantized/gguf_file.rs:534-582):
magic, version, counts, metadata (`Value::write`, :359-399), tensor table with dimensions innermost first and
offsets of 32-byte-padded tensors, padding to 32, tensor bytes each padded to 32.  Versions 1 (u32 counts and
string lengths, :139-145, :443-455) and 3 are written with the same body so that the reader's three
branches can be exercised."""
import struct

import numpy as np

U8, I8, U16, I16, U32, I32, F32, BOOL, STRING, ARRAY, U64, I64, F64 = range(13)
_FMT = {U8: "<B", I8: "<b", U16: "<H", I16: "<h", U32: "<I", I32: "<i", F32: "<f", BOOL: "<B", U64: "<Q", I64: "<q", F64: "<d"}
# GgmlDType id -> (block elements, block bytes), candle-core/src/quantized/mod.rs:153-174, 218-252
GEOMETRY = {0: (1, 4), 1: (1, 2), 2: (32, 18), 3: (32, 20), 6: (32, 22), 7: (32, 24), 8: (32, 34), 9: (32, 36),
            10: (256, 84), 11: (256, 110), 12: (256, 144), 13: (256, 176), 14: (256, 210), 15: (256, 292), 30: (1, 2)}


def _count(n, version):
    return struct.pack("<I" if version == 1 else "<Q", n)


def _string(s, version):
    b = s if isinstance(s, bytes) else s.encode()
    return _count(len(b), version) + b


def _value(vt, v, version):
    if vt == STRING:
        return _string(v, version)
    if vt == ARRAY:
        et, items = v
        return struct.pack("<I", et) + _count(len(items), version) + b"".join(_value(et, x, version) for x in items)
    return struct.pack(_FMT[vt], v)


def write_gguf(path, metadata, tensors, version=2, alignment=32, magic=0x46554747):
    """metadata: list of (key, value type id, value); arrays take (element type id, [items]).
    tensors: list of (name, ggml dtype id, shape outermost-first, bytes-like)."""
    out = bytearray()
    out += struct.pack("<II", magic, version)
    out += _count(len(tensors), version) + _count(len(metadata), version)
    for key, vt, v in metadata:
        out += _string(key, version) + struct.pack("<I", vt) + _value(vt, v, version)
    offset, offsets = 0, []
    for name, dt, shape, data in tensors:
        out += _string(name, version) + struct.pack("<I", len(shape))
        for d in reversed(shape):
            out += _count(d, version)
        out += struct.pack("<IQ", dt, offset)
        offsets.append(offset)
        n = len(bytes(data))
        offset += n + (alignment - 1 - (alignment - 1 + n) % alignment)
    out += b"\0" * (alignment - 1 - (alignment - 1 + len(out)) % alignment)
    data_start = len(out)
    for off, (name, dt, shape, data) in zip(offsets, tensors):
        assert data_start + off == len(out)
        b = bytes(data)
        out += b + b"\0" * (alignment - 1 - (alignment - 1 + len(b)) % alignment)
    with open(path, "wb") as f:
        f.write(out)
    return data_start


def moe_layer_file(path, layer, gate, w1, w3, w2, dtype, top_k, gate_dtype=0, gate_blocks=None, extra_metadata=(), version=2,
                   down_dtype=None, expert_keys=True):
    """One MoE layer under the names `ModelWeights::from_gguf` reads (quantized_llama.rs:506-512, 553-578)."""
    E, H = gate.shape
    F = np.asarray(w1[0]).size // (H // GEOMETRY[dtype][0] * GEOMETRY[dtype][1])
    md = [("general.architecture", STRING, "llama"), ("llama.embedding_length", U32, H)] + list(extra_metadata)
    if expert_keys:
        md += [("llama.expert_count", U32, E), ("llama.expert_used_count", U32, top_k)]
    if gate_dtype == 0:
        gbytes = np.ascontiguousarray(gate, dtype=np.float32).tobytes()
    elif gate_dtype == 1:
        gbytes = np.ascontiguousarray(gate, dtype=np.float16).tobytes()
    else:
        gbytes = np.asarray(gate_blocks).tobytes()  # the gate quantised by the caller
    ts = [("blk.%d.ffn_gate_inp.weight" % layer, gate_dtype, (E, H), gbytes)]
    for e in range(E):
        ts.append(("blk.%d.ffn_gate.%d.weight" % (layer, e), dtype, (F, H), np.asarray(w1[e]).tobytes()))
        ts.append(("blk.%d.ffn_down.%d.weight" % (layer, e), dtype if down_dtype is None else down_dtype, (H, F), np.asarray(w2[e]).tobytes()))
        ts.append(("blk.%d.ffn_up.%d.weight" % (layer, e), dtype, (F, H), np.asarray(w3[e]).tobytes()))
    return write_gguf(path, md, ts, version=version)
