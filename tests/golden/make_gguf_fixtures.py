"""Writes the hand-assembled GGUF byte fixtures gguf_v1.hex.txt / gguf_v2.hex.txt / gguf_v3.hex.txt.

Every field is laid down here one by one with the width `Content::read` takes for it
(candle-core/src/quantized/gguf_file.rs: magic and version :34-46, counts :443-454, `read_string` :135-150,
`Value::read` :318-357, value type ids :402-420, tensor infos :464-492, `general.alignment` and the start of the tensor
data :494-505), independently of tests/gguf_writer.py.  The output is text: one field per line, its bytes in hex, then
what the field is, so that a reader can check the layout against the reference by eye; tests/test_gguf_cpu.py turns the
hex back into a file and reads it through the library.

    python tests/golden/make_gguf_fixtures.py
"""
import os
import struct

HERE = os.path.dirname(os.path.abspath(__file__))


class Hex:
    def __init__(self):
        self.lines, self.n = [], 0

    def put(self, raw, what):
        self.lines.append("%-50s # @%d %s" % (raw.hex(), self.n, what))
        self.n += len(raw)

    def u8(self, v, what): self.put(struct.pack("<B", v), what)
    def i8(self, v, what): self.put(struct.pack("<b", v), what)
    def u16(self, v, what): self.put(struct.pack("<H", v), what)
    def i16(self, v, what): self.put(struct.pack("<h", v), what)
    def u32(self, v, what): self.put(struct.pack("<I", v), what)
    def i32(self, v, what): self.put(struct.pack("<i", v), what)
    def u64(self, v, what): self.put(struct.pack("<Q", v), what)
    def i64(self, v, what): self.put(struct.pack("<q", v), what)
    def f32(self, v, what): self.put(struct.pack("<f", v), what)
    def f64(self, v, what): self.put(struct.pack("<d", v), what)

    def count(self, v, version, what):
        # v1 stores counts, string lengths and dimensions as u32, v2 and v3 as u64 (:137-141, :443-454, :468-479)
        (self.u32 if version == 1 else self.u64)(v, what)

    def string(self, s, version, what):
        self.count(len(s), version, "length of " + what)
        self.put(s, what)

    def pad_to(self, alignment, what):
        k = (-self.n) % alignment
        if k:
            self.put(b"\0" * k, what)

    def save(self, name, header):
        with open(os.path.join(HERE, name), "w") as f:
            f.write("".join("# %s\n" % h for h in header))
            f.write("\n".join(self.lines) + "\n")


def q4k_payload():
    """Two BlockQ4K (144 bytes each): bytes (7 i + 3) mod 256."""
    return bytes((7 * i + 3) & 0xFF for i in range(288))


def f32_payload():
    return struct.pack("<4f", 1.0, -2.5, 0.0, 1e-3)


def build(version, alignment):
    h = Hex()
    h.put(b"GGUF", "magic 0x46554747 read as a little-endian u32")
    h.u32(version, "version")
    h.count(2, version, "tensor count")
    kv = 15 if alignment else 14
    h.count(kv, version, "metadata key-value count")

    def key(name, type_id, type_name):
        h.string(name.encode(), version, "key '%s'" % name)
        h.u32(type_id, "value type %s" % type_name)

    key("t.u8", 0, "U8"); h.u8(200, "value 200")
    key("t.i8", 1, "I8"); h.i8(-100, "value -100")
    key("t.u16", 2, "U16"); h.u16(50000, "value 50000")
    key("t.i16", 3, "I16"); h.i16(-20000, "value -20000")
    key("t.u32", 4, "U32"); h.u32(4000000000, "value 4000000000")
    key("t.i32", 5, "I32"); h.i32(-2000000000, "value -2000000000")
    key("t.f32", 6, "F32"); h.f32(0.5, "value 0.5")
    key("t.bool", 7, "Bool"); h.u8(1, "value true (one byte)")
    key("t.str", 8, "String"); h.string("héllo".encode(), version, "value 'héllo' (utf-8, 6 bytes)")
    key("t.arr", 9, "Array")
    h.u32(8, "element type String")
    h.count(3, version, "array length")
    for s in (b"a", b"", b"xyz\0"):
        h.string(s, version, "element %r (trailing NULs are dropped, :144-147)" % s)
    key("t.u64", 10, "U64"); h.u64(2 ** 63 + 5, "value 2^63 + 5")
    key("t.i64", 11, "I64"); h.i64(-(2 ** 62), "value -2^62")
    key("t.f64", 12, "F64"); h.f64(-1.25, "value -1.25")
    key("llama.expert_count", 4, "U32"); h.u32(8, "value 8")
    if alignment:
        key("general.alignment", 4, "U32"); h.u32(alignment, "value %d" % alignment)
    eff = alignment or 32   # DEFAULT_ALIGNMENT (:10) when the key is absent
    q4k, f32 = q4k_payload(), f32_payload()
    second_offset = (len(q4k) + eff - 1) // eff * eff
    # tensor infos: name, n_dimensions u32, dimensions innermost first, dtype u32, offset u64 (:464-492)
    h.string(b"blk.0.ffn_gate.0.weight", version, "tensor name")
    h.u32(2, "n_dimensions")
    h.count(256, version, "dimension 0 = innermost (columns); the reader reverses the list (:481)")
    h.count(2, version, "dimension 1 (rows)")
    h.u32(12, "ggml dtype Q4K")
    h.u64(0, "offset from the start of the tensor data (u64 in every version)")
    h.string(b"small.f32", version, "tensor name")
    h.u32(1, "n_dimensions")
    h.count(4, version, "dimension 0")
    h.u32(0, "ggml dtype F32")
    h.u64(second_offset, "offset from the start of the tensor data")
    h.pad_to(eff, "padding up to a multiple of the alignment: the tensor data starts here (:504)")
    data_start = h.n
    h.put(q4k, "tensor 0: two BlockQ4K, bytes (7 i + 3) mod 256")
    h.pad_to(eff, "padding")
    assert h.n - data_start == second_offset
    h.put(f32, "tensor 1: f32 1.0, -2.5, 0.0, 1e-3")
    h.save("gguf_v%d.hex.txt" % version,
           ["GGUF version %d, alignment %s; tensor data starts at byte %d; written by make_gguf_fixtures.py" % (version, alignment or "default 32", data_start),
            "format: <hex bytes>  # @<file offset> <field>"])
    return data_start


if __name__ == "__main__":
    for version, alignment in ((1, 0), (2, 64), (3, 128)):
        print("v%d: tensor data at %d" % (version, build(version, alignment)))
