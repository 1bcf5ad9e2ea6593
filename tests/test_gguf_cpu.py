"""GGUF container reader (host code of the library, no GPU needed) against files written the way the
reference's own writer does (gguf_file.rs:534-582), and against the reference's error behaviour."""
import os
import struct

import numpy as np
import pytest

import candle_amd
import gguf_writer as W


def rnd(n, seed=0):
    return np.random.default_rng(seed).integers(0, 256, n, dtype=np.uint8)


@pytest.mark.parametrize("version", [1, 2, 3])
def test_round_trip_all_value_types_and_tensors(tmp_path, version):
    md = [("a.u8", W.U8, 200), ("a.i8", W.I8, -100), ("a.u16", W.U16, 60000), ("a.i16", W.I16, -30000),
          ("a.u32", W.U32, 4000000000), ("a.i32", W.I32, -2000000000), ("a.u64", W.U64, 1 << 40), ("a.i64", W.I64, -(1 << 40)),
          ("a.f32", W.F32, 1.5), ("a.f64", W.F64, -2.25), ("a.true", W.BOOL, 1), ("a.false", W.BOOL, 0),
          ("a.str", W.STRING, b"hello\0\0"),  # trailing NULs are dropped (gguf_file.rs:145-148)
          ("a.arr", W.ARRAY, (W.U32, [1, 2, 3])), ("a.strs", W.ARRAY, (W.STRING, ["x", "yy"])),
          ("a.nested", W.ARRAY, (W.ARRAY, [(W.U8, [1, 2]), (W.U8, [])])), ("a.empty", W.ARRAY, (W.U32, []))]
    tensors = [("t.f32", 0, (3, 5), rnd(60, 1)), ("t.f16", 1, (7,), rnd(14, 2)), ("t.q4_0", 2, (4, 64), rnd(4 * 2 * 18, 3)),
               ("t.q8_0", 8, (2, 3, 32), rnd(6 * 34, 4)), ("t.q4k", 12, (2, 512), rnd(4 * 144, 5)), ("t.q6k", 14, (256,), rnd(210, 6))]
    path = tmp_path / "f.gguf"
    data_start = W.write_gguf(path, md, tensors, version=version)
    with candle_amd.GgufFile(str(path)) as g:
        assert g.version == version
        assert g.tensor_data_offset == data_start and data_start % 32 == 0
        assert g.tensor_names() == [t[0] for t in tensors]
        assert g.metadata("a.u8") == 200 and g.metadata("a.i8") == -100
        assert g.metadata("a.u16") == 60000 and g.metadata("a.i16") == -30000
        assert g.metadata("a.u32") == 4000000000 and g.metadata("a.i32") == -2000000000
        assert g.metadata("a.u64") == 1 << 40 and g.metadata("a.i64") == -(1 << 40)
        assert g.metadata("a.f32") == 1.5 and g.metadata("a.f64") == -2.25
        assert g.metadata("a.true") is True and g.metadata("a.false") is False
        assert g.metadata("a.str") == "hello"
        assert g.metadata("a.arr") == ("array", 3, W.U32) and g.metadata("a.strs") == ("array", 2, W.STRING)
        assert g.metadata("a.nested") == ("array", 2, W.ARRAY) and g.metadata("a.empty")[1] == 0
        raw = open(path, "rb").read()
        off = data_start
        for name, dt, shape, data in tensors:
            gdt, gshape, gbytes = g.tensor(name)
            assert (gdt, gshape) == (dt, shape)          # dimensions come back outermost first
            assert bytes(gbytes) == bytes(data) == raw[off: off + len(bytes(data))]
            off += (len(bytes(data)) + 31) // 32 * 32    # every tensor starts on a 32-byte boundary
        with pytest.raises(candle_amd.MoeError, match="cannot find tensor info for nope"):
            g.tensor("nope")
        with pytest.raises(candle_amd.MoeError, match="cannot find nope in metadata"):
            g.metadata("nope")


def test_alignment_key_moves_the_tensor_data(tmp_path):
    path = tmp_path / "a.gguf"
    start = W.write_gguf(path, [("general.alignment", W.U32, 256), ("k", W.STRING, "v" * 70)], [("t", 0, (4,), rnd(16))], alignment=256)
    with candle_amd.GgufFile(str(path)) as g:
        assert g.tensor_data_offset == start and start % 256 == 0
        assert bytes(g.tensor("t")[2]) == bytes(rnd(16))
    # a negative signed alignment is ignored (gguf_file.rs:497-504): the default 32 applies
    path2 = tmp_path / "b.gguf"
    start2 = W.write_gguf(path2, [("general.alignment", W.I32, -8)], [("t", 0, (4,), rnd(16))])
    with candle_amd.GgufFile(str(path2)) as g:
        assert g.tensor_data_offset == start2 and start2 % 32 == 0


def test_both_magics_are_accepted(tmp_path):
    for magic in (0x46554747, 0x47475546):  # gguf_file.rs:19
        path = tmp_path / ("m%x.gguf" % magic)
        W.write_gguf(path, [], [], magic=magic)
        with candle_amd.GgufFile(str(path)) as g:
            assert g.tensor_names() == []


def test_expert_count_keys_of_another_type_read_as_zero(tmp_path):
    # `md_get(key).and_then(|v| v.to_u32()).unwrap_or(0)` (quantized_llama.rs:507-512): `Value::to_u32`
    # (gguf_file.rs:249-254) takes the U32 variant only, so a string, a u64 or a missing key all give 0
    p = tmp_path / "keys.gguf"
    W.write_gguf(p, [("llama.expert_count", W.U32, 8), ("llama.expert_used_count", W.STRING, "2"),
                     ("llama.block_count", W.U64, 32)], [("t", 0, (4,), np.zeros(4, np.float32).tobytes())])
    with candle_amd.GgufFile(str(p)) as g:
        assert g.metadata_u32_or_zero("llama.expert_count") == 8
        assert g.metadata_u32_or_zero("llama.expert_used_count") == 0
        assert g.metadata_u32_or_zero("llama.block_count") == 0
        assert g.metadata_u32_or_zero("llama.absent") == 0
        assert g.metadata("llama.expert_used_count") == "2"


def test_malformed_files_are_rejected(tmp_path):
    good = tmp_path / "good.gguf"
    W.write_gguf(good, [("k", W.U32, 1)], [("t", 12, (256,), rnd(144))])
    raw = open(good, "rb").read()

    def expect(blob, pattern, name):
        p = tmp_path / name
        open(p, "wb").write(blob)
        with pytest.raises(candle_amd.MoeError, match=pattern):
            candle_amd.GgufFile(str(p))

    expect(b"GGML" + raw[4:], "unknown magic 0x4c4d4747", "magic.gguf")
    expect(raw[:4] + struct.pack("<I", 4) + raw[8:], "unsupported version 4", "version.gguf")
    expect(raw[:30], "end of file|truncated", "short.gguf")
    expect(raw[:3], "too short", "tiny.gguf")
    # value type 13 does not exist (gguf_file.rs:402-420)
    bad_vt = bytearray(raw)
    bad_vt[24 + 8 + 1: 24 + 8 + 1 + 4] = struct.pack("<I", 13)
    expect(bytes(bad_vt), "unrecognized value-type", "vt.gguf")
    with pytest.raises(candle_amd.MoeError, match="cannot open"):
        candle_amd.GgufFile(str(tmp_path / "missing.gguf"))
    # dtype id 5 is not a GgmlDType (quantized/mod.rs:153-174)
    p = tmp_path / "dtype.gguf"
    W.write_gguf(p, [], [("t", 12, (256,), rnd(144))])
    blob = bytearray(open(p, "rb").read())
    i = blob.index(b"t", 24) + 1 + 4 + 8           # name, n_dims, one u64 dimension
    assert struct.unpack_from("<I", blob, i)[0] == 12
    struct.pack_into("<I", blob, i, 5)
    expect(bytes(blob), "unknown dtype for tensor 5", "dtype2.gguf")


def test_tensor_size_and_bounds_checks(tmp_path):
    # 100 elements are not a whole number of Q4K blocks (gguf_file.rs:66-70)
    p = tmp_path / "div.gguf"
    W.write_gguf(p, [], [("t", 12, (100,), rnd(144))])
    with candle_amd.GgufFile(str(p)) as g:
        with pytest.raises(candle_amd.MoeError, match="the number of elements 100 is not divisible by the block size 256"):
            g.tensor("t")
    # the table promises more bytes than the file holds (gguf_file.rs:103-110)
    p2 = tmp_path / "cut.gguf"
    W.write_gguf(p2, [], [("t", 0, (1024,), rnd(4096))])
    raw = open(p2, "rb").read()
    open(p2, "wb").write(raw[:-2048])
    with candle_amd.GgufFile(str(p2)) as g:
        with pytest.raises(candle_amd.MoeError, match="tensor data extends beyond file boundary"):
            g.tensor("t")


def test_hostile_tables_are_refused_not_followed(tmp_path):
    # dimensions whose product wraps around 2^64 must not pass the size check as a small tensor
    p = tmp_path / "wrap.gguf"
    W.write_gguf(p, [], [("t", 0, (1 << 33, 1 << 33), rnd(64)), ("u", 12, (1 << 62, 1024), rnd(144))])
    with candle_amd.GgufFile(str(p)) as g:
        for name in ("t", "u"):
            with pytest.raises(candle_amd.MoeError, match="overflow"):
                g.tensor(name)
    # a data offset near 2^64 must not wrap the start address back into the file
    p2 = tmp_path / "offset.gguf"
    W.write_gguf(p2, [], [("t", 0, (16,), rnd(64))])
    blob = bytearray(open(p2, "rb").read())
    i = blob.index(b"t", 24) + 1 + 4 + 8 + 4           # name, n_dims, one u64 dimension, dtype
    assert struct.unpack_from("<Q", blob, i)[0] == 0
    struct.pack_into("<Q", blob, i, (1 << 64) - 32)
    open(p2, "wb").write(bytes(blob))
    with candle_amd.GgufFile(str(p2)) as g:
        with pytest.raises(candle_amd.MoeError, match="beyond file boundary"):
            g.tensor("t")
    # an array that claims more elements than the file has bytes left
    p3 = tmp_path / "array.gguf"
    W.write_gguf(p3, [("a", W.ARRAY, (W.U8, [1, 2, 3]))], [])
    blob = bytearray(open(p3, "rb").read())
    i = blob.index(b"a", 24) + 1 + 4 + 4               # key, value type (array), element type
    assert struct.unpack_from("<Q", blob, i)[0] == 3
    struct.pack_into("<Q", blob, i, 1 << 40)
    open(p3, "wb").write(bytes(blob))
    with pytest.raises(candle_amd.MoeError, match="array length past the end of the file"):
        candle_amd.GgufFile(str(p3))
    # an absurd alignment
    p4 = tmp_path / "align.gguf"
    W.write_gguf(p4, [("general.alignment", W.U32, 32)], [("t", 0, (8,), rnd(32))])
    blob = bytearray(open(p4, "rb").read())
    i = blob.index(b"general.alignment") + len("general.alignment") + 4
    assert struct.unpack_from("<I", blob, i)[0] == 32
    struct.pack_into("<I", blob, i, 0xFFFFFFFF)
    open(p4, "wb").write(bytes(blob))
    with pytest.raises(candle_amd.MoeError, match="general.alignment is 4294967295"):
        candle_amd.GgufFile(str(p4))


def test_reader_survives_mutated_files_under_sanitizers(tmp_path):
    # gguf.cpp (host code only) built with AddressSanitizer + UBSan around stubs that read every byte the reader
    # hands out; 2000 mutated copies of a valid MoE file (byte and bit flips, extreme 64-bit fields, truncations)
    # go through every public call of the reader.  Any out-of-bounds read, overflow or leak aborts the harness.
    import shutil
    import subprocess
    gxx = shutil.which("g++")
    if gxx is None or not os.path.isdir("/opt/rocm/include"):
        pytest.skip("needs g++ and the ROCm headers")
    here = os.path.dirname(os.path.abspath(__file__))
    exe = tmp_path / "gguf_fuzz"
    cmd = [gxx, "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=all", "-D__HIP_PLATFORM_AMD__",
           "-I/opt/rocm/include", os.path.join(here, "gguf_fuzz_harness.cpp"),
           os.path.join(here, "..", "candle_amd", "csrc", "gguf.cpp"), "-o", str(exe)]
    r = subprocess.run(cmd, capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-2000:]
    rng = np.random.default_rng(0)
    H, F, E = 256, 256, 4
    blk = lambda: rng.integers(0, 256, H * F // 256 * 144, dtype=np.uint8)
    gate = rng.standard_normal((E, H)).astype(np.float32)
    good = tmp_path / "good.gguf"
    W.moe_layer_file(good, 0, gate, [blk() for _ in range(E)], [blk() for _ in range(E)], [blk() for _ in range(E)], 12, 2,
                     extra_metadata=[("tokenizer.ggml.tokens", W.ARRAY, (W.STRING, ["a", "bb", "ccc"]))])
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0")
    r = subprocess.run([str(exe), str(good), str(tmp_path / "mut.gguf"), "2000", "7"], capture_output=True, text=True, env=env, timeout=300)
    assert r.returncode == 0, (r.stdout[-500:], r.stderr[-3000:])
    assert "2000 mutants survived" in r.stdout


# ---------------------------------------------------------------------------------------------
# Hand-assembled byte fixtures (tests/golden/gguf_v*.hex.txt): one field per line with the width Content::read takes
# for it (gguf_file.rs:34-46, 135-150, 318-357, 402-420, 443-505), written without tests/gguf_writer.py, so that a
# misreading shared by the library's reader and the test's own writer cannot hide.
def _fixture_bytes(version):
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "gguf_v%d.hex.txt" % version)
    out = bytearray()
    for line in open(path, encoding="utf-8"):
        if line.startswith("#"):
            continue
        out += bytes.fromhex(line.split("#", 1)[0].strip())
    return bytes(out)


@pytest.mark.parametrize("version,alignment,data_start", [(1, 32, 384), (2, 64, 576), (3, 128, 640)])
def test_hand_assembled_fixture(tmp_path, version, alignment, data_start):
    raw = _fixture_bytes(version)
    # what the reference's field widths give for v3: header 24 bytes, thirteen typed entries up to byte 342,
    # llama.expert_count (8 + 18 + 4 + 4) to 376, general.alignment (8 + 17 + 4 + 4) to 409, tensor infos
    # (8 + 23 + 4 + 16 + 4 + 8 = 63) to 472 and (8 + 9 + 4 + 8 + 4 + 8 = 41) to 513 -> next multiple of 128 = 640;
    # data: 288 bytes, the second tensor at +384, its 16 bytes end the file at 1040
    if version == 3:
        assert len(raw) == 1040
    path = tmp_path / ("fixture_v%d.gguf" % version)
    path.write_bytes(raw)
    with candle_amd.GgufFile(str(path)) as g:
        assert g.version == version
        assert g.tensor_data_offset == data_start and data_start % alignment == 0
        assert g.tensor_names() == ["blk.0.ffn_gate.0.weight", "small.f32"]
        assert g.metadata("t.u8") == 200 and g.metadata("t.i8") == -100
        assert g.metadata("t.u16") == 50000 and g.metadata("t.i16") == -20000
        assert g.metadata("t.u32") == 4000000000 and g.metadata("t.i32") == -2000000000
        assert g.metadata("t.f32") == 0.5 and g.metadata("t.bool") is True
        assert g.metadata("t.str") == "héllo"
        assert g.metadata("t.arr") == ("array", 3, 8)
        assert g.metadata("t.u64") == 2 ** 63 + 5 and g.metadata("t.i64") == -(2 ** 62) and g.metadata("t.f64") == -1.25
        assert g.metadata("llama.expert_count") == 8
        if version > 1:
            assert g.metadata("general.alignment") == alignment
        dt, shape, data = g.tensor("blk.0.ffn_gate.0.weight")
        assert dt == 12 and shape == (2, 256)          # outermost first: the on-disk order is reversed
        assert bytes(data) == bytes((7 * i + 3) & 0xFF for i in range(288))
        dt, shape, data = g.tensor("small.f32")
        assert dt == 0 and shape == (4,)
        assert np.array_equal(np.frombuffer(bytes(data), dtype="<f4"), np.array([1.0, -2.5, 0.0, 1e-3], dtype=np.float32))
        # the second tensor sits at the first multiple of the alignment past the 288 bytes of the first
        second = data_start + (288 + alignment - 1) // alignment * alignment
        assert raw[second:second + 16] == bytes(data)
