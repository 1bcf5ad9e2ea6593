"""Pins the CPU oracle's block formats against the reference's own known answers."""
import numpy as np
import pytest

from rand09 import std_rng_f32


def ramp(bound, size=1024):
    # get_test_vector2, candle-core/tests/quantized_tests.rs:393-405
    i = np.arange(size, dtype=np.float32)
    return (i - np.float32(size / 2)) * np.float32(bound) / np.float32(size / 2)


def ggml_like(offset, n=4096):
    # create_ggml_like_vector, quantized_tests.rs:428-432 (f32 cos of an f32 argument)
    i = np.arange(n, dtype=np.float32) + np.float32(offset)
    return (np.float32(0.1) + np.float32(2.0) * np.cos(i, dtype=np.float32)).astype(np.float32)


def test_f16_exhaustive(O):
    h = np.arange(65536, dtype=np.uint16)
    want = h.view(np.float16).astype(np.float32)
    got = np.array([O.f16_to_f32(int(v)) for v in h], dtype=np.float32)
    assert np.array_equal(got.view(np.uint32)[~np.isnan(want)], want.view(np.uint32)[~np.isnan(want)])
    assert np.isnan(got[np.isnan(want)]).all()
    # every representable half converts back to itself
    fin = ~np.isnan(want)
    back = np.array([O.f32_to_f16(float(v)) for v in want[fin]], dtype=np.uint16)
    assert np.array_equal(back, h[fin])


def test_f32_to_f16_rounding(O):
    rng = np.random.default_rng(7)
    bits = rng.integers(0, 2**32, size=200000, dtype=np.uint64).astype(np.uint32)
    # concentrate half of the samples around the f16 range incl. subnormals and ties
    e = rng.integers(127 - 27, 127 + 17, size=100000).astype(np.uint32)
    bits[:100000] = (bits[:100000] & np.uint32(0x807FFFFF)) | (e << np.uint32(23))
    bits[:20000] &= np.uint32(0xFFFFF000)  # many exact ties
    f = bits.view(np.float32)
    f = f[~np.isnan(f)]
    with np.errstate(over="ignore"):
        want = f.astype(np.float16).view(np.uint16)
    got = np.array([O.f32_to_f16(float(v)) for v in f], dtype=np.uint16)
    assert np.array_equal(got, want)


def test_q4_0_roundtrip_known_answer(O, golden):
    src = np.arange(128, dtype=np.float32)
    dst = O.dequantize(O.Q4_0, O.quantize(O.Q4_0, src), 128)
    want = np.array(golden["q4_0_roundtrip_0_127"]["expected"], dtype=np.float32)
    assert np.array_equal(dst.view(np.uint32), want.view(np.uint32))  # includes the two -0.0


def round3_half_away(v):
    # round_vector, quantized_tests.rs:407-412: f32::round(1000 x) / 1000 (ties away from zero)
    t = np.float32(1000.0) * np.asarray(v, dtype=np.float32)
    return (np.sign(t) * np.floor(np.abs(t) + np.float32(0.5))).astype(np.float32) / np.float32(1000.0)


@pytest.mark.parametrize("name,dt", [("q4_1", 3), ("q5_0", 6), ("q5_1", 7)])
def test_legacy_roundtrip_known_answers(O, golden, name, dt):
    # quantize_q4_1 / quantize_q5_0 / quantize_q5_1: 0..128 through from_float and to_float, to three decimals
    src = np.arange(128, dtype=np.float32)
    dst = O.dequantize(dt, O.quantize(dt, src), 128)
    want = np.array(golden[name + "_roundtrip_0_127"]["expected_rounded_3"], dtype=np.float32)
    assert round3_half_away(dst).tolist() == want.tolist()


@pytest.mark.parametrize("simd", [False, True])
def test_q4_0_matmul_known_answers(O, golden, simd):
    m, k, n = 3, 64, 4
    lhs = np.arange(m * k, dtype=np.float32).reshape(m, k)
    rhs = np.arange(k * n, dtype=np.float32)
    got = O.matmul(O.Q4_0, lhs, O.quantize(O.Q4_0, rhs), n, simd=simd)
    assert np.round(got).reshape(-1).tolist() == golden["q4_0_matmul_3_64_4"]["expected_rounded"]
    lhs = (np.arange(m * k, dtype=np.float32) - np.float32(m * k / 2.0)).reshape(m, k)
    rhs = np.arange(k * n, dtype=np.float32) - np.float32(k * n / 3.0)
    got = O.matmul(O.Q4_0, lhs, O.quantize(O.Q4_0, rhs), n, simd=simd)
    assert np.round(got).reshape(-1).tolist() == golden["q4_0_matmul_neg_3_64_4"]["expected_rounded"]


@pytest.mark.parametrize("name,dt", [("q2k_ramp", 10), ("q3k_ramp", 11), ("q4k_ramp", 12), ("q5k_ramp", 13), ("q6k_ramp", 14), ("q8k_ramp", 15)])
def test_kquant_ramp_spot_values(O, golden, name, dt):
    g = golden[name]
    idx = golden["ramp_spot_indices"]
    src = ramp(0.5)
    assert src[idx].tolist() == np.array(golden["ramp_src_spot"]["expected"], dtype=np.float32).tolist()
    dst = O.dequantize(dt, O.quantize(dt, src), 1024)
    assert np.abs(dst - src).max() < g["max_abs_err_bound_0p5"]
    got = (np.round(np.float32(1000.0) * dst[idx]) / np.float32(1000.0)).astype(np.float32)
    assert got.tolist() == np.array(g["spot_rounded_3"], dtype=np.float32).tolist()
    if "max_abs_err_bound_128" in g:  # the reference's Q6K test states no bound for the large ramp
        big = ramp(128.0)
        dbig = O.dequantize(dt, O.quantize(dt, big), 1024)
        assert np.abs(dbig - big).max() < g["max_abs_err_bound_128"]


@pytest.mark.parametrize("dt", [2, 3, 6, 7, 8, 10, 11, 12, 13, 14, 15])
def test_ggml_quantization_rmse(O, golden, dt):
    src = ggml_like(0.0)
    dst = O.dequantize(dt, O.quantize(dt, src), src.size)
    rmse = np.sqrt(np.sum((src - dst).astype(np.float32) ** 2, dtype=np.float32)) / src.size
    assert rmse <= golden["ggml_quantization_rmse_bound"][{10: "bound_2bits", 11: "bound_3bits"}.get(dt, "bound")]


@pytest.mark.parametrize("dt", [2, 3, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15])
def test_ggml_dot_error(O, golden, dt):
    # ggml_matmul_error_test, quantized_tests.rs:846-911
    g = golden["ggml_dot_error"]
    n = 4096
    cases = [(ggml_like(0.0), ggml_like(1.0), 1.0),
             (np.arange(n, dtype=np.float32) / np.float32(n), np.arange(n, dtype=np.float32) / np.float32(n), 2.0)]
    for a, b, err_m in cases:
        aq = O.quantize(dt, a)
        bq = O.quantize(O.VECDOT[dt], b)
        r_unopt = O.vec_dot(dt, n, aq, bq)
        r_opt = O.vec_dot(dt, n, aq, bq, simd=True)
        assert abs(r_opt - r_unopt) / n <= 1e-6
        r_mm = float(O.matmul(dt, b.reshape(1, n), aq, 1)[0, 0])
        assert abs(r_mm - r_unopt) / n <= 1e-6
        ref = float(np.sum(a * b, dtype=np.float32))
        for r in (r_unopt, r_opt, r_mm):
            err = abs(r - ref) / n
            assert err <= g["max_dot_product_error"]
            assert err - g["leniency"] <= g["reference_error"][str(dt)] * err_m


def test_vec_dot_matches_dequantised_float64(O):
    # brute force: the integer block dot must equal the float dot of the dequantised operands
    rng = np.random.default_rng(3)
    n = 2048
    for dt in (O.Q4_0, O.Q4_1, O.Q5_0, O.Q5_1, O.Q8_0, O.Q2K, O.Q3K, O.Q4K, O.Q5K, O.Q6K):
        w = rng.normal(0, 0.02, n).astype(np.float32)
        if dt in (O.Q4_1, O.Q5_1):
            w += np.float32(0.05)  # a block minimum that matters
        x = rng.normal(0, 1.0, n).astype(np.float32)
        wq, xq = O.quantize(dt, w), O.quantize(O.VECDOT[dt], x)
        wd = O.dequantize(dt, wq, n).astype(np.float64)
        if O.VECDOT[dt] == O.Q8_1:  # the reference has no to_float for Q8_1: d * qs, decoded here
            blk = xq.reshape(-1, 36)
            xd = (blk[:, :2].copy().view(np.float16).astype(np.float64) * blk[:, 4:].view(np.int8)).reshape(-1)
        else:
            xd = O.dequantize(O.VECDOT[dt], xq, n).astype(np.float64)
        want = float(wd @ xd)
        for simd in (False, True):
            got = O.vec_dot(dt, n, wq, xq, simd=simd)
            assert abs(got - want) <= 2e-5 * np.sqrt(n) * np.abs(wd).max() * np.abs(xd).max() * 8


@pytest.mark.parametrize("simd", [False, True])
def test_seeded_matmul_spot_values(O, golden, simd):
    g = golden["seeded_matmul_11_512_21"]
    m, k, n = 11, 512, 21
    v = std_rng_f32(g["seed"], (m + n) * k)
    lhs = (v[: m * k] - np.float32(0.5)).reshape(m, k)
    rhs = (v[m * k:] - np.float32(0.5)).reshape(n, k)
    pick = [0, m * n // 3, m * n * 2 // 3, m * n - 1]
    r3 = lambda a: [float(np.round(np.float32(1000.0) * np.float32(x)) / np.float32(1000.0)) for x in a]
    dense = (lhs.astype(np.float64) @ rhs.astype(np.float64).T).reshape(-1)
    assert r3(dense[pick]) == r3(g["dense"])  # validates the StdRng restatement itself
    for key, dt in (("q2k", O.Q2K), ("q3k", O.Q3K), ("q4k", O.Q4K), ("q5k", O.Q5K), ("q6k", O.Q6K), ("q8k", O.Q8K)):
        mm = O.matmul(dt, lhs, O.quantize(dt, rhs), n, simd=simd).reshape(-1)
        assert r3(mm[pick]) == r3(g[key])


def test_matmul_batch_invariance_and_threads(O):
    # qmm_batch, quantized_tests.rs:221-256: identical rows give identical outputs at any batch
    rng = np.random.default_rng(11)
    k, n = 512, 300
    w = O.quantize(O.Q4K, rng.normal(0, 0.02, (n, k)).astype(np.float32))
    lhs = rng.normal(0, 1, (2, k)).astype(np.float32)
    mm = O.matmul(O.Q4K, lhs, w, n)
    mm6 = O.matmul(O.Q4K, np.concatenate([lhs] * 3), w, n, threads=4)
    assert np.array_equal(mm6[2:4], mm) and np.array_equal(mm6[4:], mm)


def test_q8_quantizer_closed_forms(O):
    rng = np.random.default_rng(5)
    x = rng.normal(0, 1, 256).astype(np.float32)
    x[17] = -4.5  # largest magnitude is negative: Q8K must map it to +... -128*-1 -> clipped 127? no: iscale=-128/max
    b = O.quantize(O.Q8K, x)
    d = b[:4].view(np.float32)[0]
    qs = b[4:260].view(np.int8)
    bs = b[260:].view(np.int16)
    iscale = np.float32(-128.0) / np.float32(-4.5)
    assert d == np.float32(1.0) / iscale
    assert qs[17] == -128
    want = np.minimum(np.sign(iscale * x) * np.floor(np.abs(iscale * x) + np.float32(0.5)), 127).astype(np.int8)
    assert np.array_equal(qs, want)
    assert np.array_equal(bs, qs.astype(np.int32).reshape(16, 16).sum(1).astype(np.int16))
    # positive maximum: the maximum itself would be -128*... = -128 -> stays in range, others clip at 127
    x2 = -x
    q2 = O.quantize(O.Q8K, x2)[4:260].view(np.int8)
    assert q2[17] == -128 and q2.max() <= 127
    # Q8_0: d = amax/127 stored as f16, quants use the unrounded f32 reciprocal
    y = rng.normal(0, 1, 32).astype(np.float32)
    b0 = O.quantize(O.Q8_0, y)
    d32 = np.abs(y).max() / np.float32(127.0)
    assert b0[:2].view(np.float16)[0] == np.float16(d32)
    idv = np.float32(1.0) / d32
    t = y * idv
    want0 = (np.sign(t) * np.floor(np.abs(t) + np.float32(0.5))).astype(np.int8)
    assert np.array_equal(b0[2:].view(np.int8), want0)
    # all-zero blocks
    assert not O.quantize(O.Q8K, np.zeros(256, np.float32)).any()
    assert not O.quantize(O.Q8_0, np.zeros(32, np.float32)).any()
    z4 = O.quantize(O.Q4_0, np.zeros(32, np.float32))  # d = 0/-8 = -0.0, every nibble 8
    assert z4[:2].view(np.uint16)[0] == 0x8000 and (z4[2:] == 0x88).all()


def test_q8_1_closed_forms(O):
    # Q8_1 = the Q8_0 block plus s = f16(sum of quants) * d in binary16 arithmetic (k_quants.rs:716-727)
    rng = np.random.default_rng(6)
    x = rng.normal(0, 1, 32 * 64).astype(np.float32)
    x[:32] = 3.0   # sum = 32 * 127 = 4064: not a multiple of 4, so f16(sum) rounds
    x[32:64] = 0.0
    b1 = O.quantize(O.Q8_1, x).reshape(-1, 36)
    b0 = O.quantize(O.Q8_0, x).reshape(-1, 34)
    assert np.array_equal(b1[:, :2], b0[:, :2]) and np.array_equal(b1[:, 4:], b0[:, 2:])
    d = b1[:, :2].copy().view(np.float16).reshape(-1)
    sums = b1[:, 4:].view(np.int8).astype(np.int32).sum(1)
    assert sums[0] == 4064
    want = (sums.astype(np.float16).astype(np.float32) * d.astype(np.float32)).astype(np.float16)
    assert np.array_equal(b1[:, 2:4].copy().view(np.float16).reshape(-1).view(np.uint16), want.view(np.uint16))
    assert not b1[1].any()


def test_legacy_layouts_against_independent_decoders(O):
    # numpy decoders of the published block layouts: Q4_1 (d, m, 16 nibble bytes), Q5_0 (d, 32 fifth bits, nibbles),
    # Q5_1 (d, m, fifth bits, nibbles); element j < 16 is the low nibble of byte j, element j + 16 the high one,
    # and the fifth bit of element e is bit e of the 32-bit little-endian word
    rng = np.random.default_rng(12)
    x = (rng.normal(0, 1, 32 * 40) + 0.3).astype(np.float32)
    for dt, nb, has_m, has_h in ((O.Q4_1, 20, True, False), (O.Q5_0, 22, False, True), (O.Q5_1, 24, True, True)):
        blk = O.quantize(dt, x).reshape(-1, nb)
        pos = 2
        d = blk[:, :2].copy().view(np.float16).astype(np.float32)
        m = np.zeros_like(d)
        if has_m:
            m = blk[:, 2:4].copy().view(np.float16).astype(np.float32); pos = 4
        hi = np.zeros((blk.shape[0], 32), dtype=np.int32)
        if has_h:
            word = blk[:, pos:pos + 4].copy().view("<u4").reshape(-1, 1)
            hi = ((word >> np.arange(32, dtype=np.uint32)) & 1).astype(np.int32) << 4
            pos += 4
        qs = blk[:, pos:pos + 16].astype(np.int32)
        code = np.concatenate([qs & 15, qs >> 4], axis=1) | hi
        if dt == O.Q5_0:
            code = code - 16
        want = code.astype(np.float32) * d + m if has_m else code.astype(np.float32) * d
        got = O.dequantize(dt, blk.reshape(-1), x.size).reshape(-1, 32)
        assert np.array_equal(got.view(np.uint32), want.astype(np.float32).view(np.uint32))
        assert np.abs(got.reshape(-1) - x).max() <= (np.abs(d).max() * (0.51 if dt != O.Q5_0 else 1.01))


def test_q4k_layout_against_independent_decoder(O):
    # independent numpy decoder of the published Q4_K layout (d, dmin, 12 packed 6-bit scale/min bytes,
    # 128 nibble bytes: byte l of each 32-byte group holds element l (low) and l+32 (high))
    rng = np.random.default_rng(9)
    x = rng.normal(0, 0.02, 1024).astype(np.float32)
    blocks = O.quantize(O.Q4K, x).reshape(4, 144)
    out = np.empty((4, 256), dtype=np.float32)
    for b in range(4):
        raw = blocks[b]
        d = np.float32(raw[0:2].view(np.float16)[0])
        dmin = np.float32(raw[2:4].view(np.float16)[0])
        s = raw[4:16].astype(np.int32)
        sc = np.zeros(8, np.int32)
        mn = np.zeros(8, np.int32)
        for j in range(8):
            if j < 4:
                sc[j], mn[j] = s[j] & 63, s[j + 4] & 63
            else:
                sc[j] = (s[j + 4] & 0xF) | ((s[j - 4] >> 6) << 4)
                mn[j] = (s[j + 4] >> 4) | ((s[j] >> 6) << 4)
        qs = raw[16:].reshape(4, 32)
        for g in range(4):
            lo = (qs[g] & 0xF).astype(np.float32)
            hi = (qs[g] >> 4).astype(np.float32)
            out[b, 64 * g: 64 * g + 32] = (d * np.float32(sc[2 * g])) * lo - dmin * np.float32(mn[2 * g])
            out[b, 64 * g + 32: 64 * g + 64] = (d * np.float32(sc[2 * g + 1])) * hi - dmin * np.float32(mn[2 * g + 1])
    got = O.dequantize(O.Q4K, blocks.reshape(-1), 1024)
    assert np.array_equal(got.view(np.uint32), out.reshape(-1).view(np.uint32))


def test_q6k_layout_against_independent_decoder(O):
    # independent numpy decoder of the published Q6_K layout, addressed by element rather than by the
    # reference's loop nest: 128 bytes of low nibbles, 64 bytes of 2-bit highs, 16 i8 scales, f16 d.
    # Element e of a block lies in half e//128, quarter q = (e%128)//32, column l = e%32: its low
    # nibble is in ql[64*half + 32*(q&1) + l] (high nibble for q >= 2), its two high bits are bits
    # 2q..2q+1 of qh[32*half + l], and its scale is scales[e//16].
    rng = np.random.default_rng(10)
    x = rng.normal(0, 0.02, 1024).astype(np.float32)
    x[256:272] = 0.0           # one all-zero 16-element group
    blocks = O.quantize(O.Q6K, x).reshape(4, 210)
    out = np.empty((4, 256), dtype=np.float32)
    codes = np.empty((4, 256), dtype=np.int32)
    for b in range(4):
        raw = blocks[b]
        ql, qh = raw[:128].astype(np.int32), raw[128:192].astype(np.int32)
        sc = raw[192:208].view(np.int8).astype(np.float32)
        d = np.float32(raw[208:210].view(np.float16)[0])
        for e in range(256):
            half, q, l = e // 128, (e % 128) // 32, e % 32
            byte = ql[64 * half + 32 * (q & 1) + l]
            nib = (byte >> 4) if q >= 2 else (byte & 15)
            hi = (qh[32 * half + l] >> (2 * q)) & 3
            codes[b, e] = (nib | (hi << 4)) - 32
            out[b, e] = d * sc[e // 16] * np.float32(codes[b, e])
    got = O.dequantize(O.Q6K, blocks.reshape(-1), 1024)
    assert np.array_equal(got.view(np.uint32), out.reshape(-1).view(np.uint32))
    assert codes.min() >= -32 and codes.max() <= 31 and codes.max() - codes.min() > 40
    assert np.abs(got - x).max() < 0.02 * 4 / 31    # a 6-bit grid over at most ~4 sigma
    # the dot product is the integer sum the layout implies, against float64
    y = rng.normal(0, 1, 1024).astype(np.float32)
    yq = O.quantize(O.Q8K, y)
    yd = O.dequantize(O.Q8K, yq, 1024).astype(np.float64)
    want = float(out.reshape(-1).astype(np.float64) @ yd)
    for simd in (False, True):
        assert abs(O.vec_dot(O.Q6K, 1024, blocks.reshape(-1), yq, simd=simd) - want) <= 1e-5 * abs(want) + 1e-6


def test_q6k_quantizer_closed_forms(O):
    # a 16-element group holding one value c repeated maps to the extreme code: make_qx_quants
    # (utils.rs:62-94) picks iscale = -32/c, so every code is -32 and the group scale is -c/32; the
    # super-block scale d = max |scale| / 128 with sign, and the stored i8 scale of that group is -128.
    x = np.zeros(256, dtype=np.float32)
    x[32:48] = 0.5
    b = O.quantize(O.Q6K, x)
    sc = b[192:208].view(np.int8)
    d = b[208:210].view(np.float16)[0]
    assert sc[2] == -128 and not sc[[0, 1] + list(range(3, 16))].any()
    assert np.float32(d) == np.float32(np.float16(np.float32(0.5) / np.float32(32.0) / np.float32(128.0)))
    y = O.dequantize(O.Q6K, b, 256)
    assert np.array_equal(y[32:48], np.full(16, 0.5, np.float32)) and not y[:32].any() and not y[48:].any()
    # all zeros: d = -0.0 (1 / (-128 / 0)), zero scales, codes 0 (value -32 * 0)
    z = O.quantize(O.Q6K, np.zeros(256, np.float32))
    assert z[208:210].view(np.uint16)[0] == 0x8000 and not z[:208].any()
    assert not O.dequantize(O.Q6K, z, 256).any()


def test_q5k_layout_against_independent_decoder(O):
    # independent numpy decoder of the published Q5_K layout, addressed by element: d, dmin, the 12 packed
    # scale / min bytes of Q4_K, 32 bytes of high bits, 128 nibble bytes.  Element e lies in pair e//64,
    # half (e%64)//32, column l = e%32: nibble byte qs[32*pair + l] (high nibble for the second half), fifth
    # bit = bit 2*pair + half of qh[l].
    rng = np.random.default_rng(12)
    x = rng.normal(0, 0.02, 1024).astype(np.float32)
    blocks = O.quantize(O.Q5K, x).reshape(4, 176)
    out = np.empty((4, 256), dtype=np.float32)
    codes = np.empty((4, 256), dtype=np.int32)
    for b in range(4):
        raw = blocks[b]
        d = np.float32(raw[0:2].view(np.float16)[0])
        dmin = np.float32(raw[2:4].view(np.float16)[0])
        s = raw[4:16].astype(np.int32)
        qh, qs = raw[16:48].astype(np.int32), raw[48:176].astype(np.int32)
        for e in range(256):
            pair, half, l = e // 64, (e % 64) // 32, e % 32
            j = 2 * pair + half
            if j < 4:
                sc, mn = s[j] & 63, s[j + 4] & 63
            else:
                sc, mn = (s[j + 4] & 0xF) | ((s[j - 4] >> 6) << 4), (s[j + 4] >> 4) | ((s[j] >> 6) << 4)
            byte = qs[32 * pair + l]
            code = ((byte >> 4) if half else (byte & 15)) + 16 * ((qh[l] >> j) & 1)
            codes[b, e] = code
            out[b, e] = (d * np.float32(sc)) * np.float32(code) - dmin * np.float32(mn)
    got = O.dequantize(O.Q5K, blocks.reshape(-1), 1024)
    assert np.array_equal(got.view(np.uint32), out.reshape(-1).view(np.uint32))
    assert codes.min() == 0 and codes.max() == 31
    assert np.abs(got - x).max() < 0.02 * 8 / 31


def test_q2k_layout_against_independent_decoder(O):
    # independent numpy decoder of the published Q2_K layout, addressed by element: 16 bytes of
    # (4-bit scale | 4-bit min << 4) per 16 elements, 64 bytes of 2-bit codes, f16 d and dmin.  Element e
    # lies in half e//128, quarter q = (e%128)//32, column l = e%32: its code is bits 2q..2q+1 of
    # qs[32*half + l], its scale byte is scales[e//16].
    rng = np.random.default_rng(13)
    x = rng.normal(0, 0.02, 1024).astype(np.float32)
    blocks = O.quantize(O.Q2K, x).reshape(4, 84)
    out = np.empty((4, 256), dtype=np.float32)
    codes = np.empty((4, 256), dtype=np.int32)
    for b in range(4):
        raw = blocks[b]
        sc, qs = raw[:16].astype(np.int32), raw[16:80].astype(np.int32)
        d = np.float32(raw[80:82].view(np.float16)[0])
        dmin = np.float32(raw[82:84].view(np.float16)[0])
        for e in range(256):
            half, q, l = e // 128, (e % 128) // 32, e % 32
            codes[b, e] = (qs[32 * half + l] >> (2 * q)) & 3
            s = sc[e // 16]
            out[b, e] = (d * np.float32(s & 15)) * np.float32(codes[b, e]) - dmin * np.float32(s >> 4)
    got = O.dequantize(O.Q2K, blocks.reshape(-1), 1024)
    assert np.array_equal(got.view(np.uint32), out.reshape(-1).view(np.uint32))
    assert codes.min() == 0 and codes.max() == 3
    assert np.abs(got - x).max() < 0.02 * 8 / 3


def test_q3k_layout_against_independent_decoder(O):
    # independent numpy decoder of the published Q3_K layout, addressed by element: 32 bytes of high bits,
    # 64 bytes of 2-bit codes, 12 bytes holding sixteen 6-bit scales (stored + 32), f16 d.  Element e lies in
    # 32-element group G = e//32 (half G//4, quarter G%4), column l = e%32: low bits 2(G%4).. of
    # qs[32*(G//4) + l], high bit = bit G of hmask[l] (clear means -4); scale j = e//16 has its low nibble in
    # scales[j%8] (upper nibble for j >= 8) and its two high bits at 2*(j//4) of scales[8 + j%4].
    rng = np.random.default_rng(14)
    x = rng.normal(0, 0.02, 1024).astype(np.float32)
    blocks = O.quantize(O.Q3K, x).reshape(4, 110)
    out = np.empty((4, 256), dtype=np.float32)
    codes = np.empty((4, 256), dtype=np.int32)
    scs = np.empty((4, 16), dtype=np.int32)
    for b in range(4):
        raw = blocks[b]
        hmask, qs, sc = raw[:32].astype(np.int32), raw[32:96].astype(np.int32), raw[96:108].astype(np.int32)
        d = np.float32(raw[108:110].view(np.float16)[0])
        for j in range(16):
            lo = (sc[j % 8] >> (4 if j >= 8 else 0)) & 15
            hi = (sc[8 + j % 4] >> (2 * (j // 4))) & 3
            scs[b, j] = (lo | (hi << 4)) - 32
        for e in range(256):
            G, l = e // 32, e % 32
            low = (qs[32 * (G // 4) + l] >> (2 * (G % 4))) & 3
            codes[b, e] = low - (0 if (hmask[l] >> G) & 1 else 4)
            out[b, e] = (d * np.float32(scs[b, e // 16])) * np.float32(codes[b, e])
    got = O.dequantize(O.Q3K, blocks.reshape(-1), 1024)
    assert np.array_equal(got.view(np.uint32), out.reshape(-1).view(np.uint32))
    assert codes.min() == -4 and codes.max() == 3 and scs.min() == -32 and scs.max() > 0
    assert np.abs(got - x).max() < 0.02 * 8 / 4


def test_round_half_away_identity_of_the_device_quantisers():
    """The HIP activation quantisers take `(scale * x).round()` (f32::round: half away from zero) as
    trunc(v + copysign(0.49999997, v)), 0.49999997 being the float below one half; beyond |v| = 130 both sides of their
    clamp to [-128, 127] agree anyway.  Checked here over every non-negative float up to 130 (float addition and trunc
    are odd functions, so the negative half follows)."""
    c = np.float32(0.49999997)
    assert c == np.nextafter(np.float32(0.5), np.float32(0))
    hi = int(np.float32(130.0).view(np.uint32))
    step = 1 << 25
    for s0 in range(0, hi + 1, step):
        x = np.arange(s0, min(s0 + step, hi + 1), dtype=np.uint32).view(np.float32)
        got = np.trunc(x + c)                                   # f32 arithmetic, as on the device
        want = np.floor(x.astype(np.float64) + 0.5)             # round half away from zero, exactly
        assert np.array_equal(got, want), x[got != want][:4]
